// Host-side helpers shared by the matmul and conv entry points: tile-shape
// choice and the launch of one gemm_kernel instantiation.
#pragma once

#include <math.h>
#include <stdlib.h>

#include "common.h"
#include "gemm_kernel.h"

namespace tfhip {

struct TileShape {
  int bm, bn, bk, waves_m, waves_n;
};

// Shapes instantiated for every loader combination (index = case in launch_gemm_shape).
static const TileShape kTileShapes[] = {
    {128, 128, 16, 2, 2}, {128, 96, 16, 2, 2}, {128, 64, 16, 2, 2}, {64, 64, 16, 2, 2},  {256, 32, 16, 4, 1},
    {256, 16, 16, 4, 1},  {64, 96, 16, 2, 2},  {128, 128, 32, 2, 2}, {128, 96, 32, 2, 2}, {64, 64, 32, 2, 2},
    {64, 48, 32, 4, 1},   {32, 64, 32, 2, 2},  {32, 32, 32, 2, 2},
};
constexpr int kNumTileShapes = 13;

// Estimated run time in microseconds of an M x N x K product, `batch` times,
// with tile shape t on `cus` compute units. Per workgroup and K tile the matrix
// cores need mfma_us; a lone workgroup on a compute unit is bound by the latency
// of one trip round the pipeline (lat_us) instead, and up to `resident`
// workgroups overlap on one compute unit. Constants were fitted to measured
// sweeps of all shapes over BERT-base and MobileNetV2 products on an MI355X.
inline double estimate_us(const TileShape &t, long long M, long long N, long long K, long long batch, int cus) {
  const long long tiles = ((M + t.bm - 1) / t.bm) * ((N + t.bn - 1) / t.bn) * batch;
  const long long k_tiles = (K + t.bk - 1) / t.bk;
  const int tm = t.bm / t.waves_m / 16, tn = t.bn / t.waves_n / 16;
  const double mfma_us = tm * tn * (t.bk / 4) * 32 / 2400.0;
  const double lat_us = 1.15 * mfma_us + 0.184 * (t.bk / 16.0);
  const long long per_cu = (tiles + cus - 1) / cus;
  const int resident_max = t.bm * t.bn <= 64 * 96 ? 3 : 2;
  const double resident = per_cu < resident_max ? (double)per_cu : (double)resident_max;
  const double trip = mfma_us * resident / 0.85 > lat_us ? mfma_us * resident / 0.85 : lat_us;
  double compute = (double)k_tiles * trip + 2.0 + t.bm * t.bn * 0.37e-3;
  if (per_cu > resident_max) compute *= (double)per_cu / resident_max;
  const double hbm = 4.0 * ((double)M * K + (double)K * N + (double)M * N) * batch / 4.94e6;
  return (compute > hbm ? compute : hbm) + 1.9;
}

// Picks the tile shape with the lowest estimated run time.
// The "tile" tuning knob overrides the choice.
inline int choose_tile_shape(long long M, long long N, long long K, long long batch, int cus) {
  const int forced = tuning(kTuneTile);
  if (forced >= 0 && forced < kNumTileShapes) return forced;
  // Very large products: the 128x128 tile with several workgroups per compute unit
  // runs the k loop at 85% of the matrix-core rate, the small tiles at 78%.
  if (((M + 127) / 128) * ((N + 127) / 128) * batch >= 3LL * cus && K >= 512) return 0;
  // One 64 x 48 tile on (nearly) every compute unit and a long k: that tile with two groups of
  // wavefronts sharing it (choose_k_groups) beats the 32 x 32 tile the estimate below prefers
  // (1024 x 768 x 3072: 43.9 against 47.0 us back to back, 45.4 against 55.2 us with operands from
  // memory; 1024 x 768 x 768: 15.5 against 15.7, 16.9 against 18.1).
  {
    const long long tiles = ((M + 63) / 64) * ((N + 47) / 48) * batch;
    if (tiles <= cus && tiles * 4 >= 3LL * cus && K >= 768) return 10;
  }
  int best = 0;
  double best_us = 0;
  for (int i = 0; i < kNumTileShapes; ++i) {
    const double us = estimate_us(kTileShapes[i], M, N, K, batch, cus);
    if (i == 0 || us < best_us) {
      best_us = us;
      best = i;
    }
  }
  return best;
}

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int A_KIND, int B_KIND, int KG = 1>
inline int launch_gemm(GemmParams &p) {
  using T = GemmTile<BM, BN, BK, WAVES_M, WAVES_N, A_KIND, B_KIND, KG>;
  p.tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  const long long tiles = (long long)p.tiles_m * p.tiles_n * p.batch;
  if (tiles <= 0) return kOk;
  // Split K when the tiles alone leave compute units idle and K is long: each
  // copy of the tile set sums a slice of k into the workspace and gemm_finish
  // adds the slices. Time model (us): fixed + k tiles on the busiest compute unit
  // x tile time, plus the second kernel.
  p.splits = 1;
  p.k_per_split = p.K;
  p.ws = nullptr;
  {
    const int k_tiles = (p.K + BK - 1) / BK;
    const double tile_us = (BM / 16) * (BN / 16) / 4 * (BK / 4) * 32 / 2400.0 / 0.63;
    const int cus = num_cus();
    int best = 1;
    double best_us = 0;
    for (int s = 1; s <= 8; ++s) {
      if (s > 1 && k_tiles / s < 6) break;
      // the busiest compute unit runs `rounds` workgroups of `kt` k tiles each; a
      // unit holding several at once gains little (measured about 8%)
      const long long rounds = (tiles * s + cus - 1) / cus;
      const int kt = (k_tiles + s - 1) / s;
      const double us = 5.5 + (double)rounds * kt * tile_us / (rounds > 1 ? 1.08 : 1.0) +
                        (s > 1 ? 4.0 + 2e-6 * p.M * p.N * p.batch * s : 0);
      if (s == 1 || us < best_us * 0.93) {   // split further only for a clear gain
        best_us = us;
        best = s;
      }
    }
    const int forced = tuning(kTuneSplitK);   // tuning / test override
    const bool was_forced = forced > 0 && forced <= 64 && forced <= k_tiles;
    if (was_forced) best = forced;
    const size_t slice_bytes = (size_t)p.batch * p.M * p.N * sizeof(float);
    if (best > 1 && workspace_is_fixed() && (size_t)best * slice_bytes > fixed_workspace_bytes()) {
      // a caller's fixed scratch: a slice count the caller forced is refused, the library's own choice
      // comes down to what fits (one slice needs no scratch at all). The library's own choice keeps
      // slices x tiles within the compute units and a tile within 128 x 128, so on 256 units it never
      // asks for more than 16 MiB; this is for a device with more of them.
      if (was_forced)
        return fail(kBadArgument,
                    "gemm: %d K slices of a %d x %d x %d output need %zu bytes of scratch; the static array of the "
                    "entry point that allocates nothing holds %zu",
                    best, p.batch, p.M, p.N, (size_t)best * slice_bytes, fixed_workspace_bytes());
      best = (int)(fixed_workspace_bytes() / slice_bytes);
      if (best < 2) best = 1;
    }
    if (best > 1) {
      const size_t bytes = (size_t)best * slice_bytes;
      float *ws = bytes <= (size_t(1) << 30) ? static_cast<float *>(workspace(bytes)) : nullptr;
      if (ws) {
        p.splits = best;
        p.k_per_split = ((k_tiles + best - 1) / best) * BK;
        p.ws = ws;
      }
    }
  }
  note_splits(p.splits);
  const long long grid = tiles * p.splits;
  {
    // ids resident together on one XCD: its share of the grid, at most two
    // workgroups on each of its 32 compute units
    const long long per_xcd = grid / 8 < 1 ? 1 : grid / 8;
    const double together = (double)(per_xcd < 64 ? per_xcd : 64);
    int g = (int)(sqrt(together * BN / BM) + 0.5);
    g = g < 1 ? 1 : g;
    p.group_m = g > p.tiles_m ? p.tiles_m : g;
  }
  if (grid > 0x7fffffffLL) return fail(kBadArgument, "gemm: %lld tiles exceed the grid limit", grid);
  if (T::LDS_FLOATS * sizeof(float) > 64 * 1024) {   // (also with KG groups of buffers)
    // dynamic LDS above the default limit: the attribute once per instantiation and device set-up
    static int raised = 0;
    if (raised != init_count()) {
      TFHIP_CHECK_HIP(hipFuncSetAttribute(
          reinterpret_cast<const void *>(gemm_kernel<BM, BN, BK, WAVES_M, WAVES_N, A_KIND, B_KIND, KG>),
          hipFuncAttributeMaxDynamicSharedMemorySize, (int)(T::LDS_FLOATS * sizeof(float))));
      raised = init_count();
    }
  }
  note_kernel("gemm_kernel<%d, %d, %d, %d, %d, %d, %d, %d>", BM, BN, BK, WAVES_M, WAVES_N, A_KIND, B_KIND, KG);
  // The fused epilogue covers per-column operands with a relu-family activation;
  // anything else leaves raw sums for gemm_finish.
  const Epilogue &e = p.epi;
  p.inline_epilogue = p.splits == 1 && e.channel_operands && (e.activation <= TFHIP_LEAKYRELU);
  if (p.inline_epilogue) {
    TFHIP_LAUNCH((gemm_kernel<BM, BN, BK, WAVES_M, WAVES_N, A_KIND, B_KIND, KG>
                  <<<dim3((unsigned)grid), dim3(256 * KG), T::LDS_FLOATS * sizeof(float), stream()>>>(p)));
  } else {
    const long long total = (long long)p.M * p.N * p.batch;
    long long blocks = (total + 255) / 256;
    const long long cap = (long long)num_cus() * 16;
    if (blocks > cap) blocks = cap;
    TFHIP_LAUNCH((gemm_kernel<BM, BN, BK, WAVES_M, WAVES_N, A_KIND, B_KIND, KG>
                  <<<dim3((unsigned)grid), dim3(256 * KG), T::LDS_FLOATS * sizeof(float), stream()>>>(p),
                  gemm_finish<<<dim3((unsigned)blocks), dim3(256), 0, stream()>>>(p)));
  }
  return kOk;
}

// Groups of wavefronts that share a tile and split its k loop (GemmTile's KG), for the two small
// tiles with row-major operands. Measured over BERT-base and MobileNetV2 products: two groups gain
// 5-8% when every compute unit holds at most one tile, at least half of them hold one, and k spans
// 18 tiles or more (1024 x 768 x 3072 on the 64 x 48 tile: 47.0 -> 43.9 us; on the 32 x 32 tile
// 1568 x 160 x 960: 10.5 -> 9.7 us, 1568 x 160 x 576: 9.1 -> 8.6 us with operands from memory);
// with more tiles per compute unit or a shorter k the extra barrier traffic and the final sum cost
// more than the shorter loop saves, and four groups never won. The "k_groups" tuning knob overrides
// (1, 2 or 4; 4 on the 32 x 32 tile only).
inline int choose_k_groups(int shape, const GemmParams &p, int cus) {
  const TileShape &t = kTileShapes[shape];
  const long long tiles = ((p.M + t.bm - 1) / t.bm) * ((p.N + t.bn - 1) / t.bn) * (long long)p.batch;
  const int k_tiles = (p.K + t.bk - 1) / t.bk;
  const int forced = tuning(kTuneKGroups);
  if (forced > 0) return forced >= 4 ? (shape == 12 ? 4 : 2) : (forced >= 2 ? 2 : 1);
  return (tiles <= cus && tiles * 2 >= cus && k_tiles >= 18) ? 2 : 1;   // (a handful of tiles, like a batch-32 classifier: 9.8 us with one group, 10.5 with two)
}

// Dispatch over the instantiated tile shapes for one loader combination.
template <int A_KIND, int B_KIND>
inline int launch_gemm_shape(int shape, GemmParams &p) {
  if constexpr (A_KIND == kLoadKVec && B_KIND == kLoadXVec) {
    if (shape == 10 || shape == 12) {
      const int kg = choose_k_groups(shape, p, num_cus());
      if (kg == 4) return launch_gemm<32, 32, 32, 2, 2, A_KIND, B_KIND, 4>(p);
      if (kg == 2 && shape == 10) return launch_gemm<64, 48, 32, 4, 1, A_KIND, B_KIND, 2>(p);
      if (kg == 2) return launch_gemm<32, 32, 32, 2, 2, A_KIND, B_KIND, 2>(p);
    }
  }
  switch (shape) {
    case 0: return launch_gemm<128, 128, 16, 2, 2, A_KIND, B_KIND>(p);
    case 1: return launch_gemm<128, 96, 16, 2, 2, A_KIND, B_KIND>(p);
    case 2: return launch_gemm<128, 64, 16, 2, 2, A_KIND, B_KIND>(p);
    case 3: return launch_gemm<64, 64, 16, 2, 2, A_KIND, B_KIND>(p);
    case 4: return launch_gemm<256, 32, 16, 4, 1, A_KIND, B_KIND>(p);
    case 5: return launch_gemm<256, 16, 16, 4, 1, A_KIND, B_KIND>(p);
    case 6: return launch_gemm<64, 96, 16, 2, 2, A_KIND, B_KIND>(p);
    case 7: return launch_gemm<128, 128, 32, 2, 2, A_KIND, B_KIND>(p);
    case 8: return launch_gemm<128, 96, 32, 2, 2, A_KIND, B_KIND>(p);
    case 9: return launch_gemm<64, 64, 32, 2, 2, A_KIND, B_KIND>(p);
    case 10: return launch_gemm<64, 48, 32, 4, 1, A_KIND, B_KIND>(p);
    case 11: return launch_gemm<32, 64, 32, 2, 2, A_KIND, B_KIND>(p);
    default: return launch_gemm<32, 32, 32, 2, 2, A_KIND, B_KIND>(p);
  }
}

// Plain (non-im2col) GEMM launch, defined once in gemm.hip: picks the loaders
// for row-major / transposed operands; `vec` says both operands may be fetched
// with float4 loads.
int launch_plain_gemm(GemmParams &p, bool transpose_a, bool transpose_b, bool vec);

// Fills the bias / prelu part of an Epilogue from caller strides over `rank`
// output dims (3: batch,row,col; 4: n,h,w,c) after validating them. Sets
// kChannel addressing when every operand varies along the last axis only.
inline int fill_epilogue(Epilogue &e, const char *who, const int64_t *dims, int rank, const float *bias,
                         const int64_t *bias_strides, int activation, const float *prelu,
                         const int64_t *prelu_strides, double leaky_alpha, int general_addressing) {
  if (activation < TFHIP_LINEAR || activation > TFHIP_ELU) return fail(kBadArgument, "%s: unknown activation %d", who, activation);
  if (activation == TFHIP_PRELU && prelu == nullptr) return fail(kBadArgument, "%s: prelu activation without weights", who);
  e.activation = activation;
  e.leaky_alpha = leaky_alpha;
  e.bias = nullptr;
  e.prelu = nullptr;
  bool channel_only = true;
  for (int which = 0; which < 2; ++which) {
    const float *ptr = which == 0 ? bias : (activation == TFHIP_PRELU ? prelu : nullptr);
    const int64_t *st = which == 0 ? bias_strides : prelu_strides;
    const char *name = which == 0 ? "bias" : "prelu_weights";
    if (!ptr) continue;
    if (!st) return fail(kBadArgument, "%s: %s given without strides", who, name);
    long long *dst = which == 0 ? e.bias_s : e.prelu_s;
    for (int i = 0; i < rank; ++i) {
      if (st[i] < 0) return fail(kBadArgument, "%s: negative %s stride", who, name);
      dst[i] = st[i];
      if (i < rank - 1 && st[i] != 0 && dims[i] > 1) channel_only = false;
    }
    const int64_t extent = strided_extent(dims, st, rank);
    if (!range_is_live(ptr, (size_t)extent * 4))
      return fail(kOutOfRange, "%s: operand '%s' (%lld elements) is not inside a live device buffer", who, name,
                  (long long)extent);
    if (which == 0) e.bias = ptr; else e.prelu = ptr;
  }
  e.channel_operands = channel_only ? 1 : 0;
  if (channel_only) {
    e.addressing = kChannel;
    e.bias_s[3] = bias ? bias_strides[rank - 1] : 0;
    e.prelu_s[3] = (activation == TFHIP_PRELU) ? prelu_strides[rank - 1] : 0;
  } else {
    e.addressing = general_addressing;
  }
  return kOk;
}

}  // namespace tfhip
