// Host-side helpers shared by the matmul and conv entry points: tile-shape
// choice and the launch of one gemm_kernel instantiation.
#pragma once

#include <stdlib.h>

#include "common.h"
#include "gemm_kernel.h"

namespace tfhip {

struct TileShape {
  int bm, bn, bk;
  double quality;  // relative speed of a full tile of this shape
};

// Shapes instantiated for every loader combination.
static const TileShape kTileShapes[] = {
    {128, 128, 16, 1.00}, {128, 96, 16, 0.97}, {128, 64, 16, 0.90}, {64, 64, 16, 0.78},  {256, 32, 16, 0.80},
    {256, 16, 16, 0.60},  {64, 96, 16, 0.85},  {128, 128, 32, 1.02}, {128, 96, 32, 0.99}, {64, 64, 32, 0.80},
};
constexpr int kNumTileShapes = 10;

// Picks the shape with the best estimated throughput for an M x N output
// repeated `batch` times on `cus` compute units: useful fraction of the padded
// tiles, times the fill of the last round of workgroups, times tile quality.
// TFHIP_TILE=<index> in the environment overrides the choice (tuning aid).
inline int choose_tile_shape(long long M, long long N, long long K, long long batch, int cus) {
  static const int forced = [] {
    const char *e = getenv("TFHIP_TILE");
    return e ? atoi(e) : -1;
  }();
  if (forced >= 0 && forced < kNumTileShapes) return forced;
  int best = 0;
  double best_score = -1.0;
  for (int i = 0; i < kNumTileShapes; ++i) {
    const TileShape &t = kTileShapes[i];
    const long long tm = (M + t.bm - 1) / t.bm, tn = (N + t.bn - 1) / t.bn;
    const long long kp = (K + t.bk - 1) / t.bk * t.bk;
    const double useful = (double)(M * N) / (double)(tm * t.bm * tn * t.bn) * ((double)(K > 0 ? K : 1) / (double)(kp > 0 ? kp : 1));
    const long long tiles = tm * tn * batch;
    const long long rounds = (tiles + cus - 1) / cus;
    const double fill = (double)tiles / (double)(rounds * cus);
    const double score = useful * fill * t.quality;
    if (score > best_score) {
      best_score = score;
      best = i;
    }
  }
  return best;
}

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int A_KIND, int B_KIND>
inline int launch_gemm(GemmParams &p) {
  using T = GemmTile<BM, BN, BK, WAVES_M, WAVES_N, A_KIND, B_KIND>;
  p.tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  const long long grid = (long long)p.tiles_m * p.tiles_n * p.batch;
  if (grid <= 0) return kOk;
  if (grid > 0x7fffffffLL) return fail(kBadArgument, "gemm: %lld tiles exceed the grid limit", grid);
  note_kernel("gemm_kernel<%d, %d, %d, %d, %d, %d, %d>", BM, BN, BK, WAVES_M, WAVES_N, A_KIND, B_KIND);
  TFHIP_LAUNCH((gemm_kernel<BM, BN, BK, WAVES_M, WAVES_N, A_KIND, B_KIND>
                <<<dim3((unsigned)grid), dim3(256), T::LDS_FLOATS * sizeof(float), stream()>>>(p)));
  return kOk;
}

// Dispatch over the instantiated tile shapes for one loader combination.
template <int A_KIND, int B_KIND>
inline int launch_gemm_shape(int shape, GemmParams &p) {
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
    default: return launch_gemm<64, 64, 32, 2, 2, A_KIND, B_KIND>(p);
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
