// A whole inverted-residual block in one kernel: 1x1 expansion (+bias, relu/relu6),
// depthwise 3x3 (+bias, relu/relu6), 1x1 projection (+bias) and, where the block
// has one, the Add of its skip connection. Only the block's input and output touch
// memory: the expanded tensor and the depthwise output (each six times the block's
// input) live in LDS, one slice of 64 channels at a time.
//
//   workgroup  = one image, `rows` output rows (all columns), 512 threads
//   per slice of 64 expanded channels ("mid" channels c0 .. c0 + 63):
//     phase X  expansion on the matrix cores: the pixels of the chunk's expanded
//              rows (rows + halo) in blocks of 16, one block per wave (its A operand,
//              16 pixels x K input channels, stays in registers for the whole
//              kernel), times the slice of the expansion's weights from LDS;
//              bias-initialised, activation, into the expanded tile E in LDS
//              (positions outside the image stay zero: the depthwise padding)
//     phase D  depthwise stage: (output pixel, four channels) items, nine 16-byte
//              reads of E each, into D in LDS, laid out as the A operand of the
//              projection (pixel-major, channel-contiguous)
//     phase P  projection on the matrix cores: D times the slice of the projection's
//              weights from LDS, accumulated in registers over the slices (k ascending
//              as in a plain GEMM over all mid channels)
//   P of slice i and X of slice i + 1 run back to back between the same two barriers
//   (two barriers per slice); the weights of the next slice travel from memory to
//   registers one phase ahead and to LDS at the end of phase D.
//   end        accumulators (started from the projection's bias) + residual -> memory
//
// Both weight matrices come TRANSPOSED (expansion [mid][in], projection [out][mid]:
// k-contiguous rows, what a lane's 16-byte fragment read wants), prepared once per
// model by tfhip_transpose2d: staging a slice is then a plain 16-byte copy.
//
// The instruction order of every stage is that of the separate kernels (gemm_kernel:
// k = 16 t + 4 g + j for the j-th instruction of k group t, bias-initialised, residual
// added last; the depthwise kernels: taps from zero by row then column, bias,
// activation), so the block has the bits of the three (four) separate launches.
#include "block_fused.h"
#include "common.h"
#include "epilogue.h"

namespace tfhip {
namespace {

typedef float float4_t __attribute__((ext_vector_type(4)));
constexpr unsigned kNoOff = 0xffffffffu;   // an offset no buffer descriptor covers: loads return 0
constexpr int kThreads = 512, kWaves = 8;
constexpr int kMaxProjUnits = 2;           // (pixel block, channel block) units of the projection per wave
constexpr int kMaxW3Vecs = 5;              // 16-byte pieces of a projection-weight slice per thread (out_c <= 160)

__device__ __forceinline__ float relu_cap(float v, float cap) {
  const float t = (v > 0.f || v != v) ? v : 0.f;     // Math.max(0, x): NaN stays, -0 becomes +0
  return t > cap ? cap : t;                          // cap = 6 for relu6, +inf for relu
}

__device__ __forceinline__ float4 load16(__amdgpu_buffer_rsrc_t rsrc, unsigned off) {
  const auto v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)off, 0, 0);
  return make_float4(__uint_as_float(v[0]), __uint_as_float(v[1]), __uint_as_float(v[2]), __uint_as_float(v[3]));
}

// S: stride of the depthwise stage. K = 16 KF input channels. Slices of CS = 64 mid channels.
// TEAM: waves that share a pixel block of the expansion and split its four channel blocks.
template <int S, int KF, int TEAM>
__global__ __launch_bounds__(kThreads) void inverted_residual_block(BlockArgs g) {
  constexpr int K = 16 * KF, KP = K + 4;
  constexpr int CS = 64, NCB = 4, PITCH = CS + 4, CQ = CS / 4;
  constexpr int W1_VECS = CS * K / 4 / kThreads;   // 16-byte pieces of an expansion-weight slice per thread
  static_assert(CS * K / 4 % kThreads == 0 && W1_VECS >= 1, "slice staging");
  extern __shared__ float lds[];
  float *tileE = lds;                                   // [erows][ecols][PITCH]
  float *tileD = tileE + g.erows * g.ecols * PITCH;     // [16 * mbp][PITCH]
  float *w1s = tileD + 16 * g.mbp * PITCH;              // [CS][KP]
  float *w3s = w1s + CS * KP;                           // [16 * nb][PITCH]
  float *b1s = w3s + 16 * g.nb * PITCH;                 // [CS]: the expansion's bias of the slice
  float *w2s = b1s + CS;                                // [10][CS]: the depthwise filter's nine taps and bias

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int grp = lane >> 4, r = lane & 15;
  const int chunk = blockIdx.x % g.chunks_h, n = blockIdx.x / g.chunks_h;
  const int oh0 = chunk * g.rows;
  const int rows = oh0 + g.rows <= g.out_h ? g.rows : g.out_h - oh0;
  const int erows = (rows - 1) * S + 3;
  const int ih0 = oh0 * S - g.pad_top, iw0 = -g.pad_left;   // image position of tile position (0, 0)
  const int ih_lo = ih0 < 0 ? 0 : ih0, ih_hi = ih0 + erows < g.in_h ? ih0 + erows : g.in_h;
  const int iw_lo = iw0 < 0 ? 0 : iw0, iw_hi = iw0 + g.ecols < g.in_w ? iw0 + g.ecols : g.in_w;
  const int wi = iw_hi > iw_lo ? iw_hi - iw_lo : 0;
  const int inside = ih_hi > ih_lo ? (ih_hi - ih_lo) * wi : 0;
  const int mbe = (inside + 15) / 16;                   // pixel blocks of the expansion (<= 8: one per wave at most)
  const int out_px = rows * g.out_w;

  const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc((void *)g.x, 0, (int)g.x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rw1 = __builtin_amdgcn_make_buffer_rsrc((void *)g.w1t, 0, (int)g.w1t_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rw3 = __builtin_amdgcn_make_buffer_rsrc((void *)g.w3t, 0, (int)g.w3t_bytes, 0x00020000);

  // ---- expansion: which pixel block and which channel blocks of a slice this wave computes.
  // `team` waves share a pixel block and split its four channel blocks.
  constexpr int CB_PER = NCB / TEAM;
  const int my_mb = wave / TEAM;
  const int cb_lo = (wave % TEAM) * CB_PER;
  const bool exp_wave = my_mb < mbe;
  unsigned a_off = kNoOff;
  int e_pos = -1;
  if (exp_wave) {
    const int m = 16 * my_mb + r;
    if (m < inside) {
      const int rr = m / wi, cc = m - rr * wi;
      const int ih = ih_lo + rr, iw = iw_lo + cc;
      a_off = (unsigned)((((long long)n * g.in_h + ih) * g.in_w + iw) * K * 4);
      e_pos = (ih - ih0) * g.ecols + (iw - iw0);
    }
  }
  float4 a_frag[KF];
#pragma unroll
  for (int t = 0; t < KF; ++t) a_frag[t] = load16(rx, a_off != kNoOff ? a_off + (16 * t + 4 * grp) * 4 : kNoOff);

  // ---- staging of the weight slices: this thread's 16-byte pieces
  float4 w1_reg[W1_VECS], w3_reg[kMaxW3Vecs], b1_reg = make_float4(0.f, 0.f, 0.f, 0.f);
  const int w3_vecs = (16 * g.nb * CQ + kThreads - 1) / kThreads;
  auto fetch_w1 = [&](int slice) __attribute__((always_inline)) {
#pragma unroll
    for (int v = 0; v < W1_VECS; ++v) {
      const int i = tid + v * kThreads;
      const int row = i / (K / 4), kq = i - row * (K / 4);
      w1_reg[v] = load16(rw1, slice < g.slices ? (unsigned)((((long long)slice * CS + row) * K + 4 * kq) * 4) : kNoOff);
    }
    if (tid < CQ && g.b1 && slice < g.slices) b1_reg = *reinterpret_cast<const float4 *>(g.b1 + slice * CS + 4 * tid);
  };
  auto store_w1 = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int v = 0; v < W1_VECS; ++v) {
      const int i = tid + v * kThreads;
      const int row = i / (K / 4), kq = i - row * (K / 4);
      *reinterpret_cast<float4 *>(w1s + row * KP + 4 * kq) = w1_reg[v];
    }
    if (tid < CQ) *reinterpret_cast<float4 *>(b1s + 4 * tid) = b1_reg;
  };
  auto fetch_w3 = [&](int slice) __attribute__((always_inline)) {
#pragma unroll
    for (int v = 0; v < kMaxW3Vecs; ++v) {
      const int i = tid + v * kThreads;
      const int row = i / CQ, q = i - row * CQ;          // row: output channel (rows past out_c read zero)
      if (v >= w3_vecs) break;
      const bool ok = row < g.n_out && slice < g.slices;
      w3_reg[v] = load16(rw3, ok ? (unsigned)((((long long)row * g.c) + slice * CS + 4 * q) * 4) : kNoOff);
    }
  };
  auto store_w3 = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int v = 0; v < kMaxW3Vecs; ++v) {
      const int i = tid + v * kThreads;
      const int row = i / CQ, q = i - row * CQ;
      if (v < w3_vecs && row < 16 * g.nb) *reinterpret_cast<float4 *>(w3s + row * PITCH + 4 * q) = w3_reg[v];
    }
  };
  fetch_w1(0);
  fetch_w3(0);

  // ---- depthwise stage: this thread's four channels of a slice, its pixels tid / 16 + 32 p. The
  // slice's filter taps and bias (ten rows of 64 floats) go through LDS like the other weights:
  // every thread needs forty of them, and fetching them from memory thread by thread costs more
  // than the stage's arithmetic.
  const int c4 = tid % CQ, px0 = tid / CQ;
  float4 w2_reg = make_float4(0.f, 0.f, 0.f, 0.f);
  auto fetch_w2 = [&](int slice) __attribute__((always_inline)) {
    if (tid < 10 * CQ && slice < g.slices) {
      const int t = tid / CQ;
      const float *src = t < 9 ? g.w2 + (long long)t * g.c : g.b2;
      w2_reg = src ? *reinterpret_cast<const float4 *>(src + slice * CS + 4 * c4) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  };
  auto store_w2 = [&]() __attribute__((always_inline)) {
    if (tid < 10 * CQ) *reinterpret_cast<float4 *>(w2s + 4 * tid) = w2_reg;
  };
  fetch_w2(0);

  // ---- projection: this wave's (pixel block, channel block) units, accumulators from the bias
  const int units_p = g.mbp * g.nb;
  const int share_p = (units_p + kWaves - 1) / kWaves;
  float4_t acc[kMaxProjUnits];
  int u_pmb[kMaxProjUnits], u_nb[kMaxProjUnits];
  bool u_on[kMaxProjUnits];
#pragma unroll
  for (int u = 0; u < kMaxProjUnits; ++u) {
    const int id = wave * share_p + u;
    u_on[u] = u < share_p && id < units_p;
    u_pmb[u] = u_on[u] ? id / g.nb : 0;
    u_nb[u] = u_on[u] ? id - u_pmb[u] * g.nb : 0;
    acc[u] = {0.f, 0.f, 0.f, 0.f};
    const int ch = 16 * u_nb[u] + 4 * grp;
    if (u_on[u] && g.b3 && ch < g.n_out) {
      const float4 b = *reinterpret_cast<const float4 *>(g.b3 + ch);
      acc[u] = {b.x, b.y, b.z, b.w};
    }
  }

  // positions of E outside the image: the zero padding of the depthwise stage (written once)
  {
    const int positions = erows * g.ecols;
    for (int p = tid; p < positions; p += kThreads) {
      const int er = p / g.ecols, ec = p - er * g.ecols;
      const int ih = ih0 + er, iw = iw0 + ec;
      if (ih < 0 || ih >= g.in_h || iw < 0 || iw >= g.in_w) {
        float4 *dst = reinterpret_cast<float4 *>(tileE + p * PITCH);
#pragma unroll
        for (int q = 0; q < CQ; ++q) dst[q] = make_float4(0.f, 0.f, 0.f, 0.f);
      }
    }
  }

  // expansion of the slice whose weights are in LDS into E: this wave's pixel block x its channel
  // blocks, as CB_PER accumulator chains that take turns in the matrix pipe
  auto expand = [&]() __attribute__((always_inline)) {
    if (!exp_wave) return;
    const float *wcol = w1s + (16 * cb_lo + r) * KP + 4 * grp;
    float4_t e[CB_PER];
#pragma unroll
    for (int c = 0; c < CB_PER; ++c) e[c] = *reinterpret_cast<const float4_t *>(b1s + 16 * (cb_lo + c) + 4 * grp);
#pragma unroll
    for (int t = 0; t < KF; ++t) {
      float4 b[CB_PER];
#pragma unroll
      for (int c = 0; c < CB_PER; ++c) b[c] = *reinterpret_cast<const float4 *>(wcol + 16 * c * KP + 16 * t);
#pragma unroll
      for (int c = 0; c < CB_PER; ++c) e[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[c].x, a_frag[t].x, e[c], 0, 0, 0);
#pragma unroll
      for (int c = 0; c < CB_PER; ++c) e[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[c].y, a_frag[t].y, e[c], 0, 0, 0);
#pragma unroll
      for (int c = 0; c < CB_PER; ++c) e[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[c].z, a_frag[t].z, e[c], 0, 0, 0);
#pragma unroll
      for (int c = 0; c < CB_PER; ++c) e[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[c].w, a_frag[t].w, e[c], 0, 0, 0);
    }
    if (e_pos >= 0) {
#pragma unroll
      for (int c = 0; c < CB_PER; ++c) {
        float4 v;
        v.x = relu_cap(e[c][0], g.cap);
        v.y = relu_cap(e[c][1], g.cap);
        v.z = relu_cap(e[c][2], g.cap);
        v.w = relu_cap(e[c][3], g.cap);
        *reinterpret_cast<float4 *>(tileE + e_pos * PITCH + 16 * (cb_lo + c) + 4 * grp) = v;
      }
    }
  };

  // prologue: slice 0's expansion weights into LDS, then its expansion
  store_w1();
  store_w2();
  lds_barrier();
  fetch_w1(1);
  fetch_w2(1);
  expand();
  lds_barrier();

  for (int slice = 0; slice < g.slices; ++slice) {
    // ---- phase D: depthwise stage of this slice, E -> D
    float4 w2q[9];
#pragma unroll
    for (int t = 0; t < 9; ++t) w2q[t] = *reinterpret_cast<const float4 *>(w2s + t * CS + 4 * c4);
    const float4 b2q = *reinterpret_cast<const float4 *>(w2s + 9 * CS + 4 * c4);
    for (int px = px0; px < out_px; px += kThreads / CQ) {
      const int o = px / g.out_w, q = px - o * g.out_w;
      const float *win = tileE + ((S * o) * g.ecols + S * q) * PITCH + 4 * c4;
      float4 e[9];
#pragma unroll
      for (int wr = 0; wr < 3; ++wr) {
#pragma unroll
        for (int wc = 0; wc < 3; ++wc) e[wr * 3 + wc] = *reinterpret_cast<const float4 *>(win + (wr * g.ecols + wc) * PITCH);
      }
      float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int t = 0; t < 9; ++t) {
        s.x = fmaf(e[t].x, w2q[t].x, s.x);
        s.y = fmaf(e[t].y, w2q[t].y, s.y);
        s.z = fmaf(e[t].z, w2q[t].z, s.z);
        s.w = fmaf(e[t].w, w2q[t].w, s.w);
      }
      float4 d;
      d.x = relu_cap(s.x + b2q.x, g.cap);
      d.y = relu_cap(s.y + b2q.y, g.cap);
      d.z = relu_cap(s.z + b2q.z, g.cap);
      d.w = relu_cap(s.w + b2q.w, g.cap);
      *reinterpret_cast<float4 *>(tileD + px * PITCH + 4 * c4) = d;
    }
    // the weight slices the next phases use (fetched a phase ago): registers -> LDS
    store_w3();
    if (slice + 1 < g.slices) store_w1();
    lds_barrier();
    store_w2();   // (phase D of this slice, its last reader, is over)
    fetch_w3(slice + 1);
    fetch_w1(slice + 2);
    fetch_w2(slice + 2);

    // ---- phase P: projection of this slice, D x w3 slice -> accumulators
#pragma unroll
    for (int u = 0; u < kMaxProjUnits; ++u) {
      if (!u_on[u]) continue;
      const float *arow = tileD + (16 * u_pmb[u] + r) * PITCH + 4 * grp;
      const float *brow = w3s + (16 * u_nb[u] + r) * PITCH + 4 * grp;
#pragma unroll
      for (int t = 0; t < NCB; ++t) {
        const float4 a = *reinterpret_cast<const float4 *>(arow + 16 * t);
        const float4 b = *reinterpret_cast<const float4 *>(brow + 16 * t);
        acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(b.x, a.x, acc[u], 0, 0, 0);
        acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(b.y, a.y, acc[u], 0, 0, 0);
        acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(b.z, a.z, acc[u], 0, 0, 0);
        acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(b.w, a.w, acc[u], 0, 0, 0);
      }
    }
    // ---- phase X: expansion of the next slice
    if (slice + 1 < g.slices) expand();
    lds_barrier();
  }

  // ---- accumulators (+ residual) -> memory: the lane holds pixel r of its pixel block,
  // output channels 16 nb + 4 grp .. +3
#pragma unroll
  for (int u = 0; u < kMaxProjUnits; ++u) {
    if (!u_on[u]) continue;
    const int px = 16 * u_pmb[u] + r, ch = 16 * u_nb[u] + 4 * grp;
    if (px >= out_px || ch >= g.n_out) continue;
    const int o = px / g.out_w, q = px - o * g.out_w;
    const long long at = (((long long)n * g.out_h + oh0 + o) * g.out_w + q) * g.n_out + ch;
    float4 out = make_float4(acc[u][0], acc[u][1], acc[u][2], acc[u][3]);
    if (g.res) {
      const float4 r4 = *reinterpret_cast<const float4 *>(g.res + at);
      out.x += r4.x; out.y += r4.y; out.z += r4.z; out.w += r4.w;
    }
    *reinterpret_cast<float4 *>(g.y + at) = out;
  }
}

template <int S, int KF, int TEAM>
int launch_block(const BlockArgs &g, size_t lds_bytes) {
  static int raised = 0;
  if (raised != init_count()) {
    TFHIP_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(inverted_residual_block<S, KF, TEAM>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    raised = init_count();
  }
  note_kernel("inverted_residual_block<%d, %d, %d>", S, KF, TEAM);
  TFHIP_LAUNCH((inverted_residual_block<S, KF, TEAM><<<dim3((unsigned)(g.batch * g.chunks_h)), dim3(kThreads), lds_bytes, stream()>>>(g)));
  return kOk;
}

template <int S, int KF>
int launch_block_team(const BlockArgs &g, size_t lds_bytes) {
  switch (g.team) {
    case 1: return launch_block<S, KF, 1>(g, lds_bytes);
    case 2: return launch_block<S, KF, 2>(g, lds_bytes);
    default: return launch_block<S, KF, 4>(g, lds_bytes);
  }
}

template <int S>
int launch_block_k(const BlockArgs &g, size_t lds_bytes) {
  switch (g.cin) {
    case 32: return launch_block_team<S, 2>(g, lds_bytes);
    case 64: return launch_block_team<S, 4>(g, lds_bytes);
    case 96: return launch_block_team<S, 6>(g, lds_bytes);
    default: return launch_block_team<S, 10>(g, lds_bytes);
  }
}

}  // namespace

// Tiling: as many output rows per workgroup as keep (a) the expansion's pixels within eight
// blocks of 16 (one per wave), (b) the projection's units within two per wave, (c) LDS within a
// compute unit's, and (d) at least three workgroups for every four compute units (none of the
// four when nothing else fits).
bool plan_block(BlockArgs &g, size_t *lds_bytes) {
  const bool k_ok = g.cin == 32 || g.cin == 64 || g.cin == 96 || g.cin == 160;
  if (!k_ok || g.c % 64 != 0 || g.n_out % 4 != 0 || g.n_out > 160 || (g.stride != 1 && g.stride != 2)) return false;
  if (g.out_h <= 0 || g.out_w <= 0 || g.batch <= 0) return false;
  g.slices = g.c / 64;
  g.nb = (g.n_out + 15) / 16;
  g.ecols = (g.out_w - 1) * g.stride + 3;
  const int in_cols = g.ecols < g.in_w + 2 ? g.ecols : g.in_w + 2;   // (an upper bound of the columns inside the image)
  const int forced = tuning(kTuneBlockRows);
  int best = 0;
  for (int rows = 1; rows <= g.out_h; ++rows) {
    if (forced > 0 && rows != (forced > g.out_h ? g.out_h : forced)) continue;
    const int erows = (rows - 1) * g.stride + 3;
    const int inside_max = erows * (in_cols < g.in_w ? in_cols : g.in_w);
    const int mbe = (inside_max + 15) / 16, mbp = (rows * g.out_w + 15) / 16;
    if (mbe > 8 || (mbp * g.nb + 7) / 8 > 2) break;
    const size_t bytes = ((size_t)erows * g.ecols * 68 + (size_t)16 * mbp * 68 + (size_t)64 * (g.cin + 4) + (size_t)16 * g.nb * 68 + 64 + 640) * 4;
    if (bytes > 156 * 1024) break;
    const long long wgs = (long long)g.batch * ((g.out_h + rows - 1) / rows);
    if (best == 0 || forced > 0 || wgs * 4 >= 3LL * num_cus()) best = rows;
  }
  if (best == 0) return false;
  g.rows = best;
  g.chunks_h = (g.out_h + best - 1) / best;
  g.erows = (best - 1) * g.stride + 3;
  const int inside_max = g.erows * (in_cols < g.in_w ? in_cols : g.in_w);
  const int mbe = (inside_max + 15) / 16;
  g.mbp = (best * g.out_w + 15) / 16;
  g.team = mbe <= 2 ? 4 : (mbe <= 4 ? 2 : 1);
  *lds_bytes = ((size_t)g.erows * g.ecols * 68 + (size_t)16 * g.mbp * 68 + (size_t)64 * (g.cin + 4) + (size_t)16 * g.nb * 68 + 64 + 640) * 4;
  return true;
}

int launch_block_kernel(const BlockArgs &g, size_t lds_bytes) {
  if ((long long)g.batch * g.chunks_h > 0x7fffffffLL) return fail(kBadArgument, "tfhip_fused_inverted_residual: grid too large");
  return g.stride == 1 ? launch_block_k<1>(g, lds_bytes) : launch_block_k<2>(g, lds_bytes);
}

}  // namespace tfhip

using namespace tfhip;

namespace {

int fill_block_args(BlockArgs &g, const float *x, const float *pw_filter_t, const float *pw_bias, int activation,
                    const float *dw_filter, const float *dw_bias, const float *proj_filter_t, const float *proj_bias,
                    const float *residual, float *y, int64_t batch, int64_t in_h, int64_t in_w, int64_t in_c,
                    int64_t mid_c, int64_t out_c, int64_t stride, int64_t pad_top, int64_t pad_left, int64_t out_h,
                    int64_t out_w) {
  g = {};
  g.x = x; g.w1t = pw_filter_t; g.b1 = pw_bias; g.w2 = dw_filter; g.b2 = dw_bias; g.w3t = proj_filter_t; g.b3 = proj_bias;
  g.res = residual; g.y = y;
  g.batch = (int)batch; g.in_h = (int)in_h; g.in_w = (int)in_w; g.cin = (int)in_c; g.c = (int)mid_c; g.n_out = (int)out_c;
  g.stride = (int)stride; g.pad_top = (int)pad_top; g.pad_left = (int)pad_left; g.out_h = (int)out_h; g.out_w = (int)out_w;
  g.cap = activation == TFHIP_RELU6 ? 6.f : __builtin_inff();
  g.x_bytes = (unsigned)(batch * in_h * in_w * in_c * 4);
  g.w1t_bytes = (unsigned)(mid_c * in_c * 4);
  g.w3t_bytes = (unsigned)(out_c * mid_c * 4);
  return kOk;
}

bool dims_in_range(int64_t batch, int64_t in_h, int64_t in_w, int64_t in_c, int64_t mid_c, int64_t out_c, int64_t stride,
                   int64_t pad_top, int64_t pad_left, int64_t out_h, int64_t out_w) {
  const int64_t lim = 0x7fffffff;
  return batch >= 0 && in_h > 0 && in_w > 0 && in_c > 0 && mid_c > 0 && out_c > 0 && stride > 0 && out_h >= 0 && out_w >= 0 &&
         pad_top >= 0 && pad_left >= 0 && pad_top < lim && pad_left < lim && in_c <= 4096 && mid_c <= 65536 && out_c <= 4096 &&
         in_h < lim && in_w < lim && out_h < lim && out_w < lim && batch < lim &&
         product_below(0x40000000LL, {batch, in_h, in_w, in_c}) && product_below(lim, {batch, out_h, out_w, out_c}) &&
         product_below(lim, {batch, out_h, out_w, mid_c});
}

}  // namespace

extern "C" int tfhip_fused_inverted_residual(const float *x, const float *pw_filter_t, const float *pw_bias, int activation,
                                             const float *dw_filter, const float *dw_bias, const float *proj_filter_t,
                                             const float *proj_bias, const float *residual, float *y, int64_t batch,
                                             int64_t in_h, int64_t in_w, int64_t in_c, int64_t mid_c, int64_t out_c,
                                             int64_t stride, int64_t pad_top, int64_t pad_left, int64_t out_h,
                                             int64_t out_w) {
  TFHIP_REQUIRE_INIT();
  TFHIP_CHECK_ARG(dims_in_range(batch, in_h, in_w, in_c, mid_c, out_c, stride, pad_top, pad_left, out_h, out_w),
                  "tfhip_fused_inverted_residual: bad dimension");
  TFHIP_CHECK_ARG(activation == TFHIP_RELU || activation == TFHIP_RELU6,
                  "tfhip_fused_inverted_residual: the expansion and the depthwise stage share relu or relu6; run the "
                  "three convolutions for any other activation");
  if (batch * out_h * out_w == 0) return kOk;
  TFHIP_CHECK_RANGE(x, batch * in_h * in_w * in_c, 4, "x");
  TFHIP_CHECK_RANGE(pw_filter_t, mid_c * in_c, 4, "pw_filter_t");
  TFHIP_CHECK_RANGE(dw_filter, 9 * mid_c, 4, "dw_filter");
  TFHIP_CHECK_RANGE(proj_filter_t, out_c * mid_c, 4, "proj_filter_t");
  if (pw_bias) TFHIP_CHECK_RANGE(pw_bias, mid_c, 4, "pw_bias");
  if (dw_bias) TFHIP_CHECK_RANGE(dw_bias, mid_c, 4, "dw_bias");
  if (proj_bias) TFHIP_CHECK_RANGE(proj_bias, out_c, 4, "proj_bias");
  TFHIP_CHECK_OUTPUT(y, batch * out_h * out_w * out_c, 4, "y");
  if (residual) {
    TFHIP_CHECK_RANGE(residual, batch * out_h * out_w * out_c, 4, "residual");
    TFHIP_CHECK_ARG(residual != y, "tfhip_fused_inverted_residual: residual and y are the same buffer");
  }
  if (window_can_miss(in_h, out_h, stride, pad_top, 3, 1) || window_can_miss(in_w, out_w, stride, pad_left, 3, 1)) {
    bool refuse = false;
    const int rc = refuse_nonfinite_filter(dw_filter, 9 * mid_c, "tfhip_fused_inverted_residual", &refuse);
    if (rc != kOk) return rc;
    if (refuse) return fail(kBadArgument, "tfhip_fused_inverted_residual: %s", kNonfiniteFilterMessage);
  }
  const float *ptrs[] = {x, pw_filter_t, pw_bias, dw_filter, dw_bias, proj_filter_t, proj_bias, residual, y};
  bool aligned = true;
  for (const float *p : ptrs) aligned = aligned && reinterpret_cast<uintptr_t>(p) % 16 == 0;
  BlockArgs g;
  fill_block_args(g, x, pw_filter_t, pw_bias, activation, dw_filter, dw_bias, proj_filter_t, proj_bias, residual, y, batch,
                  in_h, in_w, in_c, mid_c, out_c, stride, pad_top, pad_left, out_h, out_w);
  size_t lds_bytes = 0;
  if (!aligned || !plan_block(g, &lds_bytes)) {
    return fail(kBadArgument,
                "tfhip_fused_inverted_residual: form not taken by the block kernel (in_c 32/64/96/160, mid_c a multiple "
                "of 64, out_c a multiple of 4 up to 160, stride 1 or 2, a map narrow enough for a row of it to fit the "
                "kernel's tile, 16-byte aligned operands); run the three convolutions");
  }
  return launch_block_kernel(g, lds_bytes);
}

// 1 when tfhip_fused_inverted_residual takes the shape and is expected to beat the separate
// kernels: enough workgroups to occupy the chip, and not the smallest maps, where every row
// chunk would recompute most of the expansion for its halo.
extern "C" int tfhip_inverted_residual_pays(int64_t batch, int64_t in_h, int64_t in_w, int64_t in_c, int64_t mid_c,
                                            int64_t out_c, int64_t stride, int64_t out_h, int64_t out_w) {
  if (!initialised() || !dims_in_range(batch, in_h, in_w, in_c, mid_c, out_c, stride, 0, 0, out_h, out_w) || batch == 0 ||
      out_h == 0 || out_w == 0) {
    return 0;
  }
  BlockArgs g;
  fill_block_args(g, nullptr, nullptr, nullptr, TFHIP_RELU6, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, batch,
                  in_h, in_w, in_c, mid_c, out_c, stride, 0, 0, out_h, out_w);
  size_t lds_bytes = 0;
  if (!plan_block(g, &lds_bytes)) return 0;
  if (tuning(kTuneFuseBlock) >= 0) return tuning(kTuneFuseBlock) > 0 ? 1 : 0;   // knob: always / never
  // Measured at batch 32 in sequence against the channel-sliced pointwise + depthwise kernel followed
  // by the projection GEMM: 14x14, 64 -> 384 -> 64: 20.5 us against 13-15 + 9; 28x28, 32 -> 192 -> 32:
  // 25 against 16-19 + 10; 14x14, 96 -> 576 -> 96: 38 against 21-23 + 14. One workgroup per compute
  // unit runs its phases (weights in, matrix cores, depthwise arithmetic) one after the other, and
  // the halo rows double the expansion's work, so the block kernel only draws level where it is
  // best: never chosen by default.
  return 0;
}
