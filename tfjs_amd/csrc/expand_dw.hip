// Pointwise (1x1) convolution + depthwise 3x3 convolution in one kernel: the
// expansion and the depthwise stage of an inverted-residual block.
//
// Run as two kernels, the expanded tensor - the largest of the whole network -
// is written to memory by the first and read back by the second. Here a
// workgroup produces a tile of the expanded tensor row by row into a ring of
// rows in LDS (matrix cores, the operand layout and instruction order of
// skinny_gemm_regs, so the same bits), and the depthwise stage reads its 3x3
// windows from that ring (the multiply-add order of depthwise_3x3_rows: taps
// by row then column from zero, then the bias, then the activation): only the
// block's input and the depthwise output touch memory.
//
//   workgroup  = one image, `rows` output rows, `tile_w` output columns, all channels
//   ring       = 3 + S expanded rows of ecols = 16 * pblocks pixels (tile + halo),
//                pixel pitch c + 4 floats (16-byte accesses of a wave then spread
//                over all banks)
//   step o     = depthwise output row o from ring rows S o .. S o + 2, and the S
//                expanded rows the next step needs into the free ring slots; one
//                barrier per step
//   expansion  = tasks of 16 pixels x 16 channels dealt to the four waves in turn:
//                A (16 pixels x K input channels) comes from memory as one 16-byte
//                (+ one 8-byte) load per lane, issued a step ahead; the weights
//                come from LDS, transposed so that a lane's four k values are one
//                16-byte read
//   padding    = positions of the expanded tensor outside the image are zero (what
//                the depthwise stage pads with), not activation(bias)
#include "common.h"
#include "epilogue.h"
#include "expand_dw_stream.h"
#include "expand_dw_tile.h"

namespace tfhip {
namespace {

typedef float float4_t __attribute__((ext_vector_type(4)));
constexpr unsigned kNoOff = 0xffffffffu;   // an offset no buffer descriptor covers: loads return 0

struct ExpandDwArgs {
  const float *x, *w1, *b1, *w2, *b2;
  float *y;
  int batch, in_h, in_w, cin, c;   // x [batch, in_h, in_w, cin]; expanded [batch, in_h, in_w, c]
  int pad_top, pad_left, out_h, out_w;
  int act1, act2;                  // both relu or both relu6
  int tile_w, tiles_w, rows, chunks_h, pblocks, pitch;
  unsigned x_bytes;
  // first stage a convolution over few input channels instead of a 1x1 one (TAPS > 0): x is
  // [batch, xh, xw, xc], the "expanded" tensor [batch, in_h, in_w, c] is its output
  int xh, xw, xc, conv_stride, conv_pad_top, conv_pad_left, k;
};

template <int ACT>
__device__ __forceinline__ float relu_like(float v) {
  const float t = (v > 0.f || v != v) ? v : 0.f;     // Math.max(0, x): NaN stays, -0 becomes +0
  return (ACT == TFHIP_RELU6 && t > 6.f) ? 6.f : t;
}

constexpr int kMaxPasses = 4;   // depthwise pixels per lane and step

// S: stride of the depthwise stage. K = 16 KF + (HALF ? 8 : 0) input channels.
// ACT: the activation of both stages, relu or relu6.
// TAPS > 0: the first stage is a convolution of at most 4 TAPS taps (filter height x width x
// input channels, a network stem) gathered element by element with the lane layout and
// instruction order of conv_few_taps (lane (grp, r) feeds tap 4 t + grp in k step t); KF and
// HALF are then unused.
template <int S, int KF, bool HALF, int ACT, int TAPS>
__global__ __launch_bounds__(256) void expand_dw_3x3(ExpandDwArgs g, StemTaps taps) {
  constexpr int K = TAPS > 0 ? 4 * TAPS : 16 * KF + (HALF ? 8 : 0);   // k extent of the weights in LDS
  constexpr int KP = K + 4;             // floats per column of the transposed weights in LDS
  constexpr int RING = 3 + S;
  extern __shared__ float lds[];
  const int ecols = 16 * g.pblocks;
  const int row_floats = ecols * g.pitch;
  float *ring = lds;                                  // [RING][ecols][pitch]
  float *w1t = ring + RING * row_floats;              // [c][KP]
  float *b1s = w1t + g.c * KP;                        // [c]

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int grp = lane >> 4, r = lane & 15;
  int rem = blockIdx.x;
  const int tw = rem % g.tiles_w;
  rem /= g.tiles_w;
  const int chunk = rem % g.chunks_h;
  const int n = rem / g.chunks_h;
  const int oh0 = chunk * g.rows, ow0 = tw * g.tile_w;
  const int ih0 = oh0 * S - g.pad_top, iw0 = ow0 * S - g.pad_left;   // image position of expanded (0, 0)
  const int rows = oh0 + g.rows <= g.out_h ? g.rows : g.out_h - oh0;
  const int cblocks = g.c / 16;
  const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc((void *)g.x, 0, (int)g.x_bytes, 0x00020000);

  // weights of the expansion, transposed, and its bias: 16-byte loads along the channels, eight of
  // a lane in flight at once (the fill is a memory round trip per batch of loads, paid by every
  // workgroup before its first matrix instruction)
  if (TAPS > 0) {   // rows beyond the filter's taps multiply zeros
    for (int i = threadIdx.x; i < g.c * KP; i += 256) w1t[i] = 0.f;
    __syncthreads();
  }
  {
    const int quads = g.c / 4, total = quads * (TAPS > 0 ? g.k : K);   // w1 is [K][c]
    for (int i0 = threadIdx.x; i0 < total; i0 += 256 * 8) {
      float4 v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int i = i0 + u * 256;
        v[u] = *reinterpret_cast<const float4 *>(g.w1 + 4 * (i < total ? i : total - 1));
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int i = i0 + u * 256;
        if (i < total) {
          const int k = i / quads, col = 4 * (i - k * quads);
          w1t[(col + 0) * KP + k] = v[u].x;
          w1t[(col + 1) * KP + k] = v[u].y;
          w1t[(col + 2) * KP + k] = v[u].z;
          w1t[(col + 3) * KP + k] = v[u].w;
        }
      }
    }
  }
  for (int i = threadIdx.x; i < g.c; i += 256) b1s[i] = g.b1 ? g.b1[i] : 0.f;

  // depthwise stage: this lane's four channels and its pixels of a row
  const int cq = g.c / 4, groups = 256 / cq;
  const int c4 = (int)threadIdx.x % cq, pxg = (int)threadIdx.x / cq;
  const bool dw_lane = pxg < groups;
  float4 w2q[9], b2q = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (int t = 0; t < 9; ++t) {
    w2q[t] = dw_lane ? *reinterpret_cast<const float4 *>(g.w2 + (long long)t * g.c + 4 * c4) : b2q;
  }
  if (dw_lane && g.b2) b2q = *reinterpret_cast<const float4 *>(g.b2 + 4 * c4);

  // Expansion work of one step: S expanded rows x pblocks blocks of 16 pixels ("row blocks"), each
  // with c / 16 blocks of 16 channels. The (row block, channel block) pairs are cut into four
  // contiguous shares, one per wave: a share spans at most two row blocks, and all its channel
  // blocks of one row block use the same 16 pixels x K inputs (one load per lane).
  const int per_step = S * g.pblocks * cblocks;
  const int share = (per_step + 3) / 4;
  const int t_lo = wave * share < per_step ? wave * share : per_step;
  const int t_hi = t_lo + share < per_step ? t_lo + share : per_step;
  const int rb0 = t_lo / cblocks;
  const int cb0_lo = t_lo - rb0 * cblocks;
  const int end0 = t_hi < (rb0 + 1) * cblocks ? t_hi : (rb0 + 1) * cblocks;
  const int cb0_hi = end0 - rb0 * cblocks;           // first row block: channel blocks [cb0_lo, cb0_hi)
  const int cb1_hi = t_hi - end0;                     // second row block: channel blocks [0, cb1_hi)
  const int row0 = rb0 / g.pblocks, pb0 = rb0 - row0 * g.pblocks;
  const int row1 = (rb0 + 1) / g.pblocks, pb1 = (rb0 + 1) - row1 * g.pblocks;

  struct AFrag {
    float4 full[KF > 0 ? KF : 1];
    float2 half;
    float tap[TAPS > 0 ? TAPS : 1];
  };
  int tap_dh[TAPS > 0 ? TAPS : 1], tap_dw[TAPS > 0 ? TAPS : 1];
  unsigned tap_off[TAPS > 0 ? TAPS : 1];
  if (TAPS > 0) {
#pragma unroll
    for (int t = 0; t < TAPS; ++t) {
      tap_dh[t] = taps.dh[4 * t + grp];
      tap_dw[t] = taps.dw[4 * t + grp];
      tap_off[t] = taps.off_bytes[4 * t + grp];
    }
  }
  auto load_a = [&](AFrag &a, int erow, int pb) __attribute__((always_inline)) {
    const int ih = ih0 + erow, iw = iw0 + 16 * pb + r;
    const bool inside = ih >= 0 && ih < g.in_h && iw >= 0 && iw < g.in_w;
    if (TAPS > 0) {
      // the window of first-stage output pixel (ih, iw); its top-left element may lie before
      // the image, the sum with an inside tap's offset is exact modulo 2^32
      const int xh0 = ih * g.conv_stride - g.conv_pad_top, xw0 = iw * g.conv_stride - g.conv_pad_left;
      const unsigned base = (unsigned)((((long long)n * g.xh + xh0) * g.xw + xw0) * g.xc * 4);
#pragma unroll
      for (int t = 0; t < TAPS; ++t) {
        const bool ok = inside && (unsigned)(xh0 + tap_dh[t]) < (unsigned)g.xh && (unsigned)(xw0 + tap_dw[t]) < (unsigned)g.xw;
        a.tap[t] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rx, (int)(ok ? base + tap_off[t] : kNoOff), 0, 0));
      }
      return;
    }
    const unsigned base = (unsigned)((((long long)n * g.in_h + ih) * g.in_w + iw) * (16 * KF + (HALF ? 8 : 0)) * 4);
#pragma unroll
    for (int t = 0; t < KF; ++t) {
      const auto v = __builtin_amdgcn_raw_buffer_load_b128(rx, (int)(inside ? base + (16 * t + 4 * grp) * 4 : kNoOff), 0, 0);
      a.full[t] = make_float4(__uint_as_float(v[0]), __uint_as_float(v[1]), __uint_as_float(v[2]), __uint_as_float(v[3]));
    }
    if (HALF) {
      const auto v = __builtin_amdgcn_raw_buffer_load_b64(rx, (int)(inside ? base + (16 * KF + 2 * grp) * 4 : kNoOff), 0, 0);
      a.half = make_float2(__uint_as_float(v[0]), __uint_as_float(v[1]));
    }
  };
  // channel blocks [cb_lo, cb_hi) of the row block (erow, pb) into ring slot `slot`
  auto expand_blocks = [&](const AFrag &a, int erow, int slot, int pb, int cb_lo, int cb_hi) __attribute__((always_inline)) {
    const int ih = ih0 + erow, iw = iw0 + 16 * pb + r;
    const bool inside = ih >= 0 && ih < g.in_h && iw >= 0 && iw < g.in_w;
    float *dst = ring + slot * row_floats + (16 * pb + r) * g.pitch + 4 * grp;
    const float *wcol = w1t + r * KP + 4 * grp;
    const float *bias = b1s + 4 * grp;
    for (int cb = cb_lo; cb < cb_hi; ++cb) {
      float4_t acc = *reinterpret_cast<const float4_t *>(bias + 16 * cb);
      if (TAPS > 0) {
#pragma unroll
        for (int t = 0; t < TAPS; ++t) {
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w1t[(16 * cb + r) * KP + 4 * t + grp], a.tap[t], acc, 0, 0, 0);
        }
      }
#pragma unroll
      for (int t = 0; t < (TAPS > 0 ? 0 : KF); ++t) {
        const float4 b = *reinterpret_cast<const float4 *>(wcol + 16 * cb * KP + 16 * t);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(b.x, a.full[t].x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(b.y, a.full[t].y, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(b.z, a.full[t].z, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(b.w, a.full[t].w, acc, 0, 0, 0);
      }
      if (HALF && TAPS == 0) {
        const float2 b = *reinterpret_cast<const float2 *>(w1t + (16 * cb + r) * KP + 16 * KF + 2 * grp);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(b.x, a.half.x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(b.y, a.half.y, acc, 0, 0, 0);
      }
      // the lane holds pixel 16 pb + r, channels 16 cb + 4 grp .. +3; outside the image the
      // expanded tensor is the zero padding of the depthwise stage
      float4 e;
      e.x = inside ? relu_like<ACT>(acc[0]) : 0.f;
      e.y = inside ? relu_like<ACT>(acc[1]) : 0.f;
      e.z = inside ? relu_like<ACT>(acc[2]) : 0.f;
      e.w = inside ? relu_like<ACT>(acc[3]) : 0.f;
      *reinterpret_cast<float4 *>(dst + 16 * cb) = e;
    }
  };
  // this wave's share of expanded rows first .. first + S - 1 (only those below first + nrows), whose
  // first row goes to ring slot `slot`
  AFrag a0, a1;
  auto issue_rows = [&](int first, int nrows) __attribute__((always_inline)) {
    if (cb0_hi > cb0_lo && row0 < nrows) load_a(a0, first + row0, pb0);
    if (cb1_hi > 0 && row1 < nrows) load_a(a1, first + row1, pb1);
  };
  auto expand_rows = [&](int first, int nrows, int slot) __attribute__((always_inline)) {
    if (cb0_hi > cb0_lo && row0 < nrows) {
      const int s0 = slot + row0 >= RING ? slot + row0 - RING : slot + row0;
      expand_blocks(a0, first + row0, s0, pb0, cb0_lo, cb0_hi);
    }
    if (cb1_hi > 0 && row1 < nrows) {
      const int s1 = slot + row1 >= RING ? slot + row1 - RING : slot + row1;
      expand_blocks(a1, first + row1, s1, pb1, 0, cb1_hi);
    }
  };

  // prologue: expanded rows 0, 1, 2
  __syncthreads();   // w1t, b1s
#pragma unroll
  for (int first = 0; first < 3; first += S) {
    const int nrows = 3 - first < S ? 3 - first : S;
    issue_rows(first, nrows);
    expand_rows(first, nrows, first);
  }
  lds_barrier();

  int slot0 = 0;            // ring slot of expanded row S o
  int new_slot = 3 % RING;  // ring slot of expanded row S o + 3
  for (int o = 0; o < rows; ++o) {
    // the rows the next step reads: S o + 3 .. S o + 2 + S (none after the last step)
    const bool more = o + 1 < rows;
    const int first = S * o + 3;
    if (more) issue_rows(first, S);
    // depthwise output row o
    const int oh = oh0 + o;
    if (dw_lane) {
#pragma unroll
      for (int pass = 0; pass < kMaxPasses; ++pass) {
        const int q = pxg + pass * groups;
        if (q >= g.tile_w || ow0 + q >= g.out_w) break;
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int wr = 0; wr < 3; ++wr) {
          const int slot = slot0 + wr >= RING ? slot0 + wr - RING : slot0 + wr;
          const float *erow = ring + slot * row_floats + (S * q) * g.pitch + 4 * c4;
#pragma unroll
          for (int wc = 0; wc < 3; ++wc) {
            const float4 e = *reinterpret_cast<const float4 *>(erow + wc * g.pitch);
            const float4 w = w2q[wr * 3 + wc];
            acc.x = fmaf(e.x, w.x, acc.x);
            acc.y = fmaf(e.y, w.y, acc.y);
            acc.z = fmaf(e.z, w.z, acc.z);
            acc.w = fmaf(e.w, w.w, acc.w);
          }
        }
        float4 out;
        out.x = relu_like<ACT>(acc.x + b2q.x);
        out.y = relu_like<ACT>(acc.y + b2q.y);
        out.z = relu_like<ACT>(acc.z + b2q.z);
        out.w = relu_like<ACT>(acc.w + b2q.w);
        store_result4(g.y + (((long long)n * g.out_h + oh) * g.out_w + ow0 + q) * g.c + 4 * c4, out);
      }
    }
    if (more) expand_rows(first, S, new_slot);
    slot0 = slot0 + S >= RING ? slot0 + S - RING : slot0 + S;
    new_slot = new_slot + S >= RING ? new_slot + S - RING : new_slot + S;
    lds_barrier();   // the ring lives in LDS alone: no wait for the stores of the output row
  }
}

template <int S, int KF, bool HALF, int ACT, int TAPS>
int launch_expand_dw_act(const ExpandDwArgs &g, const StemTaps &taps, size_t lds_bytes) {
  // dynamic LDS above the default limit needs the attribute once per instantiation and device set-up
  static int raised = 0;
  if (raised != init_count()) {
    TFHIP_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(expand_dw_3x3<S, KF, HALF, ACT, TAPS>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    raised = init_count();
  }
  const long long wgs = (long long)g.batch * g.chunks_h * g.tiles_w;
  note_kernel("expand_dw_3x3<%d, %d, %s, %d, %d>", S, KF, HALF ? "true" : "false", ACT, TAPS);
  TFHIP_LAUNCH((expand_dw_3x3<S, KF, HALF, ACT, TAPS><<<dim3((unsigned)wgs), dim3(256), lds_bytes, stream()>>>(g, taps)));
  return kOk;
}

template <int S, int KF, bool HALF>
int launch_expand_dw(const ExpandDwArgs &g, size_t lds_bytes) {
  const StemTaps none = {};
  if (g.act1 == TFHIP_RELU6) return launch_expand_dw_act<S, KF, HALF, TFHIP_RELU6, 0>(g, none, lds_bytes);
  return launch_expand_dw_act<S, KF, HALF, TFHIP_RELU, 0>(g, none, lds_bytes);
}

template <int S, int TAPS>
int launch_stem_dw(const ExpandDwArgs &g, const StemTaps &taps, size_t lds_bytes) {
  if (g.act1 == TFHIP_RELU6) return launch_expand_dw_act<S, 0, false, TFHIP_RELU6, TAPS>(g, taps, lds_bytes);
  return launch_expand_dw_act<S, 0, false, TFHIP_RELU, TAPS>(g, taps, lds_bytes);
}

}  // namespace

// Fills the tiling of `g` for the fused kernel; false when the shape is one it does not take.
// K: the k extent of the first stage's weights in LDS (input channels of a 1x1 first stage, 4 x k
// steps of a few-channel convolution).
bool plan_expand_dw(ExpandDwArgs &g, int stride, int K, size_t *lds_bytes) {
  if (g.c % 16 != 0 || g.c > 256 || (stride != 1 && stride != 2)) return false;
  const int cq = g.c / 4, cblocks = g.c / 16;
  const int groups = 256 / cq;
  if (groups < 1) return false;
  // output columns per workgroup: with its halo the tile is one or two blocks of 16 expanded
  // pixels; the wider candidate unless only the narrower one divides the row
  const int candidates[2][2] = {{14, 30}, {7, 15}};
  int pick = 0;
  for (int i = 1; i >= 0; --i) {
    const int tile_w = candidates[stride - 1][i] > g.out_w ? g.out_w : candidates[stride - 1][i];
    const int pblocks = ((tile_w - 1) * stride + 3 + 15) / 16;
    const size_t bytes = ((size_t)(3 + stride) * 16 * pblocks * (g.c + 4) + (size_t)g.c * (K + 4) + g.c) * sizeof(float);
    const bool fits = pblocks <= 2 && (tile_w + groups - 1) / groups <= kMaxPasses && bytes <= 156 * 1024;
    if (!fits) continue;
    // (a narrow tile that gives the four waves fewer than four blocks per step only when nothing else fits)
    const bool idle_waves = stride * pblocks * cblocks < 4;
    if (pick == 0 || (g.out_w % pick != 0 && g.out_w % tile_w == 0 && !idle_waves)) pick = tile_w;
  }
  if (pick == 0) return false;
  g.tile_w = pick;
  g.pblocks = ((pick - 1) * stride + 3 + 15) / 16;
  g.pitch = g.c + 4;
  *lds_bytes = ((size_t)(3 + stride) * 16 * g.pblocks * g.pitch + (size_t)g.c * (K + 4) + g.c) * sizeof(float);
  g.tiles_w = (g.out_w + g.tile_w - 1) / g.tile_w;
  // output rows per workgroup: every row chunk recomputes two expanded rows of halo, so as
  // many rows as still give each compute unit the workgroups its LDS holds (four at most)
  long long resident = (long long)(160 * 1024 / *lds_bytes);
  resident = resident > 4 ? 4 : resident;
  int rows = g.out_h;
  while (rows > 7 && (long long)g.batch * ((g.out_h + rows - 1) / rows) * g.tiles_w < resident * num_cus()) rows = (rows + 1) / 2;
  g.rows = rows;
  g.chunks_h = (g.out_h + rows - 1) / rows;
  return true;
}

}  // namespace tfhip

using namespace tfhip;

namespace {

// Where both fused kernels take a shape: the row-ring kernel for the wide maps of the first
// blocks (its workgroups split the map, and every one needs all expanded channels), the tile
// kernel from 28x28 down (its workgroups split the channels).
bool prefer_tile_kernel(int64_t batch, int64_t in_c, int64_t mid_c, int64_t stride, int64_t out_h, int64_t out_w) {
  (void)batch; (void)in_c; (void)mid_c; (void)out_h;
  return out_w * stride <= 28;
}

}  // namespace

extern "C" int tfhip_fused_pointwise_depthwise(const float *x, const float *pw_filter, const float *pw_bias,
                                               int pw_activation, const float *dw_filter, const float *dw_bias,
                                               int dw_activation, float *y, int64_t batch, int64_t in_h,
                                               int64_t in_w, int64_t in_c, int64_t mid_c, int64_t stride,
                                               int64_t pad_top, int64_t pad_left, int64_t out_h, int64_t out_w) {
  TFHIP_REQUIRE_INIT();
  TFHIP_CHECK_ARG(batch >= 0 && in_h > 0 && in_w > 0 && in_c > 0 && mid_c > 0 && stride > 0 && out_h >= 0 && out_w >= 0 &&
                      pad_top >= 0 && pad_left >= 0,
                  "tfhip_fused_pointwise_depthwise: bad dimension");
  const int64_t lim = 0x7fffffff;
  TFHIP_CHECK_ARG(product_below(lim, {batch, in_h, in_w, in_c > mid_c ? in_c : mid_c}) &&
                      product_below(lim, {batch, out_h, out_w, mid_c}) && stride < lim && pad_top < lim && pad_left < lim,
                  "tfhip_fused_pointwise_depthwise: tensor exceeds the supported range");
  TFHIP_CHECK_ARG(batch * in_h * in_w * in_c * 4 <= 0xfffffffeLL,
                  "tfhip_fused_pointwise_depthwise: x exceeds the 4 GiB one buffer descriptor addresses");
  TFHIP_CHECK_ARG(pw_activation >= TFHIP_LINEAR && pw_activation <= TFHIP_ELU && dw_activation >= TFHIP_LINEAR &&
                      dw_activation <= TFHIP_ELU,
                  "tfhip_fused_pointwise_depthwise: unknown activation");
  if (batch * out_h * out_w == 0) return kOk;
  TFHIP_CHECK_RANGE(x, batch * in_h * in_w * in_c, 4, "x");
  TFHIP_CHECK_RANGE(pw_filter, in_c * mid_c, 4, "pw_filter");
  TFHIP_CHECK_RANGE(dw_filter, 9 * mid_c, 4, "dw_filter");
  if (pw_bias) TFHIP_CHECK_RANGE(pw_bias, mid_c, 4, "pw_bias");
  if (dw_bias) TFHIP_CHECK_RANGE(dw_bias, mid_c, 4, "dw_bias");
  TFHIP_CHECK_OUTPUT(y, batch * out_h * out_w * mid_c, 4, "y");
  if (window_can_miss(in_h, out_h, stride, pad_top, 3, 1) || window_can_miss(in_w, out_w, stride, pad_left, 3, 1)) {
    bool refuse = false;
    const int rc = refuse_nonfinite_filter(dw_filter, 9 * mid_c, "tfhip_fused_pointwise_depthwise", &refuse);
    if (rc != kOk) return rc;
    if (refuse) return fail(kBadArgument, "tfhip_fused_pointwise_depthwise: %s", kNonfiniteFilterMessage);
  }

  const bool aligned = reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(pw_filter) % 16 == 0 &&
                       reinterpret_cast<uintptr_t>(dw_filter) % 16 == 0 &&
                       reinterpret_cast<uintptr_t>(y) % 16 == 0 &&
                       (dw_bias == nullptr || reinterpret_cast<uintptr_t>(dw_bias) % 16 == 0);
  const bool same_relu = pw_activation == dw_activation && (pw_activation == TFHIP_RELU || pw_activation == TFHIP_RELU6);

  // the row-ring kernel (all channels per workgroup: wide maps, few channels)
  ExpandDwArgs g = {};
  g.x = x; g.w1 = pw_filter; g.b1 = pw_bias; g.w2 = dw_filter; g.b2 = dw_bias; g.y = y;
  g.batch = (int)batch; g.in_h = (int)in_h; g.in_w = (int)in_w; g.cin = (int)in_c; g.c = (int)mid_c;
  g.pad_top = (int)pad_top; g.pad_left = (int)pad_left; g.out_h = (int)out_h; g.out_w = (int)out_w;
  g.act1 = pw_activation; g.act2 = dw_activation;
  g.x_bytes = (unsigned)(batch * in_h * in_w * in_c * 4);
  size_t lds_bytes = 0;
  const bool k_ok = in_c == 8 || in_c == 16 || in_c == 24 || in_c == 32;
  const bool ring_ok = aligned && same_relu && k_ok && plan_expand_dw(g, (int)stride, (int)in_c, &lds_bytes);

  // the channel-sliced tile kernel (small maps, many channels)
  ExpandDwTileArgs t = {};
  t.x = x; t.w1 = pw_filter; t.b1 = pw_bias; t.w2 = dw_filter; t.b2 = dw_bias; t.y = y;
  t.batch = (int)batch; t.in_h = (int)in_h; t.in_w = (int)in_w; t.cin = (int)in_c; t.c = (int)mid_c;
  t.stride = (int)stride; t.pad_top = (int)pad_top; t.pad_left = (int)pad_left; t.out_h = (int)out_h; t.out_w = (int)out_w;
  t.cap = pw_activation == TFHIP_RELU6 ? 6.f : __builtin_inff();
  t.x_bytes = g.x_bytes;
  size_t tile_lds_bytes = 0;
  const bool tile_ok = aligned && same_relu &&
                       (pw_bias == nullptr || reinterpret_cast<uintptr_t>(pw_bias) % 16 == 0) &&
                       plan_expand_dw_tile(t, &tile_lds_bytes);

  // the register-streaming kernel (a wavefront per strip and block of 16 channels, no LDS)
  ExpandDwStreamArgs st = {};
  st.x = x; st.w1 = pw_filter; st.b1 = pw_bias; st.w2 = dw_filter; st.b2 = dw_bias; st.y = y;
  st.batch = (int)batch; st.in_h = (int)in_h; st.in_w = (int)in_w; st.cin = (int)in_c; st.c = (int)mid_c;
  st.stride = (int)stride; st.pad_top = (int)pad_top; st.pad_left = (int)pad_left; st.out_h = (int)out_h; st.out_w = (int)out_w;
  st.cap = t.cap;
  st.x_bytes = g.x_bytes;
  const bool stream_ok = aligned && same_relu &&
                         (pw_bias == nullptr || reinterpret_cast<uintptr_t>(pw_bias) % 16 == 0) &&
                         plan_expand_dw_stream(st);
  {
    // Measured at batch 32 with operands from memory (streaming against the better of the other two):
    // 112x112 16 -> 96 stride 2: 34 against 47 us; 56x56 24 -> 144: 38 against 55 (stride 1), 21
    // against 29 (stride 2); 28x28 32 -> 192 stride 1: 14.2 against 15.5. On the smaller maps, whose
    // many input channels every wavefront would hold in registers, the tile kernel stays ahead.
    const int knob = tuning(kTunePwDwStream);
    const bool wide = out_w * stride >= 56 || (stride == 1 && out_w * stride >= 28 && in_c <= 32);
    const bool other_forced = tuning(kTunePwDwTile) >= 0 && (tile_ok || ring_ok);   // that knob names one of the other two
    if (stream_ok && (knob >= 0 ? knob > 0 : ((wide && !other_forced) || (!tile_ok && !ring_ok)))) return launch_expand_dw_stream(st);
  }

  bool use_tile = tile_ok && !ring_ok;
  if (tile_ok && ring_ok) {
    const int knob = tuning(kTunePwDwTile);
    use_tile = knob >= 0 ? knob > 0 : prefer_tile_kernel(batch, in_c, mid_c, stride, out_h, out_w);
  }
  if (use_tile) return launch_expand_dw_tile(t, tile_lds_bytes);
  if (!ring_ok) {
    return fail(kBadArgument,
                "tfhip_fused_pointwise_depthwise: form not taken by the fused kernels (in_c 8/16/24/32 with mid_c a "
                "multiple of 16 up to 256, or in_c 16/24/32/64/96/160 with mid_c a multiple of 32 on a map that "
                "fits the kernel's tile; stride 1 or 2, both activations relu or both relu6, 16-byte aligned "
                "operands); run the two convolutions");
  }
  const int key = (int)stride * 100 + (int)in_c;
  switch (key) {
    case 108: return launch_expand_dw<1, 0, true>(g, lds_bytes);
    case 116: return launch_expand_dw<1, 1, false>(g, lds_bytes);
    case 124: return launch_expand_dw<1, 1, true>(g, lds_bytes);
    case 132: return launch_expand_dw<1, 2, false>(g, lds_bytes);
    case 208: return launch_expand_dw<2, 0, true>(g, lds_bytes);
    case 216: return launch_expand_dw<2, 1, false>(g, lds_bytes);
    case 224: return launch_expand_dw<2, 1, true>(g, lds_bytes);
    default: return launch_expand_dw<2, 2, false>(g, lds_bytes);
  }
}

// 1 when tfhip_fused_pointwise_depthwise takes this shape and is expected to beat the two kernels,
// else 0. The streaming kernel and the channel-sliced one pay at every batch size: at batch 32 the
// expanded tensor no longer goes to memory and back, and at small batches, where both separate
// launches are all latency, one launch replaces two (MobileNetV2 through the graph model as a
// recorded launch sequence, all 17 pairs fused against the two kernels each: 0.284 against 0.296
// ms at batch 1, 0.298 against 0.331 at batch 4, 0.407 against 0.424 at batch 16). The row-ring
// kernel, which is what is left for shapes neither of them takes, pays from an expanded tensor of
// 48 MB (measured at batch 32 in sequence: 16 -> 96 channels at 112x112, stride 2: 43 us against
// 38 + 55; 32 -> 192 at 28x28, where the expanded tensor of 19 MB stays in cache: 38 against 21
// at stride 2).
extern "C" int tfhip_pointwise_depthwise_pays(int64_t batch, int64_t in_c, int64_t mid_c, int64_t stride,
                                              int64_t out_h, int64_t out_w) {
  if (!initialised() || batch <= 0 || out_h <= 0 || out_w <= 0 || mid_c <= 0 || mid_c > 0x7fffffff || in_c <= 0 ||
      in_c > 0x7fffffff || batch > 0x7fffffff || out_h > 0x7fffffff || out_w > 0x7fffffff) {
    return 0;
  }
  ExpandDwArgs g = {};
  g.batch = (int)batch; g.cin = (int)in_c; g.c = (int)mid_c; g.out_h = (int)out_h; g.out_w = (int)out_w;
  size_t lds_bytes = 0;
  const bool k_ok = in_c == 8 || in_c == 16 || in_c == 24 || in_c == 32;
  const bool ring_ok = k_ok && plan_expand_dw(g, (int)stride, (int)in_c, &lds_bytes);
  ExpandDwTileArgs t = {};
  t.batch = (int)batch; t.cin = (int)in_c; t.c = (int)mid_c; t.stride = (int)stride; t.out_h = (int)out_h; t.out_w = (int)out_w;
  const bool tile_ok = plan_expand_dw_tile(t, &lds_bytes);
  ExpandDwStreamArgs st = {};
  st.batch = (int)batch; st.cin = (int)in_c; st.c = (int)mid_c; st.stride = (int)stride; st.out_h = (int)out_h; st.out_w = (int)out_w;
  const bool stream_ok = tuning(kTunePwDwStream) != 0 && plan_expand_dw_stream(st);
  if (!ring_ok && !tile_ok && !stream_ok) return 0;
  if (tuning(kTuneFusePwDw) >= 0) return tuning(kTuneFusePwDw) > 0 ? 1 : 0;   // knob: always / never
  // (the maps on which the entry point runs the streaming kernel by choice; elsewhere it is only the
  // fallback for a channel count the channel-sliced kernel does not divide, and priced like the ring)
  const bool wide = out_w * stride >= 56 || (stride == 1 && out_w * stride >= 28 && in_c <= 32);
  if (tile_ok || (stream_ok && wide)) return 1;
  const int64_t expanded_bytes = batch * out_h * stride * out_w * stride * mid_c * 4;
  return expanded_bytes >= 48LL * 1000 * 1000 ? 1 : 0;
}

namespace {

// k steps of the instantiated few-channel first stages for a filter of `taps` taps (0: none)
int stem_k_steps(int64_t taps) { return taps <= 12 ? 3 : (taps <= 28 ? 7 : (taps <= 36 ? 9 : 0)); }

}  // namespace

extern "C" int tfhip_fused_conv2d_depthwise(const float *x, const float *filter, const float *bias, int activation,
                                            const float *dw_filter, const float *dw_bias, int dw_activation, float *y,
                                            int64_t batch, int64_t in_h, int64_t in_w, int64_t in_c, int64_t f_h,
                                            int64_t f_w, int64_t mid_c, int64_t stride, int64_t pad_top,
                                            int64_t pad_left, int64_t mid_h, int64_t mid_w, int64_t dw_stride,
                                            int64_t dw_pad_top, int64_t dw_pad_left, int64_t out_h, int64_t out_w) {
  TFHIP_REQUIRE_INIT();
  TFHIP_CHECK_ARG(batch >= 0 && in_h > 0 && in_w > 0 && in_c > 0 && f_h > 0 && f_w > 0 && mid_c > 0 && stride > 0 &&
                      mid_h >= 0 && mid_w >= 0 && dw_stride > 0 && out_h >= 0 && out_w >= 0 && pad_top >= 0 &&
                      pad_left >= 0 && dw_pad_top >= 0 && dw_pad_left >= 0,
                  "tfhip_fused_conv2d_depthwise: bad dimension");
  const int64_t lim = 0x7fffffff;
  TFHIP_CHECK_ARG(product_below(lim, {batch, in_h, in_w, in_c}) && product_below(lim, {batch, mid_h, mid_w, mid_c}) &&
                      product_below(lim, {batch, out_h, out_w, mid_c}) && product_below(lim, {f_h, f_w, in_c, mid_c}) &&
                      stride < lim && dw_stride < lim && pad_top < lim && pad_left < lim && dw_pad_top < lim &&
                      dw_pad_left < lim,
                  "tfhip_fused_conv2d_depthwise: tensor exceeds the supported range");
  TFHIP_CHECK_ARG(activation >= TFHIP_LINEAR && activation <= TFHIP_ELU && dw_activation >= TFHIP_LINEAR &&
                      dw_activation <= TFHIP_ELU,
                  "tfhip_fused_conv2d_depthwise: unknown activation");
  if (batch * out_h * out_w == 0) return kOk;
  const int64_t K = f_h * f_w * in_c;
  TFHIP_CHECK_RANGE(x, batch * in_h * in_w * in_c, 4, "x");
  TFHIP_CHECK_RANGE(filter, K * mid_c, 4, "filter");
  TFHIP_CHECK_RANGE(dw_filter, 9 * mid_c, 4, "dw_filter");
  if (bias) TFHIP_CHECK_RANGE(bias, mid_c, 4, "bias");
  if (dw_bias) TFHIP_CHECK_RANGE(dw_bias, mid_c, 4, "dw_bias");
  TFHIP_CHECK_OUTPUT(y, batch * out_h * out_w * mid_c, 4, "y");
  {
    bool refuse = false;
    int rc = kOk;
    if (window_can_miss(mid_h, out_h, dw_stride, dw_pad_top, 3, 1) || window_can_miss(mid_w, out_w, dw_stride, dw_pad_left, 3, 1))
      rc = refuse_nonfinite_filter(dw_filter, 9 * mid_c, "tfhip_fused_conv2d_depthwise", &refuse);
    if (rc == kOk && !refuse &&
        (window_can_miss(in_h, mid_h, stride, pad_top, f_h, 1) || window_can_miss(in_w, mid_w, stride, pad_left, f_w, 1)))
      rc = refuse_nonfinite_filter(filter, K * mid_c, "tfhip_fused_conv2d_depthwise", &refuse);
    if (rc != kOk) return rc;
    if (refuse) return fail(kBadArgument, "tfhip_fused_conv2d_depthwise: %s", kNonfiniteFilterMessage);
  }

  ExpandDwArgs g = {};
  g.x = x; g.w1 = filter; g.b1 = bias; g.w2 = dw_filter; g.b2 = dw_bias; g.y = y;
  g.batch = (int)batch; g.in_h = (int)mid_h; g.in_w = (int)mid_w; g.cin = (int)in_c; g.c = (int)mid_c;
  g.pad_top = (int)dw_pad_top; g.pad_left = (int)dw_pad_left; g.out_h = (int)out_h; g.out_w = (int)out_w;
  g.act1 = activation; g.act2 = dw_activation;
  g.x_bytes = (unsigned)(batch * in_h * in_w * in_c * 4);
  g.xh = (int)in_h; g.xw = (int)in_w; g.xc = (int)in_c; g.conv_stride = (int)stride;
  g.conv_pad_top = (int)pad_top; g.conv_pad_left = (int)pad_left; g.k = (int)K;
  const int k_steps = in_c <= 4 ? stem_k_steps(K) : 0;
  size_t lds_bytes = 0;
  const bool aligned = reinterpret_cast<uintptr_t>(filter) % 16 == 0 && reinterpret_cast<uintptr_t>(dw_filter) % 16 == 0 &&
                       reinterpret_cast<uintptr_t>(y) % 16 == 0 &&
                       (dw_bias == nullptr || reinterpret_cast<uintptr_t>(dw_bias) % 16 == 0);
  const bool same_relu = activation == dw_activation && (activation == TFHIP_RELU || activation == TFHIP_RELU6);
  if (!aligned || !same_relu || k_steps == 0 || batch * in_h * in_w * in_c * 4 > 0xfffffffeLL ||
      !plan_expand_dw(g, (int)dw_stride, 4 * k_steps, &lds_bytes)) {
    return fail(kBadArgument,
                "tfhip_fused_conv2d_depthwise: form not taken by the fused kernel (at most 4 input channels and 36 "
                "filter taps, mid_c a multiple of 16 up to 256, depthwise stride 1 or 2, both activations relu or "
                "both relu6, 16-byte aligned operands); run the two convolutions");
  }
  StemTaps taps;
  for (int k = 0; k < kMaxStemTaps; ++k) {
    const int tap = k / (int)in_c, ch = k - tap * (int)in_c;
    const int fr = tap / (int)f_w, fs = tap - fr * (int)f_w;
    taps.dh[k] = k < K ? fr : (1 << 28);
    taps.dw[k] = fs;
    taps.off_bytes[k] = (unsigned)((((long long)fr * in_w + fs) * in_c + ch) * 4);
  }
  if (tuning(kTunePwDwStream) != 0) {   // (224x224x3 -> 112x112x32 at batch 32: 40 against 52 us with operands from memory)
    ExpandDwStreamArgs st = {};
    st.x = x; st.w1 = filter; st.b1 = bias; st.w2 = dw_filter; st.b2 = dw_bias; st.y = y;
    st.batch = (int)batch; st.in_h = (int)mid_h; st.in_w = (int)mid_w; st.cin = (int)in_c; st.c = (int)mid_c;
    st.stride = (int)dw_stride; st.pad_top = (int)dw_pad_top; st.pad_left = (int)dw_pad_left;
    st.out_h = (int)out_h; st.out_w = (int)out_w;
    st.cap = activation == TFHIP_RELU6 ? 6.f : __builtin_inff();
    st.x_bytes = g.x_bytes;
    st.xh = g.xh; st.xw = g.xw; st.xc = g.xc; st.conv_stride = g.conv_stride; st.conv_pad_top = g.conv_pad_top;
    st.conv_pad_left = g.conv_pad_left; st.k = g.k; st.k_steps = k_steps;
    if ((bias == nullptr || reinterpret_cast<uintptr_t>(bias) % 16 == 0) && plan_expand_dw_stream(st))
      return launch_stem_dw_stream(st, taps);
  }
  const int key = (int)dw_stride * 10 + k_steps;
  switch (key) {
    case 13: return launch_stem_dw<1, 3>(g, taps, lds_bytes);
    case 17: return launch_stem_dw<1, 7>(g, taps, lds_bytes);
    case 19: return launch_stem_dw<1, 9>(g, taps, lds_bytes);
    case 23: return launch_stem_dw<2, 3>(g, taps, lds_bytes);
    case 27: return launch_stem_dw<2, 7>(g, taps, lds_bytes);
    default: return launch_stem_dw<2, 9>(g, taps, lds_bytes);
  }
}

// 1 when tfhip_fused_conv2d_depthwise takes this shape and is expected to beat the two kernels, else
// 0: always where the streaming kernel takes it, from a tensor of 48 MB between the stages where
// only the row-ring kernel does (as for the pointwise first stage).
extern "C" int tfhip_conv2d_depthwise_pays(int64_t batch, int64_t in_c, int64_t f_h, int64_t f_w, int64_t mid_c,
                                           int64_t mid_h, int64_t mid_w, int64_t dw_stride, int64_t out_h,
                                           int64_t out_w) {
  if (!initialised() || batch <= 0 || out_h <= 0 || out_w <= 0 || mid_c <= 0 || mid_c > 0x7fffffff || in_c <= 0 ||
      in_c > 4 || f_h <= 0 || f_w <= 0 || f_h * f_w * in_c > 36 || batch > 0x7fffffff || out_h > 0x7fffffff ||
      out_w > 0x7fffffff || mid_h <= 0 || mid_w <= 0) {
    return 0;
  }
  ExpandDwArgs g = {};
  g.batch = (int)batch; g.cin = (int)in_c; g.c = (int)mid_c; g.out_h = (int)out_h; g.out_w = (int)out_w;
  size_t lds_bytes = 0;
  if (!plan_expand_dw(g, (int)dw_stride, 4 * stem_k_steps(f_h * f_w * in_c), &lds_bytes)) return 0;
  if (tuning(kTuneFusePwDw) >= 0) return tuning(kTuneFusePwDw) > 0 ? 1 : 0;
  ExpandDwStreamArgs st = {};
  st.batch = (int)batch; st.cin = (int)in_c; st.c = (int)mid_c; st.stride = (int)dw_stride; st.out_h = (int)out_h; st.out_w = (int)out_w;
  st.k_steps = stem_k_steps(f_h * f_w * in_c);
  if (tuning(kTunePwDwStream) != 0 && plan_expand_dw_stream(st)) return 1;
  return batch * mid_h * mid_w * mid_c * 4 >= 48LL * 1000 * 1000 ? 1 : 0;
}
