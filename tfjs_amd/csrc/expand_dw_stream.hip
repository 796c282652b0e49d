// Pointwise expansion + depthwise 3x3 stage in one launch, everything in registers.
//
//   y = act(depthwise3x3(act(x * W1 + b1), W2) + b2)        act = relu or relu6 for both
//
// One wavefront owns a block of 16 expanded channels of a strip of the map and walks down its
// rows. An expanded row of the strip is one 16 x 16 block of MFMA results: lane (grp, r) ends up
// with the four channels 4 grp .. 4 grp + 3 of pixel r. The depthwise stage needs that pixel's
// left and right neighbours, which are the neighbouring lanes of the same 16-lane row (one DPP
// row shift each), and the rows above and below, which the wavefront has already added into the
// running sums of the output rows they belong to. So the expanded tensor never leaves the registers: no LDS, no barrier, and the
// wavefronts of a workgroup (the channel blocks of one strip, which read the same input) do
// not wait for one another.
//
// The strip is 16 expanded pixels wide. At stride 1 they give 14 output columns (the two outer
// pixels are halo); at stride 2 the wavefront computes two blocks per expanded row, the even and
// the odd columns, and needs one shifted copy of the even ones: 15 output columns.
//
// Products and sums are formed in the order of the separate kernels (k ascending inside the MFMA
// chain starting from the bias; the nine taps row by row from zero, then the bias), so the result
// has the bits of FusedConv2D followed by FusedDepthwiseConv2D.
#include <type_traits>

#include "common.h"
#include "epilogue.h"
#include "expand_dw_stream.h"

namespace tfhip {
namespace {

typedef float float4_t __attribute__((ext_vector_type(4)));
constexpr unsigned kNoOff = 0xffffffffu;   // an offset no buffer descriptor covers: loads return 0

// min(max(0, v), cap) as Math.max / Math.min form it: NaN stays NaN (cap = 6 for relu6, +inf for
// relu). The median of (v, 0, cap) is the answer for every v that is a number; `nan_classes` names
// the classes of v that are handed through instead (both kinds of NaN).
constexpr int kNanClasses = 0x3;
__device__ __forceinline__ float relu_cap(float v, float cap, int nan_classes = kNanClasses) {
  const float t = __builtin_amdgcn_fmed3f(v, 0.f, cap);
  return __builtin_amdgcn_classf(v, nan_classes) ? v : t;
}

// The value of the lane below (r - 1) / above (r + 1) in the 16-lane row; 0 at the row's end.
__device__ __forceinline__ float from_lane_below(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x111, 0xf, 0xf, true));   // row_shr:1
}
__device__ __forceinline__ float from_lane_above(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x101, 0xf, 0xf, true));   // row_shl:1
}
__device__ __forceinline__ float4 from_lane_below(const float4 &v) {
  return make_float4(from_lane_below(v.x), from_lane_below(v.y), from_lane_below(v.z), from_lane_below(v.w));
}
__device__ __forceinline__ float4 from_lane_above(const float4 &v) {
  return make_float4(from_lane_above(v.x), from_lane_above(v.y), from_lane_above(v.z), from_lane_above(v.w));
}

// The three horizontal taps of one expanded row at this lane's output column.
struct Taps {
  float4 t0, t1, t2;
};

// S: stride of the depthwise stage. K = 16 KF + (HALF ? 8 : 0) input channels.
// TAPS > 0: the first stage is a convolution of at most 4 TAPS taps (filter height x width x input
// channels, a network stem) gathered element by element with the lane layout and instruction
// order of the few-taps convolution kernel (lane (grp, r) feeds tap 4 t + grp in k step t); KF and
// HALF are then unused.
// NCB: blocks of 16 channels per wavefront (1 or 2). Two blocks share every input fragment, and
// the wavefront's stores cover 128 contiguous bytes of a pixel instead of 64.
// AHEAD: how many expanded rows ahead of their use the inputs are fetched (2 or 4).
// (Two wavefronts per SIMD asked for wherever the registers allow: with at most 256 registers per
// lane the matrix instructions keep their results in ordinary vector registers, where the
// activation reads them, instead of the accumulation registers they would have to be copied out of.)
template <int S, int KF, bool HALF, int TAPS, int NCB, int AHEAD>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu((S * KF * NCB >= 16 || (S == 2 && TAPS >= 7)) ? 1 : 2)))
void expand_dw_stream(ExpandDwStreamArgs g, StemTaps taps) {
  constexpr int K = 16 * KF + (HALF ? 8 : 0);
  const int lane = threadIdx.x & 63;
  const int grp = lane >> 4, r = lane & 15;
  // everything derived from the wavefront's index is the same in all its lanes: pinned to scalar
  // registers, so that row addresses, loop bounds and the in-image tests of a row cost no vector
  // instruction
  // Workgroup ids i, i + 8, i + 16, ... share an XCD and its L2: each XCD takes one contiguous band
  // of the wavefront sequence, so that the channel blocks of a strip, which read the same input
  // rows, find them in one L2 instead of fetching them into all eight.
  unsigned block = blockIdx.x;
  {
    const unsigned per_xcd = gridDim.x / 8;
    if (per_xcd > 0 && block < per_xcd * 8) block = (block % 8) * per_xcd + block / 8;
  }
  unsigned w = block * 4 + (unsigned)__builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  if (w >= (unsigned)g.waves) return;   // (whole wavefronts: nothing below synchronises across them)
  const unsigned cgroups = (unsigned)(g.cblocks + NCB - 1) / NCB;
  const int cb0 = (int)(w % cgroups) * NCB;         // first channel block of this wavefront
  w /= cgroups;
  const int strip = (int)(w % (unsigned)g.strips);
  w /= (unsigned)g.strips;
  const int chunk = (int)(w % (unsigned)g.chunks_h), n = (int)(w / (unsigned)g.chunks_h);
  const int oh0 = chunk * g.rows, ow0 = strip * g.strip_w;
  const int rows = oh0 + g.rows <= g.out_h ? g.rows : g.out_h - oh0;
  const int e0 = oh0 * S - g.pad_top;               // first expanded row this wavefront needs
  // (an odd count of channel blocks: the last wavefront's second block repeats its first and is not stored)
  int cbs[NCB], ch[NCB];                            // channel blocks, and this lane's four channels in each
#pragma unroll
  for (int u = 0; u < NCB; ++u) {
    cbs[u] = cb0 + u < g.cblocks ? cb0 + u : cb0;
    ch[u] = 16 * cbs[u] + 4 * grp;
  }
  const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc((void *)g.x, 0, (int)g.x_bytes, 0x00020000);

  int tap_dh[TAPS > 0 ? TAPS : 1], tap_dw[TAPS > 0 ? TAPS : 1];
  unsigned tap_off[TAPS > 0 ? TAPS : 1];
  int tap_row[S][TAPS > 0 ? TAPS : 1];        // filled below, once this lane's columns are known
  unsigned tap_col_off[S][TAPS > 0 ? TAPS : 1];
  if (TAPS > 0) {
#pragma unroll
    for (int t = 0; t < TAPS; ++t) {
      tap_dh[t] = taps.dh[4 * t + grp];
      tap_dw[t] = taps.dw[4 * t + grp];
      tap_off[t] = taps.off_bytes[4 * t + grp];
    }
  }
  // This lane's expanded column in block b (S == 1: one block; S == 2: even and odd columns),
  // whether it lies in the image, and its byte offset inside a row of x (1x1 first stage: the k
  // group of this lane included) or the column of its window's first element (few-taps first stage).
  int ecol[S];
  bool col_ok[S];
  unsigned col_off[S];
#pragma unroll
  for (int b = 0; b < S; ++b) {
    ecol[b] = S == 1 ? ow0 - g.pad_left + r : 2 * (ow0 + r) - g.pad_left + b;
    col_ok[b] = ecol[b] >= 0 && ecol[b] < g.in_w;
    col_off[b] = TAPS > 0 ? 0u : (unsigned)(ecol[b] * K * 4 + (HALF && KF == 0 ? 2 : 4) * grp * 4);
  }
  // The expanded tensor's padding folded into the activation: a column outside the map gets the
  // cap 0 and no NaN handed through, so whatever was computed for it comes out as 0.
  float cap_col[S];
  int nan_col[S];
#pragma unroll
  for (int b = 0; b < S; ++b) {
    cap_col[b] = col_ok[b] ? g.cap : 0.f;
    nan_col[b] = col_ok[b] ? kNanClasses : 0;
  }
  if (TAPS > 0) {
    // Few-taps first stage: whether a tap's column lies in the image does not change from row to
    // row, so it is folded into the tap's row offset once: a tap whose column (or whose pixel's
    // column) is outside gets a row offset no image reaches, and the one test a row then needs per
    // tap, "is the tap's row inside", fails for it as well. The byte offset of the tap from the
    // first element of the window's row 0 takes the window's column along.
#pragma unroll
    for (int b = 0; b < S; ++b) {
      const int xw0 = ecol[b] * g.conv_stride - g.conv_pad_left;
#pragma unroll
      for (int t = 0; t < TAPS; ++t) {
        const bool col_in = col_ok[b] & ((unsigned)(xw0 + tap_dw[t]) < (unsigned)g.xw);
        tap_row[b][t] = col_in ? tap_dh[t] : 0x40000000;
        tap_col_off[b][t] = (unsigned)(xw0 * g.xc * 4) + tap_off[t];   // (exact modulo 2^32 for a tap inside)
      }
    }
  }
  const unsigned row_bytes = TAPS > 0 ? 0u : (unsigned)(g.in_w * K * 4);
  const unsigned image_off = TAPS > 0 ? 0u : (unsigned)((long long)n * g.in_h * g.in_w * K * 4);

  struct AFrag {
    float4 full[KF > 0 ? KF : 1];
    float2 half;
    float tap[TAPS > 0 ? TAPS : 1];
  };
  // The inputs of expanded row e: one fragment per block. 1x1 first stage: the loads of a position
  // outside the image may return anything (a neighbouring row, or zero past the tensor's end; the
  // descriptor keeps them inside the tensor): expand() discards what is computed from them.
  auto load_row = [&](AFrag (&a)[S], int e) __attribute__((always_inline)) {
#pragma unroll
    for (int b = 0; b < S; ++b) {
      if (TAPS > 0) {
        // the window of first-stage output pixel (e, ecol): its first row may lie before the image,
        // the sum with an inside tap's offset is exact modulo 2^32. Row number, row limit and the
        // row's byte offset are the same in every lane (scalar); a row outside the expanded map
        // gets the limit 0, which no tap passes.
        const int xh0 = e * g.conv_stride - g.conv_pad_top;
        const unsigned limit = (e >= 0 && e < g.in_h) ? (unsigned)g.xh : 0u;
        const unsigned base = (unsigned)((((long long)n * g.xh + xh0) * g.xw) * g.xc * 4);
#pragma unroll
        for (int t = 0; t < TAPS; ++t) {
          const bool ok = (unsigned)(xh0 + tap_row[b][t]) < limit;
          a[b].tap[t] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rx, (int)(ok ? base + tap_col_off[b][t] : kNoOff), 0, 0));
        }
        continue;
      }
      const unsigned base = image_off + (unsigned)e * row_bytes + col_off[b];
#pragma unroll
      for (int t = 0; t < KF; ++t) {
        const auto v = __builtin_amdgcn_raw_buffer_load_b128(rx, (int)(base + 64 * t), 0, 0);
        a[b].full[t] = make_float4(__uint_as_float(v[0]), __uint_as_float(v[1]), __uint_as_float(v[2]), __uint_as_float(v[3]));
      }
      if (HALF) {
        // (the lane's k group is two wide here: col_off holds 16 grp bytes when KF > 0, 8 grp when the half group is alone)
        const auto v = __builtin_amdgcn_raw_buffer_load_b64(rx, (int)(base + 64 * KF - (KF > 0 ? 8 * grp : 0)), 0, 0);
        a[b].half = make_float2(__uint_as_float(v[0]), __uint_as_float(v[1]));
      }
    }
  };
  // The first rows' inputs are fetched before the weights: everything the wavefront needs before its
  // first matrix instruction is then in flight together, one memory round trip instead of two.
  // Expanded row e0 + i lives in fragment set i % AHEAD.
  AFrag fa[AHEAD][S];
#pragma unroll
  for (int i = 0; i < AHEAD; ++i) load_row(fa[i], e0 + i);

  // expansion weights of channel 16 cb + r at k = 16 t + 4 grp .. + 3 (the MFMA's first operand), bias
  float4 wq[NCB][KF > 0 ? KF : 1];
  float2 wh[NCB];
  float wt[NCB][TAPS > 0 ? TAPS : 1];
  float4_t b1q[NCB];
  float4 w2q[NCB][9], b2q[NCB];
#pragma unroll
  for (int u = 0; u < NCB; ++u) {
    wh[u] = make_float2(0.f, 0.f);
    if (TAPS > 0) {
#pragma unroll
      for (int t = 0; t < TAPS; ++t) {
        const int k = 4 * t + grp;
        wt[u][t] = k < g.k ? g.w1[(long long)k * g.c + 16 * cbs[u] + r] : 0.f;   // taps beyond the filter multiply zeros
      }
    } else {
      const float *col = g.w1 + 16 * cbs[u] + r;
#pragma unroll
      for (int t = 0; t < KF; ++t) {
        const int k = 16 * t + 4 * grp;
        wq[u][t] = make_float4(col[(long long)k * g.c], col[(long long)(k + 1) * g.c], col[(long long)(k + 2) * g.c],
                               col[(long long)(k + 3) * g.c]);
      }
      if (HALF) {
        const int k = 16 * KF + 2 * grp;
        wh[u] = make_float2(col[(long long)k * g.c], col[(long long)(k + 1) * g.c]);
      }
    }
    // (a missing bias: the fetch goes to the depthwise weights instead and is dropped; a branch around a
    // load would make the wavefront wait at its end for every fetch in flight)
    {
      const float4_t v = *reinterpret_cast<const float4_t *>((g.b1 ? g.b1 : g.w2) + ch[u]);
      b1q[u] = g.b1 ? v : float4_t{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int t = 0; t < 9; ++t) w2q[u][t] = *reinterpret_cast<const float4 *>(g.w2 + (long long)t * g.c + ch[u]);
    {
      const float4 v = *reinterpret_cast<const float4 *>((g.b2 ? g.b2 : g.w2) + ch[u]);
      b2q[u] = g.b2 ? v : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  }

  // expanded row e of block b, channel block u: activation applied, zero outside the map (the
  // depthwise stage's padding)
  auto expand = [&](const AFrag &a, int e, int b, int u) __attribute__((always_inline)) {
    float4_t acc = b1q[u];
#pragma unroll
    for (int t = 0; t < TAPS; ++t) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wt[u][t], a.tap[t], acc, 0, 0, 0);
#pragma unroll
    for (int t = 0; t < (TAPS > 0 ? 0 : KF); ++t) {
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wq[u][t].x, a.full[t].x, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wq[u][t].y, a.full[t].y, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wq[u][t].z, a.full[t].z, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wq[u][t].w, a.full[t].w, acc, 0, 0, 0);
    }
    if (HALF && TAPS == 0) {
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wh[u].x, a.half.x, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wh[u].y, a.half.y, acc, 0, 0, 0);
    }
    // (a row outside the map, the same test in every lane: like a column outside)
    const bool row_in = e >= 0 && e < g.in_h;
    const float cap = row_in ? cap_col[b] : 0.f;
    const int nan = row_in ? nan_col[b] : 0;
    return make_float4(relu_cap(acc[0], cap, nan), relu_cap(acc[1], cap, nan), relu_cap(acc[2], cap, nan),
                       relu_cap(acc[3], cap, nan));
  };
  // S == 1: the output column of lane r is expanded column r's; its taps sit in lanes r - 1, r, r + 1.
  // S == 2: output column ow0 + r reads even column r, odd column r, even column r + 1.
  auto taps_of = [&](Taps (&t)[NCB], const AFrag (&a)[S], int e) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < NCB; ++u) {
      if (S == 1) {
        t[u].t1 = expand(a[0], e, 0, u);
        t[u].t0 = from_lane_below(t[u].t1);
        t[u].t2 = from_lane_above(t[u].t1);
      } else {
        t[u].t0 = expand(a[0], e, 0, u);
        t[u].t1 = expand(a[S - 1], e, S - 1, u);
        t[u].t2 = from_lane_above(t[u].t0);
      }
    }
  };
  const int ocol = S == 1 ? ow0 + r - 1 : ow0 + r;
  const bool out_lane = (S == 1 ? (r >= 1 && r <= 14) : r <= 14) && ocol < g.out_w && ocol < ow0 + g.strip_w;
  // this lane's place in an output row (channel block 0 of the wavefront), and the rows' distance
  float *out_ptr = g.y + (((long long)n * g.out_h + oh0) * g.out_w + ocol) * g.c + ch[0];
  const long long out_row = (long long)g.out_w * g.c;
  const __amdgpu_buffer_rsrc_t rsrc_y = __builtin_amdgcn_make_buffer_rsrc(
      (void *)(g.y + (long long)n * g.out_h * g.out_w * g.c), 0, (int)((unsigned)g.out_h * g.out_w * g.c * 4u), 0x00020000);
  const unsigned out_off = (unsigned)((oh0 * g.out_w + ocol) * g.c + ch[0]) * 4u;   // (meaningful where g.through)
  // One expanded row's share of a depthwise sum: the three taps of filter row wr, left to right.
  auto add_row = [&](const float4 &sum, const Taps &t, int wr, int u) __attribute__((always_inline)) {
    float4 acc = sum;
    const float4 e[3] = {t.t0, t.t1, t.t2};
#pragma unroll
    for (int wc = 0; wc < 3; ++wc) {
      const float4 wt4 = w2q[u][wr * 3 + wc];
      acc.x = fmaf(e[wc].x, wt4.x, acc.x);
      acc.y = fmaf(e[wc].y, wt4.y, acc.y);
      acc.z = fmaf(e[wc].z, wt4.z, acc.z);
      acc.w = fmaf(e[wc].w, wt4.w, acc.w);
    }
    return acc;
  };
  auto store_row = [&](int o, int u, const float4 &acc) __attribute__((always_inline)) {
    if (out_lane && (u == 0 || cb0 + u < g.cblocks)) {
      const float4 out = make_float4(relu_cap(acc.x + b2q[u].x, g.cap), relu_cap(acc.y + b2q[u].y, g.cap),
                                     relu_cap(acc.z + b2q[u].z, g.cap), relu_cap(acc.w + b2q[u].w, g.cap));
      // (written through: against non-temporal stores behind a 1x1 first stage the GEMMs that read
      // these 19 - 38 MB maps get 2 us faster per inference, and against cached stores the launch
      // behind a few-taps first stage 1 - 2 us; an image beyond 32-bit offsets: the stores of before)
      if (g.through) {
        store_result4_through(rsrc_y, out_off + (unsigned)(o * (int)out_row + 16 * u) * 4u, out);
      } else if (TAPS == 0) {
        store_result4_streaming(out_ptr + o * out_row + 16 * u, out);
      } else {
        store_result4(out_ptr + o * out_row + 16 * u, out);
      }
    }
  };

  // The inputs of a row are fetched kAhead rows before they are used (two; four where the planner
  // expects them to come from memory rather than cache, a round trip that outlasts two rows of
  // work), into kAhead fragment sets used in turn; the loops are unrolled over one turn so that each set
  // stays in fixed registers.
  // An expanded row is used the moment it exists and then dropped: it adds filter row 2 to the
  // output row that it completes, filter row 1 to the next (stride 1) and starts the one after with
  // filter row 0. The sums of the output rows in progress are all the wavefront keeps, each still
  // formed tap by tap in filter order from zero.
  constexpr int kAhead = AHEAD;
  Taps t[NCB];
  float4 sum0[NCB], sum1[NCB];   // the output row two (stride 2: one or two) expanded rows in, and the one with one row in
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
  if (S == 1) {
    taps_of(t, fa[0], e0);
    load_row(fa[0], e0 + kAhead);
#pragma unroll
    for (int u = 0; u < NCB; ++u) sum0[u] = add_row(zero, t[u], 0, u);
    taps_of(t, fa[1 % kAhead], e0 + 1);
    load_row(fa[1 % kAhead], e0 + 1 + kAhead);
#pragma unroll
    for (int u = 0; u < NCB; ++u) {
      sum0[u] = add_row(sum0[u], t[u], 1, u);
      sum1[u] = add_row(zero, t[u], 0, u);
    }
    // output row o: the new expanded row is e0 + o + 2
    auto step = [&](auto phase, int o) __attribute__((always_inline)) {
      constexpr int F = (decltype(phase)::value + 2) % kAhead;
      taps_of(t, fa[F], e0 + o + 2);
      load_row(fa[F], e0 + o + 2 + kAhead);
#pragma unroll
      for (int u = 0; u < NCB; ++u) {
        store_row(o, u, add_row(sum0[u], t[u], 2, u));
        sum0[u] = add_row(sum1[u], t[u], 1, u);
        sum1[u] = add_row(zero, t[u], 0, u);
      }
    };
    for (int o = 0; o < rows; o += 4) {
      step(std::integral_constant<int, 0>(), o);
      if (o + 1 < rows) step(std::integral_constant<int, 1>(), o + 1);
      if (o + 2 < rows) step(std::integral_constant<int, 2>(), o + 2);
      if (o + 3 < rows) step(std::integral_constant<int, 3>(), o + 3);
    }
  } else {
    taps_of(t, fa[0], e0);
    load_row(fa[0], e0 + kAhead);
#pragma unroll
    for (int u = 0; u < NCB; ++u) sum0[u] = add_row(zero, t[u], 0, u);
    // output row o reads expanded rows e0 + 2 o .. + 2: the last is the first of the row after
    auto step = [&](auto phase, int o) __attribute__((always_inline)) {
      constexpr int F1 = (2 * decltype(phase)::value + 1) % kAhead, F2 = (2 * decltype(phase)::value + 2) % kAhead;
      taps_of(t, fa[F1], e0 + 2 * o + 1);
      load_row(fa[F1], e0 + 2 * o + 1 + kAhead);
#pragma unroll
      for (int u = 0; u < NCB; ++u) sum0[u] = add_row(sum0[u], t[u], 1, u);
      taps_of(t, fa[F2], e0 + 2 * o + 2);
      load_row(fa[F2], e0 + 2 * o + 2 + kAhead);
#pragma unroll
      for (int u = 0; u < NCB; ++u) {
        store_row(o, u, add_row(sum0[u], t[u], 2, u));
        sum0[u] = add_row(zero, t[u], 0, u);
      }
    };
    for (int o = 0; o < rows; o += 2) {
      step(std::integral_constant<int, 0>(), o);
      if (o + 1 < rows) step(std::integral_constant<int, 1>(), o + 1);
    }
  }
}

template <int S, int KF, bool HALF, int TAPS, int NCB, int AHEAD>
int launch_stream_ahead(const ExpandDwStreamArgs &g, const StemTaps &taps) {
  const long long blocks = (g.waves + 3) / 4;
  if (blocks > 0x3fffffffLL) return fail(kBadArgument, "expand_dw_stream: %lld workgroups exceed the limit of 2^30", blocks);   // (the kernel counts wavefronts in 32 bits)
  note_kernel("expand_dw_stream<%d, %d, %s, %d, %d, %d>", S, KF, HALF ? "true" : "false", TAPS, NCB, AHEAD);
  TFHIP_LAUNCH((expand_dw_stream<S, KF, HALF, TAPS, NCB, AHEAD><<<dim3((unsigned)blocks), dim3(256), 0, stream()>>>(g, taps)));
  return kOk;
}

template <int S, int KF, bool HALF, int TAPS, int NCB>
int launch_stream_ncb(const ExpandDwStreamArgs &g, const StemTaps &taps) {
  if constexpr (TAPS == 0 && NCB == 1 && KF <= 2) {
    if (g.ahead == 4) return launch_stream_ahead<S, KF, HALF, TAPS, NCB, 4>(g, taps);
  }
  return launch_stream_ahead<S, KF, HALF, TAPS, NCB, 2>(g, taps);
}

// Two channel blocks per wavefront where the input fragments are short enough for the registers
// to hold both blocks' rows and weights.
template <int S, int KF, bool HALF, int TAPS>
int launch_stream(const ExpandDwStreamArgs &g, const StemTaps &taps) {
  if constexpr (KF <= 2 && TAPS <= 7) {
    if (g.ncb == 2) return launch_stream_ncb<S, KF, HALF, TAPS, 2>(g, taps);
  }
  return launch_stream_ncb<S, KF, HALF, TAPS, 1>(g, taps);
}

template <int S>
int launch_stream_k(const ExpandDwStreamArgs &g) {
  const StemTaps none = {};
  switch (g.cin) {
    case 8: return launch_stream<S, 0, true, 0>(g, none);
    case 16: return launch_stream<S, 1, false, 0>(g, none);
    case 24: return launch_stream<S, 1, true, 0>(g, none);
    case 32: return launch_stream<S, 2, false, 0>(g, none);
    case 64: return launch_stream<S, 4, false, 0>(g, none);
    case 96: return launch_stream<S, 6, false, 0>(g, none);
    case 160: return launch_stream<S, 10, false, 0>(g, none);
    default: return fail(kBadArgument, "expand_dw_stream: %d input channels not instantiated", g.cin);
  }
}

template <int S>
int launch_stream_taps(const ExpandDwStreamArgs &g, const StemTaps &taps) {
  switch (g.k_steps) {
    case 3: return launch_stream<S, 0, false, 3>(g, taps);
    case 7: return launch_stream<S, 0, false, 7>(g, taps);
    case 9: return launch_stream<S, 0, false, 9>(g, taps);
    default: return fail(kBadArgument, "expand_dw_stream: %d k steps of filter taps not instantiated", g.k_steps);
  }
}

}  // namespace

bool expand_dw_stream_takes_k(int cin) {
  return cin == 8 || cin == 16 || cin == 24 || cin == 32 || cin == 64 || cin == 96 || cin == 160;
}

// Fills the tiling of `g`; false when the shape is one the kernel does not take.
bool plan_expand_dw_stream(ExpandDwStreamArgs &g) {
  if (g.c % 16 != 0 || (g.stride != 1 && g.stride != 2)) return false;
  if (g.k_steps > 0 ? (g.k_steps != 3 && g.k_steps != 7 && g.k_steps != 9) : !expand_dw_stream_takes_k(g.cin)) return false;
  g.strip_w = g.stride == 1 ? 14 : 15;
  g.strips = (g.out_w + g.strip_w - 1) / g.strip_w;
  g.cblocks = g.c / 16;
  {
    const int forced = tuning(kTuneStreamBlocks);
    const bool short_k = g.k_steps > 0 ? g.k_steps <= 7 : g.cin <= 32;
    // Two blocks per wavefront on a few-taps first stage, whose gathered input fragments are the
    // costly part of a row and are shared by the two blocks (MobileNetV2's stem at batch 32, inside an
    // inference: 38.8 -> 33.3 us). On a 1x1 first stage they lose 1 - 4 us on every shape measured
    // and stay off unless the "stream_blocks" knob asks (2: on, 1: off everywhere).
    const bool two = forced >= 0 ? forced >= 2 : g.k_steps > 0;
    g.ncb = two && g.cblocks >= 2 && short_k ? 2 : 1;
  }
  const int cgroups = (g.cblocks + g.ncb - 1) / g.ncb;
  // Inputs four rows ahead on the large maps (measured at batch 32, operands from memory: 112x112
  // 16 -> 96 stride 2: 33 against 37 us; 56x56 24 -> 144 stride 1: 36 against 41; a loss of 1 us on
  // 56x56 stride 2 and on 28x28).
  g.ahead = (g.k_steps == 0 && g.out_w * g.stride >= 56 && (g.stride == 1 || g.cin <= 16)) ? 4 : 2;
  // Output rows per wavefront. The launch is bound by its arithmetic, which the wavefronts of a compute
  // unit share, so it lasts as long as the compute unit with the most workgroups needs for them: the
  // number of workgroups per compute unit, rounded up, times the row steps of a wavefront (its rows,
  // the two rows of halo a stride-1 chunk computes again, and about a step and a half of set-up). A
  // single wavefront per SIMD has nobody to hide its waits behind and is priced a quarter higher.
  // The row count with the lowest price wins, the larger one on a tie. (Measured at batch 32 on
  // MobileNetV2's shapes, this order of the candidates is the measured one: 56x56 / 144 channels,
  // stride 1: 14 rows 22.1 us, 28 rows 24.2, 7 rows 23.4; stride 2: 6 rows 16.8, 7 rows 18.4, 14 rows 21.6.)
  const int forced = tuning(kTuneStreamRows);
  int rows = g.out_h;
  {
    const long long cus = num_cus();
    double best = 0;
    for (int cand = g.out_h < 4 ? g.out_h : 4; cand <= g.out_h; ++cand) {
      const long long chunks = (g.out_h + cand - 1) / cand;
      const long long groups = ((long long)g.batch * chunks * g.strips * cgroups + 3) / 4;
      const long long per_cu = (groups + cus - 1) / cus;
      const double steps = cand + (g.stride == 1 ? 2.0 : 0.5) + 1.5;
      const double price = (double)per_cu * steps * (per_cu < 2 ? 1.25 : 1.0);
      if (cand == (g.out_h < 4 ? g.out_h : 4) || price <= best) {
        best = price;
        rows = cand;
      }
    }
  }
  if (forced > 0) rows = forced < g.out_h ? forced : g.out_h;
  g.rows = rows;
  g.chunks_h = (g.out_h + rows - 1) / rows;
  g.waves = (long long)g.batch * g.chunks_h * g.strips * cgroups;
  g.through = (long long)g.out_h * g.out_w * g.c * 4 <= 0xfffffff0LL ? 1 : 0;
  return true;
}

int launch_expand_dw_stream(const ExpandDwStreamArgs &g) {
  return g.stride == 1 ? launch_stream_k<1>(g) : launch_stream_k<2>(g);
}

int launch_stem_dw_stream(const ExpandDwStreamArgs &g, const StemTaps &taps) {
  return g.stride == 1 ? launch_stream_taps<1>(g, taps) : launch_stream_taps<2>(g, taps);
}

}  // namespace tfhip
