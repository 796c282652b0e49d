// FusedDepthwiseConv2D, NHWC float32.
//
// Bandwidth-bound (about 2 flops per byte), so no matrix cores. Three kernels:
//  * depthwise_3x3_rows: 3x3, stride 1 or 2, channel multiplier 1 (every
//    MobileNet layer). A register row pipeline: each input row is fetched once
//    per lane as float4 over the contiguous channel axis and scattered into
//    rotating accumulators; no LDS, no barriers.
//  * depthwise_3x3_halo: the same shapes when a tensor is too large for 32-bit
//    buffer offsets; stages an input halo tile of 32 channels in LDS.
//  * depthwise_generic: any filter, stride, dilation, channel multiplier.
// Each output accumulates its taps in the reference's own order (filter row,
// then filter column: tfjs-backend-cpu/src/kernels/DepthwiseConv2dNative.ts:62-95)
// with one fused multiply-add per tap, which is the reference's
// "fround(y + x*w)" per tap up to double rounding.
#include <stdlib.h>

#include "common.h"
#include "epilogue.h"

namespace tfhip {
namespace {

struct DwParams {
  const float *x;
  const float *w;
  float *y;
  int batch, in_h, in_w, in_c;
  int f_h, f_w, ch_mul;
  int stride_h, stride_w, dil_h, dil_w;
  int pad_top, pad_left, out_h, out_w;
};

// ---- general kernel: any filter, stride, dilation, channel multiplier -------
__global__ __launch_bounds__(256) void depthwise_generic(DwParams p, Epilogue e, long long total) {
  const long long out_c = (long long)p.in_c * p.ch_mul;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
    const long long oc = idx % out_c;
    long long t = idx / out_c;
    const int ow = (int)(t % p.out_w);
    t /= p.out_w;
    const int oh = (int)(t % p.out_h);
    const int n = (int)(t / p.out_h);
    const int d1 = (int)(oc / p.ch_mul), q = (int)(oc % p.ch_mul);
    const float *xb = p.x + (long long)n * p.in_h * p.in_w * p.in_c;
    float acc = 0.f;
    for (int r = 0; r < p.f_h; ++r) {
      const int ih = oh * p.stride_h - p.pad_top + r * p.dil_h;
      if (ih < 0 || ih >= p.in_h) continue;
      for (int s = 0; s < p.f_w; ++s) {
        const int iw = ow * p.stride_w - p.pad_left + s * p.dil_w;
        if (iw < 0 || iw >= p.in_w) continue;
        const float xv = xb[((long long)ih * p.in_w + iw) * p.in_c + d1];
        const float wv = p.w[(((long long)r * p.f_w + s) * p.in_c + d1) * p.ch_mul + q];
        acc = fmaf(xv, wv, acc);
      }
    }
    p.y[idx] = finish(e, acc, 0, 0, oc, n, oh, ow);
  }
}

// ---- 3x3, channel multiplier 1, dilation 1, stride S in both directions -----
constexpr int kCQ = 8;              // float4 channel groups per workgroup: 32 channels
constexpr int kSlots = 256 / kCQ;   // output pixels computed per pass

template <int S>
__global__ __launch_bounds__(256) void depthwise_3x3_halo(DwParams p, Epilogue e, int tile_h, int tile_w,
                                                          int tiles_w, int c4_total) {
  extern __shared__ float4 halo[];  // [in_tile_h][in_tile_w][kCQ]
  const int in_tile_h = (tile_h - 1) * S + 3;
  const int in_tile_w = (tile_w - 1) * S + 3;
  const int tile_y = blockIdx.x / tiles_w, tile_x = blockIdx.x % tiles_w;
  const int cq0 = blockIdx.y * kCQ;
  const int n = blockIdx.z;
  const int oh0 = tile_y * tile_h, ow0 = tile_x * tile_w;
  const int ih0 = oh0 * S - p.pad_top, iw0 = ow0 * S - p.pad_left;
  const float4 *x4 = reinterpret_cast<const float4 *>(p.x) + (long long)n * p.in_h * p.in_w * c4_total;
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);

  const int halo_items = in_tile_h * in_tile_w * kCQ;
  for (int i = threadIdx.x; i < halo_items; i += 256) {
    const int c4 = i % kCQ;
    const int pos = i / kCQ;
    const int iy = pos / in_tile_w, ix = pos % in_tile_w;
    const int ih = ih0 + iy, iw = iw0 + ix;
    float4 v = zero;
    if (ih >= 0 && ih < p.in_h && iw >= 0 && iw < p.in_w && cq0 + c4 < c4_total) {
      v = x4[((long long)ih * p.in_w + iw) * c4_total + cq0 + c4];
    }
    halo[i] = v;
  }

  const int c4 = threadIdx.x % kCQ;
  const int slot = threadIdx.x / kCQ;
  const bool c_ok = cq0 + c4 < c4_total;
  float4 w[9];
  const float4 *w4 = reinterpret_cast<const float4 *>(p.w);
#pragma unroll
  for (int t = 0; t < 9; ++t) w[t] = c_ok ? w4[(long long)t * c4_total + cq0 + c4] : zero;
  __syncthreads();
  if (!c_ok) return;

  const int c = (cq0 + c4) * 4;
  float4 *y4 = reinterpret_cast<float4 *>(p.y);
  const int pixels = tile_h * tile_w;
  for (int pix = slot; pix < pixels; pix += kSlots) {
    const int oy = pix / tile_w, ox = pix % tile_w;
    const int oh = oh0 + oy, ow = ow0 + ox;
    if (oh >= p.out_h || ow >= p.out_w) continue;
    float4 acc = zero;
#pragma unroll
    for (int r = 0; r < 3; ++r) {
#pragma unroll
      for (int s = 0; s < 3; ++s) {
        const float4 xv = halo[((oy * S + r) * in_tile_w + ox * S + s) * kCQ + c4];
        const float4 wv = w[r * 3 + s];
        acc.x = fmaf(xv.x, wv.x, acc.x);
        acc.y = fmaf(xv.y, wv.y, acc.y);
        acc.z = fmaf(xv.z, wv.z, acc.z);
        acc.w = fmaf(xv.w, wv.w, acc.w);
      }
    }
    float4 o;
    o.x = finish(e, acc.x, 0, 0, c + 0, n, oh, ow);
    o.y = finish(e, acc.y, 0, 0, c + 1, n, oh, ow);
    o.z = finish(e, acc.z, 0, 0, c + 2, n, oh, ow);
    o.w = finish(e, acc.w, 0, 0, c + 3, n, oh, ow);
    store_result4(reinterpret_cast<float *>(y4 + (((long long)n * p.out_h + oh) * p.out_w + ow) * c4_total + cq0 + c4), o);
  }
}


// ---- 3x3, channel multiplier 1, dilation 1, stride S: register row pipeline ----
// Each lane owns four channels (one float4) of a strip of 4 output columns and
// walks down `rows` output rows. Every input row it needs is fetched exactly
// once by that lane (4*S + 2 float4 loads: the 8 lanes that share a pixel read
// one contiguous 128-byte line, the column overlap with the neighbouring strip
// is served by the vector cache) and is scattered at once into the accumulators
// of the up to three output rows it contributes to, which live in registers and
// rotate as rows complete. The loads of input row i+1 are issued before the
// arithmetic of row i. No barriers, no LDS: the only traffic besides the
// compulsory reads and writes is the halo rows of vertically adjacent chunks.
//
// All accesses are buffer loads/stores over the whole tensor with 32-bit byte
// offsets: padding taps and ragged edges use an offset outside the descriptor,
// which reads as zero and drops stores, so the row pipeline has no branches.
constexpr int kRowsPW = 4;   // output columns per lane
#ifndef DW_WAVES
#define DW_WAVES 1
#endif
constexpr unsigned kDwNoOffset = 0xffffffffu;
// Results of at least this many bytes are stored non-temporally: an L2 holds 4 MB,
// so such a result cannot wait there for its reader (measured with operands from
// memory: 51 MB 21.3 -> 20.3 us, 12 MB at stride 2 13.7 -> 12.7 us; written through
// instead, 21.6 and 13.6 us).
constexpr long long kDwStreamBytes = 8LL << 20;
typedef unsigned int dw_uint4 __attribute__((ext_vector_type(4)));

struct DwRowsArgs {
  int strips_w;      // column strips per output row
  int chunks_h;      // row chunks per image
  int rows;          // output rows per chunk
  int c4_total;
  long long strips;  // batch * chunks_h * strips_w
  unsigned x_bytes, y_bytes;
};

template <int S>
struct DwRowsState {
  static constexpr int NIN = (kRowsPW - 1) * S + 3;   // input columns a strip needs
  static constexpr int NSLOT = S == 1 ? 3 : 2;          // output rows in flight
  float4 acc[NSLOT][kRowsPW];
  float4 w[9];
  float4 bias4;               // per-channel bias of this lane (channel addressing)
  unsigned x_col[NIN];        // byte offset of input column j (+ channel group) within a row, or kDwNoOffset
  unsigned y_col[kRowsPW];    // same for the output columns
  unsigned x_img, y_img;      // byte offset of the image
  unsigned x_row, y_row;      // bytes per row
  int in_h, out_h, ih0, oh0, ow0, rows, rows_in, c, n;
};

__device__ __forceinline__ float4 dw_load4(__amdgpu_buffer_rsrc_t r, unsigned off) {
#ifndef TFHIP_DW_LOAD_AUX
#define TFHIP_DW_LOAD_AUX 0
#endif
  const dw_uint4 v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)off, 0, TFHIP_DW_LOAD_AUX);
  return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
}

// STREAM: a non-temporal store, for a result too large to still be in the cache
// when its reader starts (it would only push out what the reader does find there).
template <bool STREAM>
__device__ __forceinline__ void dw_store4(__amdgpu_buffer_rsrc_t r, unsigned off, float4 v) {
  dw_uint4 u;
  u.x = __float_as_uint(v.x); u.y = __float_as_uint(v.y); u.z = __float_as_uint(v.z); u.w = __float_as_uint(v.w);
  __builtin_amdgcn_raw_buffer_store_b128(u, r, (int)off, 0, (STREAM || TFHIP_NT_OUT) ? 2 : 0);
}

// Bias + activation of four channels. The common case (per-channel operands,
// relu-family activation) is a handful of instructions inline; anything else
// takes one out-of-line call so that the row pipeline stays small.
__device__ __noinline__ float4 dw_finish4_general(const Epilogue &e, float4 a, int c, int n, int oh, int ow) {
  float4 r;
  r.x = finish(e, a.x, 0, 0, c + 0, n, oh, ow);
  r.y = finish(e, a.y, 0, 0, c + 1, n, oh, ow);
  r.z = finish(e, a.z, 0, 0, c + 2, n, oh, ow);
  r.w = finish(e, a.w, 0, 0, c + 3, n, oh, ow);
  return r;
}

__device__ __forceinline__ float relu_family(float v, int act) {
  if (act == TFHIP_LINEAR) return v;
  const float t = (v > 0.f || v != v) ? v : 0.f;     // Math.max(0, x): NaN stays, -0 becomes +0
  return (act == TFHIP_RELU6 && t > 6.f) ? 6.f : t;
}

template <bool GENERAL>
__device__ __forceinline__ float4 dw_finish4(const Epilogue &e, float4 a, float4 bias4, int c, int n, int oh, int ow) {
  if (!GENERAL) {
    float4 r;
    r.x = relu_family(a.x + bias4.x, e.activation);
    r.y = relu_family(a.y + bias4.y, e.activation);
    r.z = relu_family(a.z + bias4.z, e.activation);
    r.w = relu_family(a.w + bias4.w, e.activation);
    return r;
  }
  return dw_finish4_general(e, a, c, n, oh, ow);
}

// Issues the loads of input row i of the chunk (relative to its first input row).
template <int S>
__device__ __forceinline__ void dw_load_row(const DwRowsState<S> &st, __amdgpu_buffer_rsrc_t rx, int i,
                                            float4 (&in)[DwRowsState<S>::NIN]) {
  const int ih = st.ih0 + i;
  const bool row_ok = ih >= 0 && ih < st.in_h && i < st.rows_in;
  const unsigned row_off = st.x_img + (unsigned)ih * st.x_row;
#pragma unroll
  for (int j = 0; j < DwRowsState<S>::NIN; ++j) {
    const unsigned off = (row_ok && st.x_col[j] != kDwNoOffset) ? row_off + st.x_col[j] : kDwNoOffset;
    in[j] = dw_load4(rx, off);
  }
}

// Scatters input row i into the output rows it is a tap row of; PHASE is i
// modulo the rotation period of the accumulators, so slots are compile-time.
template <int S, int PHASE, bool GENERAL, bool STREAM>
__device__ __forceinline__ void dw_compute_row(DwRowsState<S> &st, const Epilogue &e, __amdgpu_buffer_rsrc_t ry,
                                               int i, const float4 (&in)[DwRowsState<S>::NIN]) {
  using St = DwRowsState<S>;
  constexpr int PERIOD = S * St::NSLOT;
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (int wr = 0; wr < 3; ++wr) {
    constexpr int kBig = 4 * PERIOD;
    if ((PHASE - wr + kBig) % S != 0) continue;          // this input row is not tap row `wr` of any output row
    const int o = (i - wr) / S;                            // output row (relative to the chunk) it feeds
    if (i - wr < 0 || o >= st.rows) continue;
    const int slot = ((PHASE - wr + kBig) / S) % St::NSLOT;
#pragma unroll
    for (int x = 0; x < kRowsPW; ++x) {
      float4 a = wr == 0 ? zero : st.acc[slot][x];
#pragma unroll
      for (int wc = 0; wc < 3; ++wc) {
        const float4 xv = in[x * S + wc];
        const float4 wv = st.w[wr * 3 + wc];
        a.x = fmaf(xv.x, wv.x, a.x);
        a.y = fmaf(xv.y, wv.y, a.y);
        a.z = fmaf(xv.z, wv.z, a.z);
        a.w = fmaf(xv.w, wv.w, a.w);
      }
      st.acc[slot][x] = a;
    }
    if (wr == 2) {
      // the row is complete: bias + activation, one float4 store per column
      const int oh = st.oh0 + o;
      const bool row_ok = oh < st.out_h;
      const unsigned row_off = st.y_img + (unsigned)oh * st.y_row;
#pragma unroll
      for (int x = 0; x < kRowsPW; ++x) {
        const unsigned off = (row_ok && st.y_col[x] != kDwNoOffset) ? row_off + st.y_col[x] : kDwNoOffset;
        dw_store4<STREAM>(ry, off, dw_finish4<GENERAL>(e, st.acc[slot][x], st.bias4, st.c, st.n, oh, st.ow0 + x));
      }
    }
  }
}

// One pipeline step: `a` holds input row i0+K, `b` receives row i0+K+1.
template <int S, int K, bool GENERAL, bool STREAM>
__device__ __forceinline__ void dw_step(DwRowsState<S> &st, const Epilogue &e, __amdgpu_buffer_rsrc_t rx,
                                        __amdgpu_buffer_rsrc_t ry, int i0, const float4 (&a)[DwRowsState<S>::NIN],
                                        float4 (&b)[DwRowsState<S>::NIN]) {
  constexpr int PERIOD = S * DwRowsState<S>::NSLOT;
  if (i0 + K >= st.rows_in) return;
  dw_load_row<S>(st, rx, i0 + K + 1, b);
  dw_compute_row<S, K % PERIOD, GENERAL, STREAM>(st, e, ry, i0 + K, a);
}

// GENERAL = false: per-channel bias and a relu-family activation, all inline.
template <int S, bool GENERAL, bool STREAM>
__global__ __launch_bounds__(256, DW_WAVES) void depthwise_3x3_rows(DwParams p, Epilogue e, DwRowsArgs g) {
  using St = DwRowsState<S>;
  const int c4 = blockIdx.y * kCQ + (threadIdx.x % kCQ);
  const long long strip = (long long)blockIdx.x * kSlots + threadIdx.x / kCQ;
  if (c4 >= g.c4_total || strip >= g.strips) return;
  const int sw = (int)(strip % g.strips_w);
  const long long t = strip / g.strips_w;
  const int ch = (int)(t % g.chunks_h);
  const int n = (int)(t / g.chunks_h);
  const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc((void *)p.x, 0, (int)g.x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc((void *)p.y, 0, (int)g.y_bytes, 0x00020000);

  St st;
  st.in_h = p.in_h; st.out_h = p.out_h;
  st.oh0 = ch * g.rows;
  st.ow0 = sw * kRowsPW;
  st.ih0 = st.oh0 * S - p.pad_top;
  st.rows = g.rows;
  st.rows_in = (g.rows - 1) * S + 3;
  st.c = c4 * 4;
  st.n = n;
  const unsigned pix = (unsigned)g.c4_total * 16u;   // bytes per pixel
  st.x_row = (unsigned)p.in_w * pix;
  st.y_row = (unsigned)p.out_w * pix;
  st.x_img = (unsigned)n * (unsigned)p.in_h * st.x_row;
  st.y_img = (unsigned)n * (unsigned)p.out_h * st.y_row;
  const int iw0 = st.ow0 * S - p.pad_left;
#pragma unroll
  for (int j = 0; j < St::NIN; ++j) {
    const int iw = iw0 + j;
    st.x_col[j] = (iw >= 0 && iw < p.in_w) ? (unsigned)iw * pix + (unsigned)c4 * 16u : kDwNoOffset;
  }
#pragma unroll
  for (int x = 0; x < kRowsPW; ++x) {
    const int ow = st.ow0 + x;
    st.y_col[x] = ow < p.out_w ? (unsigned)ow * pix + (unsigned)c4 * 16u : kDwNoOffset;
  }
  const float4 *w4 = reinterpret_cast<const float4 *>(p.w) + c4;
#pragma unroll
  for (int k = 0; k < 9; ++k) st.w[k] = w4[(long long)k * g.c4_total];
  st.bias4 = make_float4(0.f, 0.f, 0.f, 0.f);
  if (!GENERAL && e.bias) {
    const long long bs = e.bias_s[3];
    st.bias4 = make_float4(e.bias[(st.c + 0) * bs], e.bias[(st.c + 1) * bs], e.bias[(st.c + 2) * bs],
                           e.bias[(st.c + 3) * bs]);
  }

  // The two row buffers swap roles every step, so the loop is unrolled by an
  // even multiple of the accumulator rotation period.
  constexpr int PERIOD = S * St::NSLOT;
  constexpr int UNROLL = PERIOD % 2 == 0 ? PERIOD : 2 * PERIOD;
  float4 cur[St::NIN], nxt[St::NIN];
  dw_load_row<S>(st, rx, 0, cur);
  for (int i0 = 0; i0 < st.rows_in; i0 += UNROLL) {
    dw_step<S, 0, GENERAL, STREAM>(st, e, rx, ry, i0, cur, nxt);
    dw_step<S, 1, GENERAL, STREAM>(st, e, rx, ry, i0, nxt, cur);
    dw_step<S, 2, GENERAL, STREAM>(st, e, rx, ry, i0, cur, nxt);
    dw_step<S, 3, GENERAL, STREAM>(st, e, rx, ry, i0, nxt, cur);
    if (UNROLL > 4) {
      dw_step<S, 4, GENERAL, STREAM>(st, e, rx, ry, i0, cur, nxt);
      dw_step<S, 5, GENERAL, STREAM>(st, e, rx, ry, i0, nxt, cur);
    }
  }
}

// The same strip of four output columns, but a single output row per lane with
// its three input rows fetched at once: one memory round trip instead of a
// chain of them. For feature maps so small that the whole launch is a wave or
// two of lanes, where the row pipeline above never fills.
template <int S, bool GENERAL>
__global__ __launch_bounds__(256) void depthwise_3x3_flat(DwParams p, Epilogue e, DwRowsArgs g) {
  using St = DwRowsState<S>;
  const int c4 = blockIdx.y * kCQ + (threadIdx.x % kCQ);
  const long long strip = (long long)blockIdx.x * kSlots + threadIdx.x / kCQ;
  if (c4 >= g.c4_total || strip >= g.strips) return;
  const int sw = (int)(strip % g.strips_w);
  const long long t = strip / g.strips_w;
  const int oh = (int)(t % p.out_h);
  const int n = (int)(t / p.out_h);
  const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc((void *)p.x, 0, (int)g.x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc((void *)p.y, 0, (int)g.y_bytes, 0x00020000);

  St st;
  st.in_h = p.in_h; st.out_h = p.out_h;
  st.oh0 = oh;
  st.ow0 = sw * kRowsPW;
  st.ih0 = oh * S - p.pad_top;
  st.rows = 1;
  st.rows_in = 3;
  st.c = c4 * 4;
  st.n = n;
  const unsigned pix = (unsigned)g.c4_total * 16u;   // bytes per pixel
  st.x_row = (unsigned)p.in_w * pix;
  st.y_row = (unsigned)p.out_w * pix;
  st.x_img = (unsigned)n * (unsigned)p.in_h * st.x_row;
  st.y_img = (unsigned)n * (unsigned)p.out_h * st.y_row;
  const int iw0 = st.ow0 * S - p.pad_left;
#pragma unroll
  for (int j = 0; j < St::NIN; ++j) {
    const int iw = iw0 + j;
    st.x_col[j] = (iw >= 0 && iw < p.in_w) ? (unsigned)iw * pix + (unsigned)c4 * 16u : kDwNoOffset;
  }
#pragma unroll
  for (int x = 0; x < kRowsPW; ++x) {
    const int ow = st.ow0 + x;
    st.y_col[x] = ow < p.out_w ? (unsigned)ow * pix + (unsigned)c4 * 16u : kDwNoOffset;
  }
  float4 r0[St::NIN], r1[St::NIN], r2[St::NIN];
  dw_load_row<S>(st, rx, 0, r0);
  dw_load_row<S>(st, rx, 1, r1);
  dw_load_row<S>(st, rx, 2, r2);
  const float4 *w4 = reinterpret_cast<const float4 *>(p.w) + c4;
#pragma unroll
  for (int k = 0; k < 9; ++k) st.w[k] = w4[(long long)k * g.c4_total];
  st.bias4 = make_float4(0.f, 0.f, 0.f, 0.f);
  if (!GENERAL && e.bias) {
    const long long bs = e.bias_s[3];
    st.bias4 = make_float4(e.bias[(st.c + 0) * bs], e.bias[(st.c + 1) * bs], e.bias[(st.c + 2) * bs],
                           e.bias[(st.c + 3) * bs]);
  }
  dw_compute_row<S, 0, GENERAL, false>(st, e, ry, 0, r0);
  dw_compute_row<S, 1, GENERAL, false>(st, e, ry, 1, r1);
  dw_compute_row<S, 2, GENERAL, false>(st, e, ry, 2, r2);
}

int balanced_tile(int extent, int max_tile) {
  const int tiles = (extent + max_tile - 1) / max_tile;
  return (extent + tiles - 1) / tiles;
}

// Output rows per lane for the row pipeline. A lane that walks more rows
// re-reads fewer halo rows (each chunk of r output rows fetches (r-1)*S+3 input
// rows) but is a longer serial chain of row fetches, and fewer, longer chains
// may not keep enough loads in flight. The estimate below is
// max(latency chain, traffic / bandwidth) with constants fitted to sweeps over
// r on MI355X (one row fetch per lane is about 0.8 us of memory latency, one
// wavefront sustains about 7.5 GB/s, the chip about 6.5 TB/s; halo rows of a
// working set that fits the 256 MB memory-side cache mostly hit it).
int choose_rows(int batch, int in_h, int in_w, int in_c, int out_h, int out_w, int S, int cus) {
  const double in_bytes = 4.0 * batch * in_h * in_w * in_c;
  const double out_bytes = 4.0 * batch * out_h * out_w * in_c;
  const int strips_w = (out_w + kRowsPW - 1) / kRowsPW;
  const int c_blocks = (in_c / 4 + kCQ - 1) / kCQ;
  const long long slots = (long long)cus * 8;   // resident wavefronts: two per SIMD at this kernel's register count
  const bool cached = in_bytes + out_bytes <= 250e6;
  int best = 1;
  double best_t = 1e30;
  for (int r = 1; r <= 24 && r <= out_h; ++r) {
    const int chunks = (out_h + r - 1) / r;
    const int rb = (out_h + chunks - 1) / chunks;
    if (rb != r) continue;   // the balanced tile is what runs: only score those
    const int rows_in = (rb - 1) * S + 3;
    const long long wgs = (((long long)batch * chunks * strips_w + kSlots - 1) / kSlots) * c_blocks;
    const long long waves = wgs * 4;
    const long long rounds = (waves + slots - 1) / slots;
    const double halo = (double)chunks * rows_in / in_h;
    const double traffic = in_bytes * (cached ? 1.0 + (halo - 1.0) * 0.3 : halo) + out_bytes;
    const double wave_bw = 7500.0 * (S == 2 ? 1.5 : 1.0);   // bytes per us
    const double conc = (double)(waves < slots ? waves : slots);
    const double bw = conc * wave_bw < 6.5e6 ? conc * wave_bw : 6.5e6;
    // workgroups that do not fill the compute units evenly leave some idle at the
    // end (measured at stride 1: 294 workgroups on 256 units run 8% longer than 252;
    // at stride 2 the effect is not seen)
    // (a last channel block that is partly empty counts by its share of lanes)
    const double full_wgs = (double)(wgs / c_blocks) * (in_c / 4) / kCQ;
    const double per_cu = ceil(full_wgs / cus);
    const double balance = S == 1 ? full_wgs / (per_cu * cus) : 1.0;
    const double t_bw = traffic / bw / (0.85 + 0.15 * balance);
    const double t_lat = rounds * (1.5 + rows_in * 0.8);
    const double t = t_lat > t_bw ? t_lat : t_bw;
    if (t < best_t) { best_t = t; best = r; }
  }
  return best;
}

}  // namespace
}  // namespace tfhip

using namespace tfhip;

extern "C" int tfhip_fused_depthwise_conv2d(
    const float *x, const float *filter, float *y, int64_t batch, int64_t in_h, int64_t in_w,
    int64_t in_c, int64_t f_h, int64_t f_w, int64_t ch_mul, int64_t stride_h, int64_t stride_w,
    int64_t dilation_h, int64_t dilation_w, int64_t pad_top, int64_t pad_left, int64_t out_h,
    int64_t out_w, const float *bias, const int64_t bias_strides[4], int activation,
    const float *prelu_weights, const int64_t prelu_strides[4], double leakyrelu_alpha) {
  TFHIP_REQUIRE_INIT();
  TFHIP_CHECK_ARG(batch >= 0 && in_h > 0 && in_w > 0 && in_c > 0 && f_h > 0 && f_w > 0 && ch_mul > 0 &&
                      stride_h > 0 && stride_w > 0 && dilation_h > 0 && dilation_w > 0 && out_h >= 0 &&
                      out_w >= 0,
                  "tfhip_fused_depthwise_conv2d: non-positive dimension");
  TFHIP_CHECK_ARG(activation >= TFHIP_LINEAR && activation <= TFHIP_ELU,
                  "tfhip_fused_depthwise_conv2d: unknown activation %d", activation);
  TFHIP_CHECK_ARG(activation != TFHIP_PRELU || prelu_weights != nullptr,
                  "tfhip_fused_depthwise_conv2d: prelu activation without weights");
  const int64_t lim = 0x7fffffff;
  TFHIP_CHECK_ARG(batch < lim && in_h < lim && in_w < lim && in_c * ch_mul < lim && out_h < lim && out_w < lim,
                  "tfhip_fused_depthwise_conv2d: dimension exceeds 2^31-1");
  TFHIP_CHECK_ARG(pad_top >= 0 && pad_left >= 0, "tfhip_fused_depthwise_conv2d: negative padding");
  const int64_t out_c = in_c * ch_mul;
  const int64_t total = batch * out_h * out_w * out_c;
  if (total == 0) return kOk;
  TFHIP_CHECK_RANGE(x, batch * in_h * in_w * in_c, 4, "x");
  TFHIP_CHECK_RANGE(filter, f_h * f_w * in_c * ch_mul, 4, "filter");
  TFHIP_CHECK_OUTPUT(y, total, 4, "y");
  const int64_t dims[4] = {batch, out_h, out_w, out_c};

  Epilogue e = {};
  e.activation = activation;
  e.leaky_alpha = leakyrelu_alpha;
  e.addressing = kConv;
  e.out_h = (int)out_h;
  e.out_w = (int)out_w;
  bool channel_only = true;
  if (bias) {
    TFHIP_CHECK_ARG(bias_strides != nullptr, "tfhip_fused_depthwise_conv2d: bias without strides");
    for (int i = 0; i < 4; ++i) {
      TFHIP_CHECK_ARG(bias_strides[i] >= 0, "tfhip_fused_depthwise_conv2d: negative bias stride");
      e.bias_s[i] = bias_strides[i];
      if (i < 3 && bias_strides[i] != 0) channel_only = false;
    }
    TFHIP_CHECK_RANGE(bias, strided_extent(dims, bias_strides, 4), 4, "bias");
    e.bias = bias;
  }
  if (activation == TFHIP_PRELU) {
    TFHIP_CHECK_ARG(prelu_strides != nullptr, "tfhip_fused_depthwise_conv2d: prelu weights without strides");
    for (int i = 0; i < 4; ++i) {
      TFHIP_CHECK_ARG(prelu_strides[i] >= 0, "tfhip_fused_depthwise_conv2d: negative prelu stride");
      e.prelu_s[i] = prelu_strides[i];
      if (i < 3 && prelu_strides[i] != 0) channel_only = false;
    }
    TFHIP_CHECK_RANGE(prelu_weights, strided_extent(dims, prelu_strides, 4), 4, "prelu_weights");
    e.prelu = prelu_weights;
  }
  if (channel_only) e.addressing = kChannel;

  DwParams p;
  p.x = x; p.w = filter; p.y = y;
  p.batch = (int)batch; p.in_h = (int)in_h; p.in_w = (int)in_w; p.in_c = (int)in_c;
  p.f_h = (int)f_h; p.f_w = (int)f_w; p.ch_mul = (int)ch_mul;
  p.stride_h = (int)stride_h; p.stride_w = (int)stride_w; p.dil_h = (int)dilation_h; p.dil_w = (int)dilation_w;
  p.pad_top = (int)pad_top; p.pad_left = (int)pad_left; p.out_h = (int)out_h; p.out_w = (int)out_w;

  const bool aligned16 = reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(filter) % 16 == 0 &&
                         reinterpret_cast<uintptr_t>(y) % 16 == 0;
  // The 3x3 kernels read a zero for a tap outside the image and multiply it by the filter value; the
  // reference skips the tap (DepthwiseConv2dNative.ts:72-86), which differs under a value that is not
  // finite: such a filter, where a window can reach outside, takes the general kernel, which skips.
  const bool taps_can_miss = pad_top > 0 || pad_left > 0 ||
                             (out_h - 1) * stride_h - pad_top + (f_h - 1) * dilation_h >= in_h ||
                             (out_w - 1) * stride_w - pad_left + (f_w - 1) * dilation_w >= in_w;
  bool nonfinite = false;
  if (taps_can_miss) {
    const int rc = scan_filter(filter, f_h * f_w * in_c * ch_mul, "tfhip_fused_depthwise_conv2d", &nonfinite);
    if (rc != kOk) return rc;
  }
  const bool fast = f_h == 3 && f_w == 3 && ch_mul == 1 && dilation_h == 1 && dilation_w == 1 &&
                    stride_h == stride_w && (stride_h == 1 || stride_h == 2) && in_c % 4 == 0 && aligned16 &&
                    batch <= 65535 && !nonfinite;
  // the row pipeline addresses both tensors with 32-bit byte offsets
  const bool fits32 = batch * in_h * in_w * in_c * 4 <= 0xfffffff0LL && total * 4 <= 0xfffffff0LL;
  if (fast && fits32 && tuning(kTuneDwHalo) <= 0) {
    const int S = (int)stride_h;
    DwRowsArgs g;
    g.c4_total = (int)(in_c / 4);
    g.strips_w = ((int)out_w + kRowsPW - 1) / kRowsPW;
    {
      // one output row per lane when all its wavefronts are resident at once and the
      // input is small enough for its rows, each fetched by up to three output rows,
      // to come from cache (measured against the row pipeline: 5-15% faster up to
      // about 3000 wavefronts and 24 MB, slower beyond either)
      const long long flat_strips = (long long)batch * out_h * g.strips_w;
      const long long flat_blocks = (flat_strips + kSlots - 1) / kSlots;
      const long long flat_waves = flat_blocks * ((g.c4_total + kCQ - 1) / kCQ) * 4;
      const int forced = tuning(kTuneDwFlat);
      const bool flat = forced >= 0 ? forced > 0 : (tuning(kTuneDwRows) <= 0 && flat_waves <= (long long)num_cus() * 12 &&
                                              batch * in_h * in_w * in_c * 4 <= 24000000);
      if (flat && flat_blocks <= 0x7fffffffLL) {
        g.rows = 1;
        g.chunks_h = (int)out_h;
        g.strips = flat_strips;
        g.x_bytes = (unsigned)(batch * in_h * in_w * in_c * 4);
        g.y_bytes = (unsigned)(total * 4);
        dim3 grid((unsigned)flat_blocks, (g.c4_total + kCQ - 1) / kCQ, 1);
        const bool general = !(e.addressing == kChannel && activation <= TFHIP_RELU6);
        note_kernel("depthwise_3x3_flat<%d, %s>", S, general ? "true" : "false");
        if (S == 1 && !general)
          TFHIP_LAUNCH((depthwise_3x3_flat<1, false><<<grid, 256, 0, stream()>>>(p, e, g)));
        else if (S == 1)
          TFHIP_LAUNCH((depthwise_3x3_flat<1, true><<<grid, 256, 0, stream()>>>(p, e, g)));
        else if (!general)
          TFHIP_LAUNCH((depthwise_3x3_flat<2, false><<<grid, 256, 0, stream()>>>(p, e, g)));
        else
          TFHIP_LAUNCH((depthwise_3x3_flat<2, true><<<grid, 256, 0, stream()>>>(p, e, g)));
        return kOk;
      }
    }
    int rows = choose_rows((int)batch, (int)in_h, (int)in_w, (int)in_c, (int)out_h, (int)out_w, S, num_cus());
    if (tuning(kTuneDwRows) > 0) rows = tuning(kTuneDwRows);   // tuning override
    rows = rows < 1 ? 1 : (rows > 32 ? 32 : rows);
    if (rows > out_h) rows = (int)out_h;
    g.rows = balanced_tile((int)out_h, rows);
    g.chunks_h = ((int)out_h + g.rows - 1) / g.rows;
    g.strips = (long long)batch * g.chunks_h * g.strips_w;
    g.x_bytes = (unsigned)(batch * in_h * in_w * in_c * 4);
    g.y_bytes = (unsigned)(total * 4);
    const long long blocks_x = (g.strips + kSlots - 1) / kSlots;
    if (blocks_x <= 0x7fffffffLL) {
      dim3 grid((unsigned)blocks_x, (g.c4_total + kCQ - 1) / kCQ, 1);
      const bool general = !(e.addressing == kChannel && activation <= TFHIP_RELU6);
      const bool streamed = !general && total * 4 >= kDwStreamBytes;
      note_kernel("depthwise_3x3_rows<%d, %s, %s>", S, general ? "true" : "false", streamed ? "true" : "false");
      if (S == 1 && streamed)
        TFHIP_LAUNCH((depthwise_3x3_rows<1, false, true><<<grid, 256, 0, stream()>>>(p, e, g)));
      else if (S == 1 && !general)
        TFHIP_LAUNCH((depthwise_3x3_rows<1, false, false><<<grid, 256, 0, stream()>>>(p, e, g)));
      else if (S == 1)
        TFHIP_LAUNCH((depthwise_3x3_rows<1, true, false><<<grid, 256, 0, stream()>>>(p, e, g)));
      else if (streamed)
        TFHIP_LAUNCH((depthwise_3x3_rows<2, false, true><<<grid, 256, 0, stream()>>>(p, e, g)));
      else if (!general)
        TFHIP_LAUNCH((depthwise_3x3_rows<2, false, false><<<grid, 256, 0, stream()>>>(p, e, g)));
      else
        TFHIP_LAUNCH((depthwise_3x3_rows<2, true, false><<<grid, 256, 0, stream()>>>(p, e, g)));
      return kOk;
    }
  }
  if (fast) {
    const int S = (int)stride_h;
    const int c4_total = (int)(in_c / 4);
    const int tile_w = balanced_tile((int)out_w, 16);
    // about 128 output pixels per workgroup, shrunk until the halo fits 48 KiB of LDS
    int cap_h = 128 / tile_w;
    cap_h = cap_h < 1 ? 1 : (cap_h > 16 ? 16 : cap_h);
    int tile_h = balanced_tile((int)out_h, cap_h);
    size_t lds = 0;
    for (;;) {
      const int in_tile_h = (tile_h - 1) * S + 3, in_tile_w = (tile_w - 1) * S + 3;
      lds = (size_t)in_tile_h * in_tile_w * kCQ * sizeof(float4);
      if (lds <= 48 * 1024 || tile_h == 1) break;
      tile_h = balanced_tile((int)out_h, tile_h - 1);
    }
    const int tiles_h = ((int)out_h + tile_h - 1) / tile_h, tiles_w = ((int)out_w + tile_w - 1) / tile_w;
    if (lds <= 64 * 1024) {
      dim3 grid(tiles_h * tiles_w, (c4_total + kCQ - 1) / kCQ, (unsigned)batch);
      note_kernel("depthwise_3x3_halo<%d>", S);
      if (S == 1)
        TFHIP_LAUNCH((depthwise_3x3_halo<1><<<grid, 256, lds, stream()>>>(p, e, tile_h, tile_w, tiles_w, c4_total)));
      else
        TFHIP_LAUNCH((depthwise_3x3_halo<2><<<grid, 256, lds, stream()>>>(p, e, tile_h, tile_w, tiles_w, c4_total)));
      return kOk;
    }
  }
  long long blocks = (total + 255) / 256;
  const long long cap = (long long)num_cus() * 64;
  if (blocks > cap) blocks = cap;
  note_kernel("depthwise_generic");
  TFHIP_LAUNCH((depthwise_generic<<<(int)blocks, 256, 0, stream()>>>(p, e, total)));
  return kOk;
}
