// FusedDepthwiseConv2D, NHWC float32.
//
// Bandwidth-bound (about 2 flops per byte), so no matrix cores. Three kernels:
//  * depthwise_3x3_cols: 3x3, stride 1 or 2, channel multiplier 1 (every
//    MobileNet layer). Lanes lie along an output row in memory order, one float4
//    of one column each, and walk down a chunk of rows with the input rows in a
//    register ring; no LDS, no barriers.
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


// ---- shared by the 3x3 kernels ------------------------------------------------------
// All accesses are buffer loads / stores over the whole tensor with 32-bit byte offsets: padding
// taps and ragged edges use an offset outside the descriptor, which reads as zero and drops
// stores, so the row loops have no branches.
constexpr unsigned kDwNoOffset = 0xffffffffu;
// Results of at least this many bytes are stored non-temporally: an L2 holds 4 MB,
// so such a result cannot wait there for its reader (measured with operands from
// memory: 51 MB 21.3 -> 20.3 us, 12 MB at stride 2 13.7 -> 12.7 us; written through
// instead, 21.6 and 13.6 us).
constexpr long long kDwStreamBytes = 8LL << 20;
typedef unsigned int dw_uint4 __attribute__((ext_vector_type(4)));

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

// ---- 3x3, channel multiplier 1, dilation 1, stride S: one output column per lane ----
// The lanes of a launch lie along an output row in MEMORY order: lane f of a row chunk owns
// float4 f of the row ([column][channel quad], the NHWC order), so a wavefront's store covers
// one contiguous kilobyte and its three loads per input row (the columns left of, at and right
// of its own) cover contiguous kilobytes too, each element asked for by three lanes and served
// to two of them by the vector cache. A lane walks down `rows` output rows with the input rows
// in a register ring (the three a window needs plus S fetched ahead), so a row is fetched once
// per lane; with three float4 per input row a lane is light on registers, and a launch has
// thousands of wavefronts: the bytes in flight that a memory-bound kernel needs come from
// occupancy. Taps accumulate from zero by filter row, then column, one fused multiply-add each
// (the reference's order: DepthwiseConv2dNative.ts:62-95).
// Measured on [8,112,112,96] with operands from memory, against a kernel that gave a lane a strip of
// four columns (six loads per input row, 252 workgroups, one wavefront per SIMD): 20.3 -> 18.7 us at
// stride 1, 12.7 -> 11.6 at stride 2; a plain copy of the same bytes takes 16.1 us there. What is
// left is not latency (two to four rows fetched ahead change nothing), not the rows two chunks
// both read (chunks walking towards each other, so that those rows are read at the same time:
// no change) and not arithmetic (a third of the multiply-adds: no change): reads alone take
// 9.7 us (12.7 with the two neighbour loads), stores the rest, and the two do not overlap better
// than in the copy. Staging a workgroup's row segment through LDS, so that every element is fetched
// once instead of by three lanes, gave 18.1 us; non-temporal stores are the best of the six cache
// policies a store can carry (plain and write-through: +1 us).
constexpr int kColsThreads = 64;
struct DwColsArgs {
  int c4_total;        // channel quads per pixel
  int row_quads;       // out_w * c4_total: float4 per output row
  int blocks_per_row;  // workgroups along a row
  int chunks_h, rows;  // row chunks per image, output rows per chunk
  int xcd_run;         // > 0: workgroup ids are dealt to the XCDs in contiguous runs of this many
  unsigned x_bytes, y_bytes;
};

template <int S, bool GENERAL, bool STREAM>
__global__ __launch_bounds__(kColsThreads) void depthwise_3x3_cols(DwParams p, Epilogue e, DwColsArgs g) {
  constexpr int A = S;        // input rows in flight beyond the window in use: one output row ahead (two, three and
                              // four rows ahead measured the same: the launch is not short of loads in flight)
  constexpr int NB = 3 + A;   // ring of input rows
  // workgroup ids i, i + 8, ... share an XCD: each XCD takes a contiguous run, so that the columns
  // two neighbouring workgroups both read come from one L2
  const unsigned wg = g.xcd_run ? (blockIdx.x % 8) * (unsigned)g.xcd_run + blockIdx.x / 8 : blockIdx.x;
  const int bx = (int)(wg % (unsigned)g.blocks_per_row);
  const unsigned t = wg / (unsigned)g.blocks_per_row;
  const int chunk = (int)(t % (unsigned)g.chunks_h), n = (int)(t / (unsigned)g.chunks_h);
  const int f = bx * kColsThreads + (int)threadIdx.x;
  if (f >= g.row_quads) return;
  const int ow = f / g.c4_total, q = f - ow * g.c4_total;
  const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc((void *)p.x, 0, (int)g.x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc((void *)p.y, 0, (int)g.y_bytes, 0x00020000);
  const unsigned pix = (unsigned)g.c4_total * 16u;   // bytes per pixel
  const unsigned x_row = (unsigned)p.in_w * pix, y_row = (unsigned)p.out_w * pix;
  const unsigned x_img = (unsigned)n * (unsigned)p.in_h * x_row, y_img = (unsigned)n * (unsigned)p.out_h * y_row;
  const int oh0 = chunk * g.rows;
  const int rows = oh0 + g.rows <= p.out_h ? g.rows : p.out_h - oh0;
  const int rows_in = (rows - 1) * S + 3;
  const int ih0 = oh0 * S - p.pad_top;
  unsigned x_col[3];
#pragma unroll
  for (int wc = 0; wc < 3; ++wc) {
    const int iw = ow * S - p.pad_left + wc;
    x_col[wc] = (iw >= 0 && iw < p.in_w) ? (unsigned)iw * pix + (unsigned)q * 16u : kDwNoOffset;
  }
  const unsigned y_col = (unsigned)f * 16u;
  float4 ring[NB][3];
  auto fetch = [&](float4 (&row)[3], int i) __attribute__((always_inline)) {
    const int ih = ih0 + i;
    const bool row_ok = ih >= 0 && ih < p.in_h && i < rows_in;
    const unsigned row_off = x_img + (unsigned)ih * x_row;
#pragma unroll
    for (int wc = 0; wc < 3; ++wc) row[wc] = dw_load4(rx, (row_ok && x_col[wc] != kDwNoOffset) ? row_off + x_col[wc] : kDwNoOffset);
  };
  // the first window's rows, then this lane's filter taps and bias: one round trip for all of them
#pragma unroll
  for (int i = 0; i < 3 + A - S; ++i) fetch(ring[i], i);
  float4 w[9];
  const float4 *w4 = reinterpret_cast<const float4 *>(p.w) + q;
#pragma unroll
  for (int k = 0; k < 9; ++k) w[k] = w4[(long long)k * g.c4_total];
  float4 bias4 = make_float4(0.f, 0.f, 0.f, 0.f);
  const int c = q * 4;
  if (!GENERAL && e.bias) {
    const long long bs = e.bias_s[3];
    bias4 = make_float4(e.bias[(c + 0) * bs], e.bias[(c + 1) * bs], e.bias[(c + 2) * bs], e.bias[(c + 3) * bs]);
  }
  for (int o0 = 0; o0 < rows; o0 += NB) {
#pragma unroll
    for (int k = 0; k < NB; ++k) {
      const int o = o0 + k;
      if (o < rows) {
        // input row r of the chunk lives in ring[r % NB]; o0 is a multiple of NB
#pragma unroll
        for (int j = 0; j < S; ++j) fetch(ring[(S * k + 3 + A - S + j) % NB], S * o + 3 + A - S + j);
        float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int wr = 0; wr < 3; ++wr) {
#pragma unroll
          for (int wc = 0; wc < 3; ++wc) {
            const float4 xv = ring[(S * k + wr) % NB][wc];
            const float4 wv = w[wr * 3 + wc];
            a.x = fmaf(xv.x, wv.x, a.x);
            a.y = fmaf(xv.y, wv.y, a.y);
            a.z = fmaf(xv.z, wv.z, a.z);
            a.w = fmaf(xv.w, wv.w, a.w);
          }
        }
        const int oh = oh0 + o;
        dw_store4<STREAM>(ry, y_img + (unsigned)oh * y_row + y_col, dw_finish4<GENERAL>(e, a, bias4, c, n, oh, ow));
      }
    }
  }
}

int balanced_tile(int extent, int max_tile) {
  const int tiles = (extent + max_tile - 1) / max_tile;
  return (extent + tiles - 1) / tiles;
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
  TFHIP_CHECK_ARG(batch < lim && in_h < lim && in_w < lim && product_below(lim, {in_c, ch_mul}) && out_h < lim && out_w < lim,
                  "tfhip_fused_depthwise_conv2d: dimension exceeds 2^31-1");
  TFHIP_CHECK_ARG(pad_top >= 0 && pad_left >= 0, "tfhip_fused_depthwise_conv2d: negative padding");
  TFHIP_CHECK_ARG(product_below(kMaxElems, {batch, in_h, in_w, in_c}) && product_below(kMaxElems, {batch, out_h, out_w, in_c, ch_mul}) &&
                      product_below(lim, {f_h, f_w, in_c, ch_mul}),
                  "tfhip_fused_depthwise_conv2d: tensor exceeds the supported range");
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
    DwColsArgs g;
    g.c4_total = (int)(in_c / 4);
    g.row_quads = (int)out_w * g.c4_total;
    g.blocks_per_row = (g.row_quads + kColsThreads - 1) / kColsThreads;
    // Rows per chunk: a chunk of r output rows fetches (r - 1) S + 3 input rows, so longer chunks re-read
    // fewer rows, and shorter ones make more wavefronts. 14 rows (8 at stride 2) measured best on
    // [8,112,112,96] with operands from memory (stride 1: 18.7 us at 14 rows, 19.2 at 8, 20.5 at 4, 22.2 at 28;
    // stride 2: 11.6 at 8, 13.5 at 14); smaller launches take shorter chunks until there are two
    // wavefronts for every SIMD of the chip.
    int rows = S == 1 ? 14 : 8;
    if (tuning(kTuneDwRows) > 0) {
      rows = tuning(kTuneDwRows);
    } else {
      const long long want = 8LL * num_cus();
      while (rows > 1 && (long long)g.blocks_per_row * ((out_h + rows - 1) / rows) * batch < want) rows = (rows + 1) / 2;
    }
    rows = rows > out_h ? (int)out_h : rows;
    g.rows = balanced_tile((int)out_h, rows);
    g.chunks_h = ((int)out_h + g.rows - 1) / g.rows;
    g.x_bytes = (unsigned)(batch * in_h * in_w * in_c * 4);
    g.y_bytes = (unsigned)(total * 4);
    const long long wgs = (long long)g.blocks_per_row * g.chunks_h * batch;
    if (wgs <= 0x7fffffffLL) {
      g.xcd_run = wgs % 8 == 0 ? (int)(wgs / 8) : 0;
      const bool general = !(e.addressing == kChannel && activation <= TFHIP_RELU6);
      const bool streamed = !general && total * 4 >= kDwStreamBytes;
      note_kernel("depthwise_3x3_cols<%d, %s, %s>", S, general ? "true" : "false", streamed ? "true" : "false");
      const dim3 grid((unsigned)wgs), block(kColsThreads);
      if (S == 1 && streamed)
        TFHIP_LAUNCH((depthwise_3x3_cols<1, false, true><<<grid, block, 0, stream()>>>(p, e, g)));
      else if (S == 1 && !general)
        TFHIP_LAUNCH((depthwise_3x3_cols<1, false, false><<<grid, block, 0, stream()>>>(p, e, g)));
      else if (S == 1)
        TFHIP_LAUNCH((depthwise_3x3_cols<1, true, false><<<grid, block, 0, stream()>>>(p, e, g)));
      else if (streamed)
        TFHIP_LAUNCH((depthwise_3x3_cols<2, false, true><<<grid, block, 0, stream()>>>(p, e, g)));
      else if (!general)
        TFHIP_LAUNCH((depthwise_3x3_cols<2, false, false><<<grid, block, 0, stream()>>>(p, e, g)));
      else
        TFHIP_LAUNCH((depthwise_3x3_cols<2, true, false><<<grid, block, 0, stream()>>>(p, e, g)));
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
