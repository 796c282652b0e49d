// FusedDepthwiseConv2D, NHWC float32.
//
// Bandwidth-bound (about 2 flops per byte), so no matrix cores: the 3x3 kernel
// stages an input halo tile of 32 channels in LDS once per workgroup, so each
// input element is fetched from memory once per tile instead of up to nine
// times, and every global access is a float4 over the contiguous channel axis.
// Each output accumulates its taps in the reference's own order (filter row,
// then filter column: tfjs-backend-cpu/src/kernels/DepthwiseConv2dNative.ts:62-95)
// with one fused multiply-add per tap, which is the reference's
// "fround(y + x*w)" per tap up to double rounding.
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
    y4[(((long long)n * p.out_h + oh) * p.out_w + ow) * c4_total + cq0 + c4] = o;
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
  TFHIP_CHECK_ARG(batch < lim && in_h < lim && in_w < lim && in_c * ch_mul < lim && out_h < lim && out_w < lim,
                  "tfhip_fused_depthwise_conv2d: dimension exceeds 2^31-1");
  TFHIP_CHECK_ARG(pad_top >= 0 && pad_left >= 0, "tfhip_fused_depthwise_conv2d: negative padding");
  const int64_t out_c = in_c * ch_mul;
  const int64_t total = batch * out_h * out_w * out_c;
  if (total == 0) return kOk;
  TFHIP_CHECK_RANGE(x, batch * in_h * in_w * in_c, 4, "x");
  TFHIP_CHECK_RANGE(filter, f_h * f_w * in_c * ch_mul, 4, "filter");
  TFHIP_CHECK_RANGE(y, total, 4, "y");
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
  const bool fast = f_h == 3 && f_w == 3 && ch_mul == 1 && dilation_h == 1 && dilation_w == 1 &&
                    stride_h == stride_w && (stride_h == 1 || stride_h == 2) && in_c % 4 == 0 && aligned16 &&
                    batch <= 65535;
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
