// FusedConv2D entry point: implicit GEMM over the matrix cores.
//
//   rows of A  = output pixels (n, oh, ow), M = batch * out_h * out_w
//   columns    = filter taps x input channels, K = f_h * f_w * in_c
//   B          = the HWIO filter, already a row-major [K][out_c] matrix
//   C          = the NHWC output, a row-major [M][out_c] matrix
//
// A is gathered from the image inside the tile loader; nothing is unfolded in
// memory. A 1x1 filter with stride 1 and no padding is an ordinary GEMM on the
// image itself and takes the plain loaders.
#include "gemm_host.h"

using namespace tfhip;

namespace {

// Direct convolution for images with very few input channels (a network stem:
// 3 channels, K = 27). The implicit GEMM wastes most of a k tile on such a
// short contraction and gathers the image element by element; here one lane
// owns one output pixel and OC output channels in registers, the image values
// are fetched once per tap, and the filter values are the same for every lane,
// so they come through the scalar cache as instruction operands. Taps
// accumulate in the reference's order (filter row, column, input channel:
// tfjs-backend-cpu/src/kernels/Conv2D.ts:64-96), out-of-range taps are skipped
// like there. NHWC, per-channel bias and relu-family activations only; other
// forms take the implicit GEMM.
struct FewChannelsArgs {
  const float *x, *w, *bias;
  float *y;
  long long xs_n, xs_h, xs_w, bias_stride;
  int M, out_c, in_h, in_w, in_c, f_h, f_w, stride_h, stride_w, dil_h, dil_w, pad_top, pad_left, out_h, out_w;
  int activation;   // linear, relu or relu6
};

template <int OC>
__global__ __launch_bounds__(256) void conv_few_channels(FewChannelsArgs g) {
  const int m = blockIdx.x * 256 + threadIdx.x;
  if (m >= g.M) return;
  const int oc0 = blockIdx.y * OC;
  const int ow = m % g.out_w;
  const int t2 = m / g.out_w;
  const int oh = t2 % g.out_h, n = t2 / g.out_h;
  const float *__restrict__ x = g.x + (long long)n * g.xs_n;
  const float *__restrict__ w = g.w + oc0;
  float acc[OC], bias[OC];
#pragma unroll
  for (int o = 0; o < OC; ++o) acc[o] = bias[o] = 0.f;
  if (g.bias) {   // the same values in every lane; fetched ahead of the taps
#pragma unroll
    for (int o = 0; o < OC; ++o) bias[o] = g.bias[(long long)(oc0 + o) * g.bias_stride];
  }
  for (int r = 0; r < g.f_h; ++r) {
    const int ih = oh * g.stride_h - g.pad_top + r * g.dil_h;
    for (int s = 0; s < g.f_w; ++s) {
      const int iw = ow * g.stride_w - g.pad_left + s * g.dil_w;
      const bool inside = ih >= 0 && ih < g.in_h && iw >= 0 && iw < g.in_w;
      const float *xp = x + (inside ? (long long)ih * g.xs_h + (long long)iw * g.xs_w : 0);
      for (int c = 0; c < g.in_c; ++c) {
        const float xv = xp[c];
        const float *wk = w + (long long)((r * g.f_w + s) * g.in_c + c) * g.out_c;   // the same address in every lane
        if (inside) {
#pragma unroll
          for (int o = 0; o < OC; ++o) acc[o] = fmaf(xv, wk[o], acc[o]);
        }
      }
    }
  }
  float *y = g.y + (long long)m * g.out_c + oc0;
#pragma unroll
  for (int o = 0; o < OC; o += 4) {
    float q[4] = {acc[o], acc[o + 1], acc[o + 2], acc[o + 3]};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      q[k] += bias[o + k];
      if (g.activation != TFHIP_LINEAR) {
        q[k] = (q[k] > 0.f || q[k] != q[k]) ? q[k] : 0.f;   // Math.max(0, x): NaN stays, -0 becomes +0
        if (g.activation == TFHIP_RELU6 && q[k] > 6.f) q[k] = 6.f;
      }
    }
    store_result4(y + o, make_float4(q[0], q[1], q[2], q[3]));
  }
}

// What tap k = (r * f_w + s) * in_c + c of the filter reads, relative to the
// top-left element of a pixel's window; rows beyond K hold a row offset that no
// image has. Filled on the host so that the kernel does no divisions for it.
constexpr int kMaxTaps = 36;
struct TapTable {
  int dh[kMaxTaps], dw[kMaxTaps];
  unsigned off_bytes[kMaxTaps];
};

// The same convolution on the matrix cores, for filters of at most 4 * KSTEPS
// taps (K = f_h * f_w * in_c) and 16 * NB output channels per workgroup column.
// A wave computes 64 consecutive pixels x 16 NB channels per trip as 4 x NB
// blocks of v_mfma_f32_16x16x4_f32 over KSTEPS k steps:
//  * lane (r = lane % 16, kg = lane / 16) feeds tap k = 4 t + kg in k step t: of
//    the filter (weights of channel 16 j + r, fetched once per wave and kept in
//    registers) and of the image (pixel 16 i + r of the wave's 64: one gathered
//    element load per block and k step, all 4 * KSTEPS of them in flight at once;
//    buffer loads, so a tap outside the image or beyond K reads zero through an
//    offset that the descriptor does not cover);
//  * the operands go in swapped, so the lane ends up with channels 4 kg .. +3 of
//    pixel 16 i + r for each block: bias (the accumulators start from it),
//    activation and one 16-byte store per block.
template <int KSTEPS, int NB>
__global__ __launch_bounds__(256) void conv_few_taps(FewChannelsArgs g, TapTable taps, int chunks, unsigned x_bytes) {
  // blockDim.x is 256 or 64: four wavefronts or one, 64 consecutive pixels each
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, kg = lane >> 4;
  const int oc0 = blockIdx.y * (16 * NB);
  const int K = g.f_h * g.f_w * g.in_c;
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)g.x, 0, (int)x_bytes, 0x00020000);
  float wv[KSTEPS][NB];
  unsigned tap_off[KSTEPS];
  int tap_dh[KSTEPS], tap_dw[KSTEPS];
#pragma unroll
  for (int t = 0; t < KSTEPS; ++t) {
    const int k = 4 * t + kg;
    tap_dh[t] = taps.dh[k];
    tap_dw[t] = taps.dw[k];
    tap_off[t] = taps.off_bytes[k];
#pragma unroll
    for (int j = 0; j < NB; ++j) wv[t][j] = k < K ? g.w[(long long)k * g.out_c + oc0 + 16 * j + r] : 0.f;
  }
  float4_t bias4[NB];
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    bias4[j] = (float4_t){0.f, 0.f, 0.f, 0.f};
    if (g.bias) {
#pragma unroll
      for (int q = 0; q < 4; ++q) bias4[j][q] = g.bias[(long long)(oc0 + 16 * j + 4 * kg + q) * g.bias_stride];
    }
  }
  for (int chunk = blockIdx.x; chunk < chunks; chunk += gridDim.x) {
    const int m_wave = chunk * (int)blockDim.x + wave * 64;
    // pixel of block 0; the following blocks are 16 pixels further along the row
    int m = m_wave + r;
    int ow = m % g.out_w;
    int t2 = m / g.out_w;
    int oh = t2 % g.out_h, n = t2 / g.out_h;
    float av[4][KSTEPS];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool live = m < g.M;
      const int ih0 = oh * g.stride_h - g.pad_top, iw0 = ow * g.stride_w - g.pad_left;
      // byte offset of the window's top-left element; it may lie before the
      // image, the sum with an inside tap's offset is exact modulo 2^32
      const unsigned base = (unsigned)(((long long)n * g.xs_n + (long long)ih0 * g.xs_h + (long long)iw0 * g.xs_w) * 4);
#pragma unroll
      for (int t = 0; t < KSTEPS; ++t) {
        const bool inside = live && (unsigned)(ih0 + tap_dh[t]) < (unsigned)g.in_h &&
                            (unsigned)(iw0 + tap_dw[t]) < (unsigned)g.in_w;
        av[i][t] = __uint_as_float(
            __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)(inside ? base + tap_off[t] : 0xffffffffu), 0, 0));
      }
      m += 16;
      ow += 16;
      while (ow >= g.out_w) {
        ow -= g.out_w;
        if (++oh == g.out_h) {
          oh = 0;
          ++n;
        }
      }
    }
    float4_t acc[4][NB];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < NB; ++j) acc[i][j] = bias4[j];
#pragma unroll
    for (int t = 0; t < KSTEPS; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(wv[t][j], av[i][t], acc[i][j], 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int mi = m_wave + 16 * i + r;
      if (mi >= g.M) continue;
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        float q[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          q[k] = acc[i][j][k];
          if (g.activation != TFHIP_LINEAR) {
            q[k] = (q[k] > 0.f || q[k] != q[k]) ? q[k] : 0.f;   // Math.max(0, x): NaN stays, -0 becomes +0
            if (g.activation == TFHIP_RELU6 && q[k] > 6.f) q[k] = 6.f;
          }
        }
        *reinterpret_cast<float4 *>(g.y + (long long)mi * g.out_c + oc0 + 16 * j + 4 * kg) =
            make_float4(q[0], q[1], q[2], q[3]);
      }
    }
  }
}

void fill_few_channels_args(FewChannelsArgs &g, const GemmParams &p, int f_h) {
  const ConvGeom &c = p.conv;
  g.x = p.a; g.w = p.b; g.y = p.c;
  g.bias = p.epi.bias; g.bias_stride = p.epi.bias ? p.epi.bias_s[3] : 0;
  g.xs_n = c.xs_n; g.xs_h = c.xs_h; g.xs_w = c.xs_w;
  g.M = p.M; g.out_c = p.N; g.in_h = c.in_h; g.in_w = c.in_w; g.in_c = c.in_c; g.f_h = f_h; g.f_w = c.f_w;
  g.stride_h = c.stride_h; g.stride_w = c.stride_w; g.dil_h = c.dil_h; g.dil_w = c.dil_w;
  g.pad_top = c.pad_top; g.pad_left = c.pad_left; g.out_h = c.out_h; g.out_w = c.out_w;
  g.activation = p.epi.activation;
}

template <int KSTEPS, int NB>
int launch_few_taps(const GemmParams &p, int f_h) {
  FewChannelsArgs g;
  fill_few_channels_args(g, p, f_h);
  const ConvGeom &c = p.conv;
  TapTable taps;
  for (int k = 0; k < kMaxTaps; ++k) {
    const int tap = k / c.in_c, ch = k - tap * c.in_c;
    const int fr = tap / c.f_w, fs = tap - fr * c.f_w;
    taps.dh[k] = k < p.K ? fr * c.dil_h : (1 << 28);
    taps.dw[k] = fs * c.dil_w;
    taps.off_bytes[k] = (unsigned)(((long long)fr * c.dil_h * c.xs_h + (long long)fs * c.dil_w * c.xs_w + ch) * 4);
  }
  // 256 pixels (four wavefronts) per workgroup and trip, 64 when that would leave
  // compute units without a workgroup; every workgroup makes the same number of trips
  const int threads = (p.M + 255) / 256 * (p.N / (16 * NB)) >= num_cus() ? 256 : 64;
  const int chunks = (p.M + threads - 1) / threads;
  const int at_once = num_cus() * 8 * (256 / threads);
  const int trips = (chunks + at_once - 1) / at_once;
  dim3 grid((unsigned)((chunks + trips - 1) / trips), (unsigned)(p.N / (16 * NB)), 1);
  note_kernel("conv_few_taps<%d, %d>", KSTEPS, NB);
  TFHIP_LAUNCH((conv_few_taps<KSTEPS, NB><<<grid, threads, 0, stream()>>>(g, taps, chunks, p.a_bytes)));
  return kOk;
}

template <int NB>
int launch_few_taps_k(const GemmParams &p, int f_h) {
  if (p.K <= 12) return launch_few_taps<3, NB>(p, f_h);
  if (p.K <= 28) return launch_few_taps<7, NB>(p, f_h);
  return launch_few_taps<9, NB>(p, f_h);
}

template <int OC>
int launch_few_channels(const GemmParams &p, int f_h) {
  FewChannelsArgs g;
  fill_few_channels_args(g, p, f_h);
  dim3 grid((unsigned)((p.M + 255) / 256), (unsigned)(p.N / OC), 1);
  note_kernel("conv_few_channels<%d>", OC);
  TFHIP_LAUNCH((conv_few_channels<OC><<<grid, 256, 0, stream()>>>(g)));
  return kOk;
}

// The reference's own loop, one output element per lane: taps outside the image are SKIPPED, not
// read as zero (tfjs-backend-cpu/src/kernels/Conv2D.ts:72-84). For a finite filter the two are the
// same number; a filter that holds Inf or NaN gives NaN at every border output when a zero is
// multiplied by it, and leaves those outputs alone in the reference. The MFMA kernels cannot skip
// a tap per output pixel, so a padded convolution whose filter is not finite runs here: any layout,
// stride, dilation, epilogue and residual, sums in the reference's order (filter row, filter
// column, input channel) with one float32 rounding per multiply-add.
struct SkipTapsArgs {
  const float *x, *w;
  float *y;
  int in_h, in_w, in_c, f_h, f_w, out_c;
  int stride_h, stride_w, dil_h, dil_w, pad_top, pad_left, out_h, out_w;
  long long xs_n, xs_h, xs_w, xs_c;
};

__global__ __launch_bounds__(256) void conv_skip_taps(SkipTapsArgs g, Epilogue e, long long total) {
  const long long stride = (long long)gridDim.x * 256;
  for (long long idx = (long long)blockIdx.x * 256 + threadIdx.x; idx < total; idx += stride) {
    const int oc = (int)(idx % g.out_c);
    long long t = idx / g.out_c;
    const int ow = (int)(t % g.out_w);
    t /= g.out_w;
    const int oh = (int)(t % g.out_h);
    const long long n = t / g.out_h;
    float acc = 0.f;
    for (int r = 0; r < g.f_h; ++r) {
      const int ih = oh * g.stride_h - g.pad_top + r * g.dil_h;
      if (ih < 0 || ih >= g.in_h) continue;
      for (int c = 0; c < g.f_w; ++c) {
        const int iw = ow * g.stride_w - g.pad_left + c * g.dil_w;
        if (iw < 0 || iw >= g.in_w) continue;
        const float *xp = g.x + n * g.xs_n + ih * g.xs_h + iw * g.xs_w;
        const float *wp = g.w + ((long long)(r * g.f_w + c) * g.in_c) * g.out_c + oc;
        for (int d = 0; d < g.in_c; ++d) acc = fmaf(xp[d * g.xs_c], wp[(long long)d * g.out_c], acc);
      }
    }
    float v = finish(e, acc, 0, n * g.out_h * g.out_w + (long long)oh * g.out_w + ow, oc, n, oh, ow);
    const long long at = n * e.y_s[0] + oh * e.y_s[1] + ow * e.y_s[2] + oc * e.y_s[3];
    if (e.residual) v = v + e.residual[at];
    g.y[at] = v;
  }
}

int launch_skip_taps(const GemmParams &p, int f_h, long long batch) {
  SkipTapsArgs g;
  const ConvGeom &c = p.conv;
  g.x = p.a; g.w = p.b; g.y = p.c;
  g.in_h = c.in_h; g.in_w = c.in_w; g.in_c = c.in_c; g.f_h = f_h; g.f_w = c.f_w; g.out_c = p.N;
  g.stride_h = c.stride_h; g.stride_w = c.stride_w; g.dil_h = c.dil_h; g.dil_w = c.dil_w;
  g.pad_top = c.pad_top; g.pad_left = c.pad_left; g.out_h = c.out_h; g.out_w = c.out_w;
  g.xs_n = c.xs_n; g.xs_h = c.xs_h; g.xs_w = c.xs_w; g.xs_c = c.xs_c;
  const long long total = (long long)p.M * p.N;
  long long blocks = (total + 255) / 256;
  const long long cap = (long long)num_cus() * 32;
  note_kernel("conv_skip_taps");
  TFHIP_LAUNCH((conv_skip_taps<<<dim3((unsigned)(blocks < cap ? blocks : cap)), dim3(256), 0, stream()>>>(g, p.epi, total)));
  return kOk;
}

// y += residual for the kernels whose tail does not take a residual itself.
__global__ __launch_bounds__(256) void add_residual(float *__restrict__ y, const float *__restrict__ residual,
                                                    long long total) {
  const long long stride = (long long)gridDim.x * 256;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) y[i] = y[i] + residual[i];
}

int launch_add_residual(float *y, const float *residual, long long total) {
  long long blocks = (total + 255) / 256;
  const long long cap = (long long)num_cus() * 16;
  TFHIP_LAUNCH((add_residual<<<dim3((unsigned)(blocks < cap ? blocks : cap)), dim3(256), 0, stream()>>>(y, residual,
                                                                                                     total)));
  return kOk;
}

int fused_conv2d(const float *x, const float *filter, float *y, int64_t batch, int64_t in_h,
                 int64_t in_w, int64_t in_c, int64_t f_h, int64_t f_w, int64_t out_c,
                 int64_t stride_h, int64_t stride_w, int64_t dilation_h, int64_t dilation_w,
                 int64_t pad_top, int64_t pad_left, int64_t out_h, int64_t out_w, int nchw,
                 const float *bias, const int64_t bias_strides[4], int activation,
                 const float *prelu_weights, const int64_t prelu_strides[4],
                 double leakyrelu_alpha, const float *residual) {
  TFHIP_REQUIRE_INIT();
  TFHIP_CHECK_ARG(batch >= 0 && in_h > 0 && in_w > 0 && in_c > 0 && f_h > 0 && f_w > 0 && out_c > 0 &&
                      stride_h > 0 && stride_w > 0 && dilation_h > 0 && dilation_w > 0 && out_h >= 0 && out_w >= 0,
                  "tfhip_fused_conv2d: non-positive dimension");
  TFHIP_CHECK_ARG(pad_top >= 0 && pad_left >= 0, "tfhip_fused_conv2d: negative padding");
  const int64_t lim = 0x7fffffff;
  TFHIP_CHECK_ARG(product_below(lim, {batch, out_h, out_w}) && product_below(lim, {f_h, f_w, in_c}) && out_c < lim &&
                      in_h < lim && in_w < lim && product_below(lim << 8, {batch, in_h, in_w, in_c}),
                  "tfhip_fused_conv2d: dimension exceeds the supported range");
  const int64_t M = batch * out_h * out_w, K = f_h * f_w * in_c;
  TFHIP_CHECK_ARG(batch * in_h * in_w * in_c * 4 <= 0xfffffffeLL,
                  "tfhip_fused_conv2d: an input above 4 GiB is not supported");
  if (M == 0) return kOk;
  TFHIP_CHECK_RANGE(x, batch * in_h * in_w * in_c, 4, "x");
  TFHIP_CHECK_RANGE(filter, K * out_c, 4, "filter");
  TFHIP_CHECK_OUTPUT(y, M * out_c, 4, "y");
  if (residual) TFHIP_CHECK_RANGE(residual, M * out_c, 4, "residual");

  GemmParams p = {};
  p.a = x; p.b = filter; p.c = y;
  p.M = (int)M; p.N = (int)out_c; p.K = (int)K;
  p.batch = p.batch_a = p.batch_b = 1;
  p.b_sx = 1; p.b_sk = out_c;
  p.ldc = out_c;
  ConvGeom &g = p.conv;
  g.in_h = (int)in_h; g.in_w = (int)in_w; g.in_c = (int)in_c; g.f_w = (int)f_w;
  g.stride_h = (int)stride_h; g.stride_w = (int)stride_w; g.dil_h = (int)dilation_h; g.dil_w = (int)dilation_w;
  g.pad_top = (int)pad_top; g.pad_left = (int)pad_left; g.out_h = (int)out_h; g.out_w = (int)out_w;
  if (nchw) {
    g.xs_n = in_c * in_h * in_w; g.xs_c = in_h * in_w; g.xs_h = in_w; g.xs_w = 1;
  } else {
    g.xs_n = in_h * in_w * in_c; g.xs_h = in_w * in_c; g.xs_w = in_c; g.xs_c = 1;
  }
  const int64_t dims[4] = {batch, out_h, out_w, out_c};
  int rc = fill_epilogue(p.epi, "tfhip_fused_conv2d", dims, 4, bias, bias_strides, activation, prelu_weights,
                         prelu_strides, leakyrelu_alpha, kConv);
  if (rc) return rc;
  p.epi.residual = residual;   // every GEMM-shaped path below adds it in its tail
  p.epi.out_h = (int)out_h;
  p.epi.out_w = (int)out_w;
  if (nchw) {
    // bias / prelu of a channel-only shape still index by column; only the
    // output needs the (n, oh, ow, c) split to be written channels-first
    if (p.epi.addressing == kChannel) {
      p.epi.bias_s[0] = p.epi.bias_s[1] = p.epi.bias_s[2] = 0;
      p.epi.prelu_s[0] = p.epi.prelu_s[1] = p.epi.prelu_s[2] = 0;
      p.epi.addressing = kConv;
    }
    p.epi.y_s[0] = out_c * out_h * out_w; p.epi.y_s[1] = out_w; p.epi.y_s[2] = 1; p.epi.y_s[3] = out_h * out_w;
  } else {
    p.epi.y_s[0] = out_h * out_w * out_c; p.epi.y_s[1] = out_w * out_c; p.epi.y_s[2] = out_c; p.epi.y_s[3] = 1;
  }

  const int64_t kMaxBufferBytes = 0xfffffffeLL;   // one buffer descriptor addresses at most this much
  const int64_t x_bytes = batch * in_h * in_w * in_c * 4, w_bytes = K * out_c * 4;
  p.a_bytes = (unsigned)(x_bytes <= kMaxBufferBytes ? x_bytes : 0);
  p.b_bytes = (unsigned)(w_bytes <= kMaxBufferBytes ? w_bytes : 0);
  p.c_bytes = (unsigned)(M * out_c * 4 <= kMaxBufferBytes ? M * out_c * 4 : 0);
  p.vec_store = !nchw && out_c % 4 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0;
  const bool x16 = reinterpret_cast<uintptr_t>(x) % 16 == 0 && p.a_bytes != 0,
             w16 = reinterpret_cast<uintptr_t>(filter) % 16 == 0 && p.b_bytes != 0;
  const bool vec = !nchw && x16 && w16 && in_c % 4 == 0 && out_c % 4 == 0;
  // A window can reach outside the image: the reference skips such taps, the kernels below read
  // zeros for them, which differs only under a filter value that is not finite.
  const bool taps_can_miss = pad_top > 0 || pad_left > 0 ||
                             (out_h - 1) * stride_h - pad_top + (f_h - 1) * dilation_h >= in_h ||
                             (out_w - 1) * stride_w - pad_left + (f_w - 1) * dilation_w >= in_w;
  if (taps_can_miss) {
    bool nonfinite = false;
    if ((rc = scan_filter(filter, K * out_c, "tfhip_fused_conv2d", &nonfinite)) != kOk) return rc;
    if (nonfinite) return launch_skip_taps(p, (int)f_h, batch);
  }
  const bool pointwise = !nchw && f_h == 1 && f_w == 1 && stride_h == 1 && stride_w == 1 && pad_top == 0 &&
                         pad_left == 0 && out_h == in_h && out_w == in_w;
  if (pointwise) {
    p.a_sx = in_c; p.a_sk = 1;
    return launch_plain_gemm(p, false, false, vec);
  }
  if (!nchw && in_c <= 4 && out_c % 8 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0 &&
      p.epi.channel_operands && activation <= TFHIP_RELU6) {
    const bool few_taps = K <= kMaxTaps && M < lim - 256 && p.a_bytes != 0;
    // 32 channels per wavefront when there are pixels enough to fill the chip that
    // way, else 16 (twice the wavefronts)
    if (few_taps && out_c % 32 == 0 && M >= 64LL * 4 * num_cus()) rc = launch_few_taps_k<2>(p, (int)f_h);
    else if (few_taps && out_c % 16 == 0) rc = launch_few_taps_k<1>(p, (int)f_h);
    else if (out_c % 32 == 0) rc = launch_few_channels<32>(p, (int)f_h);
    else if (out_c % 16 == 0) rc = launch_few_channels<16>(p, (int)f_h);
    else rc = launch_few_channels<8>(p, (int)f_h);
    // these direct kernels have no residual operand: a second pass over y adds it
    if (rc == kOk && residual) rc = launch_add_residual(y, residual, M * out_c);
    return rc;
  }
  if (vec) {
    const int shape = choose_tile_shape(M, out_c, K, 1, num_cus());
    return launch_gemm_shape<kLoadIm2colVec, kLoadXVec>(shape, p);
  }
  if (out_c <= 32) return launch_gemm<256, 32, 16, 4, 1, kLoadIm2colScalar, kLoadScalar>(p);
  return launch_gemm<64, 64, 16, 2, 2, kLoadIm2colScalar, kLoadScalar>(p);
}

}  // namespace

extern "C" int tfhip_fused_conv2d(const float *x, const float *filter, float *y, int64_t batch, int64_t in_h,
                                  int64_t in_w, int64_t in_c, int64_t f_h, int64_t f_w, int64_t out_c,
                                  int64_t stride_h, int64_t stride_w, int64_t dilation_h, int64_t dilation_w,
                                  int64_t pad_top, int64_t pad_left, int64_t out_h, int64_t out_w, int nchw,
                                  const float *bias, const int64_t bias_strides[4], int activation,
                                  const float *prelu_weights, const int64_t prelu_strides[4],
                                  double leakyrelu_alpha) {
  return fused_conv2d(x, filter, y, batch, in_h, in_w, in_c, f_h, f_w, out_c, stride_h, stride_w, dilation_h,
                      dilation_w, pad_top, pad_left, out_h, out_w, nchw, bias, bias_strides, activation,
                      prelu_weights, prelu_strides, leakyrelu_alpha, nullptr);
}

extern "C" int tfhip_fused_conv2d_add(const float *x, const float *filter, float *y, int64_t batch, int64_t in_h,
                                      int64_t in_w, int64_t in_c, int64_t f_h, int64_t f_w, int64_t out_c,
                                      int64_t stride_h, int64_t stride_w, int64_t dilation_h, int64_t dilation_w,
                                      int64_t pad_top, int64_t pad_left, int64_t out_h, int64_t out_w, int nchw,
                                      const float *bias, const int64_t bias_strides[4], int activation,
                                      const float *prelu_weights, const int64_t prelu_strides[4],
                                      double leakyrelu_alpha, const float *residual) {
  TFHIP_CHECK_ARG(residual != nullptr, "tfhip_fused_conv2d_add: residual is NULL");
  TFHIP_CHECK_ARG(residual != y, "tfhip_fused_conv2d_add: residual and y are the same buffer");
  return fused_conv2d(x, filter, y, batch, in_h, in_w, in_c, f_h, f_w, out_c, stride_h, stride_w, dilation_h,
                      dilation_w, pad_top, pad_left, out_h, out_w, nchw, bias, bias_strides, activation,
                      prelu_weights, prelu_strides, leakyrelu_alpha, residual);
}
