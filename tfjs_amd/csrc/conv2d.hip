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

extern "C" int tfhip_fused_conv2d(const float *x, const float *filter, float *y, int64_t batch, int64_t in_h,
                                  int64_t in_w, int64_t in_c, int64_t f_h, int64_t f_w, int64_t out_c,
                                  int64_t stride_h, int64_t stride_w, int64_t dilation_h, int64_t dilation_w,
                                  int64_t pad_top, int64_t pad_left, int64_t out_h, int64_t out_w, int nchw,
                                  const float *bias, const int64_t bias_strides[4], int activation,
                                  const float *prelu_weights, const int64_t prelu_strides[4],
                                  double leakyrelu_alpha) {
  TFHIP_REQUIRE_INIT();
  TFHIP_CHECK_ARG(batch >= 0 && in_h > 0 && in_w > 0 && in_c > 0 && f_h > 0 && f_w > 0 && out_c > 0 &&
                      stride_h > 0 && stride_w > 0 && dilation_h > 0 && dilation_w > 0 && out_h >= 0 && out_w >= 0,
                  "tfhip_fused_conv2d: non-positive dimension");
  TFHIP_CHECK_ARG(pad_top >= 0 && pad_left >= 0, "tfhip_fused_conv2d: negative padding");
  const int64_t lim = 0x7fffffff;
  const int64_t M = batch * out_h * out_w, K = f_h * f_w * in_c;
  TFHIP_CHECK_ARG(M < lim && K < lim && out_c < lim && in_h < lim && in_w < lim && batch * in_h * in_w * in_c < (lim << 8),
                  "tfhip_fused_conv2d: dimension exceeds the supported range");
  TFHIP_CHECK_ARG(batch * in_h * in_w * in_c * 4 <= 0xfffffffeLL,
                  "tfhip_fused_conv2d: an input above 4 GiB is not supported");
  if (M == 0) return kOk;
  TFHIP_CHECK_RANGE(x, batch * in_h * in_w * in_c, 4, "x");
  TFHIP_CHECK_RANGE(filter, K * out_c, 4, "filter");
  TFHIP_CHECK_RANGE(y, M * out_c, 4, "y");

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
  p.vec_store = !nchw && out_c % 4 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0;
  const bool x16 = reinterpret_cast<uintptr_t>(x) % 16 == 0 && p.a_bytes != 0,
             w16 = reinterpret_cast<uintptr_t>(filter) % 16 == 0 && p.b_bytes != 0;
  const bool vec = !nchw && x16 && w16 && in_c % 4 == 0 && out_c % 4 == 0;
  const bool pointwise = !nchw && f_h == 1 && f_w == 1 && stride_h == 1 && stride_w == 1 && pad_top == 0 &&
                         pad_left == 0 && out_h == in_h && out_w == in_w;
  if (pointwise) {
    p.a_sx = in_c; p.a_sk = 1;
    return launch_plain_gemm(p, false, false, vec);
  }
  if (vec) {
    const int shape = choose_tile_shape(M, out_c, K, 1, num_cus());
    return launch_gemm_shape<kLoadIm2colVec, kLoadXVec>(shape, p);
  }
  if (out_c <= 32) return launch_gemm<256, 32, 16, 4, 1, kLoadIm2colScalar, kLoadScalar>(p);
  return launch_gemm<64, 64, 16, 2, 2, kLoadIm2colScalar, kLoadScalar>(p);
}
