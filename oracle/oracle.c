/*
 * CPU oracle: a plain-C restatement of the tfjs-backend-cpu kernels and of the
 * tfjs-core weight decoder that the HIP backend must agree with.
 *
 * THIS FILE IS TEST INFRASTRUCTURE. It is the checker the parity tests, the
 * smoke test and the benchmark's cpu_baseline leg compare against; nothing in
 * the product path may call it.
 *
 * Arithmetic model (what JavaScript does in the reference): every typed-array
 * element is an IEEE binary32, every expression between two typed-array stores
 * is evaluated in IEEE binary64, and a store rounds to nearest-even binary32.
 * Here that is `float` storage and `double` expressions, compiled with
 * -ffp-contract=off so no multiply-add is fused.
 *
 * Loops that are independent per output element are parallelised with OpenMP;
 * each output element is still produced by one thread in the reference's own
 * order, so results do not depend on the thread count.
 *
 * All file:line citations are relative to the tensorflow/tfjs source tree.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_MAX_RANK 8

/* Activation numbering: tfjs-backend-wasm/src/cc/backend.h:32-40. */
enum {
  ORC_LINEAR = 0,
  ORC_RELU = 1,
  ORC_RELU6 = 2,
  ORC_PRELU = 3,
  ORC_LEAKYRELU = 4,
  ORC_SIGMOID = 5,
  ORC_ELU = 6
};

static int64_t size_from_shape(const int64_t *shape, int rank) {
  int64_t n = 1;
  for (int i = 0; i < rank; ++i) n *= shape[i];
  return n;
}

/* util.computeStrides (tfjs-core/src/util_base.ts:565-579): rank-1 entries. */
static void compute_strides(const int64_t *shape, int rank, int64_t *strides) {
  if (rank < 2) return;
  strides[rank - 2] = shape[rank - 1];
  for (int i = rank - 3; i >= 0; --i) strides[i] = strides[i + 1] * shape[i + 1];
}

/* ------------------------------------------------------------------ */
/* BatchMatMul: tfjs-backend-cpu/src/kernels/BatchMatMul.ts:25-133.    */
/* a is [bA, M, K] (or [bA, K, M] when transA), b is [bB, K, N] (or    */
/* [bB, N, K] when transB); out is [max(bA,bB), M, N]. Blocked by 48   */
/* (backend_cpu.ts:38); `sum` is a double over one k-block and is      */
/* added into the float32 result once per k-block (:108-119).          */
/* ------------------------------------------------------------------ */
void orc_batch_matmul(const float *a, const float *b, float *out, int64_t bA,
                      int64_t bB, int64_t M, int64_t N, int64_t K, int transA,
                      int transB) {
  const int64_t blockSize = 48;
  const int64_t batchDim = bA > bB ? bA : bB;
  /* strides of the rank-3 views (:82-87) */
  const int64_t aS0 = M * K, aS1 = transA ? M : K;
  const int64_t bS0 = K * N, bS1 = transB ? K : N;
  const int64_t aBatch = aS0, aOuterStep = transA ? 1 : aS1,
                aInnerStep = transA ? aS1 : 1;
  const int64_t bInnerStep = transB ? 1 : bS1, bOuterStep = transB ? bS1 : 1,
                bBatch = bS0;
  const int64_t size = M * N;
  memset(out, 0, sizeof(float) * (size_t)(batchDim * size));
  const int64_t iBlocks = (M + blockSize - 1) / blockSize;
#pragma omp parallel for collapse(2) schedule(dynamic)
  for (int64_t bi = 0; bi < batchDim; bi++) {
    for (int64_t ib = 0; ib < iBlocks; ib++) {
      const int64_t batchIndexA = bi % bA;
      const int64_t batchIndexB = bi % bB;
      const int64_t i0 = ib * blockSize;
      const int64_t iBlock = i0 + blockSize < M ? i0 + blockSize : M;
      for (int64_t j0 = 0; j0 < N; j0 += blockSize) {
        const int64_t jBlock = j0 + blockSize < N ? j0 + blockSize : N;
        for (int64_t k0 = 0; k0 < K; k0 += blockSize) {
          const int64_t kBlock = k0 + blockSize < K ? k0 + blockSize : K;
          for (int64_t i = i0; i < iBlock; i++) {
            for (int64_t j = j0; j < jBlock; j++) {
              double sum = 0.0;
              for (int64_t k = k0; k < kBlock; k++) {
                const double aVal =
                    a[batchIndexA * aBatch + i * aOuterStep + k * aInnerStep];
                const double bVal =
                    b[k * bInnerStep + j * bOuterStep + batchIndexB * bBatch];
                sum += aVal * bVal;
              }
              float *r = &out[bi * size + (i * N + j)];
              *r = (float)((double)*r + sum);
            }
          }
        }
      }
    }
  }
}

/* ------------------------------------------------------------------ */
/* Broadcasting binary template:                                       */
/* tfjs-backend-cpu/src/utils/binary_impl.ts:25-68, with               */
/* assertAndGetBroadcastShape / getBroadcastDims from                  */
/* tfjs-core/src/ops/broadcast_util.ts:27-41,63-90.                    */
/* op: 0 = add (kernels/Add.ts:23-24), 1 = prelu (kernels/Prelu.ts:24-25) */
/* Returns the output rank (shape in outShape) or -1 if the shapes do  */
/* not broadcast.                                                      */
/* ------------------------------------------------------------------ */
static int broadcast_shape(const int64_t *sa, int ra, const int64_t *sb, int rb,
                           int64_t *out) {
  const int l = ra > rb ? ra : rb;
  for (int i = 0; i < l; i++) {
    int64_t a = (ra - i - 1 >= 0) ? sa[ra - i - 1] : 1;
    int64_t b = (rb - i - 1 >= 0) ? sb[rb - i - 1] : 1;
    if (a == 1) {
      out[l - i - 1] = b;
    } else if (b == 1) {
      out[l - i - 1] = a;
    } else if (a != b) {
      return -1;
    } else {
      out[l - i - 1] = a;
    }
  }
  return l;
}

static int broadcast_dims(const int64_t *in, int inRank, const int64_t *out,
                          int outRank, int *dims) {
  /* dims[d] = 1 when dimension d of `in` is stretched 1 -> n */
  int count = 0;
  for (int d = 0; d < inRank; d++) dims[d] = 0;
  for (int i = 0; i < inRank; i++) {
    const int dim = inRank - 1 - i;
    const int64_t a = in[dim] ? in[dim] : 1;
    const int64_t o = out[outRank - 1 - i];
    const int64_t b = o ? o : 1;
    if (b > 1 && a == 1) {
      dims[dim] = 1;
      count++;
    }
  }
  return count;
}

static inline float binary_apply(int op, float x, float y) {
  if (op == 0) return (float)((double)x + (double)y);
  /* Sub.ts: (a, b) => a - b; Multiply.ts: (a, b) => a * b */
  if (op == 2) return (float)((double)x - (double)y);
  if (op == 3) return (float)((double)x * (double)y);
  /* prelu: xValue < 0 ? aValue * xValue : xValue */
  return x < 0 ? (float)((double)y * (double)x) : x;
}

int orc_binary_broadcast(int op, const float *aVals, const int64_t *aShape,
                         int aRank, const float *bVals, const int64_t *bShape,
                         int bRank, float *result, int64_t *outShape) {
  int64_t newShape[ORC_MAX_RANK];
  const int rank = broadcast_shape(aShape, aRank, bShape, bRank, newShape);
  if (rank < 0) return -1;
  for (int i = 0; i < rank; i++) outShape[i] = newShape[i];
  const int64_t resultSize = size_from_shape(newShape, rank);
  const int64_t aLen = size_from_shape(aShape, aRank);
  const int64_t bLen = size_from_shape(bShape, bRank);
  int64_t resultStrides[ORC_MAX_RANK], aStrides[ORC_MAX_RANK],
      bStrides[ORC_MAX_RANK];
  compute_strides(newShape, rank, resultStrides);
  compute_strides(aShape, aRank, aStrides);
  compute_strides(bShape, bRank, bStrides);
  int aB[ORC_MAX_RANK], bB[ORC_MAX_RANK];
  const int na = broadcast_dims(aShape, aRank, newShape, rank, aB);
  const int nb = broadcast_dims(bShape, bRank, newShape, rank, bB);
  if (na + nb == 0) {
    /* :46-50, wrap-around indexing */
#pragma omp parallel for
    for (int64_t i = 0; i < resultSize; ++i) {
      result[i] = binary_apply(op, aVals[i % aLen], bVals[i % bLen]);
    }
  } else {
#pragma omp parallel for
    for (int64_t i = 0; i < resultSize; ++i) {
      int64_t loc[ORC_MAX_RANK];
      int64_t index = i;
      for (int d = 0; d < rank - 1; ++d) {
        loc[d] = index / resultStrides[d];
        index -= loc[d] * resultStrides[d];
      }
      if (rank > 0) loc[rank - 1] = index;
      int64_t aIndex = 0, bIndex = 0;
      for (int d = 0; d < aRank; ++d) {
        const int64_t l = aB[d] ? 0 : loc[rank - aRank + d];
        aIndex += (d == aRank - 1) ? l : l * aStrides[d];
      }
      for (int d = 0; d < bRank; ++d) {
        const int64_t l = bB[d] ? 0 : loc[rank - bRank + d];
        bIndex += (d == bRank - 1) ? l : l * bStrides[d];
      }
      result[i] = binary_apply(op, aVals[aIndex], bVals[bIndex]);
    }
  }
  return rank;
}

/* ------------------------------------------------------------------ */
/* Unary activations: tfjs-backend-cpu/src/kernels/Relu.ts:22,         */
/* Relu6.ts:22-23, Elu.ts:22-23, Sigmoid.ts:25-26, LeakyRelu.ts:38-40. */
/* Math.max / Math.min propagate NaN and return +0 for max(0, -0).     */
/* ------------------------------------------------------------------ */
static inline double js_max0(double x) {
  if (x != x) return x;
  return x > 0 ? x : 0.0;
}

void orc_unary_activation(int act, const float *x, float *y, int64_t n,
                          double leakyAlpha) {
#pragma omp parallel for
  for (int64_t i = 0; i < n; ++i) {
    const double xi = x[i];
    double r;
    switch (act) {
      case ORC_RELU:
        r = js_max0(xi);
        break;
      case ORC_RELU6: {
        const double m = js_max0(xi);
        r = (m != m) ? m : (m < 6 ? m : 6.0);
        break;
      }
      case ORC_ELU:
        r = xi >= 0 ? xi : (exp(xi) - 1);
        break;
      case ORC_SIGMOID:
        r = 1 / (1 + exp(-xi));
        break;
      case ORC_LEAKYRELU:
        r = xi < 0 ? leakyAlpha * xi : xi;
        break;
      default:
        r = xi;
    }
    y[i] = (float)r;
  }
}

/* applyActivation: tfjs-backend-cpu/src/utils/fused_utils.ts:29-49. In place
 * on `x` of shape xShape; prelu weights broadcast as a tensor. */
static int apply_activation(int act, float *x, const int64_t *xShape, int xRank,
                            const float *prelu, const int64_t *preluShape,
                            int preluRank, double leakyAlpha) {
  const int64_t n = size_from_shape(xShape, xRank);
  if (act == ORC_LINEAR) return 0;
  if (act == ORC_PRELU) {
    int64_t outShape[ORC_MAX_RANK];
    float *tmp = (float *)malloc(sizeof(float) * (size_t)(n ? n : 1));
    const int r = orc_binary_broadcast(1, x, xShape, xRank, prelu, preluShape,
                                       preluRank, tmp, outShape);
    if (r < 0 || size_from_shape(outShape, r) != n) {
      free(tmp);
      return -1;
    }
    memcpy(x, tmp, sizeof(float) * (size_t)n);
    free(tmp);
    return 0;
  }
  orc_unary_activation(act, x, x, n, leakyAlpha);
  return 0;
}

static int add_bias(float *x, const int64_t *xShape, int xRank,
                    const float *bias, const int64_t *biasShape, int biasRank) {
  const int64_t n = size_from_shape(xShape, xRank);
  int64_t outShape[ORC_MAX_RANK];
  float *tmp = (float *)malloc(sizeof(float) * (size_t)(n ? n : 1));
  const int r = orc_binary_broadcast(0, x, xShape, xRank, bias, biasShape,
                                     biasRank, tmp, outShape);
  if (r < 0 || size_from_shape(outShape, r) != n) {
    free(tmp);
    return -1;
  }
  memcpy(x, tmp, sizeof(float) * (size_t)n);
  free(tmp);
  return 0;
}

/* ------------------------------------------------------------------ */
/* _FusedMatMul: tfjs-backend-cpu/src/kernels/_FusedMatMul.ts:26-62.   */
/* out viewed as [batch, M, N]; bias / prelu are tensors with their    */
/* own shapes, broadcast against that view (null pointer = absent).    */
/* ------------------------------------------------------------------ */
int orc_fused_matmul(const float *a, const float *b, float *out, int64_t bA,
                     int64_t bB, int64_t M, int64_t N, int64_t K, int transA,
                     int transB, const float *bias, const int64_t *biasShape,
                     int biasRank, int act, const float *prelu,
                     const int64_t *preluShape, int preluRank,
                     double leakyAlpha) {
  orc_batch_matmul(a, b, out, bA, bB, M, N, K, transA, transB);
  const int64_t shape[3] = {bA > bB ? bA : bB, M, N};
  if (bias && add_bias(out, shape, 3, bias, biasShape, biasRank)) return -1;
  return apply_activation(act, out, shape, 3, prelu, preluShape, preluRank,
                          leakyAlpha);
}

/* ------------------------------------------------------------------ */
/* computeConv2DInfo / getPadAndOutInfo:                               */
/* tfjs-core/src/ops/conv_util.ts:177-236, :421-481, :548-564.         */
/* padMode: 0 'valid', 1 'same', 2 number (padNum), 3 explicit         */
/* (top,bottom,left,right in explicitPad). roundMode: 0 none (trunc),  */
/* 1 floor, 2 round, 3 ceil. info out: [outH, outW, outC, padTop,      */
/* padBottom, padLeft, padRight, effFH, effFW].                        */
/* ------------------------------------------------------------------ */
static double round_mode(double v, int mode) {
  switch (mode) {
    case 1:
      return floor(v);
    case 2:
      return floor(v + 0.5); /* Math.round */
    case 3:
      return ceil(v);
    default:
      return trunc(v);
  }
}

static int64_t effective_filter(int64_t f, int64_t d) {
  return d <= 1 ? f : f + (f - 1) * (d - 1);
}

void orc_conv2d_info(int64_t inH, int64_t inW, int64_t inC, int64_t fH,
                     int64_t fW, int64_t filterChannels, int64_t sH, int64_t sW,
                     int64_t dH, int64_t dW, int padMode, int64_t padNum,
                     const int64_t *explicitPad, int roundMode, int depthwise,
                     int64_t *info) {
  const int64_t eH = effective_filter(fH, dH), eW = effective_filter(fW, dW);
  int64_t top = 0, bottom = 0, left = 0, right = 0, outH = 0, outW = 0;
  if (padMode == 2) {
    top = bottom = left = right = padNum;
    /* computeOutputShape2D (:350-365) uses the filter HEIGHT and the stride
     * HEIGHT for both output dimensions (:443-444). */
    outH = (int64_t)round_mode(
        (double)(inH - eH + 2 * padNum) / (double)sH + 1, roundMode);
    outW = (int64_t)round_mode(
        (double)(inW - eH + 2 * padNum) / (double)sH + 1, roundMode);
  } else if (padMode == 1) {
    outH = (int64_t)ceil((double)inH / (double)sH);
    outW = (int64_t)ceil((double)inW / (double)sW);
    int64_t padAlongH = (outH - 1) * sH + eH - inH;
    int64_t padAlongW = (outW - 1) * sW + eW - inW;
    if (padAlongH < 0) padAlongH = 0;
    if (padAlongW < 0) padAlongW = 0;
    top = padAlongH / 2;
    bottom = padAlongH - top;
    left = padAlongW / 2;
    right = padAlongW - left;
  } else if (padMode == 0) {
    outH = (int64_t)ceil((double)(inH - eH + 1) / (double)sH);
    outW = (int64_t)ceil((double)(inW - eW + 1) / (double)sW);
  } else {
    top = explicitPad[0];
    bottom = explicitPad[1];
    left = explicitPad[2];
    right = explicitPad[3];
    outH = (int64_t)round_mode(
        (double)(inH - eH + top + bottom) / (double)sH + 1, roundMode);
    outW = (int64_t)round_mode(
        (double)(inW - eW + left + right) / (double)sW + 1, roundMode);
  }
  info[0] = outH;
  info[1] = outW;
  info[2] = depthwise ? filterChannels * inC : filterChannels;
  info[3] = top;
  info[4] = bottom;
  info[5] = left;
  info[6] = right;
  info[7] = eH;
  info[8] = eW;
}

/* ------------------------------------------------------------------ */
/* Conv2D: tfjs-backend-cpu/src/kernels/Conv2D.ts:23-103.              */
/* Direct convolution; y[o] = fround(y[o] + x*w) for every tap, loop   */
/* nest b, yR, wR, yC, wC, d1, d2 (:64-96). nchw != 0 selects the      */
/* channelsFirst strides (:48-58). Filter is [fH, fW, inC, outC].      */
/* ------------------------------------------------------------------ */
void orc_conv2d(const float *xVals, const float *wVals, float *yVals,
                int64_t batch, int64_t inH, int64_t inW, int64_t inC,
                int64_t fH, int64_t fW, int64_t outC, int64_t sH, int64_t sW,
                int64_t dH, int64_t dW, int64_t padTop, int64_t padLeft,
                int64_t outH, int64_t outW, int nchw) {
  const int64_t xBatchStride = inH * inW * inC;
  const int64_t xRowStride = nchw ? inW : inW * inC;
  const int64_t xColStride = nchw ? 1 : inC;
  const int64_t xChannelStride = nchw ? inH * inW : 1;
  const int64_t yBatchStride = outH * outW * outC;
  const int64_t yRowStride = nchw ? outW : outW * outC;
  const int64_t yColStride = nchw ? 1 : outC;
  const int64_t yChannelStride = nchw ? outH * outW : 1;
  const int64_t fS0 = fW * inC * outC, fS1 = inC * outC;
  memset(yVals, 0, sizeof(float) * (size_t)(batch * yBatchStride));
#pragma omp parallel for collapse(2) schedule(dynamic)
  for (int64_t b = 0; b < batch; ++b) {
    for (int64_t yR = 0; yR < outH; ++yR) {
      const int64_t xOffset1 = b * xBatchStride;
      const int64_t yOffset1 = b * yBatchStride;
      const int64_t yOffset2 = yOffset1 + yR * yRowStride;
      const int64_t xRCorner = yR * sH - padTop;
      for (int64_t wR = 0; wR < fH; ++wR) {
        const int64_t xR = xRCorner + wR * dH;
        if (xR < 0 || xR >= inH) continue;
        const int64_t wOffset1 = wR * fS0;
        const int64_t xOffset2 = xOffset1 + xR * xRowStride;
        for (int64_t yC = 0; yC < outW; ++yC) {
          const int64_t yOffset3 = yOffset2 + yC * yColStride;
          const int64_t xCCorner = yC * sW - padLeft;
          for (int64_t wC = 0; wC < fW; ++wC) {
            const int64_t xC = xCCorner + wC * dW;
            if (xC < 0 || xC >= inW) continue;
            const int64_t wOffset2 = wOffset1 + wC * fS1;
            const int64_t xOffset3 = xOffset2 + xC * xColStride;
            int64_t wOffset3 = wOffset2;
            for (int64_t d1 = 0; d1 < inC; ++d1) {
              const double xVal = xVals[xOffset3 + d1 * xChannelStride];
              for (int64_t d2 = 0; d2 < outC; ++d2) {
                float *y = &yVals[yOffset3 + d2 * yChannelStride];
                *y = (float)((double)*y + xVal * (double)wVals[wOffset3 + d2]);
              }
              wOffset3 += outC;
            }
          }
        }
      }
    }
  }
}

/* ------------------------------------------------------------------ */
/* DepthwiseConv2dNative:                                              */
/* tfjs-backend-cpu/src/kernels/DepthwiseConv2dNative.ts:23-102.       */
/* NHWC only; filter [fH, fW, inC, chMul]; loop nest b, yR, wR, yC,    */
/* wC, d1, q (:62-95).                                                 */
/* ------------------------------------------------------------------ */
void orc_depthwise_conv2d(const float *xVals, const float *wVals, float *yVals,
                          int64_t batch, int64_t inH, int64_t inW, int64_t inC,
                          int64_t fH, int64_t fW, int64_t chMul, int64_t sH,
                          int64_t sW, int64_t dH, int64_t dW, int64_t padTop,
                          int64_t padLeft, int64_t outH, int64_t outW) {
  const int64_t outC = inC * chMul;
  const int64_t xS0 = inH * inW * inC, xS1 = inW * inC;
  const int64_t yS0 = outH * outW * outC, yS1 = outW * outC, yS2 = outC;
  const int64_t fS0 = fW * inC * chMul, fS1 = inC * chMul;
  memset(yVals, 0, sizeof(float) * (size_t)(batch * yS0));
#pragma omp parallel for collapse(2) schedule(dynamic)
  for (int64_t b = 0; b < batch; ++b) {
    for (int64_t yR = 0; yR < outH; ++yR) {
      const int64_t xOffset1 = b * xS0;
      const int64_t yOffset1 = b * yS0;
      const int64_t yOffset2 = yOffset1 + yR * yS1;
      const int64_t xRCorner = yR * sH - padTop;
      for (int64_t wR = 0; wR < fH; ++wR) {
        const int64_t xR = xRCorner + wR * dH;
        if (xR < 0 || xR >= inH) continue;
        const int64_t wOffset1 = wR * fS0;
        const int64_t xOffset2 = xOffset1 + xR * xS1;
        for (int64_t yC = 0; yC < outW; ++yC) {
          const int64_t yOffset3 = yOffset2 + yC * yS2;
          const int64_t xCCorner = yC * sW - padLeft;
          for (int64_t wC = 0; wC < fW; ++wC) {
            const int64_t xC = xCCorner + wC * dW;
            if (xC < 0 || xC >= inW) continue;
            const int64_t wOffset2 = wOffset1 + wC * fS1;
            const int64_t xOffset3 = xOffset2 + xC * inC;
            int64_t yOffset4 = yOffset3;
            int64_t wOffset3 = wOffset2;
            for (int64_t d1 = 0; d1 < inC; ++d1) {
              const double xVal = xVals[xOffset3 + d1];
              for (int64_t q = 0; q < chMul; ++q) {
                float *y = &yVals[yOffset4 + q];
                *y = (float)((double)*y + xVal * (double)wVals[wOffset3 + q]);
              }
              yOffset4 += chMul;
              wOffset3 += chMul;
            }
          }
        }
      }
    }
  }
}

/* ------------------------------------------------------------------ */
/* FusedConv2D: tfjs-backend-cpu/src/kernels/FusedConv2D.ts:26-95 and  */
/* FusedDepthwiseConv2D.ts:25-61: conv, then broadcasting add of the   */
/* bias, then the activation, each as its own float32-rounded pass.    */
/* For NCHW a 1-D bias / prelu tensor of length != 1 is reshaped to    */
/* [C,1,1] (FusedConv2D.ts:55-61, :76-86).                             */
/* ------------------------------------------------------------------ */
static int fused_tail(float *y, const int64_t *yShape, int nchw,
                      const float *bias, const int64_t *biasShape, int biasRank,
                      int act, const float *prelu, const int64_t *preluShape,
                      int preluRank, double leakyAlpha) {
  int64_t tmpShape[3];
  if (bias) {
    if (nchw && biasRank == 1 && biasShape[0] != 1) {
      tmpShape[0] = biasShape[0];
      tmpShape[1] = 1;
      tmpShape[2] = 1;
      if (add_bias(y, yShape, 4, bias, tmpShape, 3)) return -1;
    } else if (add_bias(y, yShape, 4, bias, biasShape, biasRank)) {
      return -1;
    }
  }
  if (nchw && act == ORC_PRELU && preluRank == 1 && preluShape[0] != 1) {
    tmpShape[0] = preluShape[0];
    tmpShape[1] = 1;
    tmpShape[2] = 1;
    return apply_activation(act, y, yShape, 4, prelu, tmpShape, 3, leakyAlpha);
  }
  return apply_activation(act, y, yShape, 4, prelu, preluShape, preluRank,
                          leakyAlpha);
}

int orc_fused_conv2d(const float *x, const float *w, float *y, int64_t batch,
                     int64_t inH, int64_t inW, int64_t inC, int64_t fH,
                     int64_t fW, int64_t outC, int64_t sH, int64_t sW,
                     int64_t dH, int64_t dW, int64_t padTop, int64_t padLeft,
                     int64_t outH, int64_t outW, int nchw, const float *bias,
                     const int64_t *biasShape, int biasRank, int act,
                     const float *prelu, const int64_t *preluShape,
                     int preluRank, double leakyAlpha) {
  orc_conv2d(x, w, y, batch, inH, inW, inC, fH, fW, outC, sH, sW, dH, dW,
             padTop, padLeft, outH, outW, nchw);
  int64_t yShape[4] = {batch, outH, outW, outC};
  if (nchw) {
    yShape[1] = outC;
    yShape[2] = outH;
    yShape[3] = outW;
  }
  return fused_tail(y, yShape, nchw, bias, biasShape, biasRank, act, prelu,
                    preluShape, preluRank, leakyAlpha);
}

int orc_fused_depthwise_conv2d(const float *x, const float *w, float *y,
                               int64_t batch, int64_t inH, int64_t inW,
                               int64_t inC, int64_t fH, int64_t fW,
                               int64_t chMul, int64_t sH, int64_t sW,
                               int64_t dH, int64_t dW, int64_t padTop,
                               int64_t padLeft, int64_t outH, int64_t outW,
                               const float *bias, const int64_t *biasShape,
                               int biasRank, int act, const float *prelu,
                               const int64_t *preluShape, int preluRank,
                               double leakyAlpha) {
  orc_depthwise_conv2d(x, w, y, batch, inH, inW, inC, fH, fW, chMul, sH, sW,
                       dH, dW, padTop, padLeft, outH, outW);
  const int64_t yShape[4] = {batch, outH, outW, inC * chMul};
  return fused_tail(y, yShape, 0, bias, biasShape, biasRank, act, prelu,
                    preluShape, preluRank, leakyAlpha);
}

/* ------------------------------------------------------------------ */
/* Weight dequantisation: tfjs-core/src/io/io_utils.ts:185-251.        */
/* ------------------------------------------------------------------ */

/* uint8 / uint16 -> float32 (:223-227): values[i] = v * scale + min in
 * double, stored to a Float32Array. `q` may be unaligned for uint16. */
void orc_dequant_affine_f32(const uint8_t *q, int bits, int64_t n, double scale,
                            double min, float *out) {
#pragma omp parallel for
  for (int64_t i = 0; i < n; ++i) {
    uint32_t v;
    if (bits == 8) {
      v = q[i];
    } else {
      v = (uint32_t)q[2 * i] | ((uint32_t)q[2 * i + 1] << 8);
    }
    out[i] = (float)((double)v * scale + min);
  }
}

/* Math.round: nearest integer, ties toward +infinity. */
static double js_math_round(double x) {
  if (x != x || isinf(x)) return x;
  const double f = floor(x);
  return (x - f >= 0.5) ? f + 1.0 : f;
}

/* ECMAScript ToInt32, the conversion an Int32Array store applies. */
static int32_t js_to_int32(double x) {
  if (x != x || isinf(x)) return 0;
  double t = trunc(x);
  double m = fmod(t, 4294967296.0);
  if (m < 0) m += 4294967296.0;
  return (int32_t)(uint32_t)(m);
}

/* uint8 / uint16 -> int32 (:243-247): Math.round(v * scale + min). */
void orc_dequant_affine_i32(const uint8_t *q, int bits, int64_t n, double scale,
                            double min, int32_t *out) {
#pragma omp parallel for
  for (int64_t i = 0; i < n; ++i) {
    uint32_t v;
    if (bits == 8) {
      v = q[i];
    } else {
      v = (uint32_t)q[2 * i] | ((uint32_t)q[2 * i + 1] << 8);
    }
    out[i] = js_to_int32(js_math_round((double)v * scale + min));
  }
}

/* float16 -> float32 through the three lookup tables:
 * computeFloat16MantisaTable :645-670, computeFloat16ExponentTable :678-694,
 * computeFloat16OffsetTable :702-711, decoder :720-741. */
static uint32_t f16_mantissa[2048], f16_exponent[64], f16_offset[64];
static int f16_tables_ready = 0;

static uint32_t convert_mantissa(uint32_t i) {
  uint32_t m = i << 13;
  uint32_t e = 0;
  while ((m & 0x00800000u) == 0) {
    e -= 0x00800000u;
    m <<= 1;
  }
  m &= ~0x00800000u;
  e += 0x38800000u;
  return m | e;
}

static void f16_build_tables(void) {
  f16_mantissa[0] = 0;
  for (uint32_t i = 1; i < 1024; i++) f16_mantissa[i] = convert_mantissa(i);
  for (uint32_t i = 1024; i < 2048; i++)
    f16_mantissa[i] = 0x38000000u + ((i - 1024) << 13);
  memset(f16_exponent, 0, sizeof f16_exponent);
  f16_exponent[31] = 0x47800000u;
  f16_exponent[32] = 0x80000000u;
  f16_exponent[63] = 0xc7800000u;
  for (uint32_t i = 1; i < 31; i++) f16_exponent[i] = i << 23;
  for (uint32_t i = 33; i < 63; i++)
    f16_exponent[i] = 0x80000000u + ((i - 32) << 23);
  for (int i = 0; i < 64; i++) f16_offset[i] = 1024;
  f16_offset[0] = f16_offset[32] = 0;
  f16_tables_ready = 1;
}

void orc_dequant_f16(const uint8_t *q, int64_t n, uint32_t *outBits) {
  if (!f16_tables_ready) f16_build_tables();
#pragma omp parallel for
  for (int64_t i = 0; i < n; ++i) {
    const uint32_t h = (uint32_t)q[2 * i] | ((uint32_t)q[2 * i + 1] << 8);
    /* Uint32Array store wraps modulo 2^32, as uint32_t addition does */
    outBits[i] = f16_mantissa[f16_offset[h >> 10] + (h & 0x3ff)] +
                 f16_exponent[h >> 10];
  }
}

/* ------------------------------------------------------------------ */
/* Glue kernels around the fused ops in a MobileNetV2 graph.           */
/* ------------------------------------------------------------------ */

/* Mean over the two middle axes of an NHWC tensor, the global average pool:
 * tfjs-backend-cpu/src/kernels/Mean.ts:41-48 divides every element by the
 * reduce size into a float32 tensor first; Sum.ts:67-73 then accumulates each
 * output in a double and stores float32. Sum transposes the reduced axes
 * innermost, so the order of accumulation is h-major, w-minor. */
void orc_mean_hw(const float *x, float *y, int64_t batch, int64_t H, int64_t W,
                 int64_t C) {
  const double reduceSize = (double)(float)(H * W);
#pragma omp parallel for collapse(2)
  for (int64_t b = 0; b < batch; ++b) {
    for (int64_t c = 0; c < C; ++c) {
      double sum = 0;
      for (int64_t i = 0; i < H * W; ++i) {
        const float d = (float)((double)x[(b * H * W + i) * C + c] / reduceSize);
        sum += (double)d;
      }
      y[b * C + c] = (float)sum;
    }
  }
}

/* AvgPool, NHWC: tfjs-backend-cpu/src/kernels/AvgPool.ts:25-58 over
 * utils/pool_utils.ts:20-87 with poolType 'avg' and dilation 1: the window's
 * elements inside the image are summed in a double, row by row, and divided by
 * their count; the store rounds to float32. */
void orc_avg_pool(const float *xValues, float *outputVals, int64_t batchSize,
                  int64_t inHeight, int64_t inWidth, int64_t inChannels,
                  int64_t effectiveFilterHeight, int64_t effectiveFilterWidth,
                  int64_t strideHeight, int64_t strideWidth, int64_t padTop,
                  int64_t padLeft, int64_t outHeight, int64_t outWidth) {
  const int64_t s0 = inHeight * inWidth * inChannels, s1 = inWidth * inChannels,
                s2 = inChannels;
  const int64_t outputBatchStrides = outHeight * outWidth * inChannels;
  const int64_t outputRowStrides = outWidth * inChannels;
  const int64_t outputColStrides = inChannels;
#pragma omp parallel for collapse(2)
  for (int64_t b = 0; b < batchSize; ++b) {
    for (int64_t d = 0; d < inChannels; ++d) {
      const int64_t outputBatchOffset = b * outputBatchStrides;
      const int64_t inputBatchOffset = b * s0;
      for (int64_t yR = 0; yR < outHeight; ++yR) {
        const int64_t xRCorner = yR * strideHeight - padTop;
        const int64_t xRMin = xRCorner > 0 ? xRCorner : 0;
        const int64_t xRMax = inHeight < effectiveFilterHeight + xRCorner
                                  ? inHeight
                                  : effectiveFilterHeight + xRCorner;
        const int64_t outputRowOffset = outputBatchOffset + yR * outputRowStrides;
        for (int64_t yC = 0; yC < outWidth; ++yC) {
          const int64_t xCCorner = yC * strideWidth - padLeft;
          const int64_t xCMin = xCCorner > 0 ? xCCorner : 0;
          const int64_t xCMax = inWidth < effectiveFilterWidth + xCCorner
                                    ? inWidth
                                    : effectiveFilterWidth + xCCorner;
          double avgValue = 0;
          int64_t count = 0;
          for (int64_t xR = xRMin; xR < xRMax; xR += 1) {
            const int64_t xROffset = inputBatchOffset + xR * s1;
            for (int64_t xC = xCMin; xC < xCMax; xC += 1) {
              const int64_t xCOffset = xROffset + xC * s2;
              avgValue += (double)xValues[xCOffset + d];
              count++;
            }
          }
          const int64_t outputOffset = outputRowOffset + yC * outputColStrides + d;
          outputVals[outputOffset] = (float)(avgValue / (double)count);
        }
      }
    }
  }
}

/* Cast: tfjs-backend-cpu/src/kernels/Cast.ts:28-46.
 *   to int32: Int32Array.from(values) stores ECMAScript ToInt32(v) (js_to_int32
 *     above): NaN and the infinities become 0; any other value is truncated toward
 *     zero and taken modulo 2^32 into [-2^31, 2^31);
 *   to bool: (a !== b) ? 1 : 0 against zero (NaN !== 0 is true);
 *   to float32 from int32 / bool (no encoding loss path): Float32Array store. */
void orc_cast_f32_to_i32(const float *x, int32_t *y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) y[i] = js_to_int32((double)x[i]);
}

void orc_cast_f32_to_bool(const float *x, uint8_t *y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) y[i] = (x[i] != 0.0f) ? 1 : 0;
}

void orc_cast_i32_to_bool(const int32_t *x, uint8_t *y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) y[i] = (x[i] != 0) ? 1 : 0;
}

void orc_cast_i32_to_f32(const int32_t *x, float *y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) y[i] = (float)(double)x[i];
}
