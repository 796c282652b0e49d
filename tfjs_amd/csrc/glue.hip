// The non-contraction kernels a MobileNetV2 graph needs between the fused ops,
// so that no tensor leaves the device mid-graph: the broadcasting binary ops
// (Add of the skip connections; Sub and Multiply, which a converted graph uses to
// scale its input), the stand-alone activations, the global average pool (Mean
// over H and W, or AvgPool), Cast and the rank-2 Transpose.
#include "common.h"
#include "epilogue.h"

namespace tfhip {
namespace {

constexpr int kMaxRank = 6;

struct AddParams {
  const float *a;
  const float *b;
  float *out;
  long long total;
  int rank;
  long long shape[kMaxRank];
  long long a_s[kMaxRank];
  long long b_s[kMaxRank];
};

// Binary ops: a float32 result of float32 operands equals the reference's double expression rounded
// once (one IEEE operation), so plain float arithmetic gives its bits. The compiler must not fuse
// these into anything: each is one rounded operation.
enum BinaryOp { kAdd = 0, kSub = 1, kMul = 2 };

template <int OP>
__device__ __forceinline__ float binary_apply(float u, float v) {
  return OP == kAdd ? __fadd_rn(u, v) : (OP == kSub ? __fsub_rn(u, v) : __fmul_rn(u, v));
}

__global__ __launch_bounds__(256) void add_same_shape(const float4 *__restrict__ a, const float4 *__restrict__ b,
                                                      float4 *__restrict__ out, long long groups) {
  const long long stride = (long long)gridDim.x * 256;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < groups; i += stride) {
    const float4 u = a[i], v = b[i];
    out[i] = make_float4(u.x + v.x, u.y + v.y, u.z + v.z, u.w + v.w);
  }
}

template <int OP>
__global__ __launch_bounds__(256) void binary_same_shape(const float4 *__restrict__ a, const float4 *__restrict__ b,
                                                         float4 *__restrict__ out, long long groups) {
  const long long stride = (long long)gridDim.x * 256;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < groups; i += stride) {
    const float4 u = a[i], v = b[i];
    out[i] = make_float4(binary_apply<OP>(u.x, v.x), binary_apply<OP>(u.y, v.y), binary_apply<OP>(u.z, v.z),
                         binary_apply<OP>(u.w, v.w));
  }
}

template <int OP>
__global__ __launch_bounds__(256) void binary_broadcast(AddParams p) {
  const long long stride = (long long)gridDim.x * 256;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < p.total; i += stride) {
    long long rem = i, ia = 0, ib = 0;
#pragma unroll
    for (int d = kMaxRank - 1; d >= 0; --d) {
      if (d < p.rank) {
        const long long loc = rem % p.shape[d];
        rem /= p.shape[d];
        ia += loc * p.a_s[d];
        ib += loc * p.b_s[d];
      }
    }
    p.out[i] = binary_apply<OP>(p.a[ia], p.b[ib]);
  }
}

// Stand-alone activation (the kernels Relu, Relu6, Elu, LeakyRelu, Sigmoid): the fused epilogue's
// arithmetic (epilogue.h: activate) on a tensor of its own.
__global__ __launch_bounds__(256) void unary_activation(const float *__restrict__ x, float *__restrict__ y, long long n,
                                                        int activation, double alpha) {
  const long long stride = (long long)gridDim.x * 256;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
    y[i] = activate(x[i], activation, 0.f, alpha);
  }
}

struct PoolParams {
  const float *x;
  float *y;
  int batch, in_h, in_w, c, f_h, f_w, stride_h, stride_w, pad_top, pad_left, out_h, out_w;
};

// AvgPool, NHWC: a lane per output element, consecutive lanes consecutive channels. The window's
// elements inside the image are summed in a double by row then column and divided by their count
// (tfjs-backend-cpu/src/utils/pool_utils.ts:45-84).
__global__ __launch_bounds__(256) void avg_pool(PoolParams p) {
  const long long total = (long long)p.batch * p.out_h * p.out_w * p.c;
  const long long stride = (long long)gridDim.x * 256;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
    const int d = (int)(i % p.c);
    long long rem = i / p.c;
    const int yc = (int)(rem % p.out_w);
    rem /= p.out_w;
    const int yr = (int)(rem % p.out_h), b = (int)(rem / p.out_h);
    const int r0 = yr * p.stride_h - p.pad_top, c0 = yc * p.stride_w - p.pad_left;
    const int r_lo = r0 < 0 ? 0 : r0, r_hi = r0 + p.f_h < p.in_h ? r0 + p.f_h : p.in_h;
    const int c_lo = c0 < 0 ? 0 : c0, c_hi = c0 + p.f_w < p.in_w ? c0 + p.f_w : p.in_w;
    double sum = 0.0;
    int count = 0;
    for (int r = r_lo; r < r_hi; ++r) {
      const float *row = p.x + (((long long)b * p.in_h + r) * p.in_w) * p.c + d;
      for (int cc = c_lo; cc < c_hi; ++cc) {
        sum += (double)row[(long long)cc * p.c];
        ++count;
      }
    }
    p.y[i] = (float)(sum / (double)count);   // (an empty window divides 0 by 0: NaN, as in the reference)
  }
}

// Cast between float32 (0), int32 (1) and bool (2, one byte per element):
//   -> int32: Int32Array.from(values), i.e. ECMAScript ToInt32: NaN and infinities give 0, anything
//             else is truncated toward zero and wrapped modulo 2^32
//   -> bool:  x != 0 (NaN is not equal to 0: true)
//   -> float32 from int32 / bool: the nearest float32
// (tfjs-backend-cpu/src/kernels/Cast.ts:28-46).
__device__ __forceinline__ int to_int32(float v) {
  if (!(v == v) || v == __builtin_inff() || v == -__builtin_inff()) return 0;
  const double t = trunc((double)v);
  // wrap into [0, 2^32), then reinterpret: fmod is exact
  double m = fmod(t, 4294967296.0);
  if (m < 0) m += 4294967296.0;
  return (int)(unsigned)m;
}

__global__ __launch_bounds__(256) void cast_elements(const void *__restrict__ x, void *__restrict__ y, long long n,
                                                     int from, int to) {
  const long long stride = (long long)gridDim.x * 256;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
    float f = 0.f;
    int k = 0;
    if (from == 0) {
      f = static_cast<const float *>(x)[i];
    } else if (from == 1) {
      k = static_cast<const int *>(x)[i];
    } else {
      k = static_cast<const unsigned char *>(x)[i];
    }
    if (to == 0) {
      static_cast<float *>(y)[i] = from == 0 ? f : (float)k;
    } else if (to == 1) {
      static_cast<int *>(y)[i] = from == 0 ? to_int32(f) : k;
    } else {
      static_cast<unsigned char *>(y)[i] = from == 0 ? (f != 0.f ? 1 : 0) : (k != 0 ? 1 : 0);
    }
  }
}

__global__ __launch_bounds__(256) void add_broadcast(AddParams p) {
  const long long stride = (long long)gridDim.x * 256;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < p.total; i += stride) {
    long long rem = i, ia = 0, ib = 0;
#pragma unroll
    for (int d = kMaxRank - 1; d >= 0; --d) {
      if (d < p.rank) {
        const long long loc = rem % p.shape[d];
        rem /= p.shape[d];
        ia += loc * p.a_s[d];
        ib += loc * p.b_s[d];
      }
    }
    p.out[i] = p.a[ia] + p.b[ib];
  }
}

// One lane per (n, c): consecutive lanes read consecutive channels.
__global__ __launch_bounds__(256) void mean_hw(const float *__restrict__ x, float *__restrict__ y, long long batch,
                                               long long hw, long long c) {
  const float denom = (float)hw;
  const long long total = batch * c;
  const long long stride = (long long)gridDim.x * 256;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
    const long long n = i / c, ch = i - n * c;
    const float *px = x + n * hw * c + ch;
    double sum = 0.0;
    for (long long j = 0; j < hw; ++j) sum += (double)__fdiv_rn(px[j * c], denom);
    y[i] = (float)sum;
  }
}

// The same for c % 4 == 0: a lane takes four channels (one 16-byte load per
// position) and one of eight interleaved slices of the h*w positions, so that all
// loads of a small feature map are in flight at once; the eight partial sums
// (double, positions in ascending order within a slice) are added in slice
// order through LDS.
__global__ __launch_bounds__(256) void mean_hw_vec(const float *__restrict__ x, float *__restrict__ y, long long batch,
                                                   long long hw, long long c) {
  __shared__ double part[8][32][4];
  const float denom = (float)hw;
  const int slice = threadIdx.x >> 5, q = threadIdx.x & 31;
  const long long quads = c / 4, total = batch * quads;
  for (long long base = (long long)blockIdx.x * 32; base < total; base += (long long)gridDim.x * 32) {
    const long long i = base + q;
    double sum[4] = {0.0, 0.0, 0.0, 0.0};
    if (i < total) {
      const long long n = i / quads, cq = i - n * quads;
      const float4 *px = reinterpret_cast<const float4 *>(x + n * hw * c + cq * 4);
      for (long long j0 = slice; j0 < hw; j0 += 64) {
        float4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const long long j = j0 + 8 * u;
          v[u] = j < hw ? px[j * quads] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          if (j0 + 8 * u >= hw) continue;
          sum[0] += (double)__fdiv_rn(v[u].x, denom);
          sum[1] += (double)__fdiv_rn(v[u].y, denom);
          sum[2] += (double)__fdiv_rn(v[u].z, denom);
          sum[3] += (double)__fdiv_rn(v[u].w, denom);
        }
      }
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) part[slice][q][k] = sum[k];
    __syncthreads();
    if (threadIdx.x < 128) {
      const int qq = threadIdx.x >> 2, k = threadIdx.x & 3;
      const long long o = base + qq;
      if (o < total) {
        double t = 0.0;
#pragma unroll
        for (int sl = 0; sl < 8; ++sl) t += part[sl][qq][k];
        y[o * 4 + k] = (float)t;
      }
    }
    __syncthreads();
  }
}

__global__ __launch_bounds__(256) void copy_f4(const float4 *__restrict__ src, float4 *__restrict__ dst, long long n4) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) dst[i] = src[i];
}

// One item per lane where the grid allows it: streaming kernels whose workgroups start in address
// order and drift apart use the memory channels better than a small grid of lanes striding in step
// (a 1 GiB copy: 80% of the memory bandwidth against 62% with 32 workgroups per compute unit).
int grid_for(long long items) {
  long long blocks = (items + 255) / 256;
  const long long cap = 0x3fffffLL;
  if (blocks > cap) blocks = cap;
  return blocks < 1 ? 1 : (int)blocks;
}

}  // namespace
}  // namespace tfhip

using namespace tfhip;

// y[c][r] = x[r][c] through a 32 x 33 LDS tile: reads and writes both run along rows.
__global__ __launch_bounds__(256) void transpose2d(const float *__restrict__ x, float *__restrict__ y, int rows, int cols) {
  __shared__ float tile[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  const int r0 = blockIdx.y * 32, c0 = blockIdx.x * 32;
  for (int i = ty; i < 32; i += 8) {
    const int r = r0 + i, c = c0 + tx;
    if (r < rows && c < cols) tile[i][tx] = x[(long long)r * cols + c];
  }
  __syncthreads();
  for (int i = ty; i < 32; i += 8) {
    const int c = c0 + i, r = r0 + tx;
    if (r < rows && c < cols) y[(long long)c * rows + r] = tile[tx][i];
  }
}

extern "C" {

int tfhip_transpose2d(const float *x, float *y, int64_t rows, int64_t cols) {
  TFHIP_REQUIRE_INIT();
  TFHIP_CHECK_ARG(rows >= 0 && cols >= 0 && rows < 0x7fffffff && cols < 0x7fffffff, "tfhip_transpose2d: bad dimensions");
  if (rows * cols == 0) return kOk;
  TFHIP_CHECK_ARG((rows + 31) / 32 <= 65535, "tfhip_transpose2d: more than 2 097 120 rows");
  TFHIP_CHECK_RANGE(x, rows * cols, 4, "x");
  TFHIP_CHECK_OUTPUT(y, rows * cols, 4, "y");
  TFHIP_CHECK_ARG(x != y, "tfhip_transpose2d: x and y are the same buffer");
  note_kernel("transpose2d");
  const dim3 grid((unsigned)((cols + 31) / 32), (unsigned)((rows + 31) / 32));
  TFHIP_LAUNCH((transpose2d<<<grid, 256, 0, stream()>>>(x, y, (int)rows, (int)cols)));
  return kOk;
}

int tfhip_add(const float *a, const int64_t *a_strides, const float *b, const int64_t *b_strides, float *out,
              const int64_t *out_shape, int rank) {
  TFHIP_REQUIRE_INIT();
  TFHIP_CHECK_ARG(rank >= 0 && rank <= kMaxRank, "tfhip_add: rank %d not in 0..%d", rank, kMaxRank);
  TFHIP_CHECK_ARG(rank == 0 || (a_strides && b_strides && out_shape), "tfhip_add: missing shape or strides");
  AddParams p = {};
  p.a = a; p.b = b; p.out = out; p.rank = rank;
  long long total = 1;
  bool dense = true;
  for (int d = rank - 1; d >= 0; --d) {
    TFHIP_CHECK_ARG(out_shape[d] >= 0 && a_strides[d] >= 0 && b_strides[d] >= 0, "tfhip_add: negative extent or stride");
    TFHIP_CHECK_ARG(out_shape[d] == 0 || total <= kMaxElems / out_shape[d], "tfhip_add: tensor exceeds the supported range");
    if (out_shape[d] > 1 && (a_strides[d] != total || b_strides[d] != total)) dense = false;
    p.shape[d] = out_shape[d];
    p.a_s[d] = a_strides[d];
    p.b_s[d] = b_strides[d];
    total *= out_shape[d];
  }
  p.total = total;
  if (total == 0) return kOk;
  TFHIP_CHECK_RANGE(a, strided_extent(out_shape, a_strides, rank), 4, "a");
  TFHIP_CHECK_RANGE(b, strided_extent(out_shape, b_strides, rank), 4, "b");
  TFHIP_CHECK_OUTPUT(out, total, 4, "out");
  const bool aligned = reinterpret_cast<uintptr_t>(a) % 16 == 0 && reinterpret_cast<uintptr_t>(b) % 16 == 0 &&
                       reinterpret_cast<uintptr_t>(out) % 16 == 0;
  if (dense && aligned && total % 4 == 0) {
    note_kernel("add_same_shape");
    TFHIP_LAUNCH((add_same_shape<<<grid_for(total / 4), 256, 0, stream()>>>((const float4 *)a, (const float4 *)b,
                                                                          (float4 *)out, total / 4)));
  } else {
    note_kernel("add_broadcast");
    TFHIP_LAUNCH((add_broadcast<<<grid_for(total), 256, 0, stream()>>>(p)));
  }
  return kOk;
}

int tfhip_binary(int op, const float *a, const int64_t *a_strides, const float *b, const int64_t *b_strides, float *out,
                 const int64_t *out_shape, int rank) {
  if (op == kAdd) return tfhip_add(a, a_strides, b, b_strides, out, out_shape, rank);
  TFHIP_REQUIRE_INIT();
  TFHIP_CHECK_ARG(op == kSub || op == kMul, "tfhip_binary: unknown op %d (0 add, 1 sub, 2 mul)", op);
  TFHIP_CHECK_ARG(rank >= 0 && rank <= kMaxRank, "tfhip_binary: rank %d not in 0..%d", rank, kMaxRank);
  TFHIP_CHECK_ARG(rank == 0 || (a_strides && b_strides && out_shape), "tfhip_binary: missing shape or strides");
  AddParams p = {};
  p.a = a; p.b = b; p.out = out; p.rank = rank;
  long long total = 1;
  bool dense = true;
  for (int d = rank - 1; d >= 0; --d) {
    TFHIP_CHECK_ARG(out_shape[d] >= 0 && a_strides[d] >= 0 && b_strides[d] >= 0, "tfhip_binary: negative extent or stride");
    TFHIP_CHECK_ARG(out_shape[d] == 0 || total <= kMaxElems / out_shape[d], "tfhip_binary: tensor exceeds the supported range");
    if (out_shape[d] > 1 && (a_strides[d] != total || b_strides[d] != total)) dense = false;
    p.shape[d] = out_shape[d];
    p.a_s[d] = a_strides[d];
    p.b_s[d] = b_strides[d];
    total *= out_shape[d];
  }
  p.total = total;
  if (total == 0) return kOk;
  TFHIP_CHECK_RANGE(a, strided_extent(out_shape, a_strides, rank), 4, "a");
  TFHIP_CHECK_RANGE(b, strided_extent(out_shape, b_strides, rank), 4, "b");
  TFHIP_CHECK_OUTPUT(out, total, 4, "out");
  const bool aligned = reinterpret_cast<uintptr_t>(a) % 16 == 0 && reinterpret_cast<uintptr_t>(b) % 16 == 0 &&
                       reinterpret_cast<uintptr_t>(out) % 16 == 0;
  if (dense && aligned && total % 4 == 0) {
    note_kernel("binary_same_shape<%d>", op);
    if (op == kSub) {
      TFHIP_LAUNCH((binary_same_shape<kSub><<<grid_for(total / 4), 256, 0, stream()>>>((const float4 *)a, (const float4 *)b,
                                                                                     (float4 *)out, total / 4)));
    } else {
      TFHIP_LAUNCH((binary_same_shape<kMul><<<grid_for(total / 4), 256, 0, stream()>>>((const float4 *)a, (const float4 *)b,
                                                                                     (float4 *)out, total / 4)));
    }
  } else {
    note_kernel("binary_broadcast<%d>", op);
    if (op == kSub) {
      TFHIP_LAUNCH((binary_broadcast<kSub><<<grid_for(total), 256, 0, stream()>>>(p)));
    } else {
      TFHIP_LAUNCH((binary_broadcast<kMul><<<grid_for(total), 256, 0, stream()>>>(p)));
    }
  }
  return kOk;
}

int tfhip_unary(int activation, const float *x, float *y, int64_t n, double leakyrelu_alpha) {
  TFHIP_REQUIRE_INIT();
  TFHIP_CHECK_ARG(activation == TFHIP_RELU || activation == TFHIP_RELU6 || activation == TFHIP_LEAKYRELU ||
                      activation == TFHIP_SIGMOID || activation == TFHIP_ELU,
                  "tfhip_unary: activation %d is not one of relu, relu6, leakyrelu, sigmoid, elu", activation);
  TFHIP_CHECK_ARG(n >= 0, "tfhip_unary: negative size");
  if (n == 0) return kOk;
  TFHIP_CHECK_RANGE(x, n, 4, "x");
  TFHIP_CHECK_OUTPUT(y, n, 4, "y");
  note_kernel("unary_activation");
  TFHIP_LAUNCH((unary_activation<<<grid_for(n), 256, 0, stream()>>>(x, y, n, activation, leakyrelu_alpha)));
  return kOk;
}

int tfhip_avg_pool(const float *x, float *y, int64_t batch, int64_t in_h, int64_t in_w, int64_t c, int64_t f_h,
                   int64_t f_w, int64_t stride_h, int64_t stride_w, int64_t pad_top, int64_t pad_left, int64_t out_h,
                   int64_t out_w) {
  TFHIP_REQUIRE_INIT();
  const int64_t lim = 0x7fffffff;
  TFHIP_CHECK_ARG(batch >= 0 && in_h > 0 && in_w > 0 && c >= 0 && f_h > 0 && f_w > 0 && stride_h > 0 && stride_w > 0 &&
                      pad_top >= 0 && pad_left >= 0 && out_h >= 0 && out_w >= 0,
                  "tfhip_avg_pool: bad dimensions");
  TFHIP_CHECK_ARG(batch < lim && in_h < lim && in_w < lim && c < lim && f_h < lim && f_w < lim && stride_h < lim &&
                      stride_w < lim && pad_top < lim && pad_left < lim && out_h < lim && out_w < lim,
                  "tfhip_avg_pool: dimension exceeds 2^31-1");
  // (a window may lie outside the image altogether - the reference's output extent for a numeric pad is worked
  // out from the filter height and the row stride alone, computeOutputShape2D in conv_util.ts:350-365 - and
  // averages nothing: 0 / 0, NaN, as pool_utils.ts:81 leaves it)
  TFHIP_CHECK_ARG(out_h * stride_h + f_h < lim && out_w * stride_w + f_w < lim,
                  "tfhip_avg_pool: window positions exceed 2^31-1");
  TFHIP_CHECK_ARG(product_below(kMaxElems, {batch, in_h, in_w, c}) && product_below(kMaxElems, {batch, out_h, out_w, c}),
                  "tfhip_avg_pool: tensor exceeds the supported range");
  if (batch * out_h * out_w * c == 0) return kOk;
  TFHIP_CHECK_RANGE(x, batch * in_h * in_w * c, 4, "x");
  TFHIP_CHECK_OUTPUT(y, batch * out_h * out_w * c, 4, "y");
  PoolParams p = {x, y, (int)batch, (int)in_h, (int)in_w, (int)c, (int)f_h, (int)f_w, (int)stride_h, (int)stride_w,
                  (int)pad_top, (int)pad_left, (int)out_h, (int)out_w};
  note_kernel("avg_pool");
  TFHIP_LAUNCH((avg_pool<<<grid_for(batch * out_h * out_w * c), 256, 0, stream()>>>(p)));
  return kOk;
}

int tfhip_cast(const void *x, int from_dtype, void *y, int to_dtype, int64_t n) {
  TFHIP_REQUIRE_INIT();
  TFHIP_CHECK_ARG(from_dtype >= 0 && from_dtype <= 2 && to_dtype >= 0 && to_dtype <= 2,
                  "tfhip_cast: dtypes are 0 (float32), 1 (int32), 2 (bool)");
  TFHIP_CHECK_ARG(n >= 0, "tfhip_cast: negative size");
  if (n == 0) return kOk;
  TFHIP_CHECK_RANGE(x, n, from_dtype == 2 ? 1 : 4, "x");
  TFHIP_CHECK_OUTPUT(y, n, to_dtype == 2 ? 1 : 4, "y");
  note_kernel("cast_elements");
  TFHIP_LAUNCH((cast_elements<<<grid_for(n), 256, 0, stream()>>>(x, y, n, from_dtype, to_dtype)));
  return kOk;
}

int tfhip_mean_hw(const float *x, float *y, int64_t batch, int64_t h, int64_t w, int64_t c) {
  TFHIP_REQUIRE_INIT();
  TFHIP_CHECK_ARG(batch >= 0 && h > 0 && w > 0 && c >= 0, "tfhip_mean_hw: bad dimensions");
  TFHIP_CHECK_ARG(product_below(kMaxElems, {batch, h, w, c}), "tfhip_mean_hw: tensor exceeds the supported range");
  if (batch * c == 0) return kOk;
  TFHIP_CHECK_RANGE(x, batch * h * w * c, 4, "x");
  TFHIP_CHECK_OUTPUT(y, batch * c, 4, "y");
  if (c % 4 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0) {
    long long blocks = (batch * (c / 4) + 31) / 32;
    const long long cap = (long long)num_cus() * 32;
    note_kernel("mean_hw_vec");
    TFHIP_LAUNCH((mean_hw_vec<<<(unsigned)(blocks < cap ? blocks : cap), 256, 0, stream()>>>(x, y, batch, h * w, c)));
    return kOk;
  }
  note_kernel("mean_hw");
  TFHIP_LAUNCH((mean_hw<<<grid_for(batch * c), 256, 0, stream()>>>(x, y, batch, h * w, c)));
  return kOk;
}

int tfhip_copy(void *dst, const void *src, size_t bytes) {
  TFHIP_REQUIRE_INIT();
  if (bytes == 0) return kOk;
  TFHIP_CHECK_ARG(bytes % 16 == 0 && reinterpret_cast<uintptr_t>(dst) % 16 == 0 &&
                      reinterpret_cast<uintptr_t>(src) % 16 == 0,
                  "tfhip_copy: pointers and size must be multiples of 16 bytes");
  TFHIP_CHECK_RANGE(src, bytes, 1, "src");
  TFHIP_CHECK_OUTPUT(dst, bytes, 1, "dst");
  note_kernel("copy_f4");
  TFHIP_LAUNCH((copy_f4<<<grid_for(bytes / 16), 256, 0, stream()>>>((const float4 *)src, (float4 *)dst,
                                                                      (long long)(bytes / 16))));
  return kOk;
}

}  // extern "C"
