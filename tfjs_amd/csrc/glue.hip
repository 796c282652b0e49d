// The few non-contraction kernels a MobileNetV2 graph needs between the fused
// ops, so that no tensor leaves the device mid-graph: the residual Add and the
// global average pool (Mean over H and W).
#include "common.h"

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

__global__ __launch_bounds__(256) void add_same_shape(const float4 *__restrict__ a, const float4 *__restrict__ b,
                                                      float4 *__restrict__ out, long long groups) {
  const long long stride = (long long)gridDim.x * 256;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < groups; i += stride) {
    const float4 u = a[i], v = b[i];
    out[i] = make_float4(u.x + v.x, u.y + v.y, u.z + v.z, u.w + v.w);
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

int grid_for(long long items) {
  long long blocks = (items + 255) / 256;
  const long long cap = (long long)num_cus() * 32;
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
  TFHIP_CHECK_RANGE(y, rows * cols, 4, "y");
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
  TFHIP_CHECK_RANGE(out, total, 4, "out");
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

int tfhip_mean_hw(const float *x, float *y, int64_t batch, int64_t h, int64_t w, int64_t c) {
  TFHIP_REQUIRE_INIT();
  TFHIP_CHECK_ARG(batch >= 0 && h > 0 && w > 0 && c >= 0, "tfhip_mean_hw: bad dimensions");
  if (batch * c == 0) return kOk;
  TFHIP_CHECK_RANGE(x, batch * h * w * c, 4, "x");
  TFHIP_CHECK_RANGE(y, batch * c, 4, "y");
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
  TFHIP_CHECK_RANGE(dst, bytes, 1, "dst");
  note_kernel("copy_f4");
  TFHIP_LAUNCH((copy_f4<<<grid_for(bytes / 16), 256, 0, stream()>>>((const float4 *)src, (float4 *)dst,
                                                                      (long long)(bytes / 16))));
  return kOk;
}

}  // extern "C"
