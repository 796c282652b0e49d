// Weight dequantisation on load: uint8 / uint16 affine and float16 -> float32.
//
// Bandwidth-bound: 1 or 2 bytes in, 4 bytes out per weight. The aligned kernels
// read one 32-bit (uint8) or 64-bit (uint16 / float16) word per lane and write
// one float4 per lane, so every wavefront load and store instruction covers one
// contiguous, fully used span. The byte-wise kernels take quantized data at any
// byte offset, which is how tensors sit inside a weight shard
// (tfjs-core/src/io/io_utils.ts:137-158).
//
// Arithmetic follows the reference's JavaScript exactly
// (tfjs-core/src/io/io_utils.ts:223-227): integer -> double, one double
// multiply, one double add (never fused), one round-to-nearest-even to float32.
#include "common.h"

namespace tfhip {
namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ float affine_f32(unsigned v, double scale, double min) {
  return __double2float_rn(__dadd_rn(__dmul_rn((double)v, scale), min));
}

// Math.round (ties toward +infinity) followed by the Int32Array store's ToInt32
// (io_utils.ts:243-247).
__device__ __forceinline__ int affine_i32(unsigned v, double scale, double min) {
  const double x = __dadd_rn(__dmul_rn((double)v, scale), min);
  if (x != x || isinf(x)) return 0;
  const double f = floor(x);
  const double r = (x - f >= 0.5) ? f + 1.0 : f;
  if (fabs(r) < 9.0e15) {
    return (int)(unsigned)(unsigned long long)(long long)r;
  }
  double m = fmod(r, 4294967296.0);
  if (m < 0) m += 4294967296.0;
  return (int)(unsigned)(unsigned long long)m;
}

// float16 bit pattern -> float32 bit pattern, the value the reference's three
// lookup tables produce (io_utils.ts:645-741): exact for normals, subnormals,
// zeros and infinities; a NaN keeps its payload (m << 13) and its quiet bit is
// not forced.
__device__ __forceinline__ unsigned half_bits_to_float_bits(unsigned h) {
  const unsigned sign = (h & 0x8000u) << 16;
  const unsigned exp = (h >> 10) & 0x1fu;
  const unsigned man = h & 0x3ffu;
  if (exp == 0) {
    if (man == 0) return sign;
    // subnormal: value = man * 2^-24, normalise
    const int shift = __clz(man) - 21;  // leading zeros above bit 10
    const unsigned m = (man << shift) & 0x3ffu;
    return sign | ((unsigned)(113 - shift) << 23) | (m << 13);
  }
  if (exp == 31) return sign | 0x7f800000u | (man << 13);
  return sign | ((exp + 112u) << 23) | (man << 13);
}

template <bool TO_INT>
__global__ __launch_bounds__(kThreads) void dequant_u8_vec(const unsigned *__restrict__ q,
                                                           float4 *__restrict__ out, long long groups,
                                                           double scale, double min) {
  const long long stride = (long long)gridDim.x * kThreads;
  for (long long g = (long long)blockIdx.x * kThreads + threadIdx.x; g < groups; g += stride) {
    const unsigned w = q[g];
    float4 r;
    if (TO_INT) {
      r.x = __int_as_float(affine_i32(w & 0xffu, scale, min));
      r.y = __int_as_float(affine_i32((w >> 8) & 0xffu, scale, min));
      r.z = __int_as_float(affine_i32((w >> 16) & 0xffu, scale, min));
      r.w = __int_as_float(affine_i32(w >> 24, scale, min));
    } else {
      r.x = affine_f32(w & 0xffu, scale, min);
      r.y = affine_f32((w >> 8) & 0xffu, scale, min);
      r.z = affine_f32((w >> 16) & 0xffu, scale, min);
      r.w = affine_f32(w >> 24, scale, min);
    }
    out[g] = r;
  }
}

// MODE 0: uint16 affine -> float32, 1: uint16 affine -> int32, 2: float16.
template <int MODE>
__global__ __launch_bounds__(kThreads) void dequant_u16_vec(const uint2 *__restrict__ q,
                                                            float4 *__restrict__ out, long long groups,
                                                            double scale, double min) {
  const long long stride = (long long)gridDim.x * kThreads;
  for (long long g = (long long)blockIdx.x * kThreads + threadIdx.x; g < groups; g += stride) {
    const uint2 w = q[g];
    const unsigned c0 = w.x & 0xffffu, c1 = w.x >> 16, c2 = w.y & 0xffffu, c3 = w.y >> 16;
    float4 r;
    if (MODE == 2) {
      r.x = __uint_as_float(half_bits_to_float_bits(c0));
      r.y = __uint_as_float(half_bits_to_float_bits(c1));
      r.z = __uint_as_float(half_bits_to_float_bits(c2));
      r.w = __uint_as_float(half_bits_to_float_bits(c3));
    } else if (MODE == 1) {
      r.x = __int_as_float(affine_i32(c0, scale, min));
      r.y = __int_as_float(affine_i32(c1, scale, min));
      r.z = __int_as_float(affine_i32(c2, scale, min));
      r.w = __int_as_float(affine_i32(c3, scale, min));
    } else {
      r.x = affine_f32(c0, scale, min);
      r.y = affine_f32(c1, scale, min);
      r.z = affine_f32(c2, scale, min);
      r.w = affine_f32(c3, scale, min);
    }
    out[g] = r;
  }
}

// One element per lane, source read byte by byte: any source alignment, and the
// tail of the aligned kernels. MODE 0: affine f32, 1: affine i32, 2: float16.
template <int MODE>
__global__ __launch_bounds__(kThreads) void dequant_bytes(const unsigned char *__restrict__ q,
                                                          unsigned *__restrict__ out, long long first,
                                                          long long n, int bytes_per, double scale,
                                                          double min) {
  const long long stride = (long long)gridDim.x * kThreads;
  for (long long i = first + (long long)blockIdx.x * kThreads + threadIdx.x; i < n; i += stride) {
    unsigned v = q[i * bytes_per];
    if (bytes_per == 2) v |= (unsigned)q[i * 2 + 1] << 8;
    unsigned r;
    if (MODE == 2) {
      r = half_bits_to_float_bits(v);
    } else if (MODE == 1) {
      r = (unsigned)affine_i32(v, scale, min);
    } else {
      r = __float_as_uint(affine_f32(v, scale, min));
    }
    out[i] = r;
  }
}

int grid_for(long long items) {
  long long blocks = (items + kThreads - 1) / kThreads;
  const long long cap = (long long)num_cus() * 32;
  if (blocks > cap) blocks = cap;
  return blocks < 1 ? 1 : (int)blocks;
}

// mode: 0 affine f32, 1 affine i32, 2 float16
int launch(const void *q, int bytes_per, long long n, double scale, double min, void *out, int mode) {
  const uintptr_t qa = reinterpret_cast<uintptr_t>(q);
  const uintptr_t oa = reinterpret_cast<uintptr_t>(out);
  const bool aligned = (qa % (bytes_per == 1 ? 4 : 8) == 0) && (oa % 16 == 0);
  long long groups = aligned ? n / 4 : 0;
  hipStream_t s = stream();
  if (groups > 0) {
    note_kernel(bytes_per == 1 ? "dequant_u8_vec" : "dequant_u16_vec");
    const int grid = grid_for(groups);
    if (bytes_per == 1) {
      if (mode == 1)
        TFHIP_LAUNCH((dequant_u8_vec<true><<<grid, kThreads, 0, s>>>((const unsigned *)q, (float4 *)out, groups, scale, min)));
      else
        TFHIP_LAUNCH((dequant_u8_vec<false><<<grid, kThreads, 0, s>>>((const unsigned *)q, (float4 *)out, groups, scale, min)));
    } else {
      if (mode == 2)
        TFHIP_LAUNCH((dequant_u16_vec<2><<<grid, kThreads, 0, s>>>((const uint2 *)q, (float4 *)out, groups, scale, min)));
      else if (mode == 1)
        TFHIP_LAUNCH((dequant_u16_vec<1><<<grid, kThreads, 0, s>>>((const uint2 *)q, (float4 *)out, groups, scale, min)));
      else
        TFHIP_LAUNCH((dequant_u16_vec<0><<<grid, kThreads, 0, s>>>((const uint2 *)q, (float4 *)out, groups, scale, min)));
    }
  }
  const long long first = groups * 4;
  if (first < n) {
    if (groups == 0) note_kernel("dequant_bytes");
    const int grid = grid_for(n - first);
    if (mode == 2)
        TFHIP_LAUNCH((dequant_bytes<2><<<grid, kThreads, 0, s>>>((const unsigned char *)q, (unsigned *)out, first, n, bytes_per, scale, min)));
    else if (mode == 1)
        TFHIP_LAUNCH((dequant_bytes<1><<<grid, kThreads, 0, s>>>((const unsigned char *)q, (unsigned *)out, first, n, bytes_per, scale, min)));
    else
        TFHIP_LAUNCH((dequant_bytes<0><<<grid, kThreads, 0, s>>>((const unsigned char *)q, (unsigned *)out, first, n, bytes_per, scale, min)));
  }
  return kOk;
}

}  // namespace
}  // namespace tfhip

using namespace tfhip;

extern "C" {

int tfhip_dequant_affine(const void *q, int bits, int64_t n, double scale, double min, void *out,
                         int to_int32) {
  TFHIP_REQUIRE_INIT();
  TFHIP_CHECK_ARG(bits == 8 || bits == 16, "tfhip_dequant_affine: bits must be 8 or 16, got %d", bits);
  TFHIP_CHECK_ARG(n >= 0, "tfhip_dequant_affine: negative element count");
  if (n == 0) return kOk;
  TFHIP_CHECK_RANGE(q, n, bits / 8, "q");
  TFHIP_CHECK_RANGE(out, n, 4, "out");
  TFHIP_CHECK_ARG(reinterpret_cast<uintptr_t>(out) % 4 == 0, "tfhip_dequant_affine: out is not 4-byte aligned");
  return launch(q, bits / 8, n, scale, min, out, to_int32 ? 1 : 0);
}

int tfhip_dequant_f16(const void *q, int64_t n, float *out) {
  TFHIP_REQUIRE_INIT();
  TFHIP_CHECK_ARG(n >= 0, "tfhip_dequant_f16: negative element count");
  if (n == 0) return kOk;
  TFHIP_CHECK_RANGE(q, n, 2, "q");
  TFHIP_CHECK_RANGE(out, n, 4, "out");
  TFHIP_CHECK_ARG(reinterpret_cast<uintptr_t>(out) % 4 == 0, "tfhip_dequant_f16: out is not 4-byte aligned");
  return launch(q, 2, n, 0.0, 0.0, out, 2);
}

}  // extern "C"
