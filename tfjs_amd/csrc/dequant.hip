// Weight dequantisation on load: uint8 / uint16 affine and float16 -> float32.
//
// Bandwidth-bound: 1 or 2 bytes in, 4 bytes out per weight. The aligned kernel
// reads 16 bytes of codes per lane and writes four (uint8) or two (uint16 /
// float16) float4s per lane, arranged so that every wavefront load and store
// instruction covers one contiguous 1 KB span. The byte-wise kernel takes
// quantized data at any byte offset, which is how tensors sit inside a weight
// shard (tfjs-core/src/io/io_utils.ts:137-158).
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

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// mode 0: affine -> float32, 1: affine -> int32, 2: float16 (two-byte codes only)
template <int MODE>
__device__ __forceinline__ float decode_one(unsigned code, double scale, double min) {
  if (MODE == 2) return __uint_as_float(half_bits_to_float_bits(code));
  if (MODE == 1) return __int_as_float(affine_i32(code, scale, min));
  return affine_f32(code, scale, min);
}

// The aligned kernel. A lane reads 16 bytes of codes (16 one-byte or 8 two-byte codes), so a
// wavefront's load instruction covers 1 KB in one piece. Written out directly, lane l's results
// would be the float4s 4l..4l+3 (2l, 2l+1), a 64-byte (32-byte) stride between lanes in every store
// instruction; instead the wavefront passes its 1 KB of codes through LDS and lane l decodes the
// float4s l, 64+l, 128+l, 192+l (l, 64+l) of the span, so every store instruction also covers 1 KB
// in one piece. The LDS span belongs to one wavefront, whose LDS instructions complete in order:
// no workgroup barrier, and a wavefront's lanes all run the same number of rounds. The results are
// read and written with streaming (non-temporal) loads and stores: nothing here touches either
// twice.
template <int BYTES_PER, int MODE>
__global__ __launch_bounds__(kThreads) void dequant_vec16(const u32x4 *__restrict__ q, f32x4 *__restrict__ out,
                                                          long long groups, double scale, double min) {
  __shared__ u32x4 stage[kThreads];
  const int lane = threadIdx.x & 63, wave_first = threadIdx.x & ~63;
  u32x4 *span = stage + wave_first;
  constexpr int kOutPerGroup = BYTES_PER == 1 ? 4 : 2;   // float4s decoded from one 16-byte group
  const long long out_count = groups * kOutPerGroup;
  const long long stride = (long long)gridDim.x * kThreads;
  for (long long base = (long long)blockIdx.x * kThreads + wave_first; base < groups; base += stride) {
    const long long g = base + lane;
    u32x4 w = {0u, 0u, 0u, 0u};
    if (g < groups) w = __builtin_nontemporal_load(q + g);
    span[lane] = w;
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int k = 0; k < kOutPerGroup; ++k) {
      const long long o = base * kOutPerGroup + k * 64 + lane;
      f32x4 r;
      if (BYTES_PER == 1) {
        const unsigned c = reinterpret_cast<const unsigned *>(span)[k * 64 + lane];
        r.x = decode_one<MODE>(c & 0xffu, scale, min);
        r.y = decode_one<MODE>((c >> 8) & 0xffu, scale, min);
        r.z = decode_one<MODE>((c >> 16) & 0xffu, scale, min);
        r.w = decode_one<MODE>(c >> 24, scale, min);
      } else {
        const u32x2 c = reinterpret_cast<const u32x2 *>(span)[k * 64 + lane];
        r.x = decode_one<MODE>(c.x & 0xffffu, scale, min);
        r.y = decode_one<MODE>(c.x >> 16, scale, min);
        r.z = decode_one<MODE>(c.y & 0xffffu, scale, min);
        r.w = decode_one<MODE>(c.y >> 16, scale, min);
      }
      if (o < out_count) __builtin_nontemporal_store(r, out + o);
    }
    __builtin_amdgcn_wave_barrier();
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

int grid_for(long long items, int blocks_per_cu) {
  long long blocks = (items + kThreads - 1) / kThreads;
  const long long cap = (long long)num_cus() * blocks_per_cu;
  if (blocks > cap) blocks = cap;
  return blocks < 1 ? 1 : (int)blocks;
}

template <int MODE>
int launch_bytes(const void *q, void *out, long long first, long long end, int bytes_per, double scale, double min) {
  TFHIP_LAUNCH((dequant_bytes<MODE><<<grid_for(end - first, 32), kThreads, 0, stream()>>>(
      (const unsigned char *)q, (unsigned *)out, first, end, bytes_per, scale, min)));
  return kOk;
}

int bytes_kernel(const void *q, void *out, long long first, long long end, int bytes_per, double scale, double min,
                  int mode) {
  if (first >= end) return kOk;
  if (mode == 2) return launch_bytes<2>(q, out, first, end, bytes_per, scale, min);
  if (mode == 1) return launch_bytes<1>(q, out, first, end, bytes_per, scale, min);
  return launch_bytes<0>(q, out, first, end, bytes_per, scale, min);
}

template <int BYTES_PER, int MODE>
int launch_vec16(const void *q, void *out, long long groups, double scale, double min) {
  // One round per lane: workgroups start in address order and drift apart, which spreads the
  // requests in flight over the memory channels. A grid capped at a few workgroups per compute unit,
  // every lane striding through the tensor in step with all others, measured 68% of the memory
  // bandwidth at 1.3 GB where this grid reaches 77%. (The loop in the kernel serves tensors beyond
  // 2^31 lanes.)
  const long long blocks = (groups + kThreads - 1) / kThreads;
  TFHIP_LAUNCH((dequant_vec16<BYTES_PER, MODE><<<(unsigned)(blocks > 0x3fffffLL ? 0x3fffffLL : blocks), kThreads, 0, stream()>>>(
      (const u32x4 *)q, (f32x4 *)out, groups, scale, min)));
  return kOk;
}

// mode: 0 affine f32, 1 affine i32, 2 float16.
// The 16-byte kernel takes the stretch of the tensor whose codes start on a 16-byte boundary and
// whose results do too; that needs the source on a 4-byte (one-byte codes) or 8-byte (two-byte
// codes) boundary and the output on a 16-byte one. Elements before and after that stretch, and
// tensors at any other alignment (they sit at arbitrary byte offsets inside a weight shard), go
// through the byte-wise kernel.
int launch(const void *q, int bytes_per, long long n, double scale, double min, void *out, int mode) {
  const uintptr_t qa = reinterpret_cast<uintptr_t>(q);
  const uintptr_t oa = reinterpret_cast<uintptr_t>(out);
  const int codes_per_group = 16 / bytes_per;
  long long head = 0, groups = 0;
  if (qa % (bytes_per == 1 ? 4 : 8) == 0 && oa % 16 == 0) {
    head = (long long)((16 - qa % 16) % 16) / bytes_per;   // a multiple of four elements
    if (head > n) head = n;
    groups = (n - head) / codes_per_group;
  }
  if (groups == 0) {
    note_kernel("dequant_bytes<%d>", mode);
    return bytes_kernel(q, out, 0, n, bytes_per, scale, min, mode);
  }
  note_kernel("dequant_vec16<%d, %d>", bytes_per, mode);
  int rc = bytes_kernel(q, out, 0, head, bytes_per, scale, min, mode);
  if (rc != kOk) return rc;
  const void *qv = (const unsigned char *)q + head * bytes_per;
  void *ov = (unsigned char *)out + head * 4;
  if (bytes_per == 1) {
    rc = mode == 1 ? launch_vec16<1, 1>(qv, ov, groups, scale, min) : launch_vec16<1, 0>(qv, ov, groups, scale, min);
  } else {
    rc = mode == 2 ? launch_vec16<2, 2>(qv, ov, groups, scale, min) :
         mode == 1 ? launch_vec16<2, 1>(qv, ov, groups, scale, min) : launch_vec16<2, 0>(qv, ov, groups, scale, min);
  }
  if (rc != kOk) return rc;
  return bytes_kernel(q, out, head + groups * codes_per_group, n, bytes_per, scale, min, mode);
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
  TFHIP_CHECK_OUTPUT(out, n, 4, "out");
  TFHIP_CHECK_ARG(reinterpret_cast<uintptr_t>(out) % 4 == 0, "tfhip_dequant_affine: out is not 4-byte aligned");
  return launch(q, bits / 8, n, scale, min, out, to_int32 ? 1 : 0);
}

int tfhip_dequant_f16(const void *q, int64_t n, float *out) {
  TFHIP_REQUIRE_INIT();
  TFHIP_CHECK_ARG(n >= 0, "tfhip_dequant_f16: negative element count");
  if (n == 0) return kOk;
  TFHIP_CHECK_RANGE(q, n, 2, "q");
  TFHIP_CHECK_OUTPUT(out, n, 4, "out");
  TFHIP_CHECK_ARG(reinterpret_cast<uintptr_t>(out) % 4 == 0, "tfhip_dequant_f16: out is not 4-byte aligned");
  return launch(q, 2, n, 0.0, 0.0, out, 2);
}

}  // extern "C"
