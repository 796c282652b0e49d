// _FusedMatMul / BatchMatMul entry point: validates the operands, picks the
// loaders the memory layout allows and a tile shape, and launches gemm_kernel.
#include "gemm_host.h"
#include "skinny_gemm.h"

using namespace tfhip;

int tfhip::launch_plain_gemm(GemmParams &p, bool transpose_a, bool transpose_b, bool vec) {
  if (skinny_applies(p, transpose_a, transpose_b, vec) && tuning(kTuneNoSkinny) <= 0) return launch_skinny(p);
  if (vec) {
    const int shape = choose_tile_shape(p.M, p.N, p.K, p.batch, num_cus());
    if (!transpose_a && !transpose_b) return launch_gemm_shape<kLoadKVec, kLoadXVec>(shape, p);
    if (!transpose_a && transpose_b) return launch_gemm_shape<kLoadKVec, kLoadKVec>(shape, p);
    if (transpose_a && !transpose_b) return launch_gemm_shape<kLoadXVec, kLoadXVec>(shape, p);
    return launch_gemm_shape<kLoadXVec, kLoadKVec>(shape, p);
  }
  return launch_gemm<64, 64, 16, 2, 2, kLoadScalar, kLoadScalar>(p);
}

namespace tfhip {
namespace {

// Scratch of tfhip_fused_matmul_noalloc: the split-K partial sums that
// tfhip_fused_matmul keeps in the library's growing workspace. Every GPU the
// library runs on holds its own copy of the array, at its own address, until
// the process ends; in host code the name below is only a stand-in for the
// symbol, and the per-device address is resolved once by setup_static_scratch
// (with that device current) and used from then on.
static __device__ __align__(256) float scratch[TFHIP_NOALLOC_SCRATCH_BYTES / sizeof(float)];

constexpr int kMaxDevices = 64;
float *g_scratch_ptr[kMaxDevices] = {};

}  // namespace

int setup_static_scratch(int device) {
  if (device < 0 || device >= kMaxDevices)
    return fail(kBadArgument, "tfhip_init: device %d is beyond the %d devices the static scratch table covers", device,
                kMaxDevices);
  if (g_scratch_ptr[device] != nullptr) return kOk;
  void *ptr = nullptr;
  const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
  if (e != hipSuccess || ptr == nullptr) {
    (void)hipGetLastError();
    return fail(kHipError, "tfhip_init: hipGetSymbolAddress(scratch) on device %d failed: %s", device,
                hipGetErrorString(e));
  }
  g_scratch_ptr[device] = static_cast<float *>(ptr);
  return kOk;
}

}  // namespace tfhip

static int fused_matmul_impl(const char *who, const float *a, const float *b, float *out, int64_t batch_a,
                             int64_t batch_b, int64_t M, int64_t N, int64_t K, int transpose_a, int transpose_b,
                             const float *bias, const int64_t bias_strides[3], int activation,
                             const float *prelu_weights, const int64_t prelu_strides[3], double leakyrelu_alpha);

extern "C" int tfhip_fused_matmul(const float *a, const float *b, float *out, int64_t batch_a, int64_t batch_b,
                                  int64_t M, int64_t N, int64_t K, int transpose_a, int transpose_b,
                                  const float *bias, const int64_t bias_strides[3], int activation,
                                  const float *prelu_weights, const int64_t prelu_strides[3],
                                  double leakyrelu_alpha) {
  return fused_matmul_impl("tfhip_fused_matmul", a, b, out, batch_a, batch_b, M, N, K, transpose_a, transpose_b, bias,
                           bias_strides, activation, prelu_weights, prelu_strides, leakyrelu_alpha);
}

extern "C" int tfhip_fused_matmul_noalloc(const float *a, const float *b, float *out, int64_t batch_a,
                                          int64_t batch_b, int64_t M, int64_t N, int64_t K, int transpose_a,
                                          int transpose_b, const float *bias, const int64_t bias_strides[3],
                                          int activation, const float *prelu_weights,
                                          const int64_t prelu_strides[3], double leakyrelu_alpha) {
  TFHIP_REQUIRE_INIT();
  float *ptr = g_scratch_ptr[device_index()];
  if (ptr == nullptr)
    return fail(kHipError, "tfhip_fused_matmul_noalloc: the static scratch array was not resolved on device %d",
                device_index());
  // Same kernels and the same choice of K slices as tfhip_fused_matmul; only the
  // home of the partial sums differs, so the two agree bit for bit. Nothing needs
  // clearing between calls: every slab element that gemm_finish reads was written
  // by this call's gemm_kernel.
  FixedWorkspace fixed(ptr, TFHIP_NOALLOC_SCRATCH_BYTES);
  return fused_matmul_impl("tfhip_fused_matmul_noalloc", a, b, out, batch_a, batch_b, M, N, K, transpose_a,
                           transpose_b, bias, bias_strides, activation, prelu_weights, prelu_strides,
                           leakyrelu_alpha);
}

static int fused_matmul_impl(const char *who, const float *a, const float *b, float *out, int64_t batch_a,
                             int64_t batch_b, int64_t M, int64_t N, int64_t K, int transpose_a, int transpose_b,
                             const float *bias, const int64_t bias_strides[3], int activation,
                             const float *prelu_weights, const int64_t prelu_strides[3], double leakyrelu_alpha) {
  TFHIP_REQUIRE_INIT();
  TFHIP_CHECK_ARG(batch_a >= 0 && batch_b >= 0 && M >= 0 && N >= 0 && K >= 0, "%s: negative dimension", who);
  const int64_t lim = 0x7fffffff;
  TFHIP_CHECK_ARG(M < lim && N < lim && K < lim && batch_a < lim && batch_b < lim,
                  "%s: dimension exceeds 2^31-1", who);
  const int64_t batch = batch_a > batch_b ? batch_a : batch_b;
  int rc = kOk;
  if (batch_a == 0 || batch_b == 0 || M == 0 || N == 0) return kOk;
  // three factors below 2^31 each can pass 2^63: bound every operand's element count before forming it
  const int64_t max_elems = int64_t(1) << 40;
  TFHIP_CHECK_ARG(product_below(max_elems, {batch_a, M, K > 0 ? K : 1}) && product_below(max_elems, {batch_b, K > 0 ? K : 1, N}) &&
                      product_below(max_elems, {batch, M, N}),
                  "%s: an operand exceeds 2^40 elements", who);
  auto live = [&](const void *ptr, int64_t elems, const char *name) {
    if (ptr != nullptr && range_is_live(ptr, (size_t)elems * 4)) return (int)kOk;
    return fail(kOutOfRange, "%s: operand '%s' (%lld elements of 4 bytes at %p) is not inside a live device buffer",
                who, name, (long long)elems, ptr);
  };
  if (K > 0) {
    if ((rc = live(a, batch_a * M * K, "a")) != kOk) return rc;
    if ((rc = live(b, batch_b * K * N, "b")) != kOk) return rc;
  }
  if ((rc = live(out, batch * M * N, "out")) != kOk) return rc;
  forget_filter_scans(out);

  GemmParams p = {};
  p.a = a; p.b = b; p.c = out;
  p.M = (int)M; p.N = (int)N; p.K = (int)K;
  p.batch = (int)batch; p.batch_a = (int)batch_a; p.batch_b = (int)batch_b;
  p.a_batch_stride = M * K; p.b_batch_stride = K * N; p.c_batch_stride = M * N;
  // strides folded as in tfjs-backend-cpu/src/kernels/BatchMatMul.ts:82-87
  p.a_sx = transpose_a ? 1 : K; p.a_sk = transpose_a ? M : 1;
  p.b_sx = transpose_b ? K : 1; p.b_sk = transpose_b ? 1 : N;
  p.ldc = N;
  const int64_t dims[3] = {batch, M, N};
  rc = fill_epilogue(p.epi, who, dims, 3, bias, bias_strides, activation, prelu_weights,
                         prelu_strides, leakyrelu_alpha, kMatmul);
  if (rc) return rc;

  const int64_t kMaxBufferBytes = 0xfffffffeLL;   // one buffer descriptor addresses at most this much
  p.a_bytes = (unsigned)(M * K * 4 <= kMaxBufferBytes ? M * K * 4 : 0);
  p.b_bytes = (unsigned)(K * N * 4 <= kMaxBufferBytes ? K * N * 4 : 0);
  p.c_bytes = (unsigned)(M * N * 4 <= kMaxBufferBytes ? M * N * 4 : 0);
  p.vec_store = N % 4 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
  const bool a16 = reinterpret_cast<uintptr_t>(a) % 16 == 0 && p.a_bytes != 0,
             b16 = reinterpret_cast<uintptr_t>(b) % 16 == 0 && p.b_bytes != 0;
  // float4 loads need the contiguous extent (and with it every row start and
  // batch start) to be a multiple of four elements
  const bool a_vec = a16 && K > 0 && (transpose_a ? M % 4 == 0 : K % 4 == 0) && (M * K) % 4 == 0;
  const bool b_vec = b16 && K > 0 && (transpose_b ? K % 4 == 0 : N % 4 == 0) && (K * N) % 4 == 0;
  return launch_plain_gemm(p, transpose_a != 0, transpose_b != 0, a_vec && b_vec);
}
