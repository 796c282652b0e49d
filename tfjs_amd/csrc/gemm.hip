// _FusedMatMul / BatchMatMul entry point: validates the operands, picks the
// loaders the memory layout allows and a tile shape, and launches gemm_kernel.
#include "gemm_host.h"
#include "skinny_gemm.h"
#include "small_k_gemm.h"

using namespace tfhip;

int tfhip::launch_plain_gemm(GemmParams &p, bool transpose_a, bool transpose_b, bool vec) {
  if (skinny_applies(p, transpose_a, transpose_b, vec) && tuning(kTuneNoSkinny) <= 0) return launch_skinny(p);
  // (off unless asked for: back to back it beats the tiled kernel, but inside a network, where
  // its operands come from memory rather than from the cache a repeated launch leaves them in, it
  // loses more often than it wins)
  if (small_k_applies(p, transpose_a, transpose_b, vec) && tuning(kTuneSmallK) > 0) return launch_small_k(p);
  if (vec) {
    const int shape = choose_tile_shape(p.M, p.N, p.K, p.batch, num_cus());
    if (!transpose_a && !transpose_b) return launch_gemm_shape<kLoadKVec, kLoadXVec>(shape, p);
    if (!transpose_a && transpose_b) return launch_gemm_shape<kLoadKVec, kLoadKVec>(shape, p);
    if (transpose_a && !transpose_b) return launch_gemm_shape<kLoadXVec, kLoadXVec>(shape, p);
    return launch_gemm_shape<kLoadXVec, kLoadKVec>(shape, p);
  }
  return launch_gemm<64, 64, 16, 2, 2, kLoadScalar, kLoadScalar>(p);
}

extern "C" int tfhip_fused_matmul(const float *a, const float *b, float *out, int64_t batch_a, int64_t batch_b,
                                  int64_t M, int64_t N, int64_t K, int transpose_a, int transpose_b,
                                  const float *bias, const int64_t bias_strides[3], int activation,
                                  const float *prelu_weights, const int64_t prelu_strides[3],
                                  double leakyrelu_alpha) {
  TFHIP_REQUIRE_INIT();
  TFHIP_CHECK_ARG(batch_a >= 0 && batch_b >= 0 && M >= 0 && N >= 0 && K >= 0, "tfhip_fused_matmul: negative dimension");
  const int64_t lim = 0x7fffffff;
  TFHIP_CHECK_ARG(M < lim && N < lim && K < lim && batch_a < lim && batch_b < lim,
                  "tfhip_fused_matmul: dimension exceeds 2^31-1");
  const int64_t batch = batch_a > batch_b ? batch_a : batch_b;
  if (batch_a == 0 || batch_b == 0 || M == 0 || N == 0) return kOk;
  if (K > 0) {
    TFHIP_CHECK_RANGE(a, batch_a * M * K, 4, "a");
    TFHIP_CHECK_RANGE(b, batch_b * K * N, 4, "b");
  }
  TFHIP_CHECK_RANGE(out, batch * M * N, 4, "out");

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
  int rc = fill_epilogue(p.epi, "tfhip_fused_matmul", dims, 3, bias, bias_strides, activation, prelu_weights,
                         prelu_strides, leakyrelu_alpha, kMatmul);
  if (rc) return rc;

  const int64_t kMaxBufferBytes = 0xfffffffeLL;   // one buffer descriptor addresses at most this much
  p.a_bytes = (unsigned)(M * K * 4 <= kMaxBufferBytes ? M * K * 4 : 0);
  p.b_bytes = (unsigned)(K * N * 4 <= kMaxBufferBytes ? K * N * 4 : 0);
  p.vec_store = N % 4 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
  const bool a16 = reinterpret_cast<uintptr_t>(a) % 16 == 0 && p.a_bytes != 0,
             b16 = reinterpret_cast<uintptr_t>(b) % 16 == 0 && p.b_bytes != 0;
  // float4 loads need the contiguous extent (and with it every row start and
  // batch start) to be a multiple of four elements
  const bool a_vec = a16 && K > 0 && (transpose_a ? M % 4 == 0 : K % 4 == 0) && (M * K) % 4 == 0;
  const bool b_vec = b16 && K > 0 && (transpose_b ? K % 4 == 0 : N % 4 == 0) && (K * N) % 4 == 0;
  return launch_plain_gemm(p, transpose_a != 0, transpose_b != 0, a_vec && b_vec);
}
