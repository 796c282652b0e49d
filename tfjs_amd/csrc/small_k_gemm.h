// GEMM for a very short contraction: C[M x N] = A[M x K] * B[K x N] with K <= 64
// (the first expansion convolutions of a mobile network: K = 32, 64, N = 6 K).
//
// With one to four k tiles the pipelined kernel of gemm_kernel.h is all prologue
// and epilogue (measured with launches back to back: 6-10% slower than this kernel
// at K = 32 and 64; from K = 96 on its overlap of fetches and matrix instructions
// wins, by 12-30%). Inside a network the picture turns: operands then come from
// memory, not from the cache a repeated launch leaves them in, and waiting for one
// long round trip before the first matrix instruction costs more than the tiled
// kernel's staggered fetches (seven MobileNetV2 layers, in sequence: 99.7 us with
// this kernel, 88.7 us with the tiled one). So it is only used when the "small_k"
// knob asks for it.
// Here a workgroup fetches ALL of its A rows and B columns at once (every load
// of the tile in flight together: one memory round trip), stores them to LDS
// in the x-major layout of gemm_kernel.h (row pitch k_pad + 8 floats, B transposed
// on the way), passes ONE barrier and then issues its matrix instructions back to
// back from LDS: one 16-byte fragment read per operand block feeds four MFMAs, as
// there. The accumulators start from the bias; activation and float4 stores happen
// in registers (operands passed swapped, a lane holds four consecutive columns).
//
// Row-major A and B with 16-byte aligned rows, per-column bias, linear / relu /
// relu6 / leakyrelu; anything else takes gemm_kernel.h.
#pragma once

#include <hip/hip_runtime.h>

#include "common.h"
#include "gemm_kernel.h"

namespace tfhip {

struct SmallKArgs {
  const float *a, *b, *bias;
  float *c;
  long long bias_stride;
  double leaky_alpha;
  long long a_batch_stride, b_batch_stride, c_batch_stride;
  int M, N, K, k_pad;   // k_pad: K rounded up to 16
  int batch_a, batch_b;
  int tiles_n;
  unsigned a_bytes, b_bytes;
  int activation;
};

// KQ_MAX: float4 per row of A the instantiation can hold (k_pad <= 4 * KQ_MAX).
template <int BM, int WAVES_M, int WAVES_N, int KQ_MAX>
__global__ __launch_bounds__(256) void small_k_gemm(SmallKArgs g) {
  constexpr int BN = 64;
  static_assert(WAVES_M * WAVES_N == 4 && KQ_MAX % 16 == 0, "four wavefronts; k in steps of 64");
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int TM = WM / 16, TN = WN / 16;
  constexpr int A_ROW_PASSES = BM / 16, A_K_PASSES = KQ_MAX / 16;
  constexpr int B_K_PASSES = KQ_MAX / 4;   // 16 k per pass
  extern __shared__ float lds[];
  const int pitch = g.k_pad + 8;
  float *lds_a = lds;                 // [BM][pitch]
  float *lds_b = lds + BM * pitch;    // [BN][pitch]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;
  const int tm = blockIdx.x / g.tiles_n, tn = blockIdx.x - tm * g.tiles_n;
  const int bz = blockIdx.y;
  const int m0 = tm * BM, n0 = tn * BN;
  const float *A = uniform_pointer(g.a + (long long)(bz % g.batch_a) * g.a_batch_stride);
  const float *B = uniform_pointer(g.b + (long long)(bz % g.batch_b) * g.b_batch_stride);
  const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc((void *)A, 0, (int)g.a_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc((void *)B, 0, (int)g.b_bytes, 0x00020000);

  // ---- every load of the tile, unconditionally (out of range: offset the descriptor does not cover, reads zero)
  // A: 16 lanes along k (one float4 each), 16 rows per pass
  float4 ra[A_ROW_PASSES][A_K_PASSES];
  const int a_row = tid >> 4, a_kq = tid & 15;
#pragma unroll
  for (int ri = 0; ri < A_ROW_PASSES; ++ri) {
    const int row = m0 + a_row + 16 * ri;
#pragma unroll
    for (int ki = 0; ki < A_K_PASSES; ++ki) {
      const int k = (a_kq + 16 * ki) * 4;
      const unsigned off = (row < g.M && k < g.K) ? (unsigned)(((long long)row * g.K + k) * 4) : kNoOffset;
      ra[ri][ki] = as_float4(__builtin_amdgcn_raw_buffer_load_b128(rsrc_a, (int)off, 0, 0));
    }
  }
  // B: 16 lanes along k (consecutive LDS banks when transposed), 16 float4 column groups
  float4 rb[B_K_PASSES];
  const int b_k = tid & 15, b_nq = tid >> 4;
  const int b_col = n0 + 4 * b_nq;
#pragma unroll
  for (int i = 0; i < B_K_PASSES; ++i) {
    const int k = b_k + 16 * i;
    const unsigned off = (k < g.K && b_col < g.N) ? (unsigned)(((long long)k * g.N + b_col) * 4) : kNoOffset;
    rb[i] = as_float4(__builtin_amdgcn_raw_buffer_load_b128(rsrc_b, (int)off, 0, 0));
  }
  // the accumulators start from the bias of the lane's four columns per block
  float4_t acc[TM][TN];
  {
    const int lane_col = n0 + wn0 + (lane >> 4) * 4;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      float4_t b4 = {0.f, 0.f, 0.f, 0.f};
      if (g.bias) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int col = lane_col + j * 16 + q;
          b4[q] = g.bias[(long long)(col < g.N ? col : g.N - 1) * g.bias_stride];
        }
      }
#pragma unroll
      for (int i = 0; i < TM; ++i) acc[i][j] = b4;
    }
  }

  // ---- registers -> LDS
#pragma unroll
  for (int ri = 0; ri < A_ROW_PASSES; ++ri)
#pragma unroll
    for (int ki = 0; ki < A_K_PASSES; ++ki) {
      const int k = (a_kq + 16 * ki) * 4;
      if (k < g.k_pad) *reinterpret_cast<float4 *>(lds_a + (a_row + 16 * ri) * pitch + k) = ra[ri][ki];
    }
#pragma unroll
  for (int i = 0; i < B_K_PASSES; ++i) {
    const int k = b_k + 16 * i;
    if (k < g.k_pad) {
      float *d = lds_b + (4 * b_nq) * pitch + k;
      d[0] = rb[i].x;
      d[pitch] = rb[i].y;
      d[2 * pitch] = rb[i].z;
      d[3 * pitch] = rb[i].w;
    }
  }
  __syncthreads();

  // ---- matrix instructions straight from LDS: lane (g4, r) reads k = 16 q + 4 g4 .. +3 of row r of each block
  const float *a_lane = lds_a + (wm0 + (lane & 15)) * pitch + (lane >> 4) * 4;
  const float *b_lane = lds_b + (wn0 + (lane & 15)) * pitch + (lane >> 4) * 4;
  const int quads = g.k_pad / 16;
  float4 fa[TM], fb[TN], na[TM], nb[TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) fa[i] = *reinterpret_cast<const float4 *>(a_lane + i * 16 * pitch);
#pragma unroll
  for (int j = 0; j < TN; ++j) fb[j] = *reinterpret_cast<const float4 *>(b_lane + j * 16 * pitch);
  for (int q = 0; q < quads; ++q) {
    const int nq = q + 1 < quads ? q + 1 : q;   // the last step re-reads its own fragments instead of branching
#pragma unroll
    for (int i = 0; i < TM; ++i) na[i] = *reinterpret_cast<const float4 *>(a_lane + i * 16 * pitch + nq * 16);
#pragma unroll
    for (int j = 0; j < TN; ++j) nb[j] = *reinterpret_cast<const float4 *>(b_lane + j * 16 * pitch + nq * 16);
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(quad_element(fb[j], s), quad_element(fa[i], s), acc[i][j],
                                                           0, 0, 0);
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[i] = na[i];
#pragma unroll
    for (int j = 0; j < TN; ++j) fb[j] = nb[j];
  }

  // ---- epilogue: lane l of a 16x16 block holds row l % 16, columns 4 * (l / 16) .. +3
  float *C = g.c + (long long)bz * g.c_batch_stride;
  const int lane_m = lane & 15, lane_n = (lane >> 4) * 4;
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int row = m0 + wm0 + i * 16 + lane_m;
    if (row >= g.M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = n0 + wn0 + j * 16 + lane_n;
      if (col >= g.N) continue;
      float out[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float v = acc[i][j][q];
        switch (g.activation) {
          case TFHIP_RELU: v = (v > 0.f || v != v) ? v : 0.f; break;
          case TFHIP_RELU6: v = (v > 0.f || v != v) ? v : 0.f; v = v > 6.f ? 6.f : v; break;
          case TFHIP_LEAKYRELU: v = v < 0.f ? (float)(g.leaky_alpha * (double)v) : v; break;
          default: break;
        }
        out[q] = v;
      }
      store_result4(C + (long long)row * g.N + col, make_float4(out[0], out[1], out[2], out[3]));
    }
  }
}

// True when the product fits this kernel.
inline bool small_k_applies(const GemmParams &p, bool transpose_a, bool transpose_b, bool vec) {
  if (transpose_a || transpose_b || !vec) return false;
  if (p.K < 4 || p.K > 64 || p.K % 4 != 0 || p.N % 4 != 0 || !p.vec_store || p.ldc != p.N) return false;
  if (!p.epi.channel_operands || p.epi.activation > TFHIP_LEAKYRELU || p.epi.activation == TFHIP_PRELU) return false;
  if (p.a_bytes == 0 || p.b_bytes == 0 || p.batch > 65535 || p.epi.residual) return false;
  // one round trip only pays while the k loop it replaces is short against its own set-up
  return (long long)p.M * p.batch >= 512 && p.N >= 64;
}

template <int BM, int WAVES_M, int WAVES_N, int KQ_MAX>
inline int launch_small_k_tile(SmallKArgs &g, int batch) {
  const int tiles_m = (g.M + BM - 1) / BM;
  g.tiles_n = (g.N + 63) / 64;
  const size_t lds = (size_t)(BM + 64) * (g.k_pad + 8) * sizeof(float);
  note_kernel("small_k_gemm<%d, %d, %d, %d>", BM, WAVES_M, WAVES_N, KQ_MAX);
  TFHIP_LAUNCH((small_k_gemm<BM, WAVES_M, WAVES_N, KQ_MAX>
                <<<dim3((unsigned)(tiles_m * g.tiles_n), (unsigned)batch), dim3(256), lds, stream()>>>(g)));
  return kOk;
}

inline int launch_small_k(const GemmParams &p) {
  SmallKArgs g;
  g.a = p.a; g.b = p.b; g.c = p.c;
  g.bias = p.epi.bias; g.bias_stride = p.epi.bias ? p.epi.bias_s[3] : 0;
  g.leaky_alpha = p.epi.leaky_alpha;
  g.a_batch_stride = p.a_batch_stride; g.b_batch_stride = p.b_batch_stride; g.c_batch_stride = p.c_batch_stride;
  g.M = p.M; g.N = p.N; g.K = p.K;
  g.k_pad = (p.K + 15) / 16 * 16;   // <= 64 = 4 * KQ_MAX of the instantiations below
  g.batch_a = p.batch_a; g.batch_b = p.batch_b;
  g.a_bytes = p.a_bytes; g.b_bytes = p.b_bytes;
  g.activation = p.epi.activation;
  // 64-row tiles when they still make four workgroups per compute unit, else 32-row tiles
  const long long tiles64 = (long long)((p.M + 63) / 64) * ((p.N + 63) / 64) * p.batch;
  const int forced = tuning(kTuneSmallK);
  const bool rows64 = forced == 64 ? true : (forced == 32 ? false : tiles64 >= 4LL * num_cus());
  if (rows64) return launch_small_k_tile<64, 2, 2, 16>(g, p.batch);
  return launch_small_k_tile<32, 2, 2, 16>(g, p.batch);
}

}  // namespace tfhip
