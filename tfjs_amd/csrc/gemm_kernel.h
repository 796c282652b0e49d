// Tiled float32 GEMM on the CDNA matrix cores, shared by _FusedMatMul,
// BatchMatMul and the implicit-GEMM FusedConv2D.
//
//   C[M x N] = A[M x K] * B[K x N], one workgroup of 256 threads (4 wavefronts
//   of 64) per BM x BN tile of C, K consumed in steps of BK.
//
// * Matrix core instruction: v_mfma_f32_16x16x4_f32 (64 lanes compute a 16x16
//   block over 4 values of k). Lane l feeds A[row l%16][k l/16] and
//   B[k l/16][col l%16] and receives C[rows 4*(l/16)..+3][col l%16].
// * Both operands are staged in LDS k-major ("[k][x]", x = row of A or column
//   of B), so the 16 lanes that share k read 16 consecutive words: no bank
//   conflicts whichever way the operand lies in global memory.
// * Global -> register -> LDS double buffering: while the matrix cores work on
//   LDS buffer t, the loads of tile t+1 are in flight into registers; they are
//   written to the other LDS buffer after the compute, one barrier per step.
// * Loaders (template parameter) decide how a tile is fetched:
//     kLoadKVec   operand is k-contiguous in memory (A row-major, or B given
//                 transposed): float4 loads along k, transposed into LDS
//     kLoadXVec   operand is x-contiguous (B row-major, or A given transposed):
//                 float4 loads along x, float4 LDS stores
//     kLoadScalar any strides, element loads with bounds checks
//     kLoadIm2colVec / kLoadIm2colScalar (A only): the rows of A are the
//                 receptive fields of an NHWC (or, scalar only, any-stride)
//                 image, gathered on the fly -- A is never materialised.
// * Workgroup ids are re-ordered so that the ids that land on one XCD (the
//   hardware deals consecutive ids round-robin over 8 XCDs, each with its own
//   L2) cover one contiguous band of tiles.
#pragma once

#include <hip/hip_runtime.h>

#include "epilogue.h"

namespace tfhip {

enum LoadKind { kLoadKVec = 0, kLoadXVec = 1, kLoadScalar = 2, kLoadIm2colVec = 3, kLoadIm2colScalar = 4 };

struct ConvGeom {
  // input addressing: x[n*xs_n + ih*xs_h + iw*xs_w + c*xs_c]
  long long xs_n, xs_h, xs_w, xs_c;
  int in_h, in_w, in_c;
  int f_w;            // k = (r * f_w + s) * in_c + c
  int stride_h, stride_w, dil_h, dil_w, pad_top, pad_left;
  int out_h, out_w;
};

struct GemmParams {
  const float *a;
  const float *b;
  float *c;
  int M, N, K;
  int batch, batch_a, batch_b;
  long long a_batch_stride, b_batch_stride, c_batch_stride;
  // element (i, k) of A at a[i*a_sx + k*a_sk]; element (k, j) of B at b[j*b_sx + k*b_sk]
  long long a_sx, a_sk, b_sx, b_sk;
  long long ldc;
  int tiles_m, tiles_n;
  ConvGeom conv;
  Epilogue epi;
};

typedef float float4_t __attribute__((ext_vector_type(4)));

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int A_KIND, int B_KIND>
struct GemmTile {
  static constexpr int kThreads = 256;
  static_assert(WAVES_M * WAVES_N == 4, "four wavefronts per workgroup");
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int TM = WM / 16, TN = WN / 16;
  static_assert(WM % 16 == 0 && WN % 16 == 0 && BK % 4 == 0, "tile shape");
  // Row pitch of the k-major LDS tiles: congruent to 16 modulo the 32 banks, so
  // the two k rows a half-wavefront reads never collide.
  static constexpr int LDA = BM % 32 == 0 ? BM + 16 : BM + 32;
  static constexpr int LDB = BN % 32 == 0 ? BN + 16 : BN + 32;
  // float4 fetches per thread per tile (the last round may be partly idle)
  static constexpr int A_VECS = (BM * BK / 4 + kThreads - 1) / kThreads;
  static constexpr int B_VECS = (BN * BK / 4 + kThreads - 1) / kThreads;
  static constexpr int LDS_FLOATS = 2 * BK * (LDA + LDB);
};

// Fetches this thread's share of a BX x BK operand tile into registers.
// `x0`/`k0` are the tile origin; the operand has X rows (M or N) and K columns.
template <int BX, int BK, int KIND, int VECS>
__device__ __forceinline__ void load_tile(float4 (&reg)[VECS], const float *__restrict__ base, long long sx,
                                          long long sk, int X, int K, int x0, int k0, int tid,
                                          const ConvGeom &g, const long long (&row_base)[VECS],
                                          const int (&row_ih)[VECS], const int (&row_iw)[VECS]) {
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (int i = 0; i < VECS; ++i) {
    const int f = tid + i * 256;
    if ((BX * BK / 4) % 256 != 0 && f >= BX * BK / 4) {
      reg[i] = zero;
      continue;
    }
    if (KIND == kLoadKVec) {
      // BK/4 float4 per row; K % 4 == 0 so a float4 is wholly inside or outside
      const int row = f / (BK / 4), kq = f % (BK / 4);
      const int x = x0 + row, k = k0 + kq * 4;
      reg[i] = (x < X && k < K) ? *reinterpret_cast<const float4 *>(base + (long long)x * sx + k) : zero;
    } else if (KIND == kLoadXVec) {
      // BX/4 float4 per k row; X % 4 == 0
      const int kr = f / (BX / 4), xq = f % (BX / 4);
      const int x = x0 + xq * 4, k = k0 + kr;
      reg[i] = (x < X && k < K) ? *reinterpret_cast<const float4 *>(base + (long long)k * sk + x) : zero;
    } else if (KIND == kLoadScalar) {
      // four elements along k (stride sk) of one row
      const int row = f / (BK / 4), kq = f % (BK / 4);
      const int x = x0 + row, k = k0 + kq * 4;
      float v[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = (x < X && k + j < K) ? base[(long long)x * sx + (long long)(k + j) * sk] : 0.f;
      reg[i] = make_float4(v[0], v[1], v[2], v[3]);
    } else if (KIND == kLoadIm2colVec) {
      // in_c % 4 == 0: the four k values share one filter tap (r, s)
      const int kq = f % (BK / 4);
      const int k = k0 + kq * 4;
      float4 v = zero;
      if (row_base[i] >= 0 && k < K) {
        const int tap = k / g.in_c, c = k - tap * g.in_c;
        const int r = tap / g.f_w, s = tap - r * g.f_w;
        const int ih = row_ih[i] + r * g.dil_h, iw = row_iw[i] + s * g.dil_w;
        if (ih >= 0 && ih < g.in_h && iw >= 0 && iw < g.in_w)
          v = *reinterpret_cast<const float4 *>(base + row_base[i] + ih * g.xs_h + iw * g.xs_w + c);
      }
      reg[i] = v;
    } else {  // kLoadIm2colScalar
      const int kq = f % (BK / 4);
      float v[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int k = k0 + kq * 4 + j;
        v[j] = 0.f;
        if (row_base[i] >= 0 && k < K) {
          const int tap = k / g.in_c, c = k - tap * g.in_c;
          const int r = tap / g.f_w, s = tap - r * g.f_w;
          const int ih = row_ih[i] + r * g.dil_h, iw = row_iw[i] + s * g.dil_w;
          if (ih >= 0 && ih < g.in_h && iw >= 0 && iw < g.in_w)
            v[j] = base[row_base[i] + ih * g.xs_h + iw * g.xs_w + c * g.xs_c];
        }
      }
      reg[i] = make_float4(v[0], v[1], v[2], v[3]);
    }
  }
}

// Writes the registers fetched by load_tile into a k-major LDS tile [BK][LD].
template <int BX, int BK, int LD, int KIND, int VECS>
__device__ __forceinline__ void store_tile(float *__restrict__ lds, const float4 (&reg)[VECS], int tid) {
#pragma unroll
  for (int i = 0; i < VECS; ++i) {
    const int f = tid + i * 256;
    if ((BX * BK / 4) % 256 != 0 && f >= BX * BK / 4) continue;
    if (KIND == kLoadXVec) {
      const int kr = f / (BX / 4), xq = f % (BX / 4);
      *reinterpret_cast<float4 *>(lds + kr * LD + xq * 4) = reg[i];
    } else {
      const int row = f / (BK / 4), kq = f % (BK / 4);
      float *d = lds + (kq * 4) * LD + row;
      d[0] = reg[i].x;
      d[LD] = reg[i].y;
      d[2 * LD] = reg[i].z;
      d[3 * LD] = reg[i].w;
    }
  }
}

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int A_KIND, int B_KIND>
__global__ __launch_bounds__(256) void gemm_kernel(GemmParams p) {
  using T = GemmTile<BM, BN, BK, WAVES_M, WAVES_N, A_KIND, B_KIND>;
  extern __shared__ float lds[];
  float *lds_a = lds;                      // [2][BK][LDA]
  float *lds_b = lds + 2 * BK * T::LDA;    // [2][BK][LDB]

  // Workgroup id -> (batch, tile_m, tile_n). Ids i, i+8, i+16, ... share an XCD;
  // give each XCD one contiguous band of the tile sequence.
  const int total = gridDim.x;
  int id = blockIdx.x;
  {
    const int per_xcd = total / 8;
    if (per_xcd > 0 && id < per_xcd * 8) id = (id % 8) * per_xcd + id / 8;
  }
  const int tiles_per_batch = p.tiles_m * p.tiles_n;
  const int bz = id / tiles_per_batch;
  const int t = id - bz * tiles_per_batch;
  const int tile_m = t / p.tiles_n, tile_n = t - tile_m * p.tiles_n;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const float *A = p.a + (long long)(bz % p.batch_a) * p.a_batch_stride;
  const float *B = p.b + (long long)(bz % p.batch_b) * p.b_batch_stride;
  float *C = p.c + (long long)bz * p.c_batch_stride;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave / WAVES_N) * T::WM, wn0 = (wave % WAVES_N) * T::WN;

  // im2col: the output pixel behind each A row this thread fetches is fixed
  // across k, so split it once. row_base < 0 marks a row beyond M.
  long long row_base[T::A_VECS];
  int row_ih[T::A_VECS], row_iw[T::A_VECS];
  if (A_KIND == kLoadIm2colVec || A_KIND == kLoadIm2colScalar) {
#pragma unroll
    for (int i = 0; i < T::A_VECS; ++i) {
      const int row = (tid + i * 256) / (BK / 4);
      const int m = m0 + row;
      if (row < BM && m < p.M) {
        const int ow = m % p.conv.out_w;
        const int t2 = m / p.conv.out_w;
        const int oh = t2 % p.conv.out_h, n = t2 / p.conv.out_h;
        row_base[i] = (long long)n * p.conv.xs_n;
        row_ih[i] = oh * p.conv.stride_h - p.conv.pad_top;
        row_iw[i] = ow * p.conv.stride_w - p.conv.pad_left;
      } else {
        row_base[i] = -1;
        row_ih[i] = row_iw[i] = 0;
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < T::A_VECS; ++i) {
      row_base[i] = 0;
      row_ih[i] = row_iw[i] = 0;
    }
  }
  const long long no_base[T::B_VECS] = {};
  const int no_pos[T::B_VECS] = {};

  float4_t acc[T::TM][T::TN];
#pragma unroll
  for (int i = 0; i < T::TM; ++i)
#pragma unroll
    for (int j = 0; j < T::TN; ++j) acc[i][j] = (float4_t){0.f, 0.f, 0.f, 0.f};

  float4 ra[T::A_VECS], rb[T::B_VECS];
  const int k_tiles = (p.K + BK - 1) / BK;

  load_tile<BM, BK, A_KIND, T::A_VECS>(ra, A, p.a_sx, p.a_sk, p.M, p.K, m0, 0, tid, p.conv, row_base, row_ih, row_iw);
  load_tile<BN, BK, B_KIND, T::B_VECS>(rb, B, p.b_sx, p.b_sk, p.N, p.K, n0, 0, tid, p.conv, no_base, no_pos, no_pos);
  store_tile<BM, BK, T::LDA, A_KIND, T::A_VECS>(lds_a, ra, tid);
  store_tile<BN, BK, T::LDB, B_KIND, T::B_VECS>(lds_b, rb, tid);
  __syncthreads();

  for (int kt = 0; kt < k_tiles; ++kt) {
    const int cur = kt & 1;
    const bool more = kt + 1 < k_tiles;
    if (more) {
      load_tile<BM, BK, A_KIND, T::A_VECS>(ra, A, p.a_sx, p.a_sk, p.M, p.K, m0, (kt + 1) * BK, tid, p.conv, row_base, row_ih, row_iw);
      load_tile<BN, BK, B_KIND, T::B_VECS>(rb, B, p.b_sx, p.b_sk, p.N, p.K, n0, (kt + 1) * BK, tid, p.conv, no_base, no_pos, no_pos);
    }
    const float *ta = lds_a + cur * BK * T::LDA + (lane >> 4) * T::LDA + wm0 + (lane & 15);
    const float *tb = lds_b + cur * BK * T::LDB + (lane >> 4) * T::LDB + wn0 + (lane & 15);
#pragma unroll
    for (int kk = 0; kk < BK; kk += 4) {
      float fa[T::TM], fb[T::TN];
#pragma unroll
      for (int i = 0; i < T::TM; ++i) fa[i] = ta[kk * T::LDA + i * 16];
#pragma unroll
      for (int j = 0; j < T::TN; ++j) fb[j] = tb[kk * T::LDB + j * 16];
#pragma unroll
      for (int i = 0; i < T::TM; ++i)
#pragma unroll
        for (int j = 0; j < T::TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    if (more) {
      store_tile<BM, BK, T::LDA, A_KIND, T::A_VECS>(lds_a + (cur ^ 1) * BK * T::LDA, ra, tid);
      store_tile<BN, BK, T::LDB, B_KIND, T::B_VECS>(lds_b + (cur ^ 1) * BK * T::LDB, rb, tid);
    }
    __syncthreads();
  }

  // Epilogue: lane l holds rows 4*(l/16)..+3 of column l%16 of each 16x16 block.
  const Epilogue &e = p.epi;
#pragma unroll
  for (int i = 0; i < T::TM; ++i) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = m0 + wm0 + i * 16 + (lane >> 4) * 4 + r;
      if (row >= p.M) continue;
      long long n = 0, oh = 0, ow = 0;
      long long out_row;
      if (e.addressing == kConv) {
        ow = row % e.out_w;
        const int t2 = row / e.out_w;
        oh = t2 % e.out_h;
        n = t2 / e.out_h;
        out_row = n * e.y_s[0] + oh * e.y_s[1] + ow * e.y_s[2];
      } else {
        out_row = (long long)row * p.ldc;
      }
#pragma unroll
      for (int j = 0; j < T::TN; ++j) {
        const int col = n0 + wn0 + j * 16 + (lane & 15);
        if (col >= p.N) continue;
        const float v = finish(e, acc[i][j][r], bz, row, col, n, oh, ow);
        const long long off = (e.addressing == kConv) ? out_row + col * e.y_s[3] : out_row + col;
        C[off] = v;
      }
    }
  }
}

}  // namespace tfhip
