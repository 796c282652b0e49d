// Tiled float32 GEMM on the CDNA matrix cores, shared by _FusedMatMul,
// BatchMatMul and the implicit-GEMM FusedConv2D.
//
//   C[M x N] = A[M x K] * B[K x N], one workgroup of 256 threads (4 wavefronts
//   of 64) per BM x BN tile of C, K consumed in steps of BK.
//
// * Matrix core instruction: v_mfma_f32_16x16x4_f32 (64 lanes compute a 16x16
//   block over 4 values of k). Lane l feeds A[row l%16][k l/16] and
//   B[k l/16][col l%16] and receives C[rows 4*(l/16)..+3][col l%16].
// * Both operands are staged in LDS x-major ("[x][k]", x = row of A or column
//   of B, k contiguous, row pitch BK + 8 floats). The matrix instruction only
//   needs the two operands of a lane to belong to the same k, not any particular
//   k, so lane (g, r) (g = lane / 16, r = lane % 16) takes k = 16T + 4g + j for
//   the j-th of four consecutive instructions: one 16-byte LDS read per operand
//   block feeds four MFMAs. (Element-wise fragment reads run at half the LDS
//   rate of 16-byte reads on this chip and were the bottleneck of the k loop.)
//   An operand that is k-contiguous in memory goes into LDS with 16-byte stores;
//   an x-contiguous one is transposed with element stores, consecutive lanes
//   taking consecutive k so that the stores of a wave cover consecutive banks.
// * Software pipeline: a ring of registers keeps the global loads of the next
//   three tiles in flight (buffer loads: out-of-range lanes read zero, no
//   branches); tile t+1 moves from its ring slot to one of three LDS buffers
//   during the first k steps of tile t; LDS fragments of k step s+1 (also across
//   the tile boundary) are fetched while the MFMAs of step s issue. One
//   LDS-only barrier per tile, in the middle of the tile.
// * The two MFMA operands are passed swapped (the instruction computes the
//   transposed block), so a lane ends up with four consecutive COLUMNS of one
//   output row: the epilogue applies bias + activation in registers and writes
//   one float4 per 16x16 block, with no trip through LDS and no barrier.
//   Epilogues that are not "per-column operands + relu-family activation"
//   (sigmoid, elu, bias or PReLU weights that vary along rows or batch) store
//   the raw sums and are completed in place by gemm_finish, a second kernel
//   enqueued right behind.
// * Loaders (template parameter) decide how a tile is fetched:
//     kLoadKVec   operand is k-contiguous in memory (A row-major, or B given
//                 transposed): 16-byte loads along k, transposed into LDS
//     kLoadXVec   operand is x-contiguous (B row-major, or A given transposed):
//                 16-byte loads along x, 16-byte LDS stores
//     kLoadScalar any strides, element loads with bounds checks
//     kLoadIm2colVec / kLoadIm2colScalar (A only): the rows of A are the
//                 receptive fields of an NHWC (or, scalar only, any-stride)
//                 image, gathered on the fly -- A is never materialised.
// * Workgroup ids are re-ordered so that the ids that land on one XCD (the
//   hardware deals consecutive ids round-robin over 8 XCDs, each with its own
//   L2) cover one contiguous band of tiles.
#pragma once

#include <hip/hip_runtime.h>

#include <type_traits>
#include <utility>

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
  // bytes addressable from the (per-batch) base of each operand, for the buffer descriptors
  unsigned a_bytes, b_bytes;
  // bytes addressable from the (per-batch) base of C, which is also the size of a split-K slab; 0: more
  // than a descriptor's 32-bit offsets reach (results then leave as plain stores, else written through)
  unsigned c_bytes;
  int tiles_m, tiles_n;
  int group_m;    // tile rows per panel of the tile numbering
  // split K: the grid holds `splits` copies of the tile set, copy s sums
  // k in [s * k_per_split, (s+1) * k_per_split) into ws[s][batch][M][N]
  int splits, k_per_split;
  float *ws;
  int vec_store;  // rows of C are 16-byte aligned and N % 4 == 0
  int inline_epilogue;  // bias + activation happen in gemm_kernel (else gemm_finish completes the raw sums)
  ConvGeom conv;
  Epilogue epi;
};

typedef float float4_t __attribute__((ext_vector_type(4)));
typedef unsigned int uint4_t __attribute__((ext_vector_type(4)));

constexpr unsigned kNoOffset = 0xffffffffu;  // a buffer offset no descriptor covers: loads return 0

// KG: groups of four wavefronts per workgroup. Every group runs the whole pipeline below on its own
// slice of k, with LDS buffers of its own, and the groups' sums are added through LDS at the end: a
// product with few tiles and a long k then has KG times the wavefronts per compute unit to hide the
// latencies of a k step behind, and a k loop KG times shorter.
template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int A_KIND, int B_KIND, int KG = 1>
struct GemmTile {
  static constexpr int kThreads = 256;   // per group
  static_assert(WAVES_M * WAVES_N == 4, "four wavefronts per workgroup");
  static_assert(BK == 16 || BK == 32, "k step of the tile");
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int TM = WM / 16, TN = WN / 16;
  static_assert(WM % 16 == 0 && WN % 16 == 0, "tile shape");
  static constexpr int PITCH = BK + 8;   // floats per LDS row: 16-byte fragment reads of a wave spread over all banks
  static constexpr int QUADS = BK / 16;  // groups of four MFMA k steps fed by one 16-byte read
  // 16-byte fetches per thread per tile (the last round may be partly idle)
  static constexpr int A_VECS = (BM * BK / 4 + kThreads - 1) / kThreads;
  static constexpr int B_VECS = (BN * BK / 4 + kThreads - 1) / kThreads;
  static constexpr int A_BUF = BM * PITCH, B_BUF = BN * PITCH;
  // Three LDS buffers, and three tiles in flight between global memory and LDS (the ring of register
  // slots in gemm_kernel takes any depth; six slots on the 32 x 32 x 32 and 64 x 64 x 16 tiles were
  // slower on every MobileNetV2 projection, by 0.5 - 1.5 us of 7 - 15: the k loop of these
  // launches is not waiting for a fetch that three tiles in flight fail to cover)
  static constexpr int PREFETCH = 3;
  static constexpr int GROUP_LDS_FLOATS = 3 * (A_BUF + B_BUF);
  static constexpr int LDS_FLOATS = KG * GROUP_LDS_FLOATS;
  static_assert(KG == 1 || (KG - 1) * kThreads * TM * TN * 4 <= LDS_FLOATS, "the groups' sums fit the tile buffers");
};

__device__ __forceinline__ const float *uniform_pointer(const float *ptr) {
  const unsigned long long v = reinterpret_cast<unsigned long long>(ptr);
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v);
  const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
  return reinterpret_cast<const float *>(((unsigned long long)hi << 32) | lo);
}

__device__ __forceinline__ float4 as_float4(uint4_t v) {
  return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
}

// Per-thread addressing state of one operand loader, fixed across k tiles.
template <int VECS>
struct LoaderState {
  unsigned row_off[VECS];   // byte offset of this thread's row (or kNoOffset)
  int row_ih[VECS];         // im2col: top-left input coordinate of the row's window
  int row_iw[VECS];
};

template <int BX, int BK, int KIND, int VECS>
__device__ __forceinline__ void init_loader(LoaderState<VECS> &st, long long sx, long long sk, int X, int x0, int tid,
                                            const ConvGeom &g) {
#pragma unroll
  for (int i = 0; i < VECS; ++i) {
    const int f = tid + i * 256;
    st.row_ih[i] = st.row_iw[i] = 0;
    if ((BX * BK / 4) % 256 != 0 && f >= BX * BK / 4) {
      st.row_off[i] = kNoOffset;
      continue;
    }
    if (KIND == kLoadKVec) {
      const int x = x0 + f / (BK / 4);
      st.row_off[i] = x < X ? (unsigned)((long long)x * sx * 4) : kNoOffset;
    } else if (KIND == kLoadXVec) {
      const int x = x0 + (f / BK) * 4;   // consecutive lanes: consecutive k
      st.row_off[i] = x < X ? (unsigned)(x * 4) : kNoOffset;
    } else if (KIND == kLoadIm2colVec || KIND == kLoadIm2colScalar) {
      const int m = x0 + f / (BK / 4);
      if (m < X) {
        const int ow = m % g.out_w;
        const int t2 = m / g.out_w;
        const int oh = t2 % g.out_h, n = t2 / g.out_h;
        st.row_off[i] = (unsigned)((long long)n * g.xs_n * 4);
        st.row_ih[i] = oh * g.stride_h - g.pad_top;
        st.row_iw[i] = ow * g.stride_w - g.pad_left;
      } else {
        st.row_off[i] = kNoOffset;
      }
    } else {
      st.row_off[i] = 0;
    }
  }
}

// Issues this thread's share of the loads of the BX x BK tile at (x0, k0).
template <int BX, int BK, int KIND, int VECS>
__device__ __forceinline__ void load_tile(float4 (&reg)[VECS], const LoaderState<VECS> &st,
                                          __amdgpu_buffer_rsrc_t rsrc, const float *__restrict__ base, long long sx,
                                          long long sk, int X, int K, int x0, int k0, int tid, const ConvGeom &g) {
  if (KIND == kLoadKVec) {
    // the k offset of a thread is the same for all its rows (256 % (BK/4) == 0)
    const int k = k0 + (tid % (BK / 4)) * 4;
    const bool k_ok = k < K;
#pragma unroll
    for (int i = 0; i < VECS; ++i) {
      const unsigned off = (k_ok && st.row_off[i] != kNoOffset) ? st.row_off[i] + (unsigned)(k * 4) : kNoOffset;
      reg[i] = as_float4(__builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)off, 0, 0));
    }
  } else if (KIND == kLoadXVec) {
#pragma unroll
    for (int i = 0; i < VECS; ++i) {
      const int k = k0 + (tid + i * 256) % BK;
      const unsigned off =
          (k < K && st.row_off[i] != kNoOffset) ? st.row_off[i] + (unsigned)((long long)k * sk * 4) : kNoOffset;
      reg[i] = as_float4(__builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)off, 0, 0));
    }
  } else if (KIND == kLoadIm2colVec) {
    // in_c % 4 == 0: the four k values of a fetch share one filter tap (r, s)
    const int k = k0 + (tid % (BK / 4)) * 4;
    const int tap = k / g.in_c, c = k - tap * g.in_c;
    const int r = tap / g.f_w, s = tap - r * g.f_w;
    const int dh = r * g.dil_h, dw = s * g.dil_w;
    const bool k_ok = k < K;
#pragma unroll
    for (int i = 0; i < VECS; ++i) {
      const int ih = st.row_ih[i] + dh, iw = st.row_iw[i] + dw;
      const bool ok = k_ok && st.row_off[i] != kNoOffset && ih >= 0 && ih < g.in_h && iw >= 0 && iw < g.in_w;
      const unsigned off = ok ? st.row_off[i] + (unsigned)((ih * g.xs_h + iw * g.xs_w + c) * 4) : kNoOffset;
      reg[i] = as_float4(__builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)off, 0, 0));
    }
  } else if (KIND == kLoadScalar) {
#pragma unroll
    for (int i = 0; i < VECS; ++i) {
      const int f = tid + i * 256;
      const int x = x0 + f / (BK / 4), k = k0 + (f % (BK / 4)) * 4;
      float v[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const bool ok = st.row_off[i] != kNoOffset && x < X && k + j < K;
        v[j] = ok ? base[(long long)x * sx + (long long)(k + j) * sk] : 0.f;
      }
      reg[i] = make_float4(v[0], v[1], v[2], v[3]);
    }
  } else {  // kLoadIm2colScalar
#pragma unroll
    for (int i = 0; i < VECS; ++i) {
      const int f = tid + i * 256;
      float v[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int k = k0 + (f % (BK / 4)) * 4 + j;
        v[j] = 0.f;
        if (st.row_off[i] != kNoOffset && k < K) {
          const int tap = k / g.in_c, c = k - tap * g.in_c;
          const int r = tap / g.f_w, s = tap - r * g.f_w;
          const int ih = st.row_ih[i] + r * g.dil_h, iw = st.row_iw[i] + s * g.dil_w;
          if (ih >= 0 && ih < g.in_h && iw >= 0 && iw < g.in_w)
            v[j] = base[(long long)(st.row_off[i] >> 2) + ih * g.xs_h + iw * g.xs_w + c * g.xs_c];
        }
      }
      reg[i] = make_float4(v[0], v[1], v[2], v[3]);
    }
  }
}

// Writes vectors [first, last) of the registers fetched by load_tile into an
// x-major LDS tile [BX][PITCH].
template <int BX, int BK, int PITCH, int KIND, int VECS>
__device__ __forceinline__ void store_tile(float *__restrict__ lds, const float4 (&reg)[VECS], int tid,
                                           int first = 0, int last = VECS) {
#pragma unroll
  for (int i = 0; i < VECS; ++i) {
    if (i < first || i >= last) continue;
    const int f = tid + i * 256;
    if ((BX * BK / 4) % 256 != 0 && f >= BX * BK / 4) continue;
    if (KIND == kLoadXVec) {
      // four consecutive x at one k: transposed, element by element
      const int k = f % BK, xq = f / BK;
      float *d = lds + (xq * 4) * PITCH + k;
      d[0] = reg[i].x;
      d[PITCH] = reg[i].y;
      d[2 * PITCH] = reg[i].z;
      d[3 * PITCH] = reg[i].w;
    } else {
      // four consecutive k of one row
      const int row = f / (BK / 4), kq = f % (BK / 4);
      *reinterpret_cast<float4 *>(lds + row * PITCH + kq * 4) = reg[i];
    }
  }
}

// Fragments of quad `quad` (16 k) for NT blocks of 16 rows: lane (g, r) reads
// k = 16 quad + 4 g .. +3 of row r of each block. `lane_base` points at the
// lane's (r, g) position in block 0 of buffer 0.
template <int PITCH, int NT>
__device__ __forceinline__ void load_fragment(float4 (&frag)[NT], const float *lane_base, int buf_off, int quad) {
#pragma unroll
  for (int t = 0; t < NT; ++t)
    frag[t] = *reinterpret_cast<const float4 *>(lane_base + buf_off + t * 16 * PITCH + quad * 16);
}

// f(integral_constant<int, I>) for every I of the sequence, in order.
template <int... I, typename F>
__device__ __forceinline__ void static_for(std::integer_sequence<int, I...>, F &&f) {
  (f(std::integral_constant<int, I>()), ...);
}

__device__ __forceinline__ float quad_element(const float4 &v, int j) {
  return j == 0 ? v.x : (j == 1 ? v.y : (j == 2 ? v.z : v.w));
}

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int A_KIND, int B_KIND, int KG = 1>
__global__ __launch_bounds__(256 * KG) void gemm_kernel(GemmParams p) {
  using T = GemmTile<BM, BN, BK, WAVES_M, WAVES_N, A_KIND, B_KIND, KG>;
  extern __shared__ float lds[];
  // Every kernel argument the prologue reads, asked for here in one piece: the compiler fetches an
  // argument where it is first used, and the prologue's branches and divisions would otherwise cut
  // those fetches into three or four batches, each waiting a scalar-cache miss of its own.
  asm volatile("" ::"s"(p.a), "s"(p.b), "s"(p.c), "s"(p.M), "s"(p.N), "s"(p.K), "s"(p.batch), "s"(p.a_sx), "s"(p.a_sk),
               "s"(p.b_sx), "s"(p.b_sk), "s"(p.ldc), "s"(p.a_bytes), "s"(p.b_bytes), "s"(p.tiles_m), "s"(p.tiles_n),
               "s"(p.group_m), "s"(p.splits), "s"(p.k_per_split), "s"(p.vec_store), "s"(p.inline_epilogue),
               "s"(p.epi.bias), "s"(p.epi.bias_s[3]), "s"(p.epi.activation), "s"(p.epi.residual), "s"(p.epi.addressing));
  // this wavefront's group, and its thread index inside the group
  const int kgroup = KG > 1 ? __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 8) : 0;
  float *lds_a = lds + kgroup * T::GROUP_LDS_FLOATS;   // [3][BM][PITCH]
  float *lds_b = lds_a + 3 * T::A_BUF;                 // [3][BN][PITCH]

  // Workgroup id -> (batch, tile_m, tile_n). Ids i, i+8, i+16, ... share an XCD;
  // give each XCD one contiguous band of the tile sequence.
  int id = blockIdx.x;
  {
    const int per_xcd = gridDim.x / 8;
    if (per_xcd > 0 && id < per_xcd * 8) id = (id % 8) * per_xcd + id / 8;
  }
  const int tiles_per_batch = p.tiles_m * p.tiles_n;
  int split = 0, bz = 0;
  if (p.splits * p.batch > 1) {   // (most launches: one product, not split; no division for them)
    split = id / (tiles_per_batch * p.batch);
    id -= split * tiles_per_batch * p.batch;
    bz = id / tiles_per_batch;
  }
  const int t = id - bz * tiles_per_batch;
  int k_begin = split * p.k_per_split;
  int k_end = k_begin + p.k_per_split < p.K ? k_begin + p.k_per_split : p.K;
  // the groups cut this range into KG runs of whole k tiles, all of the same tile count (a run that
  // starts beyond the range reads zeros), so that every group reaches every barrier
  int group_k_tiles = 0;
  if (KG > 1) {
    const int all_tiles = (k_end - k_begin + BK - 1) / BK;
    group_k_tiles = (all_tiles + KG - 1) / KG;
    k_begin += kgroup * group_k_tiles * BK;
    const int run_end = k_begin + group_k_tiles * BK;
    k_end = run_end < k_end ? run_end : k_end;
    if (k_end < k_begin) k_end = k_begin;
  }
  // Tiles are numbered in panels of group_m tile rows, column by column inside a
  // panel, so that the run of consecutive ids that is resident on one XCD covers
  // a near-square block of C: the rows of A and columns of B it needs per k tile
  // are as few as possible and stay in that XCD's L2.
  const int width = p.group_m * p.tiles_n;
  const int first_m = (t / width) * p.group_m;
  const int gsz = p.tiles_m - first_m < p.group_m ? p.tiles_m - first_m : p.group_m;
  const int in_group = t % width;
  const int tile_m = first_m + in_group % gsz, tile_n = in_group / gsz;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  // The operand bases are the same for the whole workgroup; readfirstlane pins
  // them to scalar registers so that the buffer descriptors built from them are
  // scalar too (a descriptor the compiler believes to vary per lane makes it
  // wrap every buffer load in a loop over the distinct values).
  const float *A = uniform_pointer(p.a + (long long)(bz % p.batch_a) * p.a_batch_stride);
  const float *B = uniform_pointer(p.b + (long long)(bz % p.batch_b) * p.b_batch_stride);
  const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc((void *)A, 0, (int)p.a_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc((void *)B, 0, (int)p.b_bytes, 0x00020000);

  const int tid = KG > 1 ? (int)threadIdx.x & 255 : (int)threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave / WAVES_N) * T::WM, wn0 = (wave % WAVES_N) * T::WN;

  LoaderState<T::A_VECS> sa;
  LoaderState<T::B_VECS> sb;
  init_loader<BM, BK, A_KIND, T::A_VECS>(sa, p.a_sx, p.a_sk, p.M, m0, tid, p.conv);
  init_loader<BN, BK, B_KIND, T::B_VECS>(sb, p.b_sx, p.b_sk, p.N, n0, tid, p.conv);

  // lane position inside the x-major tiles: row (lane % 16) of the wave's first
  // block, k group (lane / 16)
  const float *a_lane = lds_a + (wm0 + (lane & 15)) * T::PITCH + (lane >> 4) * 4;
  const float *b_lane = lds_b + (wn0 + (lane & 15)) * T::PITCH + (lane >> 4) * 4;

  const Epilogue &e = p.epi;
  const bool fused = p.inline_epilogue != 0;
  float4_t acc[T::TM][T::TN];

  // Software pipeline over k tiles, D (three or six) deep in registers, three deep in LDS:
  //  * registers: tile t lives in ring slot t % D from its global fetch (issued
  //    while tile t-D-1 computes) until it is stored to LDS (while tile t-1 computes)
  //  * LDS: tile t lives in buffer t % 3. It is written during the first k steps of
  //    tile t-1, ONE barrier in the middle of tile t-1 publishes it, and the last k
  //    step of tile t-1 already fetches its first fragments, so no wave ever waits
  //    for LDS at a tile boundary. The buffer it overwrites held tile t-3, which
  //    every wave finished before it reached the barrier inside tile t-2.
  constexpr int D = T::PREFETCH;
  float4 ra[D][T::A_VECS], rb[D][T::B_VECS];
  const int k_tiles = KG > 1 ? group_k_tiles : (k_end - k_begin + BK - 1) / BK;

  // Every fetch is unconditional: a tile past K reads as zeros through the buffer
  // descriptor at no memory cost, and with no branch around a load the compiler
  // can count exactly how many loads may stay in flight at each use (a
  // conditional load makes it assume the shortest queue and wait for all).
#pragma unroll
  for (int d = 0; d < D; ++d) {
    load_tile<BM, BK, A_KIND, T::A_VECS>(ra[d], sa, rsrc_a, A, p.a_sx, p.a_sk, p.M, k_end, m0, k_begin + d * BK, tid,
                                         p.conv);
    load_tile<BN, BK, B_KIND, T::B_VECS>(rb[d], sb, rsrc_b, B, p.b_sx, p.b_sk, p.N, k_end, n0, k_begin + d * BK, tid,
                                         p.conv);
  }
  // The accumulators start from the bias (lane l of a 16x16 block ends up with
  // columns 4 * (l / 16) .. +3 of its row, see the epilogue): its fetch is issued
  // behind the first tiles' and shares their round trip, instead of costing one of
  // its own before them or after the k loop. A product that is completed by
  // gemm_finish starts from zero.
  {
    const int lane_col = n0 + wn0 + (lane >> 4) * 4;
    const bool with_bias = fused && e.bias != nullptr && kgroup == 0;
#pragma unroll
    for (int j = 0; j < T::TN; ++j) {
      float4_t b4 = {0.f, 0.f, 0.f, 0.f};
      if (with_bias) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int col = lane_col + j * 16 + q;
          b4[q] = e.bias[(long long)(col < p.N ? col : p.N - 1) * e.bias_s[3]];
        }
      }
#pragma unroll
      for (int i = 0; i < T::TM; ++i) acc[i][j] = b4;
    }
  }
  store_tile<BM, BK, T::PITCH, A_KIND, T::A_VECS>(lds_a, ra[0], tid);
  store_tile<BN, BK, T::PITCH, B_KIND, T::B_VECS>(lds_b, rb[0], tid);
  load_tile<BM, BK, A_KIND, T::A_VECS>(ra[0], sa, rsrc_a, A, p.a_sx, p.a_sk, p.M, k_end, m0, k_begin + D * BK, tid,
                                       p.conv);
  load_tile<BN, BK, B_KIND, T::B_VECS>(rb[0], sb, rsrc_b, B, p.b_sx, p.b_sk, p.N, k_end, n0, k_begin + D * BK, tid,
                                       p.conv);
  lds_barrier();

  // fragments of the quad being multiplied and of the one after it (also across
  // the tile boundary)
  float4 fa[T::TM], fb[T::TN], na[T::TM], nb4[T::TN];
  load_fragment<T::PITCH, T::TM>(fa, a_lane, 0, 0);
  load_fragment<T::PITCH, T::TN>(fb, b_lane, 0, 0);

  // A tile is QUADS quads of four MFMA groups (one group = all TM x TN blocks at
  // one k position of the quad). Side work of the tile is cut into pieces dealt
  // out over the groups (LDS serves the four waves in order: a burst of tile
  // stores would hold up the fragment reads queued behind it):
  //   pieces 0 .. A_VECS-1              one 16-byte vector of tile kt+1 -> LDS (A)
  //   pieces A_VECS .. A_VECS+B_VECS-1  the same for B
  //   then the global fetches of tile kt+4 into the ring slot just drained, A and
  //   B as one piece each.
  // The next quad's fragments are fetched in group 2 of each quad (group 0 for the smallest
  // wave tiles, below); for the last quad of a tile they come from tile kt+1, so its stores and
  // the barrier must be over by the group before.
  // A wavefront with a single block has groups of one matrix instruction: two groups are 64
  // cycles, less than an LDS read takes, and every quad then began with a wait for its
  // fragments. There the next quad's fragments are fetched in group 0, a whole quad ahead, and
  // the barrier comes as late as that allows, so that the tile stores in front of it have the
  // longest time to complete (256 x 512 x 512 on the 32 x 32 x 32 tile: 7.0 -> 6.55 us back to
  // back; the fifteen MobileNetV2 projections on that tile 0.1 - 0.5 us each).
  constexpr int Q = T::QUADS;
  constexpr bool kFewBlocks = T::TM * T::TN == 1 && Q >= 2;
  constexpr int kFetchGroup = kFewBlocks ? 0 : 2;   // group of a quad that fetches the next quad's fragments
  constexpr int kGroups = 4 * Q;
  constexpr int kStores = T::A_VECS + T::B_VECS;
  constexpr int kPieces = kStores + 2;
  constexpr int kEven = (kPieces + kGroups - 1) / kGroups;
  constexpr int kStoreGroups = 4 * (Q - 1) + kFetchGroup;   // groups in front of the fetch from tile kt+1
  constexpr int kForStores = (kStores + kStoreGroups - 1) / kStoreGroups;
  constexpr int kPerGroup = kEven > kForStores ? kEven : kForStores;
  constexpr int kLastStoreGroup = (kStores - 1) / kPerGroup;
  constexpr int kBarrierGroup = kFewBlocks ? kStoreGroups - 1 : kLastStoreGroup;
  static_assert(kLastStoreGroup <= kBarrierGroup && kBarrierGroup < kStoreGroups,
                "the barrier follows the last store and precedes the fetch of the next tile's fragments");

  // One k tile: tile kt = L * n + i sits in LDS buffer u = i % 3, tile kt+1 in ring slot (i+1) % D and
  // goes to LDS buffer (u+1) % 3.
  auto tile_step = [&](int kt, auto i_tag) __attribute__((always_inline)) {
    constexpr int u = decltype(i_tag)::value % 3;
    constexpr int nb = (u + 1) % 3;
    constexpr int slot = (decltype(i_tag)::value + 1) % D;
    const int a_off = u * T::A_BUF, b_off = u * T::B_BUF;
#pragma unroll
    for (int quad = 0; quad < Q; ++quad) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        constexpr int kDummy = 0;
        (void)kDummy;
        const int group = quad * 4 + j;
        if (j == kFetchGroup) {
          if (quad + 1 < Q) {
            load_fragment<T::PITCH, T::TM>(na, a_lane, a_off, quad + 1);
            load_fragment<T::PITCH, T::TN>(nb4, b_lane, b_off, quad + 1);
          } else {
            load_fragment<T::PITCH, T::TM>(na, a_lane, nb * T::A_BUF, 0);
            load_fragment<T::PITCH, T::TN>(nb4, b_lane, nb * T::B_BUF, 0);
          }
        }
#pragma unroll
        for (int piece = group * kPerGroup; piece < (group + 1) * kPerGroup && piece < kPieces; ++piece) {
          if (piece < T::A_VECS) {
            store_tile<BM, BK, T::PITCH, A_KIND, T::A_VECS>(lds_a + nb * T::A_BUF, ra[slot], tid, piece, piece + 1);
          } else if (piece < kStores) {
            store_tile<BN, BK, T::PITCH, B_KIND, T::B_VECS>(lds_b + nb * T::B_BUF, rb[slot], tid, piece - T::A_VECS,
                                                            piece - T::A_VECS + 1);
          } else if (piece == kStores) {
            load_tile<BM, BK, A_KIND, T::A_VECS>(ra[slot], sa, rsrc_a, A, p.a_sx, p.a_sk, p.M, k_end, m0,
                                                 k_begin + (kt + 1 + D) * BK, tid, p.conv);
          } else {
            load_tile<BN, BK, B_KIND, T::B_VECS>(rb[slot], sb, rsrc_b, B, p.b_sx, p.b_sk, p.N, k_end, n0,
                                                 k_begin + (kt + 1 + D) * BK, tid, p.conv);
          }
        }
#pragma unroll
        for (int i = 0; i < T::TM; ++i)
#pragma unroll
          for (int jn = 0; jn < T::TN; ++jn)
            acc[i][jn] = __builtin_amdgcn_mfma_f32_16x16x4f32(quad_element(fb[jn], j), quad_element(fa[i], j),
                                                              acc[i][jn], 0, 0, 0);
        // Issue order inside the group: after every matrix instruction a little of
        // the side work, so that it issues in the shadow of the matrix pipe. A wave
        // issues in order: side work in a block in front of the MFMAs is exposed
        // whenever a SIMD holds a single wave.
#pragma unroll
        for (int m = 0; m < T::TM * T::TN; ++m) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one MFMA
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read
          __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);   // one LDS write
          __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);   // one global read
          __builtin_amdgcn_sched_group_barrier(0x006, 3, 0);   // a few vector / scalar ALU
        }
        __builtin_amdgcn_sched_barrier(0);   // groups stay in order
        if (group == kBarrierGroup) {
          lds_barrier();                     // tile kt+1 is complete in LDS
          __builtin_amdgcn_sched_barrier(0);
        }
      }
#pragma unroll
      for (int i = 0; i < T::TM; ++i) fa[i] = na[i];
#pragma unroll
      for (int jn = 0; jn < T::TN; ++jn) fb[jn] = nb4[jn];
    }
  };

  // Full turns of the two rings (L tiles: both ring positions are then constants) run without a
  // branch between them; the remainder follows with one check per tile.
  constexpr int L = D % 3 == 0 ? D : 3 * D;
  int kt = 0;
  for (; kt + L <= k_tiles; kt += L)
    static_for(std::make_integer_sequence<int, L>(), [&](auto i) __attribute__((always_inline)) { tile_step(kt + decltype(i)::value, i); });
  static_for(std::make_integer_sequence<int, L - 1>(), [&](auto i) __attribute__((always_inline)) {
    if (kt + decltype(i)::value < k_tiles) tile_step(kt + decltype(i)::value, i);
  });

  // ---- the groups' sums into group 0, through LDS (the tile buffers are free once every
  // wavefront is past its last fragment read)
  if (KG > 1) {
    lds_barrier();
    float4_t *sums = reinterpret_cast<float4_t *>(lds);   // [KG - 1][TM * TN][256]
    if (kgroup > 0) {
#pragma unroll
      for (int i = 0; i < T::TM; ++i)
#pragma unroll
        for (int j = 0; j < T::TN; ++j) sums[((kgroup - 1) * T::TM * T::TN + i * T::TN + j) * 256 + tid] = acc[i][j];
    }
    lds_barrier();
    if (kgroup > 0) return;
#pragma unroll
    for (int gk = 1; gk < KG; ++gk)
#pragma unroll
      for (int i = 0; i < T::TM; ++i)
#pragma unroll
        for (int j = 0; j < T::TN; ++j) acc[i][j] += sums[((gk - 1) * T::TM * T::TN + i * T::TN + j) * 256 + tid];
  }

  // ---- epilogue: registers -> global. Lane l of a 16x16 block holds row l % 16,
  // columns 4 * (l / 16) .. +3 (the operands went into the MFMA swapped).
  const int lane_m = lane & 15, lane_n = (lane >> 4) * 4;
  // destination: the output itself, or this split's dense [M][N] slab of the workspace
  const bool to_ws = p.splits > 1;
  float *C = to_ws ? p.ws + ((long long)split * p.batch + bz) * p.M * p.N : p.c + (long long)bz * p.c_batch_stride;
  const long long ldc = to_ws ? p.N : p.ldc;
  const bool conv_addr = !to_ws && e.addressing == kConv;
  const bool vec = to_ws ? p.N % 4 == 0 : p.vec_store != 0;
  const bool through = p.c_bytes != 0;
  const __amdgpu_buffer_rsrc_t rsrc_c =
      __builtin_amdgcn_make_buffer_rsrc((void *)uniform_pointer(C), 0, (int)p.c_bytes, 0x00020000);
  // the residual lies where the output element does
  const float *R = (fused && e.residual) ? e.residual + (long long)bz * p.c_batch_stride : nullptr;
  float alpha_q[T::TN][4];
#pragma unroll
  for (int j = 0; j < T::TN; ++j) {
    const int col = n0 + wn0 + j * 16 + lane_n;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const bool ok = fused && col + q < p.N;
      alpha_q[j][q] = (ok && e.activation == TFHIP_PRELU) ? e.prelu[(long long)(col + q) * e.prelu_s[3]] : 0.f;
    }
  }
  auto write_out = [&](auto act_tag) __attribute__((always_inline)) {
    constexpr int ACT = decltype(act_tag)::value;
#pragma unroll
    for (int i = 0; i < T::TM; ++i) {
      const int row = m0 + wm0 + i * 16 + lane_m;
      if (row >= p.M) continue;
      long long base = (long long)row * ldc, col_stride = 1;
      if (conv_addr) {
        const int ow = row % e.out_w;
        const int t2 = row / e.out_w;
        base = (long long)(t2 / e.out_h) * e.y_s[0] + (long long)(t2 % e.out_h) * e.y_s[1] + ow * e.y_s[2];
        col_stride = e.y_s[3];
      }
#pragma unroll
      for (int j = 0; j < T::TN; ++j) {
        const int col = n0 + wn0 + j * 16 + lane_n;
        if (col >= p.N) continue;
        float out[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float v = acc[i][j][q];
          if (ACT == TFHIP_RELU) {
            out[q] = (v > 0.f || v != v) ? v : 0.f;
          } else if (ACT == TFHIP_RELU6) {
            const float t = (v > 0.f || v != v) ? v : 0.f;
            out[q] = t > 6.f ? 6.f : t;
          } else if (ACT == TFHIP_PRELU) {
            out[q] = v < 0.f ? alpha_q[j][q] * v : v;
          } else if (ACT == TFHIP_LEAKYRELU) {
            out[q] = v < 0.f ? (float)(e.leaky_alpha * (double)v) : v;
          } else {
            out[q] = v;
          }
        }
        if (vec) {
          if (R) {
            const float4 r4 = *reinterpret_cast<const float4 *>(R + base + col);
            out[0] += r4.x; out[1] += r4.y; out[2] += r4.z; out[3] += r4.w;
          }
          const float4 out4 = make_float4(out[0], out[1], out[2], out[3]);
          if (through) store_result4_through(rsrc_c, (unsigned)((base + col) * 4), out4);
          else store_result4(C + base + col, out4);
        } else {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            if (col + q < p.N) {
              const long long at = base + (col + q) * col_stride;
              C[at] = R ? out[q] + R[at] : out[q];
            }
          }
        }
      }
    }
  };
  switch (fused ? e.activation : TFHIP_LINEAR) {
    case TFHIP_RELU: write_out(std::integral_constant<int, TFHIP_RELU>()); break;
    case TFHIP_RELU6: write_out(std::integral_constant<int, TFHIP_RELU6>()); break;
    case TFHIP_PRELU: write_out(std::integral_constant<int, TFHIP_PRELU>()); break;
    case TFHIP_LEAKYRELU: write_out(std::integral_constant<int, TFHIP_LEAKYRELU>()); break;
    default: write_out(std::integral_constant<int, TFHIP_LINEAR>()); break;
  }
}

// Completes an output that gemm_kernel left as raw sums (in place, or as split-K
// partial slabs in the workspace): bias with any broadcast shape and any
// activation, one element per thread and trip.
static __global__ __launch_bounds__(256) void gemm_finish(GemmParams p) {
  const Epilogue &e = p.epi;
  const long long per_batch = (long long)p.M * p.N;
  const long long total = per_batch * p.batch;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
    const long long bz = idx / per_batch;
    const long long rem = idx - bz * per_batch;
    const long long row = rem / p.N, col = rem - row * p.N;
    long long n = 0, oh = 0, ow = 0;
    long long at = bz * p.c_batch_stride + row * p.ldc + col;
    if (e.addressing == kConv) {
      ow = row % e.out_w;
      const long long t2 = row / e.out_w;
      oh = t2 % e.out_h;
      n = t2 / e.out_h;
      at = n * e.y_s[0] + oh * e.y_s[1] + ow * e.y_s[2] + col * e.y_s[3];
    }
    float v;
    if (p.splits > 1) {
      // partial sums in ascending k order
      v = p.ws[idx];
      for (int sp = 1; sp < p.splits; ++sp) v += p.ws[(long long)sp * total + idx];
    } else {
      v = p.c[at];
    }
    v = finish(e, v, bz, row, col, n, oh, ow);
    p.c[at] = e.residual ? v + e.residual[at] : v;
  }
}

}  // namespace tfhip
