// Streaming GEMM for tall products with a small B: C[M x N] = A[M x K] * B[K x N]
// with M in the tens of thousands and K * N small enough for B to sit in LDS
// (the pointwise convolutions of a mobile network: N = 16 .. 192, K = 16 .. 576).
//
// Such a product is bound by reading A and writing C once. The tiled kernel
// spends its time in per-tile set-up instead (a two- or three-step k loop never
// fills its pipeline), so this kernel turns the loop around:
//  * B is transposed into LDS once per workgroup and stays there.
//  * Each wavefront walks over blocks of 16 rows of A. A lane fetches its part of
//    A straight from global memory as float4 along k, no LDS in between: the
//    matrix instruction only needs both operands of a lane to belong to the same
//    k, so lane (g, r) (g = lane / 16, r = lane % 16) takes k = 16t + 4g + j for
//    the j-th of four consecutive instructions, which is exactly the float4 it
//    loaded, and reads the matching B[k][.] from LDS, also as one float4.
//  * The loads of the next 64 k (or of the next row block) are in flight while
//    the current ones are consumed.
//  * Operands are passed swapped, as in gemm_kernel.h, so a lane ends with four
//    consecutive columns of one row and writes float4s after bias + activation.
#pragma once

#include <hip/hip_runtime.h>

#include <type_traits>

#include "common.h"
#include "gemm_kernel.h"

namespace tfhip {

struct SkinnyArgs {
  const float *a, *b, *bias;
  const float *residual;   // [M][N] like c, added after the activation; may be null
  float *c;
  long long bias_stride;
  double leaky_alpha;
  int M, N, K, k_pad;   // k_pad: K rounded up to 64
  unsigned a_bytes;
  int activation;
};

constexpr int kSkinnyChunk = 64;   // k per pipeline step: four float4 per lane
constexpr int kSkinnyPad = 8;      // LDS row pitch k_pad + 8: the pitch the 16-byte fragment reads run fastest at

// Cache policy of the fetches of A. Every element of A is read once, so a large A (beyond what the L2
// caches hold together) is fetched non-temporally: it would only push out what later kernels still
// want to find there - weights, residuals, the network's input (MobileNetV2 at batch 32, in
// sequence: the three launches here get 5 us slower in total and the rest of the inference 17 us
// faster).
constexpr long long kSkinnyStreamBytes = 32LL << 20;

// WAVES wavefronts per workgroup share one copy of B. STREAM_A: see above.
// SV > 0 (K = 16 SV): A goes through LDS. A 16-row block of A is one contiguous piece of memory, so
// the wavefront fetches it as such - every instruction 1 KB of whole cache lines instead of 64 bytes
// of each of 16 rows, whose other halves the next instruction asks for again - parks it in a region
// of LDS of its own (rows 4 floats apart from a multiple of 16: conflict-free fragment reads) and
// takes its fragments from there; the registers are free for the next block's fetch at once.
template <int TN, int WAVES, bool STREAM_A, int SV = 0>
__global__ __launch_bounds__(WAVES * 64) void skinny_gemm(SkinnyArgs g) {
  constexpr int kThreads = WAVES * 64;
  extern __shared__ float lds_bt[];          // [16 * TN][k_pad + kSkinnyPad]: B transposed, zero padded
  const int pitch = g.k_pad + kSkinnyPad;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int grp = lane >> 4, r = lane & 15;
  const __amdgpu_buffer_rsrc_t rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)uniform_pointer(g.a), 0, (int)g.a_bytes, 0x00020000);

  const int blocks = (g.M + 15) / 16;
  const int first = blockIdx.x * WAVES + wave, step = gridDim.x * WAVES;
  const int chunks = g.k_pad / kSkinnyChunk;
  const int my_blocks = first < blocks ? (blocks - first + step - 1) / step : 0;
  const int total = my_blocks * chunks;

  // loads of one step: k = c * 64 + 16 t + 4 grp .. +3 of row b * 16 + r
  auto issue = [&](float4 (&dst)[4], int b, int c) __attribute__((always_inline)) {
    const int row = b * 16 + r;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int k = c * kSkinnyChunk + 16 * t + 4 * grp;
      const unsigned off = (row < g.M && k < g.K) ? (unsigned)(((long long)row * g.K + k) * 4) : kNoOffset;
      dst[t] = as_float4(__builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)off, 0, STREAM_A ? 2 : 0));
    }
  };

  // Two accumulators per column group when there are few groups: consecutive
  // matrix instructions then never wait for each other's result.
  constexpr int NA = TN <= 2 ? 2 : 1;
  float4_t acc[NA][TN];
#pragma unroll
  for (int h = 0; h < NA; ++h)
#pragma unroll
    for (int n = 0; n < TN; ++n) acc[h][n] = (float4_t){0.f, 0.f, 0.f, 0.f};

  // ---- prologue: the first fetch of A, the whole of B and the bias are issued before anything
  // waits, so the three share one memory round trip (a fetch behind a branch, or the bias in front
  // of A, costs a round trip of its own: 3.4 us of an 11 us launch went into them, measured with
  // timestamps inside the kernel).
  float4 cur[4], nxt[4];
  constexpr int NV = SV > 0 ? SV : 1;
  float4 blk[NV];
  unsigned park[NV];   // where this lane's fetches of a block go in the wavefront's LDS region (float index)
  const int a_pitch = g.K + 4;
  float *stage = lds_bt + 16 * TN * pitch + wave * 16 * a_pitch;
  auto issue_block = [&](int b) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const long long e = (long long)b * 16 * g.K + 4 * (lane + 64 * i);   // first of this lane's four floats
      const unsigned off = (b < blocks && e * 4 < (long long)g.a_bytes) ? (unsigned)(e * 4) : kNoOffset;
      blk[i] = as_float4(__builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)off, 0, STREAM_A ? 2 : 0));
    }
  };
  if (SV > 0) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int e = 4 * (lane + 64 * i);
      const int row = e / g.K;
      park[i] = (unsigned)(row * a_pitch + (e - row * g.K));
    }
    issue_block(first);
  } else {
    issue(cur, total > 0 ? first : blocks, 0);   // (no row block: every offset is out of range, nothing is read)
  }

  // B -> LDS, transposed. Columns >= N and rows >= K read as zero; rows beyond
  // the last 16-row group that holds real data are never read. Consecutive lanes
  // take consecutive k (conflict-free LDS stores; B itself is small and cached),
  // and a thread's fetches of a pass are all issued before the first is stored.
  const int kk = ((g.K + 15) / 16) * 16;
  const int items = kk * (16 * TN / 4);
  constexpr int kFill = 8;   // fetches per thread and pass
  float4 v[kFill];
  auto fetch_b = [&](int i0) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < kFill; ++u) {
      const int i = i0 + u * kThreads;
      const int c = (i / kk) * 4, k = i - (i / kk) * kk;
      const bool real = i < items && k < g.K && c < g.N;
      const float4 w = *reinterpret_cast<const float4 *>(g.b + (real ? (long long)k * g.N + c : 0));
      v[u] = real ? w : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  };
  auto store_b = [&](int i0) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < kFill; ++u) {
      const int i = i0 + u * kThreads;
      if (i >= items) continue;
      const int c = (i / kk) * 4, k = i - (i / kk) * kk;
      lds_bt[(c + 0) * pitch + k] = v[u].x;
      lds_bt[(c + 1) * pitch + k] = v[u].y;
      lds_bt[(c + 2) * pitch + k] = v[u].z;
      lds_bt[(c + 3) * pitch + k] = v[u].w;
    }
  };
  fetch_b(tid);

  // per-lane epilogue operands: four consecutive columns of each 16-column group (a missing
  // bias or a column beyond N: the fetch goes to B's first element and is dropped)
  float bias_q[TN][4];
#pragma unroll
  for (int n = 0; n < TN; ++n)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int col = n * 16 + grp * 4 + q;
      const bool real = g.bias != nullptr && col < g.N;
      const float w = real ? g.bias[(long long)col * g.bias_stride] : g.b[0];
      bias_q[n][q] = real ? w : 0.f;
    }

  store_b(tid);
  for (int i0 = tid + kThreads * kFill; i0 < items; i0 += kThreads * kFill) {
    fetch_b(i0);
    store_b(i0);
  }
  lds_barrier();   // B is in LDS; nobody waits for a fetch here

  // bias, activation, residual and store of the finished row block b; the accumulators start over
  auto finish_block = [&](int b) __attribute__((always_inline)) {
    // lane holds row b*16 + r, columns n*16 + 4*grp .. +3
    const int row = b * 16 + r;
#pragma unroll
    for (int n = 0; n < TN; ++n) {
      const int col = n * 16 + grp * 4;
      float out[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        float v = (NA == 2 ? acc[0][n][k] + acc[NA - 1][n][k] : acc[0][n][k]) + bias_q[n][k];
        switch (g.activation) {
          case TFHIP_RELU: v = (v > 0.f || v != v) ? v : 0.f; break;
          case TFHIP_RELU6: v = (v > 0.f || v != v) ? v : 0.f; v = v > 6.f ? 6.f : v; break;
          case TFHIP_LEAKYRELU: v = v < 0.f ? (float)(g.leaky_alpha * (double)v) : v; break;
          default: break;
        }
        out[k] = v;
      }
      if (row < g.M && col < g.N) {
        if (g.residual) {
          const float4 r4 = *reinterpret_cast<const float4 *>(g.residual + (long long)row * g.N + col);
          out[0] += r4.x; out[1] += r4.y; out[2] += r4.z; out[3] += r4.w;
        }
        store_result4(g.c + (long long)row * g.N + col, make_float4(out[0], out[1], out[2], out[3]));
      }
#pragma unroll
      for (int h = 0; h < NA; ++h) acc[h][n] = (float4_t){0.f, 0.f, 0.f, 0.f};
    }
  };
  // the four matrix instructions per column group that one float4 of A feeds
  auto multiply = [&](const float4 &a, const float *bt) __attribute__((always_inline)) {
    const float a4[4] = {a.x, a.y, a.z, a.w};
    float4 b4[TN];
#pragma unroll
    for (int n = 0; n < TN; ++n) b4[n] = *reinterpret_cast<const float4 *>(bt + n * 16 * pitch);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int n = 0; n < TN; ++n) {
        const float bv = j == 0 ? b4[n].x : (j == 1 ? b4[n].y : (j == 2 ? b4[n].z : b4[n].w));
        acc[j % NA][n] = __builtin_amdgcn_mfma_f32_16x16x4f32(bv, a4[j], acc[j % NA][n], 0, 0, 0);
      }
    }
  };

  if (SV > 0) {
    for (int b = first; b < blocks; b += step) {
      // the block in the registers -> LDS (the wavefront's own region: its LDS accesses execute in
      // order, nobody else reads them), and the registers take the next block's fetch
#pragma unroll
      for (int i = 0; i < NV; ++i) *reinterpret_cast<float4 *>(stage + park[i]) = blk[i];
      issue_block(b + step);   // past the end: every offset is out of range, nothing is read
      const float *at = stage + r * a_pitch + 4 * grp;
      const float *bt = lds_bt + r * pitch + 4 * grp;
#pragma unroll
      for (int t = 0; t < NV; ++t) multiply(*reinterpret_cast<const float4 *>(at + 16 * t), bt + 16 * t);
      finish_block(b);
    }
    return;
  }

  int b = first, c = 0;
  for (int q = 0; q < total; ++q) {
    int nb = b, nc = c + 1;
    if (nc == chunks) {
      nc = 0;
      nb = b + step;
    }
    issue(nxt, q + 1 < total ? nb : blocks, nc);   // past the end: every offset is out of range, nothing is read

    const float *bt = lds_bt + r * pitch + c * kSkinnyChunk + 4 * grp;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      if (c * kSkinnyChunk + 16 * t >= g.K) continue;   // nothing but padding (the same for all lanes)
      multiply(cur[t], bt + 16 * t);
    }
    if (c == chunks - 1) finish_block(b);
#pragma unroll
    for (int t = 0; t < 4; ++t) cur[t] = nxt[t];
    b = nb;
    c = nc;
  }
}

// The same product with B held in REGISTERS instead of LDS, for K <= 32: a B so
// small that staging it through LDS - two memory round trips and a workgroup
// barrier before the first row block - costs more than the few row blocks each
// wavefront then has to do (measured 5-20% faster up to K = 32, 25% slower at
// K = 96 and 144, where the LDS kernel stays). Every wavefront
// is on its own: it fetches its share of B once (lane (g, r) keeps
// B[k][16 n + r] for exactly the k it will feed) together with its first rows
// of A and streams over its row blocks with the next block's A in flight.
//   KF    full k groups of 16 (lane takes k = 16 t + 4 g + j, a float4 of A)
//   HALF  one more group of 8 (lane takes k = 16 KF + 2 g + j, a float2 of A):
//         K = 24 costs six matrix instructions per block instead of eight
//   STAGED  (K = 32, a streamed A) the 2 KB row block is fetched as one contiguous piece, whole
//         cache lines per instruction, and turned into the fragment layout through a region of
//         LDS that belongs to the wavefront alone (see skinny_gemm)
template <int TN, int KF, bool HALF, bool STREAM_A, bool STAGED = false>
__global__ __launch_bounds__(256) void skinny_gemm_regs(SkinnyArgs g) {
  static_assert(!STAGED || (KF == 2 && !HALF), "the staged form is the K = 32 one");
  constexpr int STEPS = 4 * KF + (HALF ? 2 : 0);
  constexpr int kPitch = 36;   // floats per staged row: 16-byte reads of eight rows on different banks
  __shared__ float staged_rows[STAGED ? 4 * 16 * kPitch : 1];
  const int lane = threadIdx.x & 63;
  const int grp = lane >> 4, r = lane & 15;
  const __amdgpu_buffer_rsrc_t rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)uniform_pointer(g.a), 0, (int)g.a_bytes, 0x00020000);
  const int blocks = (g.M + 15) / 16;
  const int waves = gridDim.x * 4;
  const int first = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int n0 = blockIdx.y * (16 * TN);   // this workgroup's slice of the columns

  struct ABlock {
    float4 full[KF > 0 ? KF : 1];
    float2 half;
  };
  auto issue = [&](ABlock &dst, int b) __attribute__((always_inline)) {
    const int row = b * 16 + r;
    const bool row_ok = b < blocks && row < g.M;
#pragma unroll
    for (int t = 0; t < KF; ++t) {
      const int k = 16 * t + 4 * grp;
      const unsigned off = (row_ok && k < g.K) ? (unsigned)(((long long)row * g.K + k) * 4) : kNoOffset;
      dst.full[t] = as_float4(__builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)off, 0, STREAM_A ? 2 : 0));
    }
    if (HALF) {
      const int k = 16 * KF + 2 * grp;
      const unsigned off = (row_ok && k < g.K) ? (unsigned)(((long long)row * g.K + k) * 4) : kNoOffset;
      const auto v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, (int)off, 0, STREAM_A ? 2 : 0);
      dst.half = make_float2(__uint_as_float(v[0]), __uint_as_float(v[1]));
    }
  };
  ABlock cur, nxt;
  float *stage = staged_rows + (threadIdx.x >> 6) * 16 * kPitch;
  const int park0 = (lane >> 3) * kPitch + 4 * (lane & 7);   // lane's float4 of the first 1 KB: row lane / 8
  auto issue_flat = [&](ABlock &dst, int b) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const long long e = (long long)b * 512 + 4 * (lane + 64 * i);
      const unsigned off = (b < blocks && e * 4 < (long long)g.a_bytes) ? (unsigned)(e * 4) : kNoOffset;
      dst.full[i < KF ? i : 0] = as_float4(__builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)off, 0, STREAM_A ? 2 : 0));
    }
  };
  if (STAGED) issue_flat(nxt, first);
  else issue(cur, first);

  // this lane's B values and epilogue operands
  float breg[STEPS][TN];
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    const int k = s < 4 * KF ? 16 * (s / 4) + 4 * grp + s % 4 : 16 * KF + 2 * grp + (s - 4 * KF);
#pragma unroll
    for (int n = 0; n < TN; ++n) {
      const int col = n0 + n * 16 + r;
      breg[s][n] = (k < g.K && col < g.N) ? g.b[(long long)k * g.N + col] : 0.f;
    }
  }
  float4_t bias4[TN];
#pragma unroll
  for (int n = 0; n < TN; ++n)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int col = n0 + n * 16 + grp * 4 + q;
      bias4[n][q] = (g.bias && col < g.N) ? g.bias[(long long)col * g.bias_stride] : 0.f;
    }

  for (int b = first; b < blocks; b += waves) {
    if (STAGED) {
      // nxt holds block b as fetched; through LDS into the fragment layout (the wavefront's LDS
      // accesses execute in order), and nxt takes the next block's fetch
      *reinterpret_cast<float4 *>(stage + park0) = nxt.full[0];
      *reinterpret_cast<float4 *>(stage + park0 + 8 * kPitch) = nxt.full[KF > 1 ? 1 : 0];
      issue_flat(nxt, b + waves);
      cur.full[0] = *reinterpret_cast<const float4 *>(stage + r * kPitch + 4 * grp);
      cur.full[KF > 1 ? 1 : 0] = *reinterpret_cast<const float4 *>(stage + r * kPitch + 16 + 4 * grp);
    } else {
      issue(nxt, b + waves);   // past the end: every offset is out of range, nothing is read
    }
    float4_t acc[TN];
#pragma unroll
    for (int n = 0; n < TN; ++n) acc[n] = bias4[n];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      float av;
      if (s < 4 * KF) {
        const float4 v = cur.full[s / 4 < KF ? s / 4 : 0];
        av = s % 4 == 0 ? v.x : (s % 4 == 1 ? v.y : (s % 4 == 2 ? v.z : v.w));
      } else {
        av = s - 4 * KF == 0 ? cur.half.x : cur.half.y;
      }
#pragma unroll
      for (int n = 0; n < TN; ++n) acc[n] = __builtin_amdgcn_mfma_f32_16x16x4f32(breg[s][n], av, acc[n], 0, 0, 0);
    }
    // lane holds row b*16 + r, columns n0 + n*16 + 4*grp .. +3
    const int row = b * 16 + r;
#pragma unroll
    for (int n = 0; n < TN; ++n) {
      const int col = n0 + n * 16 + grp * 4;
      float out[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        float v = acc[n][k];
        switch (g.activation) {
          case TFHIP_RELU: v = (v > 0.f || v != v) ? v : 0.f; break;
          case TFHIP_RELU6: v = (v > 0.f || v != v) ? v : 0.f; v = v > 6.f ? 6.f : v; break;
          case TFHIP_LEAKYRELU: v = v < 0.f ? (float)(g.leaky_alpha * (double)v) : v; break;
          default: break;
        }
        out[k] = v;
      }
      if (row < g.M && col < g.N)
        store_result4(g.c + (long long)row * g.N + col, make_float4(out[0], out[1], out[2], out[3]));
    }
    if (!STAGED) cur = nxt;
  }
}

template <int TN, int KF, bool HALF>
inline int launch_skinny_regs(const SkinnyArgs &g, int column_groups) {
  static int resident = 0;   // workgroups per compute unit at this instantiation's register count
  if (resident == 0) {
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, skinny_gemm_regs<TN, KF, HALF, false>, 256, 0) != hipSuccess || n < 1) {
      (void)hipGetLastError();
      n = 1;
    }
    resident = n;
  }
  // all workgroups resident at once; wavefront w takes row blocks w, w + waves, ...
  const long long blocks = (g.M + 15) / 16;
  long long grid = (blocks + 3) / 4;
  long long cap = (long long)num_cus() * resident / column_groups;
  if (cap < 1) cap = 1;
  if (grid > cap) grid = cap;
  const bool stream_a = (long long)g.M * g.K * 4 >= kSkinnyStreamBytes;
  if constexpr (KF == 2 && !HALF) {
    if (stream_a && g.K == 32 && tuning(kTuneSkinnyStage) != 0) {
      note_kernel("skinny_gemm_regs<%d, 2, false, true, true>", TN);
      TFHIP_LAUNCH((skinny_gemm_regs<TN, 2, false, true, true>
                    <<<dim3((unsigned)grid, (unsigned)column_groups), dim3(256), 0, stream()>>>(g)));
      return kOk;
    }
  }
  note_kernel("skinny_gemm_regs<%d, %d, %s, %s>", TN, KF, HALF ? "true" : "false", stream_a ? "true" : "false");
  if (stream_a) {
    TFHIP_LAUNCH((skinny_gemm_regs<TN, KF, HALF, true>
                  <<<dim3((unsigned)grid, (unsigned)column_groups), dim3(256), 0, stream()>>>(g)));
  } else {
    TFHIP_LAUNCH((skinny_gemm_regs<TN, KF, HALF, false>
                  <<<dim3((unsigned)grid, (unsigned)column_groups), dim3(256), 0, stream()>>>(g)));
  }
  return kOk;
}

// Dispatch over the instantiated k combinations for TN groups of 16 columns per
// wavefront; -1 when there is none.
template <int TN>
inline int launch_skinny_regs_tn(const SkinnyArgs &g, int column_groups) {
  const int kf = g.K / 16, rest = g.K % 16;
  if (rest == 0) {
    if (kf == 1) return launch_skinny_regs<TN, 1, false>(g, column_groups);
    if (kf == 2) return launch_skinny_regs<TN, 2, false>(g, column_groups);
  } else if (rest <= 8) {
    if (kf == 0) return launch_skinny_regs<TN, 0, true>(g, column_groups);
    if (kf == 1) return launch_skinny_regs<TN, 1, true>(g, column_groups);
  } else {
    if (kf == 0) return launch_skinny_regs<TN, 1, false>(g, column_groups);
    if (kf == 1) return launch_skinny_regs<TN, 2, false>(g, column_groups);
  }
  return -1;
}

// Instantiated widths in groups of 16 columns (0: too wide).
inline int skinny_groups(int n) {
  const int tn = (n + 15) / 16;
  return tn <= 4 ? tn : (tn <= 6 ? 6 : (tn <= 9 ? 9 : (tn <= 12 ? 12 : 0)));
}

// True when the product fits this kernel: row-major operands, float4-aligned,
// per-column bias with linear / relu / relu6 / leakyrelu, B small enough
// for LDS and enough rows to keep every wavefront streaming.
inline bool skinny_applies(const GemmParams &p, bool transpose_a, bool transpose_b, bool vec) {
  if (transpose_a || transpose_b || !vec || p.batch != 1) return false;
  if (p.K % 4 != 0 || p.N % 4 != 0 || !p.vec_store || p.ldc != p.N) return false;
  if (p.epi.addressing == kConv && !p.vec_store) return false;
  if (!p.epi.channel_operands || p.epi.activation > TFHIP_LEAKYRELU || p.epi.activation == TFHIP_PRELU) return false;
  const int tn = skinny_groups(p.N);
  if (tn == 0 || p.a_bytes == 0) return false;
  // enough 16-row blocks per wavefront to pay for the B fill (a wide B costs more)
  if (p.M < (tn >= 9 ? 98304 : 65536)) return false;
  const long long k_pad = (p.K + kSkinnyChunk - 1) / kSkinnyChunk * kSkinnyChunk;
  return 16LL * tn * (k_pad + kSkinnyPad) * 4 <= 64 * 1024;
}

template <int TN>
inline int launch_skinny_tn(const SkinnyArgs &g) {
  // Workgroups of four wavefronts, three per compute unit, measured best: fatter
  // workgroups fill B fewer times but start later and pipeline less.
  constexpr int WAVES = 4;
  const int blocks = (g.M + 15) / 16;
  const size_t lds = (size_t)16 * TN * (g.k_pad + kSkinnyPad) * sizeof(float);
  long long grid = (blocks + WAVES - 1) / WAVES;
  const long long cap = (long long)num_cus() * 3;
  if (grid > cap) grid = cap;
  const bool stream_a = (long long)g.M * g.K * 4 >= kSkinnyStreamBytes;
  if constexpr (TN <= 2) {
    // A through LDS (instantiated for the k of the wide early projections)
    const int sv = (stream_a && g.K % 16 == 0 && tuning(kTuneSkinnyStage) != 0) ? g.K / 16 : 0;
    const size_t lds_staged = lds + (size_t)WAVES * 16 * (g.K + 4) * sizeof(float);
    if ((sv == 6 || sv == 9 || sv == 12) && lds_staged <= 64 * 1024) {
      long long per_cu = (long long)(160 * 1024) / (long long)lds_staged;
      per_cu = per_cu > 3 ? 3 : per_cu;
      long long staged_grid = (blocks + WAVES - 1) / WAVES;
      if (staged_grid > num_cus() * per_cu) staged_grid = num_cus() * per_cu;
      note_kernel("skinny_gemm<%d, %d, true, %d>", TN, WAVES, sv);
      const dim3 grid3((unsigned)staged_grid), block3(WAVES * 64);
      if (sv == 6) TFHIP_LAUNCH((skinny_gemm<TN, WAVES, true, 6><<<grid3, block3, lds_staged, stream()>>>(g)));
      else if (sv == 9) TFHIP_LAUNCH((skinny_gemm<TN, WAVES, true, 9><<<grid3, block3, lds_staged, stream()>>>(g)));
      else TFHIP_LAUNCH((skinny_gemm<TN, WAVES, true, 12><<<grid3, block3, lds_staged, stream()>>>(g)));
      return kOk;
    }
  }
  note_kernel("skinny_gemm<%d, %d, %s>", TN, WAVES, stream_a ? "true" : "false");
  if (stream_a) {
    TFHIP_LAUNCH((skinny_gemm<TN, WAVES, true><<<dim3((unsigned)grid), dim3(WAVES * 64), lds, stream()>>>(g)));
  } else {
    TFHIP_LAUNCH((skinny_gemm<TN, WAVES, false><<<dim3((unsigned)grid), dim3(WAVES * 64), lds, stream()>>>(g)));
  }
  return kOk;
}

inline int launch_skinny(const GemmParams &p) {
  SkinnyArgs g;
  g.a = p.a; g.b = p.b; g.c = p.c;
  g.bias = p.epi.bias; g.bias_stride = p.epi.bias ? p.epi.bias_s[3] : 0;
  g.leaky_alpha = p.epi.leaky_alpha;
  g.M = p.M; g.N = p.N; g.K = p.K;
  g.k_pad = (p.K + kSkinnyChunk - 1) / kSkinnyChunk * kSkinnyChunk;
  g.a_bytes = p.a_bytes;
  g.activation = p.epi.activation;
  g.residual = p.epi.residual;
  if (tuning(kTuneSkinnyRegs) != 0 && !g.residual) {   // B in registers where an instantiation fits
    // columns per wavefront: all of them up to 96; wider outputs in slices (a
    // wavefront that keeps 144 columns of accumulators, B and bias is so heavy on
    // registers that too few of them are resident to cover each other's stores)
    const int total = skinny_groups(p.N);
    int per_wave = total <= 6 ? total : 3;
    if (tuning(kTuneSkinnyRegs) >= 2) per_wave = tuning(kTuneSkinnyRegs) - 1;   // tuning: value - 1 groups per wavefront
    const int column_groups = (((int)p.N + 15) / 16 + per_wave - 1) / per_wave;
    int rc = -1;
    switch (per_wave) {
      case 1: rc = launch_skinny_regs_tn<1>(g, column_groups); break;
      case 2: rc = launch_skinny_regs_tn<2>(g, column_groups); break;
      case 3: rc = launch_skinny_regs_tn<3>(g, column_groups); break;
      case 4: rc = launch_skinny_regs_tn<4>(g, column_groups); break;
      case 6: rc = launch_skinny_regs_tn<6>(g, column_groups); break;
      case 9: rc = launch_skinny_regs_tn<9>(g, column_groups); break;
      default: break;
    }
    if (rc >= 0) return rc;
  }
  switch (skinny_groups(p.N)) {
    case 1: return launch_skinny_tn<1>(g);
    case 2: return launch_skinny_tn<2>(g);
    case 3: return launch_skinny_tn<3>(g);
    case 4: return launch_skinny_tn<4>(g);
    case 6: return launch_skinny_tn<6>(g);
    case 9: return launch_skinny_tn<9>(g);
    default: return launch_skinny_tn<12>(g);
  }
}

}  // namespace tfhip
