// Pointwise (1x1) convolution + depthwise 3x3 convolution in one kernel, for the
// blocks whose feature map is small (56x56 and below) and whose expanded tensor is
// wide (up to 960 channels): the workgroups split the EXPANDED CHANNELS.
//
// Both stages are separable the way this split needs: a column of the expansion's
// weights produces one expanded channel from all input channels, and the
// depthwise stage works on every channel on its own. So a workgroup that owns
// `cs` expanded channels (a "slice") of one image tile computes exactly its share
// of both stages: nothing is computed twice except the tile's halo rows, and the
// expanded tensor never reaches memory.
//
//   grid       x: (image, chunk of output rows)   y: channel slice
//   LDS        the slice of the expanded tile [erows][ecols][cs + 4] (tile + the
//              halo the 3x3 windows reach into; positions outside the image hold
//              the zeros the depthwise stage pads with), and the slice of the
//              expansion's weights, transposed [cs][K + 4]
//   phase 1    expansion on the matrix cores: blocks of 16 pixels of the tile that
//              lie inside the image, dealt to the four waves in turn; a block's A
//              operand (16 pixels x K input channels) comes straight from memory in
//              the instruction's register layout, fetched one block ahead; the
//              cs / 16 column blocks of a pixel block are independent accumulator
//              chains that interleave in the matrix pipe; bias-initialised, k
//              ascending, relu / relu6, one 16-byte LDS store per lane and block
//   phase 2    depthwise stage from LDS: (output pixel, four channels) items dealt
//              to the lanes, nine independent 16-byte LDS reads each; taps from
//              zero by row then column, then bias, then the activation: the order
//              of the stand-alone kernels
//
// The instruction order of both stages is that of gemm_kernel (k = 16 t + 4 g + j
// for the j-th instruction of k group t) and of the depthwise kernels, so the
// result has the bits of the two separate launches.
#include "common.h"
#include "epilogue.h"
#include "expand_dw_tile.h"

namespace tfhip {
namespace {

typedef float float4_t __attribute__((ext_vector_type(4)));
constexpr unsigned kNoOff = 0xffffffffu;   // an offset no buffer descriptor covers: loads return 0

__device__ __forceinline__ float relu_cap(float v, float cap) {
  const float t = (v > 0.f || v != v) ? v : 0.f;     // Math.max(0, x): NaN stays, -0 becomes +0
  return t > cap ? cap : t;                          // cap = 6 for relu6, +inf for relu
}

// S: stride of the depthwise stage. K = 16 KF + (HALF ? 8 : 0) input channels.
// NCB: blocks of 16 channels per slice.
template <int S, int KF, bool HALF, int NCB>
__global__ __launch_bounds__(256) void expand_dw_tile(ExpandDwTileArgs g) {
  constexpr int K = 16 * KF + (HALF ? 8 : 0);
  constexpr int KP = K + 4;              // floats per column of the transposed weights
  constexpr int CS = 16 * NCB;
  constexpr int PITCH = CS + 4;          // floats per position of the expanded tile
  extern __shared__ float lds[];
  float *tile = lds;                                   // [erows][ecols][PITCH]
  float *w1t = lds + g.erows * g.ecols * PITCH;        // [CS][KP]

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int grp = lane >> 4, r = lane & 15;
  const int chunk = blockIdx.x % g.chunks_h, n = blockIdx.x / g.chunks_h;
  const int c0 = blockIdx.y * CS;                      // first expanded channel of the slice
  const int oh0 = chunk * g.rows;
  const int rows = oh0 + g.rows <= g.out_h ? g.rows : g.out_h - oh0;
  const int erows = (rows - 1) * S + 3;                // expanded rows this chunk reads
  const int ih0 = oh0 * S - g.pad_top, iw0 = -g.pad_left;   // image position of tile position (0, 0)
  // the part of the tile that lies inside the image
  const int ih_lo = ih0 < 0 ? 0 : ih0, ih_hi = ih0 + erows < g.in_h ? ih0 + erows : g.in_h;
  const int iw_lo = iw0 < 0 ? 0 : iw0, iw_hi = iw0 + g.ecols < g.in_w ? iw0 + g.ecols : g.in_w;
  const int wi = iw_hi > iw_lo ? iw_hi - iw_lo : 0;
  const int inside = ih_hi > ih_lo ? (ih_hi - ih_lo) * wi : 0;
  const int mblocks = (inside + 15) / 16;
  const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc((void *)g.x, 0, (int)g.x_bytes, 0x00020000);

  struct AFrag {
    float4 full[KF > 0 ? KF : 1];
    float2 half;
  };
  // pixel r of block mb: its byte offset in x and its position in the tile (-1: past the last pixel)
  auto locate = [&](int mb, unsigned &x_off, int &pos) __attribute__((always_inline)) {
    const int m = 16 * mb + r;
    if (m < inside) {
      const int rr = m / wi, cc = m - rr * wi;
      const int ih = ih_lo + rr, iw = iw_lo + cc;
      x_off = (unsigned)((((long long)n * g.in_h + ih) * g.in_w + iw) * K * 4);
      pos = (ih - ih0) * g.ecols + (iw - iw0);
    } else {
      x_off = kNoOff;
      pos = -1;
    }
  };
  auto load_a = [&](AFrag &a, unsigned x_off) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < KF; ++t) {
      const auto v = __builtin_amdgcn_raw_buffer_load_b128(rx, (int)(x_off != kNoOff ? x_off + (16 * t + 4 * grp) * 4 : kNoOff), 0, 0);
      a.full[t] = make_float4(__uint_as_float(v[0]), __uint_as_float(v[1]), __uint_as_float(v[2]), __uint_as_float(v[3]));
    }
    if (HALF) {
      const auto v = __builtin_amdgcn_raw_buffer_load_b64(rx, (int)(x_off != kNoOff ? x_off + (16 * KF + 2 * grp) * 4 : kNoOff), 0, 0);
      a.half = make_float2(__uint_as_float(v[0]), __uint_as_float(v[1]));
    }
  };

  // ---- prologue: every operand fetch is issued before anything waits for one of them, so that the
  // workgroup pays one memory round trip, with the LDS set-up done while it is under way. (Issued
  // one after the other, each behind a wait for the one before - the weights, then this wave's
  // first pixels, then the depthwise operands behind the barrier's full wait - they cost three.)
  // The slice of the expansion's weights: w1 is [K][c], 16-byte loads along the channels.
  constexpr int quads = CS / 4, total = quads * K, NV = (total + 255) / 256;
  float4 wv[NV];
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    const int i = tid + u * 256;
    const int ii = i < total ? i : total - 1;
    const int k = ii / quads, col = 4 * (ii - k * quads);
    wv[u] = *reinterpret_cast<const float4 *>(g.w1 + (long long)k * g.c + c0 + col);
  }
  // first pixel block of this wave
  AFrag a_cur, a_next;
  unsigned off_cur = kNoOff, off_next = kNoOff;
  int pos_cur = -1, pos_next = -1;
  if (wave < mblocks) locate(wave, off_cur, pos_cur);
  load_a(a_cur, off_cur);   // (no block: every offset is out of range, nothing is read)
  // this lane's biases of the expansion: channels 16 cb + 4 grp .. +3 of the slice
  float4_t bias1[NCB];
#pragma unroll
  for (int cb = 0; cb < NCB; ++cb) {
    bias1[cb] = {0.f, 0.f, 0.f, 0.f};
    if (g.b1) {
      const float4 b = *reinterpret_cast<const float4 *>(g.b1 + c0 + 16 * cb + 4 * grp);
      bias1[cb] = {b.x, b.y, b.z, b.w};
    }
  }
  // depthwise stage: this lane's four channels, its weights and bias (the lanes left over when the
  // channel quads do not divide 256 fetch like the others and sit the phase out)
  constexpr int CQ = CS / 4, SLOTS = 256 / CQ;   // lanes along the channels, output pixels served at once
  const int c4 = tid % CQ, slot = tid / CQ;
  const bool dw_lane = slot < SLOTS;
  float4 w2q[9], b2q = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (int t = 0; t < 9; ++t) w2q[t] = *reinterpret_cast<const float4 *>(g.w2 + (long long)t * g.c + c0 + 4 * c4);
  if (g.b2) b2q = *reinterpret_cast<const float4 *>(g.b2 + c0 + 4 * c4);

  // tile positions outside the image: the zero padding of the depthwise stage
  {
    const int positions = erows * g.ecols;
    for (int p = tid; p < positions; p += 256) {
      const int er = p / g.ecols, ec = p - er * g.ecols;
      const int ih = ih0 + er, iw = iw0 + ec;
      if (ih < 0 || ih >= g.in_h || iw < 0 || iw >= g.in_w) {
        float4 *dst = reinterpret_cast<float4 *>(tile + p * PITCH);
#pragma unroll
        for (int q = 0; q < CS / 4; ++q) dst[q] = make_float4(0.f, 0.f, 0.f, 0.f);
      }
    }
  }
  // the weights, transposed, into LDS (they were fetched first: the wait leaves the later fetches in flight)
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    const int i = tid + u * 256;
    if (i < total) {
      const int k = i / quads, col = 4 * (i - k * quads);
      w1t[(col + 0) * KP + k] = wv[u].x;
      w1t[(col + 1) * KP + k] = wv[u].y;
      w1t[(col + 2) * KP + k] = wv[u].z;
      w1t[(col + 3) * KP + k] = wv[u].w;
    }
  }
  lds_barrier();   // w1t and the zeros; nobody waits for a fetch here

  // ---- phase 1: the expanded tile
  const float *wcol = w1t + r * KP + 4 * grp;
  for (int mb = wave; mb < mblocks; mb += 4) {
    if (mb + 4 < mblocks) {
      locate(mb + 4, off_next, pos_next);
      load_a(a_next, off_next);
    }
    float4_t acc[NCB];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) acc[cb] = bias1[cb];
#pragma unroll
    for (int t = 0; t < KF; ++t) {
      float4 b[NCB];
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) b[cb] = *reinterpret_cast<const float4 *>(wcol + 16 * cb * KP + 16 * t);
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[cb].x, a_cur.full[t].x, acc[cb], 0, 0, 0);
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[cb].y, a_cur.full[t].y, acc[cb], 0, 0, 0);
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[cb].z, a_cur.full[t].z, acc[cb], 0, 0, 0);
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[cb].w, a_cur.full[t].w, acc[cb], 0, 0, 0);
    }
    if (HALF) {
      float2 b[NCB];
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) b[cb] = *reinterpret_cast<const float2 *>(w1t + (16 * cb + r) * KP + 16 * KF + 2 * grp);
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[cb].x, a_cur.half.x, acc[cb], 0, 0, 0);
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[cb].y, a_cur.half.y, acc[cb], 0, 0, 0);
    }
    // the lane holds pixel r of the block, channels 16 cb + 4 grp .. +3 of the slice
    if (pos_cur >= 0) {
      float *dst = tile + pos_cur * PITCH + 4 * grp;
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) {
        float4 e;
        e.x = relu_cap(acc[cb][0], g.cap);
        e.y = relu_cap(acc[cb][1], g.cap);
        e.z = relu_cap(acc[cb][2], g.cap);
        e.w = relu_cap(acc[cb][3], g.cap);
        *reinterpret_cast<float4 *>(dst + 16 * cb) = e;
      }
    }
    a_cur = a_next;
    off_cur = off_next;
    pos_cur = pos_next;
  }
  lds_barrier();

  // ---- phase 2: depthwise stage from the tile. (output pixel, four channels) items are dealt to
  // the lanes; an item's nine 16-byte reads are independent, so they travel together.
  // (this image's part of the result, for the write-through stores)
  const __amdgpu_buffer_rsrc_t rsrc_y = __builtin_amdgcn_make_buffer_rsrc(
      (void *)(g.y + (long long)n * g.out_h * g.out_w * g.c), 0, (int)((unsigned)g.out_h * g.out_w * g.c * 4u), 0x00020000);
  if (dw_lane) {
    const int items = rows * g.out_w;
    for (int it = slot; it < items; it += SLOTS) {
      const int o = it / g.out_w, q = it - o * g.out_w;
      const float *win = tile + ((S * o) * g.ecols + S * q) * PITCH + 4 * c4;
      float4 e[9];
#pragma unroll
      for (int wr = 0; wr < 3; ++wr) {
#pragma unroll
        for (int wc = 0; wc < 3; ++wc) e[wr * 3 + wc] = *reinterpret_cast<const float4 *>(win + (wr * g.ecols + wc) * PITCH);
      }
      float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int t = 0; t < 9; ++t) {
        acc.x = fmaf(e[t].x, w2q[t].x, acc.x);
        acc.y = fmaf(e[t].y, w2q[t].y, acc.y);
        acc.z = fmaf(e[t].z, w2q[t].z, acc.z);
        acc.w = fmaf(e[t].w, w2q[t].w, acc.w);
      }
      float4 out;
      out.x = relu_cap(acc.x + b2q.x, g.cap);
      out.y = relu_cap(acc.y + b2q.y, g.cap);
      out.z = relu_cap(acc.z + b2q.z, g.cap);
      out.w = relu_cap(acc.w + b2q.w, g.cap);
      if (g.stream_out) {
        store_result4_streaming(g.y + (((long long)n * g.out_h + oh0 + o) * g.out_w + q) * g.c + c0 + 4 * c4, out);
      } else {
        store_result4_through(rsrc_y, (unsigned)(((oh0 + o) * g.out_w + q) * g.c + c0 + 4 * c4) * 4u, out);
      }
    }
  }
}

template <int S, int KF, bool HALF, int NCB>
int launch_tile(const ExpandDwTileArgs &g, size_t lds_bytes) {
  // dynamic LDS above the default limit needs the attribute once per instantiation and device set-up
  static int raised = 0;
  if (raised != init_count()) {
    TFHIP_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(expand_dw_tile<S, KF, HALF, NCB>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    raised = init_count();
  }
  note_kernel("expand_dw_tile<%d, %d, %s, %d>", S, KF, HALF ? "true" : "false", NCB);
  const dim3 grid((unsigned)(g.batch * g.chunks_h), (unsigned)g.slices);
  TFHIP_LAUNCH((expand_dw_tile<S, KF, HALF, NCB><<<grid, dim3(256), lds_bytes, stream()>>>(g)));
  return kOk;
}

template <int S, int KF, bool HALF>
int launch_tile_ncb(const ExpandDwTileArgs &g, size_t lds_bytes) {
  switch (g.cs / 16) {
    case 2: return launch_tile<S, KF, HALF, 2>(g, lds_bytes);
    case 3: return launch_tile<S, KF, HALF, 3>(g, lds_bytes);
    default: return launch_tile<S, KF, HALF, 4>(g, lds_bytes);
  }
}

template <int S>
int launch_tile_k(const ExpandDwTileArgs &g, size_t lds_bytes) {
  switch (g.cin) {
    case 16: return launch_tile_ncb<S, 1, false>(g, lds_bytes);
    case 24: return launch_tile_ncb<S, 1, true>(g, lds_bytes);
    case 32: return launch_tile_ncb<S, 2, false>(g, lds_bytes);
    case 64: return launch_tile_ncb<S, 4, false>(g, lds_bytes);
    case 96: return launch_tile_ncb<S, 6, false>(g, lds_bytes);
    default: return launch_tile_ncb<S, 10, false>(g, lds_bytes);
  }
}

}  // namespace

bool expand_dw_tile_takes_k(int cin) { return cin == 16 || cin == 24 || cin == 32 || cin == 64 || cin == 96 || cin == 160; }

// Tiling, fitted to sweeps over MobileNetV2's blocks at batch 32: slices of 48 channels where they
// divide the expanded channels (two workgroups then fit a compute unit at the 14x14 maps), 64 on
// the smallest maps (a slice's weights are staged once per workgroup, and there a workgroup has
// few pixels to spend them on), else 64 or 32; then row chunks (two halo rows recomputed by each)
// until the launch has two workgroups per compute unit, but no chunk shorter than seven rows (four
// at stride 2).
// Results of at least this many bytes are stored non-temporally, smaller ones written through
// (measured at batch 32: the 9.6 and 14.4 MB maps lose 0.7 and 0.4 us per launch to write-through,
// the 3.6 - 6 MB ones nothing, and the projections that read those get 0.7 us faster each).
constexpr long long kTileStreamBytes = 8LL << 20;

bool plan_expand_dw_tile(ExpandDwTileArgs &g, size_t *lds_bytes) {
  if (!expand_dw_tile_takes_k(g.cin) || g.c % 16 != 0 || (g.stride != 1 && g.stride != 2)) return false;
  if (g.out_h <= 0 || g.out_w <= 0) return false;
  const int forced_cs = tuning(kTuneTileSlice);
  int cs = 0;
  if (forced_cs == 32 || forced_cs == 48 || forced_cs == 64) {
    if (g.c % forced_cs != 0) return false;
    cs = forced_cs;
  } else if (g.out_h * g.stride <= 8 && g.c % 64 == 0) {
    cs = 64;
  } else {
    cs = g.c % 48 == 0 ? 48 : (g.c % 64 == 0 ? 64 : (g.c % 32 == 0 ? 32 : 0));
  }
  if (cs == 0) return false;
  g.cs = cs;
  g.slices = g.c / cs;
  g.ecols = (g.out_w - 1) * g.stride + 3;
  const size_t w_floats = (size_t)cs * (g.cin + 4);
  auto rows_for = [&](int chunks) { return (g.out_h + chunks - 1) / chunks; };
  auto bytes_for = [&](int rows) { return ((size_t)((rows - 1) * g.stride + 3) * g.ecols * (cs + 4) + w_floats) * sizeof(float); };
  const size_t lds_limit = 156 * 1024;
  int chunks = 1;
  const int forced_chunks = tuning(kTuneTileChunks);
  if (forced_chunks > 0) {
    chunks = forced_chunks > g.out_h ? g.out_h : forced_chunks;
  } else {
    while (chunks < g.out_h && bytes_for(rows_for(chunks)) > lds_limit) ++chunks;
    const long long want = 2LL * num_cus();
    // (a stride-2 chunk reads 2 rows + 1 input rows, one of them again: chunks down to four rows still pay
    // there - 14x14 / 576 channels 15.0 -> 14.1 us, 28x28 / 192 channels 10.2 -> 9.9 us at batch 32)
    const int min_rows = g.stride == 2 ? 4 : 7;
    while ((long long)g.batch * g.slices * chunks < want && rows_for(chunks + 1) >= min_rows) ++chunks;
  }
  g.rows = rows_for(chunks);
  g.chunks_h = (g.out_h + g.rows - 1) / g.rows;
  g.erows = (g.rows - 1) * g.stride + 3;
  const long long image_bytes = (long long)g.out_h * g.out_w * g.c * 4;
  g.stream_out = (g.batch * image_bytes >= kTileStreamBytes || image_bytes > 0xfffffff0LL) ? 1 : 0;
  *lds_bytes = bytes_for(g.rows);
  return *lds_bytes <= lds_limit;
}

int launch_expand_dw_tile(const ExpandDwTileArgs &g, size_t lds_bytes) {
  if ((long long)g.batch * g.chunks_h > 0x7fffffffLL || g.slices > 65535)
    return fail(kBadArgument, "tfhip_fused_pointwise_depthwise: grid too large");
  return g.stride == 1 ? launch_tile_k<1>(g, lds_bytes) : launch_tile_k<2>(g, lds_bytes);
}

}  // namespace tfhip
