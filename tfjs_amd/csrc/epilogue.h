// Fused bias + activation tail shared by the matmul, conv and depthwise kernels.
//
// The reference runs three float32-rounded passes (kernel, broadcasting Add of
// the bias, activation: tfjs-backend-cpu/src/kernels/_FusedMatMul.ts:41-55,
// FusedConv2D.ts:43-92); here the same three roundings happen in registers
// before the single store.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace tfhip {

// How bias / prelu weights are addressed for an output element.
//  kChannel: base[col * s_col] only (rank-1 bias over the last axis, or scalar)
//  kMatmul:  base[batch*s[0] + row*s[1] + col*s[2]]
//  kConv:    row is split into (n, oh, ow): base[n*s[0] + oh*s[1] + ow*s[2] + col*s[3]]
enum EpilogueAddressing { kChannel = 0, kMatmul = 1, kConv = 2 };

struct Epilogue {
  const float *bias;
  const float *prelu;
  long long bias_s[4];
  long long prelu_s[4];
  double leaky_alpha;
  int activation;
  int addressing;
  int channel_operands;  // bias and PReLU weights (if any) are indexed by column alone
  // kConv only: spatial extent of the output for the row split, and the output
  // strides for (n, oh, ow, c) so NCHW outputs can be written in place.
  int out_h, out_w;
  long long y_s[4];
  // Optional tensor of the output's own shape and layout, added to the result
  // after the activation (a residual connection: the Add that follows the
  // convolution in the graph, rounded like that separate float32 Add).
  const float *residual;
};

__device__ __forceinline__ float activate(float v, int act, float alpha, double leaky) {
  switch (act) {
    case TFHIP_RELU:
      // Math.max(0, x): NaN stays NaN, -0 becomes +0 (Relu.ts:22)
      return (v > 0.f || v != v) ? v : 0.f;
    case TFHIP_RELU6: {
      // Math.min(Math.max(0, x), 6) (Relu6.ts:22-23)
      const float t = (v > 0.f || v != v) ? v : 0.f;
      return t > 6.f ? 6.f : t;
    }
    case TFHIP_PRELU:
      // x < 0 ? alpha * x : x (Prelu.ts:24-25)
      return v < 0.f ? alpha * v : v;
    case TFHIP_LEAKYRELU:
      // the reference keeps alpha as a double attribute (LeakyRelu.ts:38-40)
      return v < 0.f ? (float)(leaky * (double)v) : v;
    case TFHIP_SIGMOID:
      // 1 / (1 + exp(-x)) (Sigmoid.ts:25-26)
      return 1.f / (1.f + expf(-v));
    case TFHIP_ELU:
      // x >= 0 ? x : exp(x) - 1 (Elu.ts:22-23)
      return v >= 0.f ? v : expm1f(v);
    default:
      return v;
  }
}

// Index of the bias (which == 0) or PReLU weight (which == 1) that goes with
// output element (batch, row, col); for kConv (n, oh, ow) is the split of row.
__device__ __forceinline__ long long operand_index(const Epilogue &e, int which, long long batch, long long row,
                                                   long long col, long long n, long long oh, long long ow) {
  const long long *s = which == 0 ? e.bias_s : e.prelu_s;
  if (e.addressing == kChannel) return col * s[3];
  if (e.addressing == kMatmul) return batch * s[0] + row * s[1] + col * s[2];
  return n * s[0] + oh * s[1] + ow * s[2] + col * s[3];
}

// Applies bias and activation to `v`, the raw contraction result of output
// element (batch, row, col). For kConv, (n, oh, ow) is the split of `row`.
__device__ __forceinline__ float finish(const Epilogue &e, float v, long long batch,
                                        long long row, long long col, long long n,
                                        long long oh, long long ow) {
  if (e.bias) {
    long long idx;
    if (e.addressing == kChannel) {
      idx = col * e.bias_s[3];
    } else if (e.addressing == kMatmul) {
      idx = batch * e.bias_s[0] + row * e.bias_s[1] + col * e.bias_s[2];
    } else {
      idx = n * e.bias_s[0] + oh * e.bias_s[1] + ow * e.bias_s[2] + col * e.bias_s[3];
    }
    v = v + e.bias[idx];
  }
  float alpha = 0.f;
  if (e.activation == TFHIP_PRELU) {
    long long idx;
    if (e.addressing == kChannel) {
      idx = col * e.prelu_s[3];
    } else if (e.addressing == kMatmul) {
      idx = batch * e.prelu_s[0] + row * e.prelu_s[1] + col * e.prelu_s[2];
    } else {
      idx = n * e.prelu_s[0] + oh * e.prelu_s[1] + ow * e.prelu_s[2] + col * e.prelu_s[3];
    }
    alpha = e.prelu[idx];
  }
  return activate(v, e.activation, alpha, e.leaky_alpha);
}

// The float4 stores the kernels write their results with, in three cache policies. A result is
// written once and read by the next launch, on any of the eight XCDs, whose L2 caches do not see
// each other's dirty lines: what a kernel leaves dirty in its L2 is written back when it ends,
// and that write-back is part of the launch.
//  * store_result4_through: write-through (`sc1`), through a buffer descriptor. The line goes to
//    memory as the store is issued, so nothing is left to write back at the end, and it stays in
//    the memory-side cache, where the reader finds it. The tiled GEMMs, the register-streaming pair
//    kernel and the channel-sliced pair kernel's results below 8 MB (MobileNetV2 at batch 32, in
//    sequence: 473 -> 460 us per inference, writers and readers both faster). It is the
//    compiler's own buffer store with the scope bit set: the same instruction written as inline
//    assembly, which the compiler cannot see into, lost a float4 now and then.
//  * store_result4_streaming: non-temporal. For a result of 8 MB or more that is stored in pieces
//    of cache lines and read once: the channel-sliced pair kernel on its larger maps, where a lane
//    writes 16 bytes of a pixel's 1.5 - 2.3 KB of channels (its eleven launches 177 -> 154 us
//    against cached stores; write-through instead costs those launches 0.7 us each).
//  * store_result4: a plain cached store. The streaming GEMMs: the pair kernels that read their
//    results, every channel block once more, lose 23 us per inference when those come from
//    memory, and write-through costs the larger of them 2 us. Also every result too large for the
//    32-bit offsets of a descriptor.
// TFHIP_NT_OUT is a build-time switch for measurement that makes every result store a streaming
// one.
#ifndef TFHIP_NT_OUT
#define TFHIP_NT_OUT 0
#endif
__device__ __forceinline__ void store_result4_streaming(float *p, float4 v) {
  typedef float result4_t __attribute__((ext_vector_type(4)));
  const result4_t t = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(t, reinterpret_cast<result4_t *>(p));
}
// `byte_offset` is relative to the descriptor's base; an offset beyond its extent drops the store.
__device__ __forceinline__ void store_result4_through(__amdgpu_buffer_rsrc_t rsrc, unsigned byte_offset, float4 v) {
  typedef unsigned int result4_bits __attribute__((ext_vector_type(4)));
  const result4_bits d = {__float_as_uint(v.x), __float_as_uint(v.y), __float_as_uint(v.z), __float_as_uint(v.w)};
  __builtin_amdgcn_raw_buffer_store_b128(d, rsrc, (int)byte_offset, 0, TFHIP_NT_OUT ? 2 : 16);
}
__device__ __forceinline__ void store_result4(float *p, float4 v) {
#if TFHIP_NT_OUT
  store_result4_streaming(p, v);
#else
  *reinterpret_cast<float4 *>(p) = v;
#endif
}

// Workgroup barrier that orders LDS traffic only. __syncthreads() also fences
// global memory, which makes every wave wait for all of its outstanding global
// loads (vmcnt(0)) at each barrier and so drains the prefetch ring once per k
// tile; the tiles exchanged between waves here live in LDS alone.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

}  // namespace tfhip
