// N-API shim over the C ABI of libtfjs_hip.so (include/tfjs_hip.h): one exported
// JavaScript function per entry point, nothing else. Device buffers cross the
// boundary as plain numbers (the device address; it fits the 53-bit integer
// range of a double). A non-zero status becomes a thrown Error carrying
// tfhip_last_error(), the convention of the reference's Node binding
// (tfjs-node/binding/utils.h:46-94). All calls are synchronous on the main
// thread, as in tfjs-node/binding/tfjs_binding.cc:51-167; kernel entry points
// only enqueue work on the library's stream.
#include <node_api.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "tfjs_hip.h"

namespace {

#define NAPI_OK(call)                                                    \
  do {                                                                   \
    if ((call) != napi_ok) {                                             \
      napi_throw_error(env, nullptr, "tfjs_hip: N-API call failed: " #call); \
      return nullptr;                                                    \
    }                                                                    \
  } while (0)

#define HIP_OK(call)                                        \
  do {                                                      \
    if ((call) != 0) {                                      \
      napi_throw_error(env, nullptr, tfhip_last_error());   \
      return nullptr;                                       \
    }                                                       \
  } while (0)

constexpr size_t kMaxArgs = 32;

struct Args {
  napi_env env;
  size_t argc = kMaxArgs;
  napi_value argv[kMaxArgs];
  bool ok = true;

  Args(napi_env e, napi_callback_info info, size_t expected, const char *name) : env(e) {
    if (napi_get_cb_info(env, info, &argc, argv, nullptr, nullptr) != napi_ok) {
      ok = false;
      napi_throw_error(env, nullptr, "tfjs_hip: cannot read arguments");
    } else if (argc < expected) {
      ok = false;
      char msg[128];
      snprintf(msg, sizeof msg, "tfjs_hip.%s expects %zu arguments, got %zu", name, expected, argc);
      napi_throw_type_error(env, nullptr, msg);
    }
  }

  double num(size_t i) {
    double v = 0;
    if (ok && napi_get_value_double(env, argv[i], &v) != napi_ok) {
      ok = false;
      char msg[96];
      snprintf(msg, sizeof msg, "tfjs_hip: argument %zu must be a number", i);
      napi_throw_type_error(env, nullptr, msg);
    }
    return v;
  }
  int64_t i64(size_t i) { return (int64_t)num(i); }
  int i32(size_t i) { return (int)num(i); }
  // device pointer: a number, or null / undefined for "absent"
  void *ptr(size_t i) {
    if (!ok) return nullptr;
    napi_valuetype t;
    napi_typeof(env, argv[i], &t);
    if (t == napi_null || t == napi_undefined) return nullptr;
    return reinterpret_cast<void *>((uintptr_t)num(i));
  }
  // array of `n` integers (plain array or typed array of numbers)
  bool ints(size_t i, int64_t *out, size_t n) {
    if (!ok) return false;
    napi_valuetype t;
    napi_typeof(env, argv[i], &t);
    if (t == napi_null || t == napi_undefined) {
      for (size_t k = 0; k < n; ++k) out[k] = 0;
      return true;
    }
    // fast path: a Float64Array or Int32Array is read in place (one N-API call)
    bool typed = false;
    if (napi_is_typedarray(env, argv[i], &typed) == napi_ok && typed) {
      napi_typedarray_type type;
      size_t length = 0, offset = 0;
      void *data = nullptr;
      napi_value ab;
      if (napi_get_typedarray_info(env, argv[i], &type, &length, &data, &ab, &offset) != napi_ok ||
          length < n || (type != napi_float64_array && type != napi_int32_array)) {
        ok = false;
        napi_throw_type_error(env, nullptr, "tfjs_hip: expected a Float64Array or Int32Array of sufficient length");
        return false;
      }
      if (type == napi_float64_array) {
        for (size_t k = 0; k < n; ++k) out[k] = (int64_t) static_cast<const double *>(data)[k];
      } else {
        for (size_t k = 0; k < n; ++k) out[k] = static_cast<const int32_t *>(data)[k];
      }
      return true;
    }
    for (uint32_t k = 0; k < n; ++k) {
      napi_value el;
      double v = 0;
      if (napi_get_element(env, argv[i], k, &el) != napi_ok || napi_get_value_double(env, el, &v) != napi_ok) {
        ok = false;
        napi_throw_type_error(env, nullptr, "tfjs_hip: expected an array of numbers");
        return false;
      }
      out[k] = (int64_t)v;
    }
    return true;
  }
  // bytes of a TypedArray, DataView-less ArrayBuffer or Buffer
  bool bytes(size_t i, void **data, size_t *len) {
    if (!ok) return false;
    bool is = false;
    napi_is_typedarray(env, argv[i], &is);
    if (is) {
      napi_typedarray_type type;
      size_t length, offset;
      napi_value ab;
      if (napi_get_typedarray_info(env, argv[i], &type, &length, data, &ab, &offset) != napi_ok) {
        ok = false;
        return false;
      }
      static const size_t width[] = {1, 1, 1, 2, 2, 4, 4, 4, 8, 8, 8};
      *len = length * width[type];
      return true;
    }
    napi_is_arraybuffer(env, argv[i], &is);
    if (is && napi_get_arraybuffer_info(env, argv[i], data, len) == napi_ok) return true;
    ok = false;
    napi_throw_type_error(env, nullptr, "tfjs_hip: expected a TypedArray or ArrayBuffer");
    return false;
  }
};

napi_value make_number(napi_env env, double v) {
  napi_value r;
  napi_create_double(env, v, &r);
  return r;
}

napi_value undefined(napi_env env) {
  napi_value r;
  napi_get_undefined(env, &r);
  return r;
}

napi_value Init(napi_env env, napi_callback_info info) {
  Args a(env, info, 1, "init");
  const int dev = a.i32(0);
  if (!a.ok) return nullptr;
  HIP_OK(tfhip_init(dev));
  return undefined(env);
}

napi_value Shutdown(napi_env env, napi_callback_info) {
  HIP_OK(tfhip_shutdown());
  return undefined(env);
}

napi_value DeviceInfo(napi_env env, napi_callback_info) {
  char name[256] = "", arch[256] = "";
  int cus = 0, clock = 0;
  size_t mem = 0;
  HIP_OK(tfhip_device_info(name, sizeof name, arch, sizeof arch, &cus, &clock, &mem));
  napi_value obj, v;
  NAPI_OK(napi_create_object(env, &obj));
  napi_create_string_utf8(env, name, NAPI_AUTO_LENGTH, &v);
  napi_set_named_property(env, obj, "name", v);
  napi_create_string_utf8(env, arch, NAPI_AUTO_LENGTH, &v);
  napi_set_named_property(env, obj, "arch", v);
  napi_set_named_property(env, obj, "cus", make_number(env, cus));
  napi_set_named_property(env, obj, "clockKhz", make_number(env, clock));
  napi_set_named_property(env, obj, "hbmBytes", make_number(env, (double)mem));
  return obj;
}

napi_value Alloc(napi_env env, napi_callback_info info) {
  Args a(env, info, 1, "alloc");
  const double bytes = a.num(0);
  if (!a.ok) return nullptr;
  void *p = nullptr;
  HIP_OK(tfhip_alloc((size_t)bytes, &p));
  return make_number(env, (double)(uintptr_t)p);
}

napi_value Free(napi_env env, napi_callback_info info) {
  Args a(env, info, 1, "free");
  void *p = a.ptr(0);
  if (!a.ok) return nullptr;
  HIP_OK(tfhip_free(p));
  return undefined(env);
}

// upload(dst, dstOffset, data[, srcByteOffset, byteLength])
napi_value Upload(napi_env env, napi_callback_info info) {
  Args a(env, info, 3, "upload");
  void *dst = a.ptr(0);
  const size_t off = (size_t)a.num(1);
  void *data = nullptr;
  size_t len = 0;
  if (!a.bytes(2, &data, &len)) return nullptr;
  size_t src_off = 0;
  if (a.argc > 4) {
    src_off = (size_t)a.num(3);
    const size_t want = (size_t)a.num(4);
    if (!a.ok) return nullptr;
    if (src_off + want > len) {
      napi_throw_range_error(env, nullptr, "tfjs_hip.upload: source range exceeds the buffer");
      return nullptr;
    }
    len = want;
  }
  if (!a.ok) return nullptr;
  HIP_OK(tfhip_upload(dst, off, static_cast<char *>(data) + src_off, len));
  return undefined(env);
}

// download(src, srcOffset, typedArray): fills typedArray, blocks until done
napi_value Download(napi_env env, napi_callback_info info) {
  Args a(env, info, 3, "download");
  void *src = a.ptr(0);
  const size_t off = (size_t)a.num(1);
  void *data = nullptr;
  size_t len = 0;
  if (!a.bytes(2, &data, &len) || !a.ok) return nullptr;
  HIP_OK(tfhip_download(data, src, off, len));
  return a.argv[2];
}

napi_value Sync(napi_env env, napi_callback_info) {
  HIP_OK(tfhip_sync());
  return undefined(env);
}

napi_value MemoryInfo(napi_env env, napi_callback_info) {
  size_t live = 0, live_bytes = 0, pooled = 0;
  HIP_OK(tfhip_memory_info(&live, &live_bytes, &pooled));
  napi_value obj;
  NAPI_OK(napi_create_object(env, &obj));
  napi_set_named_property(env, obj, "live", make_number(env, (double)live));
  napi_set_named_property(env, obj, "liveBytes", make_number(env, (double)live_bytes));
  napi_set_named_property(env, obj, "pooledBytes", make_number(env, (double)pooled));
  return obj;
}

napi_value WorkspaceInfo(napi_env env, napi_callback_info) {
  size_t bytes = 0, allocations = 0;
  int splits = 0;
  HIP_OK(tfhip_workspace_info(&bytes, &allocations, &splits));
  napi_value obj;
  NAPI_OK(napi_create_object(env, &obj));
  napi_set_named_property(env, obj, "bytes", make_number(env, (double)bytes));
  napi_set_named_property(env, obj, "allocations", make_number(env, (double)allocations));
  napi_set_named_property(env, obj, "lastSplits", make_number(env, (double)splits));
  return obj;
}

napi_value EventRecord(napi_env env, napi_callback_info info) {
  Args a(env, info, 1, "eventRecord");
  const int slot = a.i32(0);
  if (!a.ok) return nullptr;
  HIP_OK(tfhip_event_record(slot));
  return undefined(env);
}

napi_value EventElapsed(napi_env env, napi_callback_info info) {
  Args a(env, info, 2, "eventElapsed");
  const int s0 = a.i32(0), s1 = a.i32(1);
  if (!a.ok) return nullptr;
  float ms = 0;
  HIP_OK(tfhip_event_elapsed(s0, s1, &ms));
  return make_number(env, ms);
}

napi_value SetLaunchRepeat(napi_env env, napi_callback_info info) {
  Args a(env, info, 1, "setLaunchRepeat");
  const int n = a.i32(0);
  if (!a.ok) return nullptr;
  HIP_OK(tfhip_set_launch_repeat(n));
  return undefined(env);
}

// setTuning(name, value): overrides a kernel-selection heuristic (value < 0 restores it)
napi_value SetTuning(napi_env env, napi_callback_info info) {
  Args a(env, info, 2, "setTuning");
  char name[64] = "";
  size_t len = 0;
  if (a.ok && napi_get_value_string_utf8(env, a.argv[0], name, sizeof name, &len) != napi_ok) {
    napi_throw_type_error(env, nullptr, "tfjs_hip.setTuning: name must be a string");
    return nullptr;
  }
  const int value = a.i32(1);
  if (!a.ok) return nullptr;
  HIP_OK(tfhip_set_tuning(name, value));
  return undefined(env);
}

napi_value LastKernel(napi_env env, napi_callback_info) {
  char name[256] = "";
  HIP_OK(tfhip_last_kernel(name, sizeof name));
  napi_value v;
  NAPI_OK(napi_create_string_utf8(env, name, NAPI_AUTO_LENGTH, &v));
  return v;
}

// fusedMatMul(a, b, out, batchA, batchB, M, N, K, transposeA, transposeB,
//             bias, biasStrides[3], activation, prelu, preluStrides[3], leakyreluAlpha)
// fusedMatMulNoAlloc: the same arguments, through tfhip_fused_matmul_noalloc.
static napi_value FusedMatMulAny(napi_env env, napi_callback_info info, bool noalloc) {
  Args a(env, info, 16, noalloc ? "fusedMatMulNoAlloc" : "fusedMatMul");
  int64_t bs[3], ps[3];
  a.ints(11, bs, 3);
  a.ints(14, ps, 3);
  const float *pa = (const float *)a.ptr(0), *pb = (const float *)a.ptr(1);
  float *out = (float *)a.ptr(2);
  const int64_t bA = a.i64(3), bB = a.i64(4), M = a.i64(5), N = a.i64(6), K = a.i64(7);
  const int tA = a.i32(8), tB = a.i32(9);
  const float *bias = (const float *)a.ptr(10), *prelu = (const float *)a.ptr(13);
  const int act = a.i32(12);
  const double leaky = a.num(15);
  if (!a.ok) return nullptr;
  if (noalloc) {
    HIP_OK(tfhip_fused_matmul_noalloc(pa, pb, out, bA, bB, M, N, K, tA, tB, bias, bs, act, prelu, ps, leaky));
  } else {
    HIP_OK(tfhip_fused_matmul(pa, pb, out, bA, bB, M, N, K, tA, tB, bias, bs, act, prelu, ps, leaky));
  }
  return undefined(env);
}
napi_value FusedMatMul(napi_env env, napi_callback_info info) { return FusedMatMulAny(env, info, false); }
napi_value FusedMatMulNoAlloc(napi_env env, napi_callback_info info) { return FusedMatMulAny(env, info, true); }

// fusedConv2D(x, filter, y, geom[15], nchw, bias, biasStrides[4], activation, prelu, preluStrides[4], alpha
//             [, residual])   with a residual: tfhip_fused_conv2d_add
// geom = [batch, inH, inW, inC, fH, fW, outC, strideH, strideW, dilH, dilW, padTop, padLeft, outH, outW]
napi_value FusedConv2D(napi_env env, napi_callback_info info) {
  Args a(env, info, 11, "fusedConv2D");
  int64_t g[15], bs[4], ps[4];
  a.ints(3, g, 15);
  a.ints(6, bs, 4);
  a.ints(9, ps, 4);
  const float *x = (const float *)a.ptr(0), *w = (const float *)a.ptr(1);
  float *y = (float *)a.ptr(2);
  const int nchw = a.i32(4), act = a.i32(7);
  const float *bias = (const float *)a.ptr(5), *prelu = (const float *)a.ptr(8);
  const double leaky = a.num(10);
  if (!a.ok) return nullptr;
  const float *residual = a.argc > 11 ? (const float *)a.ptr(11) : nullptr;
  if (!a.ok) return nullptr;
  if (residual) {
    HIP_OK(tfhip_fused_conv2d_add(x, w, y, g[0], g[1], g[2], g[3], g[4], g[5], g[6], g[7], g[8], g[9], g[10], g[11],
                                  g[12], g[13], g[14], nchw, bias, bs, act, prelu, ps, leaky, residual));
    return undefined(env);
  }
  HIP_OK(tfhip_fused_conv2d(x, w, y, g[0], g[1], g[2], g[3], g[4], g[5], g[6], g[7], g[8], g[9], g[10], g[11], g[12],
                            g[13], g[14], nchw, bias, bs, act, prelu, ps, leaky));
  return undefined(env);
}

// fusedDepthwiseConv2D(x, filter, y, geom[15], bias, biasStrides[4], activation, prelu, preluStrides[4], alpha)
// geom as above with chMul in place of outC
napi_value FusedDepthwiseConv2D(napi_env env, napi_callback_info info) {
  Args a(env, info, 10, "fusedDepthwiseConv2D");
  int64_t g[15], bs[4], ps[4];
  a.ints(3, g, 15);
  a.ints(5, bs, 4);
  a.ints(8, ps, 4);
  const float *x = (const float *)a.ptr(0), *w = (const float *)a.ptr(1);
  float *y = (float *)a.ptr(2);
  const float *bias = (const float *)a.ptr(4), *prelu = (const float *)a.ptr(7);
  const int act = a.i32(6);
  const double leaky = a.num(9);
  if (!a.ok) return nullptr;
  HIP_OK(tfhip_fused_depthwise_conv2d(x, w, y, g[0], g[1], g[2], g[3], g[4], g[5], g[6], g[7], g[8], g[9], g[10],
                                      g[11], g[12], g[13], g[14], bias, bs, act, prelu, ps, leaky));
  return undefined(env);
}

// dequantAffine(q, qByteOffset, bits, n, scale, min, out, toInt32)
napi_value DequantAffine(napi_env env, napi_callback_info info) {
  Args a(env, info, 8, "dequantAffine");
  char *q = (char *)a.ptr(0);
  const size_t off = (size_t)a.num(1);
  const int bits = a.i32(2);
  const int64_t n = a.i64(3);
  const double scale = a.num(4), min = a.num(5);
  void *out = a.ptr(6);
  const int to_int = a.i32(7);
  if (!a.ok) return nullptr;
  HIP_OK(tfhip_dequant_affine(q + off, bits, n, scale, min, out, to_int));
  return undefined(env);
}

// dequantF16(q, qByteOffset, n, out)
napi_value DequantF16(napi_env env, napi_callback_info info) {
  Args a(env, info, 4, "dequantF16");
  char *q = (char *)a.ptr(0);
  const size_t off = (size_t)a.num(1);
  const int64_t n = a.i64(2);
  float *out = (float *)a.ptr(3);
  if (!a.ok) return nullptr;
  HIP_OK(tfhip_dequant_f16(q + off, n, out));
  return undefined(env);
}

// add(a, aStrides, b, bStrides, out, outShape[, rank])   (rank = outShape.length <= 6)
napi_value Add(napi_env env, napi_callback_info info) {
  Args a(env, info, 6, "add");
  uint32_t rank = 0;
  if (a.ok && a.argc > 6) {
    rank = (uint32_t)a.i32(6);  // typed arrays: the rank comes as its own argument
  } else if (a.ok && napi_get_array_length(env, a.argv[5], &rank) != napi_ok) {
    napi_throw_type_error(env, nullptr, "tfjs_hip.add: outShape must be an array (or pass the rank)");
    return nullptr;
  }
  if (rank > 6) {
    napi_throw_range_error(env, nullptr, "tfjs_hip.add: rank above 6");
    return nullptr;
  }
  int64_t as[6] = {0}, bs[6] = {0}, shape[6] = {0};
  a.ints(1, as, rank);
  a.ints(3, bs, rank);
  a.ints(5, shape, rank);
  const float *pa = (const float *)a.ptr(0), *pb = (const float *)a.ptr(2);
  float *out = (float *)a.ptr(4);
  if (!a.ok) return nullptr;
  HIP_OK(tfhip_add(pa, as, pb, bs, out, shape, (int)rank));
  return undefined(env);
}

// binary(op, a, aStrides, b, bStrides, out, outShape, rank)   op: 0 add, 1 sub, 2 mul
napi_value Binary(napi_env env, napi_callback_info info) {
  Args a(env, info, 8, "binary");
  const int op = a.i32(0);
  const uint32_t rank = a.ok ? (uint32_t)a.i32(7) : 0;
  if (rank > 6) {
    napi_throw_range_error(env, nullptr, "tfjs_hip.binary: rank above 6");
    return nullptr;
  }
  int64_t as[6] = {0}, bs[6] = {0}, shape[6] = {0};
  a.ints(2, as, rank);
  a.ints(4, bs, rank);
  a.ints(6, shape, rank);
  const float *pa = (const float *)a.ptr(1), *pb = (const float *)a.ptr(3);
  float *out = (float *)a.ptr(5);
  if (!a.ok) return nullptr;
  HIP_OK(tfhip_binary(op, pa, as, pb, bs, out, shape, (int)rank));
  return undefined(env);
}

// unary(activation, x, y, n, leakyreluAlpha)
napi_value Unary(napi_env env, napi_callback_info info) {
  Args a(env, info, 5, "unary");
  const int act = a.i32(0);
  const float *x = (const float *)a.ptr(1);
  float *y = (float *)a.ptr(2);
  const int64_t n = a.i64(3);
  const double alpha = a.num(4);
  if (!a.ok) return nullptr;
  HIP_OK(tfhip_unary(act, x, y, n, alpha));
  return undefined(env);
}

// avgPool(x, y, geom[12] = [batch, inH, inW, c, fH, fW, strideH, strideW, padTop, padLeft, outH, outW])
napi_value AvgPool(napi_env env, napi_callback_info info) {
  Args a(env, info, 3, "avgPool");
  int64_t g[12];
  a.ints(2, g, 12);
  const float *x = (const float *)a.ptr(0);
  float *y = (float *)a.ptr(1);
  if (!a.ok) return nullptr;
  HIP_OK(tfhip_avg_pool(x, y, g[0], g[1], g[2], g[3], g[4], g[5], g[6], g[7], g[8], g[9], g[10], g[11]));
  return undefined(env);
}

// cast(x, fromDtype, y, toDtype, n)   dtypes: 0 float32, 1 int32, 2 bool
napi_value Cast(napi_env env, napi_callback_info info) {
  Args a(env, info, 5, "cast");
  const void *x = a.ptr(0);
  const int from = a.i32(1);
  void *y = a.ptr(2);
  const int to = a.i32(3);
  const int64_t n = a.i64(4);
  if (!a.ok) return nullptr;
  HIP_OK(tfhip_cast(x, from, y, to, n));
  return undefined(env);
}

// transpose2d(x, y, rows, cols)
napi_value Transpose2D(napi_env env, napi_callback_info info) {
  Args a(env, info, 4, "transpose2d");
  const float *x = (const float *)a.ptr(0);
  float *y = (float *)a.ptr(1);
  const int64_t rows = a.i64(2), cols = a.i64(3);
  if (!a.ok) return nullptr;
  HIP_OK(tfhip_transpose2d(x, y, rows, cols));
  return undefined(env);
}

// fusedInvertedResidual(x, pwFilterT, pwBias, activation, dwFilter, dwBias, projFilterT, projBias, residual, y,
//                       geom[11] = [batch, inH, inW, inC, midC, outC, stride, padTop, padLeft, outH, outW])
napi_value FusedInvertedResidual(napi_env env, napi_callback_info info) {
  Args a(env, info, 11, "fusedInvertedResidual");
  int64_t g[11];
  a.ints(10, g, 11);
  const float *x = (const float *)a.ptr(0), *w1 = (const float *)a.ptr(1), *b1 = (const float *)a.ptr(2);
  const int act = a.i32(3);
  const float *w2 = (const float *)a.ptr(4), *b2 = (const float *)a.ptr(5), *w3 = (const float *)a.ptr(6);
  const float *b3 = (const float *)a.ptr(7), *res = (const float *)a.ptr(8);
  float *y = (float *)a.ptr(9);
  if (!a.ok) return nullptr;
  HIP_OK(tfhip_fused_inverted_residual(x, w1, b1, act, w2, b2, w3, b3, res, y, g[0], g[1], g[2], g[3], g[4], g[5], g[6],
                                       g[7], g[8], g[9], g[10]));
  return undefined(env);
}

// invertedResidualPays(batch, inH, inW, inC, midC, outC, stride, outH, outW): boolean
napi_value InvertedResidualPays(napi_env env, napi_callback_info info) {
  Args a(env, info, 9, "invertedResidualPays");
  int64_t v[9];
  for (int i = 0; i < 9; ++i) v[i] = a.i64(i);
  if (!a.ok) return nullptr;
  napi_value out;
  NAPI_OK(napi_get_boolean(env, tfhip_inverted_residual_pays(v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7], v[8]) == 1, &out));
  return out;
}

// filterIsFinite(filter, elems): boolean
napi_value FilterIsFinite(napi_env env, napi_callback_info info) {
  Args a(env, info, 2, "filterIsFinite");
  const float *filter = (const float *)a.ptr(0);
  const int64_t elems = a.i64(1);
  if (!a.ok) return nullptr;
  int finite = 1;
  HIP_OK(tfhip_filter_is_finite(filter, elems, &finite));
  napi_value out;
  NAPI_OK(napi_get_boolean(env, finite == 1, &out));
  return out;
}

// meanHW(x, y, batch, h, w, c)
napi_value MeanHW(napi_env env, napi_callback_info info) {
  Args a(env, info, 6, "meanHW");
  const float *x = (const float *)a.ptr(0);
  float *y = (float *)a.ptr(1);
  const int64_t b = a.i64(2), h = a.i64(3), w = a.i64(4), c = a.i64(5);
  if (!a.ok) return nullptr;
  HIP_OK(tfhip_mean_hw(x, y, b, h, w, c));
  return undefined(env);
}

// fusedPointwiseDepthwise(x, pwFilter, pwBias, pwActivation, dwFilter, dwBias, dwActivation, y,
//                         geom[10] = [batch, inH, inW, inC, midC, stride, padTop, padLeft, outH, outW])
napi_value FusedPointwiseDepthwise(napi_env env, napi_callback_info info) {
  Args a(env, info, 9, "fusedPointwiseDepthwise");
  int64_t g[10];
  a.ints(8, g, 10);
  const float *x = (const float *)a.ptr(0), *w1 = (const float *)a.ptr(1), *b1 = (const float *)a.ptr(2);
  const float *w2 = (const float *)a.ptr(4), *b2 = (const float *)a.ptr(5);
  float *y = (float *)a.ptr(7);
  const int act1 = a.i32(3), act2 = a.i32(6);
  if (!a.ok) return nullptr;
  HIP_OK(tfhip_fused_pointwise_depthwise(x, w1, b1, act1, w2, b2, act2, y, g[0], g[1], g[2], g[3], g[4], g[5], g[6], g[7],
                                         g[8], g[9]));
  return undefined(env);
}

// fusedConv2DDepthwise(x, filter, bias, activation, dwFilter, dwBias, dwActivation, y,
//                      geom[17] = [batch, inH, inW, inC, fH, fW, midC, stride, padTop, padLeft, midH, midW,
//                                  dwStride, dwPadTop, dwPadLeft, outH, outW])
napi_value FusedConv2DDepthwise(napi_env env, napi_callback_info info) {
  Args a(env, info, 9, "fusedConv2DDepthwise");
  int64_t g[17];
  a.ints(8, g, 17);
  const float *x = (const float *)a.ptr(0), *w1 = (const float *)a.ptr(1), *b1 = (const float *)a.ptr(2);
  const float *w2 = (const float *)a.ptr(4), *b2 = (const float *)a.ptr(5);
  float *y = (float *)a.ptr(7);
  const int act1 = a.i32(3), act2 = a.i32(6);
  if (!a.ok) return nullptr;
  HIP_OK(tfhip_fused_conv2d_depthwise(x, w1, b1, act1, w2, b2, act2, y, g[0], g[1], g[2], g[3], g[4], g[5], g[6], g[7],
                                      g[8], g[9], g[10], g[11], g[12], g[13], g[14], g[15], g[16]));
  return undefined(env);
}

// conv2dDepthwisePays(batch, inC, fH, fW, midC, midH, midW, dwStride, outH, outW): boolean
napi_value Conv2DDepthwisePays(napi_env env, napi_callback_info info) {
  Args a(env, info, 10, "conv2dDepthwisePays");
  int64_t v[10];
  for (int i = 0; i < 10; ++i) v[i] = a.i64(i);
  if (!a.ok) return nullptr;
  napi_value r;
  NAPI_OK(napi_get_boolean(env, tfhip_conv2d_depthwise_pays(v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7], v[8], v[9]) == 1,
                           &r));
  return r;
}

// pointwiseDepthwisePays(batch, inC, midC, stride, outH, outW): boolean
napi_value PointwiseDepthwisePays(napi_env env, napi_callback_info info) {
  Args a(env, info, 6, "pointwiseDepthwisePays");
  const int64_t b = a.i64(0), ic = a.i64(1), mc = a.i64(2), s = a.i64(3), oh = a.i64(4), ow = a.i64(5);
  if (!a.ok) return nullptr;
  napi_value r;
  NAPI_OK(napi_get_boolean(env, tfhip_pointwise_depthwise_pays(b, ic, mc, s, oh, ow) == 1, &r));
  return r;
}

// copy(dst, src, bytes): device to device on the library's stream
napi_value Copy(napi_env env, napi_callback_info info) {
  Args a(env, info, 3, "copy");
  void *dst = a.ptr(0), *src = a.ptr(1);
  const double bytes = a.num(2);
  if (!a.ok) return nullptr;
  HIP_OK(tfhip_copy(dst, src, (size_t)bytes));
  return undefined(env);
}

napi_value CaptureBegin(napi_env env, napi_callback_info) {
  HIP_OK(tfhip_capture_begin());
  return undefined(env);
}

// captureEnd(keep): {id, nodes}; keep == false discards the recording (id 0)
napi_value CaptureEnd(napi_env env, napi_callback_info info) {
  Args a(env, info, 1, "captureEnd");
  bool keep = false;
  if (a.ok && napi_get_value_bool(env, a.argv[0], &keep) != napi_ok) {
    napi_throw_type_error(env, nullptr, "tfjs_hip.captureEnd: keep must be a boolean");
    return nullptr;
  }
  if (!a.ok) return nullptr;
  int id = 0, nodes = 0;
  HIP_OK(tfhip_capture_end(keep ? &id : nullptr, &nodes));
  napi_value obj;
  NAPI_OK(napi_create_object(env, &obj));
  napi_set_named_property(env, obj, "id", make_number(env, id));
  napi_set_named_property(env, obj, "nodes", make_number(env, nodes));
  return obj;
}

napi_value GraphLaunch(napi_env env, napi_callback_info info) {
  Args a(env, info, 1, "graphLaunch");
  const int id = a.i32(0);
  if (!a.ok) return nullptr;
  HIP_OK(tfhip_graph_launch(id));
  return undefined(env);
}

napi_value GraphDestroy(napi_env env, napi_callback_info info) {
  Args a(env, info, 1, "graphDestroy");
  const int id = a.i32(0);
  if (!a.ok) return nullptr;
  HIP_OK(tfhip_graph_destroy(id));
  return undefined(env);
}

napi_value Register(napi_env env, napi_value exports) {
  const napi_property_descriptor props[] = {
#define FN(name, fn) {name, nullptr, fn, nullptr, nullptr, nullptr, napi_enumerable, nullptr}
      FN("init", Init),
      FN("shutdown", Shutdown),
      FN("deviceInfo", DeviceInfo),
      FN("alloc", Alloc),
      FN("free", Free),
      FN("upload", Upload),
      FN("download", Download),
      FN("sync", Sync),
      FN("memoryInfo", MemoryInfo),
      FN("workspaceInfo", WorkspaceInfo),
      FN("filterIsFinite", FilterIsFinite),
      FN("eventRecord", EventRecord),
      FN("eventElapsed", EventElapsed),
      FN("setLaunchRepeat", SetLaunchRepeat),
      FN("lastKernel", LastKernel),
      FN("setTuning", SetTuning),
      FN("fusedMatMul", FusedMatMul),
      FN("fusedMatMulNoAlloc", FusedMatMulNoAlloc),
      FN("fusedConv2D", FusedConv2D),
      FN("fusedDepthwiseConv2D", FusedDepthwiseConv2D),
      FN("dequantAffine", DequantAffine),
      FN("dequantF16", DequantF16),
      FN("add", Add),
      FN("meanHW", MeanHW),
      FN("binary", Binary),
      FN("unary", Unary),
      FN("avgPool", AvgPool),
      FN("cast", Cast),
      FN("transpose2d", Transpose2D),
      FN("fusedInvertedResidual", FusedInvertedResidual),
      FN("invertedResidualPays", InvertedResidualPays),
      FN("fusedPointwiseDepthwise", FusedPointwiseDepthwise),
      FN("pointwiseDepthwisePays", PointwiseDepthwisePays),
      FN("fusedConv2DDepthwise", FusedConv2DDepthwise),
      FN("conv2dDepthwisePays", Conv2DDepthwisePays),
      FN("copy", Copy),
      FN("captureBegin", CaptureBegin),
      FN("captureEnd", CaptureEnd),
      FN("graphLaunch", GraphLaunch),
      FN("graphDestroy", GraphDestroy),
#undef FN
  };
  napi_define_properties(env, exports, sizeof props / sizeof props[0], props);
  return exports;
}

}  // namespace

NAPI_MODULE(tfjs_hip, Register)
