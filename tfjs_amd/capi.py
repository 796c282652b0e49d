"""ctypes binding of the C ABI declared in include/tfjs_hip.h.

Loads tfjs_amd/lib/libtfjs_hip.so; raises if it is missing -- there is no CPU
fallback. `check()` turns a non-zero status into HipBackendError carrying
tfhip_last_error().
"""
import ctypes
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libtfjs_hip.so")

ACTIVATIONS = {"linear": 0, "relu": 1, "relu6": 2, "prelu": 3, "leakyrelu": 4, "sigmoid": 5, "elu": 6}

c_i64 = ctypes.c_int64
c_f32p = ctypes.c_void_p
c_i64p = ctypes.POINTER(ctypes.c_int64)

# name -> (argtypes); every entry point returns int except tfhip_last_error
SIGNATURES = {
    "tfhip_init": [ctypes.c_int],
    "tfhip_shutdown": [],
    "tfhip_device_info": [ctypes.c_char_p, ctypes.c_size_t, ctypes.c_char_p, ctypes.c_size_t,
                          ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int),
                          ctypes.POINTER(ctypes.c_size_t)],
    "tfhip_alloc": [ctypes.c_size_t, ctypes.POINTER(ctypes.c_void_p)],
    "tfhip_free": [ctypes.c_void_p],
    "tfhip_upload": [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_size_t],
    "tfhip_download": [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t],
    "tfhip_sync": [],
    "tfhip_copy": [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t],
    "tfhip_set_tuning": [ctypes.c_char_p, ctypes.c_int],
    "tfhip_memory_info": [ctypes.POINTER(ctypes.c_size_t)] * 3,
    "tfhip_filter_is_finite": [c_f32p, c_i64, ctypes.POINTER(ctypes.c_int)],
    "tfhip_workspace_info": [ctypes.POINTER(ctypes.c_size_t)] * 2 + [ctypes.POINTER(ctypes.c_int)],
    "tfhip_register_external": [ctypes.c_void_p, ctypes.c_size_t],
    "tfhip_unregister_external": [ctypes.c_void_p],
    "tfhip_event_record": [ctypes.c_int],
    "tfhip_event_elapsed": [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_float)],
    "tfhip_set_launch_repeat": [ctypes.c_int],
    "tfhip_capture_begin": [],
    "tfhip_capture_end": [ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)],
    "tfhip_graph_launch": [ctypes.c_int],
    "tfhip_graph_destroy": [ctypes.c_int],
    "tfhip_last_kernel": [ctypes.c_char_p, ctypes.c_size_t],
    "tfhip_fused_matmul": [c_f32p, c_f32p, c_f32p, c_i64, c_i64, c_i64, c_i64, c_i64, ctypes.c_int,
                           ctypes.c_int, c_f32p, c_i64p, ctypes.c_int, c_f32p, c_i64p, ctypes.c_double],
    "tfhip_fused_matmul_noalloc": [c_f32p, c_f32p, c_f32p, c_i64, c_i64, c_i64, c_i64, c_i64, ctypes.c_int,
                                   ctypes.c_int, c_f32p, c_i64p, ctypes.c_int, c_f32p, c_i64p, ctypes.c_double],
    "tfhip_fused_conv2d": [c_f32p, c_f32p, c_f32p] + [c_i64] * 15 + [ctypes.c_int, c_f32p, c_i64p,
                                                                      ctypes.c_int, c_f32p, c_i64p,
                                                                      ctypes.c_double],
    "tfhip_fused_conv2d_add": [c_f32p, c_f32p, c_f32p] + [c_i64] * 15 + [ctypes.c_int, c_f32p, c_i64p,
                                                                      ctypes.c_int, c_f32p, c_i64p,
                                                                      ctypes.c_double, c_f32p],
    "tfhip_fused_pointwise_depthwise": [c_f32p, c_f32p, c_f32p, ctypes.c_int, c_f32p, c_f32p, ctypes.c_int, c_f32p] +
                                       [c_i64] * 10,
    "tfhip_pointwise_depthwise_pays": [c_i64] * 6,
    "tfhip_fused_conv2d_depthwise": [c_f32p, c_f32p, c_f32p, ctypes.c_int, c_f32p, c_f32p, ctypes.c_int, c_f32p] +
                                    [c_i64] * 17,
    "tfhip_conv2d_depthwise_pays": [c_i64] * 10,
    "tfhip_fused_depthwise_conv2d": [c_f32p, c_f32p, c_f32p] + [c_i64] * 15 + [c_f32p, c_i64p, ctypes.c_int,
                                                                                c_f32p, c_i64p, ctypes.c_double],
    "tfhip_fused_inverted_residual": [c_f32p, c_f32p, c_f32p, ctypes.c_int, c_f32p, c_f32p, c_f32p, c_f32p, c_f32p, c_f32p] +
                                     [c_i64] * 11,
    "tfhip_inverted_residual_pays": [c_i64] * 9,
    "tfhip_transpose2d": [c_f32p, c_f32p, c_i64, c_i64],
    "tfhip_dequant_affine": [ctypes.c_void_p, ctypes.c_int, c_i64, ctypes.c_double, ctypes.c_double,
                             ctypes.c_void_p, ctypes.c_int],
    "tfhip_dequant_f16": [ctypes.c_void_p, c_i64, ctypes.c_void_p],
    "tfhip_add": [c_f32p, c_i64p, c_f32p, c_i64p, c_f32p, c_i64p, ctypes.c_int],
    "tfhip_mean_hw": [c_f32p, c_f32p, c_i64, c_i64, c_i64, c_i64],
    "tfhip_binary": [ctypes.c_int, c_f32p, c_i64p, c_f32p, c_i64p, c_f32p, c_i64p, ctypes.c_int],
    "tfhip_unary": [ctypes.c_int, c_f32p, c_f32p, c_i64, ctypes.c_double],
    "tfhip_avg_pool": [c_f32p, c_f32p] + [c_i64] * 12,
    "tfhip_cast": [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int, c_i64],
}


class HipBackendError(RuntimeError):
    pass


_lib = None


def load_library():
    """Loads the shared library and declares every entry point's signature."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise HipBackendError(
                "%s is missing: build it with `python -m tfjs_amd.build` (there is no CPU fallback)" % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, argtypes in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = ctypes.c_int
        lib.tfhip_last_error.argtypes = []
        lib.tfhip_last_error.restype = ctypes.c_char_p
        _lib = lib
    return _lib


def check(status):
    if status != 0:
        raise HipBackendError(load_library().tfhip_last_error().decode("utf-8", "replace"))


def i64_array(values):
    return (ctypes.c_int64 * max(1, len(values)))(*[int(v) for v in values])


class DeviceBuffer:
    """A block of device memory from the library's pool."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        ptr = ctypes.c_void_p()
        check(load_library().tfhip_alloc(max(1, self.nbytes), ctypes.byref(ptr)))
        self.ptr = ptr.value

    @classmethod
    def from_numpy(cls, array):
        array = np.ascontiguousarray(array)
        buf = cls(array.nbytes)
        buf.upload(array)
        return buf

    def upload(self, array, offset=0):
        array = np.ascontiguousarray(array)
        check(load_library().tfhip_upload(self.ptr, offset, array.ctypes.data, array.nbytes))

    def download(self, dtype, count, offset=0):
        out = np.empty(int(count), dtype=dtype)
        check(load_library().tfhip_download(out.ctypes.data, self.ptr, offset, out.nbytes))
        return out

    def free(self):
        if self.ptr is not None:
            check(load_library().tfhip_free(self.ptr))
            self.ptr = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.free()
