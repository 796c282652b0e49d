"""tfjs-backend-hip: MI355X-native kernels for the tfjs fused-op hot path.

  csrc/    HIP kernels and the C ABI (include/tfjs_hip.h) -> lib/libtfjs_hip.so
  js/      the tfjs backend package (KernelBackend + kernel configs + N-API addon)
  capi.py  ctypes binding of the C ABI
  pyhost.py numpy-level mirror of the kernel interfaces, used by tests and bench
"""
from .capi import HipBackendError, load_library  # noqa: F401
