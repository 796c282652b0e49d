"""tfhip_fused_matmul_noalloc against tfhip_fused_matmul through the C ABI.

The entry point keeps split-K partial sums in a static device array instead of
the library's allocated workspace; the two must agree bit for bit when they cut
K into the same slices. Two calls in a row share the array, the second with a
smaller input, so stale partial sums of the first call would show in the second.

What "allocates nothing" means is checked on the library's own books
(tfhip_workspace_info: size of its scratch block and the hipMalloc calls made for
it, which tfhip_memory_info does not count) after a shutdown / init, so that no
earlier test has grown the block: the no-alloc calls leave it at zero
allocations while their launches did run with several K slices, and the same
product through tfhip_fused_matmul then does allocate it."""
import ctypes

import numpy as np
import pytest

from tfjs_amd import capi, pyhost as hip
from tfjs_amd.capi import DeviceBuffer, check, i64_array

pytestmark = pytest.mark.gpu


def _run(entry, a, b, bias, m, n, k, activation):
    lib = capi.load_library()
    da, db, dbias = DeviceBuffer.from_numpy(a), DeviceBuffer.from_numpy(b), DeviceBuffer.from_numpy(bias)
    dout = DeviceBuffer(m * n * 4)
    try:
        check(getattr(lib, entry)(da.ptr, db.ptr, dout.ptr, 1, 1, m, n, k, 0, 0, dbias.ptr, i64_array([0, 0, 1]),
                                  capi.ACTIVATIONS[activation], None, i64_array([0, 0, 0]), 0.2))
        name = ctypes.create_string_buffer(256)
        check(lib.tfhip_last_kernel(name, 256))
        splits = hip.workspace_info()["last_splits"]
        return dout.download(np.float32, m * n), name.value.decode(), splits
    finally:
        for buf in (da, db, dbias, dout):
            buf.free()


def _fresh_library():
    """The library without a scratch block: whatever earlier tests made it allocate is gone."""
    lib = capi.load_library()
    hip.init(0)
    hip.shutdown()
    hip.init(0)
    info = hip.workspace_info()
    assert info["bytes"] == 0 and info["allocations"] == 0, info
    return lib


def test_noalloc_matmul_matches_the_allocating_entry_point_twice():
    lib = _fresh_library()
    rng = np.random.default_rng(7)
    check(lib.tfhip_set_tuning(b"splitk", 4))    # partial sums of four K slices go through the scratch
    try:
        cases = [(192, 160, 2048, "relu"), (64, 96, 1024, "linear")]
        operands, got = [], []
        for (m, n, k, act) in cases:
            a = rng.standard_normal((m, k)).astype(np.float32)
            b = rng.standard_normal((k, n)).astype(np.float32)
            bias = rng.standard_normal((n,)).astype(np.float32)
            operands.append((a, b, bias))
            before = hip.memory_info()
            out, kernel, splits = _run("tfhip_fused_matmul_noalloc", a, b, bias, m, n, k, act)
            after = hip.memory_info()
            assert splits == 4, "the launch did not go through the scratch array"
            assert (after["live"], after["live_bytes"]) == (before["live"], before["live_bytes"])
            got.append((out, kernel))
        # two calls through the static array, the second smaller: the library has allocated no scratch
        info = hip.workspace_info()
        assert info["bytes"] == 0 and info["allocations"] == 0, info
        for (m, n, k, act), (a, b, bias), (out, kernel) in zip(cases, operands, got):
            want, kernel_want, splits = _run("tfhip_fused_matmul", a, b, bias, m, n, k, act)
            assert splits == 4 and kernel == kernel_want
            np.testing.assert_array_equal(out.view(np.uint32), want.view(np.uint32))
            ref = np.maximum(a.astype(np.float64) @ b + bias, 0 if act == "relu" else -np.inf).reshape(-1)
            assert np.max(np.abs(out - ref) / np.maximum(1.0, np.abs(ref))) <= 1e-3
        # ... and the allocating entry point did allocate for the same products
        info = hip.workspace_info()
        assert info["allocations"] >= 1 and info["bytes"] >= 4 * 192 * 160 * 4, info
    finally:
        check(lib.tfhip_set_tuning(b"splitk", -1))


def test_noalloc_matmul_without_forced_slices_and_size_limit():
    lib = _fresh_library()
    rng = np.random.default_rng(8)
    # the library's own choice (a long K over few tiles is cut into slices)
    m, n, k = 64, 64, 6144
    a = rng.standard_normal((m, k)).astype(np.float32)
    b = rng.standard_normal((k, n)).astype(np.float32)
    bias = np.zeros((n,), np.float32)
    got, _, splits = _run("tfhip_fused_matmul_noalloc", a, b, bias, m, n, k, "linear")
    assert splits > 1
    assert hip.workspace_info()["allocations"] == 0
    want, _, splits_want = _run("tfhip_fused_matmul", a, b, bias, m, n, k, "linear")
    assert splits_want == splits
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))

    # a forced slice count beyond the static array: refused with both sizes in the message, nothing launched
    check(lib.tfhip_set_tuning(b"splitk", 8))
    try:
        m, n, k = 1024, 1024, 512
        big = DeviceBuffer(m * max(n, k) * 4)
        out = DeviceBuffer(m * n * 4)
        rc = lib.tfhip_fused_matmul_noalloc(big.ptr, big.ptr, out.ptr, 1, 1, m, n, k, 0, 0, None, i64_array([0, 0, 0]),
                                            0, None, i64_array([0, 0, 0]), 0.2)
        msg = lib.tfhip_last_error().decode()
        assert rc != 0 and "33554432" in msg and "16777216" in msg, msg
        big.free()
        out.free()
    finally:
        check(lib.tfhip_set_tuning(b"splitk", -1))
