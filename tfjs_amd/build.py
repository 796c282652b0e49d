"""Builds the native half of tfjs-backend-hip in-tree.

  tfjs_amd/lib/libtfjs_hip.so   HIP kernels + C ABI (include/tfjs_hip.h), gfx950 only
  tfjs_amd/lib/tfjs_hip.node    N-API addon over that C ABI (only if Node headers exist)

Objects go to a temporary directory; only the two libraries stay in the tree.
"""
import concurrent.futures
import os
import shutil
import subprocess
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIB_DIR, "libtfjs_hip.so")
ADDON = os.path.join(LIB_DIR, "tfjs_hip.node")

HIP_SOURCES = ["runtime.hip", "dequant.hip", "depthwise.hip", "gemm.hip", "conv2d.hip", "glue.hip", "expand_dw.hip", "expand_dw_tile.hip", "expand_dw_stream.hip", "block_fused.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -packed-fp32-ops off: the compiler must not form packed FP32 instructions
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=on",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall",
             "-Wno-unused-command-line-argument"]
NODE_INCLUDE_CANDIDATES = ["/usr/include/node", "/usr/local/include/node"]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def node_include_dir():
    for d in NODE_INCLUDE_CANDIDATES:
        if os.path.exists(os.path.join(d, "node_api.h")):
            return d
    return None


def build_library(verbose=False):
    os.makedirs(LIB_DIR, exist_ok=True)
    tmp = tempfile.mkdtemp(prefix="tfjs_hip_build_")
    try:
        def compile_one(src):
            obj = os.path.join(tmp, src.replace(".hip", ".o"))
            out = _run([HIPCC] + HIP_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj])
            if verbose and out.strip():
                print(out)
            return obj
        with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(HIP_SOURCES))) as pool:
            objs = list(pool.map(compile_one, HIP_SOURCES))
        _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    return LIB


def build_addon():
    inc = node_include_dir()
    src = os.path.join(CSRC, "napi_addon.cc")
    if inc is None or not os.path.exists(src):
        return None
    _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-I", inc, "-I", os.path.join(HERE, "..", "include"),
          "-DNAPI_VERSION=6", src, "-o", ADDON, "-L", LIB_DIR, "-ltfjs_hip", "-Wl,-rpath,$ORIGIN"])
    return ADDON


def build_all(verbose=False):
    lib = build_library(verbose)
    addon = build_addon()
    return lib, addon


if __name__ == "__main__":
    print(build_all(verbose=True))
