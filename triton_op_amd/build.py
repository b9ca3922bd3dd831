"""Builds the HIP shared library of the decode op, in-tree, for gfx950.

    python -m triton_op_amd.build

`hipcc` cross-compiles without a GPU.  The result is triton_op_amd/libpa_decode.so, which the
ctypes binding in `_cabi.py` loads; nothing is JIT-compiled at import or call time.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = [os.path.join(HERE, "csrc", "pa_decode.hip"), os.path.join(HERE, "csrc", "pa_kv_cache.hip")]
HEADERS = [os.path.join(HERE, "..", "include", "pa_decode.h")] + [
    os.path.join(HERE, "csrc", h)
    for h in ("pa_common.h", "pa_launch.h", "pa_partition_kernel.h", "pa_partition_shared_kernel.h", "pa_plan_kernel.h",
              "pa_reduce_kernel.h", "pa_generic_kernel.h")]
LIB_PATH = os.path.join(HERE, "libpa_decode.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++20",
    "-fno-strict-aliasing",
    "-fPIC",
    "-shared",
    # packed-FP32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or put /opt/rocm/bin on PATH)")


def build(verbose: bool = True, extra_flags=()) -> str:
    cmd = [find_hipcc(), *HIPCC_FLAGS, *extra_flags, *SOURCES, "-o", LIB_PATH]
    if verbose:
        print("[triton_op_amd.build]", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass warns that it does not know the packed-fp32-ops feature; that is expected
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{res.stdout}\n{res.stderr}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return LIB_PATH


NATIVE_SMOKE_SRC = os.path.join(HERE, "..", "tests", "native", "abi_smoke.cpp")
NATIVE_SMOKE_BIN = os.path.join(HERE, "..", "tests", "native", "abi_smoke")


def build_native_smoke(verbose: bool = True) -> str:
    """The C++ caller of the C ABI that the GPU tests run (tests/native/abi_smoke.cpp): no Python, no torch."""
    cmd = [find_hipcc(), "-O2", NATIVE_SMOKE_SRC, "-I" + os.path.join(HERE, "..", "include"), "-L" + HERE,
           "-lpa_decode", "-Wl,-rpath,$ORIGIN/../../triton_op_amd", "-o", NATIVE_SMOKE_BIN]
    if verbose:
        print("[triton_op_amd.build]", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{res.stdout}\n{res.stderr}")
    return NATIVE_SMOKE_BIN


PROBE_SRC = os.path.join(HERE, "..", "tests", "native", "pa_probe.hip")
PROBE_LIB = os.path.join(HERE, "..", "tests", "native", "libpa_probe.so")


def build_probe(verbose: bool = True) -> str:
    """The measuring kernels of bench.py's probe workloads (tests/native/pa_probe.h): a library of their own, built
    from the decode kernels' headers; not part of the operator or its ABI."""
    cmd = [find_hipcc(), *HIPCC_FLAGS, PROBE_SRC, "-o", PROBE_LIB]
    if verbose:
        print("[triton_op_amd.build]", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{res.stdout}\n{res.stderr}")
    return PROBE_LIB


TRACE_LIB = os.path.join(HERE, "..", "tests", "native", "libpa_decode_trace.so")


def build_trace(verbose: bool = True) -> str:
    """The measuring build of the decode library (-DPA_DECODE_TRACE): the same sources, with per-workgroup timestamps
    in pa_partition_shared_kernel, for bench.py's `trace:` workloads.  Never loaded by the product path."""
    cmd = [find_hipcc(), *HIPCC_FLAGS, "-DPA_DECODE_TRACE", *SOURCES, "-o", TRACE_LIB]
    if verbose:
        print("[triton_op_amd.build]", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{res.stdout}\n{res.stderr}")
    return TRACE_LIB


def is_stale() -> bool:
    if not os.path.exists(LIB_PATH):
        return True
    t = os.path.getmtime(LIB_PATH)
    return any(os.path.getmtime(p) > t for p in SOURCES + HEADERS)


if __name__ == "__main__":
    build()
    build_native_smoke()
    build_probe()
    build_trace()
