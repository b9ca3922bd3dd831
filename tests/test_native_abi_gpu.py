"""The C ABI called from C++ with no Python and no torch in the process (tests/native/abi_smoke.cpp): an FP8 cache
written by pa_kv_cache_write, one pa_decode call, checked inside the program against a double-precision attention
over the bytes the cache holds (atol = rtol = 2e-2)."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu


def test_native_caller_of_the_c_abi(cuda):
    from triton_op_amd import build as B

    if not os.path.exists(B.NATIVE_SMOKE_BIN):
        B.build_native_smoke(verbose=False)
    res = subprocess.run([B.NATIVE_SMOKE_BIN], capture_output=True, text=True, timeout=100)
    print(res.stdout, res.stderr, flush=True)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "abi_smoke ok" in res.stdout
