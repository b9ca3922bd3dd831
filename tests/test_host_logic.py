"""CPU-side tests: the C-ABI library loads and exports every symbol the header declares, the ctypes
struct matches it, the host-side argument checks raise the reference's errors, the tuning layer's
choices, and the workload generators."""
import ctypes as C
import os
import re

import pytest
import torch

from triton_op_amd import _cabi, kv_layout as L, workloads as W
import triton_op_amd as T

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header():
    with open(os.path.join(ROOT, "include", "pa_decode.h")) as f:
        return f.read()


def test_library_exports_every_declared_symbol(pa_lib):
    text = re.sub(r"/\*.*?\*/", "", _header(), flags=re.S)
    declared = set(re.findall(r"\b(pa_[a-z0-9_]+)\s*\(", text))
    assert declared == set(_cabi.EXPORTED_SYMBOLS), declared ^ set(_cabi.EXPORTED_SYMBOLS)
    for name in declared:
        assert hasattr(pa_lib, name), name


def test_struct_layout_and_version(pa_lib):
    assert pa_lib.pa_decode_abi_version() == _cabi.PA_DECODE_ABI_VERSION
    assert pa_lib.pa_decode_args_size() == C.sizeof(_cabi.PaDecodeArgs)
    # every field of the header's struct, in order
    body = re.search(r"typedef struct PaDecodeArgs \{(.*?)\} PaDecodeArgs;", _header(), re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    names = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl:
            continue
        names += [n.strip().lstrip("*") for n in re.sub(r"^(const\s+)?[a-z0-9_]+\s*\**", "", decl, count=1).split(",")]
    assert names == [f[0] for f in _cabi.PaDecodeArgs._fields_]
    body = re.search(r"typedef struct PaKvWriteArgs \{(.*?)\} PaKvWriteArgs;", _header(), re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    names = []
    for decl in body.split(";"):
        decl = decl.strip()
        if decl:
            names += [n.strip().lstrip("*") for n in re.sub(r"^(const\s+)?[a-z0-9_]+\s*\**", "", decl, count=1).split(",")]
    assert names == [f[0] for f in _cabi.PaKvWriteArgs._fields_]
    assert C.sizeof(_cabi.PaKvWriteArgs) == 8 + 7 * 8 + 8 + 6 * 4 + 10 * 8


def test_workspace_size_rule(pa_lib):
    # 64 bytes of counters + one (sequence, partition) pair of int32 per possible item + one int32 per sequence
    assert pa_lib.pa_decode_workspace_bytes(256, 8) == 64 + 8 * 256 * 8 + 4 * 256
    assert pa_lib.pa_decode_workspace_bytes(1, 1) == 76
    assert pa_lib.pa_decode_workspace_bytes(0, 4) == _cabi.PA_DECODE_WORKSPACE_BYTES


def test_error_strings_and_null_arguments(pa_lib):
    assert pa_lib.pa_decode_error_string(0) == b"ok"
    for code in range(-7, 0):
        assert pa_lib.pa_decode_error_string(code) not in (b"ok", b"unknown error code")
    assert pa_lib.pa_decode(None, None) == -1
    a = _cabi.PaDecodeArgs()
    assert pa_lib.pa_decode_partition(C.byref(a), None) == -2  # struct_size not set
    a.struct_size = C.sizeof(_cabi.PaDecodeArgs)
    assert pa_lib.pa_decode_partition(C.byref(a), None) == -1  # buffers are NULL
    assert pa_lib.pa_debug_fp8_decode(None, None, 4, None) == -1
    assert pa_lib.pa_decode_noalloc(None, None) == -1
    b = _cabi.PaDecodeArgs()
    assert pa_lib.pa_decode_noalloc(C.byref(b), None) == -2
    b.struct_size = C.sizeof(_cabi.PaDecodeArgs)
    b.workspace_bytes = 64  # this entry point owns the workspace and the partition buffers: passing one is an error
    assert pa_lib.pa_decode_noalloc(C.byref(b), None) == -4


def test_partition_size_choices():
    f = T.select_partition_size
    # (num_seqs, kv heads, rows per group, longest context, block size, CUs)
    assert f(64, 8, 8, 4096, 16, 256) == 4096      # c2: one partition, four waves per workgroup, no reduce
    assert f(4, 8, 8, 131072, 16, 256) == 8192     # c4: 16 partitions x 32 (sequence, head) pairs x 4 waves
    assert f(128, 8, 16, 32768, 1024, 256) == 8192  # c3
    assert f(256, 8, 64, 65536, 16, 256) == 8192   # c5: 64 rows = 4 row tiles sharing one workgroup's page stream
    assert f(4, 8, 32, 131072, 16, 256) == 5632    # few long sequences, 2 row tiles: 24 partitions fill the GPU
    assert f(32, 4, 32, 4096, 16, 256) == 1024     # short partitions: two workgroups per CU (36.6 us against 39.4 for 768)
    assert f(4, 8, 64, 16384, 16, 256) == 1024     # measured 43.0 us against 47.6 us for 768
    assert f(64, 4, 32, 4096, 16, 256) == 1536     # measured 59.9 us against 61.9 (2048) and 64.9 (1024)
    assert f(4, 1, 8, 1024, 16, 256) == 1024       # c1: tiny; one partition, no second kernel
    assert f(48, 8, 8, 4096, 16, 256) == 4096      # three quarters of the wave slots filled: still one partition
    assert f(4, 8, 8, 4096, 16, 256) == 512        # 32 rows only: eight partitions each
    assert f(8, 8, 8, 4096, 16, 256) == 512        # measured 18.6 us against 20.2 (1024) and 27.6 (4096)
    assert f(16, 8, 8, 4096, 16, 256) == 1024      # measured 29.2 us against 30.8 (512) and 30.6 (4096)
    assert f(24, 8, 8, 4096, 16, 256) == 4096      # measured 36.4 us against 41.5 (2048)
    assert f(1, 8, 8, 4096, 16, 256) == 512
    for args in [(1, 1, 1, 1, 16, 256), (3, 5, 7, 100000, 64, 304), (1000, 8, 16, 300, 16, 64)]:
        ps = f(*args)
        assert ps >= 256 and ps % 256 == 0
    with pytest.raises(_cabi.PaDecodeLibraryError):
        f(0, 8, 8, 4096, 16, 256)


def test_partition_size_from_the_longest_context_and_the_total():
    """The tuning layer's second statistic: the sum of the context lengths.  A batch counts as total / longest
    sequences of the longest length, so a batch whose tokens sit in one or two long sequences gets the small
    partitions of a small batch (measured on the GPU: 8 sequences, one of 65536 tokens and seven of 1024, 32 rows per
    kv head: 106.7 us at 5632 against 49.6 us at 1536); an even batch, or no total, changes nothing."""
    f = T.select_partition_size
    # (num_seqs, kv heads, rows per group, longest context, block size, CUs, total tokens)
    assert f(8, 8, 32, 65536, 16, 256) == 5632 and f(8, 8, 32, 65536, 16, 256, 65536 + 7 * 1024) == 1536
    assert f(8, 8, 8, 65536, 16, 256) == 8192 and f(8, 8, 8, 65536, 16, 256, 65536 + 7 * 1024) == 2048
    assert f(32, 8, 8, 32768, 16, 256, 2 * 32768 + 30 * 512) == 2048
    assert f(64, 8, 8, 4096, 16, 256, 64 * 4096) == f(64, 8, 8, 4096, 16, 256) == 4096     # c2: even
    assert f(256, 8, 64, 28856, 16, 256, 896879) == f(256, 8, 64, 28856, 16, 256) == 7424  # c5: 8192-token cap either way
    assert f(8, 8, 32, 65536, 16, 256, 8 * 65536) == f(8, 8, 32, 65536, 16, 256)           # total = batch x longest
    assert f(8, 8, 32, 65536, 16, 256, 10 ** 12) == f(8, 8, 32, 65536, 16, 256)            # never more than the batch
    assert f(8, 8, 32, 65536, 16, 256, 5) == f(1, 8, 32, 65536, 16, 256)                   # never less than one sequence


def _cpu_args(**over):
    wl = W.make_decode_workload(name="v", seed=1, batch=2, num_q_heads=8, num_kv_heads=2,
                                context_lens=torch.tensor([40, 300], dtype=torch.int32))
    kw = dict(output=torch.empty_like(wl.query), query=wl.query, key_cache=wl.key_cache, value_cache=wl.value_cache,
              sequence_lengths=wl.context_lens, block_tables=wl.block_tables, softmax_scale=wl.softmax_scale,
              query_sequence_length=1, max_sequence_length=300, compute_type=torch.bfloat16, query_scale=None,
              key_scale=wl.key_scale, value_scale=wl.value_scale)
    kw.update(over)
    return kw


@pytest.mark.parametrize("over,msg", [
    (dict(output=torch.empty(2, 8, 128)), "output tensor only support dtype"),
    (dict(query=torch.empty(16, 128, dtype=torch.bfloat16)), "Expected 3D query tensor"),
    (dict(key_cache=torch.empty(4, 2, 16, 128, dtype=torch.float8_e4m3fn)), "Expected 5D key_cache"),
    (dict(value_cache=torch.empty(4, 2, 128, dtype=torch.float8_e4m3fn)), "Unsupported value cache shape"),
    (dict(query_sequence_length=3), "is not num_kv_heads"),
    (dict(key_scale=torch.ones(4, 2, 16), value_scale=torch.ones(4, 2, 16)), "Expected 4D key_scale"),
    (dict(key_scale=torch.ones((), dtype=torch.float64)), "key_scale tensor only support dtype"),
    (dict(key_scale=torch.ones(4, 2, 16, 1)), "same shape"),
    (dict(value_scale=None), "given together"),
    (dict(compute_type=torch.float16), "compute_type"),
    (dict(sequence_lengths=torch.tensor([40, 300])), "int32"),
    (dict(), "GPU only"),
])
def test_entry_point_rejects_bad_arguments(over, msg):
    with pytest.raises(ValueError, match=msg):
        T.plan_decode(**_cpu_args(**over))


def test_entry_point_takes_the_harness_wrappers_trailing_buffers_and_both_alibi_layouts():
    """`max_logits, exp_sums, tmp_output` follow `alibi_slopes` positionally, as in run_gluon_fp8_kernel
    (test_pa_mtp.py:566-584; its spelling `temp_output` is a keyword here) and run_triton
    (test_pa_decode_gluon_triton.py:264-281); `alibi_slopes` is one slope per packed query row (the reference
    kernels' array, pa_decode_triton_gluon_fp8.py:323-327) or one per query head.  On this GPU-less machine a call
    that passes every argument check ends at the "GPU only" error; anything else raised earlier."""
    from triton_op_amd import pa_decode_triton

    wl = W.make_decode_workload(name="v", seed=1, batch=2, num_q_heads=8, num_kv_heads=2, q_len=3,
                                context_lens=torch.tensor([40, 300], dtype=torch.int32))
    rows = 2 * 3 * 4
    ml, es = torch.zeros(2, 2, 2, 12), torch.zeros(2, 2, 2, 12)
    to = torch.zeros(2, 2, 2, 12, 128, dtype=torch.bfloat16)
    pos = (torch.empty_like(wl.query), wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables,
           wl.softmax_scale, 3, 300, torch.bfloat16, None, wl.key_scale, wl.value_scale, 0)
    for slopes in (torch.rand(rows), torch.rand(8), None):
        with pytest.raises(ValueError, match="GPU only"):
            T.plan_decode(*pos, slopes, ml, es, to)
        with pytest.raises(ValueError, match="GPU only"):
            T.paged_attention_decode(*pos, slopes, ml, es, temp_output=to)
    for bad in (torch.rand(rows + 1), torch.rand(2), torch.rand(rows, dtype=torch.float64)):
        with pytest.raises(ValueError, match="alibi_slopes must be"):
            T.plan_decode(*pos, bad)
    with pytest.raises(ValueError, match="same buffer"):
        T.plan_decode(*pos, None, ml, es, to, temp_output=to.clone())
    wl1 = W.make_decode_workload(name="v", seed=1, batch=2, num_q_heads=8, num_kv_heads=2,
                                 context_lens=torch.tensor([40, 300], dtype=torch.int32))
    with pytest.raises(ValueError, match="GPU only"):
        pa_decode_triton.paged_attention_decode(
            torch.empty_like(wl1.query), wl1.query, wl1.key_cache, wl1.value_cache, wl1.context_lens, wl1.block_tables,
            wl1.softmax_scale, 300, torch.bfloat16, wl1.key_scale, wl1.value_scale, 0, torch.rand(8),
            torch.zeros(2, 2, 2, 4), torch.zeros(2, 2, 2, 4), torch.zeros(2, 2, 2, 4, 128, dtype=torch.bfloat16))


def test_c_abi_checks_the_alibi_array_length(pa_lib):
    """The C ABI cannot see an array's length: alibi_slopes_len says which of the two layouts the caller's array
    has, and anything else is refused before a launch."""
    a = _fake_args(b=4, hq=16, hkv=2, q=3, ctx=1024, ps=256)
    buf = C.create_string_buffer(256)
    a.alibi_slopes = 0x70000000
    for n, rc in ((2 * 3 * 8, 0), (2 * 8, 0), (0, -4), (3 * 8, -4), (2 * 3 * 8 + 1, -4)):
        a.alibi_slopes_len = n
        assert pa_lib.pa_decode_launch_info(C.byref(a), buf, 256) == rc, n
    a.alibi_slopes = None  # without slopes the length is ignored
    assert pa_lib.pa_decode_launch_info(C.byref(a), buf, 256) == 0


def test_entry_point_rejects_group_and_block_size():
    wl = W.make_decode_workload(name="v", seed=1, batch=1, num_q_heads=80, num_kv_heads=1,
                                context_lens=torch.tensor([40], dtype=torch.int32))
    with pytest.raises(ValueError, match="exceeds maximum of 64"):
        T.plan_decode(torch.empty_like(wl.query), wl.query, wl.key_cache, wl.value_cache, wl.context_lens,
                      wl.block_tables, 0.1, 1, 40, torch.bfloat16, None, wl.key_scale, wl.value_scale)
    kc = torch.empty(4, 1, 8, 32, 16, dtype=torch.float8_e4m3fn)
    vc = torch.empty(4, 1, 128, 32, dtype=torch.float8_e4m3fn)
    q = torch.empty(1, 8, 128, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="not in"):
        T.plan_decode(torch.empty_like(q), q, kc, vc, torch.tensor([40], dtype=torch.int32),
                      torch.zeros(1, 4, dtype=torch.int32), 0.1, 1, 40)


def test_kv_cache_writers_reject_tensors_on_another_device(monkeypatch):
    """Every tensor handed to the cache writers is dereferenced on the GPU: one that lives elsewhere (a
    slot_mapping built on the host, a CPU scale tensor) must raise before anything is launched.  The check is
    reached on this GPU-less machine by presenting the key rows as a tensor of another device type."""
    from triton_op_amd import kv_cache as KC

    class _Launched(Exception):
        pass

    def _no_launch():
        raise _Launched("the library must not be reached")

    monkeypatch.setattr(KC._cabi, "load_library", _no_launch)
    t, h, d, bs, nblk = 32, 2, 128, 16, 4
    key = torch.zeros(t, h, d, dtype=torch.bfloat16, device="meta")
    value = torch.zeros(t, h, d, dtype=torch.bfloat16, device="meta")
    kc = torch.zeros(nblk, h, d // 16, bs, 16, dtype=torch.float8_e4m3fn, device="meta")
    vc = torch.zeros(nblk, h, d, bs, dtype=torch.float8_e4m3fn, device="meta")
    ks = torch.zeros(nblk, h, bs, 1, device="meta")
    vs = torch.zeros(nblk, h, bs, 1, device="meta")
    slots = torch.zeros(t, dtype=torch.int64, device="meta")
    monkeypatch.setattr(torch.Tensor, "is_cuda", property(lambda self: self.device.type in ("cuda", "meta")))
    good = dict(key=key, value=value, key_cache=kc, value_cache=vc, slot_mapping=slots, key_scale=ks, value_scale=vs)
    for name in ("value", "key_cache", "value_cache", "slot_mapping", "key_scale", "value_scale"):
        bad = dict(good)
        bad[name] = torch.zeros(good[name].shape, dtype=good[name].dtype)  # the same tensor on the CPU
        with pytest.raises(ValueError, match=f"{name} is on cpu"):
            KC.kv_cache_write(**bad)
    kc16 = torch.zeros(nblk, h, d // 8, bs, 8, dtype=torch.bfloat16, device="meta")
    vc16 = torch.zeros(nblk, h, d, bs, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="value_cache is on cpu"):
        KC.quantize_kv_cache_symmetric(kc16, vc16)


def test_library_path_must_exist(monkeypatch):
    monkeypatch.setattr(_cabi, "_lib", None)
    with pytest.raises(_cabi.PaDecodeLibraryError, match="is missing"):
        _cabi.load_library("/nonexistent/libpa_decode.so")
    monkeypatch.undo()
    assert _cabi.load_library() is not None


def test_workload_generators_shapes_and_bytes():
    wl = W.make_config("c1")
    assert wl.query.shape == (4, 8, 128) and wl.key_cache.shape == (256, 1, 16, 16, 8)
    assert wl.value_cache.shape == (256, 1, 128, 16) and wl.block_tables.shape == (4, 64)
    assert sorted(wl.block_tables.flatten().tolist()) == list(range(256))  # a permutation of the pool
    assert 1 <= int(wl.context_lens.min()) and int(wl.context_lens.max()) <= 1024
    c2 = W.make_config("c2", batch=2, ctx_scale=0.125)
    assert c2.key_cache.dtype == torch.float8_e4m3fn and c2.key_cache.shape[1:] == (8, 8, 16, 16)
    assert c2.key_scale.dim() == 0 and c2.meta["pool_blocks"] == 80  # 1.25 x 2 x 512 / 16
    assert c2.kv_bytes() == 2 * 512 * 8 * 128 * 2
    assert len(set(c2.block_tables.flatten().tolist())) == c2.block_tables.numel()
    c5 = W.make_config("c5", batch=6, ctx_scale=0.05)
    assert c5.key_scale.shape == (c5.key_cache.shape[0], 8, 16, 1) and c5.q_lens is not None
    assert c5.query.shape == (6, 8 * 4 * 16, 128)
    assert c5.kv_bytes() == int(c5.context_lens.sum()) * 8 * (256 + 8)
    # same seed, same tensors
    again = W.make_config("c2", batch=2, ctx_scale=0.125)
    assert torch.equal(again.key_cache.view(torch.uint8), c2.key_cache.view(torch.uint8))
    assert torch.equal(again.block_tables, c2.block_tables)


def test_per_token_quantised_cache_layout():
    g = torch.Generator().manual_seed(3)
    kc, vc = L.create_kv_cache(5, 16, 2, 128, torch.bfloat16, generator=g)
    kq, ks, vq, vs = L.quantize_kv_cache_per_token(kc, vc)
    assert kq.shape == (5, 2, 8, 16, 16) and vq.shape == (5, 2, 128, 16) and ks.shape == vs.shape == (5, 2, 16, 1)
    ktok = L.key_cache_to_tokens(kc).float()  # [blocks, bs, Hkv, D]
    back = L.key_cache_to_tokens(kq).float() * ks.permute(0, 2, 1, 3)
    assert float((back - ktok).abs().max()) <= float(ktok.abs().max()) * 2.0 ** -4
    vtok = L.value_cache_to_tokens(vc).float()
    vback = L.value_cache_to_tokens(vq).float() * vs.permute(0, 2, 1, 3)
    assert float((vback - vtok).abs().max()) <= float(vtok.abs().max()) * 2.0 ** -4
    kq2, ks2, vq2, vs2 = L.quantize_kv_cache_per_tensor(kc, vc)
    assert kq2.shape == kq.shape and ks2.dim() == 0


def test_bench_refuses_more_than_one_gpu():
    """One GPU per box: bench.py --gpus N with N > 1 must say so and exit instead of measuring anything."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True,
                         text=True, timeout=120)
    assert res.returncode != 0
    assert "one GPU" in (res.stdout + res.stderr)


def test_graft_entry_points_exist():
    import __graft_entry__ as g

    assert callable(g.build) and callable(g.smoke)


def test_header_is_plain_c_and_links(tmp_path):
    """include/pa_decode.h is the contract of a foreign-function binding: it must compile as C99 on its own, and a
    C program that uses it must link against the library and see the same struct size."""
    import os
    import shutil
    import subprocess

    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = tmp_path / "use_abi.c"
    src.write_text(
        '#include <stdio.h>\n#include "pa_decode.h"\n'
        "int main(void) {\n"
        "  PaDecodeArgs a = {0};\n"
        "  a.struct_size = sizeof a;\n"
        "  if (pa_decode_abi_version() != PA_DECODE_ABI_VERSION) return 2;\n"
        "  if (pa_decode_args_size() != sizeof(PaDecodeArgs)) return 3;\n"
        "  if (pa_decode(&a, 0) != PA_ERR_NULL_POINTER) return 4;  /* buffers are NULL: rejected before any launch */\n"
        '  printf("%s\\n", pa_decode_error_string(PA_ERR_BAD_SHAPE));\n'
        "  return 0;\n}\n")
    exe = tmp_path / "use_abi"
    libdir = os.path.join(root, "triton_op_amd")
    subprocess.run([gcc, "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", os.path.join(root, "include"), str(src),
                    "-L", libdir, "-lpa_decode", "-Wl,-rpath," + libdir, "-o", str(exe)], check=True,
                   capture_output=True, text=True)
    res = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert res.returncode == 0, (res.returncode, res.stdout, res.stderr)
    assert "stride" in res.stdout or "size" in res.stdout


def test_short_division_of_the_cache_writers_is_the_rounded_quotient(tmp_path):
    """The KV-cache write kernels divide by a row's scale with a reciprocal and ONE correction of the quotient
    (pa_kv_cache.hip: quantize8, bf16_amax_to_scale) and must still produce the correctly rounded x / scale of
    the torch formula (kv_layout.pertoken_quant).  tests/native/short_division_check.c runs the same arithmetic
    on the host against the compiler's division: exhaustively for per-token scales, widely for arbitrary ones."""
    import os
    import shutil
    import subprocess

    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = tmp_path / "short_division_check"
    subprocess.run([gcc, "-O2", "-ffp-contract=off", os.path.join(root, "tests", "native", "short_division_check.c"),
                    "-lm", "-o", str(exe)], check=True)
    res = subprocess.run([str(exe), "8000"], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stdout + res.stderr
    assert " 0 mismatches; arbitrary" in res.stdout and res.stdout.rstrip().endswith("amax/448 0 mismatches")


def _fake_args(*, b, hq, hkv, q, ctx, bs=16, ps, kv="fp8", per_token=False, ragged=False, workspace=True):
    """A PaDecodeArgs with the shapes of a call and made-up, suitably aligned addresses: the launch layer's choice
    is host arithmetic on the struct and dereferences nothing."""
    a = _cabi.PaDecodeArgs()
    a.struct_size = C.sizeof(_cabi.PaDecodeArgs)
    g = hq // hkv
    ge = q * g
    esz = 1 if kv == "fp8" else 2
    x = 16 // esz
    base = 0x10000000
    for i, name in enumerate(("output", "query", "key_cache", "value_cache", "context_lens", "block_tables", "exp_sums",
                              "max_logits", "tmp_output")):
        setattr(a, name, base + i * 0x1000000)
    if ragged:
        a.q_lens = base + 0x20000000
    if kv == "fp8":
        a.key_scale, a.value_scale = base + 0x30000000, base + 0x31000000
    a.num_seqs, a.num_kv_heads, a.group_size, a.q_len, a.head_size, a.block_size = b, hkv, g, q, 128, bs
    a.partition_size = ps
    a.max_num_partitions = -(-ctx // ps)
    a.query_dtype = _cabi.PA_DTYPE_BF16
    a.kv_dtype = _cabi.PA_DTYPE_FP8_E4M3FN if kv == "fp8" else _cabi.PA_DTYPE_BF16
    a.query_quant_mode = _cabi.PA_QUANT_NONE
    a.kv_quant_mode = (_cabi.PA_QUANT_PER_TOKEN if per_token else _cabi.PA_QUANT_PER_TENSOR) if kv == "fp8" else _cabi.PA_QUANT_NONE
    a.softmax_scale = 0.088
    a.stride_out_h = a.stride_q_h = 128
    a.stride_out_s = a.stride_q_s = 128 * hkv * ge
    a.stride_k_c, a.stride_k_h = bs * x, 128 * bs
    a.stride_k_b = a.stride_k_h * hkv
    a.stride_v_2, a.stride_v_h, a.stride_v_b = bs, 128 * bs, 128 * bs * hkv
    a.stride_bt_s = -(-ctx // bs)
    P = a.max_num_partitions
    a.stride_es_p, a.stride_es_h, a.stride_es_s = ge, ge * P, ge * P * hkv
    a.stride_tmp_g, a.stride_tmp_p, a.stride_tmp_h, a.stride_tmp_s = 128, 128 * ge, 128 * ge * P, 128 * ge * P * hkv
    a.stride_kvscale_h, a.stride_kvscale_b = bs, bs * hkv
    if workspace:
        a.workspace = base + 0x40000000
        a.workspace_bytes = 64 + 8 * b * P + 4 * b
    return a


def test_own_cut_of_the_partition_axis_invariants(pa_lib):
    """PA_DECODE_FLAG_OUTPUT_ONLY: over random shapes the library's own partition size (pa_decode_launch_info names
    it) is a multiple of the caller's, no longer than the caller's whole axis and no longer than the tuning layer's
    choice for the shape; without a workspace the factor divides the caller's partition count (the axis ends where
    the caller's ends); without the flag nothing is re-cut."""
    import random

    rng = random.Random(77)
    recut = 0
    for _ in range(1500):
        hkv = rng.choice([1, 2, 4, 8])
        g, q = rng.choice([(1, 1), (5, 1), (8, 1), (16, 1), (8, 2), (16, 2), (16, 4), (8, 4), (10, 1)])
        b = rng.choice([1, 3, 16, 64, 128, 256, 700])
        ps = rng.choice([256, 256, 512, 1024])
        ctx = rng.randint(1, 140000 if b <= 16 else 9000)
        ws = rng.random() < 0.7
        kw = dict(b=b, hq=g * hkv, hkv=hkv, q=q, ctx=ctx, bs=rng.choice([16, 64, 1024]), ps=ps,
                  per_token=rng.random() < 0.5, ragged=q > 1 and rng.random() < 0.5, workspace=ws)
        texts = []
        for flags in (0, _cabi.PA_DECODE_FLAG_OUTPUT_ONLY):
            a = _fake_args(**kw)
            a.flags = flags
            buf = C.create_string_buffer(256)
            assert pa_lib.pa_decode_launch_info(C.byref(a), buf, 256) == 0, kw
            texts.append(buf.value.decode())
        assert "own partitions" not in texts[0], (kw, texts[0])
        if "own partitions of " not in texts[1]:
            continue
        recut += 1
        P = -(-ctx // ps)
        own = int(texts[1].split("own partitions of ")[1].split()[0])
        k = own // ps
        assert own % ps == 0 and 2 <= k <= P, (kw, texts[1])
        want = pa_lib.pa_decode_select_partition_size_stats(b, hkv, g * q, P * ps, 0, kw["bs"], 256)
        assert own <= want, (kw, texts[1], want)
        if not ws:
            assert P % k == 0, (kw, texts[1])
    assert recut > 300


def test_launch_layer_choices(pa_lib):
    """Which partition kernel, in which instantiation, over which grid: the launch layer's choice for the five
    benchmark configurations at the tuning layer's partition size (256 compute units assumed when there is no
    GPU) and for the cases that take another path."""
    def info(**kw):
        buf = C.create_string_buffer(256)
        assert pa_lib.pa_decode_launch_info(C.byref(_fake_args(**kw)), buf, 256) == 0
        return buf.value.decode()

    # c2: one partition, four waves, 64 x 8 workgroups, no item list
    assert info(b=64, hq=64, hkv=8, q=1, ctx=4096, ps=4096) == "pa_partition_kernel<fp8, bs16, 4 waves> x 512"
    # c2 at the reference's partition size: 16 x 512 partitions for 2048 wave slots: one-wave walkers of four each, and
    # the four of a (sequence, kv head) in one workgroup that merges them itself
    assert info(b=64, hq=64, hkv=8, q=1, ctx=4096, ps=256) == \
        "pa_partition_kernel<fp8, bs16, 1 waves> x 512, teams of 4 waves, 4 partitions per wave, no reduce kernel"
    # ... without an output (stage 1 alone forms no teams), with too few sequences to fill three quarters of the wave
    # slots, or with more than fit the GPU at once: one-wave workgroups
    a = _fake_args(b=64, hq=64, hkv=8, q=1, ctx=4096, ps=256)
    a.output = None
    buf = C.create_string_buffer(256)
    assert pa_lib.pa_decode_launch_info(C.byref(a), buf, 256) == 0
    assert buf.value.decode() == "pa_partition_kernel<fp8, bs16, 1 waves> x 2048, 4 partitions per workgroup"
    assert info(b=40, hq=64, hkv=8, q=1, ctx=4096, ps=256) == \
        "pa_partition_kernel<fp8, bs16, 1 waves> x 2560, 2 partitions per workgroup"
    assert info(b=72, hq=64, hkv=8, q=1, ctx=4096, ps=256) == \
        "pa_partition_kernel<fp8, bs16, 1 waves> x 2304, 4 partitions per workgroup"
    # 13 partitions: 4 + 4 + 4 + 1; per-token scales: the teams of a sequence on one XCD
    assert info(b=56, hq=64, hkv=8, q=1, ctx=3200, ps=256, per_token=True) == \
        "pa_partition_kernel<fp8 per-token, bs16, 1 waves> x 448, teams of 4 waves, 4 partitions per wave, no reduce kernel, " \
        "an item's heads on one XCD"
    # ... of 1024 tokens: two each; and never more than the partition axis holds (3 partitions: one workgroup per sequence and head, four rounds of them: sorted)
    assert info(b=128, hq=64, hkv=8, q=1, ctx=4096, ps=1024) == \
        "pa_partition_kernel<fp8, bs16, 1 waves> x 2048, 2 partitions per workgroup"
    assert info(b=1024, hq=64, hkv=8, q=1, ctx=768, ps=256) == \
        "pa_partition_kernel<fp8, bs16, 1 waves> x 8192, sorted items, 3 partitions per workgroup"
    # c4: 16 partitions per sequence, one round
    assert info(b=4, hq=64, hkv=8, q=1, ctx=131072, ps=8192) == "pa_partition_kernel<fp8, bs16, 4 waves> x 512"
    # c3: block 1024 takes the run-time strides
    assert info(b=128, hq=64, hkv=8, q=2, ctx=32768, bs=1024, ps=8192) == \
        "pa_partition_kernel<fp8, strided, 4 waves> x 4096, sorted items"
    # c5: 64 rows per kv head over an FP8 cache with per-token scales
    assert info(b=256, hq=128, hkv=8, q=4, ctx=28856, ps=7424, per_token=True, ragged=True) == \
        "pa_partition_shared_kernel<fp8 per-token, bs16, 3 ring slots, 3 workgroups per CU> x 8192, sorted items, " \
        "an item's heads on one XCD"
    assert info(b=128, hq=64, hkv=4, q=2, ctx=4096, ps=4096) == \
        "pa_partition_shared_kernel<fp8, bs16, 2 ring slots, 4 workgroups per CU> x 512"
    # per-token scales: the grid is whole groups of eight (sequence, partition) items (an XCD takes every eighth, with
    # all its heads); 3 sequences x 4 partitions -> 16 items x 2 heads
    assert info(b=3, hq=64, hkv=2, q=1, ctx=4096, ps=1024, per_token=True) == \
        "pa_partition_shared_kernel<fp8 per-token, bs16, 3 ring slots, 3 workgroups per CU> x 32, an item's heads on one XCD"
    assert info(b=3, hq=16, hkv=2, q=1, ctx=4096, ps=1024, per_token=True) == \
        "pa_partition_kernel<fp8 per-token, bs16, 4 waves> x 32, an item's heads on one XCD"
    # c1: a bf16 cache, 8 rows, few workgroups
    assert info(b=4, hq=8, hkv=1, q=1, ctx=1024, ps=1024, kv="bf16") == "pa_partition_kernel<bf16, strided, 4 waves> x 4"
    # a bf16 cache with 32 rows per kv head: two row tiles per workgroup; ragged with a workspace: queued
    assert info(b=128, hq=64, hkv=4, q=2, ctx=4096, ps=4096, kv="bf16") == \
        "pa_partition_kernel<bf16, strided, 4 waves, 2 row tiles> x 512"
    assert "queued items" in info(b=64, hq=128, hkv=8, q=4, ctx=4096, ps=4096, kv="bf16", ragged=True)
    assert "queued items" not in info(b=64, hq=128, hkv=8, q=4, ctx=4096, ps=4096, kv="bf16", ragged=True, workspace=False)
    # more sequences than the item tables of the queued / sorted launches hold: plain order, no error
    # (a tile of up to 8 real rows stages half the bytes per partition: up to eight partitions per workgroup)
    assert info(b=5000, hq=8, hkv=1, q=1, ctx=4096, ps=256) == \
        "pa_partition_kernel<fp8, bs16, 1 waves> x 10000, 8 partitions per workgroup"
    assert info(b=5000, hq=16, hkv=1, q=1, ctx=4096, ps=256) == \
        "pa_partition_kernel<fp8, bs16, 1 waves> x 20000, 4 partitions per workgroup"
    # c4 at the reference's partition size: 512 partitions per sequence, eight per workgroup, one round
    assert info(b=4, hq=64, hkv=8, q=1, ctx=131072, ps=256) == \
        "pa_partition_kernel<fp8, bs16, 1 waves> x 2048, 8 partitions per workgroup"
    # bad arguments are refused as by the launch itself
    a = _fake_args(b=4, hq=8, hkv=1, q=1, ctx=1024, ps=300)
    assert pa_lib.pa_decode_launch_info(C.byref(a), C.create_string_buffer(64), 64) == -4
