"""GPU parity tests: the HIP kernels, called through the C ABI (via the Python entry point or the
raw ctypes functions), against the CPU oracle on the same seeded inputs.

Tolerances.  End to end the bar is atol 2e-2 / rtol 2e-2 on the bf16 output (torch.allclose rule
|a-b| <= atol + rtol*|b|).  Stage-wise: the cache bytes and the query reach the MFMAs exactly (a bf16
cache on the bf16 MFMAs; an FP8 cache on the FP8 MFMAs with the bf16 query carried as an FP8 head plus
an FP8 residual under a power-of-two row factor, which is exact), so max_logits and exp_sums differ
from the f32 oracle by accumulation order only and are compared at 1e-4 (bf16 cache) / 5e-4 (FP8 cache,
whose scales are applied in another order).  tmp_output carries the
rounding of P (about 2^-8 relative per element) and of the stored bf16 value and is compared at 2e-2
like the output.
"""
import ctypes as C
import math

import pytest
import torch

from oracle import pa_oracle as O

pytestmark = pytest.mark.gpu

ATOL = RTOL = 2e-2


def _ctx(*v):
    return torch.tensor(v, dtype=torch.int32)


def _run(wl, dev, *, partition_size=256, alibi=None, transposed=False, **kw):
    import triton_op_amd as T

    g = wl.to(dev)
    out = torch.full_like(g.query, float("nan"))
    res = T.paged_attention_decode(
        out, g.query, g.key_cache, g.value_cache, g.context_lens, g.block_tables, g.softmax_scale, g.q_len,
        g.max_context_len, torch.bfloat16, None, g.key_scale, g.value_scale,
        alibi_slopes=None if alibi is None else alibi.to(dev), partition_size=partition_size,
        query_lens=g.q_lens, **kw)
    torch.cuda.synchronize()
    return out.cpu(), res


def _oracle(wl, alibi=None, seq_ids=None):
    return O.paged_attention_decode_oracle(
        wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables, wl.softmax_scale,
        wl.q_len if wl.q_lens is None else wl.q_lens, wl.key_scale, wl.value_scale, alibi, seq_ids, q_max=wl.q_len)


def _check_stages(wl, res, partition_size, alibi=None):
    P = res["maximum_logits"].shape[2]
    ml, es, to = O.partition_stage(
        wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables, wl.softmax_scale,
        wl.q_len if wl.q_lens is None else wl.q_lens, wl.key_scale, wl.value_scale, alibi, partition_size, P,
        q_max=wl.q_len)
    gml, ges = res["maximum_logits"].cpu(), res["exponential_sums"].cpu()
    gto = res["temporary_output"].float().cpu()
    fin = torch.isfinite(ml)
    assert torch.equal(gml[~fin], ml[~fin]), "rows with no visible key must hold max=-inf"
    # the cache bytes and the query enter the MFMAs exactly (bf16, or FP8 with the query as an exact FP8
    # head + residual): the logits differ from the f32 oracle by accumulation order only
    if wl.key_cache.dtype == torch.bfloat16:
        torch.testing.assert_close(gml[fin], ml[fin], atol=1e-4, rtol=1e-5)
        torch.testing.assert_close(ges, es, atol=1e-4, rtol=1e-4)
    else:  # the scales are applied in another order (folded into the exponent): a few f32 roundings more
        torch.testing.assert_close(gml[fin], ml[fin], atol=5e-4, rtol=5e-5)
        torch.testing.assert_close(ges, es, atol=5e-4, rtol=1e-3)
    torch.testing.assert_close(gto, to, atol=ATOL, rtol=RTOL)
    # the reduce kernel alone, on the kernel's own partition buffers, against the closed-form merge
    merged = O.reduce_stage(gml, ges, gto, wl.context_lens, partition_size)
    return merged


def _make(**kw):
    from triton_op_amd import workloads as W

    kw.setdefault("name", "t")
    kw.setdefault("seed", 7)
    return W.make_decode_workload(**kw)


def test_fp8_dequant_table_on_device(cuda, pa_lib):
    codes = torch.arange(256, dtype=torch.uint8, device=cuda)
    out = torch.empty(256, dtype=torch.float32, device=cuda)
    assert pa_lib.pa_debug_fp8_decode(codes.data_ptr(), out.data_ptr(), 256, None) == 0
    torch.cuda.synchronize()
    tab = torch.from_numpy(O.e4m3fn_table())
    o = out.cpu()
    assert torch.equal(torch.isnan(o), torch.isnan(tab))
    ok = ~torch.isnan(tab)
    assert torch.equal(o[ok], tab[ok])


CASES = {
    # the reference sweep's awkward shapes: groups 5/10 (non power of two), ctx 4097, qlen 1..4
    "fp8_g8": dict(batch=3, num_q_heads=16, num_kv_heads=2, context_lens=_ctx(300, 64, 1000)),
    "fp8_g8_boundaries": dict(batch=6, num_q_heads=8, num_kv_heads=1, context_lens=_ctx(1, 255, 256, 257, 512, 4097)),
    "fp8_g5_q2": dict(batch=3, num_q_heads=5, num_kv_heads=1, context_lens=_ctx(257, 33, 700), q_len=2),
    "fp8_g10_q3": dict(batch=2, num_q_heads=10, num_kv_heads=1, context_lens=_ctx(513, 100), q_len=3),
    "fp8_g16_q4": dict(batch=2, num_q_heads=64, num_kv_heads=4, context_lens=_ctx(513, 4100), q_len=4),
    "fp8_g16_q1": dict(batch=2, num_q_heads=16, num_kv_heads=1, context_lens=_ctx(4096, 17)),
    "fp8_token_g16_q4": dict(batch=3, num_q_heads=32, num_kv_heads=2, context_lens=_ctx(257, 33, 700), q_len=4,
                             scale_mode="token"),
    "fp8_token_g8_q1": dict(batch=3, num_q_heads=16, num_kv_heads=2, context_lens=_ctx(257, 33, 1700),
                            scale_mode="token"),
    "fp8_token_ragged": dict(batch=4, num_q_heads=32, num_kv_heads=2, context_lens=_ctx(257, 33, 700, 5), q_len=4,
                             q_lens=_ctx(1, 2, 3, 4), scale_mode="token"),
    "bf16_g8": dict(batch=4, num_q_heads=8, num_kv_heads=1, context_lens=_ctx(1, 300, 1024, 77), kv_dtype="bf16",
                    scale_mode="none"),
    "bf16_g16_q2": dict(batch=2, num_q_heads=16, num_kv_heads=1, context_lens=_ctx(300, 77), kv_dtype="bf16",
                        scale_mode="none", q_len=2),
    "bf16_g16_q4": dict(batch=2, num_q_heads=16, num_kv_heads=1, context_lens=_ctx(600, 77), kv_dtype="bf16",
                        scale_mode="none", q_len=4),
    "fp8_bs1024_q2": dict(batch=3, num_q_heads=16, num_kv_heads=2, context_lens=_ctx(1500, 1024, 3000),
                          block_size=1024, q_len=2),
    "fp8_bs64": dict(batch=3, num_q_heads=16, num_kv_heads=2, context_lens=_ctx(1500, 63, 300), block_size=64),
    "fp8_transV_bs16": dict(batch=3, num_q_heads=16, num_kv_heads=2, context_lens=_ctx(300, 64, 1000),
                            transposed_v=True),
    "fp8_transV_bs1024": dict(batch=2, num_q_heads=16, num_kv_heads=2, context_lens=_ctx(1500, 3000),
                              block_size=1024, transposed_v=True),
    # more than 16 query rows per kv head over an FP8 cache: the row tiles share one pass over the pages
    "fp8_bs64_g16_q2": dict(batch=3, num_q_heads=32, num_kv_heads=2, context_lens=_ctx(1500, 63, 300), block_size=64,
                            q_len=2),
    "fp8_token_bs1024_g8_q4": dict(batch=3, num_q_heads=8, num_kv_heads=1, context_lens=_ctx(1500, 1024, 3000),
                                   block_size=1024, q_len=4, scale_mode="token"),
    "fp8_transV_bs16_g16_q3": dict(batch=3, num_q_heads=32, num_kv_heads=2, context_lens=_ctx(300, 64, 1000),
                                   transposed_v=True, q_len=3),
    "fp8_token_transV_bs64_g8_q3": dict(batch=2, num_q_heads=16, num_kv_heads=2, context_lens=_ctx(1500, 200),
                                        block_size=64, transposed_v=True, q_len=3, scale_mode="token"),
    "fp8_g8_q4_long": dict(batch=2, num_q_heads=8, num_kv_heads=1, context_lens=_ctx(9000, 4097), q_len=4),
    # at most two busy tiles of a four-tile group: two waves share a tile and split each step's tokens; contexts
    # so short that the second wave sees no key at all, and the padding tiles are written by the waves left over
    "fp8_ragged_two_waves_per_tile": dict(batch=5, num_q_heads=32, num_kv_heads=2, context_lens=_ctx(5, 33, 700, 31, 257),
                                          q_len=4, q_lens=_ctx(1, 2, 1, 2, 2)),
    "fp8_token_ragged_two_waves_per_tile": dict(batch=5, num_q_heads=32, num_kv_heads=2,
                                                context_lens=_ctx(17, 64, 1000, 2, 300), q_len=4,
                                                q_lens=_ctx(2, 1, 2, 2, 1), scale_mode="token"),
    # a bf16 cache with 64 rows per kv head and ragged query lengths: two workgroups of two row tiles per kv head,
    # taken from the work queue when the call has a workspace (tiles of padding rows only are no items)
    "bf16_ragged_g16_q4": dict(batch=5, num_q_heads=32, num_kv_heads=2, context_lens=_ctx(300, 33, 700, 4, 257), q_len=4,
                               q_lens=_ctx(1, 4, 2, 3, 4), kv_dtype="bf16", scale_mode="none"),
    "bf16_transV_bs64": dict(batch=2, num_q_heads=8, num_kv_heads=2, context_lens=_ctx(150, 300), block_size=64,
                             kv_dtype="bf16", scale_mode="none", transposed_v=True),
}


@pytest.mark.parametrize("name", list(CASES))
@pytest.mark.parametrize("partition_size", [256, 512, 1024, 4096])
def test_parity_stagewise_and_end_to_end(cuda, name, partition_size):
    wl = _make(**CASES[name])
    print(f"case={name} partition_size={partition_size}", flush=True)
    out, res = _run(wl, cuda, partition_size=partition_size)
    assert res["partition_size"] == partition_size
    ref = _oracle(wl)
    assert not torch.isnan(out.float()).any()
    torch.testing.assert_close(out.float(), ref.float(), atol=ATOL, rtol=RTOL)
    merged = _check_stages(wl, res, partition_size)
    torch.testing.assert_close(out.float(), merged.float(), atol=4e-3, rtol=8e-3)  # bf16 rounding only
    thr = O.error_stats(out, ref)["max_diff_thr"]
    assert thr < 1e-2, thr


@pytest.mark.parametrize("name", ["fp8_g8", "fp8_g10_q3", "fp8_token_g16_q4", "bf16_g16_q4", "fp8_token_ragged"])
@pytest.mark.parametrize("layout", ["per_row", "per_head"])
def test_alibi(cuda, name, layout):
    """ALiBi slopes in both layouts the entry point takes: one per packed query row, [Hkv*q*G] -- the array the
    reference kernels index with kv_head*QUERY_GROUP_SIZE + row (pa_decode_triton_gluon_fp8.py:323-327, 803-810) --
    and one per query head.  With several new tokens the per-row slopes are all different, so a kernel that read
    them per head (or in another row order) misses the oracle."""
    wl = _make(**CASES[name])
    n = wl.query.shape[1] if layout == "per_row" else wl.num_q_heads
    slopes = torch.linspace(0.01, 0.3, n, dtype=torch.float32)
    out, res = _run(wl, cuda, alibi=slopes)
    ref = _oracle(wl, slopes)
    torch.testing.assert_close(out.float(), ref.float(), atol=ATOL, rtol=RTOL)
    _check_stages(wl, res, 256, slopes)
    if layout == "per_row" and wl.q_len > 1:  # the other reading of the same numbers is a different result
        other = _oracle(wl, slopes[:wl.num_q_heads])
        assert float((other.float() - ref.float()).abs().max()) > 5e-2


@pytest.mark.parametrize("q_len", [2, 4])
@pytest.mark.parametrize("ctx", [(300, 64, 1000), (100, 40, 250)])
def test_attention_sinks(cuda, ctx, q_len):
    import triton_op_amd as T

    wl = _make(batch=3, num_q_heads=16, num_kv_heads=2, context_lens=_ctx(*ctx), q_len=q_len)
    g = wl.to(cuda)
    sinks = torch.linspace(-2.0, 3.0, wl.query.shape[1], dtype=torch.float32)
    out = torch.full_like(g.query, float("nan"))
    T.paged_attention_decode(out, g.query, g.key_cache, g.value_cache, g.context_lens, g.block_tables,
                             g.softmax_scale, q_len, g.max_context_len, torch.bfloat16, None, g.key_scale,
                             g.value_scale, sinks=sinks.to(cuda))
    torch.cuda.synchronize()
    ref = O.paged_attention_decode_oracle(wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables,
                                          wl.softmax_scale, q_len, wl.key_scale, wl.value_scale, sinks=sinks)
    torch.testing.assert_close(out.float().cpu(), ref.float(), atol=ATOL, rtol=RTOL)
    plain = _oracle(wl)
    assert float((plain.float() - ref.float()).abs().max()) > 5e-2  # the sinks do change the result


def test_golden_fixtures(cuda):
    import glob
    import os

    import triton_op_amd as T
    from tests.golden.make_golden import load_case

    files = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz")))
    assert files
    for f in files:
        c = load_case(f)
        d = {k: (v.to(cuda) if torch.is_tensor(v) else v) for k, v in c.items()}
        out = torch.empty_like(d["query"])
        T.paged_attention_decode(out, d["query"], d["key_cache"], d["value_cache"], d["context_lens"],
                                 d["block_tables"], c["softmax_scale"], c["q_len"], int(c["context_lens"].max()),
                                 torch.bfloat16, None, d["key_scale"], d["value_scale"])
        torch.cuda.synchronize()
        torch.testing.assert_close(out.double().cpu(), c["expected"], atol=ATOL, rtol=RTOL)
        err = float(((out.double().cpu() - c["expected"]).abs() / (1 + c["expected"].abs())).max())
        assert err < 6e-3, (f, err)


@pytest.mark.parametrize("q_len", [2, 4])
def test_stale_cache_contents_are_never_used(cuda, q_len):
    """Slots past context_len in the last page, pages named by unused block-table entries, and their
    per-token scales, hold NaN bytes: the result must not change (and must not be NaN)."""
    wl = _make(batch=3, num_q_heads=16, num_kv_heads=2, context_lens=_ctx(5, 250, 1001), scale_mode="token",
               q_len=q_len)
    ref_out, _ = _run(wl, cuda)
    kc, vc = wl.key_cache.clone().view(torch.uint8), wl.value_cache.clone().view(torch.uint8)
    ks, vs = wl.key_scale.clone(), wl.value_scale.clone()
    used = set()
    for b in range(3):
        ctx = int(wl.context_lens[b])
        for i in range((ctx + 15) // 16):
            page = int(wl.block_tables[b, i])
            used.add(page)
            live = min(16, ctx - 16 * i)
            kc[page, :, :, live:, :] = 0x7F
            vc[page, :, :, live:] = 0x7F
            ks[page, :, live:] = float("nan")
            vs[page, :, live:] = float("nan")
    spare = [p for p in range(kc.shape[0]) if p not in used]
    for p in spare:
        kc[p], vc[p], ks[p], vs[p] = 0x7F, 0x7F, float("nan"), float("nan")
    bt = wl.block_tables.clone()
    for b in range(3):
        n = (int(wl.context_lens[b]) + 15) // 16
        bt[b, n:] = spare[0]
    wl2 = type(wl)(**{**wl.__dict__, "key_cache": kc.view(torch.float8_e4m3fn), "value_cache": vc.view(torch.float8_e4m3fn),
                     "key_scale": ks, "value_scale": vs, "block_tables": bt})
    out, _ = _run(wl2, cuda)
    assert torch.equal(out.view(torch.int16), ref_out.view(torch.int16))


@pytest.mark.parametrize("q_len", [2, 3])
def test_block_permutation_invariance_bit_exact(cuda, q_len):
    wl = _make(batch=4, num_q_heads=16, num_kv_heads=2, context_lens=_ctx(700, 64, 2049, 300), q_len=q_len)
    base, _ = _run(wl, cuda)
    n = wl.key_cache.shape[0]
    perm = torch.randperm(n, generator=torch.Generator().manual_seed(3))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(n)
    wl2 = type(wl)(**{**wl.__dict__, "key_cache": wl.key_cache[perm], "value_cache": wl.value_cache[perm],
                     "block_tables": inv[wl.block_tables.long()].to(torch.int32)})
    out, _ = _run(wl2, cuda)
    assert torch.equal(out.view(torch.int16), base.view(torch.int16))


def test_caller_buffers_strided_inputs_and_twin_entry_point(cuda):
    from triton_op_amd import pa_decode_triton

    wl = _make(batch=3, num_q_heads=16, num_kv_heads=2, context_lens=_ctx(300, 64, 1000))
    g = wl.to(cuda)
    ref = _oracle(wl)
    P, ge = 4, 8
    es = torch.full((3, 2, P + 2, ge), 7.0, device=cuda)[:, :, :P]  # non-contiguous partition axis
    ml = torch.full((3, 2, P + 2, ge), 7.0, device=cuda)[:, :, :P]
    to = torch.full((3, 2, P, ge, 128), 7.0, dtype=torch.bfloat16, device=cuda)
    qpad = torch.zeros(3, 16, 256, dtype=torch.bfloat16, device=cuda)
    qpad[:, :, :128] = g.query
    q = qpad[:, :, :128]  # row stride 256
    out = torch.empty(3, 16, 128, dtype=torch.bfloat16, device=cuda)
    res = pa_decode_triton.paged_attention_decode(out, q, g.key_cache, g.value_cache, g.context_lens, g.block_tables,
                                                  g.softmax_scale, g.max_context_len, torch.bfloat16, g.key_scale,
                                                  g.value_scale, exp_sums=es, max_logits=ml, tmp_output=to)
    torch.cuda.synchronize()
    assert res["exp_sums"].data_ptr() == es.data_ptr() and res["partition_size"] == 256
    torch.testing.assert_close(out.float().cpu(), ref.float(), atol=ATOL, rtol=RTOL)
    # partitions a sequence does not reach are left untouched (sequence 1 has 64 tokens: 1 partition)
    assert (es[1, :, 1:] == 7.0).all() and (to[1, :, 1:] == 7.0).all()


def test_teams_with_strided_caller_buffers_and_output(cuda):
    """A launch in teams through caller-owned buffers that are not contiguous: partition buffers with a longer
    partition axis, a query and an output whose rows are 256 elements apart, a block table with a longer row."""
    import triton_op_amd as T

    batch, hkv, group, P = 50, 8, 8, 8
    gen = torch.Generator().manual_seed(71)
    ctx = torch.randint(1, 256 * P + 1, (batch,), generator=gen, dtype=torch.int32)
    ctx[0], ctx[1] = 256 * P, 200
    wl = _make(batch=batch, num_q_heads=hkv * group, num_kv_heads=hkv, context_lens=ctx)
    g = wl.to(cuda)
    es = torch.full((batch, hkv, P + 3, group), 7.0, device=cuda)[:, :, :P]
    ml = torch.full((batch, hkv, P + 3, group), 7.0, device=cuda)[:, :, :P]
    to = torch.full((batch, hkv, P + 1, group, 128), 7.0, dtype=torch.bfloat16, device=cuda)[:, :, :P]
    qpad = torch.zeros(batch, hkv * group, 256, dtype=torch.bfloat16, device=cuda)
    qpad[:, :, :128] = g.query
    opad = torch.full((batch, hkv * group, 256), float("nan"), dtype=torch.bfloat16, device=cuda)
    out = opad[:, :, :128]
    bt = torch.zeros(batch, g.block_tables.shape[1] + 5, dtype=torch.int32, device=cuda)
    bt[:, :g.block_tables.shape[1]] = g.block_tables
    plan = T.plan_decode(out, qpad[:, :, :128], g.key_cache, g.value_cache, g.context_lens,
                         bt[:, :g.block_tables.shape[1]], g.softmax_scale, 1, 256 * P, torch.bfloat16, None, g.key_scale,
                         g.value_scale, 0, None, ml, es, to, partition_size=256)
    assert "teams of 4 waves, 2 partitions per wave" in plan.launch_info(), plan.launch_info()
    plan.run()
    torch.cuda.synchronize()
    torch.testing.assert_close(out.float().cpu(), _oracle(wl).float(), atol=ATOL, rtol=RTOL)
    assert bool(torch.isnan(opad[:, :, 128:].float()).all())  # nothing written between the output's rows
    merged = O.reduce_stage(ml.cpu(), es.cpu(), to.float().cpu(), wl.context_lens, 256)
    torch.testing.assert_close(out.float().cpu(), merged.float(), atol=2e-3, rtol=2e-2)
    # partitions a sequence does not reach are left untouched (sequence 1 has 200 tokens: 1 partition)
    assert (es[1, :, 1:] == 7.0).all() and (to[1, :, 1:] == 7.0).all()


@pytest.mark.parametrize("q_len", [2, 4])
def test_fp8_query_with_scales(cuda, q_len):
    """FP8 query with a per-row scale, the reference Gluon entry point's own contract
    (pa_decode_triton_gluon_fp8.py:747-755,889-903)."""
    import triton_op_amd as T
    from triton_op_amd import kv_layout as L

    wl = _make(batch=3, num_q_heads=16, num_kv_heads=2, context_lens=_ctx(300, 64, 1000), q_len=q_len,
               scale_mode="token")
    qq, qs = L.pertoken_quant(wl.query.float())
    g = wl.to(cuda)
    out = torch.empty_like(g.query)
    T.paged_attention_decode(out, qq.to(cuda), g.key_cache, g.value_cache, g.context_lens, g.block_tables,
                             g.softmax_scale, q_len, g.max_context_len, torch.bfloat16, qs.to(cuda), g.key_scale,
                             g.value_scale)
    torch.cuda.synchronize()
    ref = O.paged_attention_decode_oracle(qq, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables,
                                          wl.softmax_scale, q_len, wl.key_scale, wl.value_scale, query_scale=qs)
    torch.testing.assert_close(out.float().cpu(), ref.float(), atol=ATOL, rtol=RTOL)
    qs0 = torch.tensor(float(wl.query.float().abs().max()) / 448.0)
    qq0 = (wl.query.float() / qs0).to(torch.float8_e4m3fn)
    T.paged_attention_decode(out, qq0.to(cuda), g.key_cache, g.value_cache, g.context_lens, g.block_tables,
                             g.softmax_scale, q_len, g.max_context_len, torch.bfloat16, qs0.to(cuda), g.key_scale,
                             g.value_scale)
    torch.cuda.synchronize()
    ref0 = O.paged_attention_decode_oracle(qq0, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables,
                                           wl.softmax_scale, q_len, wl.key_scale, wl.value_scale, query_scale=qs0)
    torch.testing.assert_close(out.float().cpu(), ref0.float(), atol=ATOL, rtol=RTOL)


@pytest.mark.parametrize("with_sinks", [False, True])
def test_many_rows_take_the_four_rows_per_wave_reduce(cuda, with_sinks):
    """16384 output rows and more are merged four rows per wave: up to 8 partitions through the all-loads-first
    path, more through the row loop; padding rows of a ragged batch and single-partition sequences are mixed in."""
    import triton_op_amd as T

    gen = torch.Generator().manual_seed(11)
    ctx = torch.randint(1, 1200, (128,), generator=gen, dtype=torch.int32)
    ctx[:6] = torch.tensor([3000, 2049, 256, 257, 1, 2900], dtype=torch.int32)
    ql = torch.randint(1, 3, (128,), generator=gen, dtype=torch.int32)
    wl = _make(batch=128, num_q_heads=64, num_kv_heads=8, context_lens=torch.maximum(ctx, ql), q_len=2, q_lens=ql)
    g = wl.to(cuda)
    sinks = torch.linspace(-2.0, 3.0, wl.query.shape[1], dtype=torch.float32) if with_sinks else None
    out = torch.full_like(g.query, float("nan"))
    T.paged_attention_decode(out, g.query, g.key_cache, g.value_cache, g.context_lens, g.block_tables,
                             g.softmax_scale, 2, g.max_context_len, torch.bfloat16, None, g.key_scale, g.value_scale,
                             partition_size=256, query_lens=g.q_lens, sinks=None if sinks is None else sinks.to(cuda))
    torch.cuda.synchronize()
    ref = O.paged_attention_decode_oracle(wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables,
                                          wl.softmax_scale, wl.q_lens, wl.key_scale, wl.value_scale, sinks=sinks)
    assert not torch.isnan(out.float()).any()
    torch.testing.assert_close(out.float().cpu(), ref.float(), atol=ATOL, rtol=RTOL)


@pytest.mark.parametrize("group,q_len,scale_mode", [(8, 1, "tensor"), (16, 3, "token"), (4, 2, "tensor")])
def test_sorted_dispatch_of_a_many_round_launch(cuda, group, q_len, scale_mode):
    """Launches with several rounds of workgroups take their (sequence, partition) items from the planning
    kernel's list (whole partitions first, last partitions by decreasing length).  The result must be the one the
    plain grid order gives, bit for bit, with a minimal workspace (no list) and with none of the counters left
    behind; one-token sequences and exact multiples of the partition size are in the batch."""
    import triton_op_amd as T

    gen = torch.Generator().manual_seed(21)
    # one row tile per kv head: one-wave workgroups walk up to four partitions each, so it takes 600 sequences
    # before the coarser items still make more than two rounds (600 x 8 x ceil(5 / 4)); the shared-stream kernel
    # (48 rows) has one item per partition and 96 sequences are plenty
    batch = 96 if group * q_len > 16 else 600
    top = 2600 if group * q_len > 16 else 1280
    ctx = torch.randint(1, top, (batch,), generator=gen, dtype=torch.int32)
    ctx[:5] = torch.tensor([512, 256, top - 40, 1, 255], dtype=torch.int32)
    ctx = torch.clamp(ctx, min=q_len)
    wl = _make(batch=batch, num_q_heads=group * 8, num_kv_heads=8, context_lens=ctx, q_len=q_len, scale_mode=scale_mode)
    g = wl.to(cuda)
    outs = []
    parts = -(-int(ctx.max()) // 256)
    # None: the entry point sizes the workspace for both lists (sorted dispatch, listed reduce); room for the item
    # list only (sorted dispatch, reduce over every sequence); 64: counters only (grid order)
    for ws_bytes in (None, 64 + 8 * batch * parts, 64):
        ws = None if ws_bytes is None else torch.zeros(ws_bytes // 4, dtype=torch.int32, device=cuda)
        out = torch.full_like(g.query, float("nan"))
        plan = T.plan_decode(out, g.query, g.key_cache, g.value_cache, g.context_lens, g.block_tables,
                             g.softmax_scale, q_len, g.max_context_len, torch.bfloat16, None, g.key_scale,
                             g.value_scale, partition_size=256, workspace=ws)
        assert plan.args.max_num_partitions * batch * 8 > 4096  # far more workgroups than the GPU holds
        info = plan.launch_info()
        print(f"workspace {ws_bytes}: {info}", flush=True)
        # the first two launches really take their items from the list, the third really does not
        assert ("sorted items" in info) == (ws_bytes != 64), info
        plan.run()
        plan.run()  # the list is rebuilt by every call
        torch.cuda.synchronize()
        outs.append(out.cpu())
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))
    assert torch.equal(outs[0].view(torch.int16), outs[2].view(torch.int16))
    torch.testing.assert_close(outs[0].float(), _oracle(wl).float(), atol=ATOL, rtol=RTOL)


@pytest.mark.parametrize("kv,scale_mode,group,q_len,ragged,block_size,ps,span,alibi,batch,max_ctx",
                         [("fp8", "tensor", 2, 1, False, 16, 256, 3, False, 200, 1100), ("fp8", "token", 4, 2, False, 16, 256, 3, False, 200, 1100),
                          ("fp8", "tensor", 8, 2, False, 64, 256, 3, False, 200, 1100), ("fp8", "tensor", 8, 2, False, 1024, 512, 2, False, 200, 1100),
                          ("bf16", "none", 16, 4, True, 16, 256, 4, False, 200, 1100), ("fp8", "token", 8, 1, False, 16, 256, 3, True, 200, 1100),
                          # 600 x 8 x ceil(5 / 4) coarse items are more than two rounds: the walk AND the sorted dispatch
                          # (8 rows per kv head: half-size slots, all five partitions in one workgroup)
                          ("fp8", "tensor", 8, 1, False, 16, 256, 5, False, 600, 1100), ("fp8", "token", 4, 2, False, 16, 256, 5, True, 600, 1100),
                          ("fp8", "tensor", 16, 1, False, 16, 256, 4, False, 600, 1100),
                          # nine partitions, eight rows: eight partitions per workgroup, then one
                          ("fp8", "tensor", 8, 1, False, 16, 256, 8, False, 400, 2100), ("fp8", "token", 2, 3, False, 16, 256, 8, True, 400, 2100)])
def test_workgroups_that_walk_several_partitions(cuda, kv, scale_mode, group, q_len, ragged, block_size, ps, span, alibi, batch, max_ctx):
    """A caller-fixed small partition size and several rounds of one-wave workgroups: every workgroup then walks
    several consecutive partitions in one pass over the pages (the launch layer says so) and writes one partial
    result per partition.  The partition buffers are held against the oracle's partition stage, the merged result
    against the oracle.  The partition axis (5 of 256 tokens, 3 of 512) is not a multiple of the span (3 or 4, 2),
    contexts end on, before and
    after partition boundaries, and in the ragged bf16 case a 32-row tile of some sequences holds padding rows
    only (launched without a workspace, in plain order: with one, such batches take the queued launch).  With ALiBi
    every step goes through the masked variant of the loop, boundaries included.  The two cases of 600 sequences
    still have more than two rounds of the coarser items, so the planning kernel lists (sequence, first partition of
    a walk) items and the workgroups take them from the list: there one sequence is empty, and the call is made a
    second time with the flag that says the list is still good."""
    import triton_op_amd as T
    from triton_op_amd import _cabi

    gen = torch.Generator().manual_seed(33)
    ctx = torch.randint(1, max_ctx + 1, (batch,), generator=gen, dtype=torch.int32)
    ctx[:9] = torch.tensor([1, 255, 256, 257, 512, 768, 769, 1024, max_ctx], dtype=torch.int32)
    ctx = torch.clamp(ctx, min=q_len)
    q_lens = None
    if ragged:
        q_lens = torch.randint(1, q_len + 1, (batch,), generator=gen, dtype=torch.int32)
        q_lens[:4] = torch.tensor([1, q_len, 2, 1], dtype=torch.int32)
    wl = _make(batch=batch, num_q_heads=group * 8, num_kv_heads=8, context_lens=ctx, q_len=q_len, q_lens=q_lens,
               kv_dtype=kv, scale_mode=scale_mode, block_size=block_size)
    sorted_too = batch >= 400
    if sorted_too:  # an empty sequence among them (the generator wants a page per sequence: declared empty afterwards)
        ctx = ctx.clone()
        ctx[11] = 0
        wl = type(wl)(**{**wl.__dict__, "context_lens": ctx})
    live = [b for b in range(batch) if int(ctx[b]) > 0]
    g = wl.to(cuda)
    out = torch.full_like(g.query, float("nan"))
    slopes = torch.linspace(0.01, 0.3, wl.query.shape[1], dtype=torch.float32) if alibi else None
    plan = T.plan_decode(out, g.query, g.key_cache, g.value_cache, g.context_lens, g.block_tables, g.softmax_scale,
                         q_len, max_ctx, torch.bfloat16, None, g.key_scale, g.value_scale, partition_size=ps,
                         query_lens=g.q_lens, alibi_slopes=None if slopes is None else slopes.to(cuda))
    P = -(-max_ctx // ps)
    assert plan.args.max_num_partitions == P
    if ragged:
        plan.args.workspace = None
        plan.args.workspace_bytes = 0
    # 8000 items for 2048 wave slots: three partitions each (4800 of 512 tokens: two); 16000 two-tile items for 1024
    # slots: four, the most there is
    assert f"{span} partitions per workgroup" in plan.launch_info(), plan.launch_info()
    assert ("sorted items" in plan.launch_info()) == sorted_too, plan.launch_info()
    plan.exp_sums.fill_(float("nan"))
    plan.max_logits.fill_(float("nan"))
    plan.run()
    torch.cuda.synchronize()
    if sorted_too:
        # the next layer of the same step: same lengths, the list of coarse items is reused
        first = out.clone()
        out.fill_(float("nan"))
        plan.exp_sums.fill_(float("nan"))
        plan.max_logits.fill_(float("nan"))
        plan.args.flags = _cabi.PA_DECODE_FLAG_REUSE_ITEM_LIST
        plan.run()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), first.view(torch.int16))
        assert bool((out[11] == 0).all())
    # partitions a sequence does not reach are not written; the oracle leaves them at its fill values
    reach = (torch.arange(P)[None, :] * ps < ctx[:, None])  # [batch, P]
    ml, es, to = O.partition_stage(
        wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables, wl.softmax_scale,
        wl.q_len if wl.q_lens is None else wl.q_lens, wl.key_scale, wl.value_scale, slopes, ps, P, q_max=wl.q_len)
    gml, ges, gto = plan.max_logits.cpu(), plan.exp_sums.cpu(), plan.tmp_output.float().cpu()
    sel = reach[:, None, :, None].expand_as(ml)
    fin = torch.isfinite(ml) & sel
    assert torch.equal(gml[sel & ~torch.isfinite(ml)], ml[sel & ~torch.isfinite(ml)])
    tight = kv == "bf16"
    torch.testing.assert_close(gml[fin], ml[fin], atol=1e-4 if tight else 5e-4, rtol=1e-5 if tight else 5e-5)
    torch.testing.assert_close(ges[sel], es[sel], atol=1e-4 if tight else 5e-4, rtol=1e-4 if tight else 1e-3)
    sel_o = reach[:, None, :, None, None].expand_as(to)
    torch.testing.assert_close(gto[sel_o], to[sel_o], atol=ATOL, rtol=RTOL)
    assert not torch.isnan(out.float()).any()
    torch.testing.assert_close(out.float().cpu()[live], _oracle(wl, slopes, seq_ids=live).float()[live], atol=ATOL, rtol=RTOL)


@pytest.mark.parametrize("scale_mode,group,q_len,ragged,block_size,ps,max_ctx,batch,per_wave,alibi",
                         [("tensor", 8, 1, False, 16, 256, 4096, 64, 4, False),   # the reference's shape: 16 partitions, 4 per wave
                          ("token", 8, 1, False, 16, 256, 4096, 64, 4, False),
                          ("tensor", 16, 1, False, 16, 256, 4096, 48, 4, False),  # 16 rows: full-size slots; 384 teams
                          ("token", 4, 4, True, 16, 256, 3200, 64, 4, False),     # 13 partitions: 4 + 4 + 4 + 1; padding rows
                          ("tensor", 4, 2, False, 64, 256, 1100, 64, 2, True),    # 5 partitions: 2 + 2 + 1 and an idle wave
                          ("token", 8, 2, False, 16, 512, 2048, 64, 1, False),    # 4 partitions: one each
                          ("tensor", 2, 3, True, 1024, 512, 2048, 64, 1, True),
                          ("tensor", 8, 1, False, 16, 256, 7000, 64, 7, False)])  # 28 partitions of 8 rows: 7 per wave
@pytest.mark.parametrize("output_only", [False, True])
def test_teams_merge_in_the_partition_kernel(cuda, scale_mode, group, q_len, ragged, block_size, ps, max_ctx, batch, per_wave,
                                             alibi, output_only):
    """A caller-fixed small partition size on a batch whose (sequence, kv head) units are all resident at once, four waves each: four
    one-wave walkers share a workgroup, cover the sequence's whole partition axis between them and merge their partial
    results into `output` themselves; pa_decode launches no reduce kernel (the launch layer says so).  Contexts end
    on, before and after partition and walk boundaries, reach one partition only (written by the wave that finished
    them), leave whole waves of a team without a partition, or are empty (zero rows).  The partition buffers are
    held against the oracle's partition stage (with the output-only flag the library cuts the partition axis its own
    way -- one partition for these shapes, no teams -- and the same rows are checked), the
    result against the oracle; a second call with the same arguments is bit-identical.  With attention sinks no teams
    are formed."""
    import triton_op_amd as T

    gen = torch.Generator().manual_seed(61)
    ctx = torch.randint(1, max_ctx + 1, (batch,), generator=gen, dtype=torch.int32)
    edge = [1, ps - 1, ps, ps + 1, per_wave * ps, per_wave * ps + 1, 2 * per_wave * ps + 63, 3 * per_wave * ps, max_ctx, max_ctx - 1]
    ctx[:len(edge)] = torch.tensor([min(max(e, 1), max_ctx) for e in edge], dtype=torch.int32)
    ctx = torch.clamp(ctx, min=q_len)
    q_lens = None
    if ragged:
        q_lens = torch.randint(1, q_len + 1, (batch,), generator=gen, dtype=torch.int32)
        q_lens[:4] = torch.tensor([1, q_len, 2, 1], dtype=torch.int32)
    wl = _make(batch=batch, num_q_heads=group * 8, num_kv_heads=8, context_lens=ctx, q_len=q_len, q_lens=q_lens,
               kv_dtype="fp8", scale_mode=scale_mode, block_size=block_size)
    ctx = ctx.clone()
    ctx[13] = 0  # (the generator wants a page per sequence: declared empty afterwards)
    wl = type(wl)(**{**wl.__dict__, "context_lens": ctx})
    live = [b for b in range(batch) if int(ctx[b]) > 0]
    g = wl.to(cuda)
    out = torch.full_like(g.query, float("nan"))
    slopes = torch.linspace(0.01, 0.3, wl.query.shape[1], dtype=torch.float32) if alibi else None
    kw = dict(partition_size=ps, query_lens=g.q_lens, alibi_slopes=None if slopes is None else slopes.to(cuda))
    plan = T.plan_decode(out, g.query, g.key_cache, g.value_cache, g.context_lens, g.block_tables, g.softmax_scale,
                         q_len, max_ctx, torch.bfloat16, None, g.key_scale, g.value_scale, output_only=output_only, **kw)
    P = -(-max_ctx // ps)
    assert plan.args.max_num_partitions == P
    info = plan.launch_info()
    if output_only:  # the partition buffers are scratch: the library cuts the axis its own way (here: one partition)
        assert "teams" not in info and "own partitions of" in info, info
    else:
        assert f"teams of 4 waves, {per_wave} partitions per wave, no reduce kernel" in info and f"x {batch * 8}," in info, info
    plan.exp_sums.fill_(float("nan"))
    plan.max_logits.fill_(float("nan"))
    plan.tmp_output.fill_(float("nan"))
    plan.run()
    torch.cuda.synchronize()
    first = out.clone()
    rows = (torch.ones(batch, dtype=torch.int32) * q_len if q_lens is None else q_lens)
    gml, ges, gto = plan.max_logits.cpu(), plan.exp_sums.cpu(), plan.tmp_output.float().cpu()
    if not output_only:
        reach = (torch.arange(P)[None, :] * ps < ctx[:, None])  # [batch, P]
        ml, es, to = O.partition_stage(
            wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables, wl.softmax_scale,
            wl.q_len if wl.q_lens is None else wl.q_lens, wl.key_scale, wl.value_scale, slopes, ps, P, q_max=wl.q_len)
        sel = reach[:, None, :, None].expand_as(ml)
        fin = torch.isfinite(ml) & sel
        assert torch.equal(gml[sel & ~torch.isfinite(ml)], ml[sel & ~torch.isfinite(ml)])
        torch.testing.assert_close(gml[fin], ml[fin], atol=5e-4, rtol=5e-5)
        torch.testing.assert_close(ges[sel], es[sel], atol=5e-4, rtol=1e-3)
        sel_o = reach[:, None, :, None, None].expand_as(to)
        torch.testing.assert_close(gto[sel_o], to[sel_o], atol=ATOL, rtol=RTOL)
    # rows of a sequence: [kv head, query position, head of the group]
    by_pos = lambda t: t.float().cpu().view(batch, 8, q_len, group, -1)
    want = by_pos(_oracle(wl, slopes, seq_ids=live))
    got = by_pos(out)
    for b in live:
        n = int(rows[b])
        assert not torch.isnan(got[b, :, :n]).any(), b
        torch.testing.assert_close(got[b, :, :n], want[b, :, :n], atol=ATOL, rtol=RTOL)
        if not output_only:
            assert bool((got[b, :, n:] == 0).all()), b
    assert bool((got[13] == 0).all())
    out.fill_(float("nan"))
    plan.run()
    torch.cuda.synchronize()
    keep = ~torch.isnan(first.float())
    assert torch.equal(torch.isnan(out.float()), ~keep)
    assert torch.equal(out.view(torch.int16)[keep], first.view(torch.int16)[keep])
    # with attention sinks (here of no weight) no teams are formed; the reduce kernel agrees with the team's merge (the
    # same bf16 partials, merged in another order of additions)
    out2 = torch.full_like(g.query, float("nan"))
    plan2 = T.plan_decode(out2, g.query, g.key_cache, g.value_cache, g.context_lens, g.block_tables, g.softmax_scale,
                          q_len, max_ctx, torch.bfloat16, None, g.key_scale, g.value_scale,
                          sinks=torch.full((g.query.shape[1],), -1e30, dtype=torch.float32, device=cuda), **kw)
    assert "teams" not in plan2.launch_info(), plan2.launch_info()
    plan2.run()
    torch.cuda.synchronize()
    got2 = by_pos(out2)
    for b in live:
        n = int(rows[b])
        # (with the output-only flag `got` comes from one long partition: no bf16 rounding of partial results)
        torch.testing.assert_close(got2[b, :, :n], got[b, :, :n], atol=ATOL if output_only else 2e-3, rtol=2e-2)


@pytest.mark.parametrize("seed", range(12))
def test_teams_seeded_sweep(cuda, seed):
    """Random shapes the launch layer gives to teams (384 to 512 (sequence, kv head) units, up to 16 rows, 4 to 32
    partitions of 256 or 512 tokens, per-tensor or per-token scales, ragged query lengths, ALiBi, pages of 16 or 64
    tokens), random context lengths from one token to the whole partition axis: the result against the oracle."""
    import random

    import triton_op_amd as T

    rng = random.Random(9100 + seed)
    hkv = rng.choice([4, 8])
    batch = rng.randint(384 // hkv, 512 // hkv)
    group, q_len = rng.choice([(8, 1), (4, 2), (2, 4), (16, 1), (4, 4), (8, 2), (1, 3), (5, 3), (3, 1)])
    ge = group * q_len
    ps = rng.choice([256, 256, 512])
    per_wave_max = min(8 if ge <= 8 else 4, 2048 // ps)
    p_min = -(-2048 // (batch * hkv))  # one wave per workgroup: as many items as wave slots
    P = rng.randint(max(p_min, 2), 4 * per_wave_max)
    max_ctx = P * ps - rng.randint(0, ps - 1)
    block_size = rng.choice([16, 16, 64])
    scale_mode = rng.choice(["tensor", "token"])
    ragged = q_len > 1 and rng.random() < 0.5
    alibi = rng.random() < 0.3
    gen = torch.Generator().manual_seed(9100 + seed)
    ctx = torch.randint(1, max_ctx + 1, (batch,), generator=gen, dtype=torch.int32)
    ctx[0], ctx[1] = max_ctx, 1
    ctx = torch.clamp(ctx, min=q_len)
    q_lens = torch.randint(1, q_len + 1, (batch,), generator=gen, dtype=torch.int32) if ragged else None
    wl = _make(batch=batch, num_q_heads=group * hkv, num_kv_heads=hkv, context_lens=ctx, q_len=q_len, q_lens=q_lens,
               kv_dtype="fp8", scale_mode=scale_mode, block_size=block_size, seed=9100 + seed)
    g = wl.to(cuda)
    out = torch.full_like(g.query, float("nan"))
    slopes = torch.linspace(0.01, 0.3, wl.query.shape[1], dtype=torch.float32) if alibi else None
    plan = T.plan_decode(out, g.query, g.key_cache, g.value_cache, g.context_lens, g.block_tables, g.softmax_scale,
                         q_len, max_ctx, torch.bfloat16, None, g.key_scale, g.value_scale, partition_size=ps,
                         query_lens=g.q_lens, alibi_slopes=None if slopes is None else slopes.to(cuda))
    case = f"seed {seed}: batch {batch} hkv {hkv} group {group} q_len {q_len} ps {ps} P {P} bs {block_size} {scale_mode}"
    assert "teams of 4 waves" in plan.launch_info(), case + " -> " + plan.launch_info()
    print(case, flush=True)
    plan.run()
    torch.cuda.synchronize()
    by_pos = lambda t: t.float().cpu().view(batch, hkv, q_len, group, -1)
    got, want = by_pos(out), by_pos(_oracle(wl, slopes))
    for b in range(batch):
        n = q_len if q_lens is None else int(q_lens[b])
        assert not torch.isnan(got[b, :, :n]).any(), case
        torch.testing.assert_close(got[b, :, :n], want[b, :, :n], atol=ATOL, rtol=RTOL, msg=lambda m: case + ": " + m)
        assert bool((got[b, :, n:] == 0).all()), case


@pytest.mark.parametrize("group,q_len,scale_mode", [(8, 1, "tensor"), (16, 3, "token")])
def test_item_list_reused_by_the_next_layer(cuda, group, q_len, scale_mode):
    """Two layers of one decode step share the sequence lengths and a workspace: the second is told to reuse the
    item list the first one's planning kernel left there.  Its result must be the one it computes on its own."""
    import triton_op_amd as T
    from triton_op_amd import _cabi

    gen = torch.Generator().manual_seed(23)
    # (one row tile per kv head: workgroups walk four partitions each, and it takes 600 sequences for the coarser
    # items to still be listed)
    batch = 96 if group * q_len > 16 else 600
    ctx = torch.clamp(torch.randint(1, 2600 if batch == 96 else 1280, (batch,), generator=gen, dtype=torch.int32), min=q_len)
    kw = dict(batch=batch, num_q_heads=group * 8, num_kv_heads=8, context_lens=ctx, q_len=q_len, scale_mode=scale_mode)
    layers = [_make(**kw, seed=7).to(cuda), _make(**kw, seed=8).to(cuda)]
    parts = -(-int(ctx.max()) // 256)
    ws = torch.zeros(int(_cabi.load_library().pa_decode_workspace_bytes(batch, parts)) // 4 + 1, dtype=torch.int32, device=cuda)
    outs = []
    for i, g in enumerate(layers):
        out = torch.full_like(g.query, float("nan"))
        plan = T.plan_decode(out, g.query, g.key_cache, g.value_cache, g.context_lens, g.block_tables, g.softmax_scale,
                             q_len, g.max_context_len, torch.bfloat16, None, g.key_scale, g.value_scale,
                             partition_size=256, workspace=ws, reuse_item_list=i > 0)
        assert "sorted items" in plan.launch_info(), plan.launch_info()
        plan.run()
        outs.append(out)
    alone = torch.full_like(layers[1].query, float("nan"))
    g = layers[1]
    T.paged_attention_decode(alone, g.query, g.key_cache, g.value_cache, g.context_lens, g.block_tables, g.softmax_scale,
                             q_len, g.max_context_len, torch.bfloat16, None, g.key_scale, g.value_scale, partition_size=256)
    torch.cuda.synchronize()
    assert not torch.isnan(outs[1].float()).any()
    assert torch.equal(outs[1].view(torch.int16), alone.view(torch.int16))
    with pytest.raises(ValueError):
        T.paged_attention_decode(alone, g.query, g.key_cache, g.value_cache, g.context_lens, g.block_tables,
                                 g.softmax_scale, q_len, g.max_context_len, torch.bfloat16, None, g.key_scale,
                                 g.value_scale, reuse_item_list=True)


@pytest.mark.parametrize("case", ["one_partition", "partitions", "shared", "sorted", "queue"])
def test_empty_sequences_get_zero_rows(cuda, case):
    """A sequence with context length 0 has nothing to attend to: its output rows are zero in every launch mode
    (also when no reduce kernel runs), and its neighbours are unaffected."""
    import triton_op_amd as T

    kw, ps = dict(
        one_partition=(dict(batch=4, num_q_heads=16, num_kv_heads=2, context_lens=_ctx(100, 0, 200, 0)), 256),
        partitions=(dict(batch=4, num_q_heads=16, num_kv_heads=2, context_lens=_ctx(700, 0, 200, 0)), 256),
        shared=(dict(batch=4, num_q_heads=32, num_kv_heads=2, context_lens=_ctx(100, 0, 200, 0), q_len=3), 256),
        sorted=(dict(batch=600, num_q_heads=16, num_kv_heads=8,
                     context_lens=torch.cat([_ctx(0, 1100, 0), torch.randint(1, 1280, (597,),
                                            generator=torch.Generator().manual_seed(5), dtype=torch.int32)])), 256),
        # (a bf16 cache takes two 16-row tiles per workgroup: the queued launch needs more than 32 rows per kv head)
        queue=(dict(batch=4, num_q_heads=32, num_kv_heads=2, context_lens=_ctx(300, 0, 200, 0), q_len=4,
                    q_lens=_ctx(4, 2, 1, 4), kv_dtype="bf16", scale_mode="none"), 512),
    )[case]
    # the generator wants at least one page per sequence: build with length 1, then declare the sequences empty
    empty = kw["context_lens"] == 0
    wl = _make(**{**kw, "context_lens": torch.clamp(kw["context_lens"], min=kw.get("q_len", 1))})
    ctx = wl.context_lens.clone()
    ctx[empty] = 0
    wl = type(wl)(**{**wl.__dict__, "context_lens": ctx})
    out, _ = _run(wl, cuda, partition_size=ps)
    if case in ("sorted", "queue"):  # the launch mode the case is named for is the one that ran
        g = wl.to(cuda)
        info = T.plan_decode(torch.empty_like(g.query), g.query, g.key_cache, g.value_cache, g.context_lens, g.block_tables,
                             g.softmax_scale, g.q_len, g.max_context_len, torch.bfloat16, None, g.key_scale, g.value_scale,
                             partition_size=ps, query_lens=g.q_lens).launch_info()
        assert ("sorted items" if case == "sorted" else "queued items") in info, info
    assert not torch.isnan(out.float()).any()
    assert bool((out[empty] == 0).all())
    live = [i for i in range(len(ctx)) if not bool(empty[i])]
    ref = _oracle(wl, seq_ids=live)
    torch.testing.assert_close(out[live].float(), ref[live].float(), atol=ATOL, rtol=RTOL)


@pytest.mark.parametrize("name", ["fp8_g8", "fp8_token_g16_q4", "fp8_g10_q3"])
@pytest.mark.parametrize("gain", [4.0, 12.0])
def test_large_logits(cuda, name, gain):
    """Queries scaled up until the scaled logits reach tens (sharp softmax, as trained models produce): the
    FP8 MFMAs must see the bf16 query exactly (a power-of-two row factor makes head + residual exact), or the
    logit error, proportional to the logit, breaks the output tolerance."""
    wl = _make(**CASES[name])
    wl = type(wl)(**{**wl.__dict__, "query": (wl.query.float() * gain).to(wl.query.dtype)})
    out, res = _run(wl, cuda, partition_size=512)
    torch.testing.assert_close(out.float(), _oracle(wl).float(), atol=ATOL, rtol=RTOL)
    _check_stages(wl, res, 512)


@pytest.mark.parametrize("case", ["queue", "sorted", "plain", "teams", "own_cut"])
def test_graph_capture_and_replay(cuda, case):
    """A decode plan allocates nothing and only launches kernels on the given stream, so it can be captured
    in a HIP graph: every replay (with eager work and synchronisations in between, and with new inputs written
    into the captured tensors) must reproduce the eager result bit for bit.  Covers the launch modes that keep
    state in the workspace: the work queue (its counters return to zero) and the sorted dispatch (its list is
    rebuilt by every call); a launch in teams; and the output-only flag with the library's own cut of a prime
    partition count (the kernel that limits the context lengths is part of the graph)."""
    import triton_op_amd as T

    gen = torch.Generator().manual_seed(31)
    if case == "queue":  # bf16 cache, 64 query rows (two workgroups of two row tiles), ragged query lengths: the queued launch
        kw = dict(batch=6, num_q_heads=32, num_kv_heads=2, context_lens=_ctx(300, 64, 1000, 17, 700, 256), q_len=4,
                  q_lens=_ctx(1, 4, 2, 3, 4, 1), kv_dtype="bf16", scale_mode="none")
    elif case == "sorted":  # several rounds of workgroups: the planning kernel runs inside the graph
        # (32 rows per kv head: one item per partition; with up to 16 rows the workgroups would walk four
        # partitions each and 96 sequences would be a single round)
        kw = dict(batch=96, num_q_heads=128, num_kv_heads=8, q_len=2,
                  context_lens=torch.randint(2, 2600, (96,), generator=gen, dtype=torch.int32))
    elif case == "teams":  # one workgroup per (sequence, kv head) that merges its partitions itself: a single kernel
        kw = dict(batch=52, num_q_heads=64, num_kv_heads=8,
                  context_lens=torch.randint(1, 2049, (52,), generator=gen, dtype=torch.int32))
    elif case == "own_cut":  # output-only, a prime partition count: the limited context lengths are made inside the graph
        kw = dict(batch=16, num_q_heads=16, num_kv_heads=2,
                  context_lens=torch.cat([torch.randint(1, 3328, (15,), generator=gen, dtype=torch.int32), _ctx(3328)]))
    else:
        kw = dict(batch=3, num_q_heads=16, num_kv_heads=2, context_lens=_ctx(300, 64, 1000))
    wl = _make(**kw)
    g = wl.to(cuda)
    out = torch.full_like(g.query, float("nan"))
    plan = T.plan_decode(out, g.query, g.key_cache, g.value_cache, g.context_lens, g.block_tables, g.softmax_scale,
                         g.q_len, g.max_context_len, torch.bfloat16, None, g.key_scale, g.value_scale,
                         partition_size=256, query_lens=g.q_lens, output_only=case == "own_cut")
    if case != "plain":  # the launch mode the case is named for is the one that is captured
        mode = {"queue": "queued items", "sorted": "sorted items", "teams": "teams of 4 waves", "own_cut": "own partitions of 512 tokens"}
        assert mode[case] in plan.launch_info(), plan.launch_info()
    plan.run()
    torch.cuda.synchronize()
    eager = out.clone()
    torch.testing.assert_close(eager.float().cpu(), _oracle(wl).float(), atol=ATOL, rtol=RTOL)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        plan.run(stream=side.cuda_stream)  # warm-up on the capture stream
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            plan.run(stream=side.cuda_stream)
    torch.cuda.synchronize()
    q2 = (g.query.float() * 0.5).to(g.query.dtype)
    for i in range(3):
        out.fill_(float("nan"))
        (g.key_cache.float()[:1] * 1.0).sum().item()  # unrelated eager work and a host sync between replays
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), eager.view(torch.int16)), f"replay {i}"
    # new inputs through the captured tensors: the graph computes the new result
    g.query.copy_(q2)
    graph.replay()
    torch.cuda.synchronize()
    wl2 = type(wl)(**{**wl.__dict__, "query": q2.cpu()})
    torch.testing.assert_close(out.float().cpu(), _oracle(wl2).float(), atol=ATOL, rtol=RTOL)


@pytest.mark.parametrize("name", ["fp8_g8", "fp8_token_g16_q4"])
def test_negative_softmax_scale(cuda, name):
    """A negative scale turns the row maximum of the raw logits into the minimum of the scaled ones: the
    kernels must not assume the scale's sign when they take maxima before scaling."""
    wl = _make(**CASES[name])
    wl = type(wl)(**{**wl.__dict__, "softmax_scale": -wl.softmax_scale})
    out, _ = _run(wl, cuda, partition_size=512)
    torch.testing.assert_close(out.float(), _oracle(wl).float(), atol=ATOL, rtol=RTOL)


def test_c_abi_rejects_bad_arguments(cuda, pa_lib):
    import triton_op_amd as T
    from triton_op_amd import _cabi

    wl = _make(batch=2, num_q_heads=8, num_kv_heads=1, context_lens=_ctx(100, 300)).to(cuda)
    out = torch.empty_like(wl.query)
    plan = T.plan_decode(out, wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables,
                         wl.softmax_scale, 1, 300, torch.bfloat16, None, wl.key_scale, wl.value_scale)
    a = plan.args
    assert pa_lib.pa_decode(None, None) == -1
    for field, bad, code in (("struct_size", 8, -2), ("head_size", 96, -3), ("block_size", 32, -3), ("stride_bt_s", 0, -4),
                             ("partition_size", 100, -4), ("key_cache", None, -1), ("num_seqs", 0, -4),
                             ("stride_k_b", 8, -4)):
        good = getattr(a, field)
        setattr(a, field, bad)
        assert pa_lib.pa_decode(C.byref(a), None) == code, field
        setattr(a, field, good)
    assert pa_lib.pa_decode(C.byref(a), C.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0
    torch.cuda.synchronize()
    assert pa_lib.pa_decode_error_string(-3).decode().startswith("unsupported")


@pytest.mark.parametrize("name,batch,ctx_scale", [
    ("c1", None, 1.0), ("c2", 8, 0.25), ("c3", 6, 0.125), ("c4", 1, 1 / 32), ("c5", 12, 0.25)])
def test_scaled_down_benchmark_configs(cuda, name, batch, ctx_scale):
    from triton_op_amd import workloads as W

    wl = W.make_config(name, batch=batch, ctx_scale=ctx_scale)
    print(f"config={wl.name} ctx={wl.context_lens.tolist()}", flush=True)
    out, res = _run(wl, cuda, partition_size=None)
    torch.testing.assert_close(out.float(), _oracle(wl).float(), atol=ATOL, rtol=RTOL)
    # the tuning layer with the second statistic, the sum of the context lengths (a host value)
    out2, res2 = _run(wl, cuda, partition_size=None, total_context_tokens=int(wl.context_lens.sum()))
    torch.testing.assert_close(out2.float(), _oracle(wl).float(), atol=ATOL, rtol=RTOL)
    assert res2["partition_size"] <= res["partition_size"]  # fewer tokens than batch x longest: never coarser


def _random_case(seed):
    """One seeded draw over the whole supported parameter space of the op."""
    gen = torch.Generator().manual_seed(1000 + seed)

    def pick(options):
        return options[int(torch.randint(0, len(options), (1,), generator=gen))]

    kv_dtype = pick(["fp8", "fp8", "fp8", "bf16"])
    block_size = pick([16, 16, 64, 1024])
    q_len = pick([1, 1, 2, 3, 4])
    group = pick([g for g in (1, 2, 3, 4, 5, 7, 8, 10, 12, 16, 16, 16) if g * q_len <= 64 and (kv_dtype == "fp8" or g * q_len <= 16)])
    hkv = pick([1, 2, 3])
    batch = pick([1, 2, 3, 5])
    max_ctx = pick([40, 300, 1100, 2600])
    ctx = torch.randint(q_len, max_ctx + 1, (batch,), generator=gen, dtype=torch.int32)
    kw = dict(batch=batch, num_q_heads=group * hkv, num_kv_heads=hkv, context_lens=ctx, q_len=q_len,
              block_size=block_size, kv_dtype=kv_dtype, seed=seed,
              scale_mode="none" if kv_dtype == "bf16" else pick(["tensor", "token"]),
              transposed_v=pick([False, True]))
    if q_len > 1 and pick([False, True]):
        kw["q_lens"] = torch.randint(1, q_len + 1, (batch,), generator=gen, dtype=torch.int32)
    ps = pick([256, 512, 768, 2048, None])
    alibi = pick([False, False, True])
    return kw, ps, alibi


def _sweep_seeds():
    """48 seeds in every run; PA_SWEEP_SEEDS=lo:hi (e.g. 48:14048) runs that range instead -- a soak for whoever
    changes the kernels (about a minute per 2000 seeds on the GPU)."""
    import os

    span = os.environ.get("PA_SWEEP_SEEDS", "")
    if span:
        lo, _, hi = span.partition(":")
        return range(int(lo), int(hi))
    return range(48)


@pytest.mark.parametrize("seed", _sweep_seeds())
def test_seeded_random_sweep(cuda, seed):
    """Random shapes, layouts, scale modes, partition sizes and ALiBi: the HIP path against the oracle end to
    end and stage by stage."""
    kw, ps, alibi = _random_case(seed)
    print(f"seed={seed} ps={ps} alibi={alibi} " + " ".join(f"{k}={v.tolist() if torch.is_tensor(v) else v}" for k, v in kw.items()),
          flush=True)
    wl = _make(**kw)
    # odd seeds: one slope per packed query row (the reference kernels' array), even seeds: one per query head
    slopes = torch.linspace(0.02, 0.4, wl.query.shape[1] if seed % 2 else wl.num_q_heads, dtype=torch.float32) if alibi else None
    out, res = _run(wl, cuda, partition_size=ps, alibi=slopes)
    assert not torch.isnan(out.float()).any()
    torch.testing.assert_close(out.float(), _oracle(wl, slopes).float(), atol=ATOL, rtol=RTOL)
    _check_stages(wl, res, res["partition_size"], slopes)


@pytest.mark.parametrize("num_q_heads,q_len,scale_mode", [(16, 1, "tensor"), (32, 2, "token")])
def test_understated_max_sequence_length_cuts_the_context_off(cuda, num_q_heads, q_len, scale_mode):
    """max_sequence_length sizes the partition axis; a context that is longer than the axis covers is attended to up
    to the end of the last partition only, whatever the length of the axis.  With an axis of length ONE that used to
    leave the output rows unwritten (the partition kernel wrote them only for contexts inside the partition, and no
    reduce kernel follows a single partition): now the single partition's result is the output, as the clamped
    merge gives it for longer axes.  Checked against the oracle on the cut-off context (q_len 1: the cut is the
    whole difference; q_len 2: the new tokens' causal offsets still count from the true context length, so only
    the sequences that fit are compared with the oracle and the long one with the two-partition call's clamp)."""
    import triton_op_amd as T

    ctx_true = _ctx(700, 100, 512)
    wl = _make(batch=3, num_q_heads=num_q_heads, num_kv_heads=2, context_lens=ctx_true, q_len=q_len, scale_mode=scale_mode)
    g = wl.to(cuda)
    for stated, ps in ((512, 512), (1024, 512)):
        out = torch.full_like(g.query, float("nan"))
        print(f"stated max_sequence_length={stated} partition_size={ps} heads={num_q_heads} q_len={q_len}", flush=True)
        res = T.paged_attention_decode(out, g.query, g.key_cache, g.value_cache, g.context_lens, g.block_tables,
                                       g.softmax_scale, q_len, stated, torch.bfloat16, None, g.key_scale, g.value_scale,
                                       partition_size=ps)
        torch.cuda.synchronize()
        assert res["maximum_logits"].shape[2] == stated // ps
        assert not torch.isnan(out.float()).any()  # every row written
        if stated == 1024:
            ref = _oracle(wl)  # the axis covers every context: nothing is cut
            torch.testing.assert_close(out.float().cpu(), ref.float(), atol=ATOL, rtol=RTOL)
            continue
        fits = [1, 2]
        ref = _oracle(wl, seq_ids=fits)
        torch.testing.assert_close(out[fits].float().cpu(), ref[fits].float(), atol=ATOL, rtol=RTOL)
        if q_len == 1:
            cut = type(wl)(**{**wl.__dict__, "context_lens": _ctx(512, 100, 512)})
            ref_cut = _oracle(cut, seq_ids=[0])
            torch.testing.assert_close(out[0].float().cpu(), ref_cut[0].float(), atol=ATOL, rtol=RTOL)


def _set_token_scales(wl, which, fn):
    """Replaces the per-token K or V scale of token tau of every sequence by fn(tau) (a tensor of ctx values)."""
    sc = getattr(wl, which).clone()
    for b in range(wl.batch):
        ctx = int(wl.context_lens[b])
        tau = torch.arange(ctx)
        pages = wl.block_tables[b, tau // wl.block_size].long()
        sc[pages, :, tau % wl.block_size, 0] = fn(tau)[:, None].expand(ctx, sc.shape[1])
    return type(wl)(**{**wl.__dict__, which: sc})


def _adversarial(wl, kind):
    """Data built to drive the softmax bookkeeping of the kernels to its corners; returns (workload, alibi slopes)."""
    step = lambda tau: tau // 64  # the kernels work in steps of 64 tokens
    slopes = None
    if kind in ("gain64", "gain64_vscales"):
        # logits of +-200: step maxima jump up and down by tens of powers of two, the softmax is nearly one-hot
        wl = type(wl)(**{**wl.__dict__, "query": (wl.query.float() * 64.0).to(wl.query.dtype)})
    if kind == "alibi2":
        # the bias climbs 128 (184 powers of two) per 64-token step: every step lies > 60 powers of two above the last
        slopes = torch.full((wl.query.shape[1],), 2.0)
    if kind == "kscale_waves":
        # per-token K scales x1, x64, x1, ... by step under a query gain of 8: step maxima rise by more than 60
        # powers of two from one step to the next and fall by as much in the one after
        wl = type(wl)(**{**wl.__dict__, "query": (wl.query.float() * 8.0).to(wl.query.dtype)})
        base = wl.key_scale
        wl = _set_token_scales(wl, "key_scale", lambda tau: float(base.mean()) * torch.where(step(tau) % 2 == 1, 64.0, 1.0))
    if kind in ("vscales", "gain64_vscales"):
        # per-token V scales 2^-40 ... 2^+40 ... 2^-40 inside one partition: a triangle over the steps, and +-3 powers of
        # two from token to token
        def vs(tau):
            ns = int(step(tau).max()) + 1
            tri = 40.0 - 80.0 * (step(tau).float() / max(ns - 1, 1) - 0.5).abs() * 2.0 if ns > 1 else torch.zeros(len(tau))
            return torch.exp2(torch.round(tri) + (tau % 7).float() - 3.0)
        wl = _set_token_scales(wl, "value_scale", vs)
    if kind == "vscales_rising":
        # V scales that only grow, 2^-60 to 2^+60: the accumulator's unit has to follow them up
        wl = _set_token_scales(wl, "value_scale", lambda tau: torch.exp2(torch.round(-60.0 + 120.0 * tau.float() / max(len(tau) - 1, 1))))
    if kind == "vscales_falling_logits_rising":
        # the V scales fall by 2^100 while the logits climb by as much: each alone is far outside the window the
        # kernel follows without re-basing, together they cancel and every token carries about the same weight
        wl = type(wl)(**{**wl.__dict__, "query": (wl.query.float() * 0.0).to(wl.query.dtype)})
        n_tok = lambda tau: max(len(tau) - 1, 1)
        wl = _set_token_scales(wl, "value_scale", lambda tau: torch.exp2(50.0 - torch.round(100.0 * tau.float() / n_tok(tau))))
        slopes = torch.full((wl.query.shape[1],), 100.0 * math.log(2.0) / max(int(wl.context_lens.max()) - 1, 1))
    return wl, slopes


@pytest.mark.parametrize("rows", ["g8_q1", "g8_q4", "g16_q4", "g16_q3_bs1024", "g8_q4_head64", "g16_q4_head256"])
@pytest.mark.parametrize("kind", ["gain64", "alibi2", "kscale_waves", "vscales", "gain64_vscales", "vscales_rising",
                                  "vscales_falling_logits_rising"])
def test_adversarial_softmax_levels(cuda, kind, rows):
    """The softmax state of the kernels under data that drives it to its corners: logits that jump by more than 60
    powers of two between 64-token steps, up and down; per-token V scales that span 2^-40 ... 2^+40 (and 2^-60 ...
    2^+60) inside one partition; both at once; V scales and logits that drift 100 powers of two in opposite
    directions.  8 query rows per kv head run pa_partition_kernel (running maximum), 32 rows the shared-stream
    kernel with two waves per row tile, 64 and 48 rows with one (reference maximum that is re-based).  Every output
    must be finite and meet the oracle at the usual bar, measured against each row's own magnitude (the outputs
    reach 2^40); the partition buffers are held against the oracle's partition stage."""
    g, q_len, bs, hd = dict(g8_q1=(8, 1, 16, 128), g8_q4=(8, 4, 16, 128), g16_q4=(16, 4, 16, 128),
                            g16_q3_bs1024=(16, 3, 1024, 128), g8_q4_head64=(8, 4, 16, 64),
                            g16_q4_head256=(16, 4, 16, 256))[rows]  # (the last two: the generic kernels)
    wl = _make(batch=3, num_q_heads=2 * g, num_kv_heads=2, context_lens=_ctx(2048, 700, 1030), q_len=q_len,
               scale_mode="token", block_size=bs, seed=17, head_size=hd)
    wl, slopes = _adversarial(wl, kind)
    ref = _oracle(wl, slopes).float()
    assert bool(torch.isfinite(ref).all())
    mag = ref.abs().amax(dim=-1, keepdim=True).clamp_min(1e-30)
    for ps in (2048, 512):
        print(f"kind={kind} rows={rows} partition_size={ps}", flush=True)
        out, res = _run(wl, cuda, partition_size=ps, alibi=slopes)
        o = out.float()
        assert bool(torch.isfinite(o).all()), "non-finite output"
        torch.testing.assert_close(o / mag, ref / mag, atol=ATOL, rtol=RTOL)
        P = res["maximum_logits"].shape[2]
        ml, es, to = O.partition_stage(wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables,
                                       wl.softmax_scale, wl.q_len, wl.key_scale, wl.value_scale, slopes, ps, P, q_max=wl.q_len)
        gml, ges, gto = res["maximum_logits"].cpu(), res["exponential_sums"].cpu(), res["temporary_output"].float().cpu()
        reach = (torch.arange(P)[None, :] * ps < wl.context_lens[:, None])[:, None, :, None].expand_as(ml)
        fin = torch.isfinite(ml) & reach
        assert torch.equal(gml[reach & ~torch.isfinite(ml)], ml[reach & ~torch.isfinite(ml)])
        # (logits in the hundreds carry f32 rounding of a few 1e-3 absolute, in the kernel and in the oracle alike, and
        # a near one-hot softmax turns that into parts in a hundred of the sum of exponentials)
        torch.testing.assert_close(gml[fin], ml[fin], atol=2e-3, rtol=2e-4)
        torch.testing.assert_close(ges[reach], es[reach], atol=2e-3, rtol=2e-2)
        tmag = to.abs().amax(dim=-1, keepdim=True).clamp_min(1e-30)
        assert bool(torch.isfinite(gto[reach[..., None].expand_as(to)]).all())
        sel = reach[..., None].expand_as(to)
        torch.testing.assert_close((gto / tmag)[sel], (to / tmag)[sel], atol=ATOL, rtol=RTOL)


@pytest.mark.parametrize("group,q_len,ragged,with_sinks", [(8, 1, False, False), (6, 4, True, False), (8, 3, False, True),
                                                          (16, 2, True, True)])
def test_many_partitions_of_few_rows_take_the_wide_reduce(cuda, group, q_len, ragged, with_sinks):
    """A handful of long sequences at the reference's 256-token partitions: few 16-row units with 64 partitions or
    more each go to the reduce kernel whose workgroup splits the partition axis over its sixteen waves.  In the
    batch: 79 and 67 partitions, two partitions, one partition (finished by the partition kernel: the merge must
    leave its rows alone in pa_decode and reproduce them in pa_decode_reduce), an empty sequence; 8, 24, 24 and 32
    rows per kv head (units of 8 and 16 rows, padding rows of a ragged batch, rows of padding query positions)."""
    import triton_op_amd as T

    ctx = _ctx(20000, 300, 17000, 100, q_len)
    q_lens = _ctx(q_len, 1, max(1, q_len - 1), q_len, 1) if ragged else None
    wl = _make(batch=5, num_q_heads=group * 2, num_kv_heads=2, context_lens=ctx, q_len=q_len, q_lens=q_lens, seed=29)
    ctx0 = ctx.clone()
    ctx0[4] = 0  # declared empty after the generator gave it a page
    wl = type(wl)(**{**wl.__dict__, "context_lens": ctx0})
    g = wl.to(cuda)
    sinks = torch.linspace(-2.0, 3.0, wl.query.shape[1], dtype=torch.float32) if with_sinks else None
    out = torch.full_like(g.query, float("nan"))
    plan = T.plan_decode(out, g.query, g.key_cache, g.value_cache, g.context_lens, g.block_tables, g.softmax_scale, q_len,
                         20000, torch.bfloat16, None, g.key_scale, g.value_scale, partition_size=256, query_lens=g.q_lens,
                         sinks=None if sinks is None else sinks.to(cuda))
    assert plan.args.max_num_partitions == 79
    plan.run()
    torch.cuda.synchronize()
    live = [0, 1, 2, 3]
    ref = O.paged_attention_decode_oracle(wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables,
                                          wl.softmax_scale, q_len if q_lens is None else q_lens, wl.key_scale, wl.value_scale,
                                          seq_ids=live, sinks=sinks, q_max=q_len)
    assert not torch.isnan(out.float()).any()
    assert bool((out[4] == 0).all())
    torch.testing.assert_close(out.float().cpu()[live], ref.float()[live], atol=ATOL, rtol=RTOL)
    # the merge alone (every sequence, also the one-partition one) on the kernel's own buffers against the closed form
    first = out.clone()
    out.fill_(float("nan"))
    plan.run_reduce()
    torch.cuda.synchronize()
    if sinks is None:
        merged = O.reduce_stage(plan.max_logits.cpu(), plan.exp_sums.cpu(), plan.tmp_output.float().cpu(), wl.context_lens, 256)
        torch.testing.assert_close(out.float().cpu(), merged.float(), atol=4e-3, rtol=8e-3)  # bf16 rounding only
    torch.testing.assert_close(out.float().cpu(), first.float().cpu(), atol=4e-3, rtol=8e-3)


@pytest.mark.parametrize("num_q_heads,q_len,batch", [(16, 1, 8), (16, 1, 9), (32, 2, 8), (32, 4, 16)])
def test_heads_of_an_item_on_one_xcd_in_plain_order(cuda, num_q_heads, q_len, batch):
    """Per-token scales: workgroup ids are mapped so that an XCD takes every eighth (sequence, partition) item with
    all its kv heads, the grid is padded to whole groups of eight items, and in plain (unsorted) order each partition
    index starts the batch one sequence further on.  A skewed batch whose partition count exceeds the batch size
    (the rotation wraps) and is not a multiple of eight, both partition kernels, stage-wise and end to end."""
    import triton_op_amd as T

    ctx = torch.full((batch,), 100, dtype=torch.int32)
    ctx[1] = 256 * 11 - 7          # 11 partitions of 256: more than a batch of 8 or 9
    ctx[batch - 1] = 700
    wl = _make(batch=batch, num_q_heads=num_q_heads, num_kv_heads=2, context_lens=ctx, q_len=q_len, scale_mode="token")
    g = wl.to(cuda)
    info = T.plan_decode(torch.empty_like(g.query), g.query, g.key_cache, g.value_cache, g.context_lens, g.block_tables,
                         g.softmax_scale, g.q_len, g.max_context_len, torch.bfloat16, None, g.key_scale, g.value_scale,
                         partition_size=256).launch_info()
    assert "an item's heads on one XCD" in info and "sorted items" not in info, info
    out, res = _run(wl, cuda, partition_size=256)
    _check_stages(wl, res, 256)
    ref = _oracle(wl)
    assert torch.allclose(out.float(), ref.float(), atol=ATOL, rtol=RTOL)


@pytest.mark.parametrize("name", ["fp8_g8", "fp8_g16_q4", "fp8_token_ragged", "fp8_ragged_two_waves_per_tile",
                                  "fp8_token_ragged_two_waves_per_tile", "bf16_ragged_g16_q4", "bf16_g16_q4",
                                  "fp8_g8_q4_long", "fp8_bs1024_q2", "fp8_token_g8_q1"])
@pytest.mark.parametrize("partition_size", [256, 1024, 4096])
@pytest.mark.parametrize("with_sinks", [False, True])
def test_output_only_flag(cuda, pa_lib, name, partition_size, with_sinks):
    """PA_DECODE_FLAG_OUTPUT_ONLY: the caller reads only the real query rows of `output`.  Those rows equal, bit for
    bit, the flagless call's at the partition size the library cuts the axis into under the flag (a multiple of the
    caller's; `pa_decode_launch_info` names it), and so the oracle's, which that call is tested against; rows beyond a sequence's
    query length are never NaN-poisoned into real rows; a sequence that stage 1 finishes leaves its padding rows as
    they were and its partition-buffer entries untouched; the two stage entry points called one by one with the flag
    give the same rows as pa_decode."""
    import triton_op_amd as T

    wl = _make(**CASES[name])
    g = wl.to(cuda)
    G = g.query.shape[1] // (g.q_len * g.key_cache.shape[1])
    sinks = None
    if with_sinks:
        sinks = torch.linspace(-1.0, 1.0, g.query.shape[1], dtype=torch.float32, device=cuda)

    def plan(out, **kw):
        return T.plan_decode(out, g.query, g.key_cache, g.value_cache, g.context_lens, g.block_tables, g.softmax_scale,
                             g.q_len, g.max_context_len, torch.bfloat16, None, g.key_scale, g.value_scale,
                             partition_size=partition_size, query_lens=g.q_lens, sinks=sinks, **kw)

    out = torch.full_like(g.query, 7.0)
    p = plan(out, output_only=True)
    p.exp_sums.fill_(-3.0)
    p.run()
    # with the flag the library may cut the partition axis into fewer, longer partitions (the launch says so): the
    # flagless call to compare with is the one at that partition size
    info = p.launch_info()
    own_size = int(info.split("own partitions of ")[1].split()[0]) if "own partitions of" in info else partition_size
    assert own_size % partition_size == 0, info
    ref = torch.full_like(g.query, float("nan"))
    T.plan_decode(ref, g.query, g.key_cache, g.value_cache, g.context_lens, g.block_tables, g.softmax_scale,
                  g.q_len, g.max_context_len, torch.bfloat16, None, g.key_scale, g.value_scale,
                  partition_size=own_size, query_lens=g.q_lens, sinks=sinks).run()
    two = torch.full_like(g.query, 7.0)
    p2 = plan(two, output_only=True)
    p2.run_partition()
    p2.run_reduce()
    torch.cuda.synchronize()
    Hkv, q_max = g.key_cache.shape[1], g.q_len
    qls = g.q_lens.cpu().tolist() if g.q_lens is not None else [q_max] * g.query.shape[0]
    ctxs = g.context_lens.cpu().tolist()
    view = lambda t: t.view(t.shape[0], Hkv, q_max, G, -1)
    for b, (ql, ctx) in enumerate(zip(qls, ctxs)):
        live = (view(out)[b, :, :ql], view(two)[b, :, :ql], view(ref)[b, :, :ql])
        assert torch.equal(live[0], live[2]) and torch.equal(live[1], live[2]), f"sequence {b}"
        finished_by_stage_1 = (ctx <= partition_size or p.max_logits.shape[2] == 1) and sinks is None
        if finished_by_stage_1 and ctx > 0:
            assert torch.all(view(out)[b, :, ql:] == 7.0), f"padding rows of sequence {b} were written"
            assert torch.all(p.exp_sums[b] == -3.0), f"partition-buffer entries of sequence {b} were written"


@pytest.mark.parametrize("batch,hkv,group,q_len,P,scale_mode,own",
                         [(16, 2, 8, 1, 13, "tensor", 512), (24, 8, 8, 1, 29, "tensor", 2560),
                          (40, 4, 8, 4, 29, "token", 1536), (12, 8, 16, 4, 13, "token", 768)])
def test_output_only_cut_that_does_not_divide_the_partition_count(cuda, batch, hkv, group, q_len, P, scale_mode, own):
    """PA_DECODE_FLAG_OUTPUT_ONLY with reference-shaped buffers (256-token partitions) whose partition count is a
    prime: the library's own, longer partitions do not end where the caller's axis ends, so the kernels get the
    context lengths with the caller's limit applied (a copy in the workspace).  One sequence's true context is
    longer than the stated maximum: it is cut off at the end of the caller's axis, as without the flag (compared with
    the oracle on the cut context when there is one new token; with several, the causal offsets of a cut-off sequence
    count from the cut, and it is only checked to be finite).  The stage entry points called one by one give the
    same bits; without a workspace the cut falls back to a divisor of the partition count (none for a prime: the
    caller's partitions), with the same rows to the parity tolerance."""
    import triton_op_amd as T

    ps, axis = 256, 256 * P
    gen = torch.Generator().manual_seed(4242 + P + batch)
    ctx = torch.randint(1, axis + 1, (batch,), generator=gen, dtype=torch.int32)
    ctx[0], ctx[1], ctx[2] = axis, 1, axis + 300  # (the third: longer than the stated maximum)
    ctx = torch.clamp(ctx, min=q_len)
    q_lens = torch.randint(1, q_len + 1, (batch,), generator=gen, dtype=torch.int32) if q_len > 1 else None
    wl = _make(batch=batch, num_q_heads=group * hkv, num_kv_heads=hkv, context_lens=ctx, q_len=q_len, q_lens=q_lens,
               kv_dtype="fp8", scale_mode=scale_mode, block_size=16, seed=4242 + P)
    g = wl.to(cuda)

    def plan(out, **kw):
        return T.plan_decode(out, g.query, g.key_cache, g.value_cache, g.context_lens, g.block_tables, g.softmax_scale,
                             q_len, axis, torch.bfloat16, None, g.key_scale, g.value_scale, partition_size=ps,
                             query_lens=g.q_lens, output_only=True, **kw)

    out = torch.full_like(g.query, 7.0)
    p = plan(out)
    assert p.args.max_num_partitions == P
    assert f"own partitions of {own} tokens" in p.launch_info() and P % (own // ps) != 0, p.launch_info()
    p.run()
    two = torch.full_like(g.query, 7.0)
    p2 = plan(two)
    p2.run_partition()
    p2.run_reduce()
    bare = torch.full_like(g.query, 7.0)
    p3 = plan(bare)
    p3.args.workspace = None
    p3.args.workspace_bytes = 0
    assert "own partitions" not in p3.launch_info(), p3.launch_info()
    p3.run()
    torch.cuda.synchronize()
    by_pos = lambda t: t.float().cpu().view(batch, hkv, q_len, group, -1)
    cut = type(wl)(**{**wl.__dict__, "context_lens": torch.clamp(ctx, max=axis)})
    want = by_pos(_oracle(cut))
    got, got2, got3 = by_pos(out), by_pos(two), by_pos(bare)
    for b in range(batch):
        n = q_len if q_lens is None else int(q_lens[b])
        assert torch.equal(got[b, :, :n], got2[b, :, :n]), b
        assert torch.isfinite(got[b, :, :n]).all() and torch.isfinite(got3[b, :, :n]).all(), b
        if b == 2 and q_len > 1:
            continue
        torch.testing.assert_close(got[b, :, :n], want[b, :, :n], atol=ATOL, rtol=RTOL)
        torch.testing.assert_close(got3[b, :, :n], want[b, :, :n], atol=ATOL, rtol=RTOL)


def _random_case_wide(seed):
    """A second seeded draw: larger batches (launches of several rounds: sorted dispatch, grids padded to whole groups
    of eight items, the item list's reuse), attention sinks, an FP8 query with per-row or per-tensor scale, the
    caller's total-token statistic and PA_DECODE_FLAG_OUTPUT_ONLY, in any combination."""
    gen = torch.Generator().manual_seed(777000 + seed)

    def pick(options):
        return options[int(torch.randint(0, len(options), (1,), generator=gen))]

    kv_dtype = pick(["fp8", "fp8", "fp8", "bf16"])
    q_len = pick([1, 2, 4])
    group = pick([g for g in (1, 4, 8, 16) if g * q_len <= 64])
    hkv = pick([1, 2, 8])
    batch = pick([3, 17, 40, 64])
    shape = pick(["short", "mixed", "skewed"])
    hi = {"short": 300, "mixed": 1500, "skewed": 200}[shape]
    ctx = torch.randint(q_len, hi + 1, (batch,), generator=gen, dtype=torch.int32)
    if shape == "skewed":
        ctx[int(torch.randint(0, batch, (1,), generator=gen))] = pick([3000, 6000])
    kw = dict(batch=batch, num_q_heads=group * hkv, num_kv_heads=hkv, context_lens=ctx, q_len=q_len,
              block_size=pick([16, 16, 64]), kv_dtype=kv_dtype, seed=seed,
              scale_mode="none" if kv_dtype == "bf16" else pick(["tensor", "token"]), transposed_v=pick([False, True]))
    if q_len > 1 and pick([False, True]):
        kw["q_lens"] = torch.randint(1, q_len + 1, (batch,), generator=gen, dtype=torch.int32)
    opts = dict(partition_size=pick([256, 256, 512, None]), sinks=pick([False, True]),
                fp8_query=pick(["no", "no", "row", "tensor"]), output_only=pick([False, True]),
                total=pick([False, True]), alibi=pick([False, False, True]))
    # every third seed on one of the generic kernels' head sizes (not drawn: the draws above stay what they were)
    if seed % 3 == 2:
        kw["head_size"] = 64 if seed % 2 else 256
    return kw, opts


def _wide_seeds():
    import os

    span = os.environ.get("PA_SWEEP_SEEDS_WIDE", "")
    if span:
        lo, _, hi = span.partition(":")
        return range(int(lo), int(hi))
    return range(32)


@pytest.mark.parametrize("seed", _wide_seeds())
def test_seeded_random_sweep_wide(cuda, seed):
    """The features the first sweep does not draw, against the oracle end to end (real query rows only when the call
    is made with output_only); PA_SWEEP_SEEDS_WIDE=lo:hi runs another range of the draw."""
    import triton_op_amd as T
    from triton_op_amd import kv_layout as L

    kw, o = _random_case_wide(seed)
    print(f"seed={seed} {o} " + " ".join(f"{k}={v.tolist() if torch.is_tensor(v) else v}" for k, v in kw.items()), flush=True)
    wl = _make(**kw)
    g = wl.to(cuda)
    rows = wl.query.shape[1]
    query, qscale = wl.query, None
    if o["fp8_query"] == "row":
        query, qscale = L.pertoken_quant(wl.query.float())
    elif o["fp8_query"] == "tensor":
        qscale = torch.tensor(max(float(wl.query.float().abs().max()), 1e-6) / 448.0)
        query = (wl.query.float() / qscale).to(torch.float8_e4m3fn)
    sinks = torch.linspace(-2.0, 2.0, rows, dtype=torch.float32) if o["sinks"] else None
    slopes = torch.linspace(0.02, 0.4, rows if seed % 2 else wl.num_q_heads, dtype=torch.float32) if o["alibi"] else None
    out = torch.full_like(g.query, float("nan"))
    dev = lambda t: None if t is None else t.to(cuda)
    T.paged_attention_decode(
        out, dev(query), g.key_cache, g.value_cache, g.context_lens, g.block_tables, g.softmax_scale, g.q_len,
        g.max_context_len, torch.bfloat16, dev(qscale), g.key_scale, g.value_scale, alibi_slopes=dev(slopes),
        partition_size=o["partition_size"], query_lens=g.q_lens, sinks=dev(sinks), output_only=o["output_only"],
        total_context_tokens=int(wl.context_lens.sum()) if o["total"] else 0)
    torch.cuda.synchronize()
    ref = O.paged_attention_decode_oracle(
        query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables, wl.softmax_scale,
        wl.q_len if wl.q_lens is None else wl.q_lens, wl.key_scale, wl.value_scale, slopes, None, query_scale=qscale,
        q_max=wl.q_len, sinks=sinks)
    got = out.float().cpu()
    hkv, q_max = wl.key_cache.shape[1], wl.q_len
    view = lambda t: t.view(t.shape[0], hkv, q_max, -1, t.shape[-1])
    qls = wl.q_lens.tolist() if wl.q_lens is not None else [q_max] * wl.batch
    for b, ql in enumerate(qls):  # the real query rows (the others are unspecified under output_only)
        torch.testing.assert_close(view(got)[b, :, :ql], view(ref.float())[b, :, :ql], atol=ATOL, rtol=RTOL)
    if not o["output_only"]:
        assert not torch.isnan(got).any()
        torch.testing.assert_close(got, ref.float(), atol=ATOL, rtol=RTOL)


GENERIC_HEAD_CASES = ["fp8_g8", "fp8_g8_boundaries", "fp8_g5_q2", "fp8_g16_q4", "fp8_token_ragged", "fp8_token_g8_q1",
                      "bf16_g8", "bf16_g16_q4", "fp8_bs1024_q2", "fp8_bs64", "fp8_transV_bs16", "fp8_transV_bs1024",
                      "fp8_token_transV_bs64_g8_q3", "bf16_ragged_g16_q4", "bf16_transV_bs64",
                      "fp8_ragged_two_waves_per_tile"]


@pytest.mark.parametrize("head_size", [64, 256])
@pytest.mark.parametrize("name", GENERIC_HEAD_CASES)
@pytest.mark.parametrize("partition_size", [256, 1024])
def test_head_sizes_64_and_256(cuda, head_size, name, partition_size):
    """Head sizes other than 128 run on the generic kernels (plain f32 arithmetic): the same cases as the tuned
    kernels', stage by stage and end to end against the oracle."""
    import triton_op_amd as T

    wl = _make(**CASES[name], head_size=head_size)
    g = wl.to(cuda)
    info = T.plan_decode(torch.empty_like(g.query), g.query, g.key_cache, g.value_cache, g.context_lens, g.block_tables,
                         g.softmax_scale, g.q_len, g.max_context_len, torch.bfloat16, None, g.key_scale, g.value_scale,
                         partition_size=partition_size, query_lens=g.q_lens).launch_info()
    assert info.startswith(f"pa_partition_generic_kernel<head size {head_size}"), info
    out, res = _run(wl, cuda, partition_size=partition_size)
    assert not torch.isnan(out.float()).any()
    _check_stages(wl, res, partition_size)
    torch.testing.assert_close(out.float(), _oracle(wl).float(), atol=ATOL, rtol=RTOL)


@pytest.mark.parametrize("head_size", [64, 256])
@pytest.mark.parametrize("feature", ["alibi_rows", "alibi_heads", "sinks", "fp8_query_rows", "fp8_query_tensor",
                                     "output_only", "noalloc", "stale_nan"])
def test_head_sizes_64_and_256_options(cuda, head_size, feature):
    """... and the operator's options on those head sizes."""
    import triton_op_amd as T
    from triton_op_amd import kv_layout as L

    wl = _make(batch=4, num_q_heads=32, num_kv_heads=2, context_lens=_ctx(700, 33, 300, 5), q_len=2,
               q_lens=_ctx(2, 1, 2, 2), scale_mode="token", head_size=head_size)
    g = wl.to(cuda)
    rows = wl.query.shape[1]
    query, qscale, slopes, sinks = wl.query, None, None, None
    if feature == "alibi_rows":
        slopes = torch.linspace(0.02, 0.4, rows, dtype=torch.float32)
    if feature == "alibi_heads":
        slopes = torch.linspace(0.02, 0.4, wl.num_q_heads, dtype=torch.float32)
    if feature == "sinks":
        sinks = torch.linspace(-2.0, 3.0, rows, dtype=torch.float32)
    if feature == "fp8_query_rows":
        query, qscale = L.pertoken_quant(wl.query.float())
    if feature == "fp8_query_tensor":
        qscale = torch.tensor(float(wl.query.float().abs().max()) / 448.0)
        query = (wl.query.float() / qscale).to(torch.float8_e4m3fn)
    if feature == "stale_nan":  # cache bytes past every sequence's end decode to NaN: they must never reach a result
        kc, vc = g.key_cache.view(torch.uint8).clone(), g.value_cache.view(torch.uint8).clone()
        bs = wl.key_cache.shape[-2]
        for b in range(wl.batch):
            ctx = int(wl.context_lens[b])
            blk = int(wl.block_tables[b, (ctx - 1) // bs])
            kc[blk, :, :, ctx % bs if ctx % bs else bs:, :] = 0x7f
            vc[blk, :, :, ctx % bs if ctx % bs else bs:] = 0x7f
        g = type(g)(**{**g.__dict__, "key_cache": kc.view(g.key_cache.dtype), "value_cache": vc.view(g.value_cache.dtype)})
    dev = lambda t: None if t is None else t.to(cuda)
    out = torch.full_like(g.query, 7.0)
    plan = T.plan_decode(out, dev(query), g.key_cache, g.value_cache, g.context_lens, g.block_tables, g.softmax_scale,
                         g.q_len, g.max_context_len, torch.bfloat16, dev(qscale), g.key_scale, g.value_scale,
                         alibi_slopes=dev(slopes), partition_size=256, query_lens=g.q_lens, sinks=dev(sinks),
                         output_only=feature == "output_only")
    if feature == "noalloc":
        plan.run_noalloc()
    else:
        plan.run()
    torch.cuda.synchronize()
    ref = O.paged_attention_decode_oracle(
        query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables, wl.softmax_scale, wl.q_lens,
        wl.key_scale, wl.value_scale, slopes, None, query_scale=qscale, q_max=wl.q_len, sinks=sinks)
    got = out.float().cpu()
    hkv, q_max = wl.key_cache.shape[1], wl.q_len
    view = lambda t: t.view(t.shape[0], hkv, q_max, -1, t.shape[-1])
    for b, ql in enumerate(wl.q_lens.tolist()):
        torch.testing.assert_close(view(got)[b, :, :ql], view(ref.float())[b, :, :ql], atol=ATOL, rtol=RTOL)
        if feature == "output_only":
            assert torch.all(view(got)[b, :, ql:] == 7.0)
    if feature != "output_only":
        torch.testing.assert_close(got, ref.float(), atol=ATOL, rtol=RTOL)


@pytest.mark.parametrize("num_q_heads,q_len", [(16, 1), (32, 4)])
def test_one_block_table_row_expanded_over_the_batch(cuda, num_q_heads, q_len):
    """Sequences that share their pages through ONE block-table row expanded over the batch (row stride 0): the entry
    point gives every row a stride of its own (the kernels request a row's first entries before they know the
    sequence's length and keep the index inside the row's stride; the C ABI refuses a stride below 1)."""
    import triton_op_amd as T

    wl = _make(batch=3, num_q_heads=num_q_heads, num_kv_heads=2, context_lens=_ctx(700, 700, 700), q_len=q_len,
               scale_mode="token")
    row = wl.block_tables[:1]
    shared = type(wl)(**{**wl.__dict__, "block_tables": row.expand(3, -1), "context_lens": _ctx(700, 33, 300)})
    g = shared.to(cuda)
    bt = g.block_tables[:1].expand(3, -1)
    assert bt.stride(0) == 0
    out = torch.full_like(g.query, float("nan"))
    T.paged_attention_decode(out, g.query, g.key_cache, g.value_cache, g.context_lens, bt, g.softmax_scale, g.q_len,
                             g.max_context_len, torch.bfloat16, None, g.key_scale, g.value_scale, partition_size=256)
    torch.cuda.synchronize()
    ref = _oracle(type(wl)(**{**shared.__dict__, "block_tables": row.expand(3, -1).contiguous()}))
    torch.testing.assert_close(out.float().cpu(), ref.float(), atol=ATOL, rtol=RTOL)
