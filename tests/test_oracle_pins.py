"""Pins the CPU oracle (oracle/pa_oracle.py) without running the reference: library routines,
closed forms, invariants and brute force on tiny inputs.  A dropped term, a wrong sign, a wrong
index or a transposed operand in the oracle fails at least one of these."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import pa_oracle as O
from triton_op_amd import kv_layout as L
from triton_op_amd import workloads as W


def _ctx(*v):
    return torch.tensor(v, dtype=torch.int32)


def test_e4m3fn_table_matches_torch_cast():
    tab = torch.from_numpy(O.e4m3fn_table())
    ref = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).to(torch.float32)
    assert torch.equal(torch.isnan(tab), torch.isnan(ref))
    assert int(torch.isnan(tab).sum()) == 2  # 0x7f and 0xff only; e4m3fn has no infinities
    ok = ~torch.isnan(ref)
    assert torch.equal(tab[ok], ref[ok])
    assert tab[0x7E] == 448.0 and tab[0xFE] == -448.0 and tab[0x01] == 2.0 ** -9


@pytest.mark.parametrize("qlen,klen,hq,hkv", [(1, 37, 8, 1), (2, 19, 6, 2), (4, 64, 4, 4), (3, 3, 5, 1)])
def test_masked_attention_matches_sdpa(qlen, klen, hq, hkv):
    g = torch.Generator().manual_seed(qlen * 100 + klen)
    q = torch.randn(qlen, hq, 32, generator=g)
    k = torch.randn(klen, hkv, 32, generator=g)
    v = torch.randn(klen, hkv, 32, generator=g)
    scale = 0.37
    out = O.masked_attention(q, k, v, scale, torch.float32, True)
    kk = k.repeat_interleave(hq // hkv, 1).permute(1, 0, 2)
    vv = v.repeat_interleave(hq // hkv, 1).permute(1, 0, 2)
    mask = torch.ones(qlen, klen, dtype=torch.bool).tril(diagonal=klen - qlen)
    ref = F.scaled_dot_product_attention(q.permute(1, 0, 2), kk, vv, attn_mask=mask, scale=scale).permute(1, 0, 2)
    torch.testing.assert_close(out, ref, atol=2e-6, rtol=1e-5)


def test_causal_rule_equals_tril_exhaustively():
    # test_pa_mtp.py:211 tril(diagonal=key_len-query_len)  ==  col + (q-1-t) < ctx  (kernel rule)
    for q in range(1, 5):
        for ctx in range(q, 9):
            tril = torch.ones(q, ctx, dtype=torch.bool).tril(diagonal=ctx - q)
            for t in range(q):
                for col in range(ctx):
                    assert bool(tril[t, col]) == (col + (q - 1 - t) < ctx)


def _tiny(kv_dtype="fp8", scale_mode="tensor", q_len=1, hq=4, hkv=2, bs=16, ctx=(5, 33, 16), seed=11, d=128):
    return W.make_decode_workload(
        name="tiny", seed=seed, batch=len(ctx), num_q_heads=hq, num_kv_heads=hkv, head_size=d, block_size=bs,
        context_lens=_ctx(*ctx), q_len=q_len, kv_dtype=kv_dtype, scale_mode=scale_mode)


def _oracle(wl, **kw):
    return O.paged_attention_decode_oracle(
        wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables, wl.softmax_scale,
        wl.q_len if wl.q_lens is None else wl.q_lens, wl.key_scale, wl.value_scale, **kw)


@pytest.mark.parametrize("kv_dtype,scale_mode,q_len", [
    ("fp8", "tensor", 1), ("fp8", "token", 2), ("bf16", "none", 1), ("fp8", "tensor", 3)])
def test_oracle_matches_double_precision_brute_force(kv_dtype, scale_mode, q_len):
    wl = _tiny(kv_dtype, scale_mode, q_len, hq=2, hkv=1, ctx=(q_len, 19, 35))
    bf = O.brute_force_decode(wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables,
                              wl.softmax_scale, q_len, wl.key_scale, wl.value_scale)
    ref = torch.tensor(bf, dtype=torch.float64)
    out = _oracle(wl).to(torch.float64)
    # the oracle's result is rounded to bf16 (8 significant bits)
    torch.testing.assert_close(out, ref, atol=2e-3, rtol=2 ** -8)


def test_block_permutation_invariance_is_bit_exact():
    wl = _tiny("fp8", "token", 2, ctx=(40, 7, 64))
    base = _oracle(wl)
    n = wl.key_cache.shape[0]
    perm = torch.randperm(n, generator=torch.Generator().manual_seed(3))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(n)
    kc, vc = wl.key_cache[perm], wl.value_cache[perm]  # new block i holds old block perm[i]
    ks, vs = wl.key_scale[perm], wl.value_scale[perm]
    bt = inv[wl.block_tables.long()].to(torch.int32)
    out = O.paged_attention_decode_oracle(wl.query, kc, vc, wl.context_lens, bt, wl.softmax_scale, 2, ks, vs)
    assert torch.equal(out, base)


def test_layout_round_trips_and_transposed_v():
    wl = _tiny("fp8", "tensor", 1)
    ktok = L.key_cache_to_tokens(wl.key_cache)
    assert torch.equal(L.tokens_to_key_cache(ktok).view(torch.uint8), wl.key_cache.view(torch.uint8))
    # flatten == the documented element rule K[page, h, d//x, tok, d%x]
    flat = O.flatten_key_cache(wl.key_cache).view(torch.uint8)
    kc = wl.key_cache.view(torch.uint8)
    for page, h, dd, tok in [(0, 0, 0, 0), (3, 1, 77, 5), (2, 0, 127, 15)]:
        assert flat[page * 16 + tok, h, dd] == kc[page, h, dd // 16, tok, dd % 16]
    vflat = O.flatten_value_cache(wl.value_cache).view(torch.uint8)
    vcu = wl.value_cache.view(torch.uint8)
    for page, h, dd, tok in [(0, 0, 0, 0), (3, 1, 77, 5), (2, 0, 127, 15)]:
        assert vflat[page * 16 + tok, h, dd] == vcu[page, h, dd, tok]
    vt = L.shuffle_value_cache_layout(wl.value_cache)
    assert vt.shape == (wl.value_cache.shape[0], 2, 1, 128, 16)
    assert torch.equal(L.unshuffle_value_cache_layout(vt).view(torch.uint8), vcu)
    assert torch.equal(O.flatten_value_cache(vt).view(torch.uint8), vflat)
    out_t = O.paged_attention_decode_oracle(wl.query, wl.key_cache, vt, wl.context_lens, wl.block_tables,
                                            wl.softmax_scale, 1, wl.key_scale, wl.value_scale)
    assert torch.equal(out_t, _oracle(wl))


def test_mtp_pack_round_trip_and_token_major_agreement():
    b, q, hkv, g = 3, 2, 2, 3
    wl = _tiny("fp8", "tensor", q, hq=hkv * g, hkv=hkv, ctx=(9, 40, 17))
    tok_major = O.mtp_unpack(wl.query, b, q, hkv)  # [B*q, Hq, D]
    assert torch.equal(O.mtp_pack(tok_major, b, q, hkv), wl.query)
    assert torch.equal(L.mtp_pack(tok_major, b, q, hkv), wl.query)
    assert torch.equal(L.mtp_unpack(wl.query, b, q, hkv), tok_major)
    # row h*(q*G) + t*G + g of the packed tensor is token t, head h*G+g
    assert torch.equal(wl.query[1, 1 * q * g + 1 * g + 2], tok_major[1 * q + 1, 1 * g + 2])
    indptr = [0, q, 2 * q, 3 * q]
    ref = O.mha_extend(tok_major, wl.key_cache, wl.value_cache, wl.block_tables, wl.context_lens, indptr,
                       wl.key_scale, wl.value_scale)
    assert torch.equal(O.mtp_pack(ref, b, q, hkv), _oracle(wl))


@pytest.mark.parametrize("q_len", [1, 2])
def test_partition_size_independence_and_one_partition_identity(q_len):
    wl = _tiny("fp8", "tensor", q_len, hq=8, hkv=2, ctx=(1000, 257, 256, 600))
    ref = _oracle(wl).float()
    outs = []
    for ps in (256, 512, 1024):
        ml, es, to = O.partition_stage(wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables,
                                       wl.softmax_scale, q_len, wl.key_scale, wl.value_scale, None, ps)
        out = O.reduce_stage(ml, es, to, wl.context_lens, ps, torch.float32)
        outs.append(out)
        torch.testing.assert_close(out.to(torch.bfloat16).float(), ref, atol=1e-2, rtol=1e-2)
        if ps == 1024:  # one partition: the merge is the identity on tmp_output
            assert ml.shape[2] == 1
            torch.testing.assert_close(out.view(4, 2, -1, 128), to[:, :, 0], atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(outs[0], outs[1], atol=2e-6, rtol=1e-5)
    torch.testing.assert_close(outs[0], outs[2], atol=2e-6, rtol=1e-5)


def test_reduce_stage_closed_form():
    # two partitions, one row, D=2: out = (l0 e^{m0-M} o0 + l1 e^{m1-M} o1) / (l0 e^{m0-M} + l1 e^{m1-M})
    ml = torch.tensor([1.0, 3.0]).view(1, 1, 2, 1)
    es = torch.tensor([2.0, 5.0]).view(1, 1, 2, 1)
    to = torch.tensor([[1.0, -2.0], [0.5, 4.0]]).view(1, 1, 2, 1, 2)
    out = O.reduce_stage(ml, es, to, _ctx(300), 256, torch.float32)
    w0, w1 = 2.0 * math.exp(1.0 - 3.0), 5.0
    exp = [(w0 * 1.0 + w1 * 0.5) / (w0 + w1), (w0 * -2.0 + w1 * 4.0) / (w0 + w1)]
    torch.testing.assert_close(out.view(-1), torch.tensor(exp), atol=1e-6, rtol=1e-6)
    # only ceil(ctx/partition) partitions count
    out1 = O.reduce_stage(ml, es, to, _ctx(256), 256, torch.float32)
    torch.testing.assert_close(out1.view(-1), torch.tensor([1.0, -2.0]))


def test_fully_masked_partition_row_has_zero_weight():
    # ctx=257, q=2: row t=0 sees keys [0,256), so in partition 1 (token 256 only) it sees nothing
    wl = _tiny("fp8", "tensor", 2, hq=2, hkv=1, ctx=(257,))
    ml, es, to = O.partition_stage(wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables,
                                   wl.softmax_scale, 2, wl.key_scale, wl.value_scale, None, 256)
    g = 2
    assert torch.isinf(ml[0, 0, 1, :g]).all() and (es[0, 0, 1, :g] == 0).all() and (to[0, 0, 1, :g] == 0).all()
    assert torch.isfinite(ml[0, 0, 1, g:]).all() and (es[0, 0, 1, g:] == 1).all()
    out = O.reduce_stage(ml, es, to, wl.context_lens, 256)
    assert torch.isfinite(out.float()).all()
    torch.testing.assert_close(out.float(), _oracle(wl).float(), atol=1e-2, rtol=1e-2)


def test_ragged_query_lens_match_per_sequence_calls():
    wl = W.make_decode_workload(name="rag", seed=5, batch=3, num_q_heads=4, num_kv_heads=2, context_lens=_ctx(20, 50, 9),
                                q_len=3, q_lens=_ctx(1, 3, 2), scale_mode="token")
    out = _oracle(wl)
    g = 2
    for b, qb in enumerate((1, 3, 2)):
        qv = wl.query[b].view(2, 3, g, 128)[:, :qb].reshape(1, 2 * qb * g, 128)
        o = O.paged_attention_decode_oracle(qv, wl.key_cache, wl.value_cache, wl.context_lens[b:b + 1],
                                            wl.block_tables[b:b + 1], wl.softmax_scale, qb, wl.key_scale, wl.value_scale)
        assert torch.equal(out[b].view(2, 3, g, 128)[:, :qb], o.view(2, qb, g, 128))
        assert (out[b].view(2, 3, g, 128)[:, qb:] == 0).all()


def test_alibi_matches_explicit_bias():
    wl = _tiny("bf16", "none", 1, hq=4, hkv=2, ctx=(30,))
    slopes = torch.tensor([0.5, 0.25, 0.125, 0.0625])
    out = _oracle(wl, alibi_slopes=slopes)
    k, v = O.gather_sequence(O.flatten_key_cache(wl.key_cache), O.flatten_value_cache(wl.value_cache), None, None,
                             wl.block_tables[0], 30, 16)
    q = wl.query[0].float()  # [Hq, D] since q_len=1
    for hq in range(4):
        s = (k[:, hq // 2] @ q[hq]) * wl.softmax_scale + slopes[hq] * (torch.arange(30) - 29).float()
        o = torch.softmax(s, 0) @ v[:, hq // 2]
        torch.testing.assert_close(out[0, hq].float(), o.to(torch.bfloat16).float(), atol=1e-2, rtol=1e-2)


def test_quantisers_closed_form():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(4, 2, 16, 128, generator=g)
    q, s = L.quantize_per_tensor(x)
    assert s.dim() == 0 and s.dtype == torch.float32
    assert float(s) == pytest.approx(float(x.abs().max()) / 448.0, rel=1e-6)
    assert float(q.float().abs().max()) == 448.0
    qt, st = L.pertoken_quant(x)
    assert st.shape == (4, 2, 16, 1)
    torch.testing.assert_close(st.squeeze(-1), x.abs().amax(-1) / 448.0)
    # dequantised error bounded by half an e4m3 ulp (2^-4 relative) of each element, plus subnormal step
    err = (qt.float() * st - x).abs()
    assert bool((err <= x.abs() * 2.0 ** -4 + st * 2.0 ** -10).all())
    z, sz = L.pertoken_quant(torch.zeros(2, 8))
    assert (sz == 1).all() and (z.float() == 0).all()


def test_golden_fixtures_match_oracle():
    import glob
    import os

    files = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz")))
    assert files, "no golden fixtures"
    from tests.golden.make_golden import load_case

    for f in files:
        case = load_case(f)
        out = O.paged_attention_decode_oracle(
            case["query"], case["key_cache"], case["value_cache"], case["context_lens"], case["block_tables"],
            case["softmax_scale"], case["q_len"], case["key_scale"], case["value_scale"])
        torch.testing.assert_close(out.double(), case["expected"], atol=2e-3, rtol=2 ** -8)


def test_sink_term_closed_form():
    # one query row, two keys: out = (e^{s0} v0 + e^{s1} v1) / (e^{s0} + e^{s1} + e^{sink})
    q = torch.tensor([[[1.0, 0.0]]])                       # [q=1, Hq=1, D=2]
    k = torch.tensor([[[2.0, 0.0]], [[-1.0, 0.0]]])        # [ctx=2, Hkv=1, D=2]
    v = torch.tensor([[[1.0, 10.0]], [[3.0, -4.0]]])
    sink = torch.tensor([[0.5]])
    out = O.masked_attention(q, k, v, 1.0, torch.float32, True, None, sink)
    e0, e1, es = math.exp(2.0), math.exp(-1.0), math.exp(0.5)
    exp = torch.tensor([(e0 * 1.0 + e1 * 3.0) / (e0 + e1 + es), (e0 * 10.0 + e1 * -4.0) / (e0 + e1 + es)])
    torch.testing.assert_close(out.view(-1), exp, atol=1e-6, rtol=1e-6)


def test_query_scale_equals_prescaled_query():
    """An FP8 query with its scale must give what the f32 product (query * scale) gives as the query: per row
    ([B, rows, 1]) and per tensor (0-dim).  A scale applied to the wrong row, or dropped, changes the logits."""
    wl = _tiny("fp8", "token", q_len=2, hq=8, hkv=2, ctx=(7, 40))
    q8, qs = L.pertoken_quant(wl.query.float())      # [B, rows, D] e4m3fn, [B, rows, 1]
    assert qs.shape == (2, 2 * 2 * 4, 1) and float(qs.min()) != float(qs.max())
    args = (wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables, wl.softmax_scale, 2, wl.key_scale,
            wl.value_scale)
    out_scaled = O.paged_attention_decode_oracle(q8, *args, query_scale=qs)
    out_product = O.paged_attention_decode_oracle(q8.float() * qs, *args)
    torch.testing.assert_close(out_scaled.float(), out_product.to(torch.bfloat16).float(), atol=0, rtol=0)
    # the rows' scales differ, so swapping two rows' scales must change those rows
    qs_swapped = qs.clone()
    qs_swapped[:, [0, 5]] = qs[:, [5, 0]]
    moved = O.paged_attention_decode_oracle(q8, *args, query_scale=qs_swapped)
    assert not torch.equal(moved[:, 0], out_scaled[:, 0]) and torch.equal(moved[:, 1], out_scaled[:, 1])
    # per tensor
    s0 = torch.tensor(0.37)
    out_t = O.paged_attention_decode_oracle(q8, *args, query_scale=s0)
    out_p = O.paged_attention_decode_oracle(q8.float() * 0.37, *args)
    torch.testing.assert_close(out_t.float(), out_p.to(torch.bfloat16).float(), atol=0, rtol=0)


def test_sinks_follow_the_packed_row_order():
    """sinks holds one logit per PACKED query row (kv head h, new token t, head g) -> h*q*G + t*G + g.  Checked
    row by row against the closed form softmax with one extra, value-less column: a (h, t, g) permutation
    applied in the wrong order pairs rows with other rows' sinks."""
    q_len, hq, hkv = 3, 4, 2
    g = hq // hkv
    wl = _tiny("bf16", "none", q_len=q_len, hq=hq, hkv=hkv, ctx=(9, 21))
    rows = hkv * q_len * g
    sinks = torch.linspace(-2.0, 3.0, rows)  # all different
    out = _oracle(wl, sinks=sinks)
    kf, vf = O.flatten_key_cache(wl.key_cache), O.flatten_value_cache(wl.value_cache)
    for b, ctx in enumerate((9, 21)):
        k, v = O.gather_sequence(kf, vf, None, None, wl.block_tables[b], ctx, 16)  # [ctx, Hkv, D]
        for h in range(hkv):
            for t in range(q_len):
                for gg in range(g):
                    row = h * q_len * g + t * g + gg
                    nvis = ctx - (q_len - 1 - t)
                    s = (k[:nvis, h].double() @ wl.query[b, row].double()) * wl.softmax_scale
                    m = max(float(s.max()), float(sinks[row]))
                    e = torch.exp(s - m)
                    o = (e[:, None] * v[:nvis, h].double()).sum(0) / (e.sum() + math.exp(float(sinks[row]) - m))
                    torch.testing.assert_close(out[b, row].double(), o.to(torch.bfloat16).double(), atol=1e-2, rtol=1e-2)


def test_alibi_in_the_two_stage_form_matches_the_end_to_end_oracle():
    """partition_stage applies the ALiBi term per partition; merged by reduce_stage it must give the end-to-end
    oracle's output (which test_alibi_matches_explicit_bias pins), for MTP rows and several partitions."""
    wl = _tiny("fp8", "tensor", q_len=2, hq=4, hkv=2, bs=16, ctx=(300, 70, 513))
    slopes = torch.tensor([0.3, 0.05, 0.011, 0.2])
    end_to_end = _oracle(wl, alibi_slopes=slopes)
    ml, es, to = O.partition_stage(wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables,
                                   wl.softmax_scale, 2, wl.key_scale, wl.value_scale, slopes, 256)
    merged = O.reduce_stage(ml, es, to, wl.context_lens, 256)
    torch.testing.assert_close(merged.float(), end_to_end.float(), atol=2e-3, rtol=2 ** -7)
    # and the term is really there: without it the result differs
    plain = _oracle(wl)
    assert float((plain.float() - end_to_end.float()).abs().max()) > 1e-2


def test_error_stats_on_a_hand_computed_pair():
    """error_stats restates compare_arrays (utils.py:50-56): max |a-b| and max |a-b| / (1 + |b|)."""
    a = torch.tensor([[1.0, -2.0], [0.5, 10.0]])
    b = torch.tensor([[1.5, -2.0], [0.0, 7.0]])
    st = O.error_stats(a, b)
    assert st["diff_abs_max"] == pytest.approx(3.0)
    # |a-b| / (1+|b|) = 0.5/2.5, 0, 0.5/1, 3/8
    assert st["max_diff_thr"] == pytest.approx(0.5)
    assert st["nan_result"] == 0 and st["nan_ref"] == 0
    st = O.error_stats(torch.tensor([float("nan"), 1.0]), torch.tensor([0.0, 1.0]))
    assert st["nan_result"] == 1 and st["nan_ref"] == 0


def test_alibi_per_packed_row_matches_explicit_bias():
    """One ALiBi slope per PACKED query row, [Hkv*q*G] at h*q*G + t*G + g: what the reference kernels read with
    alibi_slopes_ptr + kv_head*QUERY_GROUP_SIZE + row (pa_decode_triton_gluon_fp8.py:323-327, 803-810) and add as
    slope[row] * (col - ctx + 1) (:906-908).  Three new tokens, two kv heads, all slopes different; every row is
    held against a dense softmax with the bias written out as a matrix.  A slope array read in (t, h, g) or
    (h, g, t) order pairs rows with other rows' slopes and fails; so does a bias that counts columns from the
    row's own last visible key instead of from the context's end."""
    q_len, hq, hkv = 3, 4, 2
    g = hq // hkv
    wl = _tiny("bf16", "none", q_len=q_len, hq=hq, hkv=hkv, ctx=(9, 21, 40))
    rows = hkv * q_len * g
    slopes = torch.linspace(0.02, 0.9, rows)  # one per packed row, all different
    out = _oracle(wl, alibi_slopes=slopes)
    kf, vf = O.flatten_key_cache(wl.key_cache), O.flatten_value_cache(wl.value_cache)
    for b, ctx in enumerate((9, 21, 40)):
        k, v = O.gather_sequence(kf, vf, None, None, wl.block_tables[b], ctx, 16)  # [ctx, Hkv, D]
        bias = slopes.double()[:, None] * (torch.arange(ctx) - ctx + 1).double()[None, :]  # [rows, ctx]
        for h in range(hkv):
            for t in range(q_len):
                for gg in range(g):
                    row = h * q_len * g + t * g + gg
                    nvis = ctx - (q_len - 1 - t)
                    s = (k[:nvis, h].double() @ wl.query[b, row].double()) * wl.softmax_scale + bias[row, :nvis]
                    o = torch.softmax(s, 0) @ v[:nvis, h].double()
                    torch.testing.assert_close(out[b, row].double(), o.to(torch.bfloat16).double(), atol=1e-2, rtol=1e-2)
    # swapping the slopes of two rows moves exactly those rows
    sw = slopes.clone()
    sw[[1, 8]] = slopes[[8, 1]]
    moved = _oracle(wl, alibi_slopes=sw)
    same = [r for r in range(rows) if r not in (1, 8)]
    assert torch.equal(moved[:, same], out[:, same])
    assert not torch.equal(moved[:, 1], out[:, 1]) and not torch.equal(moved[:, 8], out[:, 8])
    # one slope per query head is the per-row array with the head's slope repeated for its new tokens
    per_head = torch.tensor([0.5, 0.25, 0.125, 0.0625])
    expanded = per_head.view(hkv, 1, g).expand(hkv, q_len, g).reshape(-1)
    assert torch.equal(_oracle(wl, alibi_slopes=per_head), _oracle(wl, alibi_slopes=expanded))
    # and the two-stage form reads the same array the same way
    ml, es, to = O.partition_stage(wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables,
                                   wl.softmax_scale, q_len, wl.key_scale, wl.value_scale, slopes, 256)
    merged = O.reduce_stage(ml, es, to, wl.context_lens, 256)
    torch.testing.assert_close(merged.float(), out.float(), atol=2e-3, rtol=2 ** -7)
