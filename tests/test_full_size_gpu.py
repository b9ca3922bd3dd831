"""The five benchmark configurations at full size on the GPU.

The CPU oracle takes seconds per long sequence, so a few sequences of each configuration (the
shortest, the longest and one in between) are checked against it at the 2e-2 bar, and the whole
batch through size-independent properties: (i) the result does not depend on the partition size
(reference partition 256 vs the tuning layer's choice, and the reference-shaped buffers as scratch, where the
library cuts the axis its own way), (ii) relabelling the
physical pages (a permutation applied to the pool and to the block tables) leaves every output bit
unchanged, (iii) no NaN/Inf anywhere, padded query rows are zero."""
import pytest
import torch

from oracle import pa_oracle as O

pytestmark = pytest.mark.gpu


def _decode(wl, dev_wl, partition_size, **kw):
    import triton_op_amd as T

    out = torch.full_like(dev_wl.query, float("nan"))
    res = T.paged_attention_decode(
        out, dev_wl.query, dev_wl.key_cache, dev_wl.value_cache, dev_wl.context_lens, dev_wl.block_tables,
        dev_wl.softmax_scale, dev_wl.q_len, dev_wl.max_context_len, torch.bfloat16, None, dev_wl.key_scale,
        dev_wl.value_scale, partition_size=partition_size, query_lens=dev_wl.q_lens, **kw)
    torch.cuda.synchronize()
    return out, res


def _subset_for_oracle(wl, ids):
    """Copy only the pages the chosen sequences use to the host (the pools are GBs)."""
    bs = wl.block_size
    ids = list(ids)
    ctx = wl.context_lens[ids].cpu()
    need = ((ctx.long() + bs - 1) // bs).tolist()
    bt_rows = [wl.block_tables[b, :n].long() for b, n in zip(ids, need)]
    pages = torch.cat(bt_rows)
    uniq, inv = torch.unique(pages, return_inverse=True)
    kc = wl.key_cache[uniq].cpu()
    vc = wl.value_cache[uniq].cpu()
    ks = vs = None
    if wl.key_scale is not None:
        ks = wl.key_scale.cpu() if wl.key_scale.dim() == 0 else wl.key_scale[uniq].cpu()
        vs = wl.value_scale.cpu() if wl.value_scale.dim() == 0 else wl.value_scale[uniq].cpu()
    bt = torch.zeros(len(ids), max(need), dtype=torch.int32)
    off = 0
    inv = inv.cpu()
    for r, n in enumerate(need):
        bt[r, :n] = inv[off:off + n].to(torch.int32)
        off += n
    q = wl.query[ids].cpu()
    ql = wl.q_len if wl.q_lens is None else wl.q_lens[ids].cpu()
    return q, kc, vc, ctx, bt, ql, ks, vs


@pytest.mark.parametrize("name", ["c1", "c2", "c3", "c4", "c5"])
def test_full_size_configuration(cuda, name):
    from triton_op_amd import workloads as W

    print(f"building {name} at full size", flush=True)
    wl = W.make_config(name, device=cuda)
    ctx = wl.context_lens.cpu()
    print(f"config={wl.name} batch={wl.batch} kv_bytes={wl.kv_bytes()} max_ctx={int(ctx.max())}", flush=True)
    out, res = _decode(wl, wl, None)
    o = out.float()
    assert bool(torch.isfinite(o).all())

    # oracle on a few sequences
    order = torch.argsort(ctx)
    ids = {int(order[0]), int(order[len(order) // 2]), int(order[-1])}
    if wl.q_lens is not None:
        # a ragged batch: the sample must hold a sequence of every query length (1 new token = one 16-row tile
        # per kv head ... 4 new tokens = all four tiles of the shared-stream kernel's workgroup busy), each the
        # sequence of that query length whose context is closest to the median (seconds on the CPU)
        ql_cpu = wl.q_lens.cpu()
        med = int(ctx[order[len(order) // 2]])
        for qv in range(1, wl.q_len + 1):
            cand = torch.nonzero(ql_cpu == qv).flatten()
            assert cand.numel() > 0, f"no sequence with {qv} new tokens in {wl.name}"
            ids.add(int(cand[torch.argmin((ctx[cand] - med).abs())]))
        assert {int(ql_cpu[i]) for i in ids} >= set(range(1, wl.q_len + 1))
    ids = sorted(ids)
    q, kc, vc, sctx, bt, ql, ks, vs = _subset_for_oracle(wl, ids)
    ref = O.paged_attention_decode_oracle(q, kc, vc, sctx, bt, wl.softmax_scale, ql, ks, vs, q_max=wl.q_len)
    torch.testing.assert_close(o[ids].cpu(), ref.float(), atol=2e-2, rtol=2e-2)
    thr = O.error_stats(o[ids].cpu(), ref)["max_diff_thr"]
    print(f"  oracle on sequences {ids}: max_diff_thr={thr:.2e}, partition_size={res['partition_size']}", flush=True)
    assert thr < 1.5e-2, thr
    if wl.q_lens is not None:  # padded query rows are written as zero
        g = wl.num_q_heads // wl.num_kv_heads
        b = int(torch.argmin(wl.q_lens))
        qb = int(wl.q_lens[b])
        pad = out[b].view(wl.num_kv_heads, wl.q_len, g, wl.head_size)[:, qb:]
        assert pad.numel() == 0 or bool((pad == 0).all())

    # (i) partition-size independence
    out256, res256 = _decode(wl, wl, 256)
    assert res256["partition_size"] == 256
    # the two results differ by the bf16 rounding of the partials (whose magnitude is not bounded by the
    # merged value's) and of the output: held to the parity bar, and to a much tighter bound on average
    diff = (out256.float() - o).abs()
    worst = float((diff - (2e-2 + 2e-2 * o.abs())).max())
    assert worst <= 0, worst
    assert float(diff.mean()) < 1e-3
    del out256, res256
    # ... nor, with the same reference-shaped buffers declared scratch, on the library's own cut of the partition
    # axis inside them (the real query rows; the others are left as they were)
    lean, _ = _decode(wl, wl, 256, output_only=True)
    g = wl.num_q_heads // wl.num_kv_heads
    rows = (torch.arange(wl.q_len, device=cuda)[None, :] <
            (wl.q_lens if wl.q_lens is not None else torch.full((wl.batch,), wl.q_len, device=cuda))[:, None])
    live = rows[:, None, :, None, None].expand(wl.batch, wl.num_kv_heads, wl.q_len, g, wl.head_size)
    lean5 = lean.float().view(wl.batch, wl.num_kv_heads, wl.q_len, g, wl.head_size)
    o5 = o.view(wl.batch, wl.num_kv_heads, wl.q_len, g, wl.head_size)
    diff = (lean5 - o5).abs()[live]
    assert bool(torch.isfinite(lean5[live]).all())
    assert float((diff - (2e-2 + 2e-2 * o5.abs()[live])).max()) <= 0
    assert float(diff.mean()) < 1e-3
    del lean, lean5, diff

    # (ii) page relabelling is invisible, bit for bit
    if name != "c3":  # c3's pool (5.4 GB) is permuted in place below instead of copied
        n = wl.key_cache.shape[0]
        perm = torch.randperm(n, device=cuda, generator=torch.Generator(device=cuda).manual_seed(11))
        inv = torch.empty_like(perm)
        inv[perm] = torch.arange(n, device=cuda)
        wl2 = type(wl)(**{**wl.__dict__, "key_cache": wl.key_cache[perm], "value_cache": wl.value_cache[perm],
                         "block_tables": inv[wl.block_tables.long()].to(torch.int32),
                         "key_scale": wl.key_scale if wl.key_scale is None or wl.key_scale.dim() == 0 else wl.key_scale[perm],
                         "value_scale": wl.value_scale if wl.value_scale is None or wl.value_scale.dim() == 0 else wl.value_scale[perm]})
        out2, _ = _decode(wl2, wl2, None)
        assert torch.equal(out2.view(torch.int16), out.view(torch.int16))
    else:
        # swap two pages of one sequence and its block-table entries
        b = int(order[-1])
        p0, p1 = int(wl.block_tables[b, 0]), int(wl.block_tables[b, 1])
        for t in (wl.key_cache, wl.value_cache):
            tmp = t[p0].clone()
            t[p0] = t[p1]
            t[p1] = tmp
        wl.block_tables[b, 0], wl.block_tables[b, 1] = p1, p0
        out2, _ = _decode(wl, wl, None)
        assert torch.equal(out2.view(torch.int16), out.view(torch.int16))
