"""CPU oracle for split-KV paged-attention decode.  TEST INFRASTRUCTURE ONLY.

This module is a checker: tests, the smoke entry and the bench's CPU-baseline leg
may import it; the product package must never do so.

It restates, in plain torch/numpy f32 on the CPU, the algorithm the reference checks
its own kernels against, and the two-stage (partition + reduce) form of it:

* ``masked_attention``      follows reference test_pa_mtp.py:175-220 (reference_masked_attention)
* ``mha_extend``            follows reference test_pa_mtp.py:223-291 (torch_mha_extend)
* ``flatten_*``/``token_indices`` follow test_pa_mtp.py:259-260, :271-274 and the transposed
  V layout of :472-497 (shuffle_value_cache_layout)
* ``mtp_pack``/``mtp_unpack`` follow test_pa_mtp.py:792-822 and :903-909
* ``partition_stage``       follows pa_decode_triton_gluon_fp8.py:733-1002 / :232-501 (what one
  partition writes: scaled-logit max, un-normalised exp sum, normalised partial output)
  with the mask rule of :912-925 and the early exit of :785-788
* ``reduce_stage``          follows pa_decode_triton_gluon_fp8.py:1233-1333 (log-sum-exp merge)
* ``e4m3fn_table``          is the OCP FP8 e4m3fn bit formula (the format gfx950 uses; the
  reference asserts the gfx942 fnuz variant, pa_decode_triton_gluon_fp8.py:602-604)

Pinning (what makes these trustworthy without running the reference, which needs the
un-installed ``aiter`` package and a gfx942 GPU):
  - e4m3fn_table      vs torch's float8_e4m3fn cast of all 256 codes (library routine)
  - masked_attention  vs torch.nn.functional.scaled_dot_product_attention and vs a
                      pure-Python double-precision brute force on tiny inputs
  - gather/layouts    by round trips and by block-permutation invariance
  - causal MTP mask   by exhaustive enumeration against tril(diagonal=key_len-query_len)
  - partition/reduce  by independence of the result from the partition size, by the
                      one-partition identity, and by the closed-form log-sum-exp merge
  - ALiBi             by an explicit per-row bias matrix added to a dense softmax (one slope per packed row,
                      several new tokens and kv heads, all slopes different; swapping two rows' slopes must
                      move exactly those rows), and per-head slopes by equality with their per-row expansion
The reference holds no golden vectors or known-answer tests for this path (its logs keep only
md5s of GPU-RNG outputs in fnuz FP8); bit-exact agreement with the reference's *kernels*
(accumulation order, exp2 implementation, P->FP8 rounding) is therefore "parity unpinned";
agreement with the reference's *oracle* is what is pinned here.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple, Union

import numpy as np
import torch

FP8 = torch.float8_e4m3fn
FP8_MAX = 448.0


# --------------------------------------------------------------------------------------
# FP8 e4m3fn
# --------------------------------------------------------------------------------------
def e4m3fn_table() -> np.ndarray:
    """All 256 e4m3fn codes as float32, from the bit formula (bias 7, no inf, S.1111.111 = NaN)."""
    out = np.empty(256, dtype=np.float32)
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        e = (code >> 3) & 0xF
        m = code & 0x7
        if e == 0xF and m == 0x7:
            out[code] = np.nan
        elif e == 0:
            out[code] = sign * (m / 8.0) * 2.0 ** (-6)
        else:
            out[code] = sign * (1.0 + m / 8.0) * 2.0 ** (e - 7)
    return out


def _to_f32(raw: torch.Tensor) -> torch.Tensor:
    """Cache element -> float32 (FP8 bytes are decoded with torch's e4m3fn cast)."""
    return raw.to(torch.float32)


# --------------------------------------------------------------------------------------
# layouts
# --------------------------------------------------------------------------------------
def flatten_key_cache(key_cache: torch.Tensor) -> torch.Tensor:
    """[nblk, Hkv, D/x, bs, x] -> [nblk*bs, Hkv, D]   (test_pa_mtp.py:259)"""
    nblk, hkv, dx, bs, x = key_cache.shape
    return key_cache.permute(0, 3, 1, 2, 4).contiguous().view(nblk * bs, hkv, dx * x)


def flatten_value_cache(value_cache: torch.Tensor) -> torch.Tensor:
    """[nblk, Hkv, D, bs] or transposed [nblk, Hkv, bs/x, D, x] -> [nblk*bs, Hkv, D]
    (test_pa_mtp.py:260; transposed form is the inverse of :472-497)"""
    if value_cache.dim() == 4:
        nblk, hkv, d, bs = value_cache.shape
        return value_cache.permute(0, 3, 1, 2).contiguous().view(nblk * bs, hkv, d)
    nblk, hkv, bsx, d, x = value_cache.shape
    return value_cache.permute(0, 2, 4, 1, 3).contiguous().view(nblk * bsx * x, hkv, d)


def flatten_scale(scale: Optional[torch.Tensor], hkv: int) -> Optional[torch.Tensor]:
    """entry-point scale -> [Hkv, nblk*bs] (test_pa_mtp.py:351,360) or a python float for 0-dim."""
    if scale is None:
        return None
    if scale.dim() == 0:
        return scale
    nblk, h, bs, one = scale.shape
    assert h == hkv and one == 1
    return scale.permute(1, 0, 2, 3).contiguous().view(hkv, nblk * bs)


def token_indices(block_table_row: torch.Tensor, ctx: int, bs: int) -> torch.Tensor:
    """flat token slot of each of the first ctx tokens (test_pa_mtp.py:271-274)"""
    return (
        block_table_row.to(torch.int64).repeat_interleave(bs)[:ctx] * bs
        + torch.arange(ctx, dtype=torch.int64) % bs
    )


def gather_sequence(
    key_flat: torch.Tensor,
    value_flat: torch.Tensor,
    kscale_flat,
    vscale_flat,
    block_table_row: torch.Tensor,
    ctx: int,
    bs: int,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """dense dequantised f32 K, V [ctx, Hkv, D] of one sequence (test_pa_mtp.py:277-283)"""
    idx = token_indices(block_table_row, ctx, bs)
    k = _to_f32(key_flat[idx])
    v = _to_f32(value_flat[idx])
    if kscale_flat is not None:
        if kscale_flat.dim() == 0:
            k = k * kscale_flat.to(torch.float32)
        else:
            k = k * kscale_flat[:, idx].t().unsqueeze(-1)
    if vscale_flat is not None:
        if vscale_flat.dim() == 0:
            v = v * vscale_flat.to(torch.float32)
        else:
            v = v * vscale_flat[:, idx].t().unsqueeze(-1)
    return k, v


def mtp_pack(x: torch.Tensor, batch: int, qlen: int, hkv: int) -> torch.Tensor:
    """token-major [B*q, Hq, D] -> kernel layout [B, Hkv*q*G, D], row = h*(q*G) + t*G + g
    (test_pa_mtp.py:799-804)"""
    hq, d = x.shape[1], x.shape[2]
    g = hq // hkv
    return x.reshape(batch, qlen, hkv, g, d).transpose(1, 2).reshape(batch, hkv * qlen * g, d)


def mtp_unpack(x: torch.Tensor, batch: int, qlen: int, hkv: int) -> torch.Tensor:
    """inverse of mtp_pack (test_pa_mtp.py:903-909)"""
    d = x.shape[2]
    g = x.shape[1] // (hkv * qlen)
    return x.reshape(batch, hkv, qlen, g, d).transpose(1, 2).reshape(batch * qlen, hkv * g, d)


# --------------------------------------------------------------------------------------
# dense attention (the reference's oracle)
# --------------------------------------------------------------------------------------
def masked_attention(
    query: torch.Tensor,  # [q, Hq, D]
    key: torch.Tensor,  # [ctx, Hkv, D] f32
    value: torch.Tensor,  # [ctx, Hkv, D] f32
    softmax_scale: float,
    output_dtype: torch.dtype,
    is_causal: bool = True,
    alibi_slopes: Optional[torch.Tensor] = None,  # [Hq] (shared by the q new tokens), or [q, Hq]: one per query row
    sinks: Optional[torch.Tensor] = None,  # [q, Hq] attention-sink logits
) -> torch.Tensor:
    hq, hkv = query.shape[1], key.shape[1]
    key = key.repeat_interleave(hq // hkv, dim=1)
    value = value.repeat_interleave(hq // hkv, dim=1)
    scores = torch.einsum("qhd,khd->hqk", query.float(), key.float()) * softmax_scale
    qlen, klen = query.shape[0], key.shape[0]
    if alibi_slopes is not None:
        # pa_decode_triton_gluon_fp8.py:906-908: slope_of_row * (col - ctx + 1); the column offset is the same for
        # every new token, the slope is read per packed query row (:323-327, :803-810)
        pos = torch.arange(klen, dtype=torch.float32) - klen + 1
        sl = alibi_slopes.float()
        sl = sl[:, None].expand(hq, qlen) if sl.dim() == 1 else sl.t()  # [Hq, q]
        scores = scores + sl[:, :, None] * pos[None, None, :]
    if is_causal:
        bias = torch.zeros(qlen, klen, dtype=torch.float32)
        keep = torch.ones(qlen, klen, dtype=torch.bool).tril(diagonal=klen - qlen)
        bias.masked_fill_(keep.logical_not(), float("-inf"))
        scores = scores + bias
    if sinks is not None:
        # pa_decode_triton_gluon_fp8.py:1118-1123: exp(sink - max) joins the denominator, no value attached:
        # a key column with that logit whose value row is zero
        scores = torch.cat([scores, sinks.float().t().unsqueeze(-1)], dim=-1)
        weights = torch.softmax(scores, dim=-1)[..., :-1]
    else:
        weights = torch.softmax(scores, dim=-1)
    out = torch.einsum("hqk,khd->qhd", weights.float(), value.float())
    return out.to(output_dtype)


def mha_extend(
    query: torch.Tensor,  # [total_q, Hq, D] token-major
    key_cache: torch.Tensor,
    value_cache: torch.Tensor,
    block_tables: torch.Tensor,
    seq_lens: torch.Tensor,
    qo_indptr: Sequence[int],
    key_scale: Optional[torch.Tensor] = None,
    value_scale: Optional[torch.Tensor] = None,
    softmax_scale: Optional[float] = None,
    alibi_slopes: Optional[torch.Tensor] = None,
    seq_ids: Optional[Sequence[int]] = None,
) -> torch.Tensor:
    """Paged multi-head attention, one dense f32 attention per sequence.

    Scales are given in the entry point's shapes (0-dim, or [nblk, Hkv, bs, 1]).  ``seq_ids``
    restricts the work to some sequences (rows of the others are left zero) so that
    full-size workloads can be spot-checked in seconds."""
    bs = key_cache.shape[-2]
    hkv = key_cache.shape[1]
    d = query.shape[-1]
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(d)
    key_flat = flatten_key_cache(key_cache)
    value_flat = flatten_value_cache(value_cache)
    ks = flatten_scale(key_scale, hkv)
    vs = flatten_scale(value_scale, hkv)
    out = torch.zeros_like(query)
    batch = len(qo_indptr) - 1
    for b in (range(batch) if seq_ids is None else seq_ids):
        q = query[qo_indptr[b] : qo_indptr[b + 1]]
        ctx = int(seq_lens[b])
        k, v = gather_sequence(key_flat, value_flat, ks, vs, block_tables[b], ctx, bs)
        out[qo_indptr[b] : qo_indptr[b + 1]] = masked_attention(
            q, k, v, softmax_scale, query.dtype, True, alibi_slopes
        )
    return out


def _alibi_of_rows(alibi_slopes: Optional[torch.Tensor], hkv: int, qmax: int, g: int) -> Optional[torch.Tensor]:
    """ALiBi slopes of the packed query rows, [Hkv, qmax, G].  The entry point takes one slope per packed row,
    [Hkv*qmax*G] at h*(qmax*G) + t*G + g -- the array the reference kernels index with
    kv_head*QUERY_GROUP_SIZE + row (pa_decode_triton_gluon_fp8.py:323-327, 803-810) -- or one per query head,
    [Hkv*G], shared by the head's new tokens; for one new token the two are the same array."""
    if alibi_slopes is None:
        return None
    sl = alibi_slopes.float().reshape(-1)
    if sl.numel() == hkv * qmax * g:
        return sl.view(hkv, qmax, g)
    assert sl.numel() == hkv * g, (sl.numel(), hkv, qmax, g)
    return sl.view(hkv, 1, g).expand(hkv, qmax, g)


def _row_qlens(batch: int, qlen: Union[int, torch.Tensor, Sequence[int]], q_max: Optional[int] = None):
    """per-sequence query lengths and the number of query positions the packed rows are laid out for"""
    if isinstance(qlen, int):
        return [qlen] * batch, (q_max or qlen)
    ql = [int(v) for v in qlen]
    return ql, (q_max or max(ql))


def paged_attention_decode_oracle(
    query: torch.Tensor,  # [B, Hkv*qmax*G, D] kernel (MTP-packed) layout
    key_cache: torch.Tensor,
    value_cache: torch.Tensor,
    seq_lens: torch.Tensor,
    block_tables: torch.Tensor,
    softmax_scale: float,
    query_sequence_length: Union[int, torch.Tensor, Sequence[int]] = 1,
    key_scale: Optional[torch.Tensor] = None,
    value_scale: Optional[torch.Tensor] = None,
    alibi_slopes: Optional[torch.Tensor] = None,
    seq_ids: Optional[Sequence[int]] = None,
    query_scale: Optional[torch.Tensor] = None,
    q_max: Optional[int] = None,
    sinks: Optional[torch.Tensor] = None,  # [Hkv*qmax*G], one logit per packed query row
) -> torch.Tensor:
    """The oracle behind the entry point's own conventions: output [B, Hkv*qmax*G, D] in
    query's 16-bit dtype (bf16 when the query is FP8).  Rows of padded query positions
    (t >= q_b for ragged q) are zero."""
    batch = query.shape[0]
    hkv = key_cache.shape[1]
    d = query.shape[-1]
    bs = key_cache.shape[-2]
    qls, qmax = _row_qlens(batch, query_sequence_length, q_max)
    g = query.shape[1] // (hkv * qmax)
    out_dtype = query.dtype if query.dtype in (torch.bfloat16, torch.float16) else torch.bfloat16
    qf = query.to(torch.float32)
    if query_scale is not None:
        qf = qf * (query_scale.to(torch.float32) if query_scale.dim() == 0 else query_scale.to(torch.float32))
    key_flat = flatten_key_cache(key_cache)
    value_flat = flatten_value_cache(value_cache)
    ks = flatten_scale(key_scale, hkv)
    vs = flatten_scale(value_scale, hkv)
    out = torch.zeros(query.shape, dtype=out_dtype)
    for b in (range(batch) if seq_ids is None else seq_ids):
        ctx, qb = int(seq_lens[b]), qls[b]
        k, v = gather_sequence(key_flat, value_flat, ks, vs, block_tables[b], ctx, bs)
        # [Hkv, qmax, G, D] -> token-major [qb, Hq, D]
        qv = qf[b].view(hkv, qmax, g, d)[:, :qb].permute(1, 0, 2, 3).reshape(qb, hkv * g, d)
        sk = al = None
        if sinks is not None:
            sk = sinks.float().view(hkv, qmax, g)[:, :qb].permute(1, 0, 2).reshape(qb, hkv * g)
        if alibi_slopes is not None:  # token-major like the query: [qb, Hq]
            al = _alibi_of_rows(alibi_slopes, hkv, qmax, g)[:, :qb].permute(1, 0, 2).reshape(qb, hkv * g)
        o = masked_attention(qv, k, v, softmax_scale, torch.float32, True, al, sk)
        o = o.view(qb, hkv, g, d).permute(1, 0, 2, 3)  # [Hkv, qb, G, D]
        out[b].view(hkv, qmax, g, d)[:, :qb] = o.to(out_dtype)
    return out


# --------------------------------------------------------------------------------------
# two-stage form: what the partition buffers hold, and the merge
# --------------------------------------------------------------------------------------
def partition_stage(
    query: torch.Tensor,
    key_cache: torch.Tensor,
    value_cache: torch.Tensor,
    seq_lens: torch.Tensor,
    block_tables: torch.Tensor,
    softmax_scale: float,
    query_sequence_length: Union[int, torch.Tensor, Sequence[int]] = 1,
    key_scale: Optional[torch.Tensor] = None,
    value_scale: Optional[torch.Tensor] = None,
    alibi_slopes: Optional[torch.Tensor] = None,
    partition_size: int = 256,
    max_num_partitions: Optional[int] = None,
    seq_ids: Optional[Sequence[int]] = None,
    q_max: Optional[int] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(max_logits, exp_sums, tmp_output): [B,Hkv,P,Ge] f32 x2 and [B,Hkv,P,Ge,D] f32.

    max_logits is the max of the scaled logits (natural-log domain), exp_sums the
    un-normalised sum of exp(logit - max), tmp_output the partition's normalised output.
    A row with no visible key in a partition gets max=-inf, sum=0, output=0 (the reference
    stores -1e38 / 256 / mean(V) there, whose weight in the merge is exp(-1e38 - M) = 0 as
    well).  Slots of partitions at or beyond ceil(ctx/partition) are left zero, as the
    reference leaves its zero-initialised buffers (pa_decode_triton_gluon_fp8.py:785-788)."""
    batch = query.shape[0]
    hkv = key_cache.shape[1]
    d = query.shape[-1]
    bs = key_cache.shape[-2]
    qls, qmax = _row_qlens(batch, query_sequence_length, q_max)
    g = query.shape[1] // (hkv * qmax)
    ge = qmax * g
    if max_num_partitions is None:
        max_num_partitions = (int(seq_lens.max()) + partition_size - 1) // partition_size
    P = max_num_partitions
    ml = torch.zeros(batch, hkv, P, ge, dtype=torch.float32)
    es = torch.zeros(batch, hkv, P, ge, dtype=torch.float32)
    to = torch.zeros(batch, hkv, P, ge, d, dtype=torch.float32)
    key_flat = flatten_key_cache(key_cache)
    value_flat = flatten_value_cache(value_cache)
    ks = flatten_scale(key_scale, hkv)
    vs = flatten_scale(value_scale, hkv)
    qf = query.to(torch.float32)
    for b in (range(batch) if seq_ids is None else seq_ids):
        ctx, qb = int(seq_lens[b]), qls[b]
        k, v = gather_sequence(key_flat, value_flat, ks, vs, block_tables[b], ctx, bs)
        qv = qf[b].view(hkv, ge, d)  # rows r = t*G + g
        scores = torch.einsum("hrd,khd->hrk", qv, k) * softmax_scale  # [Hkv, Ge, ctx]
        col = torch.arange(ctx)
        if alibi_slopes is not None:
            sl = _alibi_of_rows(alibi_slopes, hkv, qmax, g).reshape(hkv, ge)
            scores = scores + sl[:, :, None] * (col - ctx + 1).float()[None, None, :]
        t_of_row = torch.arange(ge) // g
        # visible: col + (q-1-t) < ctx   (pa_decode_triton_gluon_fp8.py:917-918); padded t masked
        vis = (col[None, :] + (qb - 1 - t_of_row)[:, None] < ctx) & (t_of_row < qb)[:, None]
        scores = scores.masked_fill(~vis[None], float("-inf"))
        nparts = (ctx + partition_size - 1) // partition_size
        for p in range(min(nparts, P)):
            lo, hi = p * partition_size, min((p + 1) * partition_size, ctx)
            s = scores[:, :, lo:hi]
            m = s.max(dim=-1).values  # [Hkv, Ge]
            m_safe = torch.where(torch.isinf(m), torch.zeros_like(m), m)
            e = torch.exp(s - m_safe[..., None])
            l = e.sum(-1)
            o = torch.einsum("hrk,khd->hrd", e, v[lo:hi])
            o = torch.where(l[..., None] > 0, o / l[..., None].clamp_min(1e-38), torch.zeros_like(o))
            ml[b, :, p], es[b, :, p], to[b, :, p] = m, l, o
    return ml, es, to


def reduce_stage(
    max_logits: torch.Tensor,
    exp_sums: torch.Tensor,
    tmp_output: torch.Tensor,
    seq_lens: torch.Tensor,
    partition_size: int = 256,
    output_dtype: torch.dtype = torch.bfloat16,
) -> torch.Tensor:
    """log-sum-exp merge over the first ceil(ctx/partition) partitions -> [B, Hkv*Ge, D]
    (pa_decode_triton_gluon_fp8.py:1233-1333: M = max m_p; w_p = l_p e^{m_p-M};
    out = sum_p tmp_p w_p / sum_p w_p)"""
    batch, hkv, P, ge = max_logits.shape
    d = tmp_output.shape[-1]
    out = torch.zeros(batch, hkv * ge, d, dtype=output_dtype)
    for b in range(batch):
        n = min((int(seq_lens[b]) + partition_size - 1) // partition_size, P)
        if n == 0:
            continue
        m = max_logits[b, :, :n].float()  # [Hkv, n, Ge]
        l = exp_sums[b, :, :n].float()
        M = m.max(dim=1, keepdim=True).values
        M_safe = torch.where(torch.isinf(M), torch.zeros_like(M), M)
        w = l * torch.exp(m - M_safe)
        w = torch.where(l > 0, w, torch.zeros_like(w))
        tot = w.sum(dim=1)  # [Hkv, Ge]
        acc = (tmp_output[b, :, :n].float() * w[..., None]).sum(dim=1)  # [Hkv, Ge, D]
        o = torch.where(tot[..., None] > 0, acc / tot[..., None].clamp_min(1e-38), torch.zeros_like(acc))
        out[b] = o.reshape(hkv * ge, d).to(output_dtype)
    return out


# --------------------------------------------------------------------------------------
# brute force (tiny inputs only): pure-Python double precision, no torch arithmetic
# --------------------------------------------------------------------------------------
def brute_force_decode(
    query, key_cache, value_cache, seq_lens, block_tables, softmax_scale,
    qlen: int = 1, key_scale=None, value_scale=None,
):
    """Element-by-element restatement straight from the cache indexing rules
    K[page,h,d//x,tok,d%x], V[page,h,d,tok]; returns nested lists [B][rows][D] of python floats."""
    tab = e4m3fn_table().astype(np.float64)

    def elem(t, *idx):
        v = t[idx]
        if t.dtype == FP8:
            return float(tab[int(t.view(torch.uint8)[idx])])
        return float(v)

    B = query.shape[0]
    hkv = key_cache.shape[1]
    x = key_cache.shape[-1]
    bs = key_cache.shape[-2]
    D = query.shape[-1]
    G = query.shape[1] // (hkv * qlen)
    out = [[[0.0] * D for _ in range(query.shape[1])] for _ in range(B)]
    for b in range(B):
        ctx = int(seq_lens[b])
        for h in range(hkv):
            for t in range(qlen):
                for g in range(G):
                    row = h * qlen * G + t * G + g
                    nvis = ctx - (qlen - 1 - t)
                    if nvis <= 0:
                        continue
                    logits = []
                    for c in range(nvis):
                        page, tok = int(block_tables[b, c // bs]), c % bs
                        ksc = 1.0 if key_scale is None else (
                            float(key_scale) if key_scale.dim() == 0 else float(key_scale[page, h, tok, 0]))
                        acc = 0.0
                        for dd in range(D):
                            acc += float(query[b, row, dd]) * elem(key_cache, page, h, dd // x, tok, dd % x) * ksc
                        logits.append(acc * softmax_scale)
                    mx = max(logits)
                    ws = [math.exp(v - mx) for v in logits]
                    tot = sum(ws)
                    for c in range(nvis):
                        page, tok = int(block_tables[b, c // bs]), c % bs
                        vsc = 1.0 if value_scale is None else (
                            float(value_scale) if value_scale.dim() == 0 else float(value_scale[page, h, tok, 0]))
                        w = ws[c] / tot
                        for dd in range(D):
                            out[b][row][dd] += w * elem(value_cache, page, h, dd, tok) * vsc
    return out


# --------------------------------------------------------------------------------------
# error vocabulary of the reference (utils.py:50-56 compare_arrays)
# --------------------------------------------------------------------------------------
def error_stats(result: torch.Tensor, ref: torch.Tensor) -> dict:
    a = result.detach().float().cpu()
    b = ref.detach().float().cpu()
    diff = (a - b).abs()
    return {
        "diff_abs_max": float(diff.max()) if diff.numel() else 0.0,
        "max_diff_thr": float((diff / (1.0 + b.abs())).max()) if diff.numel() else 0.0,
        "nan_result": int(torch.isnan(a).sum()),
        "nan_ref": int(torch.isnan(b).sum()),
    }
