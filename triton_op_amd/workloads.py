"""Seeded synthetic decode workloads: the five benchmark configurations and scaled-down
variants of them for parity tests.

Every tensor is drawn from ``torch.Generator`` objects seeded from (seed, tensor tag, chunk
index), in chunks of KV pages, on the device the workload is built for, so a multi-GB cache
never needs a multi-GB float32 staging copy.  A workload built on "cpu" and one built on
"cuda" use different random streams; parity tests build once and copy.

Shapes follow the decode entry point: query [B, Hkv*q*G, D] (rows r = t*G + g inside a
kv-head group), key_cache [nblk,Hkv,D/x,bs,x], value_cache [nblk,Hkv,D,bs], int32
block_tables [B, max_blocks] and context_lens [B].
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Optional

import torch

from . import kv_layout as L


@dataclass
class Workload:
    name: str
    query: torch.Tensor
    key_cache: torch.Tensor
    value_cache: torch.Tensor
    context_lens: torch.Tensor  # int32 [B]
    block_tables: torch.Tensor  # int32 [B, max_blocks]
    softmax_scale: float
    q_len: int  # rows per head group are q_len * G
    q_lens: Optional[torch.Tensor]  # int32 [B] when ragged, else None
    key_scale: Optional[torch.Tensor]
    value_scale: Optional[torch.Tensor]
    partition_size: int
    num_kv_heads: int
    num_q_heads: int
    head_size: int
    block_size: int
    max_context_len: int
    meta: dict = field(default_factory=dict)

    @property
    def batch(self) -> int:
        return self.query.shape[0]

    def kv_bytes(self) -> int:
        """Algorithmic KV-stream bytes of one call: every live token's K and V row once,
        plus the per-token scales when there are any."""
        tok = int(self.context_lens.to(torch.int64).sum())
        per_tok = self.num_kv_heads * self.head_size * (
            self.key_cache.element_size() + self.value_cache.element_size()
        )
        if self.key_scale is not None and self.key_scale.dim() == 4:
            per_tok += self.num_kv_heads * 2 * 4
        return tok * per_tok

    def flops(self) -> int:
        ql = self.q_lens.to(torch.int64) if self.q_lens is not None else torch.full(
            (self.batch,), self.q_len, dtype=torch.int64)
        return int(4 * (ql.cpu() * self.context_lens.to(torch.int64).cpu()).sum()) * self.num_q_heads * self.head_size

    def to(self, device) -> "Workload":
        kw = {}
        for k, v in self.__dict__.items():
            kw[k] = v.to(device) if isinstance(v, torch.Tensor) else v
        kw["meta"] = {k: (v.to(device) if isinstance(v, torch.Tensor) else v) for k, v in self.meta.items()}
        return Workload(**kw)


def _gen(device, seed: int, tag: int, chunk: int = 0) -> torch.Generator:
    g = torch.Generator(device=device)
    g.manual_seed((seed * 1_000_003 + tag) * 1_000_003 + chunk)
    return g


def _block_tables(ctx: torch.Tensor, block_size: int, pool_factor: float, gen_cpu: torch.Generator):
    """Random permutation of a pool of ceil(pool_factor * needed) pages; sequence b takes the
    next ceil(ctx_b/bs) entries.  Unused slots of a row repeat the row's first page."""
    need = (ctx.to(torch.int64) + block_size - 1) // block_size
    total = int(need.sum())
    pool = max(int(math.ceil(pool_factor * total)), total)
    perm = torch.randperm(pool, generator=gen_cpu)[:total].to(torch.int32)
    max_blocks = int(need.max())
    bt = torch.empty(len(ctx), max_blocks, dtype=torch.int32)
    off = 0
    for b, n in enumerate(need.tolist()):
        bt[b, :n] = perm[off : off + n]
        bt[b, n:] = perm[off]
        off += n
    return bt, pool


_CHUNK_PAGES_BYTES = 256 << 20  # f32 staging per chunk


def _fill_fp8_per_tensor(shape, device, seed, tag):
    """N(0,1) -> scale = amax/448 -> e4m3fn, in page chunks (two passes over the same streams)."""
    nblk = shape[0]
    per_page = 1
    for s in shape[1:]:
        per_page *= s
    step = max(1, _CHUNK_PAGES_BYTES // (per_page * 4))
    amax = torch.zeros((), dtype=torch.float32, device=device)
    for i, lo in enumerate(range(0, nblk, step)):
        n = min(step, nblk - lo)
        t = torch.empty((n,) + tuple(shape[1:]), dtype=torch.float32, device=device)
        t.normal_(0.0, 1.0, generator=_gen(device, seed, tag, i))
        amax = torch.maximum(amax, t.abs().amax())
    scale = (amax / L.FP8_MAX).to(torch.float32)
    out = torch.empty(shape, dtype=L.FP8_DTYPE, device=device)
    for i, lo in enumerate(range(0, nblk, step)):
        n = min(step, nblk - lo)
        t = torch.empty((n,) + tuple(shape[1:]), dtype=torch.float32, device=device)
        t.normal_(0.0, 1.0, generator=_gen(device, seed, tag, i))
        out[lo : lo + n] = (t / scale).clamp_(-L.FP8_MAX, L.FP8_MAX).to(L.FP8_DTYPE)
    return out, scale


def _fill_fp8_per_token(nblk, hkv, d, bs, device, seed, tag, sigma_mag):
    """values N(0,1) * m with m ~ LogNormal(0, sigma_mag) per (page, head, token); quantised per
    (page, head, token) over head_size.  Returns token-major FP8 [nblk,Hkv,bs,D] and scales
    [nblk,Hkv,bs,1]."""
    step = max(1, _CHUNK_PAGES_BYTES // (hkv * d * bs * 4))
    q = torch.empty(nblk, hkv, bs, d, dtype=L.FP8_DTYPE, device=device)
    sc = torch.empty(nblk, hkv, bs, 1, dtype=torch.float32, device=device)
    for i, lo in enumerate(range(0, nblk, step)):
        n = min(step, nblk - lo)
        g = _gen(device, seed, tag, i)
        t = torch.empty(n, hkv, bs, d, dtype=torch.float32, device=device).normal_(0.0, 1.0, generator=g)
        m = torch.empty(n, hkv, bs, 1, dtype=torch.float32, device=device).normal_(0.0, sigma_mag, generator=g).exp_()
        qq, ss = L.pertoken_quant(t * m)
        q[lo : lo + n] = qq
        sc[lo : lo + n] = ss
    return q, sc


def make_decode_workload(
    *,
    name: str,
    seed: int,
    batch: int,
    num_q_heads: int,
    num_kv_heads: int,
    head_size: int = 128,
    block_size: int = 16,
    context_lens: torch.Tensor,
    q_len: int = 1,
    q_lens: Optional[torch.Tensor] = None,
    kv_dtype: str = "fp8",  # "fp8" | "bf16"
    scale_mode: str = "tensor",  # "tensor" | "token" | "none"
    pool_factor: float = 1.25,
    fixed_pool_blocks: Optional[int] = None,
    partition_size: int = 256,
    device="cpu",
    transposed_v: bool = False,
) -> Workload:
    g_cpu = _gen("cpu", seed, 0)
    ctx = context_lens.to(torch.int32)
    g = num_q_heads // num_kv_heads
    ge = q_len * g
    q = torch.empty(batch, num_kv_heads * ge, head_size, dtype=torch.float32)
    q.normal_(0.0, 1.0, generator=_gen("cpu", seed, 1))
    q = q.to(torch.bfloat16)
    if fixed_pool_blocks is not None:
        perm = torch.randperm(fixed_pool_blocks, generator=g_cpu).to(torch.int32)
        need = (ctx.to(torch.int64) + block_size - 1) // block_size
        max_blocks = fixed_pool_blocks // batch
        assert int(need.max()) <= max_blocks
        bt = perm[: batch * max_blocks].view(batch, max_blocks).contiguous()
        pool = fixed_pool_blocks
    else:
        bt, pool = _block_tables(ctx, block_size, pool_factor, g_cpu)
    ks = vs = None
    if kv_dtype == "bf16":
        shape_k = L.key_cache_shape(pool, num_kv_heads, head_size, block_size, torch.bfloat16)
        shape_v = L.value_cache_shape(pool, num_kv_heads, head_size, block_size)
        kc = torch.empty(shape_k, dtype=torch.float32, device=device).normal_(
            0.0, 1.0, generator=_gen(device, seed, 2)).to(torch.bfloat16)
        vc = torch.empty(shape_v, dtype=torch.float32, device=device).normal_(
            0.0, 1.0, generator=_gen(device, seed, 3)).to(torch.bfloat16)
    elif scale_mode == "tensor":
        shape_k = L.key_cache_shape(pool, num_kv_heads, head_size, block_size, L.FP8_DTYPE)
        shape_v = L.value_cache_shape(pool, num_kv_heads, head_size, block_size)
        kc, ks = _fill_fp8_per_tensor(shape_k, device, seed, 2)
        vc, vs = _fill_fp8_per_tensor(shape_v, device, seed, 3)
    elif scale_mode == "token":
        kt, ks = _fill_fp8_per_token(pool, num_kv_heads, head_size, block_size, device, seed, 2, 0.5)
        vt, vs = _fill_fp8_per_token(pool, num_kv_heads, head_size, block_size, device, seed, 3, 0.5)
        kc = L.tokens_to_key_cache(kt.permute(0, 2, 1, 3), L.FP8_DTYPE)
        vc = L.tokens_to_value_cache(vt.permute(0, 2, 1, 3), L.FP8_DTYPE)
        del kt, vt
    else:
        raise ValueError(scale_mode)
    if transposed_v:
        vc = L.shuffle_value_cache_layout(vc)
    return Workload(
        name=name,
        query=q.to(device),
        key_cache=kc,
        value_cache=vc,
        context_lens=ctx.to(device),
        block_tables=bt.to(device),
        softmax_scale=1.0 / math.sqrt(head_size),
        q_len=q_len,
        q_lens=None if q_lens is None else q_lens.to(torch.int32).to(device),
        key_scale=ks,
        value_scale=vs,
        partition_size=partition_size,
        num_kv_heads=num_kv_heads,
        num_q_heads=num_q_heads,
        head_size=head_size,
        block_size=block_size,
        max_context_len=int(ctx.max()),
        meta={"seed": seed, "pool_blocks": pool, "kv_dtype": kv_dtype, "scale_mode": scale_mode},
    )


def _lognormal_ctx(batch, median, sigma, lo, hi, gen):
    z = torch.empty(batch, dtype=torch.float64).normal_(0.0, 1.0, generator=gen)
    return torch.clamp(torch.round(torch.exp(math.log(median) + sigma * z)), lo, hi).to(torch.int32)


CONFIG_NAMES = ("c1_plumbing_bf16", "c2_fp8_b64_ctx4k", "c3_fp8_mtp2_bs1024", "c4_fp8_ctx128k", "c5_ragged_mix")


def make_config(name: str, device="cpu", *, batch: Optional[int] = None, ctx_scale: float = 1.0) -> Workload:
    """The five benchmark configurations.  ``batch`` and ``ctx_scale`` shrink a configuration
    (fewer sequences, proportionally shorter contexts) for tests; the defaults are full size."""
    if name.startswith("c1"):
        seed, b = 1, batch or 4
        gen = _gen("cpu", seed, 9)
        ctx = torch.randint(1, int(1024 * ctx_scale) + 1, (b,), generator=gen, dtype=torch.int32)
        return make_decode_workload(
            name=CONFIG_NAMES[0], seed=seed, batch=b, num_q_heads=8, num_kv_heads=1, block_size=16,
            context_lens=ctx, kv_dtype="bf16", scale_mode="none", fixed_pool_blocks=64 * b, device=device)
    if name.startswith("c2"):
        seed, b = 2, batch or 64
        ctx = torch.full((b,), int(4096 * ctx_scale), dtype=torch.int32)
        return make_decode_workload(
            name=CONFIG_NAMES[1], seed=seed, batch=b, num_q_heads=64, num_kv_heads=8, block_size=16,
            context_lens=ctx, device=device)
    if name.startswith("c3"):
        seed, b = 3, batch or 128
        gen = _gen("cpu", seed, 9)
        ctx = torch.randint(int(1024 * ctx_scale), int(32768 * ctx_scale) + 1, (b,), generator=gen,
                            dtype=torch.int32)
        return make_decode_workload(
            name=CONFIG_NAMES[2], seed=seed, batch=b, num_q_heads=64, num_kv_heads=8, block_size=1024,
            context_lens=ctx, q_len=2, device=device)
    if name.startswith("c4"):
        seed, b = 4, batch or 4
        ctx = torch.full((b,), int(131072 * ctx_scale), dtype=torch.int32)
        return make_decode_workload(
            name=CONFIG_NAMES[3], seed=seed, batch=b, num_q_heads=64, num_kv_heads=8, block_size=16,
            context_lens=ctx, device=device)
    if name.startswith("c5"):
        seed, b = 5, batch or 256
        gen = _gen("cpu", seed, 9)
        ctx = _lognormal_ctx(b, 2048 * ctx_scale, 1.0, 16, int(65536 * ctx_scale), gen)
        ql = torch.randint(1, 5, (b,), generator=gen, dtype=torch.int32)
        ctx = torch.maximum(ctx, ql)
        return make_decode_workload(
            name=CONFIG_NAMES[4], seed=seed, batch=b, num_q_heads=128, num_kv_heads=8, block_size=16,
            context_lens=ctx, q_len=4, q_lens=ql, scale_mode="token", device=device)
    raise ValueError(f"unknown configuration {name!r}; expected one of {CONFIG_NAMES}")
