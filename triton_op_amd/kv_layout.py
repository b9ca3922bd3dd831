"""Paged KV-cache layouts, FP8 quantisers and the MTP row packing used around the decode op.

Cache layouts (x = 16 // itemsize, i.e. 16 for FP8 and 8 for bf16):
  key_cache    [num_blocks, num_kv_heads, head_size // x, block_size, x]
  value_cache  [num_blocks, num_kv_heads, head_size, block_size]
  value_cache  [num_blocks, num_kv_heads, block_size // x, head_size, x]   ("transposed")
Scales: a 0-dim f32 tensor (per tensor) or [num_blocks, num_kv_heads, block_size, 1] f32
(per token and head).  These mirror reference test_pa_mtp.py:109-172 (create_kv_cache),
:294-369 (quantize_kv_cache_symmetric), :472-497 (shuffle_value_cache_layout) and
:792-822 / :903-909 (MTP reshape and its inverse); FP8 here is OCP e4m3fn (max 448), the
format gfx950 computes in.  Everything is plain torch and runs on CPU or GPU tensors.

The torch quantisers in this file (`quantize_per_tensor`, `pertoken_quant`, `quantize_kv_cache_per_tensor`,
`quantize_kv_cache_per_token`) build synthetic caches for the workloads and are the formulas the HIP cache
writers (`kv_cache.py`, `csrc/pa_kv_cache.hip`) are tested against; the writers themselves never call them.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

FP8_DTYPE = torch.float8_e4m3fn
FP8_MAX = 448.0


def elements_per_16b(dtype: torch.dtype) -> int:
    return 16 // torch.empty((), dtype=dtype).element_size()


def key_cache_shape(num_blocks: int, num_kv_heads: int, head_size: int, block_size: int, dtype: torch.dtype):
    x = elements_per_16b(dtype)
    if head_size % x:
        raise ValueError(f"head_size {head_size} is not a multiple of {x} for {dtype}")
    return (num_blocks, num_kv_heads, head_size // x, block_size, x)


def value_cache_shape(num_blocks: int, num_kv_heads: int, head_size: int, block_size: int):
    return (num_blocks, num_kv_heads, head_size, block_size)


def tokens_to_key_cache(k_tok: torch.Tensor, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """[num_blocks, block_size, num_kv_heads, head_size] -> key-cache layout (same values)."""
    nblk, bs, hkv, d = k_tok.shape
    dtype = dtype or k_tok.dtype
    x = elements_per_16b(dtype)
    return k_tok.to(dtype).view(nblk, bs, hkv, d // x, x).permute(0, 2, 3, 1, 4).contiguous()


def tokens_to_value_cache(v_tok: torch.Tensor, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """[num_blocks, block_size, num_kv_heads, head_size] -> value-cache layout [nblk,Hkv,D,bs]."""
    dtype = dtype or v_tok.dtype
    return v_tok.to(dtype).permute(0, 2, 3, 1).contiguous()


def key_cache_to_tokens(key_cache: torch.Tensor) -> torch.Tensor:
    nblk, hkv, dx, bs, x = key_cache.shape
    return key_cache.permute(0, 3, 1, 2, 4).reshape(nblk, bs, hkv, dx * x)


def value_cache_to_tokens(value_cache: torch.Tensor) -> torch.Tensor:
    if value_cache.dim() == 5:
        value_cache = unshuffle_value_cache_layout(value_cache)
    return value_cache.permute(0, 3, 1, 2)


def create_kv_cache(
    num_blocks: int,
    block_size: int,
    num_kv_heads: int,
    head_size: int,
    dtype: torch.dtype = torch.bfloat16,
    generator: Optional[torch.Generator] = None,
    device="cpu",
    distribution: str = "uniform",
) -> Tuple[torch.Tensor, torch.Tensor]:
    """A 16-bit cache filled with uniform(-1,1) (the reference's choice) or N(0,1) values."""
    ks = key_cache_shape(num_blocks, num_kv_heads, head_size, block_size, dtype)
    vs = value_cache_shape(num_blocks, num_kv_heads, head_size, block_size)
    out = []
    for shape in (ks, vs):
        t = torch.empty(shape, dtype=torch.float32, device=device)
        if distribution == "uniform":
            t.uniform_(-1.0, 1.0, generator=generator)
        else:
            t.normal_(0.0, 1.0, generator=generator)
        out.append(t.to(dtype))
    return out[0], out[1]


def quantize_per_tensor(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """scale = amax / 448 (0-dim f32); q = (x / scale) -> e4m3fn.  Layout is preserved."""
    amax = x.abs().amax().to(torch.float32)
    scale = torch.where(amax > 0, amax / FP8_MAX, torch.ones_like(amax))
    q = (x.to(torch.float32) / scale).clamp_(-FP8_MAX, FP8_MAX).to(FP8_DTYPE)
    return q, scale


def pertoken_quant(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """amax over the last axis: scale = amax/448 (1 where the row is all zero), keepdim f32."""
    xf = x.to(torch.float32)
    amax = xf.abs().amax(dim=-1, keepdim=True)
    scale = torch.where(amax > 0, amax / FP8_MAX, torch.ones_like(amax))
    q = (xf / scale).clamp_(-FP8_MAX, FP8_MAX).to(FP8_DTYPE)
    return q, scale


def quantize_kv_cache_per_tensor(key_cache: torch.Tensor, value_cache: torch.Tensor):
    kq, ks = quantize_per_tensor(key_cache)
    vq, vs = quantize_per_tensor(value_cache)
    # a 16-bit key cache has x=8; the FP8 cache must be re-laid-out with x=16
    kq = tokens_to_key_cache(key_cache_to_tokens(kq), FP8_DTYPE)
    return kq, ks, vq, vs


def quantize_kv_cache_per_token(key_cache: torch.Tensor, value_cache: torch.Tensor):
    """Per (block, head, token) symmetric FP8 quantisation over head_size.

    Returns (key_q [nblk,Hkv,D/16,bs,16], key_scale [nblk,Hkv,bs,1],
             value_q [nblk,Hkv,D,bs],     value_scale [nblk,Hkv,bs,1])."""
    k_tok = key_cache_to_tokens(key_cache).permute(0, 2, 1, 3)  # [nblk,Hkv,bs,D]
    v_tok = value_cache_to_tokens(value_cache).permute(0, 2, 1, 3)
    kq, ks = pertoken_quant(k_tok)
    vq, vs = pertoken_quant(v_tok)
    kq = tokens_to_key_cache(kq.permute(0, 2, 1, 3), FP8_DTYPE)
    vq = tokens_to_value_cache(vq.permute(0, 2, 1, 3), FP8_DTYPE)
    return kq, ks.contiguous(), vq, vs.contiguous()


def shuffle_value_cache_layout(value_cache: torch.Tensor) -> torch.Tensor:
    """[nblk,Hkv,D,bs] -> [nblk,Hkv,bs/x,D,x]"""
    x = 16 // value_cache.element_size()
    nblk, hkv, d, bs = value_cache.shape
    return value_cache.view(nblk, hkv, d, bs // x, x).permute(0, 1, 3, 2, 4).contiguous()


def unshuffle_value_cache_layout(value_cache: torch.Tensor) -> torch.Tensor:
    """[nblk,Hkv,bs/x,D,x] -> [nblk,Hkv,D,bs]"""
    nblk, hkv, bsx, d, x = value_cache.shape
    return value_cache.permute(0, 1, 3, 2, 4).reshape(nblk, hkv, d, bsx * x)


def mtp_pack(x: torch.Tensor, batch: int, qlen: int, num_kv_heads: int) -> torch.Tensor:
    """token-major [B*q, Hq, D] -> op layout [B, Hkv*q*G, D] with row = h*(q*G) + t*G + g."""
    hq, d = x.shape[1], x.shape[2]
    g = hq // num_kv_heads
    return (
        x.reshape(batch, qlen, num_kv_heads, g, d).transpose(1, 2).reshape(batch, num_kv_heads * qlen * g, d)
    )


def mtp_unpack(x: torch.Tensor, batch: int, qlen: int, num_kv_heads: int) -> torch.Tensor:
    d = x.shape[2]
    g = x.shape[1] // (num_kv_heads * qlen)
    return (
        x.reshape(batch, num_kv_heads, qlen, g, d).transpose(1, 2).reshape(batch * qlen, num_kv_heads * g, d)
    )
