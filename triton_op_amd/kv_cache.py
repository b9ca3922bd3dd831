"""KV-cache write and quantisation on the GPU: the step that produces the paged FP8 caches the decode op reads.

`quantize_kv_cache_symmetric` keeps the name, arguments and six results of the reference's offline
routine (test_pa_mtp.py:294-369, built there on aiter.pertoken_quant); `kv_cache_write` is the
serving-time form of the same step (new tokens into their slots, quantised on the way).  Both run
HIP kernels from libpa_decode.so; the torch helpers in `kv_layout` compute the same formulas on any device
and are what the tests compare them with.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional, Tuple

import torch

from . import _cabi
from ._cabi import PaKvWriteArgs

FP8_DTYPE = torch.float8_e4m3fn


def _stream(dev) -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)


def quantize_kv_cache_symmetric(
    key_cache: torch.Tensor,    # [num_blocks, num_heads, head_size // 8, block_size, 8] bf16
    value_cache: torch.Tensor,  # [num_blocks, num_heads, head_size, block_size] bf16
    quant_dtype: torch.dtype = FP8_DTYPE,
    scale_dtype: torch.dtype = torch.float32,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Per (block, head, token) symmetric FP8 quantisation of a 16-bit cache.

    Returns (quantized_keys [nblk,H,D/16,bs,16], key_scales_flat [H, nblk*bs], quantized_values [nblk,H,D,bs],
    value_scales_flat, key_scales [nblk,H,bs,1], value_scales [nblk,H,bs,1])."""
    if quant_dtype != FP8_DTYPE or scale_dtype != torch.float32:
        raise ValueError("only float8_e4m3fn with float32 scales is supported")
    if key_cache.dtype != torch.bfloat16 or value_cache.dtype != torch.bfloat16:
        raise ValueError("quantize_kv_cache_symmetric takes a bfloat16 cache")
    if not key_cache.is_cuda:
        raise ValueError("quantize_kv_cache_symmetric runs on the GPU only (kv_layout has the torch form)")
    if value_cache.device != key_cache.device:
        raise ValueError(f"value_cache is on {value_cache.device}, key_cache on {key_cache.device}")
    nblk, h, d, bs = value_cache.shape
    if tuple(key_cache.shape) != (nblk, h, d // 8, bs, 8) or d != 128:
        raise ValueError(f"key_cache shape {tuple(key_cache.shape)} does not match value_cache {tuple(value_cache.shape)}")
    kc, vc = key_cache.contiguous(), value_cache.contiguous()
    dev = kc.device
    kq = torch.empty(nblk, h, d // 16, bs, 16, dtype=FP8_DTYPE, device=dev)
    vq = torch.empty(nblk, h, d, bs, dtype=FP8_DTYPE, device=dev)
    ks = torch.empty(nblk, h, bs, 1, dtype=torch.float32, device=dev)
    vs = torch.empty(nblk, h, bs, 1, dtype=torch.float32, device=dev)
    lib = _cabi.load_library()
    _cabi.check(lib.pa_quantize_kv_cache(kc.data_ptr(), vc.data_ptr(), kq.data_ptr(), vq.data_ptr(), ks.data_ptr(),
                                         vs.data_ptr(), nblk, h, d, bs, _stream(dev)), "pa_quantize_kv_cache")
    ks_flat = ks.permute(1, 0, 2, 3).contiguous().view(h, nblk * bs)
    vs_flat = vs.permute(1, 0, 2, 3).contiguous().view(h, nblk * bs)
    return kq, ks_flat, vq, vs_flat, ks, vs


def kv_cache_write(
    key: torch.Tensor,           # [num_tokens, num_kv_heads, head_size] bf16
    value: torch.Tensor,
    key_cache: torch.Tensor,     # [blocks, Hkv, D/x, bs, x]  bf16 or float8_e4m3fn
    value_cache: torch.Tensor,   # [blocks, Hkv, D, bs], or transposed [blocks, Hkv, bs/x, D, x]
    slot_mapping: torch.Tensor,  # [num_tokens] int64, block * block_size + offset; negative = skip
    key_scale: Optional[torch.Tensor] = None,    # FP8 cache: [blocks, Hkv, bs, 1] (written) or 0-dim (read)
    value_scale: Optional[torch.Tensor] = None,
) -> None:
    if key.dtype != torch.bfloat16 or value.dtype != torch.bfloat16 or key.shape != value.shape or key.dim() != 3:
        raise ValueError("key and value must be bfloat16 [num_tokens, num_kv_heads, head_size]")
    if not key.is_cuda:
        raise ValueError("kv_cache_write runs on the GPU only")
    # every pointer below is dereferenced by the kernel: a host tensor (a slot_mapping built on the CPU, say)
    # would be a GPU memory fault, not an exception
    for name, t_ in (("value", value), ("key_cache", key_cache), ("value_cache", value_cache),
                     ("slot_mapping", slot_mapping), ("key_scale", key_scale), ("value_scale", value_scale)):
        if t_ is not None and t_.device != key.device:
            raise ValueError(f"{name} is on {t_.device}, key on {key.device}")
    t, h, d = key.shape
    if key.stride(2) != 1 or value.stride(2) != 1:
        raise ValueError("key/value must be contiguous in the last dimension")
    if slot_mapping.dtype != torch.int64 or slot_mapping.numel() != t or not slot_mapping.is_contiguous():
        raise ValueError("slot_mapping must be contiguous int64 [num_tokens]")
    if key_cache.dtype not in (torch.bfloat16, FP8_DTYPE) or value_cache.dtype != key_cache.dtype:
        raise ValueError("caches must both be bfloat16 or float8_e4m3fn")
    x = 16 // key_cache.element_size()
    bs = key_cache.shape[-2]
    v_transposed = value_cache.dim() == 5
    v_inner = (bs // x, d, x) if v_transposed else (d, bs)
    if key_cache.dim() != 5 or tuple(key_cache.shape[1:]) != (h, d // x, bs, x) or \
            tuple(value_cache.shape[1:]) != (h,) + v_inner or (v_transposed and bs % x):
        raise ValueError("cache shapes must be [blocks, Hkv, D/x, bs, x] and [blocks, Hkv, D, bs] "
                         "(or [blocks, Hkv, bs/x, D, x] for the transposed V layout)")
    v_dense = (d * x, x, 1) if v_transposed else (bs, 1)
    def _dense(t, want):  # the stride of a dimension of size 1 means nothing
        return all(n == 1 or st == w for n, st, w in zip(t.shape, t.stride(), want))

    if not _dense(key_cache[0, 0], (bs * x, x, 1)) or not _dense(value_cache[0, 0], v_dense):
        raise ValueError("the cache dimensions inside a (block, head) must be dense")
    a = PaKvWriteArgs()
    a.struct_size = C.sizeof(PaKvWriteArgs)
    a.key, a.value, a.slot_mapping = key.data_ptr(), value.data_ptr(), slot_mapping.data_ptr()
    a.key_cache, a.value_cache = key_cache.data_ptr(), value_cache.data_ptr()
    a.num_tokens, a.num_kv_heads, a.head_size, a.block_size = t, h, d, bs
    a.cache_dtype = _cabi.PA_DTYPE_FP8_E4M3FN if key_cache.dtype == FP8_DTYPE else _cabi.PA_DTYPE_BF16
    mode = _cabi.PA_QUANT_NONE
    if key_scale is not None or value_scale is not None:
        if key_scale is None or value_scale is None or key_scale.shape != value_scale.shape or \
                key_scale.dtype != torch.float32 or value_scale.dtype != torch.float32:
            raise ValueError("key_scale and value_scale must be float32 tensors of the same shape")
        if key_cache.dtype != FP8_DTYPE:
            raise ValueError("scales need an FP8 cache")
        if key_scale.dim() == 0:
            mode = _cabi.PA_QUANT_PER_TENSOR
        else:
            if tuple(key_scale.shape) != (key_cache.shape[0], h, bs, 1) or key_scale.stride(2) != 1 or \
                    key_scale.stride() != value_scale.stride():
                raise ValueError(f"per-token scales must be [blocks, {h}, {bs}, 1], dense over tokens, same strides")
            mode = _cabi.PA_QUANT_PER_TOKEN
            a.stride_scale_b, a.stride_scale_h = key_scale.stride(0), key_scale.stride(1)
        a.key_scale, a.value_scale = key_scale.data_ptr(), value_scale.data_ptr()
    a.kv_quant_mode = mode
    a.v_transposed = 1 if v_transposed else 0
    a.stride_k_t, a.stride_k_h, a.stride_v_t, a.stride_v_h = key.stride(0), key.stride(1), value.stride(0), value.stride(1)
    a.stride_kc_b, a.stride_kc_h = key_cache.stride(0), key_cache.stride(1)
    a.stride_vc_b, a.stride_vc_h = value_cache.stride(0), value_cache.stride(1)
    lib = _cabi.load_library()
    _cabi.check(lib.pa_kv_cache_write(C.byref(a), _stream(key.device)), "pa_kv_cache_write")
