"""Writes the small golden fixtures in this folder:  python -m tests.golden.make_golden

Each .npz holds the inputs of one tiny paged-decode case (raw cache bytes, block tables, scales) and
the expected output computed by `oracle.pa_oracle.brute_force_decode`: pure-Python double-precision
loops straight from the cache indexing rules, sharing no arithmetic with the torch oracle or the HIP
kernels.  The reference repository ships no golden vectors for this path (only md5s of outputs
from GPU random streams in gfx942's fnuz FP8), so these stand in for them.
"""
from __future__ import annotations

import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))

CASES = {
    # name: (kv_dtype, scale_mode, q_len, Hq, Hkv, block_size, context_lens)
    "fp8_tensor_g8_q1": ("fp8", "tensor", 1, 8, 1, 16, (1, 17, 40)),
    "fp8_token_g2_q2": ("fp8", "token", 2, 4, 2, 16, (2, 33, 21)),
    "bf16_g4_q1": ("bf16", "none", 1, 4, 1, 16, (16, 5, 31)),
    "fp8_tensor_g5_q3_bs64": ("fp8", "tensor", 3, 5, 1, 64, (3, 70)),
}


def _np(t: torch.Tensor) -> np.ndarray:
    if t.dtype == torch.bfloat16:
        return t.contiguous().view(torch.int16).numpy()
    if t.dtype == torch.float8_e4m3fn:
        return t.contiguous().view(torch.uint8).numpy()
    return t.contiguous().numpy()


def load_case(path: str) -> dict:
    z = np.load(path, allow_pickle=False)
    kv_dtype = str(z["kv_dtype"])
    kvt = torch.float8_e4m3fn if kv_dtype == "fp8" else torch.bfloat16

    def kv(a):
        t = torch.from_numpy(a.copy())
        return t.view(kvt)

    case = {
        "query": torch.from_numpy(z["query"].copy()).view(torch.bfloat16),
        "key_cache": kv(z["key_cache"]),
        "value_cache": kv(z["value_cache"]),
        "context_lens": torch.from_numpy(z["context_lens"].copy()),
        "block_tables": torch.from_numpy(z["block_tables"].copy()),
        "softmax_scale": float(z["softmax_scale"]),
        "q_len": int(z["q_len"]),
        "key_scale": None,
        "value_scale": None,
        "expected": torch.from_numpy(z["expected"].copy()),
    }
    if "key_scale" in z.files:
        case["key_scale"] = torch.from_numpy(z["key_scale"].copy())
        case["value_scale"] = torch.from_numpy(z["value_scale"].copy())
    return case


def main() -> None:
    from oracle import pa_oracle as O
    from triton_op_amd import workloads as W

    for i, (name, (kv_dtype, scale_mode, q_len, hq, hkv, bs, ctx)) in enumerate(CASES.items()):
        wl = W.make_decode_workload(
            name=name, seed=100 + i, batch=len(ctx), num_q_heads=hq, num_kv_heads=hkv, block_size=bs,
            context_lens=torch.tensor(ctx, dtype=torch.int32), q_len=q_len, kv_dtype=kv_dtype, scale_mode=scale_mode)
        exp = O.brute_force_decode(wl.query, wl.key_cache, wl.value_cache, wl.context_lens, wl.block_tables,
                                   wl.softmax_scale, q_len, wl.key_scale, wl.value_scale)
        arrays = dict(
            query=_np(wl.query), key_cache=_np(wl.key_cache), value_cache=_np(wl.value_cache),
            context_lens=_np(wl.context_lens), block_tables=_np(wl.block_tables),
            softmax_scale=np.float64(wl.softmax_scale), q_len=np.int32(q_len), kv_dtype=np.str_(kv_dtype),
            expected=np.asarray(exp, dtype=np.float64))
        if wl.key_scale is not None:
            arrays["key_scale"] = _np(wl.key_scale)
            arrays["value_scale"] = _np(wl.value_scale)
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **arrays)
        print("wrote", name)


if __name__ == "__main__":
    main()
