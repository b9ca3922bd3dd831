"""Drop-in module for the reference's pa_decode_triton: the entry point with the shorter signature
(pa_decode_triton.py:523-537: bf16 query, no query_sequence_length / query_scale) and its result
keys (`tmp_output`, `exp_sums`, `max_logits`)."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from . import pa_decode as _impl


def paged_attention_decode(
    output: torch.Tensor,        # [num_seqs, num_kv_heads*query_grp_sz, head_sz]
    query: torch.Tensor,         # [num_seqs, num_kv_heads*query_grp_sz, head_sz]
    key_cache: torch.Tensor,     # [num_blks, num_kv_heads, head_sz/x, kv_blk_sz, x]
    value_cache: torch.Tensor,   # [num_blks, num_kv_heads, head_sz, kv_blk_sz]
    seq_lens: torch.Tensor,      # [num_seqs]
    block_tables: torch.Tensor,  # [num_seqs, max_num_blks_per_seq]
    attn_scale: float,
    max_seq_len: int,
    compute_type=None,
    k_scale: Optional[torch.Tensor] = None,
    v_scale: Optional[torch.Tensor] = None,
    num_seq_partitions: int = 0,
    alibi_slopes: Optional[torch.Tensor] = None,
    max_logits: Optional[torch.Tensor] = None,   # trailing positions of run_triton (test_pa_decode_gluon_triton.py:264-281)
    exp_sums: Optional[torch.Tensor] = None,
    tmp_output: Optional[torch.Tensor] = None,
    *,
    partition_size: Optional[int] = None,
) -> Dict[str, object]:
    # The reference reads the scalar scales with .item() (a host sync per call, :619-620); here the
    # kernel reads the 0-dim device tensors itself.  A 16-bit cache takes no scales.
    if key_cache.dtype == torch.bfloat16:
        k_scale = v_scale = None
    res = _impl.paged_attention_decode(
        output, query, key_cache, value_cache, seq_lens, block_tables, attn_scale, 1, max_seq_len,
        compute_type, None, k_scale, v_scale, num_seq_partitions, alibi_slopes, max_logits, exp_sums, tmp_output,
        partition_size=partition_size)
    return {
        "tmp_output": res["temporary_output"],
        "exp_sums": res["exponential_sums"],
        "max_logits": res["maximum_logits"],
        "partition_size": res["partition_size"],
        "triton_decode": None,
        "triton_reduce": None,
        "triton": None,
    }
