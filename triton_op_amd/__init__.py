"""MI355X-native split-KV paged-attention decode (FP8 / bf16 KV cache) behind the reference's
Python entry point.  The arithmetic lives in hand-written HIP kernels for gfx950 in
`libpa_decode.so` (C ABI: include/pa_decode.h); this package is the thin host side."""
from .pa_decode import (  # noqa: F401
    DecodePlan,
    paged_attention_decode,
    plan_decode,
    select_partition_size,
)
from .kv_cache import kv_cache_write, quantize_kv_cache_symmetric  # noqa: F401
from . import kv_layout, workloads  # noqa: F401

__all__ = ["paged_attention_decode", "plan_decode", "DecodePlan", "select_partition_size", "kv_cache_write",
           "quantize_kv_cache_symmetric", "kv_layout", "workloads"]
