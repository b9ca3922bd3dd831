"""Drop-in module for the reference's pa_decode_triton_gluon_fp8: same function name, same
parameter order (pa_decode_triton_gluon_fp8.py:1659-1675), HIP kernels behind it."""
from .pa_decode import paged_attention_decode  # noqa: F401

__all__ = ["paged_attention_decode"]
