"""ctypes binding of libpa_decode.so (the C ABI in include/pa_decode.h).

The library is loaded lazily and never built here: a missing library is an error, not a reason
to fall back to another implementation.
"""
from __future__ import annotations

import ctypes as C
import os
import threading

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libpa_decode.so")

PA_DECODE_ABI_VERSION = 5
PA_DECODE_WORKSPACE_BYTES = 64
PA_DECODE_NOALLOC_SCRATCH_BYTES = 64 << 20
PA_ERR_SCRATCH_TOO_SMALL = -7
PA_DECODE_FLAG_REUSE_ITEM_LIST = 1
PA_DECODE_FLAG_OUTPUT_ONLY = 2
PA_DTYPE_BF16, PA_DTYPE_FP8_E4M3FN = 0, 1
PA_QUANT_NONE, PA_QUANT_PER_TENSOR, PA_QUANT_PER_TOKEN = -1, 0, 1

EXPORTED_SYMBOLS = (
    "pa_decode_abi_version",
    "pa_decode_args_size",
    "pa_decode_error_string",
    "pa_decode_last_hip_error",
    "pa_decode_workspace_bytes",
    "pa_decode_select_partition_size",
    "pa_decode_select_partition_size_stats",
    "pa_decode_partition",
    "pa_decode_reduce",
    "pa_decode",
    "pa_decode_noalloc",
    "pa_decode_launch_info",
    "pa_debug_fp8_decode",
    "pa_kv_cache_write",
    "pa_quantize_kv_cache",
)


class PaDecodeArgs(C.Structure):
    _fields_ = (
        [("struct_size", C.c_uint32), ("flags", C.c_int32)]
        + [(n, C.c_void_p) for n in (
            "output", "query", "key_cache", "value_cache", "context_lens", "block_tables", "q_lens",
            "query_scale", "key_scale", "value_scale", "alibi_slopes", "sinks", "exp_sums", "max_logits", "tmp_output",
            "workspace")]
        + [(n, C.c_int32) for n in (
            "num_seqs", "num_kv_heads", "group_size", "q_len", "head_size", "block_size",
            "max_num_partitions", "partition_size", "query_dtype", "kv_dtype", "query_quant_mode",
            "kv_quant_mode", "v_transposed", "alibi_slopes_len", "reserved0")]
        + [("softmax_scale", C.c_float)]
        + [(n, C.c_int64) for n in (
            "stride_out_s", "stride_out_h", "stride_q_s", "stride_q_h",
            "stride_k_b", "stride_k_h", "stride_k_c", "stride_v_b", "stride_v_h", "stride_v_2",
            "stride_bt_s", "stride_es_s", "stride_es_h", "stride_es_p",
            "stride_tmp_s", "stride_tmp_h", "stride_tmp_p", "stride_tmp_g",
            "stride_qscale_s", "stride_kvscale_b", "stride_kvscale_h", "workspace_bytes")]
    )


class PaKvWriteArgs(C.Structure):
    _fields_ = (
        [("struct_size", C.c_uint32), ("reserved0", C.c_int32)]
        + [(n, C.c_void_p) for n in ("key", "value", "slot_mapping", "key_cache", "value_cache", "key_scale", "value_scale")]
        + [("num_tokens", C.c_int64)]
        + [(n, C.c_int32) for n in ("num_kv_heads", "head_size", "block_size", "cache_dtype", "kv_quant_mode", "v_transposed")]
        + [(n, C.c_int64) for n in (
            "stride_k_t", "stride_k_h", "stride_v_t", "stride_v_h", "stride_kc_b", "stride_kc_h", "stride_vc_b",
            "stride_vc_h", "stride_scale_b", "stride_scale_h")]
    )


class PaDecodeLibraryError(RuntimeError):
    pass


_lib = None
_lock = threading.Lock()


def load_library(path: str = None) -> C.CDLL:
    """dlopen the HIP library and check that its struct layout matches this binding.
    The environment variable PA_DECODE_LIB names another build of the library to load instead."""
    global _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = path or os.environ.get("PA_DECODE_LIB") or LIB_PATH
        if not os.path.exists(path):
            raise PaDecodeLibraryError(
                f"{path} is missing: build it with `python -m triton_op_amd.build` "
                "(there is no fallback implementation)")
        lib = C.CDLL(path)
        lib.pa_decode_abi_version.restype = C.c_int
        lib.pa_decode_args_size.restype = C.c_uint32
        lib.pa_decode_error_string.restype = C.c_char_p
        lib.pa_decode_error_string.argtypes = [C.c_int]
        lib.pa_decode_last_hip_error.restype = C.c_int
        lib.pa_decode_workspace_bytes.restype = C.c_int64
        lib.pa_decode_workspace_bytes.argtypes = [C.c_int32, C.c_int32]
        lib.pa_decode_select_partition_size.restype = C.c_int
        lib.pa_decode_select_partition_size.argtypes = [C.c_int32] * 6
        lib.pa_decode_select_partition_size_stats.restype = C.c_int
        lib.pa_decode_select_partition_size_stats.argtypes = [C.c_int32] * 4 + [C.c_int64, C.c_int32, C.c_int32]
        for name in ("pa_decode_partition", "pa_decode_reduce", "pa_decode", "pa_decode_noalloc"):
            fn = getattr(lib, name)
            fn.restype = C.c_int
            fn.argtypes = [C.POINTER(PaDecodeArgs), C.c_void_p]
        lib.pa_decode_launch_info.restype = C.c_int
        lib.pa_decode_launch_info.argtypes = [C.POINTER(PaDecodeArgs), C.c_char_p, C.c_int32]
        lib.pa_debug_fp8_decode.restype = C.c_int
        lib.pa_debug_fp8_decode.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p]
        lib.pa_kv_cache_write.restype = C.c_int
        lib.pa_kv_cache_write.argtypes = [C.POINTER(PaKvWriteArgs), C.c_void_p]
        lib.pa_quantize_kv_cache.restype = C.c_int
        lib.pa_quantize_kv_cache.argtypes = [C.c_void_p] * 6 + [C.c_int64, C.c_int32, C.c_int32, C.c_int32, C.c_void_p]
        if lib.pa_decode_abi_version() != PA_DECODE_ABI_VERSION:
            raise PaDecodeLibraryError("libpa_decode.so has a different ABI version; rebuild it")
        if lib.pa_decode_args_size() != C.sizeof(PaDecodeArgs):
            raise PaDecodeLibraryError(
                f"PaDecodeArgs is {lib.pa_decode_args_size()} bytes in the library but "
                f"{C.sizeof(PaDecodeArgs)} in the binding")
        _lib = lib
        return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        lib = load_library()
        msg = lib.pa_decode_error_string(rc).decode()
        raise PaDecodeLibraryError(f"{what} failed: {msg} (code {rc}, hipError {lib.pa_decode_last_hip_error()})")
