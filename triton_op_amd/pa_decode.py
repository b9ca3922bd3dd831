"""Host side of the paged-attention decode op: argument checking, buffer allocation, partition-size
choice and the two launches through the C ABI.

`paged_attention_decode` keeps the parameter order, tensor conventions, error conditions and the
returned dictionary of the reference entry point (pa_decode_triton_gluon_fp8.py:1659-1897);
`triton_op_amd.pa_decode_triton.paged_attention_decode` is the twin with the shorter signature of
pa_decode_triton.py:523-685.  Differences, all additive:

* `query` may be bf16 (no `query_scale`) as well as FP8 e4m3fn with a per-tensor or per-token scale;
* the caches may be bf16 (no scales) as well as FP8 with per-tensor (0-dim) or per-token scales;
* the partition buffers can be passed in, in which case nothing is allocated: `max_logits`, `exp_sums`,
  `tmp_output` (or `temp_output`) follow `alibi_slopes`, positionally or by keyword, as in the reference's harness
  wrappers (test_pa_mtp.py:566-584 run_gluon_fp8_kernel, test_pa_decode_gluon_triton.py:264-297 run_triton, which
  accept and ignore them);
* `alibi_slopes` holds one slope per packed query row ([num_kv_heads * query_sequence_length * group], what the
  reference kernels index, :323-327) or one per query head ([num_kv_heads * group]);
* `partition_size` may be any multiple of 256 (the reference's constant); by default the tuning
  layer picks it from the batch shape and the longest context;
* `total_context_tokens` (a host integer: the sum of `sequence_lengths`, which a serving engine has at hand) is the
  second context-length statistic the tuning layer uses beside `max_sequence_length`; nothing is read back from the
  device for it;
* `query_lens` gives a per-sequence number of new tokens (ragged MTP batches);
* `sinks` gives an attention-sink logit per query row ([num_kv_heads * query_group_size], as the reference's
  Gluon reduce kernel indexes it, pa_decode_triton_gluon_fp8.py:1118-1123): exp(sink - max) joins the softmax
  denominator;
* `workspace` is an int32 tensor of at least 64 bytes whose first 64 bytes are zero (a work-item counter for
  ragged batches); with `pa_decode_workspace_bytes(num_seqs, partitions)` bytes it also has room for the item
  list of the sorted dispatch.  One is allocated per call/plan when it is not given; calls that may overlap on
  the GPU need one each.

There is no eager/torch implementation behind this function: without the HIP library it raises.
"""
from __future__ import annotations

import ctypes as C
import functools
from typing import Dict, Optional

import torch

from . import _cabi
from ._cabi import PaDecodeArgs

PARTITION_GRANULE = 256  # the reference's _SEQUENCE_PARTITION_SIZE (pa_decode_triton_gluon_fp8.py:24)
FP8_DTYPE = torch.float8_e4m3fn
_SUPPORTED_BLOCK_SIZES = (16, 64, 1024)


def _dtype_code(t: torch.Tensor, what: str) -> int:
    if t.dtype == torch.bfloat16:
        return _cabi.PA_DTYPE_BF16
    if t.dtype == FP8_DTYPE:
        return _cabi.PA_DTYPE_FP8_E4M3FN
    raise ValueError(f"{what} tensor only supports dtype bfloat16 or float8_e4m3fn, but got {t.dtype}")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


@functools.lru_cache(maxsize=4096)
def select_partition_size(num_seqs: int, num_kv_heads: int, rows_per_group: int, max_context_len: int,
                          block_size: int, num_cus: int = 0, total_context_tokens: int = 0) -> int:
    """The tuning layer's choice of tokens per partition (a multiple of 256) from the batch shape and the context
    lengths' statistics: the longest and, when the caller knows it (a host value: nothing is read back from the
    device), their sum.  A pure function of its arguments (and of the GPU's CU count when num_cus is 0), hence cached."""
    lib = _cabi.load_library()
    ps = lib.pa_decode_select_partition_size_stats(num_seqs, num_kv_heads, rows_per_group, max(1, max_context_len),
                                                   int(total_context_tokens), block_size, num_cus)
    if ps < 0:
        _cabi.check(ps, "pa_decode_select_partition_size_stats")
    return ps


class DecodePlan:
    """A validated call: the filled C struct plus the tensors it points to (kept alive).
    `run()` enqueues partition + reduce on a stream; it allocates nothing and can be replayed."""

    def __init__(self, args: PaDecodeArgs, keep, exp_sums, max_logits, tmp_output, output, workspace=None):
        self.args = args
        self._keep = keep
        self.exp_sums, self.max_logits, self.tmp_output, self.output = exp_sums, max_logits, tmp_output, output
        self.workspace = workspace
        self._lib = _cabi.load_library()

    def run(self, stream: Optional[int] = None) -> None:
        if stream is None:
            stream = torch.cuda.current_stream(self.output.device).cuda_stream
        _cabi.check(self._lib.pa_decode(C.byref(self.args), C.c_void_p(stream)), "pa_decode")

    def launch_info(self) -> str:
        """The partition kernel instantiation, grid and item source the launch layer chooses for this call."""
        buf = C.create_string_buffer(256)
        _cabi.check(self._lib.pa_decode_launch_info(C.byref(self.args), buf, 256), "pa_decode_launch_info")
        return buf.value.decode()

    def run_noalloc(self, stream: Optional[int] = None) -> None:
        """The same call through `pa_decode_noalloc`: the partition buffers and the workspace of this plan are
        left alone, the library uses its own per-GPU scratch array instead (64 MiB; larger calls raise).  Calls
        that may overlap on one GPU share that array and race."""
        if stream is None:
            stream = torch.cuda.current_stream(self.output.device).cuda_stream
        a = PaDecodeArgs.from_buffer_copy(self.args)
        a.exp_sums = a.max_logits = a.tmp_output = a.workspace = None
        a.workspace_bytes = 0
        a.flags &= _cabi.PA_DECODE_FLAG_OUTPUT_ONLY
        _cabi.check(self._lib.pa_decode_noalloc(C.byref(a), C.c_void_p(stream)), "pa_decode_noalloc")

    def run_partition(self, stream: Optional[int] = None) -> None:
        if stream is None:
            stream = torch.cuda.current_stream(self.output.device).cuda_stream
        _cabi.check(self._lib.pa_decode_partition(C.byref(self.args), C.c_void_p(stream)), "pa_decode_partition")

    def run_reduce(self, stream: Optional[int] = None) -> None:
        if stream is None:
            stream = torch.cuda.current_stream(self.output.device).cuda_stream
        _cabi.check(self._lib.pa_decode_reduce(C.byref(self.args), C.c_void_p(stream)), "pa_decode_reduce")


def plan_decode(
    output: torch.Tensor,
    query: torch.Tensor,
    key_cache: torch.Tensor,
    value_cache: torch.Tensor,
    sequence_lengths: torch.Tensor,
    block_tables: torch.Tensor,
    softmax_scale: float,
    query_sequence_length: int,
    max_sequence_length: int,
    compute_type=None,
    query_scale: Optional[torch.Tensor] = None,
    key_scale: Optional[torch.Tensor] = None,
    value_scale: Optional[torch.Tensor] = None,
    num_sequence_partitions: int = 0,
    alibi_slopes: Optional[torch.Tensor] = None,
    max_logits: Optional[torch.Tensor] = None,
    exp_sums: Optional[torch.Tensor] = None,
    tmp_output: Optional[torch.Tensor] = None,
    *,
    temp_output: Optional[torch.Tensor] = None,
    partition_size: Optional[int] = None,
    query_lens: Optional[torch.Tensor] = None,
    workspace: Optional[torch.Tensor] = None,
    sinks: Optional[torch.Tensor] = None,
    reuse_item_list: bool = False,
    total_context_tokens: int = 0,
    output_only: bool = False,
) -> DecodePlan:
    if temp_output is not None:  # the spelling of run_gluon_fp8_kernel (test_pa_mtp.py:566-584)
        if tmp_output is not None and tmp_output is not temp_output:
            raise ValueError("tmp_output and temp_output name the same buffer: pass one of them")
        tmp_output = temp_output
    # ---- shapes (pa_decode_triton_gluon_fp8.py:1703-1722) ------------------------------------
    if output.dim() != 3:
        raise ValueError(f"Expected 3D output tensor, but got shape {tuple(output.shape)}")
    if query.dim() != 3:
        raise ValueError(f"Expected 3D query tensor, but got shape {tuple(query.shape)}")
    if key_cache.dim() != 5:
        raise ValueError(f"Expected 5D key_cache tensor, but got shape {tuple(key_cache.shape)}")
    if value_cache.dim() not in (4, 5):
        raise ValueError(f"Unsupported value cache shape: {tuple(value_cache.shape)}")
    dev = output.device
    for name, t in (("query", query), ("key_cache", key_cache), ("value_cache", value_cache),
                    ("sequence_lengths", sequence_lengths), ("block_tables", block_tables),
                    ("query_scale", query_scale), ("key_scale", key_scale), ("value_scale", value_scale),
                    ("alibi_slopes", alibi_slopes), ("exp_sums", exp_sums), ("max_logits", max_logits),
                    ("tmp_output", tmp_output), ("query_lens", query_lens)):
        if t is not None and t.device != dev:
            raise ValueError(f"{name} is on {t.device}, output on {dev}")

    q_len = int(query_sequence_length)
    num_seqs, rows_total, head_size = query.shape
    num_kv_heads = key_cache.shape[1]
    block_size = key_cache.shape[-2]
    if q_len < 1 or rows_total % (q_len * num_kv_heads):
        raise ValueError(
            f"query.shape[1]={rows_total} is not num_kv_heads*query_sequence_length*group "
            f"({num_kv_heads}*{q_len}*G)")
    group = rows_total // (q_len * num_kv_heads)
    ge = q_len * group
    ge_pow2 = 16 if ge <= 16 else 1 << (ge - 1).bit_length()
    if tuple(output.shape) != tuple(query.shape):
        raise ValueError(f"output shape {tuple(output.shape)} differs from query shape {tuple(query.shape)}")

    # ---- dtypes and constraints (:1742-1750) --------------------------------------------------------
    q_code = _dtype_code(query, "query")
    kv_code = _dtype_code(key_cache, "key_cache")
    if value_cache.dtype != key_cache.dtype:
        raise ValueError(f"value_cache dtype {value_cache.dtype} differs from key_cache dtype {key_cache.dtype}")
    if output.dtype != torch.bfloat16:
        raise ValueError(f"output tensor only support dtype == torch.bfloat16, but got output.dtype == {output.dtype}")
    if compute_type is not None and compute_type != torch.bfloat16:
        raise ValueError(f"compute_type must be torch.bfloat16 (or None), got {compute_type}")
    if ge_pow2 > 64:
        raise ValueError(f"equivalent_query_group_size_pow2={ge_pow2} exceeds maximum of 64")
    if block_size not in _SUPPORTED_BLOCK_SIZES:
        raise ValueError(f"kv_block_size == {block_size} not in {list(_SUPPORTED_BLOCK_SIZES)}")
    if head_size not in (64, 128, 256):  # (128 on the tuned kernels, 64 and 256 on the generic ones)
        raise ValueError(f"head_size == {head_size} is not supported (64, 128 or 256)")
    x = 16 // key_cache.element_size()
    if key_cache.shape[-1] != x or key_cache.shape[2] * x != head_size:
        raise ValueError(f"key_cache shape {tuple(key_cache.shape)} is not [blocks, kv_heads, {head_size}//{x}, bs, {x}]")
    if sequence_lengths.dtype != torch.int32 or block_tables.dtype != torch.int32:
        raise ValueError("sequence_lengths and block_tables must be int32")
    if sequence_lengths.numel() != num_seqs or block_tables.shape[0] != num_seqs:
        raise ValueError("sequence_lengths / block_tables do not have one row per sequence")

    # ---- value layout (:1793-1799) -------------------------------------------------------------------
    v_transposed = value_cache.dim() == 5
    if v_transposed:
        if tuple(value_cache.shape[1:]) != (num_kv_heads, block_size // x, head_size, x):
            raise ValueError(f"transposed value_cache shape {tuple(value_cache.shape)} is not [blocks, kv_heads, bs/{x}, D, {x}]")
        dense = value_cache.stride(4) == 1 and value_cache.stride(3) == x
    else:
        if tuple(value_cache.shape[1:]) != (num_kv_heads, head_size, block_size):
            raise ValueError(f"value_cache shape {tuple(value_cache.shape)} is not [blocks, kv_heads, D, bs]")
        dense = value_cache.stride(3) == 1
    if not dense or key_cache.stride(4) != 1 or key_cache.stride(3) != x:
        raise ValueError("the innermost cache dimensions must be dense")
    if query.stride(2) != 1 or output.stride(2) != 1 or block_tables.stride(1) != 1 or not sequence_lengths.is_contiguous():
        raise ValueError("query/output/block_tables must be contiguous in their last dimension")
    if block_tables.stride(0) < max(1, block_tables.shape[1]):
        # rows that overlap (one row expanded over the batch): the kernels want every row in a stride of its own
        block_tables = block_tables.contiguous()

    # ---- quantisation modes (:1753-1790) ---------------------------------------------------------------
    q_mode, stride_qs = _cabi.PA_QUANT_NONE, 0
    if query_scale is not None:
        if not isinstance(query_scale, torch.Tensor) or query_scale.dtype != torch.float32:
            raise ValueError("query_scale tensor only support dtype == torch.float32")
        if query_scale.dim() == 0:
            q_mode = _cabi.PA_QUANT_PER_TENSOR
        else:
            if query_scale.dim() != 3:
                raise ValueError(f"Expected 3D query_scale tensor, but got shape {tuple(query_scale.shape)}")
            if query_scale.shape[-1] != 1 or tuple(query_scale.shape[:2]) != (num_seqs, rows_total):
                raise ValueError(f"Expected query_scale shape [{num_seqs}, {rows_total}, 1], got {tuple(query_scale.shape)}")
            if query_scale.stride(1) != 1:
                raise ValueError("query_scale must be dense over the row dimension")
            q_mode = _cabi.PA_QUANT_PER_TOKEN
            stride_qs = query_scale.stride(0)
    elif q_code == _cabi.PA_DTYPE_FP8_E4M3FN:
        q_mode = _cabi.PA_QUANT_NONE
    kv_mode, stride_kvs_b, stride_kvs_h = _cabi.PA_QUANT_NONE, 0, 0
    if key_scale is not None and value_scale is not None:
        for nm, sc in (("key_scale", key_scale), ("value_scale", value_scale)):
            if not isinstance(sc, torch.Tensor) or sc.dtype != torch.float32:
                raise ValueError(f"{nm} tensor only support dtype == torch.float32")
        if key_scale.shape != value_scale.shape:
            raise ValueError(f"Key and value scales must have same shape, but got key: {tuple(key_scale.shape)}, value: {tuple(value_scale.shape)}")
        if key_scale.dim() == 0:
            kv_mode = _cabi.PA_QUANT_PER_TENSOR
        else:
            if key_scale.dim() != 4:
                raise ValueError(f"Expected 4D key_scale tensor, but got shape {tuple(key_scale.shape)}")
            if key_scale.shape[-1] != 1:
                raise ValueError(f"Expected key_scale.shape[-1] == 1, but got key_scale.shape[-1]={key_scale.shape[-1]}")
            if tuple(key_scale.shape[1:3]) != (num_kv_heads, block_size) or key_scale.shape[0] != key_cache.shape[0]:
                raise ValueError(f"Expected key_scale shape [blocks, {num_kv_heads}, {block_size}, 1], got {tuple(key_scale.shape)}")
            if key_scale.stride() != value_scale.stride() or key_scale.stride(2) != 1:
                raise ValueError("per-token key/value scales must share strides and be dense over tokens")
            if kv_code != _cabi.PA_DTYPE_FP8_E4M3FN:
                raise ValueError("per-token scales need an FP8 cache")
            kv_mode = _cabi.PA_QUANT_PER_TOKEN
            stride_kvs_b, stride_kvs_h = key_scale.stride(0), key_scale.stride(1)
    elif (key_scale is None) != (value_scale is None):
        raise ValueError("key_scale and value_scale must be given together")
    if alibi_slopes is not None:
        # one slope per packed query row, [num_kv_heads * query_sequence_length * group] at h*Ge + t*G + g: the array the
        # reference kernels index (:323-327, :803-810); or one per query head, [num_kv_heads * group]
        if alibi_slopes.dtype != torch.float32 or not alibi_slopes.is_contiguous() or \
                alibi_slopes.numel() not in (rows_total, num_kv_heads * group):
            raise ValueError(f"alibi_slopes must be contiguous float32 [{rows_total}] (one slope per query row) "
                             f"or [{num_kv_heads * group}] (one per query head)")
    if sinks is not None:
        if sinks.dtype != torch.float32 or sinks.numel() != rows_total or not sinks.is_contiguous() or sinks.device != dev:
            raise ValueError(f"sinks must be contiguous float32 [{rows_total}] (one logit per query row) on {dev}")
    if query_lens is not None:
        if query_lens.dtype != torch.int32 or query_lens.numel() != num_seqs or not query_lens.is_contiguous():
            raise ValueError("query_lens must be contiguous int32 [num_seqs]")

    if not output.is_cuda:
        raise ValueError("paged_attention_decode runs on the GPU only (there is no CPU path); got a CPU tensor")
    if reuse_item_list and workspace is None:
        raise ValueError("reuse_item_list needs the workspace the earlier call left its item list in")

    # ---- partitioning: the launch / tuning layer ---------------------------------------------------------
    max_seq = max(1, int(max_sequence_length))
    given = [t is not None for t in (exp_sums, max_logits, tmp_output)]
    if any(given) and not all(given):
        raise ValueError("exp_sums, max_logits and tmp_output must be passed together")
    if partition_size is None:
        if all(given):
            partition_size = PARTITION_GRANULE
            while exp_sums.shape[2] * partition_size < max_seq:
                partition_size += PARTITION_GRANULE
        elif num_sequence_partitions and num_sequence_partitions > 0:
            per = -(-max_seq // int(num_sequence_partitions))
            partition_size = -(-per // PARTITION_GRANULE) * PARTITION_GRANULE
        elif head_size != 128:
            # the generic kernels run one wave per (sequence, partition, kv head, 16-row tile), four waves per SIMD
            # (two at head size 256): the longest partitions of up to 1024 tokens that still give every wave slot a
            # wave (measured at 64 sequences x 8 kv heads x 4096 tokens: head 64 67 / 61 / 59 us per call at 256 / 512 /
            # 1024, head 256 207 / 196 / 228 us at 512 / 1024 / 2048), longer ones only to keep the launch under a few
            # dozen waves per SIMD
            def waves(ps):
                return num_seqs * num_kv_heads * -(-ge // 16) * -(-max_seq // ps)

            slots = torch.cuda.get_device_properties(dev).multi_processor_count * 4 * (2 if head_size == 256 else 4)
            partition_size = PARTITION_GRANULE
            while partition_size < 1024 and waves(2 * partition_size) >= slots:
                partition_size *= 2
            while waves(partition_size) > 32768 and partition_size < 4096:
                partition_size *= 2
        else:
            partition_size = select_partition_size(num_seqs, num_kv_heads, ge, max_seq, block_size, 0,
                                                   int(total_context_tokens))
    partition_size = int(partition_size)
    if partition_size <= 0 or partition_size % PARTITION_GRANULE:
        raise ValueError(f"partition_size must be a positive multiple of {PARTITION_GRANULE}, got {partition_size}")
    needed_parts = -(-max_seq // partition_size)
    if all(given):
        shape = (num_seqs, num_kv_heads, exp_sums.shape[2], ge)
        if tuple(exp_sums.shape) != shape or tuple(max_logits.shape) != shape or tuple(tmp_output.shape) != shape + (head_size,):
            raise ValueError(f"partition buffers must be [{num_seqs}, {num_kv_heads}, P, {ge}] (+[{head_size}])")
        if exp_sums.shape[2] < needed_parts:
            raise ValueError(f"partition buffers hold {exp_sums.shape[2]} partitions, {needed_parts} are needed")
        if exp_sums.dtype != torch.float32 or max_logits.dtype != torch.float32 or tmp_output.dtype != torch.bfloat16:
            raise ValueError("exp_sums/max_logits must be float32 and tmp_output bfloat16")
        if exp_sums.stride() != max_logits.stride() or exp_sums.stride(3) != 1 or tmp_output.stride(4) != 1:
            raise ValueError("exp_sums and max_logits must share strides; last dimensions must be dense")
        max_parts = exp_sums.shape[2]
    else:
        max_parts = needed_parts
        shape = (num_seqs, num_kv_heads, max_parts, ge)
        # zero-filled like the reference's (:1729-1733): slots of partitions a sequence does not reach
        # are never written or read by the kernels.  One allocation and one fill for the three buffers (and the
        # workspace, when the caller brought none): each torch.zeros is a kernel launch and ~5 us of host time.
        n = num_seqs * num_kv_heads * max_parts * ge
        sizes = [4 * n, 4 * n, 2 * n * head_size]
        if workspace is None:
            sizes.append(int(_cabi.load_library().pa_decode_workspace_bytes(num_seqs, max_parts)))
        offs, total = [], 0
        for sz in sizes:
            offs.append(total)
            total += -(-sz // 256) * 256
        pool = torch.zeros(total, dtype=torch.uint8, device=dev)
        max_logits = pool[offs[0]:offs[0] + sizes[0]].view(torch.float32).view(shape)
        exp_sums = pool[offs[1]:offs[1] + sizes[1]].view(torch.float32).view(shape)
        tmp_output = pool[offs[2]:offs[2] + sizes[2]].view(torch.bfloat16).view(shape + (head_size,))
        if workspace is None:
            workspace = pool[offs[3]:offs[3] + -(-sizes[3] // 4) * 4].view(torch.int32)

    a = PaDecodeArgs()
    a.struct_size = C.sizeof(PaDecodeArgs)
    a.output, a.query = output.data_ptr(), query.data_ptr()
    a.key_cache, a.value_cache = key_cache.data_ptr(), value_cache.data_ptr()
    a.context_lens, a.block_tables = sequence_lengths.data_ptr(), block_tables.data_ptr()
    a.q_lens = _ptr(query_lens)
    a.query_scale = _ptr(query_scale) if q_mode != _cabi.PA_QUANT_NONE else None
    a.key_scale = _ptr(key_scale) if kv_mode != _cabi.PA_QUANT_NONE else None
    a.value_scale = _ptr(value_scale) if kv_mode != _cabi.PA_QUANT_NONE else None
    a.alibi_slopes = _ptr(alibi_slopes)
    a.alibi_slopes_len = 0 if alibi_slopes is None else alibi_slopes.numel()
    a.sinks = _ptr(sinks)
    a.exp_sums, a.max_logits, a.tmp_output = exp_sums.data_ptr(), max_logits.data_ptr(), tmp_output.data_ptr()
    # zeroed work-item counter for ragged batches (the kernels leave it zero, so the plan can be replayed) plus
    # room for the item list of the sorted dispatch
    if workspace is None:
        need = int(_cabi.load_library().pa_decode_workspace_bytes(num_seqs, max_parts))
        workspace = torch.zeros((need + 3) // 4, dtype=torch.int32, device=dev)
    elif workspace.dtype != torch.int32 or workspace.numel() * 4 < _cabi.PA_DECODE_WORKSPACE_BYTES or \
            not workspace.is_contiguous() or workspace.device != dev:
        raise ValueError(f"workspace must be a contiguous int32 tensor of >= {_cabi.PA_DECODE_WORKSPACE_BYTES} bytes on {dev}")
    a.workspace = workspace.data_ptr()
    a.workspace_bytes = workspace.numel() * 4
    # the caller's word that `workspace` already holds the item list of a call with the same sequence lengths
    # and partitioning (the previous layer of this decode step): the planning kernel is skipped
    a.flags = (_cabi.PA_DECODE_FLAG_REUSE_ITEM_LIST if reuse_item_list else 0) | \
        (_cabi.PA_DECODE_FLAG_OUTPUT_ONLY if output_only else 0)
    a.num_seqs, a.num_kv_heads, a.group_size, a.q_len = num_seqs, num_kv_heads, group, q_len
    a.head_size, a.block_size = head_size, block_size
    a.max_num_partitions, a.partition_size = max_parts, partition_size
    a.query_dtype, a.kv_dtype = q_code, kv_code
    a.query_quant_mode, a.kv_quant_mode = q_mode, kv_mode
    a.v_transposed = int(v_transposed)
    a.softmax_scale = float(softmax_scale)
    a.stride_out_s, a.stride_out_h = output.stride(0), output.stride(1)
    a.stride_q_s, a.stride_q_h = query.stride(0), query.stride(1)
    a.stride_k_b, a.stride_k_h, a.stride_k_c = key_cache.stride(0), key_cache.stride(1), key_cache.stride(2)
    a.stride_v_b, a.stride_v_h, a.stride_v_2 = value_cache.stride(0), value_cache.stride(1), value_cache.stride(2)
    a.stride_bt_s = block_tables.stride(0)
    a.stride_es_s, a.stride_es_h, a.stride_es_p = exp_sums.stride(0), exp_sums.stride(1), exp_sums.stride(2)
    a.stride_tmp_s, a.stride_tmp_h, a.stride_tmp_p, a.stride_tmp_g = (tmp_output.stride(i) for i in range(4))
    a.stride_qscale_s, a.stride_kvscale_b, a.stride_kvscale_h = stride_qs, stride_kvs_b, stride_kvs_h
    keep = (output, query, key_cache, value_cache, sequence_lengths, block_tables, query_scale, key_scale,
            value_scale, alibi_slopes, query_lens, workspace, sinks)
    return DecodePlan(a, keep, exp_sums, max_logits, tmp_output, output, workspace)


def paged_attention_decode(
    output: torch.Tensor,            # [num_seqs, num_kv_heads * query_group_size, head_size]
    query: torch.Tensor,             # [num_seqs, num_kv_heads * query_group_size, head_size]
    key_cache: torch.Tensor,         # [num_blocks, num_kv_heads, head_size/x, kv_block_size, x]
    value_cache: torch.Tensor,       # [num_blocks, num_kv_heads, head_size, kv_block_size] or transposed 5-D
    sequence_lengths: torch.Tensor,  # [num_seqs] int32
    block_tables: torch.Tensor,      # [num_seqs, max_num_blocks_per_seq] int32
    softmax_scale: float,
    query_sequence_length: int,
    max_sequence_length: int,
    compute_type=None,
    query_scale: Optional[torch.Tensor] = None,  # 0-dim or [num_seqs, num_kv_heads * query_group_size, 1]
    key_scale: Optional[torch.Tensor] = None,    # 0-dim or [num_blocks, num_kv_heads, kv_block_size, 1]
    value_scale: Optional[torch.Tensor] = None,
    num_sequence_partitions: int = 0,
    alibi_slopes: Optional[torch.Tensor] = None,
    max_logits: Optional[torch.Tensor] = None,
    exp_sums: Optional[torch.Tensor] = None,
    tmp_output: Optional[torch.Tensor] = None,
    *,
    temp_output: Optional[torch.Tensor] = None,
    partition_size: Optional[int] = None,
    query_lens: Optional[torch.Tensor] = None,
    workspace: Optional[torch.Tensor] = None,
    sinks: Optional[torch.Tensor] = None,
    reuse_item_list: bool = False,
    total_context_tokens: int = 0,
    output_only: bool = False,
) -> Dict[str, object]:
    """Split-KV paged-attention decode; writes `output` in place on torch's current stream and
    returns the partition buffers under the reference's keys.  `output_only=True` (PA_DECODE_FLAG_OUTPUT_ONLY): the
    caller reads nothing but the rows of `output` that belong to real query rows; the partition buffers are scratch
    with unspecified contents afterwards, and rows beyond a sequence's `query_lens` entry are left as they were.
    With a caller-fixed small `partition_size` the library then cuts the partition axis into fewer, longer partitions
    of its own inside the same buffers (`plan.launch_info()` names their size)."""
    plan = plan_decode(
        output, query, key_cache, value_cache, sequence_lengths, block_tables, softmax_scale,
        query_sequence_length, max_sequence_length, compute_type, query_scale, key_scale, value_scale,
        num_sequence_partitions, alibi_slopes, max_logits, exp_sums, tmp_output, temp_output=temp_output,
        partition_size=partition_size, query_lens=query_lens, workspace=workspace,
        sinks=sinks, reuse_item_list=reuse_item_list, total_context_tokens=total_context_tokens, output_only=output_only)
    plan.run()
    return {
        "temporary_output": plan.tmp_output,
        "final_output": output,
        "exponential_sums": plan.exp_sums,
        "maximum_logits": plan.max_logits,
        "partition_size": int(plan.args.partition_size),
        # the reference's perftest timings have no counterpart: this op does not time itself
        "triton_decode_time": None,
        "triton_reduce_time": None,
        "total_triton_time": None,
    }
