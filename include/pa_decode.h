/*
 * pa_decode.h -- C ABI of the MI355X (gfx950) split-KV paged-attention decode library.
 *
 * The reference exposes this path as a Python function that launches Triton/Gluon kernels
 * (pa_decode_triton_gluon_fp8.py:1659-1897 `paged_attention_decode`, twin
 * pa_decode_triton.py:523-685); it has no C interface of its own.  The entry points below are
 * what a foreign-function binding for that path binds instead: plain device pointers, element
 * strides exactly as the reference passes them to its kernels
 * (pa_decode_triton_gluon_fp8.py:1822-1841), sizes, enums, and a HIP stream handle.
 *
 * All functions return 0 on success or a negative PA_ERR_* code; none throws, allocates device
 * memory, synchronises the host with the device, or keeps a pointer after it returns.  All
 * kernels are enqueued on the given stream.  The library is re-entrant.
 */
#ifndef PA_DECODE_H_
#define PA_DECODE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PA_DECODE_ABI_VERSION 5
/* Smallest useful size of the optional device workspace.  Its first 64 bytes hold a work-item counter: with
 * it, batches with per-sequence query lengths are launched as a resident grid that pulls live (sequence,
 * partition, row tile, head) items from the counter instead of one workgroup per possible item.  These 64
 * bytes must be zero before the first call; every call leaves the counters (the first 8 bytes) zero, the rest of
 * the 64 bytes is scratch that a call writes before it reads it.  A workspace of
 * pa_decode_workspace_bytes() bytes also has room for the work-item list of the sorted dispatch: in launches of
 * several rounds of workgroups a small planning kernel lists the live (sequence, partition) items (with a small
 * caller-fixed partition_size: runs of up to four consecutive partitions that one workgroup walks), whole
 * partitions first and the sequences' last, partial partitions by decreasing length, and the partition kernel
 * takes its items from the list (longest-first keeps the end of a ragged batch's launch busy); it also lists the
 * sequences that have more than one partition, which are all that pa_decode's reduce stage then visits.  The
 * lists are rewritten by every call (unless PA_DECODE_FLAG_REUSE_ITEM_LIST says they are still good).  Calls that
 * may overlap on the GPU need a workspace each. */
#define PA_DECODE_WORKSPACE_BYTES 64
/*
 * flags: the workspace still holds the item list that an earlier call built for the SAME context_lens contents,
 * num_seqs, num_kv_heads, q_len, group_size, block_size, max_num_partitions, partition_size and
 * PA_DECODE_FLAG_OUTPUT_ONLY setting (the previous layer
 * of one decode step, say; the items a launch lists also depend on how many partitions it gives a workgroup, which
 * follows from those shapes): the planning kernel is skipped (about 4.5 us).  Ignored by launches that use no item
 * list.
 */
#define PA_DECODE_FLAG_REUSE_ITEM_LIST 1
/*
 * flags (the same value in pa_decode_partition and pa_decode_reduce when the stages are called one by one: stage 2
 * then passes over the sequences stage 1 finished, as it does inside pa_decode): the caller reads nothing but
 * the rows of `output` that belong to real query rows.  The partition buffers are then scratch whose contents
 * after the call are unspecified -- stage 1 does not write the entries of a sequence it finishes itself (one that
 * fits in one partition: nobody merges them) -- and, with per-sequence query lengths (q_lens), the rows of `output`
 * beyond a sequence's own query length are left as they were instead of being zeroed.  Writes cost this GPU about
 * three times what reads cost: on a ragged batch of 256 sequences with 1-4 new tokens in buffers padded to 4
 * (70 MB of partial results, zeros and outputs per call) this is 6 % of the call.
 * Scratch buffers also leave the cut of the partition axis to the library: a caller whose buffers are laid out for a
 * small fixed partition_size (the reference's 256) gets fewer, longer partitions inside the same buffers -- the
 * largest multiple of partition_size that is not above the tuning layer's own choice for the shape
 * (pa_decode_launch_info says "own partitions of N tokens"; 64 sequences x 8 kv heads x 4096 tokens at 256: 89-91 ->
 * 83 us).  Contexts are still cut off at max_num_partitions * partition_size tokens and no block-table entry beyond
 * that token is read; when the factor does not divide max_num_partitions this needs a workspace of
 * pa_decode_workspace_bytes (a limited copy of context_lens is kept there; without one the factor is the largest
 * divisor), and a sequence that IS cut off counts the causal offsets of its new tokens from the cut.
 */
#define PA_DECODE_FLAG_OUTPUT_ONLY 2

/* element types */
enum { PA_DTYPE_BF16 = 0, PA_DTYPE_FP8_E4M3FN = 1 };
/* quantisation modes, numbered as the reference numbers them
 * (pa_decode_triton_gluon_fp8.py:1753-1790): -1 no scale, 0 one f32 per tensor (read from
 * device memory), 1 one f32 per token and kv-head ([num_blocks, num_kv_heads, block_size, 1]) */
enum { PA_QUANT_NONE = -1, PA_QUANT_PER_TENSOR = 0, PA_QUANT_PER_TOKEN = 1 };

enum {
  PA_OK = 0,
  PA_ERR_NULL_POINTER = -1,   /* a required pointer is NULL */
  PA_ERR_BAD_STRUCT = -2,     /* struct_size does not match this library */
  PA_ERR_UNSUPPORTED = -3,    /* dtype / head size / block size / group size not supported */
  PA_ERR_BAD_SHAPE = -4,      /* non-positive size, bad partition size, stride the kernels cannot take */
  PA_ERR_LAUNCH = -5,         /* the HIP runtime refused the launch (see pa_decode_last_hip_error) */
  PA_ERR_NO_DEVICE = -6,
  PA_ERR_SCRATCH_TOO_SMALL = -7 /* pa_decode_noalloc: the call's buffers exceed PA_DECODE_NOALLOC_SCRATCH_BYTES */
};

/*
 * Arguments of one decode call.  Shapes (B = num_seqs, Hkv = num_kv_heads, G = group_size
 * = query heads per kv head, q = q_len, Ge = q*G, D = head_size, bs = block_size,
 * P = max_num_partitions, x = 16 / sizeof(kv element)):
 *
 *   output        bf16 [B, Hkv*Ge, D]      row of (kv head h, new token t, head g) = h*Ge + t*G + g
 *   query         bf16 or fp8 [B, Hkv*Ge, D]   same row order
 *   key_cache     [num_blocks, Hkv, D/x, bs, x]
 *   value_cache   [num_blocks, Hkv, D, bs]           (v_transposed = 0)
 *                 [num_blocks, Hkv, bs/x, D, x]      (v_transposed = 1)
 *   context_lens  int32 [B]   tokens in the cache for each sequence, the q new ones included (0: the
 *                 sequence's output rows are written as zero)
 *   block_tables  int32 [B, >= ceil(ctx/bs)]
 *   q_lens        int32 [B] or NULL: per-sequence number of new tokens (1..q); rows t >= q_lens[b]
 *                 are padding and their output rows are written as zero
 *   exp_sums, max_logits   f32 [B, Hkv, P, Ge]
 *   tmp_output             bf16 [B, Hkv, P, Ge, D]
 *
 * Strides are in elements.  The innermost dimension of every tensor must be contiguous; for the
 * caches the two innermost ones ([bs, x] of K, [bs] of V, [D, x] of transposed V) must be dense.
 */
typedef struct PaDecodeArgs {
  uint32_t struct_size; /* = sizeof(PaDecodeArgs) */
  int32_t flags;         /* 0 or PA_DECODE_FLAG_* */

  void* output;
  const void* query;
  const void* key_cache;
  const void* value_cache;
  const int32_t* context_lens;
  const int32_t* block_tables;
  const int32_t* q_lens;      /* optional */
  const float* query_scale;   /* optional; per tensor: 1 value, per token: [B, Hkv*Ge, 1] */
  const float* key_scale;     /* optional */
  const float* value_scale;   /* optional */
  const float* alibi_slopes;  /* optional, alibi_slopes_len f32 values: one slope per packed query ROW, [Hkv*q*G] at
                                 h*Ge + t*G + g, as the reference kernels index it (pa_decode_triton_gluon_fp8.py:323-327,
                                 803-810: alibi_slopes_ptr + kv_head*QUERY_GROUP_SIZE + row), or one per query HEAD,
                                 [Hkv*G] at h*G + g, shared by the q new tokens of a head; the same array for q_len == 1 */
  const float* sinks;         /* optional, [Hkv*Ge]: attention-sink logit of every query row (natural-log domain) */
  float* exp_sums;
  float* max_logits;
  void* tmp_output;
  int32_t* workspace;         /* optional, workspace_bytes long; first 64 bytes zero on entry, left zero on return */

  int32_t num_seqs;
  int32_t num_kv_heads;
  int32_t group_size;          /* G */
  int32_t q_len;               /* q (the maximum over the batch when q_lens is given) */
  int32_t head_size;           /* D: 128 (the tuned kernels), or 64 / 256 (generic kernels: same results, about half the
                                  rate); anything else is PA_ERR_UNSUPPORTED */
  int32_t block_size;          /* 16, 64 or 1024 */
  int32_t max_num_partitions;  /* P: partition axis length of the three buffers; P * partition_size must cover the
                                  longest context_len (the caller's max_sequence_length sizes it): tokens beyond it
                                  are not attended to, whatever P is */
  int32_t partition_size;      /* tokens per partition, a multiple of 256 */
  int32_t query_dtype;         /* PA_DTYPE_* */
  int32_t kv_dtype;            /* PA_DTYPE_* */
  int32_t query_quant_mode;    /* PA_QUANT_* */
  int32_t kv_quant_mode;       /* PA_QUANT_* */
  int32_t v_transposed;
  int32_t alibi_slopes_len;    /* elements of alibi_slopes: num_kv_heads*q_len*group_size (per row) or
                                  num_kv_heads*group_size (per head); anything else is PA_ERR_BAD_SHAPE; ignored
                                  when alibi_slopes is NULL */
  int32_t reserved0;           /* 0 */
  float softmax_scale;

  int64_t stride_out_s, stride_out_h;
  int64_t stride_q_s, stride_q_h;
  int64_t stride_k_b, stride_k_h, stride_k_c;     /* block, kv head, 16-byte chunk row */
  int64_t stride_v_b, stride_v_h, stride_v_2;     /* block, kv head, dim 2 (D rows, or bs/x rows) */
  int64_t stride_bt_s;                            /* >= the number of entries of a row (rows do not overlap) */
  int64_t stride_es_s, stride_es_h, stride_es_p;  /* shared by exp_sums and max_logits */
  int64_t stride_tmp_s, stride_tmp_h, stride_tmp_p, stride_tmp_g;
  int64_t stride_qscale_s;                        /* per-token query scale: stride of dim 0 */
  int64_t stride_kvscale_b, stride_kvscale_h;     /* per-token kv scales: block, kv head */
  int64_t workspace_bytes;                        /* size of workspace (>= PA_DECODE_WORKSPACE_BYTES), 0 without one */
} PaDecodeArgs;

/* Library / ABI identification. */
int pa_decode_abi_version(void);
uint32_t pa_decode_args_size(void);
const char* pa_decode_error_string(int code);
/* hipError_t of the last failed launch on the calling thread (0 if none). */
int pa_decode_last_hip_error(void);
/* Workspace size that enables every launch mode for a batch of this shape (see PA_DECODE_WORKSPACE_BYTES):
 * 64 + 8 * num_seqs * max_num_partitions + 4 * num_seqs. */
int64_t pa_decode_workspace_bytes(int32_t num_seqs, int32_t max_num_partitions);

/*
 * Launch-time tuning layer; replaces the constants and the 15 lines of kernel selection in
 * pa_decode_triton_gluon_fp8.py:24,1492-1509,1563-1564.  Given the batch shape and the longest
 * context (the caller's max_sequence_length), returns the partition size (a multiple of 256) the partition kernel should use.
 * Pure host arithmetic; num_cus <= 0 means "ask the current device".
 */
int pa_decode_select_partition_size(int32_t num_seqs, int32_t num_kv_heads, int32_t rows_per_group,
                                    int32_t max_context_len, int32_t block_size, int32_t num_cus);
/*
 * The same with one more statistic of the context lengths, which every serving engine has on the host: their sum
 * (0 or less: unknown, every sequence is taken to be as long as the longest).  A batch whose tokens sit in a few
 * long sequences gets the smaller partitions that fill the GPU from those few.
 */
int pa_decode_select_partition_size_stats(int32_t num_seqs, int32_t num_kv_heads, int32_t rows_per_group,
                                          int32_t max_context_len, int64_t total_context_tokens, int32_t block_size,
                                          int32_t num_cus);

/*
 * Stage 1: for every (sequence, kv head, partition) gathers the partition's KV pages through
 * block_tables, computes softmax(scale * Q K^T + mask) V over the partition on MFMA and writes
 * max_logits (max of the scaled logits), exp_sums (un-normalised) and tmp_output (normalised).
 * Replaces paged_attention_decode_v2_gluon_fp8 / _large_block_fp8
 * (pa_decode_triton_gluon_fp8.py:514-1002, :27-501) and
 * _paged_attn_decode_v2_w_dot_kernel_reshape_noloop_qk (pa_decode_triton.py:26-224).
 * Partitions at or beyond ceil(context_len / partition_size) are not written.  When output is not NULL
 * and there are no sinks, the output rows of every sequence with context_len <= partition_size are
 * written here as well (their single partial is the result).
 */
int pa_decode_partition(const PaDecodeArgs* args, void* hip_stream);

/*
 * Stage 2: merges the first ceil(context_len / partition_size) partitions of every row into
 * output (every sequence, also those with one partition; attention sinks enter the denominator here).
 * Replaces paged_attention_decode_v2_reduce_kernel
 * (pa_decode_triton_gluon_fp8.py:1187-1333) and _paged_attn_decode_v2_w_dot_reduce_kernel
 * (pa_decode_triton.py:227-324).
 */
int pa_decode_reduce(const PaDecodeArgs* args, void* hip_stream);

/* Both stages back to back on one stream: the body of the reference's paged_attention_decode.  Stage 2
 * skips the sequences stage 1 has finished, and is not launched when max_num_partitions == 1 (no sinks), nor when
 * stage 1 runs in teams: for a small partition size on a batch that fits the GPU at once, one workgroup of four
 * waves covers a (sequence, kv head)'s whole partition axis, writes its partition-buffer entries as stage 1 does and
 * merges them into output itself (pa_decode_launch_info says "teams of 4 waves ... no reduce kernel"). */
int pa_decode(const PaDecodeArgs* args, void* hip_stream);

/*
 * What the launch layer would do with these arguments, as text: the partition kernel's instantiation, its grid
 * and where its workgroups take their items from, e.g.
 *   "pa_partition_kernel<fp8, bs16, 4 waves> x 512"
 *   "pa_partition_shared_kernel<fp8 per-token, bs16, 3 ring slots, 3 workgroups per CU> x 6512, sorted items".
 * With a non-NULL output the text is pa_decode's launch; with output == NULL it is pa_decode_partition's (which forms
 * no teams).  The choice is a function of the arguments and the device's CU count alone.  (The reference's counterpart is
 * the kernel selection in pa_decode_triton_gluon_fp8.py:1492-1509.)  Launches nothing.
 *
 * Limits of the two launch modes that need a workspace (beyond them the call is launched in plain order, with
 * the same results): the queued launch of ragged batches holds its item table in LDS and takes at most 2048
 * sequences; the sorted dispatch's planning kernel takes at most 4096.
 *
 * Environment: none of the library's behaviour depends on environment variables unless the process was started
 * with PA_DECODE_DEBUG=1, which enables the tuning switches PA_DECODE_WAVES, PA_DECODE_ROW_TILES, PA_DECODE_SPAN,
 * PA_DECODE_QUEUE, PA_DECODE_SHARED, PA_DECODE_SORTED, PA_DECODE_LDS_PAD, PA_DECODE_P_RESIDUAL, PA_DECODE_XCD,
 * PA_DECODE_TEAM and PA_DECODE_REPARTITION (read once, at the first launch).
 */
int pa_decode_launch_info(const PaDecodeArgs* args, char* text, int32_t text_bytes);

/*
 * pa_decode for callers that cannot allocate device memory and have no partition buffers to pass: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference (whose entry point allocates its three buffers with torch.zeros on every call,
 * pa_decode_triton_gluon_fp8.py:1726-1733).  args is filled as for pa_decode, except that exp_sums, max_logits,
 * tmp_output and workspace must be NULL and workspace_bytes 0 (the strides of the partition buffers are
 * ignored): the library places all four in a device array of PA_DECODE_NOALLOC_SCRATCH_BYTES that it holds on
 * every GPU it runs on until the process ends, and calls no hipMalloc, hipFree or other allocating routine.
 * Bytes needed, each term rounded up to a multiple of 256, with n = num_seqs * num_kv_heads *
 * max_num_partitions * q_len * group_size:
 *     pa_decode_workspace_bytes(num_seqs, max_num_partitions) + 4 n + 4 n + 2 n * head_size;
 * a call that needs more returns PA_ERR_SCRATCH_TOO_SMALL and launches nothing (choose a larger partition_size,
 * as pa_decode_select_partition_size does, or use pa_decode with buffers of your own).  The partition buffers
 * are not handed back.  All calls on one GPU share that GPU's array: calls that may overlap on the GPU (two
 * streams, two threads) race; calls on one stream, or ordered by events, do not.  The array keeps the last
 * call's contents; the call clears the counters it needs zero with a small kernel (no memset node, so it can be
 * captured into a graph) and ignores PA_DECODE_FLAG_REUSE_ITEM_LIST.
 */
#define PA_DECODE_NOALLOC_SCRATCH_BYTES (64u << 20)
int pa_decode_noalloc(const PaDecodeArgs* args, void* hip_stream);

/*
 * KV-cache write: the step before the decode path.  Writes num_tokens new (key, value) rows
 * [num_tokens, Hkv, D] (bf16) into the paged caches at slot_mapping[t] = block * block_size + offset
 * (negative = skip), in the layouts the decode kernels read.  With an FP8 cache the rows are
 * quantised on the way: per token and kv head (scale = amax / 448 written to the scale tensors), per
 * tensor (the given scales are read), or cast as they are.  The reference has this step only as an
 * offline whole-cache routine, quantize_kv_cache_symmetric (test_pa_mtp.py:294-369, over
 * aiter.pertoken_quant), which pa_quantize_kv_cache below replaces directly.
 * Calls with 2048 tokens or more whose rows, caches and strides are 16-byte aligned (and block_size a
 * multiple of 16) are written in runs of up to 16 tokens that land in consecutive slots; any slot_mapping is
 * valid (runs are found on the device), the bytes written are the same either way.
 */
typedef struct PaKvWriteArgs {
  uint32_t struct_size; /* = sizeof(PaKvWriteArgs) */
  int32_t reserved0;
  const void* key;             /* bf16 [num_tokens, Hkv, D] */
  const void* value;           /* bf16 [num_tokens, Hkv, D] */
  const int64_t* slot_mapping; /* [num_tokens] */
  void* key_cache;             /* [blocks, Hkv, D/x, bs, x] */
  void* value_cache;           /* [blocks, Hkv, D, bs], or [blocks, Hkv, bs/x, D, x] with v_transposed */
  float* key_scale;            /* per token: [blocks, Hkv, bs, 1] written; per tensor: 1 value read */
  float* value_scale;
  int64_t num_tokens;
  int32_t num_kv_heads;
  int32_t head_size;           /* 128; 64 and 256 are written token by token whatever num_tokens is */
  int32_t block_size;
  int32_t cache_dtype;         /* PA_DTYPE_* */
  int32_t kv_quant_mode;       /* PA_QUANT_* */
  int32_t v_transposed;        /* 0: value_cache [.., D, bs]; 1: [.., bs/x, D, x] (shuffle_value_cache_layout, test_pa_mtp.py:472-497) */
  int64_t stride_k_t, stride_k_h, stride_v_t, stride_v_h; /* elements; last dim contiguous */
  int64_t stride_kc_b, stride_kc_h, stride_vc_b, stride_vc_h; /* cache block / head strides; inner dims dense */
  int64_t stride_scale_b, stride_scale_h;
} PaKvWriteArgs;

int pa_kv_cache_write(const PaKvWriteArgs* args, void* hip_stream);

/*
 * Whole-cache per-token FP8 quantisation of a dense bf16 cache (x = 8) into a dense FP8 cache (x = 16)
 * plus scales [num_blocks, Hkv, block_size, 1]: quantize_kv_cache_symmetric (test_pa_mtp.py:294-369).
 */
int pa_quantize_kv_cache(const void* key_cache_bf16, const void* value_cache_bf16, void* key_cache_fp8,
                         void* value_cache_fp8, float* key_scale, float* value_scale, int64_t num_blocks,
                         int32_t num_kv_heads, int32_t head_size, int32_t block_size, void* hip_stream);

/*
 * Test hook: decodes n FP8 e4m3fn bytes (device pointer) to f32 (device pointer) with the same
 * conversion instructions the partition kernel uses, so the dequantisation table can be compared
 * with the format definition code by code.
 */
int pa_debug_fp8_decode(const uint8_t* codes, float* out, int32_t n, void* hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* PA_DECODE_H_ */
