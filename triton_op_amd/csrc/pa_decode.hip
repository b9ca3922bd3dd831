// Split-KV paged-attention decode for MI355X (gfx950 / CDNA4): the two partition kernels, the reduce
// kernel and the C ABI declared in include/pa_decode.h.
//
// pa_partition_kernel (up to 16 query rows per kv head, and every bf16 cache) and pa_partition_shared_kernel
// (17..64 rows over an FP8 cache: the same arithmetic with the row tiles of a kv head sharing one pass over the
// pages through LDS) are stage 1, pa_reduce_kernel is stage 2.
//
// This file holds the host side: argument checks, the launch / tuning layer and the extern "C" entry points.
// The kernels live in pa_partition_kernel.h, pa_partition_shared_kernel.h and pa_reduce_kernel.h.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>

#include "../../include/pa_decode.h"
#include "pa_common.h"
#include "pa_launch.h"
#include "pa_partition_kernel.h"
#include "pa_partition_shared_kernel.h"
#include "pa_generic_kernel.h"
#include "pa_plan_kernel.h"
#include "pa_reduce_kernel.h"

// Scratch of pa_decode_noalloc, the entry point for callers that can neither allocate nor pass partition buffers:
// the item-list workspace and the three partition buffers of one call.  Every GPU the library runs on holds its
// own copy at its own address; host code reaches it only through the address hipGetSymbolAddress returns there.
static __device__ __align__(256) unsigned char scratch[PA_DECODE_NOALLOC_SCRATCH_BYTES];

thread_local int pa_last_hip_error = 0;

namespace {

// context lengths with a limit applied (the end of a caller's partition axis)
__global__ void pa_limit_lens_kernel(const int32_t* lens, int32_t* out, int n, int limit) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = lens[i] < limit ? lens[i] : limit;
}

// the first `n` int32 words at p become zero (a launch, not a memset node: callers may be capturing a graph)
__global__ void pa_clear_words_kernel(int32_t* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

__global__ void pa_fp8_decode_kernel(const uint8_t* codes, float* out, int n) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  // same path as the partition kernel: byte -> bf16 bit pattern -> f32
  uint32_t w = (uint32_t)codes[i] | ((uint32_t)codes[i] << 16);
  uint32_t lo = fp8x2_to_bf16x2(w, false);
  uint32_t hi = fp8x2_to_bf16x2(w, true);
  float a = bf16_bits_to_f32(lo & 0xffffu);
  float b = bf16_bits_to_f32(hi & 0xffffu);
  out[i] = (i & 1) ? b : a;
}

int check_common(const PaDecodeArgs* a) {
  if (!a) return PA_ERR_NULL_POINTER;
  if (a->struct_size != sizeof(PaDecodeArgs)) return PA_ERR_BAD_STRUCT;
  if (!a->context_lens || !a->exp_sums || !a->max_logits || !a->tmp_output) return PA_ERR_NULL_POINTER;
  if (a->num_seqs <= 0 || a->num_kv_heads <= 0 || a->group_size <= 0 || a->q_len <= 0 ||
      a->max_num_partitions <= 0)
    return PA_ERR_BAD_SHAPE;
  if (a->partition_size <= 0 || a->partition_size % 256) return PA_ERR_BAD_SHAPE;
  if (a->flags & ~(PA_DECODE_FLAG_REUSE_ITEM_LIST | PA_DECODE_FLAG_OUTPUT_ONLY)) return PA_ERR_BAD_SHAPE;
  if (a->workspace ? a->workspace_bytes < PA_DECODE_WORKSPACE_BYTES : a->workspace_bytes != 0) return PA_ERR_BAD_SHAPE;
  if (a->head_size != kHeadSize && a->head_size != 64 && a->head_size != 256) return PA_ERR_UNSUPPORTED;
  if (a->q_len * a->group_size > 64) return PA_ERR_UNSUPPORTED;  // the reference's limit
  return PA_OK;
}

int device_num_cus() {
  static const int n = [] {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 256;
    return prop.multiProcessorCount;
  }();
  return n;
}

// Experiment switches.  They exist for tuning runs only and are dead unless the process was started with
// PA_DECODE_DEBUG=1, so a serving process's launches never depend on stray environment variables:
//   PA_DECODE_WAVES=n    waves per workgroup of pa_partition_kernel
//   PA_DECODE_ROW_TILES=1  a bf16 cache with more than 16 query rows per kv head: one workgroup per 16-row tile
//   PA_DECODE_QUEUE=0    no queued launch          PA_DECODE_SHARED=0   one workgroup per 16-row tile, always
//   PA_DECODE_SORTED=0|1 never / always the sorted dispatch (when the workspace has room)
//   PA_DECODE_LDS_PAD=n  unused LDS per workgroup of the shared-stream kernel (lowers its occupancy)
//   PA_DECODE_P_RESIDUAL=0  shared-stream kernel: P without its FP8 residual (every element rounded to e4m3)
//   PA_DECODE_XCD=0         shared-stream kernel: the kv head fastest in the workgroup id (heads spread over the XCDs)
// All are read once, at the first launch.
int debug_switch(const char* name, int unset) {
  static const bool enabled = [] {
    const char* e = getenv("PA_DECODE_DEBUG");
    return e && e[0] == '1';
  }();
  if (!enabled) return unset;
  const char* e = getenv(name);
  return e ? atoi(e) : unset;
}

// Bytes of workspace the sorted dispatch needs: the header and one (sequence, partition) pair per possible item.
long long plan_workspace_bytes(int num_seqs, int max_num_partitions) {
  return 4LL * kPlanHeaderWords + 8LL * num_seqs * max_num_partitions;
}
// ... and one more word per sequence for the list of the sequences with more than one partition
long long full_workspace_bytes(int num_seqs, int max_num_partitions) {
  return plan_workspace_bytes(num_seqs, max_num_partitions) + 4LL * num_seqs;
}

// pa_partition_kernel, waves per workgroup: 128 tokens (2 steps) per wave at least, and at most 4 waves (the
// merge buffer of a workgroup is WAVES * 8 KiB of LDS).  Eight waves (one partition where four waves take two)
// were measured and lose: a wave's chain of 1.4 us steps is what a small batch waits for, and more partitions
// shorten it where more waves per workgroup cannot go below the second kernel's cost anyway.
int waves_for_partition_size(int partition_size) { return partition_size >= 512 ? 4 : 2; }

// More than one 16-row query tile per kv head over an FP8 cache: the tiles share one pass over the pages
// (pa_partition_shared_kernel).
bool use_shared_stream(int kv_dtype, int rows_per_group) {
  static const bool off = debug_switch("PA_DECODE_SHARED", 1) == 0;
  return !off && kv_dtype == PA_DTYPE_FP8_E4M3FN && rows_per_group > 16;
}

// Everything the launch layer decides for one call, from the arguments alone (pure host arithmetic): which
// partition kernel in which instantiation, how many workgroups, and how they get their items.
struct LaunchChoice {
  bool shared;      // pa_partition_shared_kernel (else pa_partition_kernel, one workgroup per 16-row tile)
  bool fp8;         // FP8 cache (else bf16)
  bool per_token;   // per-token kv scales
  bool bs16;        // constant in-page strides: block size 16 with the default dense layout
  int waves;        // waves per workgroup
  int row_tiles;    // pa_partition_kernel: 16-row query tiles one workgroup computes in its pass over the pages (1 or 2)
  int per_cu;       // workgroups of this instantiation that fit a CU
  int span;         // consecutive partitions a one-wave workgroup walks in one pass (1: one partition per workgroup)
  bool team;        // four one-wave span walkers per workgroup cover a sequence's whole partition axis and merge it themselves
  bool queue;       // a resident grid pulls live items from a counter in the workspace
  bool sorted;      // items come from the planning kernel's list in the workspace
  bool listed_reduce;  // ... and pa_decode's reduce stage walks the planning kernel's list of multi-partition sequences
  bool heads_share_xcd;  // pa_partition_shared_kernel: an item's kv heads are consecutive workgroups of one XCD
  long long blocks; // workgroups launched
};

// `fused`: the call is pa_decode's (both stages, `output` is written): the partition kernel may finish sequences of
// several partitions itself
LaunchChoice choose_launch(const PaDecodeArgs& a, bool fused) {
  LaunchChoice c{};
  const int ge = a.q_len * a.group_size;
  c.fp8 = a.kv_dtype == PA_DTYPE_FP8_E4M3FN;
  c.per_token = a.kv_quant_mode == PA_QUANT_PER_TOKEN;
  c.bs16 = c.fp8 && a.block_size == 16 && a.stride_k_c == 256 &&
           (a.v_transposed ? a.stride_v_2 == 2048 : a.stride_v_2 == 16);
  c.shared = use_shared_stream(a.kv_dtype, ge);
  static const bool xcd_off = debug_switch("PA_DECODE_XCD", 1) == 0;
  long long items;  // (sequence, partition) pairs times kv heads times row tiles
  c.row_tiles = 1;
  if (c.shared) {
    // ring depth / waves per SIMD: without per-token scales the kernel fits 128 registers, and a fourth
    // workgroup per CU is worth more than a deeper ring (measured); with them it needs about 140
    c.waves = 4;
    c.per_cu = c.per_token ? 3 : 4;
    // Per-token scales: an XCD takes every eighth (sequence, partition) item with all its kv heads (the heads' scales of a
    // page share 128-byte lines, which then meet in one L2; measured on the ragged 64-row mix: 341 -> 336 us, uniform
    // batches 1 %); the grid is whole groups of eight items.  PA_DECODE_XCD=0: the head fastest in the workgroup id.
    c.heads_share_xcd = c.per_token && !xcd_off;
    items = (long long)a.num_seqs * a.max_num_partitions;
    if (c.heads_share_xcd) items = (items + 7) / 8 * 8;
    items *= a.num_kv_heads;
  } else {
    // no more waves than it takes to fill the GPU's wave slots (8 per CU): with 8 workgroups or more per CU one
    // wave each is best (no merge, more independent streams: 256 sequences x 8 kv heads x 512 tokens 57.7 ->
    // 44.8 us), with 4 per CU two.  But a wave keeps at most 16 steps (1024 tokens) to itself, or the longest
    // items of a ragged batch finish the launch alone, one slow wave each (256 sequences of 1..4096 tokens:
    // 196 us with one wave per workgroup against 179 us with four).
    static const int forced = debug_switch("PA_DECODE_WAVES", 0);
    // A bf16 cache with more than 16 query rows per kv head: two row tiles per workgroup share one pass over the
    // pages (one wave per SIMD then, with twice the accumulators); an FP8 cache has the shared-stream kernel.
    static const int forced_tiles = debug_switch("PA_DECODE_ROW_TILES", 0);
    c.row_tiles = !c.fp8 && ge > 16 && forced_tiles != 1 ? 2 : 1;
    items = (long long)a.num_seqs * a.num_kv_heads * a.max_num_partitions * ((ge + 16 * c.row_tiles - 1) / (16 * c.row_tiles));
    int w = waves_for_partition_size(a.partition_size);
    if (forced > 0) {
      w = forced;
    } else {
      const long long slots = (c.row_tiles == 2 ? 4LL : 8LL) * device_num_cus();
      int need = 1;  // waves per workgroup that fill the slots, or keep a wave's share at 1024 tokens
      while (need < w && (items * need < slots || a.partition_size > 1024 * need)) need *= 2;
      w = need;
    }
    c.waves = w >= 4 ? 4 : (w >= 2 ? 2 : 1);
    c.per_cu = (c.row_tiles == 2 ? 4 : 8) / c.waves;
  }
  c.blocks = items;
  // The queued launch is used when the caller gave a workspace and per-sequence query lengths and a kv head has
  // more than one 16-row query tile (tiles of padding rows only are then common): a resident grid pulls live
  // items from a counter.  Otherwise the only workgroups with nothing to do are partitions past a sequence's
  // end, which the plain launch orders last; there the queue's bookkeeping costs more than it saves (measured:
  // +10 % on a uniform batch).  Batches of more than kQueueMaxSeqs sequences (the item table in LDS) are
  // launched plainly.
  static const bool queue_off = debug_switch("PA_DECODE_QUEUE", 1) == 0;
  c.queue = !c.shared && !queue_off && a.workspace != nullptr && a.num_seqs <= kQueueMaxSeqs && a.q_lens != nullptr &&
            ge > 16 * c.row_tiles;
  if (c.queue) {
    const long long resident = (long long)device_num_cus() * c.per_cu;
    c.blocks = resident < items ? resident : items;
  }
  // One-wave workgroups in several rounds (a caller whose buffers fix a small partition size, the reference's 256):
  // each workgroup walks `span` consecutive partitions in one pass over the pages and writes a partial result per
  // partition, so the query set-up and the ramp of the page stream are paid once per span.  As many partitions
  // as still leave a workgroup for every wave slot, no wave with more than 2048 tokens, and at most four (the
  // partial results wait in LDS for the end of the pass).
  c.span = 1;
  static const int forced_span = debug_switch("PA_DECODE_SPAN", 0);  // 1 switches it off
  if (!c.shared && !c.queue && c.waves == 1 && a.max_num_partitions > 1) {
    const long long slots = (c.row_tiles == 2 ? 4LL : 8LL) * device_num_cus();
    long long span = items / slots;
    const long long cap = 2048 / a.partition_size;
    span = span > cap ? cap : span;
    // (measured, kernel + reduce, against one partition per workgroup: 64 sequences x 8 kv heads x 4096 tokens at
    // 256: 110 -> 95 us; 4 x 8 x 131072 at 256: 235 -> 223 us; 256 x 8 x 2048 at 512: 200 -> 180 us; 512 x 8 x 4096
    // at 256, eight rounds: 829 -> 808 us; pages of 1024 tokens, 128 x 8 x 16384, at 512: 847 -> 832 us, but at
    // 256: 920 -> 936 us, so not there)
    if (a.block_size > 64 && a.partition_size < 512) span = 1;
    if (forced_span > 0) span = forced_span;
    span = span > a.max_num_partitions ? a.max_num_partitions : span;
    // (a tile of up to 8 real rows stages half the bytes per partition and may walk twice as many)
    const long long span_max = c.row_tiles == 1 && ge <= 8 ? kSpanMaxFewRows : kSpanMax;
    span = span > span_max ? span_max : span;
    // A TEAM: when four such walkers cover the whole partition axis they share a workgroup, which then holds every
    // partial result of its (sequence, kv head, row tile) in LDS and merges them into `output` itself: no second
    // kernel.  Only when every team is resident at once (two per CU) and the teams' waves fill three quarters of the
    // wave slots or more: in a second round a team's waves would each have half the work of the one-wave workgroups
    // that fill the slots in one (measured, 128 sequences x 8 kv heads x 1024 tokens at 256: 53.1 against 52.3 us;
    // ragged, up to 8192 tokens: 198 against 183 us), and fewer teams lose to more, shorter workgroups (40 sequences x
    // 8 x 4096 at 256: 70.3 against 67.8 us).  Measured, call against call with the reduce kernel: 64 x 8 x 4096 at
    // 256: 93.2 -> 89.1 us; per-token scales, 56 sequences: 96.2 -> 84.3; 16 rows: 100.6 -> 95.9; 48 sequences: 75.6 ->
    // 73.5; ragged, up to 4096 tokens: 67.3 -> 65.0; 64 x 8 x 1024: 29.4 -> 28.0; 64 x 8 x 7000: 157.7 -> 157.1.
    // PA_DECODE_TEAM=0: never.
    static const bool team_off = debug_switch("PA_DECODE_TEAM", 1) == 0;
    const long long team_span = (a.max_num_partitions + kTeamWaves - 1) / kTeamWaves;
    const long long teams = items / a.max_num_partitions;
    if (fused && !team_off && c.fp8 && c.row_tiles == 1 && !a.sinks && a.output != nullptr && team_span <= span_max &&
        team_span * a.partition_size <= 2048 && !(a.block_size > 64 && a.partition_size < 512 && team_span > 1) &&
        forced_span != 1 && teams * kTeamWaves <= slots && teams * kTeamWaves * 4 >= slots * 3)
    {
      c.team = true;
      c.span = (int)team_span;
      c.per_cu = 2;
      items = teams;
      c.blocks = items;
    } else if (span >= 2) {
      c.span = (int)span;
      const long long coarse = (a.max_num_partitions + span - 1) / span;
      items = items / a.max_num_partitions * coarse;
      c.blocks = items;
    }
  }
  // The sorted dispatch pays a small extra kernel, and ordering only matters when workgroups are handed out in
  // several rounds: it is used when the launch has more than twice as many workgroups as the GPU holds at once
  // and the caller's workspace has room for the list (batches of more than kPlanMaxSeqs sequences, the planning
  // kernel's LDS tables, are launched in plain order).
  static const int sorted_mode = debug_switch("PA_DECODE_SORTED", -1);
  c.sorted = !c.queue && !c.team && sorted_mode != 0 && a.workspace != nullptr && a.num_seqs <= kPlanMaxSeqs &&
             a.workspace_bytes >= plan_workspace_bytes(a.num_seqs, a.max_num_partitions) &&
             (sorted_mode == 1 || items > 2LL * device_num_cus() * c.per_cu);
  // (with several partitions per workgroup the planning kernel lists those coarser items, and its list of the
  // sequences with more than one of them is not the list of the sequences the reduce stage has to merge)
  c.listed_reduce = c.sorted && c.span == 1 && !a.sinks &&
                    a.workspace_bytes >= full_workspace_bytes(a.num_seqs, a.max_num_partitions);
  // pa_partition_kernel with per-token scales: the same placement of an item's heads (and row tiles) on one XCD
  if (!c.shared && !c.queue && c.fp8 && c.per_token && !xcd_off) {
    c.heads_share_xcd = true;
    const long long units = (long long)a.num_kv_heads * ((ge + 16 * c.row_tiles - 1) / (16 * c.row_tiles));
    c.blocks = (items / units + 7) / 8 * 8 * units;  // whole groups of eight (sequence, partition) items
  }
  return c;
}

int launch_plan(const PaDecodeArgs& a, hipStream_t stream) {
  return pa_launch(pa_plan_kernel, dim3(1), dim3(1024), 0, stream, a);
}

// pa_partition_kernel is instantiated with one 16-row query tile per workgroup (NT = 1): a bf16 cache with
// more than 16 query rows per kv head gets one workgroup per tile (they read the same pages at the same time
// from the same L2, and tiles that hold only padding rows cost nothing).
template <int NT, int KVT, bool PT, bool BS16, int W>
int launch_partition_w(const PaDecodeArgs& k, const LaunchChoice& c, hipStream_t stream) {
  constexpr int OCC = NT == 1 ? 2 : 1;
  const dim3 grid((unsigned)c.blocks), block(64 * W);
  if constexpr (NT == 2) {
    // more rows per kv head than one workgroup's two tiles: another workgroup reads the same pages (see REREAD)
    if (k.q_len * k.group_size > 32)
      return c.queue ? pa_launch(pa_partition_kernel<NT, KVT, PT, BS16, W, OCC, true, true>, grid, block, 0, stream, k)
                     : pa_launch(pa_partition_kernel<NT, KVT, PT, BS16, W, OCC, false, true>, grid, block, 0, stream, k);
  }
  if constexpr (NT == 1 && W == 1 && KVT == PA_DTYPE_FP8_E4M3FN) {
    if (c.team)
      return pa_launch(pa_partition_kernel<1, KVT, PT, BS16, 1, OCC, false, false, true>, grid, dim3(64 * kTeamWaves), 0, stream, k);
  }
  if (c.queue) return pa_launch(pa_partition_kernel<NT, KVT, PT, BS16, W, OCC, true>, grid, block, 0, stream, k);
  return pa_launch(pa_partition_kernel<NT, KVT, PT, BS16, W, OCC, false>, grid, block, 0, stream, k);
}

template <int NT, int KVT, bool PT, bool BS16>
int launch_partition_tile(const PaDecodeArgs& k, const LaunchChoice& c, hipStream_t stream) {
  if (c.waves == 4) return launch_partition_w<NT, KVT, PT, BS16, 4>(k, c, stream);
  if (c.waves == 2) return launch_partition_w<NT, KVT, PT, BS16, 2>(k, c, stream);
  return launch_partition_w<NT, KVT, PT, BS16, 1>(k, c, stream);
}

template <bool PT, bool BS16>
int launch_partition_shared(const PaDecodeArgs& a, const LaunchChoice& c, hipStream_t stream) {
  static const int pad = debug_switch("PA_DECODE_LDS_PAD", 0);  // experiment: unused LDS that lowers the occupancy
  const PaDecodeArgs& k = a;
  if constexpr (PT)
    return pa_launch(pa_partition_shared_kernel<true, BS16, 3, 3>, dim3((unsigned)c.blocks), dim3(256), (unsigned)pad, stream, k);
  else
    return pa_launch(pa_partition_shared_kernel<false, BS16, 2, 4>, dim3((unsigned)c.blocks), dim3(256), (unsigned)pad, stream, k);
}

int check_reduce(const PaDecodeArgs* a);

// Head sizes other than 128 (64 and 256) run on the two generic kernels (pa_generic_kernel.h): plain order, one wave
// per (sequence, partition, kv head, 16-row tile), and a merge that always runs.
bool generic_head_size(const PaDecodeArgs& a) { return a.head_size != kHeadSize; }

long long generic_partition_blocks(const PaDecodeArgs& a) {
  return (long long)a.num_seqs * a.max_num_partitions * a.num_kv_heads * ((a.q_len * a.group_size + 15) / 16);
}

int launch_partition_generic(const PaDecodeArgs& a, hipStream_t stream) {
  const long long blocks = generic_partition_blocks(a);
  if (blocks > 0x7fffffffLL) return PA_ERR_BAD_SHAPE;
  PaDecodeArgs k = a;
  k.flags = (a.flags & PA_DECODE_FLAG_OUTPUT_ONLY) ? kFlagOutputOnly : 0;
  const dim3 grid((unsigned)blocks), block(64);
  const bool fp8 = a.kv_dtype == PA_DTYPE_FP8_E4M3FN;
  if (a.head_size == 64)
    return fp8 ? pa_launch(pa_partition_generic_kernel<64, true>, grid, block, 0, stream, k)
               : pa_launch(pa_partition_generic_kernel<64, false>, grid, block, 0, stream, k);
  return fp8 ? pa_launch(pa_partition_generic_kernel<256, true>, grid, block, 0, stream, k)
             : pa_launch(pa_partition_generic_kernel<256, false>, grid, block, 0, stream, k);
}

int launch_reduce_generic(const PaDecodeArgs* a, void* hip_stream) {
  const int rc = check_reduce(a);
  if (rc) return rc;
  const long long blocks = (long long)a->num_seqs * a->num_kv_heads * a->q_len * a->group_size;
  if (blocks > 0x7fffffffLL) return PA_ERR_BAD_SHAPE;
  hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
  if (a->head_size == 64) return pa_launch(pa_reduce_generic_kernel<64>, dim3((unsigned)blocks), dim3(64), 0, stream, *a);
  return pa_launch(pa_reduce_generic_kernel<256>, dim3((unsigned)blocks), dim3(64), 0, stream, *a);
}

// stage 1 as chosen: the planning kernel when the items are to be sorted, then the partition kernel
int launch_partition(const PaDecodeArgs& a, const LaunchChoice& c, hipStream_t stream) {
  if (c.blocks > 0x7fffffffLL) return PA_ERR_BAD_SHAPE;
  PaDecodeArgs k = a;
  k.flags = 0;
  if (c.sorted) {
    if (!(a.flags & PA_DECODE_FLAG_REUSE_ITEM_LIST)) {
      PaDecodeArgs items = a;  // what the planning kernel lists: a workgroup's `span` partitions are one item
      items.partition_size = a.partition_size * c.span;
      items.max_num_partitions = (a.max_num_partitions + c.span - 1) / c.span;
      const int rc = launch_plan(items, stream);
      if (rc) return rc;
    }
    k.flags = kFlagSortedItems;
  }
  if (c.span > 1) k.flags |= c.span << kFlagSpanShift;
  if (c.heads_share_xcd) k.flags |= kFlagHeadsShareXcd;
  if (a.flags & PA_DECODE_FLAG_OUTPUT_ONLY) k.flags |= kFlagOutputOnly;
  // experiment (PA_DECODE_DEBUG=1): PA_DECODE_P_RESIDUAL=0 drops the FP8 residual of P in the shared-stream kernel
  // (every P rounded to e4m3, as the reference's kernel rounds it)
  static const int p_residual = debug_switch("PA_DECODE_P_RESIDUAL", 1);
  if (p_residual == 0) k.flags |= kFlagResidualNever;
  if (!c.fp8) {
    if (c.row_tiles == 2) return launch_partition_tile<2, PA_DTYPE_BF16, false, false>(k, c, stream);
    return launch_partition_tile<1, PA_DTYPE_BF16, false, false>(k, c, stream);
  }
  if (c.shared) {
    if (c.bs16)
      return c.per_token ? launch_partition_shared<true, true>(k, c, stream) : launch_partition_shared<false, true>(k, c, stream);
    return c.per_token ? launch_partition_shared<true, false>(k, c, stream) : launch_partition_shared<false, false>(k, c, stream);
  }
  if (c.bs16)
    return c.per_token ? launch_partition_tile<1, PA_DTYPE_FP8_E4M3FN, true, true>(k, c, stream)
                       : launch_partition_tile<1, PA_DTYPE_FP8_E4M3FN, false, true>(k, c, stream);
  return c.per_token ? launch_partition_tile<1, PA_DTYPE_FP8_E4M3FN, true, false>(k, c, stream)
                     : launch_partition_tile<1, PA_DTYPE_FP8_E4M3FN, false, false>(k, c, stream);
}

// the argument checks of stage 1
int check_partition(const PaDecodeArgs* a) {
  int rc = check_common(a);
  if (rc) return rc;
  if (!a->query || !a->key_cache || !a->value_cache || !a->block_tables) return PA_ERR_NULL_POINTER;
  // a sequence's block-table row is at least one entry long and rows do not overlap (the kernels request a row's
  // first entries before they know how many of them the sequence uses, and keep the index inside the row's stride)
  if (a->stride_bt_s < 1 || a->stride_bt_s > 0x7fffffffLL) return PA_ERR_BAD_SHAPE;
  if (a->block_size != 16 && a->block_size != 64 && a->block_size != 1024) return PA_ERR_UNSUPPORTED;
  if (a->kv_dtype != PA_DTYPE_BF16 && a->kv_dtype != PA_DTYPE_FP8_E4M3FN) return PA_ERR_UNSUPPORTED;
  if (a->query_dtype != PA_DTYPE_BF16 && a->query_dtype != PA_DTYPE_FP8_E4M3FN) return PA_ERR_UNSUPPORTED;
  if (a->kv_quant_mode != PA_QUANT_NONE && (!a->key_scale || !a->value_scale)) return PA_ERR_NULL_POINTER;
  if (a->query_quant_mode != PA_QUANT_NONE && !a->query_scale) return PA_ERR_NULL_POINTER;
  if (a->kv_quant_mode < -1 || a->kv_quant_mode > 1 || a->query_quant_mode < -1 || a->query_quant_mode > 1)
    return PA_ERR_UNSUPPORTED;
  if (a->kv_quant_mode == PA_QUANT_PER_TOKEN && a->kv_dtype != PA_DTYPE_FP8_E4M3FN)
    return PA_ERR_UNSUPPORTED;  // per-token scales belong to the FP8 cache
  // ALiBi: one slope per packed query row (the reference kernels' array) or one per query head
  if (a->alibi_slopes && a->alibi_slopes_len != a->num_kv_heads * a->q_len * a->group_size &&
      a->alibi_slopes_len != a->num_kv_heads * a->group_size)
    return PA_ERR_BAD_SHAPE;
  const int esz = a->kv_dtype == PA_DTYPE_FP8_E4M3FN ? 1 : 2;
  // 16-byte vector loads: every stride that moves a vector must keep it 16-byte aligned
  if ((a->stride_k_b * esz) % 16 || (a->stride_k_h * esz) % 16 || (a->stride_k_c * esz) % 16 ||
      (a->stride_v_b * esz) % 16 || (a->stride_v_h * esz) % 16 || (a->stride_v_2 * esz) % 16)
    return PA_ERR_BAD_SHAPE;
  const int qsz = a->query_dtype == PA_DTYPE_FP8_E4M3FN ? 1 : 2;
  if ((a->stride_q_s * qsz) % 16 || (a->stride_q_h * qsz) % 16) return PA_ERR_BAD_SHAPE;
  if ((a->stride_tmp_g * 2) % 16 || (a->stride_tmp_p * 2) % 16 || (a->stride_tmp_h * 2) % 16 || (a->stride_tmp_s * 2) % 16 ||
      (reinterpret_cast<uintptr_t>(a->tmp_output) & 15))
    return PA_ERR_BAD_SHAPE;
  if (a->kv_quant_mode == PA_QUANT_PER_TOKEN && (a->stride_kvscale_b % 4 || a->stride_kvscale_h % 4))
    return PA_ERR_BAD_SHAPE;
  if ((long long)(4 * 3 + 3) * a->stride_k_c * esz + 15 * 16 >= (1LL << 32)) return PA_ERR_BAD_SHAPE;
  if ((reinterpret_cast<uintptr_t>(a->key_cache) | reinterpret_cast<uintptr_t>(a->value_cache) |
       reinterpret_cast<uintptr_t>(a->query)) & 15)
    return PA_ERR_BAD_SHAPE;
  return PA_OK;
}

// ... and of stage 2
int check_reduce(const PaDecodeArgs* a) {
  int rc = check_common(a);
  if (rc) return rc;
  if (!a->output) return PA_ERR_NULL_POINTER;
  if (a->stride_out_h % 2 || a->stride_out_s % 2 || a->stride_tmp_g % 2 || a->stride_tmp_p % 2 ||
      a->stride_tmp_h % 2 || a->stride_tmp_s % 2)
    return PA_ERR_BAD_SHAPE;
  return PA_OK;
}

int launch_reduce(const PaDecodeArgs* a, void* hip_stream, bool skip_single) {
  int rc = check_reduce(a);
  if (rc) return rc;
  const long long blocks = (long long)a->num_seqs * a->num_kv_heads * ((a->q_len * a->group_size + 15) / 16);
  if (blocks > 0x7fffffffLL) return PA_ERR_BAD_SHAPE;
  hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
  // enough rows to fill the GPU's wave slots several times over: four rows per wave
  const bool big = blocks * 16 >= 16384;
  const dim3 grid((unsigned)blocks);
  // Few 16-row units, many partitions each (a caller-fixed small partition size on a handful of long sequences): a
  // unit is cut along the head dimension into several workgroups, whose waves split the partition axis.  Needs
  // 16-byte aligned rows of tmp_output.
  if (blocks <= 2LL * device_num_cus() && a->max_num_partitions >= 64 && (a->stride_tmp_g * 2) % 16 == 0 &&
      (a->stride_tmp_p * 2) % 16 == 0 && (a->stride_tmp_h * 2) % 16 == 0 && (a->stride_tmp_s * 2) % 16 == 0 &&
      (reinterpret_cast<uintptr_t>(a->tmp_output) & 15) == 0)
  {
    const dim3 wide((unsigned)((blocks + 7) / 8 * 8 * kWideDimSplit));  // (whole groups of eight units: see the kernel)
    return skip_single ? pa_launch(pa_reduce_wide_kernel<true>, wide, dim3(64 * kWideWaves), 0, stream, *a)
                       : pa_launch(pa_reduce_wide_kernel<false>, wide, dim3(64 * kWideWaves), 0, stream, *a);
  }
  if (skip_single)
    return big ? pa_launch(pa_reduce_kernel<true, 4>, grid, dim3(256), 0, stream, *a)
               : pa_launch(pa_reduce_kernel<true, 1>, grid, dim3(1024), 0, stream, *a);
  return big ? pa_launch(pa_reduce_kernel<false, 4>, grid, dim3(256), 0, stream, *a)
             : pa_launch(pa_reduce_kernel<false, 1>, grid, dim3(1024), 0, stream, *a);
}

// The reduce stage of a call whose partition stage went through the planning kernel: only the sequences with
// more than one partition are visited, by a grid of at most eight workgroups per CU that walks their units.
int launch_reduce_listed(const PaDecodeArgs* a, void* hip_stream) {
  const long long units = (long long)a->num_seqs * a->num_kv_heads * ((a->q_len * a->group_size + 15) / 16);
  const long long cap = 8LL * device_num_cus();
  const unsigned blocks = (unsigned)(units < cap ? units : cap);
  hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
  if (units * 16 >= 16384) return pa_launch(pa_reduce_listed_kernel<4>, dim3(blocks), dim3(256), 0, stream, *a);
  return pa_launch(pa_reduce_listed_kernel<1>, dim3(blocks), dim3(1024), 0, stream, *a);
}

}  // namespace

extern "C" {
#ifdef PA_DECODE_TRACE
// the measuring build only: the workgroups' timestamps of the last pa_partition_shared_kernel launch (8 words per
// workgroup id; workgroups that exited at once, or never ran, leave what was there: clear with pa_decode_trace_clear)
int pa_decode_trace_read(void* dst, unsigned long long bytes) {
  if (bytes > sizeof(pa_trace)) return PA_ERR_BAD_SHAPE;
  return hipMemcpyFromSymbol(dst, HIP_SYMBOL(pa_trace), bytes) == hipSuccess ? PA_OK : PA_ERR_LAUNCH;
}
int pa_decode_trace_clear(void) {
  void* p = nullptr;
  if (hipGetSymbolAddress(&p, HIP_SYMBOL(pa_trace)) != hipSuccess) return PA_ERR_LAUNCH;
  return hipMemset(p, 0, sizeof(pa_trace)) == hipSuccess ? PA_OK : PA_ERR_LAUNCH;
}
#endif


int pa_decode_abi_version(void) { return PA_DECODE_ABI_VERSION; }
uint32_t pa_decode_args_size(void) { return (uint32_t)sizeof(PaDecodeArgs); }
int pa_decode_last_hip_error(void) { return pa_last_hip_error; }

int64_t pa_decode_workspace_bytes(int32_t num_seqs, int32_t max_num_partitions) {
  if (num_seqs <= 0 || max_num_partitions <= 0) return PA_DECODE_WORKSPACE_BYTES;
  return full_workspace_bytes(num_seqs, max_num_partitions);
}

const char* pa_decode_error_string(int code) {
  switch (code) {
    case PA_OK: return "ok";
    case PA_ERR_NULL_POINTER: return "a required pointer is NULL";
    case PA_ERR_BAD_STRUCT: return "PaDecodeArgs.struct_size does not match this library";
    case PA_ERR_UNSUPPORTED: return "unsupported dtype, head size, block size or group size";
    case PA_ERR_BAD_SHAPE: return "bad size, partition size or stride";
    case PA_ERR_LAUNCH: return "HIP launch failed";
    case PA_ERR_NO_DEVICE: return "no HIP device";
    case PA_ERR_SCRATCH_TOO_SMALL: return "the call's partition buffers do not fit the library's scratch array";
  }
  return "unknown error code";
}

int pa_decode_select_partition_size(int32_t num_seqs, int32_t num_kv_heads, int32_t rows_per_group,
                                    int32_t max_context_len, int32_t block_size, int32_t num_cus) {
  return pa_decode_select_partition_size_stats(num_seqs, num_kv_heads, rows_per_group, max_context_len, 0, block_size,
                                               num_cus);
}

int pa_decode_select_partition_size_stats(int32_t num_seqs_given, int32_t num_kv_heads, int32_t rows_per_group,
                                          int32_t max_context_len, int64_t total_context_tokens, int32_t block_size,
                                          int32_t num_cus) {
  (void)block_size;
  if (num_seqs_given <= 0 || num_kv_heads <= 0 || max_context_len <= 0 || rows_per_group <= 0) return PA_ERR_BAD_SHAPE;
  if (num_cus <= 0) num_cus = device_num_cus();
  // The longest context sets how long the longest sequence's workgroups run; how many workgroups there are to fill
  // the GPU with is a matter of the batch's TOTAL length.  A batch of uneven lengths counts as total / longest
  // sequences of the longest length (8 sequences of which one holds nine tenths of the tokens are little more than
  // one sequence, and want the many small partitions that a batch of one wants).  Unknown total: every sequence
  // is taken to be as long as the longest.
  int num_seqs = num_seqs_given;
  if (total_context_tokens > 0) {
    const long long eff = (total_context_tokens + max_context_len - 1) / max_context_len;
    num_seqs = (int)(eff < 1 ? 1 : (eff > num_seqs_given ? num_seqs_given : eff));
  }
  const int total_tiles = (rows_per_group + 15) / 16;
  if (use_shared_stream(PA_DTYPE_FP8_E4M3FN, rows_per_group)) {
    // All row tiles of a kv head in one workgroup that walks its partition alone: three workgroups fit a CU, and
    // no workgroup gets more than 8192 tokens (measured on a ragged batch with the sorted dispatch: 6144-12288
    // is the flat optimum, 2048 costs 12 % in partials and merge, 32768 costs 45 % in balance; without the sorted
    // dispatch the optimum is 3072-4096 and 8192 costs 3 % more).
    const long long slots = (long long)num_cus * 3;
    const long long items = (long long)num_seqs * num_kv_heads;
    // one partition, hence no second kernel, is worth leaving up to 40 % of the workgroup slots empty (measured:
    // 128 sequences x 4 kv heads x 4096 tokens, 32 rows: 111 us against 126 us for two partitions; with 64
    // sequences three partitions win, 63 us against 83 us)
    const int whole = (max_context_len + 255) / 256 * 256;
    if (whole <= 8192 && items * 5 >= slots * 3) return whole;
    // otherwise the fewest partitions that fill the three slots per CU; but partitions of under 1024 tokens pay
    // their set-up and partials dearly, so there two workgroups per CU are enough (measured: 32 sequences x 4 kv
    // heads x 4096 tokens, 1024 -> 36.6 us against 39.4 us for 768; 4 x 8 x 16384: 43.0 against 47.6 us)
    const auto fewest_parts_for = [&](long long want) {
      for (int parts = 1;; ++parts) {
        int ps = (max_context_len + parts - 1) / parts;
        ps = (ps + 255) / 256 * 256;
        if (ps <= 256) return 256;
        if (ps <= 8192 && items * parts >= want) return ps;
      }
    };
    const int ps3 = fewest_parts_for(slots);
    return ps3 >= 1024 ? ps3 : fewest_parts_for((long long)num_cus * 2);
  }
  // One workgroup per 16-row query tile, up to 4 waves (at least 128 tokens each) per workgroup, no wave with
  // more than 2048 tokens (which keeps ragged batches balanced).  The number of partitions per sequence is the
  // one a small cost model likes best (times in microseconds on this GPU):
  //   a wave costs 1.3 us to set up; each of its 64-token steps costs the root sum of squares of 1.4 us (one
  //   wave alone: the step's own chain of loads, MFMAs and softmax) and its share of the HBM stream when
  //   `waves` of them run at once, 16 KiB * waves / 6.5 TB/s; the GPU holds 8 waves per CU, more run in rounds;
  //   splitting a sequence costs the second kernel (7 us) and its partials (written, read back: 2 ns per
  //   16-row tile and partition).
  // Few rows and long contexts want many partitions; 256 or more rows want one, even if that leaves a quarter
  // of the wave slots empty (measured at 48 sequences x 8 kv heads x 4096 tokens: 71 us against 78 us for two).
  // Measured against sweeps over 256..4096 at 1..64 sequences of 4096 tokens: the choice is the best or within
  // 2 % of it.
  const double rows = (double)num_seqs * num_kv_heads * total_tiles;
  const double step_us_per_wave = 16384.0 / 6.5e6;  // one more wave streaming a 16 KiB step at 6.5 TB/s
  const double wave_slots = 8.0 * num_cus;
  int best_ps = 256;
  double best_t = 1e30;
  for (int parts = 1;; ++parts) {
    int ps = (max_context_len + parts - 1) / parts;
    ps = (ps + 255) / 256 * 256;
    const int w = waves_for_partition_size(ps);
    if (ps <= 2048 * w) {
      const int steps_per_wave = ((ps + 63) / 64 + w - 1) / w;
      const double waves = rows * parts * w;
      const double at_once = waves < wave_slots ? waves : wave_slots;
      const double rounds = waves / at_once;
      const double share = at_once * step_us_per_wave;
      const double step_us = __builtin_sqrt(1.4 * 1.4 + share * share);
      const double t = rounds * (1.3 + steps_per_wave * step_us) + (parts > 1 ? 7.0 + 0.002 * rows * parts : 0.0);
      if (t < best_t * 0.999) {  // ties go to fewer partitions
        best_t = t;
        best_ps = ps;
      }
    }
    if (ps <= 256) return best_ps;
  }
}

// PA_DECODE_FLAG_OUTPUT_ONLY: the partition buffers are scratch, so how the partition axis is cut is the library's
// business.  A caller's small fixed partition size (the reference's constant 256) is replaced by the largest multiple
// of it that is not above the tuning layer's own choice for the shape: fewer, longer partitions, every entry of which
// lies inside the caller's buffers, at the caller's strides.  The axis must still end where the caller's ends
// (contexts beyond it are cut off at the same token, and no block-table entry beyond it is read).  With a factor that
// divides the caller's partition count it does; with another factor the last partition reaches further, and the
// kernels are then given a copy of the context lengths with the caller's limit applied (made by a small kernel, in
// the caller's workspace behind the item list; without a workspace of pa_decode_workspace_bytes the factor is the
// largest divisor).  The three entry points derive the same cut from the same arguments; `stream` is null when
// nothing may be launched (pa_decode_launch_info).  PA_DECODE_REPARTITION=0 (debug): never.
struct OwnPartitions {
  PaDecodeArgs args;
  int rc;
};

static OwnPartitions with_own_partitions(const PaDecodeArgs& a, bool launch, hipStream_t stream) {
  OwnPartitions r{a, PA_OK};
  static const bool off = debug_switch("PA_DECODE_REPARTITION", 1) == 0;
  if (off || !(a.flags & PA_DECODE_FLAG_OUTPUT_ONLY) || a.max_num_partitions <= 1 || generic_head_size(a)) return r;
  const long long axis = (long long)a.max_num_partitions * a.partition_size;
  if (axis > 0x7fffffffLL) return r;
  const int want = pa_decode_select_partition_size_stats(a.num_seqs, a.num_kv_heads, a.q_len * a.group_size, (int)axis, 0,
                                                         a.block_size, 0);
  const int P = a.max_num_partitions;
  long long k = want / a.partition_size;
  k = k > P ? P : k;
  if (k < 2) return r;
  if (P % k) {
    const long long parts = (P + k - 1) / k;
    // words of the workspace: header, item list of the new cut, [the limited lengths], ..., list of the sequences to merge
    const long long first = kPlanHeaderWords + 2LL * a.num_seqs * parts;
    const bool room = a.workspace != nullptr && a.workspace_bytes >= full_workspace_bytes(a.num_seqs, P) &&
                      first + 2LL * a.num_seqs <= a.workspace_bytes / 4;
    if (room) {
      r.args.context_lens = a.workspace + first;
      if (launch)  // (also when the item list is reused: 2 us, and the copy then never depends on an earlier call)
        r.rc = pa_launch(pa_limit_lens_kernel, dim3((unsigned)((a.num_seqs + 255) / 256)), dim3(256), 0, stream,
                         a.context_lens, a.workspace + first, (int)a.num_seqs, (int)axis);
    } else {
      while (P % k) --k;  // the largest divisor below
      if (k < 2) return r;
    }
  }
  r.args.partition_size = (int32_t)(a.partition_size * k);
  r.args.max_num_partitions = (int32_t)((P + k - 1) / k);
  return r;
}

int pa_decode_partition(const PaDecodeArgs* caller, void* hip_stream) {
  const int rc = check_partition(caller);
  if (rc) return rc;
  const OwnPartitions own = with_own_partitions(*caller, true, reinterpret_cast<hipStream_t>(hip_stream));
  if (own.rc) return own.rc;
  const PaDecodeArgs* a = &own.args;
  if (generic_head_size(*a)) return launch_partition_generic(*a, reinterpret_cast<hipStream_t>(hip_stream));
  return launch_partition(*a, choose_launch(*a, false), reinterpret_cast<hipStream_t>(hip_stream));
}

int pa_decode_reduce(const PaDecodeArgs* caller, void* hip_stream) {
  // PA_DECODE_FLAG_OUTPUT_ONLY: stage 1 ran with the same flag, cut the partition axis as with_own_partitions cuts
  // it and left no entries for the sequences it finished itself; stage 2 passes over them, as it does inside pa_decode
  if (caller && caller->struct_size == sizeof(PaDecodeArgs) && generic_head_size(*caller))
    return launch_reduce_generic(caller, hip_stream);
  const bool lean = caller && caller->struct_size == sizeof(PaDecodeArgs) && (caller->flags & PA_DECODE_FLAG_OUTPUT_ONLY);
  OwnPartitions own;
  const PaDecodeArgs* a = caller;
  if (lean) {
    const int rc = check_reduce(caller);  // (before the arguments are used)
    if (rc) return rc;
    // (the limited context lengths are made again: stage 2 does not rely on what stage 1 left in the workspace)
    own = with_own_partitions(*caller, true, reinterpret_cast<hipStream_t>(hip_stream));
    if (own.rc) return own.rc;
    a = &own.args;
  }
  if (lean && a->max_num_partitions == 1 && !a->sinks) {
    const int rc = check_reduce(a);
    return rc;  // every sequence was finished by stage 1
  }
  return launch_reduce(a, hip_stream, lean);
}

int pa_decode(const PaDecodeArgs* caller, void* hip_stream) {
  int rc = check_partition(caller);
  if (rc) return rc;
  rc = check_reduce(caller);  // before anything is launched
  if (rc) return rc;
  const OwnPartitions own = with_own_partitions(*caller, true, reinterpret_cast<hipStream_t>(hip_stream));
  if (own.rc) return own.rc;
  const PaDecodeArgs* a = &own.args;
  if (generic_head_size(*a)) {
    rc = launch_partition_generic(*a, reinterpret_cast<hipStream_t>(hip_stream));
    return rc ? rc : launch_reduce_generic(a, hip_stream);
  }
  const LaunchChoice c = choose_launch(*a, true);
  rc = launch_partition(*a, c, reinterpret_cast<hipStream_t>(hip_stream));
  if (rc) return rc;
  // the partition kernel has written the rows of every sequence that has a single partition itself
  if (a->max_num_partitions == 1 && !a->sinks) return PA_OK;
  if (c.team) return PA_OK;  // ... and a team those of every sequence
  if (c.listed_reduce) return launch_reduce_listed(a, hip_stream);
  return launch_reduce(a, hip_stream, true);
}

int pa_decode_launch_info(const PaDecodeArgs* a, char* text, int32_t text_bytes) {
  const int rc = check_partition(a);
  if (rc) return rc;
  if (!text || text_bytes <= 0) return PA_ERR_NULL_POINTER;
  if (generic_head_size(*a)) {
    snprintf(text, (size_t)text_bytes, "pa_partition_generic_kernel<head size %d, %s> x %lld", a->head_size,
             a->kv_dtype == PA_DTYPE_FP8_E4M3FN ? "fp8" : "bf16", generic_partition_blocks(*a));
    return PA_OK;
  }
  const OwnPartitions own = with_own_partitions(*a, false, nullptr);
  const bool recut = own.args.partition_size != a->partition_size;
  a = &own.args;
  const LaunchChoice c = choose_launch(*a, a->output != nullptr);  // (pa_decode's launch; pa_decode_partition forms no teams)
  const char* cache = !c.fp8 ? "bf16" : (c.per_token ? "fp8 per-token" : "fp8");
  const char* placed = c.heads_share_xcd ? ", an item's heads on one XCD" : "";
  if (c.shared)
    snprintf(text, (size_t)text_bytes, "pa_partition_shared_kernel<%s, %s, %d ring slots, %d workgroups per CU> x %lld%s%s",
             cache, c.bs16 ? "bs16" : "strided", c.per_token ? 3 : 2, c.per_cu, c.blocks, c.sorted ? ", sorted items" : "",
             placed);
  else
  {
    char span_text[96] = "";
    if (c.team)
      snprintf(span_text, sizeof(span_text), ", teams of %d waves, %d partitions per wave, no reduce kernel", kTeamWaves, c.span);
    else if (c.span > 1)
      snprintf(span_text, sizeof(span_text), ", %d partitions per workgroup", c.span);
    snprintf(text, (size_t)text_bytes, "pa_partition_kernel<%s, %s, %d waves%s> x %lld%s%s%s", cache,
             c.bs16 ? "bs16" : "strided", c.waves, c.row_tiles == 2 ? ", 2 row tiles" : "", c.blocks,
             c.queue ? ", queued items" : (c.sorted ? ", sorted items" : ""), span_text, placed);
  }
  if (recut) {  // PA_DECODE_FLAG_OUTPUT_ONLY: the library's own cut of the caller's partition axis
    const size_t used = strlen(text);
    if (used + 1 < (size_t)text_bytes)
      snprintf(text + used, (size_t)text_bytes - used, ", own partitions of %d tokens", a->partition_size);
  }
  return PA_OK;
}

int pa_decode_noalloc(const PaDecodeArgs* a, void* hip_stream) {
  if (!a) return PA_ERR_NULL_POINTER;
  if (a->struct_size != sizeof(PaDecodeArgs)) return PA_ERR_BAD_STRUCT;
  // the library owns these four in this entry point: a caller that passes its own wants pa_decode
  if (a->exp_sums || a->max_logits || a->tmp_output || a->workspace || a->workspace_bytes) return PA_ERR_BAD_SHAPE;
  // Every other check of pa_decode runs on the caller's arguments first, with stand-ins for the four buffers the
  // library brings: the sizes below are then products of checked, positive int32 values.
  {
    PaDecodeArgs probe = *a;
    probe.exp_sums = probe.max_logits = reinterpret_cast<float*>(uintptr_t{256});
    probe.tmp_output = reinterpret_cast<void*>(uintptr_t{256});
    probe.stride_es_s = probe.stride_es_h = probe.stride_es_p = 0;  // the caller's strides of these buffers are ignored
    probe.stride_tmp_s = probe.stride_tmp_h = probe.stride_tmp_p = probe.stride_tmp_g = 0;
    int rc = check_partition(&probe);
    if (rc) return rc;
    rc = check_reduce(&probe);
    if (rc) return rc;
  }

  // ---- this device's copy of the scratch array: its address is asked for once per device, with that device
  // current.  The stream must belong to the current device (a stream of another GPU would get a pointer into the
  // wrong GPU's array): checked, not assumed.
  constexpr int kMaxDevices = 64;
  static unsigned char* scratch_of_device[kMaxDevices] = {};
  static std::mutex scratch_lock;
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return PA_ERR_NO_DEVICE;
  if (hip_stream != nullptr) {
    int stream_dev = -1;
    if (hipStreamGetDevice(reinterpret_cast<hipStream_t>(hip_stream), &stream_dev) != hipSuccess || stream_dev != dev)
      return PA_ERR_NO_DEVICE;
  }
  unsigned char* base;
  {
    std::lock_guard<std::mutex> guard(scratch_lock);
    if (!scratch_of_device[dev]) {
      void* p = nullptr;
      const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
      if (e != hipSuccess || !p) {
        pa_last_hip_error = (int)e;
        return PA_ERR_LAUNCH;
      }
      scratch_of_device[dev] = static_cast<unsigned char*>(p);
    }
    base = scratch_of_device[dev];
  }

  // ---- layout: workspace, max_logits, exp_sums, tmp_output, each at a multiple of 256 bytes ------------------
  // (the four factors are positive int32 values and ge <= 64: every product is formed with an overflow check)
  const auto round256 = [](long long n) { return (n + 255) / 256 * 256; };
  const long long ge = (long long)a->q_len * a->group_size;
  const long long limit = (long long)PA_DECODE_NOALLOC_SCRATCH_BYTES;
  long long rows = 0, tmp_bytes = 0;
  if (__builtin_mul_overflow((long long)a->num_seqs * a->num_kv_heads, (long long)a->max_num_partitions * ge, &rows) ||
      __builtin_mul_overflow(rows, 2LL * a->head_size, &tmp_bytes) || tmp_bytes > limit)
    return PA_ERR_SCRATCH_TOO_SMALL;
  // (rows * 128 <= 64 MiB bounds num_seqs * max_num_partitions by 2^19: the workspace size cannot overflow either)
  const long long ws_bytes = full_workspace_bytes(a->num_seqs, a->max_num_partitions);
  if (ws_bytes > limit) return PA_ERR_SCRATCH_TOO_SMALL;
  const long long off_ml = round256(ws_bytes);
  const long long off_es = off_ml + round256(4 * rows);
  const long long off_tmp = off_es + round256(4 * rows);
  const long long total = off_tmp + round256(tmp_bytes);
  if (total > limit) return PA_ERR_SCRATCH_TOO_SMALL;

  PaDecodeArgs k = *a;
  k.workspace = reinterpret_cast<int32_t*>(base);
  k.workspace_bytes = ws_bytes;
  k.max_logits = reinterpret_cast<float*>(base + off_ml);
  k.exp_sums = reinterpret_cast<float*>(base + off_es);
  k.tmp_output = base + off_tmp;
  k.stride_es_p = ge;
  k.stride_es_h = ge * a->max_num_partitions;
  k.stride_es_s = k.stride_es_h * a->num_kv_heads;
  k.stride_tmp_g = a->head_size;
  k.stride_tmp_p = ge * a->head_size;
  k.stride_tmp_h = k.stride_tmp_p * a->max_num_partitions;
  k.stride_tmp_s = k.stride_tmp_h * a->num_kv_heads;
  // the array keeps the last call's contents (a call that was cut short may have left its counters non-zero, and
  // an item list of another batch): the counters are cleared, the lists are rebuilt
  k.flags &= ~PA_DECODE_FLAG_REUSE_ITEM_LIST;
  const int rc = pa_launch(pa_clear_words_kernel, dim3(1), dim3(64), 0, reinterpret_cast<hipStream_t>(hip_stream),
                           k.workspace, (int)kPlanHeaderWords);
  if (rc) return rc;
  return pa_decode(&k, hip_stream);
}

int pa_debug_fp8_decode(const uint8_t* codes, float* out, int32_t n, void* hip_stream) {
  if (!codes || !out) return PA_ERR_NULL_POINTER;
  if (n <= 0) return PA_ERR_BAD_SHAPE;
  return pa_launch(pa_fp8_decode_kernel, dim3((n + 255) / 256), dim3(256), 0, reinterpret_cast<hipStream_t>(hip_stream),
                   codes, out, (int)n);
}

}  // extern "C"
