// pa_partition_kernel: stage 1 for up to 16 query rows per kv head (and for every bf16 cache).
//
// Work decomposition.  A workgroup of 1, 2 or 4 waves owns one item: (sequence, partition, 16-row
// query tile, kv head).  The waves take the partition's steps of 64 tokens (four 16-token tiles) round
// robin, each with private online-softmax state (m, l, O), and merge through LDS at the end.  A sequence that fits in one partition gets its final output from this kernel directly.
//
//   K tile  (16 tokens x 128 dims): every lane loads 16 bytes = one [token][16-byte chunk] cell of
//           the cache; lanes 0-15 are the 16 tokens of a page, lane>>4 picks the chunk row, so a
//           wave load covers 4 x 256 contiguous bytes in storage order.  The dot product does not care
//           in which order the head dimension is summed, so the query operand is built in the order
//           the loads deliver it.
//   S^T = K Q^T: tokens are the M rows, query rows (GQA group x MTP position, padded to 16) are
//           the N columns, so a lane ends up with 4 tokens of ONE query row per tile and the softmax
//           max/sum need only two cross-lane steps (lane^16, lane^32).
//   V tile  (128 dims x 16 tokens): every lane loads 16 bytes = 16 tokens of one head dim, lanes
//           0-15 are 16 consecutive dims (256 contiguous bytes with block 16), lane>>4 picks one of
//           the four tiles of the step.  O^T = V^T P^T accumulates in 8 MFMA tiles of [16 dims x 16 rows].
//
// FP8 cache: the cache bytes are MFMA operands as they are (v_mfma_f32_16x16x128_f8f6f4 for Q K^T,
// v_mfma_f32_16x16x32_fp8_fp8 for P V); the bf16 query and P are each carried as an FP8 head plus an
// FP8 residual (x*c = hi + lo, every product exact in the f32 accumulator), about 2^-8 relative per
// element, so there is no FP8->bf16 conversion work at all; P reaches the B-operand layout through a 4x4
// (lane group x register) transpose with v_permlane{16,32}_swap, not through LDS.  Per-tensor scales
// fold into the softmax scale (K) and the epilogue (V); per-token scales multiply S and P in f32.
// bf16 cache: bf16 MFMA (v_mfma_f32_16x16x32_bf16), P through a wave-private LDS tile.
#ifndef PA_PARTITION_KERNEL_H_
#define PA_PARTITION_KERNEL_H_

#include "pa_common.h"

namespace {

// One step's worth of cache data, as loaded (still FP8 / bf16 bit patterns).
template <int KVT, bool PER_TOKEN>
struct StepData {
  static constexpr int NKL = KVT == PA_DTYPE_FP8_E4M3FN ? 2 : 4;  // 16-byte K loads per lane per tile
  static constexpr int NVL = KVT == PA_DTYPE_FP8_E4M3FN ? 1 : 2;  // 16-byte V loads per lane per 16 dims
  u32x4 k[4][NKL];
  u32x4 v[8][NVL];
  f32x4 ks[PER_TOKEN ? 4 : 1];
  f32x4 vs[PER_TOKEN ? 4 : 1];
};

// The partition kernel.  OCC is the number of waves per SIMD the register budget is cut for.
//
// Software pipeline of one wave (each line is issued in order; loads return in order):
//   QK(s)      needs K(s)            -> then K(s+1) is loaded into the registers K(s) just left
//   softmax(s)                          (K(s+1) and V(s) in flight)
//   PV(s)      needs V(s)            -> then V(s+1) is loaded into the registers V(s) just left
// so about one step (16 KiB) of cache data per wave is in flight at any time without a second
// register copy.  Steps that need no masking and have a successor run in a branch-free loop, so
// the compiler's vmcnt waits stay partial; the last step(s) go through the masked variants.
//
// BS16 (block size 16) turns every stride inside a page into a compile-time constant, so the loads
// of a tile share one address register pair and differ by immediate offsets.
constexpr int kQueueMaxSeqs = 2048;  // sequences the item table of the queued launch can hold

// REREAD: the kv head has more row tiles than a workgroup takes (a bf16 cache with more than 32 query rows), so a
// second workgroup streams the same pages at about the same time: the cache is then read with ordinary loads (the
// lines had better still be in L2 when the other workgroup asks; non-temporal loads mark them for early eviction).
// TEAM (with WAVES = 1): four one-wave span walkers in ONE workgroup, wave w walking partitions w * span .. of the
// same (sequence, kv head, row tile), each exactly as a one-wave workgroup would.  When the four spans cover the
// whole partition axis, every partial result of the sequence is in this workgroup's LDS at the end, and the
// workgroup merges them into `output` itself: no second kernel (a caller's fixed 256-token partitions over a 4096-
// token context: 6 us of a 95 us call).
template <int NT, int KVT, bool PER_TOKEN, bool BS16, int WAVES, int OCC, bool QUEUE, bool REREAD = false, bool TEAM = false>
__global__ __launch_bounds__(TEAM ? 256 : 64 * WAVES) __attribute__((amdgpu_waves_per_eu(OCC, OCC)))
void pa_partition_kernel(const PaDecodeArgs a) {
  static_assert(!TEAM || (WAVES == 1 && !QUEUE && NT == 1), "a team is four one-wave span walkers of one row tile");
  constexpr bool kFp8 = KVT == PA_DTYPE_FP8_E4M3FN;
  constexpr bool FP8MATH = kFp8;  // an FP8 cache is multiplied on the FP8 MFMAs, a bf16 cache on the bf16 ones
  constexpr int esz = kFp8 ? 1 : 2;
  typedef StepData<KVT, PER_TOKEN> SD;

  __shared__ __attribute__((aligned(16))) char p_lds[FP8MATH ? 1 : WAVES][FP8MATH ? 1 : NT][FP8MATH ? 16 : 16 * kPRowBytes];
  // SPAN: the partial results of the partitions a workgroup walks wait here for the end of the pass (stores in the
  // middle of the page stream would hold up the loads issued after them: memory operations of a wave retire in
  // order), the last partition's included.  Per partition and row tile: the staged bf16 rows (16, or 8 when the
  // tile has no more real rows than that: half the bytes, twice the partitions), then 16 maxima and 16 sums.
  constexpr bool kSpanCapable = WAVES == 1 && !QUEUE;
  __shared__ __attribute__((aligned(16))) char o_lds[1][kSpanCapable ? 16 : 16 * kORowBytes];
  __shared__ __attribute__((aligned(16))) char span_lds[kSpanCapable ? (TEAM ? kTeamWaves : 1) * NT * kSpanPoolBytes : 16];

  const int lane = threadIdx.x & 63;
  const int team_wave = TEAM ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) : 0;
  const int wave = TEAM ? 0 : __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  char* const span_pool = &span_lds[0] + (kSpanCapable ? team_wave * NT * kSpanPoolBytes : 0);  // this wave's staging pool
  const int li = lane & 15;
  const int kg = lane >> 4;

  // ---- which (sequence, head, partition): all wave-uniform -----------------------------------------
  const int P = a.max_num_partitions;
  const int Hkv = a.num_kv_heads;
  // The WAVES waves of a workgroup share one item: (sequence, partition, group of NT 16-row query tiles,
  // kv head).  The head varies fastest, so the workgroups that stream the same pages (the other heads, and
  // the other row tiles of the same head, 8 ids apart with 8 kv heads: the same XCD and L2) run together.
  const int Ge = a.q_len * a.group_size;  // rows per kv head in the buffers
  const int RT = (Ge + 16 * NT - 1) / (16 * NT);

  // QUEUE: a resident grid of workgroups pulls live items from a counter in the caller's workspace.  Only
  // partitions a sequence reaches and row tiles that hold real query rows are items, so a ragged batch
  // launches no workgroup that would exit at once (each of those still costs a wave slot for a
  // microsecond).  Every workgroup builds, once, the exclusive prefix sum of the per-sequence item counts
  // in LDS and decodes an item index by binary search in it.
  __shared__ int q_cum[QUEUE ? kQueueMaxSeqs + 1 : 1];
  __shared__ int q_ctx[QUEUE ? kQueueMaxSeqs : 1];
  __shared__ int q_tiles[QUEUE ? kQueueMaxSeqs : 1];
  __shared__ int q_item;
  int total_items = 0;
  if constexpr (QUEUE) {
    if (wave == 0) {
      int running = 0;
      for (int b0 = 0; b0 < a.num_seqs; b0 += 64) {
        const int bb = b0 + lane;
        const int c = bb < a.num_seqs ? a.context_lens[bb] : 0;
        int np = (c + a.partition_size - 1) / a.partition_size;
        np = np <= 0 ? 1 : (np > P ? P : np);  // an empty sequence keeps one item: its workgroups zero its output rows
        const int ql = bb < a.num_seqs ? (a.q_lens ? a.q_lens[bb] : a.q_len) : 0;
        int tiles = (ql * a.group_size + 16 * NT - 1) / (16 * NT);
        tiles = tiles > RT ? RT : tiles;
        const int n = np * tiles;
        int x = n;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
          const int y = __shfl_up(x, d);
          if (lane >= d) x += y;
        }
        if (bb < a.num_seqs) {
          q_cum[bb] = running + x - n;
          q_ctx[bb] = c;
          q_tiles[bb] = tiles;
        }
        running += __builtin_amdgcn_readlane(x, 63);
      }
      if (lane == 0) q_cum[a.num_seqs] = running;
    }
    __syncthreads();
    total_items = q_cum[a.num_seqs] * Hkv;
  }

  // SPAN (one-wave workgroups, plain or sorted launch order): the workgroup walks `span` consecutive partitions in one pass
  // over the pages, and writes the partial result of each as it crosses into the next.  For callers whose buffers
  // fix a small partition size (the reference's constant 256): the query set-up and the ramp of the page stream
  // are paid once per span instead of once per four steps.
  // rows staged per tile and the bytes of a tile's slot in the pool
  const int span_rows = (NT == 1 && Ge <= 8) ? 8 : 16;
  const int span_slot_bytes = span_rows * kORowBytes + 2 * 16 * 4;
  int span = 1;
  if constexpr (kSpanCapable) {
    const int span_max = span_rows == 8 ? kSpanMaxFewRows : kSpanMax;
    span = (a.flags >> kFlagSpanShift) & 0xff;
    span = span < 1 ? 1 : (span > span_max ? span_max : span);
  }
  static_assert(kSpanMax * (16 * kORowBytes + 2 * 16 * 4) <= kSpanPoolBytes, "the pool holds kSpanMax full tiles");

  for (;;) {  // one pass without the queue
  int h, rt, b, part, tiles_b = RT;
  if constexpr (QUEUE) {
    if (threadIdx.x == 0) q_item = atomicAdd(a.workspace, 1);
    __syncthreads();
    const int item = __builtin_amdgcn_readfirstlane(q_item);
    __syncthreads();  // everybody has read q_item (and is done with the LDS buffers of the previous item)
    if (item >= total_items) break;
    h = item % Hkv;
    const int j = item / Hkv;
    int lo = 0, hi = a.num_seqs;  // q_cum[lo] <= j < q_cum[hi]
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (__builtin_amdgcn_readfirstlane(q_cum[mid]) <= j)
        lo = mid;
      else
        hi = mid;
    }
    b = lo;
    tiles_b = __builtin_amdgcn_readfirstlane(q_tiles[b]);
    const int local = j - __builtin_amdgcn_readfirstlane(q_cum[b]);
    part = local / tiles_b;
    rt = local - part * tiles_b;
  } else {
    // The partition index varies slowest: in a ragged batch the partitions that only the longest
    // sequences reach (workgroups that exit at once for everybody else) come last.
    // (32-bit unsigned arithmetic: the grid has fewer than 2^31 workgroups, and a 64-bit division by a run-time
    // value is a hundred instructions in front of the workgroup's first request)
    const uint32_t wid = blockIdx.x;
    uint32_t item;
    if (PER_TOKEN && (a.flags & kFlagHeadsShareXcd)) {
      // Workgroup ids go round the eight XCDs: an XCD takes every eighth item with all its kv heads and row tiles one
      // after the other, so the 128-byte lines that hold the per-token scales of two neighbouring heads are
      // fetched into one L2 once (with the head fastest in the id every head sits on another XCD)
      const uint32_t xcd = wid & 7u;
      const uint32_t slot = wid >> 3;
      const uint32_t units = (uint32_t)(Hkv * RT);
      const uint32_t unit = slot % units;
      h = (int)(unit % (uint32_t)Hkv);
      rt = (int)(unit / (uint32_t)Hkv);
      item = (slot / units) * 8u + xcd;
      if (!(a.flags & kFlagSortedItems) && item >= (uint32_t)a.num_seqs * (uint32_t)(TEAM ? 1 : (P + span - 1) / span)) return;
    } else {
      h = (int)(wid % (uint32_t)Hkv);
      rt = (int)((wid / (uint32_t)Hkv) % (uint32_t)RT);
      item = wid / (uint32_t)(Hkv * RT);
    }
    if (a.flags & kFlagSortedItems) {
      // the planning kernel has listed the live (sequence, partition) items, longest last partitions first
      if (item >= (uint32_t)sload_i32(a.workspace + 2)) return;
      b = sload_i32(a.workspace + kPlanHeaderWords + 2 * (int64_t)item);
      part = sload_i32(a.workspace + kPlanHeaderWords + 2 * (int64_t)item + 1) * span;
    } else {
      b = (int)(item % (uint32_t)a.num_seqs);
      const int coarse = (int)(item / (uint32_t)a.num_seqs);
      part = coarse * span;
      // (items go to the XCDs round robin: with a batch that is a multiple of eight every partition of a sequence
      // would sit on the same XCD, and a batch's one long sequence on one eighth of the GPU; each partition index
      // therefore starts the batch one sequence further on)
      if (PER_TOKEN && (a.flags & kFlagHeadsShareXcd)) b = (b + coarse % a.num_seqs) % a.num_seqs;
    }
  }
  const int row0 = 16 * NT * rt;  // first query row of this workgroup inside its kv-head group
  if constexpr (TEAM) part += team_wave * span;  // (a team's item is the sequence's whole axis: its first partition is 0)
  do {  // the body of one item; `break` leaves it
  if constexpr (TEAM) {
    if (part >= P) break;  // (a wave of the team with no partition left)
  }

  // The block-table entries of this wave's first step are requested together with the context length, not after it
  // (dependent scalar loads are round trips under full memory load; the first request of a workgroup waits for
  // all of them).  They are entries of this sequence's row (the index is kept inside the row); one that lies beyond
  // the sequence's end is read but never used.
  const int log2_bs = 31 - __builtin_clz(a.block_size);
  const int* bt = a.block_tables + (int64_t)b * a.stride_bt_s;
  int early_page[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    int idx = (part * a.partition_size + wave * kStepTokens + 16 * j) >> log2_bs;
    idx = idx < (int)a.stride_bt_s ? idx : (int)a.stride_bt_s - 1;  // (stride_bt_s >= 1: checked by the launch layer)
    early_page[j] = sload_i32(bt + idx);
  }
  const int ctx = sload_i32(a.context_lens + b);
  const int wg_start = part * a.partition_size;
  if (wg_start >= ctx) {
    if (ctx <= 0 && part == 0 && !TEAM) {
      if constexpr (QUEUE) {  // only tiles with real query rows are items: the first one zeroes the whole group
        if (rt == 0) zero_output_rows(a, b, h, 0, Ge);
      } else {
        zero_output_rows(a, b, h, row0, row0 + 16 * NT < Ge ? row0 + 16 * NT : Ge);
      }
    }
    break;
  }
  const int span_here = min(span, P - part);  // partitions of this workgroup that the buffers have room for
  const int wg_end = min(wg_start + span_here * a.partition_size, ctx);
  // The waves take the partition's 64-token steps round robin (wave w: steps w, w + WAVES, ...), so at any
  // time the workgroup reads WAVES * 64 consecutive tokens: with large blocks that is whole 128-byte lines of
  // every V row and long runs of every K chunk row, requested by the waves together.  A wave with no step
  // idles until the merge.
  const int wg_steps = (wg_end - wg_start + kStepTokens - 1) / kStepTokens;
  constexpr int kWaveStride = WAVES * kStepTokens;
  const int part_start = wg_start + wave * kStepTokens;
  const bool active = part_start < wg_end;
  const int G = a.group_size;
  const int qb = a.q_lens ? sload_i32(a.q_lens + b) : a.q_len;
  const int rows_valid = qb * G;
  if (row0 >= rows_valid) {
    // only padding rows (a ragged batch): nothing to stream; the rows read as "no visible key"
    if (wave == 0 && !(a.flags & kFlagOutputOnly)) {
      auto write_padding = [&](int pp) {
        const int64_t eo = (int64_t)b * a.stride_es_s + (int64_t)h * a.stride_es_h + (int64_t)pp * a.stride_es_p;
        char* tp = (char*)a.tmp_output + ((int64_t)b * a.stride_tmp_s + (int64_t)h * a.stride_tmp_h +
                                          (int64_t)pp * a.stride_tmp_p) * 2;
        char* op = (char*)a.output + ((int64_t)b * a.stride_out_s + (int64_t)h * Ge * a.stride_out_h) * 2;
        const bool dir = (ctx <= a.partition_size || a.max_num_partitions == 1) && a.output != nullptr && a.sinks == nullptr;
        for (int r = row0 + kg; r < row0 + 16 * NT && r < Ge; r += 4) {
          if (li == 0) {
            a.max_logits[eo + r] = -INFINITY;
            a.exp_sums[eo + r] = 0.f;
          }
          *reinterpret_cast<u32x4*>(tp + (int64_t)r * a.stride_tmp_g * 2 + li * 16) = u32x4{0, 0, 0, 0};
          if (dir) *reinterpret_cast<u32x4*>(op + (int64_t)r * a.stride_out_h * 2 + li * 16) = u32x4{0, 0, 0, 0};
        }
      };
      if constexpr (WAVES == 1 && !QUEUE) {
        for (int pp = part; pp * a.partition_size < wg_end; ++pp) write_padding(pp);  // every partition of the span
      } else {
        write_padding(part);
      }
    }
    break;
  }

  // ---- cache addressing -------------------------------------------------------------------------------
  const int bs_mask = a.block_size - 1;
  const char* kbase = (const char*)a.key_cache + (int64_t)h * a.stride_k_h * esz;
  const char* vbase = (const char*)a.value_cache + (int64_t)h * a.stride_v_h * esz;
  const int64_t k_block_bytes = a.stride_k_b * esz;
  const int64_t v_block_bytes = a.stride_v_b * esz;
  const float* ksbase = PER_TOKEN ? a.key_scale + (int64_t)h * a.stride_kvscale_h : nullptr;
  const float* vsbase = PER_TOKEN ? a.value_scale + (int64_t)h * a.stride_kvscale_h : nullptr;
  const uint32_t k_chunk_bytes = BS16 ? 256u : (uint32_t)(a.stride_k_c * esz);
  uint32_t k_lane_off[SD::NKL];  // per-lane byte offset of K load ld inside a tile
#pragma unroll
  for (int ld = 0; ld < SD::NKL; ++ld) k_lane_off[ld] = (uint32_t)(kg * k_chunk_bytes + li * 16) + 4 * ld * k_chunk_bytes;
  // V: byte offset of this lane's head dim inside a tile, distance of the second 8-token half
  // (bf16 only) and, for the transposed layout, of consecutive 16-token tiles of a page
  // (with block size 16 the plain and the transposed FP8 layouts are the same bytes; for bf16 they
  // differ, so the constant-stride form is used for the plain layout only)
  const bool vt = a.v_transposed;
  const bool v_whole_lines = KVT == PA_DTYPE_FP8_E4M3FN && (a.v_transposed || a.block_size <= 64);
  const uint32_t v_row_bytes = BS16 ? 16u * esz : (vt ? 16u : (uint32_t)(a.stride_v_2 * esz));
  const uint32_t v_half_bytes = BS16 ? 16u : (vt ? (uint32_t)(a.stride_v_2 * esz) : 16u);
  const int64_t v_tile_bytes = BS16 ? 16 * esz : (vt ? a.stride_v_2 * esz * esz : 16 * esz);
  uint32_t v_lane_off[8];
#pragma unroll
  for (int db = 0; db < 8; ++db) v_lane_off[db] = li * v_row_bytes + 16 * db * v_row_bytes;

  const int last_tile_tok = (wg_end - 1) & ~15;  // first token of the last tile that holds a live token

  // page ids of the four tiles of the step that starts at token tok0 (scalar loads; tiles past the
  // last live one repeat it, so no block-table slot or page beyond the sequence is ever touched)
  struct Pages {
    int p[4];
    int off[4];  // token offset of the tile inside its page
  };
  auto load_pages = [&](int tok0) {
    Pages pg;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int t = tok0 + 16 * j;
      t = t > last_tile_tok ? last_tile_tok : t;
      pg.p[j] = sload_i32(bt + (t >> log2_bs));
      pg.off[j] = t & bs_mask;
    }
    return pg;
  };
  constexpr bool read_once = !REREAD;  // (a choice made per load at run time costs a tenth of the kernel's rate)
  auto issue_k = [&](SD& sd, const Pages& pg) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const char* tb = kbase + (int64_t)pg.p[j] * k_block_bytes + (int64_t)pg.off[j] * 16;
      if constexpr (read_once) {
#pragma unroll
        for (int ld = 0; ld < SD::NKL; ++ld) sd.k[j][ld] = load16_stream(tb + k_lane_off[ld]);
      } else {
#pragma unroll
        for (int ld = 0; ld < SD::NKL; ++ld) sd.k[j][ld] = load16(tb + k_lane_off[ld]);
      }
      if constexpr (PER_TOKEN) {
        const int64_t so = (int64_t)pg.p[j] * a.stride_kvscale_b + pg.off[j] + 4 * kg;
        sd.ks[j] = *reinterpret_cast<const f32x4*>(ksbase + so);
      }
    }
  };
  auto issue_v = [&](SD& sd, const Pages& pg) {
    // lane group kg owns tile kg of the step
    const int page = kg == 0 ? pg.p[0] : (kg == 1 ? pg.p[1] : (kg == 2 ? pg.p[2] : pg.p[3]));
    const int off = kg == 0 ? pg.off[0] : (kg == 1 ? pg.off[1] : (kg == 2 ? pg.off[2] : pg.off[3]));
    const char* tb = vbase + (int64_t)page * v_block_bytes + (int64_t)(off >> 4) * v_tile_bytes;
    // Non-temporal where one load covers whole 128-byte lines.  With plain V and pages of more than 64 tokens
    // a 64-token step takes half a line of every head dim's row and the next step the other half: those lines
    // must stay in L2 in between (streaming them costs 13 % on 1024-token pages).
    if ((BS16 || v_whole_lines) && read_once) {
#pragma unroll
      for (int db = 0; db < 8; ++db) {
#pragma unroll
        for (int hf = 0; hf < SD::NVL; ++hf) sd.v[db][hf] = load16_stream(tb + v_lane_off[db] + hf * v_half_bytes);
      }
    } else {
#pragma unroll
      for (int db = 0; db < 8; ++db) {
#pragma unroll
        for (int hf = 0; hf < SD::NVL; ++hf) sd.v[db][hf] = load16(tb + v_lane_off[db] + hf * v_half_bytes);
      }
    }
    if constexpr (PER_TOKEN) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int64_t so = (int64_t)pg.p[j] * a.stride_kvscale_b + pg.off[j] + 4 * kg;
        sd.vs[j] = *reinterpret_cast<const f32x4*>(vsbase + so);
      }
    }
  };

  // ---- first loads go out before anything else is set up ---------------------------------------------
  const int n_steps = active ? (wg_steps - wave + WAVES - 1) / WAVES : 0;
  SD buf_a;  // one step of cache data, refilled in place for the next step
  if (active) {
    Pages pg0;
    if (part_start + 48 <= last_tile_tok) {  // (the early requests were for these four tiles)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        pg0.p[j] = early_page[j];
        pg0.off[j] = (part_start + 16 * j) & bs_mask;
      }
    } else {
      pg0 = load_pages(part_start);
    }
    issue_k(buf_a, pg0);
    issue_v(buf_a, pg0);
  }

  // ---- per-lane row bookkeeping -------------------------------------------------------------------------
  int limit[NT];      // number of visible keys of this lane's query row
  float slope2[NT];   // ALiBi slope * log2e
  const bool has_alibi = a.alibi_slopes != nullptr;
  const bool alibi_per_row = a.alibi_slopes_len == Hkv * Ge;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    int row = row0 + 16 * nt + li;
    int t = row / G;
    limit[nt] = row < rows_valid ? ctx - (qb - 1 - t) : 0;
    slope2[nt] = 0.f;
    // one slope per packed row (the reference kernels' indexing) or one per query head, shared by its new tokens
    if (has_alibi && row < rows_valid)
      slope2[nt] = a.alibi_slopes[alibi_per_row ? h * Ge + row : h * G + (row - t * G)] * kLog2e;
  }
  const int min_limit = ctx - (qb - 1);  // keys below this index are visible to every real row

  // ---- query: B operand of S^T = K Q^T --------------------------------------------------------------------
  // k-step s of a tile covers, for lane group kg, the 8 head dims the K load puts in that slot.
  // Rows past the last real one are loaded from row 0 and zeroed, which keeps this branch-free.
  bf16x8 qreg[NT][4];
  {
    const char* q_ptr = (const char*)a.query;
    // all loads of the tile rows go out together (one choice of the query's type around them, not one inside each:
    // the compiler would wait for every load before it issues the next)
    const bool q_bf16 = a.query_dtype == PA_DTYPE_BF16;
    u32x4 raw[NT][4];
    bool ok[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int row = row0 + 16 * nt + li;
      ok[nt] = row < rows_valid;
      const int64_t e0 = (int64_t)b * a.stride_q_s + (int64_t)(h * Ge + (ok[nt] ? row : 0)) * a.stride_q_h;
      if (q_bf16) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const int dim = kFp8 ? (64 * (s >> 1) + 16 * kg + 8 * (s & 1)) : (32 * s + 8 * kg);
          raw[nt][s] = load16(q_ptr + (e0 + dim) * 2);
        }
      } else {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const int dim = kFp8 ? (64 * (s >> 1) + 16 * kg + 8 * (s & 1)) : (32 * s + 8 * kg);
          const u32x2 r8 = *reinterpret_cast<const u32x2*>(q_ptr + e0 + dim);
          raw[nt][s] = u32x4{r8[0], r8[1], 0, 0};
        }
      }
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        Bf16x8Bits q;
        q.u = raw[nt][s];
        if (!q_bf16) q.v = fp8x8_to_bf16x8(raw[nt][s][0], raw[nt][s][1]);
        if (!ok[nt]) q.u = u32x4{0, 0, 0, 0};
        qreg[nt][s] = q.v;
      }
    }
  }
  // per-row query scale (FP8 query) multiplies the logits of that row
  float k_tensor_scale = 1.f, v_tensor_scale = 1.f;
  if (a.kv_quant_mode == PA_QUANT_PER_TENSOR) {
    k_tensor_scale = sload_f32(a.key_scale);
    v_tensor_scale = sload_f32(a.value_scale);
  }
  const float scale2 = a.softmax_scale * k_tensor_scale * kLog2e;
  float rscale[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int row = row0 + 16 * nt + li;
    float qs = 1.f;
    if (a.query_quant_mode == PA_QUANT_PER_TENSOR) qs = sload_f32(a.query_scale);
    if (a.query_quant_mode == PA_QUANT_PER_TOKEN && row < rows_valid)
      qs = a.query_scale[(int64_t)b * a.stride_qscale_s + h * Ge + row];
    rscale[nt] = scale2 * qs;
  }
  // FP8 math: q * cq = hi + lo with hi, lo in e4m3 and cq a power of two (exact); the logits are divided by cq again
  i32x8 qhi[FP8MATH ? NT : 1], qlo[FP8MATH ? NT : 1];
  if constexpr (FP8MATH) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      float f[32];
      float amax = 0.f;
#pragma unroll
      for (int s4 = 0; s4 < 4; ++s4) {
        Bf16x8Bits q;
        q.v = qreg[nt][s4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          f[8 * s4 + 2 * e] = bf16_bits_to_f32(q.u[e] & 0xffffu);
          f[8 * s4 + 2 * e + 1] = __uint_as_float(q.u[e] & 0xffff0000u);
        }
      }
#pragma unroll
      for (int e = 0; e < 32; ++e) amax = fmaxf(amax, fabsf(f[e]));
      amax = quad_row_max(amax);
      float cq_inv;
      const float cq = query_pow2_factor(amax, cq_inv);
      rscale[nt] *= cq_inv;
#pragma unroll
      for (int w = 0; w < 8; ++w) {
        const float x0 = f[4 * w] * cq, x1 = f[4 * w + 1] * cq, x2 = f[4 * w + 2] * cq, x3 = f[4 * w + 3] * cq;
        int hi = 0, lo = 0;
        hi = __builtin_amdgcn_cvt_pk_fp8_f32(x0, x1, hi, false);
        hi = __builtin_amdgcn_cvt_pk_fp8_f32(x2, x3, hi, true);
        const f32x2 b01 = __builtin_amdgcn_cvt_pk_f32_fp8(hi, false);
        const f32x2 b23 = __builtin_amdgcn_cvt_pk_f32_fp8(hi, true);
        lo = __builtin_amdgcn_cvt_pk_fp8_f32(x0 - b01[0], x1 - b01[1], lo, false);
        lo = __builtin_amdgcn_cvt_pk_fp8_f32(x2 - b23[0], x3 - b23[1], lo, true);
        qhi[nt][w] = hi;
        qlo[nt][w] = lo;
      }
    }
  }
  // FP8 math with per-token V scales: the unit the row's accumulator is kept in.  A step's P * v_scale is at most
  // (the step's largest P) * (the step's largest scale); the unit is that bound, unless the accumulator, decayed
  // by alpha like everything the row has seen, still needs a larger one:
  //     v_run <- max(vmx * exp2(step max - running max), v_run * alpha).
  // So P * v_scale / v_run never exceeds 1 and the step's own largest term is never far below it, whichever way
  // logits and scales drift against each other over a partition (a fixed unit, the running maximum of the scales,
  // loses a late token that carries the result through a large V scale but lies below an early token's logit).
  // Floored at 1e-30.
  float v_run[NT];
  float m_run[NT];      // running max of the scaled logits, log2 domain (-inf before the first visible key)
  float l_run[NT];      // this lane's share of the running sum of exp2(s - m)
  f32x4 acc[NT][8];     // O^T: acc[nt][db][r] is head dim 16*db + 4*kg + r of query row 16*nt + li
  auto reset_state = [&]() {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      v_run[nt] = 1e-30f;
      m_run[nt] = -INFINITY;
      l_run[nt] = 0.f;
#pragma unroll
      for (int db = 0; db < 8; ++db) acc[nt][db] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
  };
  reset_state();

  char* plds = &p_lds[wave][0][0];

  // ---- one step of 64 tokens ------------------------------------------------------------------------------
  // FULL: every token of the step is visible to every row and there is no ALiBi term.
  // PREFETCH: a next step exists; its K and V are requested as soon as this step's are consumed.
  auto step = [&]<bool FULL, bool PREFETCH>(SD& sd, int tok0, const Pages& pg_next) {
    // S^T tiles
    f32x4 s[NT][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) s[nt][j] = f32x4{0.f, 0.f, 0.f, 0.f};
      if constexpr (FP8MATH) {
        const i32x8 ka = {(int)sd.k[j][0][0], (int)sd.k[j][0][1], (int)sd.k[j][0][2], (int)sd.k[j][0][3],
                          (int)sd.k[j][1][0], (int)sd.k[j][1][1], (int)sd.k[j][1][2], (int)sd.k[j][1][3]};
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          s[nt][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ka, qhi[nt], s[nt][j], 0, 0, 0, 0, 0, 0);
          s[nt][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ka, qlo[nt], s[nt][j], 0, 0, 0, 0, 0, 0);
        }
      } else
#pragma unroll
      for (int ld = 0; ld < SD::NKL; ++ld) {
        Bf16x8Bits ka;
        ka.u = sd.k[j][ld];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          s[nt][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka.v, qreg[nt][ld], s[nt][j], 0, 0, 0);
      }
    }
    f32x4 ks_cur[PER_TOKEN ? 4 : 1];
    if constexpr (PER_TOKEN) {
#pragma unroll
      for (int j = 0; j < 4; ++j) ks_cur[j] = sd.ks[j];
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (PREFETCH) issue_k(sd, pg_next);
    __builtin_amdgcn_sched_barrier(0);

    // FP8 math, per-token V scales: P carries v_scale / v_run (<= 1); the row's accumulator is kept in units of v_run
    // FP8 math: P is produced already multiplied by pmul = 256 / v_run; log2(pmul) rides in the exponent's
    // additive term, so the factor costs nothing per element
    f32x4 vs_cur[(PER_TOKEN && FP8MATH) ? 4 : 1];
    float vmx = 0.f;  // the largest V scale of the step (the same in every lane)
    if constexpr (PER_TOKEN && FP8MATH) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        vs_cur[j] = sd.vs[j];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if constexpr (!FULL) {
            const int col = tok0 + 16 * j + 4 * kg + r;
            vs_cur[j][r] = col < ctx ? vs_cur[j][r] : 0.f;
          }
          vmx = fmaxf(vmx, vs_cur[j][r]);
        }
      }
      vmx = quad_row_max(vmx);
    }
    uint32_t ph[FP8MATH ? NT : 1][4], pl[FP8MATH ? NT : 1][4];  // FP8 math: P head / residual, 4 tokens per dword

#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const float rs = rscale[nt];
      float mx = -INFINITY;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          // FULL: the row's scale (>= 0 on this path) is applied inside the exponent's fma, and to the maximum once
          float v = s[nt][j][r];
          if constexpr (PER_TOKEN) v *= ks_cur[j][r];
          if constexpr (!FULL) {
            const int col = tok0 + 16 * j + 4 * kg + r;
            v = v * rs + slope2[nt] * (float)(col - ctx + 1);
            v = col < limit[nt] ? v : -INFINITY;
          }
          s[nt][j][r] = v;
          mx = fmaxf(mx, v);
        }
      }
      mx = quad_row_max(mx);
      if constexpr (FULL) mx *= rs;
      const float m_new = fmaxf(m_run[nt], mx);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      const float alpha = fast_exp2(m_run[nt] - m_safe);  // exp2(-inf) = 0 on the first visible step
      m_run[nt] = m_new;
      float alpha_acc = alpha, log2_pmul = FP8MATH ? 8.f : 0.f, inv_pmul = FP8MATH ? 1.f / 256.f : 1.f;
      if constexpr (PER_TOKEN && FP8MATH) {
        // the accumulator has just decayed by alpha: its unit may come down by as much, and no further
        const float v_old = v_run[nt] * alpha;
        const float v_step = vmx * fast_exp2(mx - m_safe);  // (0 for a row that sees no key of this step)
        const float v_new = fmaxf(fmaxf(v_step, v_old), 1e-30f);
        alpha_acc = v_new == v_old ? 1.f : v_old * __builtin_amdgcn_rcpf(v_new);  // <= 1
        log2_pmul = 8.f - __builtin_amdgcn_logf(v_new);
        inv_pmul = v_new * (1.f / 256.f);
        v_run[nt] = v_new;
      }
      const float e_add = log2_pmul - m_safe;
      const float e_mul = FULL ? rs : 1.f;
      float psum = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float p0 = fast_exp2(__builtin_fmaf(s[nt][j][0], e_mul, e_add));
        float p1 = fast_exp2(__builtin_fmaf(s[nt][j][1], e_mul, e_add));
        float p2 = fast_exp2(__builtin_fmaf(s[nt][j][2], e_mul, e_add));
        float p3 = fast_exp2(__builtin_fmaf(s[nt][j][3], e_mul, e_add));
        psum += (p0 + p1) + (p2 + p3);
        if constexpr (FP8MATH) {
          if constexpr (PER_TOKEN) {
            p0 *= vs_cur[j][0];
            p1 *= vs_cur[j][1];
            p2 *= vs_cur[j][2];
            p3 *= vs_cur[j][3];
          }
          // both halves of a packed word are written, so its previous value is irrelevant: a register whose
          // value is dead (a logit) stands in for it; an explicit zero would cost a move per word
          int hi = (int)__float_as_uint(s[nt][j][0]), lo = (int)__float_as_uint(s[nt][j][1]);
          hi = __builtin_amdgcn_cvt_pk_fp8_f32(p0, p1, hi, false);
          hi = __builtin_amdgcn_cvt_pk_fp8_f32(p2, p3, hi, true);
          const f32x2 b01 = __builtin_amdgcn_cvt_pk_f32_fp8(hi, false);
          const f32x2 b23 = __builtin_amdgcn_cvt_pk_f32_fp8(hi, true);
          lo = __builtin_amdgcn_cvt_pk_fp8_f32(p0 - b01[0], p1 - b01[1], lo, false);
          lo = __builtin_amdgcn_cvt_pk_fp8_f32(p2 - b23[0], p3 - b23[1], lo, true);
          ph[nt][j] = (uint32_t)hi;
          pl[nt][j] = (uint32_t)lo;
          continue;
        }
        if constexpr (PER_TOKEN) {
          // a masked token's scale may be stale memory (NaN): its weight must stay exactly 0
          f32x4 vsc = sd.vs[j];
          if constexpr (!FULL) {
#pragma unroll
            for (int r = 0; r < 4; ++r) vsc[r] = s[nt][j][r] == -INFINITY ? 0.f : vsc[r];
          }
          p0 *= vsc[0];
          p1 *= vsc[1];
          p2 *= vsc[2];
          p3 *= vsc[3];
        }
        u32x2 pk;
        pk[0] = pack_bf16x2(p0, p1);
        pk[1] = pack_bf16x2(p2, p3);
        *reinterpret_cast<u32x2*>(plds + nt * (16 * kPRowBytes) + li * kPRowBytes + (16 * j + 4 * kg) * 2) = pk;
      }
      l_run[nt] = l_run[nt] * alpha + psum * inv_pmul;
#pragma unroll
      for (int db = 0; db < 8; ++db) acc[nt][db] *= alpha_acc;
    }

    if constexpr (!FULL) {
      // zero the V bytes of tokens at or beyond ctx (stale cache contents may decode to NaN)
      int nvalid = ctx - (tok0 + 16 * kg);
      nvalid = nvalid < 0 ? 0 : (nvalid > 16 ? 16 : nvalid);
#pragma unroll
      for (int db = 0; db < 8; ++db) {
        if constexpr (kFp8) {
          sd.v[db][0] = keep_first_bytes(sd.v[db][0], nvalid);
        } else {
          sd.v[db][0] = keep_first_bytes(sd.v[db][0], 2 * (nvalid > 8 ? 8 : nvalid));
          sd.v[db][1] = keep_first_bytes(sd.v[db][1], 2 * (nvalid > 8 ? nvalid - 8 : 0));
        }
      }
    }

    if constexpr (FP8MATH) {
      // lane group kg holds, per tile j, tokens 4kg..4kg+3; the B operand of O^T += V^T P^T wants lane
      // group kg to hold all 16 tokens of tile kg: a 4x4 transpose over (lane group, register)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        quad_transpose(ph[nt]);
        quad_transpose(pl[nt]);
      }
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
        for (int db = 0; db < 8; ++db) {
          const long va = (long)(((uint64_t)sd.v[db][0][2 * hf + 1] << 32) | sd.v[db][0][2 * hf]);
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) {
            const long bh = (long)(((uint64_t)ph[nt][2 * hf + 1] << 32) | ph[nt][2 * hf]);
            const long bl = (long)(((uint64_t)pl[nt][2 * hf + 1] << 32) | pl[nt][2 * hf]);
            acc[nt][db] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(va, bh, acc[nt][db], 0, 0, 0);
            acc[nt][db] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(va, bl, acc[nt][db], 0, 0, 0);
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (PREFETCH) issue_v(sd, pg_next);
      __builtin_amdgcn_sched_barrier(0);
      return;
    }

    // the P tile is written and read by this wave only; LDS operations of one wave complete in order
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // O^T += V^T P^T
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      bf16x8 pb[NT];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        Bf16x8Bits t;
        t.u = *reinterpret_cast<const u32x4*>(plds + nt * (16 * kPRowBytes) + li * kPRowBytes +
                                              (16 * kg + 8 * hf) * 2);
        pb[nt] = t.v;
      }
#pragma unroll
      for (int db = 0; db < 8; ++db) {
        Bf16x8Bits va;
        va.u = sd.v[db][hf];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          acc[nt][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va.v, pb[nt], acc[nt][db], 0, 0, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (PREFETCH) issue_v(sd, pg_next);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  };

  // ---- main loop -------------------------------------------------------------------------------------------
  // the unmasked variant of the step scales the row maximum after taking it: only right for scales >= 0
  bool rs_neg = false;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) rs_neg = rs_neg || rscale[nt] < 0.f;
  // leading steps of this wave that need no masking: part_start + i * stride + 64 <= min_limit
  int n_full = 0;
  if (!has_alibi && __builtin_amdgcn_ballot_w64(rs_neg) == 0 && min_limit - part_start >= kStepTokens)
    n_full = (min_limit - part_start - kStepTokens) / kWaveStride + 1;
  int sidx = 0;
  int tok0 = part_start;
  // SPAN: the partition being accumulated, and the steps left in it; at the boundary its partial result is
  // set aside in LDS and the running state starts again (the page stream does not notice)
  int part_cur = part;
  const int steps_per_part = a.partition_size / kStepTokens;
  int steps_left_in_part = steps_per_part;
  auto cross_boundary = [&]() {
    if constexpr (kSpanCapable) {
      if (span > 1 && --steps_left_in_part == 0) {
        // (the one-wave epilogue below, up to the staging in LDS, for a partition that is not the workgroup's last)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          const float acc_unit = FP8MATH ? (PER_TOKEN ? v_run[nt] : 1.f) * (1.f / 256.f) : 1.f;
          char* slot = span_pool + ((part_cur - part) * NT + nt) * span_slot_bytes;
          float l_tot = quad_row_sum(l_run[nt]);
          float m_out = m_run[nt];
          if (row0 + 16 * nt + li >= rows_valid) {  // padding rows of a ragged batch: no visible key
            l_tot = 0.f;
            m_out = -INFINITY;
          }
          const float inv = l_tot > 0.f ? v_tensor_scale * acc_unit / l_tot : 0.f;
          if (kg == 0) {
            reinterpret_cast<float*>(slot + span_rows * kORowBytes)[li] = m_out * (1.0f / kLog2e);
            reinterpret_cast<float*>(slot + span_rows * kORowBytes)[16 + li] = l_tot;
          }
          stage_partial_tile(slot, acc[nt], inv, lane, span_rows);
        }
        reset_state();
        ++part_cur;
        steps_left_in_part = steps_per_part;
      }
    }
  };
  if (active) {
    const int n_fast = n_full < n_steps - 1 ? n_full : n_steps - 1;
    Pages pg_next = load_pages(part_start + kWaveStride);
    for (; sidx < n_fast; ++sidx) {
      // Waves that share a SIMD do not progress evenly by themselves (the older one wins every
      // arbitration and finishes a third earlier, leaving the SIMD half empty at the end): the further a
      // wave is from its end, the higher its issue priority.
      {
        const int rem4 = (n_steps - sidx) * 4 / n_steps;
        if (rem4 >= 3)
          __builtin_amdgcn_s_setprio(3);
        else if (rem4 == 2)
          __builtin_amdgcn_s_setprio(2);
        else if (rem4 == 1)
          __builtin_amdgcn_s_setprio(1);
        else
          __builtin_amdgcn_s_setprio(0);
      }
      const Pages pg_after = load_pages(tok0 + 2 * kWaveStride);
      step.template operator()<true, true>(buf_a, tok0, pg_next);
      pg_next = pg_after;
      tok0 += kWaveStride;
      cross_boundary();
    }
    for (; sidx < n_steps - 1; ++sidx) {
      const Pages pg_after = load_pages(tok0 + 2 * kWaveStride);
      step.template operator()<false, true>(buf_a, tok0, pg_next);
      pg_next = pg_after;
      tok0 += kWaveStride;
      cross_boundary();
    }
    if (n_full >= n_steps)
      step.template operator()<true, false>(buf_a, tok0, pg_next);
    else
      step.template operator()<false, false>(buf_a, tok0, pg_next);
  }
  // ---- epilogue ------------------------------------------------------------------------------------------------
  // max_logits holds the maximum of the scaled logits in the natural-log domain, exp_sums the
  // un-normalised sum, tmp_output the normalised bf16 partial.  For a sequence that fits in one partition the
  // partial is the result, and it is written to output as well.
  const int64_t es_off = (int64_t)b * a.stride_es_s + (int64_t)h * a.stride_es_h + (int64_t)part_cur * a.stride_es_p;
  char* tmp = (char*)a.tmp_output + ((int64_t)b * a.stride_tmp_s + (int64_t)h * a.stride_tmp_h +
                                     (int64_t)part_cur * a.stride_tmp_p) * 2;
  // a sequence with one partition needs no merge: its partial is the result.  (With a partition axis of length
  // 1 every sequence has one: a context longer than the partition is cut off at its end, as the partition axis
  // cuts off longer contexts for any other length.)
  const bool direct = (ctx <= a.partition_size || a.max_num_partitions == 1) && a.output != nullptr && a.sinks == nullptr;
  char* outp = (char*)a.output + ((int64_t)b * a.stride_out_s + (int64_t)h * Ge * a.stride_out_h) * 2;
  // PA_DECODE_FLAG_OUTPUT_ONLY: rows beyond the sequence's query length are nobody's, and a sequence finished here
  // leaves no partition-buffer entries
  const bool output_only = a.flags & kFlagOutputOnly;
  const bool no_partial = output_only && direct;
  const int rows_live = output_only ? rows_valid : Ge;
  float l_tot[NT], acc_unit[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    acc_unit[nt] = FP8MATH ? (PER_TOKEN ? v_run[nt] : 1.f) * (1.f / 256.f) : 1.f;
    l_tot[nt] = quad_row_sum(l_run[nt]);
    if (row0 + 16 * nt + li >= rows_valid) {  // padding rows of a ragged batch: no visible key
      l_tot[nt] = 0.f;
      m_run[nt] = -INFINITY;
    }
  }
  if constexpr (WAVES == 1) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int row = row0 + 16 * nt + li;
      const float inv = l_tot[nt] > 0.f ? v_tensor_scale * acc_unit[nt] / l_tot[nt] : 0.f;
      if (row < rows_live && kg == 0 && !no_partial) {
        a.max_logits[es_off + row] = m_run[nt] * (1.0f / kLog2e);
        a.exp_sums[es_off + row] = l_tot[nt];
      }
      if constexpr (TEAM) {  // (the team's merge reads every partition's maximum and sum from the staging pools)
        if (kg == 0) {
          float* ml = reinterpret_cast<float*>(span_pool + ((part_cur - part) * NT + nt) * span_slot_bytes + span_rows * kORowBytes);
          ml[li] = m_run[nt] * (1.0f / kLog2e);
          ml[16 + li] = l_tot[nt];
        }
      }
      // (one-wave workgroups stage the last partition's tile in the next free slot of the pool)
      char* stage_at = kSpanCapable ? span_pool + ((part_cur - part) * NT + nt) * span_slot_bytes : &o_lds[0][0];
      char* out_tile = outp + (int64_t)(row0 + 16 * nt) * a.stride_out_h * 2;
      if (no_partial)
        store_partial_tile(stage_at, acc[nt], inv, out_tile, a.stride_out_h * 2, nullptr, 0, rows_live - row0 - 16 * nt,
                           lane, kSpanCapable ? span_rows : 16);
      else
        store_partial_tile(stage_at, acc[nt], inv, tmp + (int64_t)(row0 + 16 * nt) * a.stride_tmp_g * 2,
                           a.stride_tmp_g * 2, direct ? out_tile : nullptr, a.stride_out_h * 2, rows_live - row0 - 16 * nt,
                           lane, kSpanCapable ? span_rows : 16);
    }
  } else {
    // merge the waves' (m, l, O): every wave holds the same (row, head dim) in the same lane and register,
    // so the merge is lane-wise; wave w merges head-dim blocks [w*8/WAVES, (w+1)*8/WAVES)
    __shared__ float mg_m[WAVES][NT * 16];
    __shared__ float mg_l[WAVES][NT * 16];
    __shared__ f32x4 mg_acc[WAVES][NT][8][64];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      if (kg == 0) {
        mg_m[wave][16 * nt + li] = m_run[nt];
        mg_l[wave][16 * nt + li] = l_tot[nt];
      }
#pragma unroll
      for (int db = 0; db < 8; ++db) mg_acc[wave][nt][db][lane] = acc[nt][db] * acc_unit[nt];
    }
    __syncthreads();
    constexpr int DBW = 8 / WAVES;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int lrow = 16 * nt + li;
      const int row = row0 + lrow;
      float M = -INFINITY;
#pragma unroll
      for (int w2 = 0; w2 < WAVES; ++w2) M = fmaxf(M, mg_m[w2][lrow]);
      const float M_safe = M == -INFINITY ? 0.f : M;
      float e[WAVES];
      float L = 0.f;
#pragma unroll
      for (int w2 = 0; w2 < WAVES; ++w2) {
        e[w2] = fast_exp2(mg_m[w2][lrow] - M_safe);
        L += mg_l[w2][lrow] * e[w2];
      }
      const float inv = L > 0.f ? v_tensor_scale / L : 0.f;
#pragma unroll
      for (int d = 0; d < DBW; ++d) {
        const int db = wave * DBW + d;
        f32x4 o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w2 = 0; w2 < WAVES; ++w2) o += mg_acc[w2][nt][db][lane] * e[w2];
        o *= inv;
        u32x2 pk;
        pk[0] = pack_bf16x2(o[0], o[1]);
        pk[1] = pack_bf16x2(o[2], o[3]);
        *reinterpret_cast<u32x2*>(&o_lds[0][0] + li * kORowBytes + (16 * db + 4 * kg) * 2) = pk;
      }
      if (wave == 0 && kg == 0 && row < rows_live && !no_partial) {
        a.max_logits[es_off + row] = M * (1.0f / kLog2e);
        a.exp_sums[es_off + row] = L;
      }
      __syncthreads();
      for (int i = wave; i < 4; i += WAVES) {
        const int r = 4 * i + kg;
        const u32x4 v = *reinterpret_cast<const u32x4*>(&o_lds[0][0] + r * kORowBytes + li * 16);
        if (r < rows_live - row0 - 16 * nt) {
          if (!no_partial) *reinterpret_cast<u32x4*>(tmp + (int64_t)(row0 + 16 * nt + r) * a.stride_tmp_g * 2 + li * 16) = v;
          if (direct)
            *reinterpret_cast<u32x4*>(outp + (int64_t)(row0 + 16 * nt + r) * a.stride_out_h * 2 + li * 16) = v;
        }
      }
      if (nt + 1 < NT) __syncthreads();
    }
  }
  if constexpr (kSpanCapable) {
    // SPAN: the partitions left behind on the way (a sequence that crosses a boundary has more than one
    // partition: nothing of it goes to `output` directly)
    for (int pc = part; pc < part_cur; ++pc) {
      const int64_t eo = (int64_t)b * a.stride_es_s + (int64_t)h * a.stride_es_h + (int64_t)pc * a.stride_es_p;
      char* tp = (char*)a.tmp_output + ((int64_t)b * a.stride_tmp_s + (int64_t)h * a.stride_tmp_h +
                                        (int64_t)pc * a.stride_tmp_p) * 2;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const char* slot = span_pool + ((pc - part) * NT + nt) * span_slot_bytes;
        const int row = row0 + 16 * nt + li;
        if (row < rows_live && kg == 0) {
          a.max_logits[eo + row] = reinterpret_cast<const float*>(slot + span_rows * kORowBytes)[li];
          a.exp_sums[eo + row] = reinterpret_cast<const float*>(slot + span_rows * kORowBytes)[16 + li];
        }
        copy_staged_tile(slot, tp + (int64_t)(row0 + 16 * nt) * a.stride_tmp_g * 2, a.stride_tmp_g * 2, nullptr, 0,
                         rows_live - row0 - 16 * nt, lane);
      }
    }
  }
  if constexpr (QUEUE) {
    // rows of padding query positions beyond the last real tile: this workgroup fills them
    if (rt == tiles_b - 1 && wave == 0 && !output_only) {
      for (int r = 16 * NT * tiles_b + kg; r < Ge; r += 4) {
        if (li == 0) {
          a.max_logits[es_off + r] = -INFINITY;
          a.exp_sums[es_off + r] = 0.f;
        }
        *reinterpret_cast<u32x4*>(tmp + (int64_t)r * a.stride_tmp_g * 2 + li * 16) = u32x4{0, 0, 0, 0};
        if (direct) *reinterpret_cast<u32x4*>(outp + (int64_t)r * a.stride_out_h * 2 + li * 16) = u32x4{0, 0, 0, 0};
      }
    }
  }
  } while (0);
  if constexpr (TEAM) {
    // ---- the team's merge: every partial result of the sequence is staged in this workgroup's LDS ---------------
    // (the sequence's lengths again: a wave without a partition has not read them; asked for ahead of the barrier)
    const int ctx_t = sload_i32(a.context_lens + b);
    const int qb_t = a.q_lens ? sload_i32(a.q_lens + b) : a.q_len;
    int n_live = (ctx_t + a.partition_size - 1) / a.partition_size;
    n_live = n_live > P ? P : n_live;
    __syncthreads();
    const int rows_valid_t = n_live > 0 ? qb_t * a.group_size : 0;
    const bool output_only_t = a.flags & kFlagOutputOnly;
    // (a sequence of one partition got its rows from the wave that finished it; with attention sinks or without an
    // output the launch layer does not form teams)
    const bool finished = n_live == 1 && ctx_t > 0;
    char* outp_t = (char*)a.output + ((int64_t)b * a.stride_out_s + (int64_t)h * Ge * a.stride_out_h) * 2;
    if (!finished) {
      // A half-wave per row (lane: four head dims), two rows of the tile per wave and pass.  Every lane takes the
      // row's maximum over the partitions, then adds up its four dims with the partitions' weights (the maxima and
      // sums are LDS broadcasts: no lane exchanges, and the reads of an unrolled group are independent).
      const int half = lane >> 5, hl = lane & 31;
      const int rows_here = Ge - row0 < 16 ? Ge - row0 : 16;  // rows of this tile that the buffers hold
      for (int r0 = 2 * team_wave; r0 < rows_here; r0 += 2 * kTeamWaves) {
        const int r = r0 + half;
        const bool in_buf = r < rows_here;
        const bool live = in_buf && row0 + r < rows_valid_t;
        const int r_read = in_buf ? r : r0;  // (a row the pools hold)
        // (wave w2's partitions are the slots of pool w2, in order: no division by the run-time span)
        // Straight-line groups of four partitions: the LDS reads of a group are all requested before the first is
        // used (an index past the pool's last live slot is clamped and its weight set to zero).
        float M = -INFINITY;
        for (int w2 = 0, p0 = 0; w2 < kTeamWaves && p0 < n_live; ++w2, p0 += span) {
          const int cnt = n_live - p0 < span ? n_live - p0 : span;
          const char* ml0 = &span_lds[0] + w2 * (NT * kSpanPoolBytes) + span_rows * kORowBytes + r_read * 4;
          for (int j2 = 0; j2 < cnt; j2 += 4) {
            float mp[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              const int jj = j2 + u < cnt ? j2 + u : cnt - 1;
              mp[u] = *reinterpret_cast<const float*>(ml0 + jj * span_slot_bytes);
            }
            M = fmaxf(fmaxf(M, fmaxf(mp[0], mp[1])), fmaxf(mp[2], mp[3]));
          }
        }
        const float M_safe = M == -INFINITY ? 0.f : M;
        float L = 0.f;
        float o[4] = {0.f, 0.f, 0.f, 0.f};
        for (int w2 = 0, p0 = 0; w2 < kTeamWaves && p0 < n_live; ++w2, p0 += span) {
          const int cnt = n_live - p0 < span ? n_live - p0 : span;
          const char* pool = &span_lds[0] + w2 * (NT * kSpanPoolBytes);
          for (int j2 = 0; j2 < cnt; j2 += 4) {
            float lp[4], mp[4];
            u32x2 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              const int jj = j2 + u < cnt ? j2 + u : cnt - 1;
              const char* slot = pool + jj * span_slot_bytes;
              const float* ml = reinterpret_cast<const float*>(slot + span_rows * kORowBytes);
              lp[u] = ml[16 + r_read];
              mp[u] = ml[r_read];
              v[u] = *reinterpret_cast<const u32x2*>(slot + r_read * kORowBytes + hl * 8);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              // (a sum of zero comes with a maximum of -inf: weight zero; such a partition's rows may hold anything)
              float wp = lp[u] * __expf(mp[u] - M_safe);
              wp = j2 + u < cnt ? wp : 0.f;
              const uint32_t keep = wp != 0.f ? 0xffffffffu : 0u;
              const uint32_t v0 = v[u][0] & keep, v1 = v[u][1] & keep;
              L += wp;
              o[0] = fmaf(wp, bf16_bits_to_f32(v0 & 0xffffu), o[0]);
              o[1] = fmaf(wp, __uint_as_float(v0 & 0xffff0000u), o[1]);
              o[2] = fmaf(wp, bf16_bits_to_f32(v1 & 0xffffu), o[2]);
              o[3] = fmaf(wp, __uint_as_float(v1 & 0xffff0000u), o[3]);
            }
          }
        }
        const float inv = L > 0.f ? 1.f / L : 0.f;
#pragma unroll
        for (int i2 = 0; i2 < 4; ++i2) o[i2] *= inv;
        if (in_buf) {
          u32x2* dst = reinterpret_cast<u32x2*>(outp_t + (int64_t)(row0 + r) * a.stride_out_h * 2 + hl * 8);
          if (live)
            *dst = u32x2{pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3])};
          else if (!output_only_t || n_live <= 0)
            *dst = u32x2{0u, 0u};  // padding rows (and every row of an empty sequence) read as zero
        }
      }
    }
  }
  if constexpr (!QUEUE) break;
  }  // for (;;)
  if constexpr (QUEUE) {
    // the last workgroup out leaves the workspace as it found it: zero
    if (threadIdx.x == 0) {
      __threadfence();
      if (atomicAdd(a.workspace + 1, 1) == (int)gridDim.x - 1) {
        a.workspace[0] = 0;
        a.workspace[1] = 0;
      }
    }
  }
}

}  // namespace

#endif  // PA_PARTITION_KERNEL_H_
