// pa_partition_shared_kernel: stage 1 for 17..64 query rows per kv head over an FP8 cache.
#ifndef PA_PARTITION_SHARED_KERNEL_H_
#define PA_PARTITION_SHARED_KERNEL_H_

#include "pa_common.h"

namespace {

// ---------------------------------------------------------------------------------------------
// Partition kernel for more than 16 query rows per kv head (large GQA groups, MTP) over an FP8 cache.
// The up to four 16-row query tiles of one (sequence, kv head, partition) are the four waves of ONE
// workgroup and share a single pass over the pages.  Of every 64-token step wave w fetches tile w (K 2 KiB,
// V 2 KiB, the tile's per-token scales) straight from global memory into LDS (global_load_lds, no
// registers), laid out in exactly the per-lane operand order of the MFMAs; after a workgroup barrier every
// wave reads the whole step back with lane-contiguous 16-byte LDS reads and runs the step's arithmetic for
// its own 16 rows.  LDS holds a ring of NB steps: NB-1 travel from HBM while one is multiplied; one barrier
// per step.  Against one workgroup per row tile this reads every page once instead of once per tile (the
// repeats hit the L2, but each costs a full trip through the vector memory path) and sets an item up once.
//
// The asynchronous loads are invisible to the compiler, which therefore inserts no waits for them: the wave
// that issued them waits with dma_wait<n>() before the barrier.  Nothing inside the step loop may use
// scratch memory (a spill, an indexed private array): the compiler would wait for such a load with
// vmcnt(0) and drain the ring.
// ---------------------------------------------------------------------------------------------
struct StepLds {
  u32x4 k[4][2][64];  // [tile][load][lane]: the K operand of a tile as its two loads deliver it
  u32x4 v[4][128];    // [tile][head dim]: 16 tokens of one head dim
  float sc[4][2][16]; // [tile][K scales, V scales][token]
};

template <bool PER_TOKEN, bool BS16, int NB, int OCC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(OCC, OCC)))
void pa_partition_shared_kernel(const PaDecodeArgs a) {
  __shared__ __attribute__((aligned(16))) StepLds stage[NB];  // ring of steps: NB-1 in flight, one being read
  static_assert(sizeof(StepLds) * NB >= 4 * 16 * kORowBytes, "the output tiles reuse the stage buffers");
  static_assert(sizeof(StepLds) * NB <= 65536, "the LDS address of an asynchronous load travels in 16 bits of M0");
  constexpr int kLoadsPerStep = PER_TOKEN ? 5 : 4;  // vector memory operations one wave issues per step

  PA_TRACE_DECL;
  PA_TRACE_MARK(0);  // entry
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int li = lane & 15;
  const int kg = lane >> 4;

  // ---- which (sequence, head, partition): workgroup-uniform; head fastest, partition slowest ----------
  const int Hkv = a.num_kv_heads;
  const int G = a.group_size;
  const int Ge = a.q_len * G;
  // (32-bit unsigned arithmetic: the grid has fewer than 2^31 workgroups, and a 64-bit division by a run-time value
  // is a hundred instructions in front of the workgroup's first request)
  const uint32_t wid = blockIdx.x;
  int h;
  uint32_t item;
  if (a.flags & kFlagHeadsShareXcd) {
    // Workgroup ids go round the eight XCDs.  With the head fastest in the id, the kv heads of an item land on
    // eight different XCDs and each fetches the 128-byte lines that hold its own 64 bytes of per-token scales of a
    // page AND its neighbour's; here an XCD takes every eighth item with all its heads one after the other, so the
    // heads' scale lines (and nothing else: K and V are disjoint) meet in one L2.
    const uint32_t xcd = wid & 7u;
    const uint32_t slot = wid >> 3;
    h = (int)(slot % (uint32_t)Hkv);
    item = (slot / (uint32_t)Hkv) * 8u + xcd;
  } else {
    h = (int)(wid % (uint32_t)Hkv);
    item = wid / (uint32_t)Hkv;
  }
  int b, part;
  if (a.flags & kFlagSortedItems) {
    // the planning kernel has listed the live (sequence, partition) items, longest last partitions first
    // (the number of listed items and this item's record are requested together: the list area is sized for every
    // (sequence, partition) pair, and the grid's padding items read the last record)
    const uint32_t pairs = (uint32_t)a.num_seqs * (uint32_t)a.max_num_partitions;
    const int64_t rec = item < pairs ? item : pairs - 1;
    const int listed = sload_i32(a.workspace + 2);
    b = sload_i32(a.workspace + kPlanHeaderWords + 2 * rec);
    part = sload_i32(a.workspace + kPlanHeaderWords + 2 * rec + 1);
    if (item >= (uint32_t)listed) return;
  } else {
    if (item >= (uint32_t)a.num_seqs * (uint32_t)a.max_num_partitions) return;  // (the grid is whole groups of eight items)
    b = (int)(item % (uint32_t)a.num_seqs);
    part = (int)(item / (uint32_t)a.num_seqs);
    // (items go to the XCDs round robin: with a batch that is a multiple of eight every partition of a sequence
    // would sit on the same XCD, and a batch's one long sequence on one eighth of the GPU; each partition index
    // therefore starts the batch one sequence further on)
    if (a.flags & kFlagHeadsShareXcd) b = (b + part % a.num_seqs) % a.num_seqs;
  }

  // The block-table entries of this wave's tile of the first NB-1 steps are requested together with the context
  // length, not after it (every dependent scalar load is a round trip under full memory load, and three of them in
  // a row were 4 us before a workgroup's first request went out).  They are entries of this sequence's row (the
  // index is kept inside the row); one that lies beyond the sequence's end is read but never used.
  const int log2_bs = 31 - __builtin_clz(a.block_size);
  const int* bt = a.block_tables + (int64_t)b * a.stride_bt_s;
  int early_page[NB - 1];
#pragma unroll
  for (int i = 0; i < NB - 1; ++i) {
    int idx = (part * a.partition_size + i * kStepTokens + 16 * wave) >> log2_bs;
    idx = idx < (int)a.stride_bt_s ? idx : (int)a.stride_bt_s - 1;  // (stride_bt_s >= 1: checked by the launch layer)
    early_page[i] = sload_i32(bt + idx);
  }
  const int ctx = sload_i32(a.context_lens + b);
  const int wg_start = part * a.partition_size;
  if (wg_start >= ctx) {
    if (ctx <= 0 && part == 0) zero_output_rows(a, b, h, 0, Ge);
    return;
  }
  const int wg_end = min(wg_start + a.partition_size, ctx);
  const int n_steps = (wg_end - wg_start + kStepTokens - 1) / kStepTokens;
  const int qb = a.q_lens ? sload_i32(a.q_lens + b) : a.q_len;
  const int rows_valid = qb * G;
  // The waves of a workgroup are spread over the CU's four SIMDs, and in a ragged batch tile 0 is always busy
  // while tile 3 rarely is: which wave computes which tile rotates from workgroup to workgroup, so that no
  // SIMD collects the busy tiles of every resident workgroup (worth ~3 % on ragged query lengths).  Which
  // wave fetches which quarter of a step does not rotate.
  // With at most two busy tiles (32 query rows) two of the four waves would only fetch, and a busy wave's chain of
  // 64 tokens' logits, softmax and P per step is what the step waits for.  Then each tile is shared by TWO waves
  // that take half of every step's tokens each (tiles 0-1 and 2-3 of the step), with (m, l, O) of their own, merged
  // through LDS at the end: half the chain per wave, all four waves busy (measured on 32 rows: 104 -> 95 us with
  // per-token scales, 94 -> 85 us without).
  const int role = (wave + b + h + part) & 3;
  const bool half_mode = rows_valid <= 32;
  const int half = half_mode ? role >> 1 : 0;             // which half of every step's tokens this wave takes
  const int row0 = 16 * (half_mode ? role & 1 : role);    // this wave's query tile
  const bool has_rows = row0 < rows_valid;  // else the wave only helps to fetch

  // ---- cache addressing ----------------------------------------------------------------------------------
  const int bs_mask = a.block_size - 1;
  const char* kbase = (const char*)a.key_cache + (int64_t)h * a.stride_k_h;
  const char* vbase = (const char*)a.value_cache + (int64_t)h * a.stride_v_h;
  const int64_t k_block_bytes = a.stride_k_b;
  const int64_t v_block_bytes = a.stride_v_b;
  const float* ksbase = PER_TOKEN ? a.key_scale + (int64_t)h * a.stride_kvscale_h : nullptr;
  const float* vsbase = PER_TOKEN ? a.value_scale + (int64_t)h * a.stride_kvscale_h : nullptr;
  const uint32_t k_chunk_bytes = BS16 ? 256u : (uint32_t)a.stride_k_c;
  uint32_t k_lane_off[2];
#pragma unroll
  for (int ld = 0; ld < 2; ++ld) k_lane_off[ld] = (uint32_t)(kg * k_chunk_bytes + li * 16) + 4 * ld * k_chunk_bytes;
  const bool vt = a.v_transposed;
  const bool v_whole_lines = a.v_transposed || a.block_size <= 64;
  const uint32_t v_row_bytes = BS16 ? 16u : (vt ? 16u : (uint32_t)a.stride_v_2);
  const int64_t v_tile_bytes = BS16 ? 16 : (vt ? a.stride_v_2 : 16);
  uint32_t v_lane_off[2];  // V loads: lane = head dim (0..63, 64..127) of one tile
#pragma unroll
  for (int i = 0; i < 2; ++i) v_lane_off[i] = (uint32_t)(lane + 64 * i) * v_row_bytes;
  const float* sc_lane = PER_TOKEN ? ((lane & 16) ? vsbase : ksbase) + li : nullptr;

  const int last_tile_tok = (wg_end - 1) & ~15;
  // wave w fetches tile w of every step: its page id (a scalar load) and the tile's token offset inside the
  // page.  Tiles past the last live one repeat it, so no block-table slot or page beyond the sequence is touched.
  struct TilePage {
    int page;
    int off;
  };
  auto load_page = [&](int tok0) {
    int t = tok0 + 16 * wave;
    t = t > last_tile_tok ? last_tile_tok : t;
    TilePage tp;
    tp.page = sload_i32(bt + (t >> log2_bs));
    tp.off = t & bs_mask;
    return tp;
  };
  // this wave's quarter of the step whose page ids are pg, sent to ring slot `slot`
  const uint32_t stage_base = lds_offset_of(&stage[0]);
  auto fetch = [&](int slot, const TilePage& tp) {
    const uint32_t st = stage_base + (uint32_t)slot * (uint32_t)sizeof(StepLds);
    // every address is a wave-uniform base plus a per-lane constant
    const int page = tp.page;
    const int off = tp.off;
    const char* kt = kbase + (int64_t)page * k_block_bytes + (int64_t)off * 16;
    const uint32_t kdst = st + (uint32_t)offsetof(StepLds, k) + (uint32_t)wave * 2048u;
    dma_load16(kt, k_lane_off[0], kdst);
    dma_load16(kt, k_lane_off[1], kdst + 1024u);
    const char* vt_ = vbase + (int64_t)page * v_block_bytes + (int64_t)(off >> 4) * v_tile_bytes;
    const uint32_t vdst = st + (uint32_t)offsetof(StepLds, v) + (uint32_t)wave * 2048u;
    // non-temporal where a load covers whole 128-byte lines; plain V in pages of more than 64 tokens gives a
    // step half a line of every head dim's row, and the other half must still be in L2 for the next step
    if (BS16 || v_whole_lines) {
      dma_load16<true>(vt_, v_lane_off[0], vdst);            // head dims 0..63 (lane = dim)
      dma_load16<true>(vt_, v_lane_off[1], vdst + 1024u);    // head dims 64..127
    } else {
      dma_load16<false>(vt_, v_lane_off[0], vdst);
      dma_load16<false>(vt_, v_lane_off[1], vdst + 1024u);
    }
    if constexpr (PER_TOKEN) {
      // lanes 0-15: the K scales of the tile's 16 tokens, lanes 16-31: the V scales
      // (ordinary loads: the other half of the line belongs to the neighbouring head, whose workgroup runs beside
      // this one on the same XCD)
      if (lane < 32)
        dma_load4<false>(sc_lane + ((int64_t)page * a.stride_kvscale_b + off),
                  st + (uint32_t)offsetof(StepLds, sc) + (uint32_t)wave * 128u);
    }
  };

  // ---- the first NB-1 steps go out before anything else is set up ----------------------------------------------
  int fetch_tok = wg_start;
#pragma unroll
  for (int i = 0; i < NB - 1; ++i) {
    if (i < n_steps) {
      const int t = fetch_tok + 16 * wave;
      TilePage tp;
      if (t <= last_tile_tok) {  // (the early request was for this tile)
        tp.page = early_page[i];
        tp.off = t & bs_mask;
      } else {
        tp = load_page(fetch_tok);
      }
      fetch(i, tp);
      fetch_tok += kStepTokens;
    }
  }
  TilePage pg_next = load_page(fetch_tok);  // of the next step to fetch

  PA_TRACE_MARK(1);  // the first steps are requested
  // ---- buffers of this item ---------------------------------------------------------------------------------
  const int64_t es_off = (int64_t)b * a.stride_es_s + (int64_t)h * a.stride_es_h + (int64_t)part * a.stride_es_p;
  char* tmp = (char*)a.tmp_output + ((int64_t)b * a.stride_tmp_s + (int64_t)h * a.stride_tmp_h +
                                     (int64_t)part * a.stride_tmp_p) * 2;
  const bool direct = (ctx <= a.partition_size || a.max_num_partitions == 1) && a.output != nullptr && a.sinks == nullptr;
  char* outp = (char*)a.output + ((int64_t)b * a.stride_out_s + (int64_t)h * Ge * a.stride_out_h) * 2;
  // ---- per-lane row bookkeeping ---------------------------------------------------------------------------------
  const bool has_alibi = a.alibi_slopes != nullptr;
  const int row = row0 + li;
  const bool row_ok = row < rows_valid;
  const int t_row = row / G;
  const int limit = row_ok ? ctx - (qb - 1 - t_row) : 0;  // number of visible keys of this lane's query row
  float slope2 = 0.f;
  // one slope per packed row (the reference kernels' indexing) or one per query head, shared by its new tokens
  if (has_alibi && row_ok)
    slope2 = a.alibi_slopes[a.alibi_slopes_len == Hkv * Ge ? h * Ge + row : h * G + (row - t_row * G)] * kLog2e;
  const int min_limit = ctx - (qb - 1);

  // ---- query: q * cq = hi + lo in e4m3, cq a power of two (exact), the B operand of S^T = K Q^T ---------
  float k_tensor_scale = 1.f, v_tensor_scale = 1.f;
  if (a.kv_quant_mode == PA_QUANT_PER_TENSOR) {
    k_tensor_scale = sload_f32(a.key_scale);
    v_tensor_scale = sload_f32(a.value_scale);
  }
  float rscale = a.softmax_scale * k_tensor_scale * kLog2e;
  if (a.query_quant_mode == PA_QUANT_PER_TENSOR) rscale *= sload_f32(a.query_scale);
  if (a.query_quant_mode == PA_QUANT_PER_TOKEN && row_ok)
    rscale *= a.query_scale[(int64_t)b * a.stride_qscale_s + h * Ge + row];
  i32x8 qhi, qlo;
  // an FP8 query times a power of two is its own FP8 head: the residual is zero and its MFMAs are skipped
  const bool q_has_residual = a.query_dtype == PA_DTYPE_BF16;
  {
    const char* q_ptr = (const char*)a.query;
    const int64_t e0 = (int64_t)b * a.stride_q_s + (int64_t)(h * Ge + (row_ok ? row : 0)) * a.stride_q_h;
    // the four loads of a row's 32 elements go out together (one choice of the query's type around them, not one
    // inside each: the compiler would wait for every load before it issues the next)
    u32x4 raw[4];
    const bool q_bf16 = a.query_dtype == PA_DTYPE_BF16;
    if (q_bf16) {
#pragma unroll
      for (int s = 0; s < 4; ++s) raw[s] = load16(q_ptr + (e0 + 64 * (s >> 1) + 16 * kg + 8 * (s & 1)) * 2);
    } else {
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const u32x2 r8 = *reinterpret_cast<const u32x2*>(q_ptr + e0 + 64 * (s >> 1) + 16 * kg + 8 * (s & 1));
        raw[s] = u32x4{r8[0], r8[1], 0, 0};
      }
    }
    float f[32];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      Bf16x8Bits q;
      q.u = raw[s];
      if (!q_bf16) q.v = fp8x8_to_bf16x8(raw[s][0], raw[s][1]);
      if (!row_ok) q.u = u32x4{0, 0, 0, 0};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        f[8 * s + 2 * e] = bf16_bits_to_f32(q.u[e] & 0xffffu);
        f[8 * s + 2 * e + 1] = __uint_as_float(q.u[e] & 0xffff0000u);
      }
    }
    float amax = 0.f;
#pragma unroll
    for (int e = 0; e < 32; ++e) amax = fmaxf(amax, fabsf(f[e]));
    amax = quad_row_max(amax);
    float cq_inv;
    const float cq = query_pow2_factor(amax, cq_inv);
    rscale *= cq_inv;
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
      qhi[w] = hi;
      qlo[w] = lo;
    }
  }

  PA_TRACE_MARK(2);  // the query operands are ready
  const bool rs_nonneg = __builtin_amdgcn_ballot_w64(rscale < 0.f) == 0;
  // Online softmax against a reference that (almost) never moves.  l and the accumulator are kept relative to
  // m_ref, the row's maximum at its first visible step, and in units of 2^k_ref (per-token V scales: the exponent
  // of the largest V scale of that step).  Every later step produces its P relative to ITS OWN maximum and V-scale
  // unit, rounded up to whole powers of two: P = exp2(x - m_ref - n) * v_scale * 2^(kPBits - k), n = ceil(max - m_ref)
  // and k = exponent(largest V scale of the step), so P always fills the FP8 range, whatever the step's level.
  // The power of two that brings the step's P V back to the reference, 2^(n + k - k_ref), is the E8M0 block scale of
  // the P operand of the scaled MFMA -- exact, and free.  Nothing is rescaled per step: no exp2 of a maximum's
  // movement, no multiplication of the 32 accumulator registers (with an exact running maximum some row of the
  // sixteen moves on most steps of a long context).  The reference is re-based only when a step's level --
  // logits and V-scale unit TOGETHER, (max - m_ref) + (k - k_ref) -- has run more than kMaxAhead powers of two
  // ahead of it, which ordinary data never does.  f32 headroom: a step adds at most 2^(kMaxAhead + 1) (level) x
  // 2^kPBits (P) x 2^9 (an e4m3 value) x 64 tokens = 2^85 to an accumulator register, and a partition has fewer
  // than 2^25 steps.  Levels far BELOW the reference cost nothing: P is formed against the step's own level down
  // to kMaxBehind powers of two under the reference (below that its weight against the reference step's own
  // contribution to l is under 2^-200), and a block scale that would leave E8M0's range is clamped, which only
  // misstates terms of under 2^-100 of the accumulator's unit.
  // (m_ref, l) stay a consistent pair; the epilogue restates l against the true maximum for the partition buffers.
  constexpr int kPBits = 8;            // P is produced times 2^kPBits (at most 256; e4m3 reaches 448)
  constexpr float kMaxAhead = 60.f;    // (max - m_ref) + (k - k_ref) stays at or below this
  constexpr float kMaxBehind = 200.f;  // a step's own level is followed this far down
  // Experiment switch (never set by the launch layer outside PA_DECODE_DEBUG runs): P without its FP8 residual, every
  // element rounded to e4m3 as the reference's kernel rounds it.  Measured: a quarter of the step's vector
  // instructions and 6 % of the run time of a uniform 64-row batch, and 91 of the 363 parity cases then miss the
  // 2e-2 bar (every kind of case: short or peaked contexts leave the rounding of the few large elements in the result).
  const bool p_residual = !(a.flags & kFlagResidualNever);
  float m_ref = -INFINITY;
  float m_ref_safe = 0.f;   // m_ref, or 0 while it is -inf
  float m_true = -INFINITY;
  int k_ref = 0;            // per-token V scales: the accumulator's unit is 2^k_ref
  float l_run = 0.f;
  f32x4 acc[8];
#pragma unroll
  for (int db = 0; db < 8; ++db) acc[db] = f32x4{0.f, 0.f, 0.f, 0.f};

  // ---- one step of 64 tokens out of LDS: the arithmetic of pa_partition_kernel's FP8 step, one row tile ----
  // HALF: this wave takes tiles 2*half, 2*half+1 of the step (32 tokens) instead of all four
  // QRES: the query has an FP8 residual (a bf16 query); an FP8 query is its own head
  auto compute = [&]<bool FULL, bool HALF, bool QRES>(const StepLds& st, int tok0) {
    constexpr int T = HALF ? 2 : 4;       // 16-token tiles of the step this wave works on
    const int jb = HALF ? 2 * half : 0;   // the first of them
    f32x4 s[T];
#pragma unroll
    for (int jj = 0; jj < T; ++jj) {
      const int j = jb + jj;
      const u32x4 k0 = st.k[j][0][lane], k1 = st.k[j][1][lane];
      const i32x8 ka = {(int)k0[0], (int)k0[1], (int)k0[2], (int)k0[3], (int)k1[0], (int)k1[1], (int)k1[2], (int)k1[3]};
      s[jj] = f32x4{0.f, 0.f, 0.f, 0.f};
      s[jj] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ka, qhi, s[jj], 0, 0, 0, 0, 0, 0);
      if constexpr (QRES) s[jj] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ka, qlo, s[jj], 0, 0, 0, 0, 0, 0);
    }
    f32x4 ks_cur[PER_TOKEN ? T : 1], vs_cur[PER_TOKEN ? T : 1];
    int k = 0;  // per-token V scales: exponent of the step's largest V scale (the same in every lane)
    if constexpr (PER_TOKEN) {
      float vmx = 0.f;
#pragma unroll
      for (int jj = 0; jj < T; ++jj) {
        const int j = jb + jj;
        ks_cur[jj] = *reinterpret_cast<const f32x4*>(&st.sc[j][0][4 * kg]);
        vs_cur[jj] = *reinterpret_cast<const f32x4*>(&st.sc[j][1][4 * kg]);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if constexpr (!FULL) {
            const int col = tok0 + 16 * j + 4 * kg + r;
            vs_cur[jj][r] = col < ctx ? vs_cur[jj][r] : 0.f;
          }
          vmx = fmaxf(vmx, vs_cur[jj][r]);
        }
      }
      vmx = quad_row_max(vmx);
      // vmx = f * 2^k, f in [0.5, 1); 0 for vmx == 0.  The same in every lane: kept in a scalar register
      k = __builtin_amdgcn_readfirstlane(__builtin_amdgcn_frexp_expf(vmx));
    }
    // FULL: the row's scale (>= 0 on this path) is applied inside the exponent's fma, and to the maximum once
    float mx = -INFINITY;
#pragma unroll
    for (int jj = 0; jj < T; ++jj) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float v = s[jj][r];
        if constexpr (PER_TOKEN) v *= ks_cur[jj][r];
        if constexpr (!FULL) {
          const int col = tok0 + 16 * (jb + jj) + 4 * kg + r;
          v = v * rscale + slope2 * (float)(col - ctx + 1);
          v = col < limit ? v : -INFINITY;
        }
        s[jj][r] = v;
        mx = fmaxf(mx, v);
      }
    }
    mx = quad_row_max(mx);
    if constexpr (FULL) mx *= rscale;
    m_true = fmaxf(m_true, mx);
    // the rare step: a row sees its first key, or this step's level -- its logits' and its V scales' together -- is
    // too far ahead of the reference.  Then the V-scale unit moves to this step's, and every row whose maximum
    // lies above its reference moves the reference up to it.
    float ahead = mx - m_ref;  // +inf at a row's first visible key, NaN while it has seen none (compares false)
    const float level = PER_TOKEN ? ahead + (float)(k - k_ref) : ahead;
    if (__builtin_amdgcn_ballot_w64(level > kMaxAhead) != 0) {
      float alpha = 1.f;
      if (ahead > 0.f) {
        alpha = fast_exp2(m_ref - mx);  // exp2(-inf) = 0 on the first visible step
        m_ref = mx;
        m_ref_safe = mx;
        ahead = 0.f;
      }
      l_run *= alpha;
      if constexpr (PER_TOKEN) {
        // (the first step of all lands here with the accumulator still zero, and fixes the unit)
        alpha *= __builtin_ldexpf(1.f, k_ref - k < -126 ? -126 : (k_ref - k > 126 ? 126 : k_ref - k));
        k_ref = k;
      }
#pragma unroll
      for (int db = 0; db < 8; ++db) acc[db] *= alpha;
    }
    // n: whole powers of two from the reference up (or down) to this step's maximum
    const float nf = __builtin_ceilf(fmaxf(ahead, -kMaxBehind));  // (NaN, -inf: no visible key; every P is 0)
    const int n = (int)nf;
    const float e_add = (float)(kPBits - k) - m_ref_safe - nf;
    // E8M0 block scale of P, 2^(p_scale - 127): n + (k - k_ref) is at most kMaxAhead + 1; 255 would be a NaN
    int p_scale = n + (127 + k - k_ref);
    p_scale = p_scale < 1 ? 1 : (p_scale > 254 ? 254 : p_scale);
    const float e_mul = FULL ? rscale : 1.f;
    float psum = 0.f;
    uint32_t ph[4] = {0u, 0u, 0u, 0u}, pl[4] = {0u, 0u, 0u, 0u};  // (HALF: the tiles that are not this wave's hold P = 0)
    auto make_p = [&]<bool RESIDUAL>() {
#pragma unroll
      for (int j = 0; j < T; ++j) {
        float p0 = fast_exp2(__builtin_fmaf(s[j][0], e_mul, e_add));
        float p1 = fast_exp2(__builtin_fmaf(s[j][1], e_mul, e_add));
        float p2 = fast_exp2(__builtin_fmaf(s[j][2], e_mul, e_add));
        float p3 = fast_exp2(__builtin_fmaf(s[j][3], e_mul, e_add));
        psum += (p0 + p1) + (p2 + p3);
        if constexpr (PER_TOKEN) {
          p0 *= vs_cur[j][0];
          p1 *= vs_cur[j][1];
          p2 *= vs_cur[j][2];
          p3 *= vs_cur[j][3];
        }
        // both halves of a packed word are written, so its previous value is irrelevant: a register whose value
        // is dead (a logit) stands in for it; an explicit zero would cost a move per word
        int hi = (int)__float_as_uint(s[j][0]);
        hi = __builtin_amdgcn_cvt_pk_fp8_f32(p0, p1, hi, false);
        hi = __builtin_amdgcn_cvt_pk_fp8_f32(p2, p3, hi, true);
        ph[j] = (uint32_t)hi;
        if constexpr (RESIDUAL) {
          int lo = (int)__float_as_uint(s[j][1]);
          const f32x2 b01 = __builtin_amdgcn_cvt_pk_f32_fp8(hi, false);
          const f32x2 b23 = __builtin_amdgcn_cvt_pk_f32_fp8(hi, true);
          lo = __builtin_amdgcn_cvt_pk_fp8_f32(p0 - b01[0], p1 - b01[1], lo, false);
          lo = __builtin_amdgcn_cvt_pk_fp8_f32(p2 - b23[0], p3 - b23[1], lo, true);
          pl[j] = (uint32_t)lo;
        }
      }
    };
    if (p_residual)
      make_p.template operator()<true>();
    else
      make_p.template operator()<false>();
    // psum = sum of exp2(x - m_ref - n) * 2^(kPBits - k): back to the reference
    l_run += __builtin_ldexpf(psum, n + k - kPBits);

    // One 128-deep MFMA per 16 head dims covers head and residual of P at once.  Its reduction index is laid out
    // so that every lane's 32 bytes of V are 32 DIFFERENT tokens: lane groups 0 and 1 take the step's tiles 0-1
    // and 2-3 against the head of P, lane groups 2 and 3 the same tiles against the residual.  Before, lane group
    // g holds tokens 4g..4g+3 of every tile; two 4x4 (lane group x register) transposes bring every group the 16
    // tokens of its first tile (pa) and of its second (pb).
    // HALF: the wave has two tiles only, 64 of the 128 reduction slots: every lane group takes ONE tile in the first
    // half of its 32 slots (groups 0/1: the two tiles against the head of P, groups 2/3 against the residual) and
    // zeros in the second half, so one transpose and one LDS read of V per 16 head dims do.
    uint32_t pa[4], pb[4];
    if constexpr (HALF) {
      pa[0] = ph[0], pa[1] = ph[1], pa[2] = pl[0], pa[3] = pl[1];
      pb[0] = pb[1] = pb[2] = pb[3] = 0u;
    } else {
      pa[0] = ph[0], pa[1] = ph[2], pa[2] = pl[0], pa[3] = pl[2];
      pb[0] = ph[1], pb[1] = ph[3], pb[2] = pl[1], pb[3] = pl[3];
    }
    quad_transpose(pa);
    if constexpr (!HALF) quad_transpose(pb);
    const i32x8 pv = {(int)pa[0], (int)pa[1], (int)pa[2], (int)pa[3], (int)pb[0], (int)pb[1], (int)pb[2], (int)pb[3]};
    const int vj = HALF ? jb + (kg & 1) : 2 * (kg & 1);  // this lane group's (first) tile
    int nvalid0 = 16, nvalid1 = 16;
    if constexpr (!FULL) {
      // V bytes of tokens at or beyond ctx are zeroed (stale cache contents may decode to NaN)
      nvalid0 = ctx - (tok0 + 16 * vj);
      nvalid0 = nvalid0 < 0 ? 0 : (nvalid0 > 16 ? 16 : nvalid0);
      nvalid1 = ctx - (tok0 + 16 * vj + 16);
      nvalid1 = nvalid1 < 0 ? 0 : (nvalid1 > 16 ? 16 : nvalid1);
    }
#pragma unroll
    for (int db = 0; db < 8; ++db) {
      u32x4 v0 = st.v[vj][16 * db + li];
      u32x4 v1 = u32x4{0u, 0u, 0u, 0u};  // HALF: meets P = 0
      if constexpr (!HALF) v1 = st.v[vj + 1][16 * db + li];
      if constexpr (!FULL) {
        v0 = keep_first_bytes(v0, nvalid0);
        if constexpr (!HALF) v1 = keep_first_bytes(v1, nvalid1);
      }
      const i32x8 va = {(int)v0[0], (int)v0[1], (int)v0[2], (int)v0[3], (int)v1[0], (int)v1[1], (int)v1[2], (int)v1[3]};
      acc[db] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(va, pv, acc[db], 0, 0, 0, 127, 0, p_scale);
    }
  };

  // ---- main loop ---------------------------------------------------------------------------------------------
  int n_full = has_alibi ? 0 : (min_limit - wg_start) / kStepTokens;  // leading steps that need no masking
  n_full = n_full < 0 ? 0 : n_full;
  int tok0 = wg_start;
  int slot = 0;             // ring slot of step s
  int fetch_slot = NB - 1;  // ring slot the next fetch goes to
  int s = 0;
  // what every wave does at the head of step s, whether it has rows to compute or not
  auto enter_step = [&]() {
    // step s has landed once at most the loads of the steps after it are outstanding
    const int after = n_steps - 1 - s;
    if (after >= NB - 2)
      dma_wait<(NB - 2) * kLoadsPerStep>();
    else if (NB > 3 && after == 1)
      dma_wait<kLoadsPerStep>();
    else
      dma_wait<0>();
    // everybody's quarter of step s is in LDS, and everybody is done reading step s-1, whose slot is refilled now
    __syncthreads();
#ifdef PA_DECODE_TRACE
    if (s == 0) PA_TRACE_MARK(3);  // the first step has landed
#endif
    if (s + NB - 1 < n_steps) {
      fetch(fetch_slot, pg_next);
      fetch_tok += kStepTokens;
      pg_next = load_page(fetch_tok);
    }
  };
  auto leave_step = [&]() {
    ++s;
    tok0 += kStepTokens;
    slot = slot + 1 == NB ? 0 : slot + 1;
    fetch_slot = fetch_slot + 1 == NB ? 0 : fetch_slot + 1;
  };
  // Three loops, each with one variant of the step (one loop with a choice inside would make the compiler
  // copy the whole accumulator state where the variants join, every step).  The waves of a workgroup may be
  // in different loops: all of them pass the same number of barriers.
  // one pair of loops per variant: first the steps that need no masking, then the rest
  auto run_steps = [&]<bool HALF, bool QRES>(int n_fast) {
    while (s < n_fast) {
      enter_step();
      compute.template operator()<true, HALF, QRES>(stage[slot], tok0);
      leave_step();
    }
    while (s < n_steps) {
      enter_step();
      compute.template operator()<false, HALF, QRES>(stage[slot], tok0);
      leave_step();
    }
  };
  if (has_rows) {
    const int n_fast = rs_nonneg ? (n_full < n_steps ? n_full : n_steps) : 0;
    if (half_mode) {
      if (q_has_residual)
        run_steps.template operator()<true, true>(n_fast);
      else
        run_steps.template operator()<true, false>(n_fast);
    } else {
      if (q_has_residual)
        run_steps.template operator()<false, true>(n_fast);
      else
        run_steps.template operator()<false, false>(n_fast);
    }
  } else {
    while (s < n_steps) {
      enter_step();
      leave_step();
    }
  }
  __syncthreads();  // the stage buffers are free
  PA_TRACE_MARK(4);  // the last step is done

  // a tile of padding rows only (a ragged batch): the rows read as "no visible key"
  const bool output_only = a.flags & kFlagOutputOnly;
  auto write_padding_rows = [&](int first_row) {
    if (output_only) return;  // nobody reads them (the merge of a longer sequence writes what it finds to rows nobody reads)
    for (int r = first_row + kg; r < first_row + 16 && r < Ge; r += 4) {
      if (li == 0) {
        a.max_logits[es_off + r] = -INFINITY;
        a.exp_sums[es_off + r] = 0.f;
      }
      *reinterpret_cast<u32x4*>(tmp + (int64_t)r * a.stride_tmp_g * 2 + li * 16) = u32x4{0, 0, 0, 0};
      if (direct) *reinterpret_cast<u32x4*>(outp + (int64_t)r * a.stride_out_h * 2 + li * 16) = u32x4{0, 0, 0, 0};
    }
  };

  // ---- two waves per tile: the second hands its (m, l, O) to the first ------------------------------------------
  float acc_unit = __builtin_ldexpf(1.f, k_ref - kPBits);
  if (half_mode) {
    // per tile: reference maximum, l and true maximum of the 16 rows (lanes 0..15) and the 32 accumulator
    // registers of all 64 lanes, in units of 1
    constexpr int kMergeFloats = 3 * 16 + 32 * 64;
    static_assert(sizeof(StepLds) * NB >= 2 * kMergeFloats * 4 + 2 * 16 * kORowBytes, "room for the merge buffers");
    float* mb = reinterpret_cast<float*>(&stage[0]) + (row0 >> 4) * kMergeFloats;
    if (has_rows && half == 1) {
      const float lt = quad_row_sum(l_run);
      if (kg == 0) {
        mb[li] = m_ref;
        mb[16 + li] = lt;
        mb[32 + li] = m_true;
      }
#pragma unroll
      for (int db = 0; db < 8; ++db) {
#pragma unroll
        for (int r = 0; r < 4; ++r) mb[48 + (4 * db + r) * 64 + lane] = acc[db][r] * acc_unit;
      }
    }
    __syncthreads();
    if (half == 1) {
      // done with its tile; the tiles 2 and 3 of a larger group hold padding rows only, which these two waves write
      write_padding_rows(32 + row0);
      return;
    }
    if (has_rows) {
      const float m1 = mb[li], l1 = mb[16 + li];
      const float l0 = quad_row_sum(l_run);
      const float mm = fmaxf(m_ref, m1);
      const float m_safe = mm == -INFINITY ? 0.f : mm;
      const float w0 = fast_exp2(m_ref - m_safe), w1 = fast_exp2(m1 - m_safe);  // exp2(-inf) = 0: a half that saw no key
#pragma unroll
      for (int db = 0; db < 8; ++db) {
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[db][r] = acc[db][r] * (acc_unit * w0) + mb[48 + (4 * db + r) * 64 + lane] * w1;
      }
      m_ref = mm;
      m_true = fmaxf(m_true, mb[32 + li]);
      // l_run becomes this lane's share of the merged sum: the row total in lane group 0, nothing elsewhere
      l_run = kg == 0 ? l0 * w0 + l1 * w1 : 0.f;
      acc_unit = 1.f;
    }
  }

  // ---- epilogue: every wave writes its own row tile -----------------------------------------------------------
  if (!has_rows) {
    write_padding_rows(row0);
    return;
  }
  float l_tot = quad_row_sum(l_run);
  if (!row_ok) {
    l_tot = 0.f;
    m_true = -INFINITY;
  }
  const float inv = l_tot > 0.f ? v_tensor_scale * acc_unit / l_tot : 0.f;
  const bool no_partial = output_only && direct;  // finished here: nobody merges this sequence
  if (row < Ge && kg == 0 && !no_partial) {
    // the partition buffers hold the true maximum and the sum taken against it
    a.max_logits[es_off + row] = m_true * (1.0f / kLog2e);
    a.exp_sums[es_off + row] = l_tot > 0.f ? l_tot * fast_exp2(m_ref - m_true) : 0.f;
  }
  // wave-private staging for the transposed store (two waves per tile: behind the merge buffers, one per tile)
  char* olds = reinterpret_cast<char*>(&stage[0]) +
               (half_mode ? 2 * (3 * 16 + 32 * 64) * 4 + (row0 >> 4) * (16 * kORowBytes) : wave * (16 * kORowBytes));
  const int rows_out = (output_only ? rows_valid : Ge) - row0;
  if (no_partial)
    store_partial_tile(olds, acc, inv, outp + (int64_t)row0 * a.stride_out_h * 2, a.stride_out_h * 2, nullptr, 0,
                       rows_out, lane);
  else
    store_partial_tile(olds, acc, inv, tmp + (int64_t)row0 * a.stride_tmp_g * 2, a.stride_tmp_g * 2,
                       direct ? outp + (int64_t)row0 * a.stride_out_h * 2 : nullptr, a.stride_out_h * 2, rows_out, lane);
#ifdef PA_DECODE_TRACE
  if (lane == 0 && row0 == 0 && half == 0 && blockIdx.x < kTraceWorkgroups) {  // (these waves run to the end)
    unsigned long long* t = pa_trace + 8ull * blockIdx.x;
#pragma unroll
    for (int i = 0; i < 5; ++i) t[i] = pa_trace_t[i];
    t[5] = wall_clock64();
    t[6] = (unsigned long long)n_steps;
    // live rows, and where the workgroup ran: HW_ID (CU, shader array, shader engine) and XCC_ID
    const unsigned hw = __builtin_amdgcn_s_getreg((4 << 0) | (0 << 6) | (31 << 11));   // HW_REG_HW_ID, 32 bits
    const unsigned xcc = __builtin_amdgcn_s_getreg((20 << 0) | (0 << 6) | (31 << 11)); // HW_REG_XCC_ID
    t[7] = (unsigned long long)rows_valid | ((unsigned long long)(hw & 0xffffu) << 16) | ((unsigned long long)(xcc & 0xfu) << 32);
  }
#endif
}

}  // namespace

#endif  // PA_PARTITION_SHARED_KERNEL_H_
