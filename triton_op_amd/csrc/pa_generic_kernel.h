// pa_partition_generic_kernel / pa_reduce_generic_kernel: both stages for head sizes other than 128.
#ifndef PA_GENERIC_KERNEL_H_
#define PA_GENERIC_KERNEL_H_

#include "pa_common.h"

namespace {

// ---------------------------------------------------------------------------------------------
// The reference's kernels take any power-of-two head size (pa_decode_triton_gluon_fp8.py:514-1002 pads it to
// HEAD_SIZE_POW2); its sweep, its published numbers and the tuned kernels of this library are all at 128.  Head
// sizes 64 and 256 run on the two kernels of this file: every layout, dtype, scale mode and option of the operator,
// on bf16 MFMAs without a software pipeline -- the same results, not the same speed.
//
// Stage 1: one wave per (sequence, partition, kv head, 16-row query tile).  A 64-token step is four 16-token
// blocks (pages, when the page size is 16).  v_mfma_f32_16x16x16_bf16 holds, in lane l (li = l % 16, kg = l / 16),
// four consecutive reduction indices 4 kg .. 4 kg + 3 of row / column li of its operands and rows 4 kg .. 4 kg + 3 of
// column li of its result, so:
//   S^T[token, row] = K Q^T:  A = 4 head dims of a token (a quarter of a 16-byte piece of the cache, as bf16),
//                             B = the same 4 head dims of query row li; the result holds 4 tokens of row li;
//   O^T[dim, row]   = V^T P:  A = 4 tokens of head dim li of a 16-dim block, B = P of those 4 tokens for row li --
//                             exactly what the lane holds of S^T, so P never moves between lanes.
// Which token is row i of K tile j is free: tile j takes tokens 4 j .. 4 j + 3 of EVERY block (row i: block i / 4,
// token 4 j + i % 4), so that lane group kg ends up with the logits, and then P, of all 16 tokens of block kg -- and
// its V operands of the step's four MFMAs per 16-dim block are one 16-byte piece of the cache (16 tokens of head dim
// li), not four 4-byte pieces of four blocks.
// Row maximum and sum: 16 values in the lane, then the four lanes of a row (quad_row_max / quad_row_sum).
// ---------------------------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(4))) short bf16x4_bits;

// four consecutive cache elements starting at p as bf16 (FP8 values are exact in bf16)
template <bool FP8>
__device__ __forceinline__ bf16x4_bits load_cache4(const char* p) {
  union {
    bf16x4_bits v;
    uint32_t u[2];
  } r;
  if constexpr (FP8) {
    const uint32_t w = *reinterpret_cast<const uint32_t*>(p);
    r.u[0] = fp8x2_to_bf16x2(w, false);
    r.u[1] = fp8x2_to_bf16x2(w, true);
  } else {
    const u32x2 w = *reinterpret_cast<const u32x2*>(p);
    r.u[0] = w[0];
    r.u[1] = w[1];
  }
  return r.v;
}

// (there is no prefetch: the waves of a SIMD hide each other's load latency, so the registers are capped for four
// waves per SIMD, two with the 64 accumulator registers of head size 256)
template <int D, bool FP8>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(D > 128 ? 2 : 4, D > 128 ? 2 : 4)))
void pa_partition_generic_kernel(const PaDecodeArgs a) {
  constexpr int X = FP8 ? 16 : 8;  // cache elements per 16 bytes
  constexpr int ESZ = FP8 ? 1 : 2;
  constexpr int DB = D / 16;       // 16-dim blocks of the head
  static_assert(D % 16 == 0, "the head is cut into 16-dim blocks");

  const int lane = threadIdx.x;
  const int li = lane & 15, kg = lane >> 4;
  const int Hkv = a.num_kv_heads;
  const int G = a.group_size;
  const int Ge = a.q_len * G;
  const int RT = (Ge + 15) / 16;
  const uint32_t wid = blockIdx.x;
  const int h = (int)(wid % (uint32_t)Hkv);
  const int rt = (int)((wid / (uint32_t)Hkv) % (uint32_t)RT);
  const uint32_t item = wid / (uint32_t)(Hkv * RT);
  const int b = (int)(item % (uint32_t)a.num_seqs);
  const int part = (int)(item / (uint32_t)a.num_seqs);
  const int row0 = 16 * rt;

  const int ctx = sload_i32(a.context_lens + b);
  const int wg_start = part * a.partition_size;
  if (wg_start >= ctx && !(ctx <= 0 && part == 0)) return;  // (an empty sequence keeps its first partition: zeros)
  const int wg_end = min(wg_start + a.partition_size, ctx);
  const int qb = a.q_lens ? sload_i32(a.q_lens + b) : a.q_len;
  const int rows_valid = qb * G;
  const bool output_only = a.flags & kFlagOutputOnly;

  const int64_t es_off = (int64_t)b * a.stride_es_s + (int64_t)h * a.stride_es_h + (int64_t)part * a.stride_es_p;
  char* tmp = (char*)a.tmp_output +
              ((int64_t)b * a.stride_tmp_s + (int64_t)h * a.stride_tmp_h + (int64_t)part * a.stride_tmp_p) * 2;

  // ---- this lane's query row: its B operands (4 head dims per 16-dim block), its scale, its mask ------------------
  const int row = row0 + li;
  const bool row_ok = row < rows_valid;
  const int t_row = row / G;
  const int limit = row_ok ? ctx - (qb - 1 - t_row) : 0;  // number of visible keys (causal over the new tokens)
  float k_tensor_scale = 1.f, v_tensor_scale = 1.f;
  if (a.kv_quant_mode == PA_QUANT_PER_TENSOR) {
    k_tensor_scale = sload_f32(a.key_scale);
    v_tensor_scale = sload_f32(a.value_scale);
  }
  const bool per_token = a.kv_quant_mode == PA_QUANT_PER_TOKEN;
  float rscale = a.softmax_scale * k_tensor_scale * kLog2e;  // logits in the log2 domain
  if (a.query_quant_mode == PA_QUANT_PER_TENSOR) rscale *= sload_f32(a.query_scale);
  if (a.query_quant_mode == PA_QUANT_PER_TOKEN && row_ok)
    rscale *= a.query_scale[(int64_t)b * a.stride_qscale_s + h * Ge + row];
  float slope2 = 0.f;
  if (a.alibi_slopes && row_ok)
    slope2 = a.alibi_slopes[a.alibi_slopes_len == Hkv * Ge ? h * Ge + row : h * G + (row - t_row * G)] * kLog2e;
  // (the order of the reduction index is free as long as both operands agree: MFMA c = 4 g + m takes head dims
  // 64 g + 16 kg + 4 m .. + 3 from lane group kg, so a lane's K bytes of four MFMAs are ONE 16-byte piece of the cache)
  bf16x4_bits qreg[DB];
  {
    const int64_t e0 = (int64_t)b * a.stride_q_s + (int64_t)(h * Ge + (row_ok ? row : 0)) * a.stride_q_h + 16 * kg;
#pragma unroll
    for (int c = 0; c < DB; ++c) {
      const int d = 64 * (c >> 2) + 4 * (c & 3);
      if (a.query_dtype == PA_DTYPE_BF16)
        qreg[c] = load_cache4<false>((const char*)a.query + (e0 + d) * 2);
      else
        qreg[c] = load_cache4<true>((const char*)a.query + (e0 + d));
      if (!row_ok) qreg[c] = bf16x4_bits{0, 0, 0, 0};
    }
  }

  const int log2_bs = 31 - __builtin_clz(a.block_size);
  const int bs_mask = a.block_size - 1;
  const int* bt = a.block_tables + (int64_t)b * a.stride_bt_s;
  const char* kbase = (const char*)a.key_cache + (int64_t)h * a.stride_k_h * ESZ;
  const char* vbase = (const char*)a.value_cache + (int64_t)h * a.stride_v_h * ESZ;
  const int last_tile_tok = (max(wg_end, 1) - 1) & ~15;

  float m_run = -INFINITY, l_run = 0.f;  // of row li (the same in the row's four lanes)
  f32x4 acc[DB];                         // O^T: head dims 16 db + 4 kg .. + 3 of row li
#pragma unroll
  for (int db = 0; db < DB; ++db) acc[db] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int sub_k = li >> 2;  // the 16-token block this lane's K rows come from (see the token order above)
  // pages of a step's four 16-token blocks (blocks past the last live one repeat it); asked for one step ahead
  int page_next[4];
  auto load_pages = [&](int t0) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int t = t0 + 16 * j;
      t = t > last_tile_tok ? last_tile_tok : t;
      page_next[j] = sload_i32(bt + (t >> log2_bs));
    }
  };
  load_pages(wg_start);
  for (int tok0 = wg_start; tok0 < wg_end; tok0 += kStepTokens) {
    int page[4], off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int t = tok0 + 16 * j;
      t = t > last_tile_tok ? last_tile_tok : t;
      page[j] = page_next[j];
      off[j] = t & bs_mask;
    }
    load_pages(tok0 + kStepTokens);  // (an index past the sequence's last live block is clamped to it)
    // this lane's block as a row of K (li / 4) and as a holder of logits, P, scales and V (kg)
    const int page_k = sub_k == 0 ? page[0] : (sub_k == 1 ? page[1] : (sub_k == 2 ? page[2] : page[3]));
    const int off_k = (sub_k == 0 ? off[0] : (sub_k == 1 ? off[1] : (sub_k == 2 ? off[2] : off[3]))) + (li & 3);
    const int page_v = kg == 0 ? page[0] : (kg == 1 ? page[1] : (kg == 2 ? page[2] : page[3]));
    const int off_v = kg == 0 ? off[0] : (kg == 1 ? off[1] : (kg == 2 ? off[2] : off[3]));
    // ---- S^T = K Q^T: tile j takes tokens 4 j .. 4 j + 3 of every block ---------------------------------------------
    f32x4 s[4];
    const char* kt = kbase + (int64_t)page_k * a.stride_k_b * ESZ;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      s[j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int g = 0; g < D / 64; ++g) {
        // this lane's 16 head dims of the 64-dim group: one 16-byte piece (FP8) or two (bf16)
        union {
          u32x4 q[2];
          uint32_t u[8];
        } kv;
        if constexpr (FP8) {
          kv.q[0] = load16(kt + (int64_t)(4 * g + kg) * a.stride_k_c + (off_k + 4 * j) * 16);
        } else {
          kv.q[0] = load16(kt + ((int64_t)(8 * g + 2 * kg) * a.stride_k_c + (off_k + 4 * j) * 8) * 2);
          kv.q[1] = load16(kt + ((int64_t)(8 * g + 2 * kg + 1) * a.stride_k_c + (off_k + 4 * j) * 8) * 2);
        }
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          union {
            bf16x4_bits v;
            uint32_t u[2];
          } ka;
          if constexpr (FP8) {
            ka.u[0] = fp8x2_to_bf16x2(kv.u[m], false);
            ka.u[1] = fp8x2_to_bf16x2(kv.u[m], true);
          } else {
            ka.u[0] = kv.u[2 * m];
            ka.u[1] = kv.u[2 * m + 1];
          }
          s[j] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(ka.v, qreg[4 * g + m], s[j], 0, 0, 0);
        }
      }
    }
    // ---- scales, ALiBi, mask; row maximum (s[j][r]: token 16 kg + 4 j + r of the step) ------------------------------
    f32x4 vs[4];
    float mx = -INFINITY;
    const int col0 = tok0 + 16 * kg;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f32x4 ks = {1.f, 1.f, 1.f, 1.f};
      vs[j] = f32x4{1.f, 1.f, 1.f, 1.f};
      if (per_token) {
        const int64_t so = (int64_t)page_v * a.stride_kvscale_b + (int64_t)h * a.stride_kvscale_h + off_v + 4 * j;
        ks = *reinterpret_cast<const f32x4*>(a.key_scale + so);
        vs[j] = *reinterpret_cast<const f32x4*>(a.value_scale + so);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int col = col0 + 4 * j + r;
        float x = s[j][r] * ks[r] * rscale + slope2 * (float)(col - ctx + 1);
        x = col < limit ? x : -INFINITY;  // (a select: stale cache bytes may have made the logit a NaN)
        s[j][r] = x;
        mx = fmaxf(mx, x);
      }
    }
    mx = quad_row_max(mx);
    const float m_new = fmaxf(m_run, mx);
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = fast_exp2(m_run - m_safe);  // exp2(-inf) = 0 while the row has seen no key
    m_run = m_new;
    float psum = 0.f;
    bf16x4_bits pb[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float p[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        p[r] = fast_exp2(s[j][r] - m_safe);
        psum += p[r];
        p[r] *= vs[j][r];
      }
      union {
        bf16x4_bits v;
        uint32_t u[2];
      } pk;
      pk.u[0] = pack_bf16x2(p[0], p[1]);
      pk.u[1] = pack_bf16x2(p[2], p[3]);
      pb[j] = pk.v;
    }
    l_run = l_run * alpha + quad_row_sum(psum);
#pragma unroll
    for (int db = 0; db < DB; ++db) acc[db] *= alpha;
    // ---- O^T += V^T P: the lane's 16 tokens of head dim li are ONE 16-byte piece of the cache (two with bf16) ----------
    // stale bytes past the context may decode to NaN, and 0 * NaN is NaN: those tokens' V is zero (masks per 4 tokens:
    // FP8, one byte a token; bf16, two dwords of two tokens)
    const int n_live = ctx - col0;  // live tokens of this lane's block (may be <= 0 or >= 16)
    uint32_t keep[FP8 ? 4 : 8];
#pragma unroll
    for (int w = 0; w < (FP8 ? 4 : 8); ++w) {
      const int per = FP8 ? 4 : 2;  // tokens in dword w
      const int v = n_live - per * w;
      keep[w] = v >= per ? 0xffffffffu : (v <= 0 ? 0u : (FP8 ? (1u << (8 * v)) - 1u : 0xffffu));
    }
    const char* vt = vbase + (int64_t)page_v * a.stride_v_b * ESZ;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int d = 16 * db + li;
      union {
        u32x4 q[2];
        uint32_t u[8];
      } vw;
      if constexpr (FP8) {
        const int64_t e = a.v_transposed ? (int64_t)(off_v / X) * a.stride_v_2 + (int64_t)d * X : (int64_t)d * a.stride_v_2 + off_v;
        vw.q[0] = load16(vt + e);
      } else {
        const int64_t e0 = a.v_transposed ? (int64_t)(off_v / X) * a.stride_v_2 + (int64_t)d * X : (int64_t)d * a.stride_v_2 + off_v;
        const int64_t e1 = a.v_transposed ? e0 + a.stride_v_2 : e0 + 8;
        vw.q[0] = load16(vt + e0 * 2);
        vw.q[1] = load16(vt + e1 * 2);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        union {
          bf16x4_bits v;
          uint32_t u[2];
        } va;
        if constexpr (FP8) {
          const uint32_t w = vw.u[j] & keep[j];
          va.u[0] = fp8x2_to_bf16x2(w, false);
          va.u[1] = fp8x2_to_bf16x2(w, true);
        } else {
          va.u[0] = vw.u[2 * j] & keep[2 * j];
          va.u[1] = vw.u[2 * j + 1] & keep[2 * j + 1];
        }
        acc[db] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(va.v, pb[j], acc[db], 0, 0, 0);
      }
    }
  }

  // ---- the partition's result: (max, sum, O / sum) of row li ---------------------------------------------------------
  const int rows_live = output_only ? rows_valid : Ge;
  if (row < rows_live) {
    const float inv = l_run > 0.f ? v_tensor_scale / l_run : 0.f;
    if (kg == 0) {
      a.max_logits[es_off + row] = m_run * (1.0f / kLog2e);
      a.exp_sums[es_off + row] = l_run;
    }
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      u32x2 pk;
      pk[0] = pack_bf16x2(acc[db][0] * inv, acc[db][1] * inv);
      pk[1] = pack_bf16x2(acc[db][2] * inv, acc[db][3] * inv);
      *reinterpret_cast<u32x2*>(tmp + ((int64_t)row * a.stride_tmp_g + 16 * db + 4 * kg) * 2) = pk;
    }
  }
}

// Stage 2 for those head sizes: one wave per (sequence, kv head, output row); lane l owns head dims l, l + 64, ...
template <int D>
__global__ __launch_bounds__(64) void pa_reduce_generic_kernel(const PaDecodeArgs a) {
  constexpr int DPL = D / 64;
  const int lane = threadIdx.x;
  const int Ge = a.q_len * a.group_size;
  const uint32_t wid = blockIdx.x;
  const int row = (int)(wid % (uint32_t)Ge);
  const int h = (int)((wid / (uint32_t)Ge) % (uint32_t)a.num_kv_heads);
  const int b = (int)(wid / (uint32_t)(Ge * a.num_kv_heads));
  const int ctx = a.context_lens[b];
  int n = (ctx + a.partition_size - 1) / a.partition_size;
  n = n > a.max_num_partitions ? a.max_num_partitions : n;
  const int qb = a.q_lens ? a.q_lens[b] : a.q_len;
  const bool live = n > 0 && row < qb * a.group_size;
  __bf16* out = (__bf16*)a.output + (int64_t)b * a.stride_out_s + (int64_t)(h * Ge + row) * a.stride_out_h;
  if (!live) {
    if (!(a.flags & PA_DECODE_FLAG_OUTPUT_ONLY) || n <= 0) {
#pragma unroll
      for (int i = 0; i < DPL; ++i) out[lane + 64 * i] = (__bf16)0.f;
    }
    return;
  }
  const int64_t es = (int64_t)b * a.stride_es_s + (int64_t)h * a.stride_es_h + row;
  const __bf16* tmp = (const __bf16*)a.tmp_output + (int64_t)b * a.stride_tmp_s + (int64_t)h * a.stride_tmp_h +
                      (int64_t)row * a.stride_tmp_g;
  float M = a.sinks ? a.sinks[h * Ge + row] : -INFINITY;  // (the sink takes part in the maximum)
  // (the loads of four partitions go out together: the loops are round trips to memory otherwise)
#pragma unroll 4
  for (int p = 0; p < n; ++p) M = fmaxf(M, a.max_logits[es + (int64_t)p * a.stride_es_p]);
  const float M_safe = M == -INFINITY ? 0.f : M;
  float L = 0.f;
  float o[DPL];
#pragma unroll
  for (int i = 0; i < DPL; ++i) o[i] = 0.f;
#pragma unroll 4
  for (int p = 0; p < n; ++p) {
    const float w = a.exp_sums[es + (int64_t)p * a.stride_es_p] *
                    __expf(a.max_logits[es + (int64_t)p * a.stride_es_p] - M_safe);
    L += w;
#pragma unroll
    for (int i = 0; i < DPL; ++i) o[i] += w * (float)tmp[(int64_t)p * a.stride_tmp_p + lane + 64 * i];
  }
  if (a.sinks) L += __expf(a.sinks[h * Ge + row] - M_safe);
  const float inv = L > 0.f ? 1.f / L : 0.f;
#pragma unroll
  for (int i = 0; i < DPL; ++i) out[lane + 64 * i] = (__bf16)(o[i] * inv);
}

}  // namespace

#endif  // PA_GENERIC_KERNEL_H_
