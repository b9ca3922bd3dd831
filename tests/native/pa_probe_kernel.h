// pa_gather_probe_kernel: a read-only probe of the partition kernel's memory access pattern.
#ifndef PA_PROBE_KERNEL_H_
#define PA_PROBE_KERNEL_H_

#include "../../triton_op_amd/csrc/pa_common.h"

namespace {

// Reads what pa_partition_kernel<fp8, bs16, 4 waves> reads for the same arguments, in the same grouping and order
// -- one workgroup of four waves per (sequence, partition, kv head), head fastest; wave w takes the 64-token
// steps w, w + 4, ...; per step every lane issues eight 16-byte non-temporal loads of K (four 16-token tiles, two
// loads each, lanes 0-15 = the tile's tokens, lane >> 4 = the chunk row) and eight of V (lanes 0-15 = 16 head dims,
// lane >> 4 = the tile), one step ahead of the step whose bytes it folds together -- and does no arithmetic beyond
// an XOR per loaded word.  What it reaches is what the memory system gives this gather pattern; the gap between it
// and the partition kernel is what the kernel's arithmetic and its tail cost.
// Block size 16, FP8 cache in the dense default layout only.  `sink` receives a word only if the fold of all the
// bytes read is a value it cannot be (which keeps the loads alive without a store per workgroup).
template <bool BS16>  // block size 16 in the dense layout: constant in-page strides, as in the kernel's own variant
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
void pa_gather_probe_kernel(const PaDecodeArgs a, int* sink) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int li = lane & 15, kg = lane >> 4;
  const int Hkv = a.num_kv_heads;
  const long long wid = blockIdx.x;
  const int h = (int)(wid % Hkv);
  const long long item = wid / Hkv;
  const int b = (int)(item % a.num_seqs);
  const int part = (int)(item / a.num_seqs);
  const int ctx = sload_i32(a.context_lens + b);
  const int wg_start = part * a.partition_size;
  if (wg_start >= ctx) return;
  const int wg_end = min(wg_start + a.partition_size, ctx);
  const int wg_steps = (wg_end - wg_start + kStepTokens - 1) / kStepTokens;
  const int n_steps = wave < wg_steps ? (wg_steps - wave + 3) / 4 : 0;
  if (n_steps == 0) return;
  const char* kbase = (const char*)a.key_cache + (int64_t)h * a.stride_k_h;
  const char* vbase = (const char*)a.value_cache + (int64_t)h * a.stride_v_h;
  const int* bt = a.block_tables + (int64_t)b * a.stride_bt_s;
  const int last_tile_tok = (wg_end - 1) & ~15;
  // (any block size and the plain V layout: the strides come from the arguments; with pages of more than 64 tokens
  // the V rows are read with ordinary loads, as the kernel reads them: a step takes half a 128-byte line of a row)
  const int log2_bs = BS16 ? 4 : 31 - __builtin_clz(a.block_size);
  const int bs_mask = BS16 ? 15 : a.block_size - 1;
  const uint32_t k_chunk = BS16 ? 256u : (uint32_t)a.stride_k_c;
  const uint32_t k_off = (uint32_t)(kg * k_chunk + li * 16);
  const uint32_t v_row = BS16 ? 16u : (uint32_t)a.stride_v_2;
  const bool v_stream = BS16 || a.block_size <= 64;
  struct Step {
    u32x4 k[4][2];
    u32x4 v[8];
  };
  auto issue = [&](Step& st, int tok0) {
    int page[4], off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int t = tok0 + 16 * j;
      t = t > last_tile_tok ? last_tile_tok : t;
      page[j] = sload_i32(bt + (t >> log2_bs));
      off[j] = t & bs_mask;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const char* tb = kbase + (int64_t)page[j] * a.stride_k_b + (int64_t)off[j] * 16;
      st.k[j][0] = load16_stream(tb + k_off);
      st.k[j][1] = load16_stream(tb + k_off + 4 * k_chunk);
    }
    const int vp = kg == 0 ? page[0] : (kg == 1 ? page[1] : (kg == 2 ? page[2] : page[3]));
    const int vo = kg == 0 ? off[0] : (kg == 1 ? off[1] : (kg == 2 ? off[2] : off[3]));
    const char* tb = vbase + (int64_t)vp * a.stride_v_b + vo;
    if (v_stream) {
#pragma unroll
      for (int db = 0; db < 8; ++db) st.v[db] = load16_stream(tb + (li + 16 * db) * v_row);
    } else {
#pragma unroll
      for (int db = 0; db < 8; ++db) st.v[db] = load16(tb + (li + 16 * db) * v_row);
    }
  };
  uint32_t fold = 0;
  auto consume = [&](const Step& st) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int ld = 0; ld < 2; ++ld) fold ^= st.k[j][ld][0] ^ st.k[j][ld][1] ^ st.k[j][ld][2] ^ st.k[j][ld][3];
#pragma unroll
    for (int db = 0; db < 8; ++db) fold ^= st.v[db][0] ^ st.v[db][1] ^ st.v[db][2] ^ st.v[db][3];
  };
  int tok0 = wg_start + wave * kStepTokens;
  Step cur, nxt;
  issue(cur, tok0);
  for (int s = 0; s + 1 < n_steps; ++s) {
    tok0 += 4 * kStepTokens;
    issue(nxt, tok0);
    consume(cur);
    cur = nxt;
  }
  consume(cur);
  // FP8 cache bytes of real workloads never fold to this exact word in every lane at once
  if (__builtin_amdgcn_ballot_w64(fold != 0x9e3779b9u) == 0) sink[lane] = (int)fold;
}

// pa_stream_probe_kernel: the same pages read the way a workgroup would read them whose four waves work on the SAME
// 64-token step: wave w loads K of the step's tile w (2 KiB), the 32 head dims 32 w .. 32 w + 31 of V for all four
// tiles (2 KiB) and, with per-token scales, the tile's 16 + 16 scales, DEPTH steps ahead of the step it folds, in
// registers; one workgroup barrier per step stands for the exchange of the step's probabilities.  OCC workgroups per
// CU.  (variant bits: 1 no barrier, 2 no scale loads, 4 V by tile.)  What this reaches is what such a kernel could reach before its arithmetic.
template <int DEPTH, int OCC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(OCC, OCC)))
void pa_stream_probe_kernel(const PaDecodeArgs a, int* sink, int variant) {
  const bool with_barrier = !(variant & 1);  // variant bit 0: no barrier between the steps
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int li = lane & 15, kg = lane >> 4;
  const int Hkv = a.num_kv_heads;
  const long long wid = blockIdx.x;
  const int h = (int)(wid % Hkv);
  const long long item = wid / Hkv;
  const int b = (int)(item % a.num_seqs);
  const int part = (int)(item / a.num_seqs);
  const int ctx = sload_i32(a.context_lens + b);
  const int wg_start = part * a.partition_size;
  if (wg_start >= ctx) return;
  const int wg_end = min(wg_start + a.partition_size, ctx);
  const int n_steps = (wg_end - wg_start + kStepTokens - 1) / kStepTokens;
  const char* kbase = (const char*)a.key_cache + (int64_t)h * a.stride_k_h;
  const char* vbase = (const char*)a.value_cache + (int64_t)h * a.stride_v_h;
  const bool per_token = a.kv_quant_mode == PA_QUANT_PER_TOKEN && !(variant & 2);  // bit 1: the scales are not read
  // (without per-token scales the load reads one word of the context lengths instead: no branch around a load)
  const float* sc_lane = per_token ? ((lane & 16) ? a.value_scale : a.key_scale) + (int64_t)h * a.stride_kvscale_h + li
                                   : reinterpret_cast<const float*>(a.context_lens);
  const int64_t sc_page_stride = per_token ? a.stride_kvscale_b : 0;
  const int* bt = a.block_tables + (int64_t)b * a.stride_bt_s;
  const int last_tile_tok = (wg_end - 1) & ~15;
  const uint32_t k_off = (uint32_t)(kg * 256 + li * 16);
  // variant bit 2: wave w reads all 128 head dims of V for the step's tile w (what pa_partition_shared_kernel's
  // waves fetch: 2 KiB in one piece) instead of 32 head dims for all four tiles (four pieces of 512 bytes)
  const bool v_by_tile = variant & 4;
  const uint32_t v_off = v_by_tile ? (uint32_t)(lane * 16) : (uint32_t)((32 * wave + li) * 16);
  const uint32_t v_off2 = v_by_tile ? 1024u : 256u;
  struct Step {
    u32x4 k[2];
    u32x4 v[2];
    float sc;
  };
  auto issue = [&](Step& st, int tok0) {
    int page[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int t = tok0 + 16 * j;
      t = t > last_tile_tok ? last_tile_tok : t;
      page[j] = sload_i32(bt + (t >> 4));
    }
    int tw = tok0 + 16 * wave;
    tw = tw > last_tile_tok ? last_tile_tok : tw;
    const int kp = sload_i32(bt + (tw >> 4));
    const char* tb = kbase + (int64_t)kp * a.stride_k_b;
    st.k[0] = load16_stream(tb + k_off);
    st.k[1] = load16_stream(tb + k_off + 1024);
    int vp = page[0];  // (lane-wise selects, no branches)
    vp = kg == 1 ? page[1] : vp;
    vp = kg == 2 ? page[2] : vp;
    vp = kg == 3 ? page[3] : vp;
    vp = v_by_tile ? kp : vp;
    const char* vb = vbase + (int64_t)vp * a.stride_v_b;
    st.v[0] = load16_stream(vb + v_off);
    st.v[1] = load16_stream(vb + v_off + v_off2);
    st.sc = __builtin_nontemporal_load(sc_lane + (int64_t)kp * sc_page_stride);
    __builtin_amdgcn_sched_barrier(0);
  };
  uint32_t fold = 0;
  auto consume = [&](const Step& st) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
      fold ^= st.k[i][0] ^ st.k[i][1] ^ st.k[i][2] ^ st.k[i][3] ^ st.v[i][0] ^ st.v[i][1] ^ st.v[i][2] ^ st.v[i][3];
    fold ^= __float_as_uint(st.sc);
    // the step's registers are needed HERE (the compiler may not gather the folds of a round at its end)
    asm volatile("" ::"v"(st.k[0]), "v"(st.k[1]), "v"(st.v[0]), "v"(st.v[1]), "v"(st.sc));
    __builtin_amdgcn_sched_barrier(0);
  };
  // whole rounds of DEPTH steps (steps past the end re-read the last tile's lines): every path to a use has issued
  // the same loads in the same order, so the compiler's counted waits stay partial
  Step st[DEPTH];
  int tok = wg_start;
#pragma unroll
  for (int i = 0; i < DEPTH; ++i) {
    issue(st[i], tok);
    tok += kStepTokens;
  }
  const int rounds = (n_steps + DEPTH - 1) / DEPTH;
  for (int r = 0; r < rounds; ++r) {
#pragma unroll
    for (int i = 0; i < DEPTH; ++i) {
      consume(st[i]);
      if (with_barrier) __syncthreads();
      issue(st[i], tok);
      tok += kStepTokens;
    }
  }
  if (__builtin_amdgcn_ballot_w64(fold != 0x9e3779b9u) == 0) sink[lane] = (int)fold;
}

// pa_issue_probe_kernel: what instructions of the decode step cost the issue port of a SIMD.  Every wave runs
// `iters` iterations of 128 instructions of one kind on eight independent registers (MODE 0: v_fma_f32, the
// full-rate yardstick; 3: v_exp_f32; 4: v_cvt_pk_fp8_f32; 5: v_permlane32_swap), or of 16 MFMAs
// (v_mfma_f32_16x16x128_f8f6f4, MODE 1), or of the 16 MFMAs with eight independent v_fma_f32 behind each (MODE 2:
// 128 fmas and 16 MFMAs per iteration; if the matrix pipe ran entirely beside the vector ALU this would take as long
// as the longer of MODE 0 and MODE 1).  One workgroup of four waves is one wave per SIMD.
template <int MODE>
__global__ __launch_bounds__(256) void pa_issue_probe_kernel(int* sink, int iters) {
  float x[8];
  uint32_t u[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    x[i] = 0.001f * (float)(threadIdx.x + i + 1);
    u[i] = threadIdx.x * 8u + (uint32_t)i;
  }
  i32x8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = (int)(threadIdx.x * 0x01010101u + (uint32_t)i);
    b[i] = (int)(0x38383838u + (uint32_t)i);
  }
  f32x4 c[4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      if constexpr (MODE == 1 || MODE == 2)
        c[r & 3] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c[r & 3], 0, 0, 0, 0, 0, 0);
      if constexpr (MODE != 1) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          if constexpr (MODE == 0 || MODE == 2) x[i] = __builtin_fmaf(x[i], 1.0001f, 0.5f);
          if constexpr (MODE == 3) x[i] = fast_exp2(x[i]);
          if constexpr (MODE == 4) u[i] = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(x[i], x[(i + 3) & 7], (int)u[i], false);
          if constexpr (MODE == 5) {
            auto t = __builtin_amdgcn_permlane32_swap(u[i], u[(i + 1) & 7], false, false);
            u[i] = t[0];
            u[(i + 1) & 7] = t[1];
          }
        }
      }
    }
  }
  float r = c[0][0] + c[1][1] + c[2][2] + c[3][3];
#pragma unroll
  for (int i = 0; i < 8; ++i) r += x[i] + (float)u[i];
  if (r == 12345.678f) sink[threadIdx.x & 63] = (int)r;  // keeps the work alive
}

}  // namespace

#endif  // PA_PROBE_KERNEL_H_
