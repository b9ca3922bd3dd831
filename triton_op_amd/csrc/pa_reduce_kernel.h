// pa_reduce_kernel: stage 2, the merge of the partitions.
#ifndef PA_REDUCE_KERNEL_H_
#define PA_REDUCE_KERNEL_H_

#include "pa_common.h"

namespace {

// ---------------------------------------------------------------------------------------------
// reduce: a workgroup owns 16 consecutive output rows of one (sequence, kv head); a wave works on one row at
// a time, two head dims per lane.  Lane p of a 64-partition chunk owns (m_p, l_p); the weights
// w_p = l_p e^{m_p - M} are broadcast with v_readlane while the partial outputs stream in.  A sequence with one
// partition was finished by the partition kernel: its workgroups leave after one scalar load.
//   ROWS = 1: 16 waves, one row each -- the least code and the shortest critical path, for batches with few rows
//             (a launch this short is dominated by fetching its own code and by one or two memory latencies).
//   ROWS = 4: 4 waves, four rows each -- for big batches, where the number of resident waves is the limit: with up
//             to 8 partitions (the tuning layer picks few, large ones) all loads of the four rows go out before
//             anything is waited for.
// ---------------------------------------------------------------------------------------------
// one row, any number of partitions; returns two packed bf16 head dims
__device__ __forceinline__ uint32_t reduce_row(const PaDecodeArgs& a, int b, int h, int row, int n, int lane) {
  const int Ge = a.q_len * a.group_size;
  const int64_t es_off = (int64_t)b * a.stride_es_s + (int64_t)h * a.stride_es_h + row;
  const float* ml = a.max_logits + es_off;
  const float* es = a.exp_sums + es_off;
  const char* tmp = (const char*)a.tmp_output +
                    ((int64_t)b * a.stride_tmp_s + (int64_t)h * a.stride_tmp_h + (int64_t)row * a.stride_tmp_g) * 2 +
                    lane * 4;
  const int64_t tp = a.stride_tmp_p * 2;
  const int64_t sp = a.stride_es_p;

  // this lane's (m, l) of the first chunk and the first eight partials (indices past the end repeat the last
  // partition and get weight 0), requested together
  float m0 = lane < n ? ml[(int64_t)lane * sp] : -INFINITY;
  float l0 = lane < n ? es[(int64_t)lane * sp] : 0.f;
  uint32_t t0[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) t0[i] = *reinterpret_cast<const uint32_t*>(tmp + (int64_t)(i < n ? i : n - 1) * tp);
  float M = m0;
  for (int p = lane + 64; p < n; p += 64) M = fmaxf(M, ml[p * sp]);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) M = fmaxf(M, __shfl_xor(M, o));
  const float M_safe = M == -INFINITY ? 0.f : M;

  float acc0 = 0.f, acc1 = 0.f, wsum = 0.f;
  for (int c0 = 0; c0 < n; c0 += 64) {
    const int cnt = n - c0 < 64 ? n - c0 : 64;
    float m = m0, l = l0;
    if (c0) {
      m = lane < cnt ? ml[(int64_t)(c0 + lane) * sp] : -INFINITY;
      l = lane < cnt ? es[(int64_t)(c0 + lane) * sp] : 0.f;
    }
    const float w = l > 0.f ? l * __expf(m - M_safe) : 0.f;  // 0 in lanes at or past cnt
    wsum += w;
    const char* tc = tmp + (int64_t)c0 * tp;
    int u = 0;
    if (c0 == 0) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float wi = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(w), i));
        acc0 += bf16_bits_to_f32(t0[i] & 0xffffu) * wi;
        acc1 += __uint_as_float(t0[i] & 0xffff0000u) * wi;
      }
      u = 8;
    }
    for (; u + 8 <= cnt; u += 8) {
      uint32_t t[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) t[i] = *reinterpret_cast<const uint32_t*>(tc + (int64_t)(u + i) * tp);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float wi = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(w), u + i));
        acc0 += bf16_bits_to_f32(t[i] & 0xffffu) * wi;
        acc1 += __uint_as_float(t[i] & 0xffff0000u) * wi;
      }
    }
    for (; u < cnt; ++u) {
      const uint32_t t = *reinterpret_cast<const uint32_t*>(tc + (int64_t)u * tp);
      const float wi = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(w), u));
      acc0 += bf16_bits_to_f32(t & 0xffffu) * wi;
      acc1 += __uint_as_float(t & 0xffff0000u) * wi;
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) wsum += __shfl_xor(wsum, o);
  // attention sink: one more term in the softmax denominator, exp(sink - M), with no value attached
  if (a.sinks) wsum += __expf(a.sinks[h * Ge + row] - M_safe);
  const float inv = wsum > 0.f ? 1.f / wsum : 0.f;
  return pack_bf16x2(acc0 * inv, acc1 * inv);
}

// rows row0, row0+4, row0+8, row0+12 with 1 <= n <= 8 partitions: every load goes out first; maximum and sum
// are taken over v_readlane broadcasts, which every lane computes alike
__device__ __forceinline__ void reduce_four_rows(const PaDecodeArgs& a, int b, int h, int row0, int n, int rows_valid,
                                                 char* outp, int lane) {
  const int Ge = a.q_len * a.group_size;
  const int64_t sp = a.stride_es_p;
  const int64_t tp = a.stride_tmp_p * 2;
  float m[4], l[4];
  uint32_t t[4][8];
#pragma unroll
  for (int rr = 0; rr < 4; ++rr) {
    const int row = row0 + 4 * rr;
    const bool live = row < rows_valid;
    const int64_t es_off = (int64_t)b * a.stride_es_s + (int64_t)h * a.stride_es_h + (live ? row : 0);
    const bool mine = live && lane < n;
    m[rr] = mine ? a.max_logits[es_off + (int64_t)lane * sp] : -INFINITY;
    l[rr] = mine ? a.exp_sums[es_off + (int64_t)lane * sp] : 0.f;
    const char* tmp = (const char*)a.tmp_output +
                      ((int64_t)b * a.stride_tmp_s + (int64_t)h * a.stride_tmp_h + (int64_t)(live ? row : 0) * a.stride_tmp_g) * 2 +
                      lane * 4;
#pragma unroll
    for (int i = 0; i < 8; ++i)
      t[rr][i] = live ? *reinterpret_cast<const uint32_t*>(tmp + (int64_t)(i < n ? i : n - 1) * tp) : 0u;
  }
#pragma unroll
  for (int rr = 0; rr < 4; ++rr) {
    const int row = row0 + 4 * rr;
    float M = -INFINITY;
#pragma unroll
    for (int i = 0; i < 8; ++i) M = fmaxf(M, __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(m[rr]), i)));
    const float M_safe = M == -INFINITY ? 0.f : M;
    const float w = l[rr] > 0.f ? l[rr] * __expf(m[rr] - M_safe) : 0.f;
    float wsum = 0.f, acc0 = 0.f, acc1 = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float wi = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(w), i));
      wsum += wi;
      acc0 += bf16_bits_to_f32(t[rr][i] & 0xffffu) * wi;
      acc1 += __uint_as_float(t[rr][i] & 0xffff0000u) * wi;
    }
    if (a.sinks && row < rows_valid) wsum += __expf(a.sinks[h * Ge + row] - M_safe);
    const float inv = wsum > 0.f ? 1.f / wsum : 0.f;
    if (row < Ge) *reinterpret_cast<uint32_t*>(outp + (int64_t)row * a.stride_out_h * 2) = pack_bf16x2(acc0 * inv, acc1 * inv);
  }
}

// one unit of the reduce: 16 output rows (row tile rt) of kv head h of sequence b, by one workgroup
template <bool SKIP_SINGLE, int ROWS>
__device__ __forceinline__ void reduce_unit(const PaDecodeArgs& a, int b, int h, int rt, int lane, int wave) {
  const int Ge = a.q_len * a.group_size;
  const int row0 = 16 * rt + wave;  // ROWS = 4: this wave's rows are row0 + 4 * rr
  if (row0 >= Ge) return;

  const int ctx = sload_i32(a.context_lens + b);
  int n = (ctx + a.partition_size - 1) / a.partition_size;
  n = n > a.max_num_partitions ? a.max_num_partitions : n;
  // SKIP_SINGLE: the partition kernel of the same call has written the rows of sequences with one partition
  if (SKIP_SINGLE && n == 1 && !a.sinks) return;
  const int qb = a.q_lens ? sload_i32(a.q_lens + b) : a.q_len;
  const int rows_valid = n <= 0 ? 0 : qb * a.group_size;  // rows at or beyond read as zero

  char* outp = (char*)a.output + ((int64_t)b * a.stride_out_s + (int64_t)h * Ge * a.stride_out_h) * 2 + lane * 4;
  if (ROWS == 4 && n >= 1 && n <= 8) {
    reduce_four_rows(a, b, h, row0, n, rows_valid, outp, lane);
    return;
  }
  for (int rr = 0; rr < ROWS; ++rr) {
    const int row = row0 + 4 * rr;
    if (row >= Ge) break;
    const uint32_t v = row < rows_valid ? reduce_row(a, b, h, row, n, lane) : 0u;
    *reinterpret_cast<uint32_t*>(outp + (int64_t)row * a.stride_out_h * 2) = v;
  }
}

template <bool SKIP_SINGLE, int ROWS>
__global__ __launch_bounds__(1024 / ROWS) void pa_reduce_kernel(const PaDecodeArgs a) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int RT = (a.q_len * a.group_size + 15) / 16;
  const long long wid = blockIdx.x;
  const int rt = (int)(wid % RT);
  const int h = (int)((wid / RT) % a.num_kv_heads);
  const int b = (int)(wid / ((long long)RT * a.num_kv_heads));
  reduce_unit<SKIP_SINGLE, ROWS>(a, b, h, rt, lane, wave);
}

// The same over the planning kernel's list of the sequences that have more than one partition (the others got
// their output rows from the partition kernel): a launch of a few hundred workgroups that walk the list's units,
// instead of one workgroup per (sequence, head, row tile) of which most would only find out that they have
// nothing to do (8192 of them cost 9 us on a ragged batch of 256 sequences).
template <int ROWS>
__global__ __launch_bounds__(1024 / ROWS) void pa_reduce_listed_kernel(const PaDecodeArgs a) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int RT = (a.q_len * a.group_size + 15) / 16;
  const int per_seq = RT * a.num_kv_heads;
  const int* list = a.workspace + (a.workspace_bytes / 4 - a.num_seqs);
  const long long units = (long long)sload_i32(a.workspace + kPlanMultiWord) * per_seq;
  for (long long u = blockIdx.x; u < units; u += gridDim.x) {
    const int b = sload_i32(list + u / per_seq);
    const int r = (int)(u % per_seq);
    reduce_unit<false, ROWS>(a, b, r / RT, r % RT, lane, wave);
  }
}

}  // namespace

#endif  // PA_REDUCE_KERNEL_H_
