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

// ---------------------------------------------------------------------------------------------
// The merge of MANY partitions for FEW rows (a handful of very long sequences cut into the reference's 256-token
// partitions: 4 sequences x 8 kv heads x 512 partitions).  pa_reduce_kernel gives such a call one wave per output
// row, which walks the row's partitions one after the other: 32 workgroups of 8 busy waves on 32 of the GPU's
// CUs, each wave waiting for its own chain of loads, and a CU can take in only so many bytes per cycle.  Here a
// 16-row unit is cut along the HEAD DIMENSION into kWideDimSplit workgroups (no exchange between them: their
// output columns are disjoint), and inside a workgroup the sixteen waves split the PARTITION axis into
// interleaved streams: one 16-byte load per lane fetches eight head dims of one row, a wave's load
// instruction covers all sixteen rows of kWideParts partitions (two partitions of a unit with at most eight rows),
// eight such loads go out before anything is waited for.
//   phase A  M[row] = max over the partitions of max_logits                  (lanes: row, partition slot)
//   phase B  acc += exp_sums * exp(max_logits - M) * partial                  (lanes: row, 8 head dims)
//   phase C  the waves' acc and sums of the weights meet in LDS; a thread owns one head dim of one row
// ---------------------------------------------------------------------------------------------
constexpr int kWideWaves = 16;
constexpr int kWideDimSplit = 4;                          // workgroups per 16-row unit
constexpr int kWideDims = kHeadSize / kWideDimSplit;      // head dims of one workgroup
constexpr int kWideRowLanes = kWideDims / 8;              // lanes that share a row (eight head dims each)
constexpr int kWideParts = 64 / (16 * kWideRowLanes);     // partitions one load instruction of a wave covers (16-row unit)
constexpr int kWideStreamsMax = kWideWaves * kWideParts * 2;  // ... twice as many when the unit has at most 8 rows
static_assert(kWideRowLanes >= 1 && kWideParts >= 1 && kWideParts * 16 * kWideRowLanes == 64, "lane map of the wide reduce");
template <bool SKIP_SINGLE>
__global__ __launch_bounds__(64 * kWideWaves) void pa_reduce_wide_kernel(const PaDecodeArgs a) {
  __shared__ float s_max[kWideStreamsMax][16];
  __shared__ float s_sum[kWideStreamsMax][16];
  __shared__ float s_acc[kWideStreamsMax][16][kWideDims + 4];  // a stream's partial results (rows padded against bank conflicts)
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int Ge = a.q_len * a.group_size;
  const int RT = (Ge + 15) / 16;
  // Workgroup ids go round the GPU's eight XCDs, each with an L2 of its own; the workgroups of one unit share the
  // 128-byte lines of its rows, so they get ids that land on ONE XCD: id = xcd + 8 * (chunk + kWideDimSplit * (unit / 8)),
  // unit % 8 == xcd (the grid is padded to whole groups of eight units).
  long long wid = blockIdx.x;
  const int xcd = (int)(wid % 8);
  wid /= 8;
  const int chunk = (int)(wid % kWideDimSplit);
  wid = (wid / kWideDimSplit) * 8 + xcd;
  if (wid >= (long long)RT * a.num_kv_heads * a.num_seqs) return;
  const int rt = (int)(wid % RT);
  const int h = (int)((wid / RT) % a.num_kv_heads);
  const int b = (int)(wid / ((long long)RT * a.num_kv_heads));
  const int row0 = 16 * rt;

  const int ctx = sload_i32(a.context_lens + b);
  int n = (ctx + a.partition_size - 1) / a.partition_size;
  n = n > a.max_num_partitions ? a.max_num_partitions : n;
  if (SKIP_SINGLE && n == 1 && !a.sinks) return;  // the partition kernel has written these rows
  const int qb = a.q_lens ? sload_i32(a.q_lens + b) : a.q_len;
  const int rows_valid = n <= 0 ? 0 : qb * a.group_size;     // rows at or beyond read as zero
  const int rows_here = min(16, Ge - row0);                  // rows of this unit that exist in the buffers
  const int rows_live = max(0, min(16, rows_valid - row0));  // ... and hold a result
  // this lane's partition stream, its row of the unit and its eight head dims of the chunk: a unit of at most 8 rows
  // gives the lanes of rows 8..15 a second partition instead (partition p belongs to stream p % streams)
  const int row_bits = rows_here <= 8 ? 3 : 4;
  const int dl = lane % kWideRowLanes, r = (lane / kWideRowLanes) & ((1 << row_bits) - 1), pp = lane / (kWideRowLanes << row_bits);
  const int parts = 64 / (kWideRowLanes << row_bits);
  const int streams = kWideWaves * parts;
  const int stream = wave * parts + pp;
  const bool live = r < rows_live;

  const int64_t sp = a.stride_es_p;
  const float* ml = a.max_logits + (int64_t)b * a.stride_es_s + (int64_t)h * a.stride_es_h + row0 + (live ? r : 0);
  const float* es = a.exp_sums + (int64_t)b * a.stride_es_s + (int64_t)h * a.stride_es_h + row0 + (live ? r : 0);
  const char* tmp = (const char*)a.tmp_output +
                    ((int64_t)b * a.stride_tmp_s + (int64_t)h * a.stride_tmp_h + (int64_t)(row0 + (live ? r : 0)) * a.stride_tmp_g) * 2 +
                    (chunk * kWideDims + 8 * dl) * 2;
  const int64_t tp = a.stride_tmp_p * 2;

  // ---- phase A: the lanes of a row walk the stream's partitions in turn
  float M = -INFINITY;
  if (live)
    for (int p = stream + streams * dl; p < n; p += kWideRowLanes * streams) M = fmaxf(M, ml[(int64_t)p * sp]);
#pragma unroll
  for (int o = 1; o < kWideRowLanes; o <<= 1) M = fmaxf(M, __shfl_xor(M, o));
  if (dl == 0) s_max[stream][r] = M;
  __syncthreads();
  M = s_max[0][r];
  for (int w = 1; w < streams; ++w) M = fmaxf(M, s_max[w][r]);
  const float M_safe = M == -INFINITY ? 0.f : M;

  // ---- phase B: this stream's partitions, eight at a time; every load of a batch goes out first
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  float wsum = 0.f;
  for (int p0 = stream; p0 - pp < n; p0 += 8 * streams) {  // (the lanes of a wave leave together)
    float m[8], l[8];
    u32x4 t[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int p = p0 + streams * q;
      const bool on = live && p < n;
      const int pc = p < n ? p : 0;  // (an address inside the buffers for the lanes that load nothing real)
      m[q] = on ? ml[(int64_t)pc * sp] : -INFINITY;
      l[q] = on ? es[(int64_t)pc * sp] : 0.f;
      t[q] = on ? load16(tmp + (int64_t)pc * tp) : u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const float w = l[q] > 0.f ? l[q] * __expf(m[q] - M_safe) : 0.f;
      wsum += w;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        acc[2 * e] += bf16_bits_to_f32(t[q][e] & 0xffffu) * w;
        acc[2 * e + 1] += __uint_as_float(t[q][e] & 0xffff0000u) * w;
      }
    }
  }

  // ---- phase C: the streams' sums meet in LDS (the lanes of a row hold the same sum of weights)
  if (dl == 0) s_sum[stream][r] = wsum;
  *reinterpret_cast<f32x4*>(&s_acc[stream][r][8 * dl]) = f32x4{acc[0], acc[1], acc[2], acc[3]};
  *reinterpret_cast<f32x4*>(&s_acc[stream][r][8 * dl + 4]) = f32x4{acc[4], acc[5], acc[6], acc[7]};
  __syncthreads();
  // thread t < 16 * kWideDims: row t / kWideDims, head dim t % kWideDims of the chunk
  const int row = (int)threadIdx.x / kWideDims, d = (int)threadIdx.x % kWideDims;
  if (threadIdx.x >= 16 * kWideDims || row >= rows_here) return;
  float o = 0.f, tot = 0.f;
  for (int w = 0; w < streams; ++w) {
    o += s_acc[w][row][d];
    tot += s_sum[w][row];
  }
  float Mr = s_max[0][row];
  for (int w = 1; w < streams; ++w) Mr = fmaxf(Mr, s_max[w][row]);
  // attention sink: one more term in the softmax denominator, exp(sink - M), with no value attached
  if (a.sinks && row < rows_live) tot += __expf(a.sinks[h * Ge + row0 + row] - (Mr == -INFINITY ? 0.f : Mr));
  const float inv = tot > 0.f ? 1.f / tot : 0.f;
  __bf16* outp = (__bf16*)a.output + (int64_t)b * a.stride_out_s + (int64_t)(h * Ge + row0 + row) * a.stride_out_h +
                 chunk * kWideDims + d;
  *outp = row < rows_live ? (__bf16)(o * inv) : (__bf16)0.f;
}

}  // namespace

#endif  // PA_REDUCE_KERNEL_H_
