// pa_plan_kernel: the work-item list of the sorted dispatch.
#ifndef PA_PLAN_KERNEL_H_
#define PA_PLAN_KERNEL_H_

#include "pa_common.h"

namespace {

constexpr int kPlanMaxSeqs = 4096;  // sequences the planning kernel's LDS tables can hold
constexpr int kPlanClasses = 64;    // length classes of the partial partitions

// One workgroup lists the live (sequence, partition) items of a call in the order the partition kernel's
// workgroups should take them: every whole partition first (they all cost the same), then the last, partial
// partition of every sequence by decreasing length (a counting sort into 64 length classes).  The hardware
// hands workgroup ids to free slots in order, so the launch becomes longest-first list scheduling: the
// end of a ragged batch's launch is filled with short items instead of whatever the batch order left over.
// The order inside a class depends on the timing of LDS atomics; the results do not (an item's arithmetic
// does not depend on its position in the list).
__global__ __launch_bounds__(1024) void pa_plan_kernel(const PaDecodeArgs a) {
  __shared__ int s_pf[kPlanMaxSeqs + 1];  // exclusive prefix of whole partitions per sequence
  __shared__ int s_wave[16];
  __shared__ int s_hist[kPlanClasses];
  __shared__ int s_base[kPlanClasses];
  __shared__ int s_multi;  // sequences with more than one partition
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int B = a.num_seqs, ps = a.partition_size, P = a.max_num_partitions;
  const int per = (B + 1023) / 1024;  // sequences per thread (contiguous), at most 4
  int nfull[4], tail[4];
  int mine = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int b = tid * per + i;
    nfull[i] = 0;
    tail[i] = 0;
    if (i < per && b < B) {
      int c = a.context_lens[b];
      c = c < 0 ? 0 : c;
      int np = (c + ps - 1) / ps;
      np = np > P ? P : np;
      int f = c / ps;
      f = f > P ? P : f;
      nfull[i] = f;
      tail[i] = np > f ? c - f * ps : 0;
      if (c == 0) tail[i] = 1;  // an empty sequence: one (shortest) item, whose workgroups zero its output rows
      mine += f;
    }
  }
  // exclusive scan of `mine` over the 1024 threads
  int incl = mine;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int y = __shfl_up(incl, d);
    if (lane >= d) incl += y;
  }
  if (lane == 63) s_wave[wave] = incl;
  if (tid < kPlanClasses) s_hist[tid] = 0;
  if (tid == 0) s_multi = 0;
  __syncthreads();
  // the sequences the reduce kernel has work for, in any order, at the end of a workspace that has room for them
  const bool has_multi_list = a.workspace_bytes >= 4LL * kPlanHeaderWords + 8LL * B * P + 4LL * B;
  if (has_multi_list) {
    int* multi = a.workspace + (a.workspace_bytes / 4 - B);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int b = tid * per + i;
      if (i < per && b < B && nfull[i] + (tail[i] > 0 ? 1 : 0) > 1) multi[atomicAdd(&s_multi, 1)] = b;
    }
  }
  int wave_off = 0, total_full = 0;
#pragma unroll
  for (int w = 0; w < 16; ++w) {
    const int v = s_wave[w];
    wave_off += w < wave ? v : 0;
    total_full += v;
  }
  int run = wave_off + incl - mine;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int b = tid * per + i;
    if (i < per && b < B) {
      s_pf[b] = run;
      run += nfull[i];
    }
  }
  if (tid == 0) s_pf[B] = total_full;
  int cls[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    cls[i] = 0;
    if (tail[i] > 0) {
      const long long q = (long long)(tail[i] - 1) * kPlanClasses / ps;  // 0 .. 63, longer = larger
      cls[i] = kPlanClasses - 1 - (int)(q > kPlanClasses - 1 ? kPlanClasses - 1 : q);
      atomicAdd(&s_hist[cls[i]], 1);
    }
  }
  __syncthreads();
  if (tid == 0) {
    int acc = 0;
    for (int c = 0; c < kPlanClasses; ++c) {
      s_base[c] = acc;
      acc += s_hist[c];
      s_hist[c] = 0;  // becomes the class's cursor
    }
    a.workspace[2] = total_full + acc;
    a.workspace[kPlanMultiWord] = has_multi_list ? s_multi : -1;
  }
  __syncthreads();
  int* items = a.workspace + kPlanHeaderWords;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (tail[i] > 0) {
      const int pos = total_full + s_base[cls[i]] + atomicAdd(&s_hist[cls[i]], 1);
      items[2 * pos] = tid * per + i;
      items[2 * pos + 1] = nfull[i];
    }
  }
  // whole partitions, sequence-major: item -> sequence by binary search in the prefix table
  for (int it = tid; it < total_full; it += 1024) {
    int lo = 0, hi = B;  // s_pf[lo] <= it < s_pf[hi]
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (s_pf[mid] <= it)
        lo = mid;
      else
        hi = mid;
    }
    items[2 * it] = lo;
    items[2 * it + 1] = it - s_pf[lo];
  }
}

}  // namespace

#endif  // PA_PLAN_KERNEL_H_
