// Shared by the decode kernels: vector types, FP8 / bf16 conversions, scalar loads, the cross-lane
// exchanges of the softmax, the partial-tile store and the global-to-LDS loads.  Included by exactly one
// translation unit (pa_decode.hip), hence the unnamed namespace.
#ifndef PA_COMMON_H_
#define PA_COMMON_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/pa_decode.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(8))) int i32x8;

// -DPA_DECODE_TRACE (the measuring build tests/native/libpa_decode_trace.so, never the product library): one wave of
// every workgroup of pa_partition_shared_kernel leaves six timestamps of the 100 MHz wall clock, its step count
// and its live rows in pa_trace; pa_decode_trace_read copies them out.  PA_TRACE_MARK(i) is nothing otherwise.
#ifdef PA_DECODE_TRACE
constexpr int kTraceWorkgroups = 16384;
__device__ unsigned long long pa_trace[kTraceWorkgroups * 8];
#define PA_TRACE_DECL unsigned long long pa_trace_t[6] = {0, 0, 0, 0, 0, 0}
#define PA_TRACE_MARK(i) pa_trace_t[i] = wall_clock64()
#else
#define PA_TRACE_DECL
#define PA_TRACE_MARK(i)
#endif

constexpr int kHeadSize = 128;
// PaDecodeArgs.flags as the kernels see it (the launch layer sets it in its own copy of the arguments)
constexpr int kFlagSortedItems = 0x10000;  // the workspace holds the planning kernel's item list
// PA_DECODE_FLAG_OUTPUT_ONLY as the kernels see it: no partition-buffer entries for a sequence this stage finishes,
// nothing written for rows beyond a sequence's query length
constexpr int kFlagOutputOnly = 0x20000;
constexpr int kFlagSpanShift = 20;         // bits 20..27: partitions a one-wave workgroup walks in one pass (0 = 1)
// experiment switch of pa_partition_shared_kernel: P without its FP8 residual
constexpr int kFlagResidualNever = 0x40000;
// pa_partition_shared_kernel: the kv heads of an item are consecutive workgroups of ONE XCD (see the kernel)
constexpr int kFlagHeadsShareXcd = 0x80000;
// ... at most: their partial results wait in LDS for the end of the pass, in a pool of kSpanPoolBytes per 16-row
// tile; a tile of up to 8 real rows stages only those (half the bytes) and may walk twice as many partitions
constexpr int kSpanMax = 4;
constexpr int kSpanMaxFewRows = 8;
constexpr int kTeamWaves = 4;  // one-wave span walkers that share a workgroup and merge their partial results in it
// Workspace layout (int32 words): [0], [1] counters of the queued launch, [2] number of listed items,
// [16 + 2i], [17 + 2i] sequence and partition index of item i.
constexpr int kPlanHeaderWords = 16;
// word of the workspace header: how many sequences have more than one partition (their numbers are the last
// num_seqs words of a workspace that is long enough for them)
constexpr int kPlanMultiWord = 5;
constexpr int kStepTokens = 64;     // tokens per pipeline step (4 tiles of 16)
constexpr float kLog2e = 1.4426950408889634f;
constexpr int kPRowBytes = 144;     // 64 tokens * 2 B + 16 B pad per query row of the P tile

union Bf16x8Bits {
  bf16x8 v;
  bf16x2 p[4];
  u32x4 u;
};

// two FP8 e4m3fn bytes -> two bf16, exactly (an e4m3 value has 3 mantissa bits, bf16 keeps 7)
__device__ __forceinline__ uint32_t fp8x2_to_bf16x2(uint32_t word, bool high_half) {
  // v_cvt_scalef32_pk_bf16_fp8 with a scale of one: one instruction for the two values (all 256 codes are held
  // against the host's table by the library's debug entry point and its test)
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_native;
  union {
    bf16x2_native v;
    uint32_t u;
  } r;
  r.v = high_half ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(word, 1.0f, true)
                  : __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(word, 1.0f, false);
  return r.u;
}

__device__ __forceinline__ bf16x8 fp8x8_to_bf16x8(uint32_t lo, uint32_t hi) {
  Bf16x8Bits r;
  r.u[0] = fp8x2_to_bf16x2(lo, false);
  r.u[1] = fp8x2_to_bf16x2(lo, true);
  r.u[2] = fp8x2_to_bf16x2(hi, false);
  r.u[3] = fp8x2_to_bf16x2(hi, true);
  return r.v;
}

__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  union {
    bf16x2 v;
    uint32_t u;
  } r;
  r.v[0] = (__bf16)a;
  r.v[1] = (__bf16)b;
  return r.u;
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ u32x4 load16(const void* p) { return *reinterpret_cast<const u32x4*>(p); }
// The same for bytes that are read once and never again (the K/V cache stream): a non-temporal load.  A plain
// read-only stream reaches 6.0-6.3 TB/s on this GPU, a non-temporal one 6.7-7.0 TB/s (measured on 4 GiB).
__device__ __forceinline__ u32x4 load16_stream(const void* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}

// wave-uniform 32-bit load through the scalar (constant) path: no VGPR, no vmcnt slot
__device__ __forceinline__ int sload_i32(const int* p) {
  return *reinterpret_cast<const __attribute__((address_space(4))) int*>(reinterpret_cast<uintptr_t>(p));
}
__device__ __forceinline__ float sload_f32(const float* p) {
  return *reinterpret_cast<const __attribute__((address_space(4))) float*>(reinterpret_cast<uintptr_t>(p));
}

// Power-of-two factor that brings a row of query values with largest magnitude amax into [128, 256): a bf16
// (8 significant bits) or FP8 value times a power of two is then EXACTLY an e4m3 head (4 significant bits)
// plus an e4m3 residual, so the FP8 MFMAs see the query without rounding (elements more than 2^15 below the
// row maximum lose bits to e4m3's subnormal range: an absolute error below 2^-17 of the row maximum).
// inv receives 1 / factor.  amax == 0 (or not finite) gives 1.
__device__ __forceinline__ float query_pow2_factor(float amax, float& inv) {
  const int e = (int)((__float_as_uint(amax) >> 23) & 0xffu) - 127;
  if (!(amax > 0.f) || e < -100 || e > 100) {
    inv = 1.f;
    return 1.f;
  }
  inv = __uint_as_float((uint32_t)(127 - 7 + e) << 23);
  return __uint_as_float((uint32_t)(127 + 7 - e) << 23);
}

// max / sum over the four lanes {l, l^16, l^32, l^48}: v_permlane{16,32}_swap exchange 16- and
// 32-lane halves inside the VALU (no LDS round trip).  Written out as instructions: a swap of a register with
// its own copy leaves {x[l], x[l^32]} (then {y[l], y[l^16]}) in the two registers of every lane, one move, one
// swap and one max per level.  (From the builtins the compiler makes ten instructions of these six: it
// re-canonicalises both results of every swap before it takes their maximum.)
__device__ __forceinline__ float quad_row_max(float x) {
  float t;
  asm("v_mov_b32 %1, %0\n\t"
      "s_nop 1\n\t"
      "v_permlane32_swap_b32 %0, %1\n\t"
      "v_max_f32 %0, %0, %1\n\t"
      "v_mov_b32 %1, %0\n\t"
      "s_nop 1\n\t"
      "v_permlane16_swap_b32 %0, %1\n\t"
      "v_max_f32 %0, %0, %1"
      : "+v"(x), "=&v"(t));
  return x;
}
__device__ __forceinline__ float quad_row_sum(float x) {
  uint32_t u = __float_as_uint(x);
  auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  x = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  u = __float_as_uint(x);
  auto b = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// 4x4 transpose over (lane group l>>4, register): afterwards register k of lane group g holds what
// register g of lane group k held
__device__ __forceinline__ void quad_transpose(uint32_t (&d)[4]) {
  auto s02 = __builtin_amdgcn_permlane32_swap(d[0], d[2], false, false);
  auto s13 = __builtin_amdgcn_permlane32_swap(d[1], d[3], false, false);
  auto s01 = __builtin_amdgcn_permlane16_swap(s02[0], s13[0], false, false);
  auto s23 = __builtin_amdgcn_permlane16_swap(s02[1], s13[1], false, false);
  d[0] = s01[0];
  d[1] = s01[1];
  d[2] = s23[0];
  d[3] = s23[1];
}

// keep the first `n` (0..16) bytes of a 16-byte vector, zero the rest
__device__ __forceinline__ u32x4 keep_first_bytes(u32x4 v, int n) {
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    int k = n - 4 * w;
    uint32_t m = k >= 4 ? 0xffffffffu : (k <= 0 ? 0u : ((1u << (8 * k)) - 1u));
    v[w] &= m;
  }
  return v;
}

// Writes one 16-row x 128-dim f32 tile of O^T (acc[db][r] = head dim 16*db + 4*kg + r of row li) as bf16
// rows of the partial output.  The tile is transposed through a wave-private LDS buffer so that every
// store instruction writes four whole 256-byte rows (16 bytes per lane) instead of 32-byte fragments.
constexpr int kORowBytes = 272;  // 256 B of bf16 + 16 B pad
constexpr int kSpanPoolBytes = kSpanMaxFewRows * (8 * kORowBytes + 2 * 16 * 4);  // >= kSpanMax slots of 16 rows
// first half: the tile, scaled and rounded to bf16, into the LDS buffer (row li at li * kORowBytes); only the first
// `rows` rows are staged (the buffer may be no longer than that)
__device__ __forceinline__ void stage_partial_tile(char* lds, const f32x4 (&acc)[8], float inv, int lane, int rows = 16) {
  const int li = lane & 15, kg = lane >> 4;
#pragma unroll
  for (int db = 0; db < 8; ++db) {
    const f32x4 o = acc[db] * inv;
    u32x2 pk;
    pk[0] = pack_bf16x2(o[0], o[1]);
    pk[1] = pack_bf16x2(o[2], o[3]);
    if (li < rows) *reinterpret_cast<u32x2*>(lds + li * kORowBytes + (16 * db + 4 * kg) * 2) = pk;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
// second half: the staged rows to memory, four whole rows per store instruction (and to dst2, if given)
__device__ __forceinline__ void copy_staged_tile(const char* lds, char* dst, int64_t row_stride_bytes, char* dst2,
                                                 int64_t row_stride2_bytes, int rows_to_write, int lane) {
  const int li = lane & 15, kg = lane >> 4;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = 4 * i + kg;
    if (r < rows_to_write) {  // (rows at or beyond may not exist in the buffer)
      const u32x4 v = *reinterpret_cast<const u32x4*>(lds + r * kORowBytes + li * 16);
      *reinterpret_cast<u32x4*>(dst + (int64_t)r * row_stride_bytes + li * 16) = v;
      if (dst2) *reinterpret_cast<u32x4*>(dst2 + (int64_t)r * row_stride2_bytes + li * 16) = v;
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
}
__device__ __forceinline__ void store_partial_tile(char* lds, const f32x4 (&acc)[8], float inv, char* dst,
                                                   int64_t row_stride_bytes, char* dst2, int64_t row_stride2_bytes,
                                                   int rows_to_write, int lane, int rows_staged = 16) {
  stage_partial_tile(lds, acc, inv, lane, rows_staged);
  copy_staged_tile(lds, dst, row_stride_bytes, dst2, row_stride2_bytes, rows_to_write, lane);
}

// A sequence with no tokens at all (context length <= 0): nobody streams anything, and when the call has a
// single partition per sequence no second kernel runs either, so the workgroups of partition 0 zero the
// sequence's output rows [row_begin, row_end) of kv head h themselves.  Called by a whole workgroup.
__device__ __forceinline__ void zero_output_rows(const PaDecodeArgs& a, int b, int h, int row_begin, int row_end) {
  if (a.output == nullptr) return;
  const int Ge = a.q_len * a.group_size;
  char* outp = (char*)a.output + ((int64_t)b * a.stride_out_s + (int64_t)h * Ge * a.stride_out_h) * 2;
  const int li = threadIdx.x & 15;
  for (int r = row_begin + (int)(threadIdx.x >> 4); r < row_end; r += (int)(blockDim.x >> 4))
    *reinterpret_cast<u32x4*>(outp + (int64_t)r * a.stride_out_h * 2 + li * 16) = u32x4{0, 0, 0, 0};
}

// Global memory -> LDS without passing through registers: lane i's 16 (4) bytes land at lds_offset + 16 (4) * i.
// They are non-temporal (the cache is streamed once).
// The loads count in vmcnt like any other vector load, but the compiler does not see them: whoever reads
// the LDS bytes waits with dma_wait<N>() (at most N vector memory operations still outstanding) first.
// M0 carries the LDS address and is named as clobbered, so the compiler keeps no value of its own in it across
// the statement (it reserves M0 and warns about any clobber that names it; that is what is wanted here).
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void dma_load16(const void* gptr, uint32_t lds_offset) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt" ::"v"(gptr), "s"(lds_offset) : "memory", "m0");
}
template <bool STREAM = true>
__device__ __forceinline__ void dma_load4(const void* gptr, uint32_t lds_offset) {
  if constexpr (STREAM)
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off nt" ::"v"(gptr), "s"(lds_offset) : "memory", "m0");
  else
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(gptr), "s"(lds_offset) : "memory", "m0");
}
// the same with the address split into a wave-uniform base and a 32-bit per-lane byte offset; STREAM = false
// for bytes whose 128-byte lines other loads will touch again soon (those must stay in L2)
template <bool STREAM = true>
__device__ __forceinline__ void dma_load16(const void* base, uint32_t lane_offset, uint32_t lds_offset) {
  // the base is wave-uniform by construction; readfirstlane makes the compiler keep it in scalar registers
  const uint64_t b = reinterpret_cast<uint64_t>(base);
  // (the builtin returns a signed int: widen through uint32_t, or a low word with bit 31 set would smear
  // ones over the high word)
  const uint32_t b_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
  const uint32_t b_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32));
  const uint64_t sb = ((uint64_t)b_hi << 32) | (uint64_t)b_lo;
  if constexpr (STREAM)
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt" ::"v"(lane_offset), "s"(sb),
                 "s"(lds_offset)
                 : "memory", "m0");
  else
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_offset), "s"(sb),
                 "s"(lds_offset)
                 : "memory", "m0");
}
#pragma clang diagnostic pop
template <int N>
__device__ __forceinline__ void dma_wait() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
__device__ __forceinline__ uint32_t lds_offset_of(const void* p) {
  return (uint32_t)reinterpret_cast<uintptr_t>(
      (const __attribute__((address_space(3))) char*)(const char*)p);
}

}  // namespace

#endif  // PA_COMMON_H_
