// KV-cache write and quantisation kernels for the paged layouts the decode kernels read:
//   key_cache   [blocks, Hkv, D/x, bs, x]     x = 16 / sizeof(element)
//   value_cache [blocks, Hkv, D, bs], or transposed [blocks, Hkv, bs/x, D, x]
//   scales      [blocks, Hkv, bs, 1] f32 (one per token and kv head) or one f32 per tensor
// FP8 is OCP e4m3fn.  Quantisation is symmetric: scale = amax / 448 (1 for an all-zero row),
// q = round_to_nearest_even(x / scale), both with IEEE division so the bytes match a float32 host
// computation of the same formula bit for bit.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/pa_decode.h"
#include "pa_launch.h"

namespace {

constexpr float kFp8Max = 448.f;

__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }

__device__ __forceinline__ uint8_t f32_to_fp8(float x) {
  x = fminf(fmaxf(x, -kFp8Max), kFp8Max);
  return (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(x, 0.f, 0, false) & 0xff);
}

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

// element index of (head dim d, token offset off) inside one (block, head) of the V cache: rows of block_size
// tokens per head dim, or, transposed, tiles of X tokens (X = 16 / element size) with the head dims inside a tile
template <int X, int D = 128>
__device__ __forceinline__ int64_t v_index(const PaKvWriteArgs& a, int d, int off) {
  return a.v_transposed ? ((int64_t)(off / X) * D + d) * X + off % X : (int64_t)d * a.block_size + off;
}

// ---- one (token, kv head) by one wave; lane l owns head dims 2l, 2l+1 (+ 128 per further pass: head size 256 takes
// two passes, head size 64 uses half the lanes) ---------------------------------------------------------------------
template <bool TO_FP8, int D = 128>
__device__ __forceinline__ void write_token(const PaKvWriteArgs& a, long long t, int h, long long slot, int lane) {
  constexpr int PASSES = (D + 127) / 128;
  const long long block = slot / a.block_size;
  const int off = (int)(slot - block * a.block_size);
  const int bs = a.block_size;

  uint32_t kraw[PASSES], vraw[PASSES];
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    const int d0 = 128 * p + 2 * lane;
    kraw[p] = vraw[p] = 0u;
    if (d0 < D) {
      kraw[p] = *reinterpret_cast<const uint32_t*>((const uint16_t*)a.key + t * a.stride_k_t + h * a.stride_k_h + d0);
      vraw[p] = *reinterpret_cast<const uint32_t*>((const uint16_t*)a.value + t * a.stride_v_t + h * a.stride_v_h + d0);
    }
  }
  if constexpr (!TO_FP8) {
    // 16-bit cache: x = 8; the two dims of a lane are adjacent in a chunk
    uint16_t* kc = (uint16_t*)a.key_cache + block * a.stride_kc_b + h * a.stride_kc_h;
    uint16_t* vc = (uint16_t*)a.value_cache + block * a.stride_vc_b + h * a.stride_vc_h;
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      const int d0 = 128 * p + 2 * lane;
      if (d0 >= D) continue;
      *reinterpret_cast<uint32_t*>(kc + (int64_t)(d0 / 8) * bs * 8 + off * 8 + d0 % 8) = kraw[p];
      vc[v_index<8, D>(a, d0, off)] = (uint16_t)(vraw[p] & 0xffffu);
      vc[v_index<8, D>(a, d0 + 1, off)] = (uint16_t)(vraw[p] >> 16);
    }
  } else {
    float ks, vs;
    if (a.kv_quant_mode == PA_QUANT_PER_TOKEN) {
      float ka = 0.f, va = 0.f;
#pragma unroll
      for (int p = 0; p < PASSES; ++p) {
        ka = fmaxf(ka, fmaxf(fabsf(bf16_to_f32(kraw[p] & 0xffffu)), fabsf(bf16_to_f32(kraw[p] >> 16))));
        va = fmaxf(va, fmaxf(fabsf(bf16_to_f32(vraw[p] & 0xffffu)), fabsf(bf16_to_f32(vraw[p] >> 16))));
      }
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) {
        ka = fmaxf(ka, __shfl_xor(ka, o));
        va = fmaxf(va, __shfl_xor(va, o));
      }
      ks = ka > 0.f ? __fdiv_rn(ka, kFp8Max) : 1.f;
      vs = va > 0.f ? __fdiv_rn(va, kFp8Max) : 1.f;
      if (lane == 0) {
        const int64_t so = block * a.stride_scale_b + h * a.stride_scale_h + off;
        a.key_scale[so] = ks;
        a.value_scale[so] = vs;
      }
    } else if (a.kv_quant_mode == PA_QUANT_PER_TENSOR) {
      ks = a.key_scale[0];
      vs = a.value_scale[0];
    } else {
      ks = vs = 1.f;
    }
    uint8_t* kc = (uint8_t*)a.key_cache + block * a.stride_kc_b + h * a.stride_kc_h;
    uint8_t* vc = (uint8_t*)a.value_cache + block * a.stride_vc_b + h * a.stride_vc_h;
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      const int d0 = 128 * p + 2 * lane;
      if (d0 >= D) continue;
      const float k0 = bf16_to_f32(kraw[p] & 0xffffu), k1 = bf16_to_f32(kraw[p] >> 16);
      const float v0 = bf16_to_f32(vraw[p] & 0xffffu), v1 = bf16_to_f32(vraw[p] >> 16);
      const uint8_t qk0 = f32_to_fp8(__fdiv_rn(k0, ks)), qk1 = f32_to_fp8(__fdiv_rn(k1, ks));
      const uint8_t qv0 = f32_to_fp8(__fdiv_rn(v0, vs)), qv1 = f32_to_fp8(__fdiv_rn(v1, vs));
      *reinterpret_cast<uint16_t*>(kc + (int64_t)(d0 / 16) * bs * 16 + off * 16 + d0 % 16) = (uint16_t)(qk0 | (qk1 << 8));
      vc[v_index<16, D>(a, d0, off)] = qv0;
      vc[v_index<16, D>(a, d0 + 1, off)] = qv1;
    }
  }
}

// ---- append, a few tokens (decode): one wave per (token, kv head) ------------------------------------------------
template <bool TO_FP8, int D = 128>
__global__ __launch_bounds__(256) void kv_cache_write_kernel(const PaKvWriteArgs a) {
  const int lane = threadIdx.x & 63;
  const long long item = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= (long long)a.num_tokens * a.num_kv_heads) return;
  const int h = (int)(item % a.num_kv_heads);
  const long long t = item / a.num_kv_heads;
  const long long slot = a.slot_mapping[t];
  if (slot < 0) return;  // padding token
  write_token<TO_FP8, D>(a, t, h, slot, lane);
}

// lane exchanges inside a row of 16 lanes on the vector ALU (DPP), not through the LDS crossbar
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, true);
}
constexpr int kDppSwap1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kDppSwap2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // lane i <-> 7 - i of each 8
constexpr int kDppMirror = 0x140;      // lane i <-> 15 - i
// maximum over the 16 lanes of a row (the operation commutes, so mirrors do for the last two steps)
__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, __uint_as_float(dpp_u32<kDppSwap1>(__float_as_uint(v))));
  v = fmaxf(v, __uint_as_float(dpp_u32<kDppSwap2>(__float_as_uint(v))));
  v = fmaxf(v, __uint_as_float(dpp_u32<kDppHalfMirror>(__float_as_uint(v))));
  v = fmaxf(v, __uint_as_float(dpp_u32<kDppMirror>(__float_as_uint(v))));
  return v;
}

// amax / 448 for a row maximum that is a bf16 value: the correctly rounded float32 quotient from the constant
// reciprocal and one correction of the quotient (the residual amax - 448 q is exact in one fma); checked on the
// host against the division for every positive bf16 value, subnormal ones included.
__device__ __forceinline__ float bf16_amax_to_scale(float amax) {
  constexpr float r = 1.f / kFp8Max;
  if (__builtin_expect(!(amax < 0x1p127f), 0)) return __fdiv_rn(amax, kFp8Max);  // infinity stays infinity
  const float q0 = amax * r;
  return __builtin_fmaf(__builtin_fmaf(-kFp8Max, q0, amax), r, q0);
}

// Eight values of one row divided by the row's scale and rounded to e4m3fn, four bytes per word.
// x / s must be the correctly rounded float32 quotient (what the host-side formula computes).  A float division
// expands to a reciprocal, one correction of it and two corrections of the quotient.  With one divisor for the
// whole row the reciprocal part is done once, and for a bf16 x one correction of the quotient is enough: the
// once corrected reciprocal is within an ulp of 1/s, so q0 = x r is within an ulp of x/s, the residual x - s q0
// is exact in one fma and q0 + residual r rounds to the quotient (on the host: every bf16 x against every
// scale a bf16 row maximum can give, and 3e5 arbitrary scales, with a first reciprocal 1 ulp off either way;
// only scales whose significand is all ones can miss) -- three instructions per value instead of ten.
// That short form needs nothing to over- or underflow on the way: it is used for scales within 2^-40 .. 2^40 and
// values below 2^80 (`xbound` is any bound of |x|; a quotient too small for its residual to be exact is far
// below the smallest FP8 value and rounds to zero either way); anything else takes the full division.
// CLAMP = false: the caller knows |x / s| <= 448 (1 + 2^-23), which converts to +-448 as it is (per-token scales:
// s = amax / 448 of a row that holds x).
template <bool CLAMP>
__device__ __forceinline__ void quantize8(const float (&x)[8], float s, float xbound, u32x2& out) {
  float q[8];
  const float as = fabsf(s);
  if (as > 0x1p-40f && as < 0x1p40f && xbound < 0x1p80f && (__float_as_uint(s) & 0x7fffffu) != 0x7fffffu) {
    const float r0 = __builtin_amdgcn_rcpf(s);
    const float r = __builtin_fmaf(__builtin_fmaf(-s, r0, 1.f), r0, r0);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float q0 = x[e] * r;
      q[e] = __builtin_fmaf(__builtin_fmaf(-s, q0, x[e]), r, q0);
    }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) q[e] = __fdiv_rn(x[e], s);
  }
#pragma unroll
  for (int w = 0; w < 2; ++w) {
    // clamp like fminf(fmaxf(x, -448), 448) (a NaN becomes -448), then two conversions of two values each
    float c0 = q[4 * w], c1 = q[4 * w + 1], c2 = q[4 * w + 2], c3 = q[4 * w + 3];
    if constexpr (CLAMP) {
      c0 = __builtin_amdgcn_fmed3f(c0, -kFp8Max, kFp8Max);
      c1 = __builtin_amdgcn_fmed3f(c1, -kFp8Max, kFp8Max);
      c2 = __builtin_amdgcn_fmed3f(c2, -kFp8Max, kFp8Max);
      c3 = __builtin_amdgcn_fmed3f(c3, -kFp8Max, kFp8Max);
    }
    int word = __builtin_amdgcn_cvt_pk_fp8_f32(c0, c1, 0, false);
    word = __builtin_amdgcn_cvt_pk_fp8_f32(c2, c3, word, true);
    out[w] = (uint32_t)word;
  }
}

// ---- append, many tokens (prefill): one workgroup per (16 tokens, up to 4 kv heads) -----------------------------
// Written token by token the V cache takes 128 separate one-byte stores per token and head (a token is one
// byte of every head dim's row) and the K cache 2-byte ones; prefill appends runs of tokens to consecutive slots,
// so here a GROUP, a run of up to 16 tokens that fill consecutive slots of one 16-slot aligned segment of a
// page, is quantised together: 256 threads load the rows 16 bytes at a time, K leaves as 16-byte (token, chunk)
// cells, and V is turned through LDS so that each head dim's row gets its 16 tokens in one 16-byte store.
// A workgroup owns the groups that START among its 16 tokens (a group may reach into the next workgroup's
// tokens, which then skips them); with more than four groups among its tokens (scattered slots) it writes its
// tokens one by one like the kernel above.
// HPW: kv heads one workgroup of the tile kernel walks, their rows all requested first.  Measured on 262,144 tokens
// x 8 heads: with per-token scales (more arithmetic per row between the loads and the stores) 2 heads per
// workgroup beat 4 (block 16: 333 against 344 us, block 1024: 343 against 351 us); with per-tensor scales or a
// 16-bit cache 4 are as good or better (block 16, per tensor: 327 against 350 us); 1 and 8 lose everywhere.

// one kv head of a group: kr, vr are this thread's 16 bytes of the token's K and V row
template <bool TO_FP8>
__device__ __forceinline__ void write_group_head(const PaKvWriteArgs& a, int n, long long block, int off0, int h, int tid,
                                                 u32x4 kr, u32x4 vr, uint8_t (*s_v)[256]) {
  const int bs = a.block_size;
  const int tk = tid >> 4, c = tid & 15;  // token of the group; 16-byte piece of its row (head dims 8c..8c+7)
  const bool on = tk < n;
  if constexpr (!TO_FP8) {
    if (on) {
      // K: the 16 bytes are one (chunk, token) cell of the cache as they are
      uint16_t* kc = (uint16_t*)a.key_cache + block * a.stride_kc_b + h * a.stride_kc_h;
      *reinterpret_cast<u32x4*>(kc + ((int64_t)c * bs + off0 + tk) * 8) = kr;
      *reinterpret_cast<u32x4*>(&s_v[tk][16 * c]) = vr;
    }
    __syncthreads();
    if (tid < 128) {  // thread = head dim: its n tokens are 2n consecutive bytes of the dim's row
      uint16_t* vc = (uint16_t*)a.value_cache + block * a.stride_vc_b + h * a.stride_vc_h;
      if (n == 16 && (off0 & 7) == 0) {
        u32x4 lo, hi;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          lo[e] = (uint32_t)*reinterpret_cast<const uint16_t*>(&s_v[2 * e][2 * tid]) |
                  ((uint32_t)*reinterpret_cast<const uint16_t*>(&s_v[2 * e + 1][2 * tid]) << 16);
          hi[e] = (uint32_t)*reinterpret_cast<const uint16_t*>(&s_v[8 + 2 * e][2 * tid]) |
                  ((uint32_t)*reinterpret_cast<const uint16_t*>(&s_v[9 + 2 * e][2 * tid]) << 16);
        }
        *reinterpret_cast<u32x4*>(vc + v_index<8>(a, tid, off0)) = lo;  // tokens 0..7: one 8-token tile if transposed
        *reinterpret_cast<u32x4*>(vc + v_index<8>(a, tid, off0 + 8)) = hi;
      } else {
        for (int k = 0; k < n; ++k) vc[v_index<8>(a, tid, off0 + k)] = *reinterpret_cast<const uint16_t*>(&s_v[k][2 * tid]);
      }
    }
    __syncthreads();  // s_v is free for the next group
  } else {
    float kf[8], vf[8];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      kf[2 * e] = bf16_to_f32(kr[e] & 0xffffu);
      kf[2 * e + 1] = bf16_to_f32(kr[e] >> 16);
      vf[2 * e] = bf16_to_f32(vr[e] & 0xffffu);
      vf[2 * e + 1] = bf16_to_f32(vr[e] >> 16);
    }
    float ks, vs;
    float ka = 0.f, va = 0.f;  // bounds of |x| in this thread's values (per-token scales: in the token's row)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      ka = fmaxf(ka, fabsf(kf[e]));
      va = fmaxf(va, fabsf(vf[e]));
    }
    if (a.kv_quant_mode == PA_QUANT_PER_TOKEN) {
      ka = row16_max(ka);  // the 16 lanes of a token
      va = row16_max(va);
      ks = ka > 0.f ? bf16_amax_to_scale(ka) : 1.f;
      vs = va > 0.f ? bf16_amax_to_scale(va) : 1.f;
      if (on && c == 0) {
        const int64_t so = block * a.stride_scale_b + h * a.stride_scale_h + off0 + tk;
        a.key_scale[so] = ks;
        a.value_scale[so] = vs;
      }
    } else if (a.kv_quant_mode == PA_QUANT_PER_TENSOR) {
      ks = a.key_scale[0];
      vs = a.value_scale[0];
    } else {
      ks = vs = 1.f;
    }
    u32x2 kq, vq;
    if (a.kv_quant_mode == PA_QUANT_PER_TOKEN && ka <= 0x1.fffffep127f && va <= 0x1.fffffep127f) {
      quantize8<false>(kf, ks, ka, kq);
      quantize8<false>(vf, vs, va, vq);
    } else {
      quantize8<true>(kf, ks, ka, kq);
      quantize8<true>(vf, vs, va, vq);
    }
    // K: lanes c, c+1 hold the two halves of one 16-byte (chunk, token) cell; the even one stores it
    const uint32_t p0 = dpp_u32<kDppSwap1>(kq[0]), p1 = dpp_u32<kDppSwap1>(kq[1]);
    if (on) {
      if ((c & 1) == 0) {
        uint8_t* kc = (uint8_t*)a.key_cache + block * a.stride_kc_b + h * a.stride_kc_h;
        *reinterpret_cast<u32x4*>(kc + ((int64_t)(c >> 1) * bs + off0 + tk) * 16) = u32x4{kq[0], kq[1], p0, p1};
      }
      *reinterpret_cast<u32x2*>(&s_v[tk][8 * c]) = vq;
    }
    __syncthreads();
    if (tid < 128) {  // thread = head dim: its n tokens are n consecutive bytes of the dim's row
      uint8_t* vc = (uint8_t*)a.value_cache + block * a.stride_vc_b + h * a.stride_vc_h;
      if (n == 16 && (off0 & 15) == 0) {
        u32x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          o[e] = (uint32_t)s_v[4 * e][tid] | ((uint32_t)s_v[4 * e + 1][tid] << 8) | ((uint32_t)s_v[4 * e + 2][tid] << 16) |
                 ((uint32_t)s_v[4 * e + 3][tid] << 24);
        *reinterpret_cast<u32x4*>(vc + v_index<16>(a, tid, off0)) = o;
      } else {
        for (int k = 0; k < n; ++k) vc[v_index<16>(a, tid, off0 + k)] = s_v[k][tid];
      }
    }
    __syncthreads();  // s_v is free for the next group
  }
}

// a group of n tokens from token t_first on, landing at slot0 .. slot0 + n - 1, for kv heads h0 .. h0 + nh - 1
template <bool TO_FP8, int HPW>
__device__ __forceinline__ void write_group(const PaKvWriteArgs& a, long long t_first, int n, long long slot0, int bs_shift,
                                            int h0, int nh, int tid, uint8_t (*s_v)[256]) {
  // bs_shift: log2 of the block size when that is a power of two (no 64-bit division then), else -1
  const long long block = bs_shift >= 0 ? slot0 >> bs_shift : slot0 / a.block_size;
  const int off0 = (int)(slot0 - block * a.block_size);
  const int tk = tid >> 4, c = tid & 15;
  u32x4 kr[HPW], vr[HPW];
#pragma unroll
  for (int i = 0; i < HPW; ++i) {
    kr[i] = vr[i] = u32x4{0, 0, 0, 0};
    if (tk < n && i < nh) {  // the rows are read once: non-temporal
      const long long t = t_first + tk;
      kr[i] = __builtin_nontemporal_load(
          reinterpret_cast<const u32x4*>((const uint16_t*)a.key + t * a.stride_k_t + (h0 + i) * a.stride_k_h + 8 * c));
      vr[i] = __builtin_nontemporal_load(
          reinterpret_cast<const u32x4*>((const uint16_t*)a.value + t * a.stride_v_t + (h0 + i) * a.stride_v_h + 8 * c));
    }
  }
#pragma unroll
  for (int i = 0; i < HPW; ++i) {
    if (i < nh) write_group_head<TO_FP8>(a, n, block, off0, h0 + i, tid, kr[i], vr[i], s_v);
  }
}

// With pages of more than 16 tokens the groups of neighbouring 16-token windows write neighbouring 16-byte
// pieces of the same 128-byte lines of the V cache, and the pieces only merge into whole lines if they pass
// through the same L2 close together.  Workgroups go to the eight XCDs (each with an L2 of its own) round robin
// in id order, so with `regroup` set the window a workgroup takes is chosen such that the eight windows of a
// 128-token stretch are the next eight workgroups of ONE XCD.  The grid is then a multiple of 64 windows.
template <bool TO_FP8, int HPW>
__global__ __launch_bounds__(256) void kv_cache_write_tile_kernel(const PaKvWriteArgs a, const int regroup, const int bs_shift) {
  __shared__ long long s_slot[33];  // slots of tokens t0-1 .. t0+31
  __shared__ __attribute__((aligned(16))) uint8_t s_v[16][256];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  // workgroup id -> (16-token window, group of kv heads), the head groups of a window next to each other: they
  // read the two halves of the same token rows and write neighbouring parts of the same pages
  const int head_groups = (a.num_kv_heads + HPW - 1) / HPW;
  long long window;
  int hg;
  if (regroup) {
    const long long q = blockIdx.x >> 3, xcd = blockIdx.x & 7;
    const long long unit = ((q >> 3) << 3) + xcd;  // (128-token stretch, head group): eight turns of one XCD
    window = unit / head_groups * 8 + (q & 7);
    hg = (int)(unit % head_groups);
  } else {
    window = blockIdx.x / head_groups;
    hg = (int)(blockIdx.x % head_groups);
  }
  const long long t0 = window * 16;
  if (t0 >= a.num_tokens) return;
  const int h0 = hg * HPW;
  const int nh = min(HPW, a.num_kv_heads - h0);
  if (tid < 33) {
    const long long t = t0 - 1 + tid;
    s_slot[tid] = (t >= 0 && t < a.num_tokens) ? a.slot_mapping[t] : -1;
  }
  __syncthreads();
  // bit j of `starts`: token t0+j is live and does not continue its predecessor's run inside a 16-slot segment;
  // bit j of `breaks`: a group that reaches token t0+j ends before it.  Every wave computes both.
  bool is_start = false, is_live = false;
  if (lane < 32) {
    const long long cur = s_slot[lane + 1], prev = s_slot[lane];
    is_live = cur >= 0;
    is_start = is_live && (prev < 0 || cur != prev + 1 || (cur & 15) == 0);
  }
  const uint64_t starts = __builtin_amdgcn_ballot_w64(is_start);
  const uint64_t breaks = starts | (~__builtin_amdgcn_ballot_w64(is_live) & 0xffffffffull) | (1ull << 32);
  uint32_t own = (uint32_t)starts & 0xffffu;  // the groups that start among this workgroup's 16 tokens
  if (own == 0) return;
  if (__builtin_popcount(own) > 4) {
    // scattered slots: token by token, the waves taking turns.  Token t0+k is this workgroup's if the last
    // start at or before it is among the first 16 tokens.
    const int wave = tid >> 6;
    for (int k = wave; k < 32; k += 4) {
      const uint64_t upto = starts & ((2ull << k) - 1);
      if (((breaks >> k) & 1) && !((starts >> k) & 1)) continue;  // not live
      if (upto == 0 || (63 - __builtin_clzll(upto)) >= 16) continue;
      for (int i = 0; i < nh; ++i) write_token<TO_FP8>(a, t0 + k, h0 + i, s_slot[k + 1], lane);
    }
    return;
  }
  while (own) {
    const int j = __builtin_ctz(own);
    own &= own - 1;
    const int n = __builtin_ctzll(breaks >> (j + 1)) + 1;
    write_group<TO_FP8, HPW>(a, t0 + j, n, s_slot[j + 1], bs_shift, h0, nh, tid, s_v);
  }
}

// ---- whole cache, per token, 16 tokens of one (block, kv head) per workgroup ------------------------------------
// The 16-bit cache (x = 8) is read in its own layout, 16 bytes per thread: K cells as they lie, V rows (8 tokens of
// one head dim) through LDS into the per-token form the append kernel works on; from there on it IS the append of
// a full group.  a.key / a.value are the 16-bit caches here.  Windows of one page are regrouped by XCD as above.
__global__ __launch_bounds__(256) void quantize_kv_cache_tile_kernel(const PaKvWriteArgs a, const long long num_windows,
                                                                    const int regroup) {
  __shared__ __attribute__((aligned(16))) uint8_t s_v[16][256];
  __shared__ uint32_t s_in[128][9];  // V rows of the window: 16 bf16 tokens per head dim, padded to 9 words
  const int tid = threadIdx.x;
  long long window = blockIdx.x;
  if (regroup) {
    const long long q = window >> 3, xcd = window & 7;
    window = (((q >> 3) << 3) + xcd) * 8 + (q & 7);
  }
  if (window >= num_windows) return;
  const int bs = a.block_size;
  const int wins_per_page = bs >> 4;
  const long long bh = window / wins_per_page;  // (block, head)
  const int tok0 = (int)(window - bh * wins_per_page) * 16;
  const long long block = bh / a.num_kv_heads;
  const int h = (int)(bh - block * a.num_kv_heads);
  const uint16_t* kin = (const uint16_t*)a.key + bh * 128 * bs;    // [16 chunks][bs][8]
  const uint16_t* vin = (const uint16_t*)a.value + bh * 128 * bs;  // [128][bs]
  const int tk = tid >> 4, c = tid & 15;
  const u32x4 kr = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(kin + ((int64_t)c * bs + tok0 + tk) * 8));
  {
    const int d = tid >> 1, half = tid & 1;
    // with more than one window per page a window reads a piece of each 128-byte line and its neighbours (same
    // XCD) the rest: those lines must stay in L2, so only whole-page windows read V non-temporally
    const u32x4* vp = reinterpret_cast<const u32x4*>(vin + (int64_t)d * bs + tok0 + 8 * half);
    const u32x4 v = regroup ? *vp : __builtin_nontemporal_load(vp);
#pragma unroll
    for (int e = 0; e < 4; ++e) s_in[d][4 * half + e] = v[e];
  }
  __syncthreads();
  u32x4 vr;
#pragma unroll
  for (int e = 0; e < 4; ++e) {  // head dims 8c + 2e, 8c + 2e + 1 of token tk
    const uint32_t w0 = s_in[8 * c + 2 * e][tk >> 1], w1 = s_in[8 * c + 2 * e + 1][tk >> 1];
    const int sh = 16 * (tk & 1);
    vr[e] = ((w0 >> sh) & 0xffffu) | (((w1 >> sh) & 0xffffu) << 16);
  }
  write_group_head<true>(a, 16, block, tok0, h, tid, kr, vr, s_v);
}

// ---- whole cache, per token: one thread per (block, kv head, token) -------------------------------------------
// Reads the 16-bit cache in its own layout (x = 8) and writes the FP8 cache (x = 16) and the scales.
__global__ __launch_bounds__(256) void quantize_kv_cache_kernel(const uint16_t* __restrict__ kin, const uint16_t* __restrict__ vin,
                                                                uint8_t* __restrict__ kout, uint8_t* __restrict__ vout,
                                                                float* __restrict__ kscale, float* __restrict__ vscale,
                                                                long long num_block_heads, int bs) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= num_block_heads * bs) return;
  const long long bh = idx / bs;
  const int tok = (int)(idx - bh * bs);
  const uint16_t* kp = kin + bh * 128 * bs;  // [16 chunks][bs][8]
  const uint16_t* vp = vin + bh * 128 * bs;  // [128][bs]
  float ka = 0.f, va = 0.f;
  u32x4 kc[16];
#pragma unroll
  for (int c = 0; c < 16; ++c) {
    kc[c] = *reinterpret_cast<const u32x4*>(kp + ((int64_t)c * bs + tok) * 8);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      ka = fmaxf(ka, fabsf(bf16_to_f32(kc[c][e] & 0xffffu)));
      ka = fmaxf(ka, fabsf(bf16_to_f32(kc[c][e] >> 16)));
    }
  }
  for (int d = 0; d < 128; ++d) va = fmaxf(va, fabsf(bf16_to_f32(vp[(int64_t)d * bs + tok])));
  const float ks = ka > 0.f ? __fdiv_rn(ka, kFp8Max) : 1.f;
  const float vs = va > 0.f ? __fdiv_rn(va, kFp8Max) : 1.f;
  kscale[idx] = ks;
  vscale[idx] = vs;
  uint8_t* ko = kout + bh * 128 * bs;  // [8 chunks][bs][16]
#pragma unroll
  for (int c = 0; c < 8; ++c) {
    u32x4 o;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const u32x4 in = kc[2 * c + half];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        uint32_t w = 0;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          const uint32_t pair = in[2 * e + q];
          const uint32_t b0 = f32_to_fp8(__fdiv_rn(bf16_to_f32(pair & 0xffffu), ks));
          const uint32_t b1 = f32_to_fp8(__fdiv_rn(bf16_to_f32(pair >> 16), ks));
          w |= (b0 | (b1 << 8)) << (16 * q);
        }
        o[2 * half + e] = w;
      }
    }
    *reinterpret_cast<u32x4*>(ko + ((int64_t)c * bs + tok) * 16) = o;
  }
  uint8_t* vo = vout + bh * 128 * bs;
  for (int d = 0; d < 128; ++d)
    vo[(int64_t)d * bs + tok] = f32_to_fp8(__fdiv_rn(bf16_to_f32(vp[(int64_t)d * bs + tok]), vs));
}

}  // namespace

extern "C" {

int pa_kv_cache_write(const PaKvWriteArgs* a, void* hip_stream) {
  if (!a) return PA_ERR_NULL_POINTER;
  if (a->struct_size != sizeof(PaKvWriteArgs)) return PA_ERR_BAD_STRUCT;
  if (!a->key || !a->value || !a->slot_mapping || !a->key_cache || !a->value_cache) return PA_ERR_NULL_POINTER;
  if (a->num_tokens < 0 || a->num_kv_heads <= 0 || a->block_size <= 0) return PA_ERR_BAD_SHAPE;
  if (a->head_size != 128 && a->head_size != 64 && a->head_size != 256) return PA_ERR_UNSUPPORTED;
  if (a->cache_dtype != PA_DTYPE_BF16 && a->cache_dtype != PA_DTYPE_FP8_E4M3FN) return PA_ERR_UNSUPPORTED;
  if (a->v_transposed != 0 && a->v_transposed != 1) return PA_ERR_BAD_SHAPE;
  if (a->v_transposed && a->block_size % (a->cache_dtype == PA_DTYPE_FP8_E4M3FN ? 16 : 8)) return PA_ERR_BAD_SHAPE;
  if (a->cache_dtype == PA_DTYPE_FP8_E4M3FN && a->kv_quant_mode != PA_QUANT_NONE && (!a->key_scale || !a->value_scale))
    return PA_ERR_NULL_POINTER;
  if (a->cache_dtype == PA_DTYPE_BF16 && a->kv_quant_mode != PA_QUANT_NONE) return PA_ERR_UNSUPPORTED;
  if (a->stride_k_t % 2 || a->stride_k_h % 2 || a->stride_v_t % 2 || a->stride_v_h % 2) return PA_ERR_BAD_SHAPE;
  if (a->num_tokens == 0) return PA_OK;
  const long long items = (long long)a->num_tokens * a->num_kv_heads;
  const long long blocks = (items + 3) / 4;
  if (blocks > 0x7fffffffLL) return PA_ERR_BAD_SHAPE;
  hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
  // Many tokens (prefill) go 16 at a time when the rows can be read 16 bytes at a time; a few tokens (decode)
  // get one wave per (token, head) each, which has more of the GPU working on them.
  const bool rows_16b = a->stride_k_t % 8 == 0 && a->stride_k_h % 8 == 0 && a->stride_v_t % 8 == 0 && a->stride_v_h % 8 == 0 &&
                        ((reinterpret_cast<uintptr_t>(a->key) | reinterpret_cast<uintptr_t>(a->value)) & 15) == 0 &&
                        ((reinterpret_cast<uintptr_t>(a->key_cache) | reinterpret_cast<uintptr_t>(a->value_cache)) & 15) == 0 &&
                        a->stride_kc_b % 16 == 0 && a->stride_kc_h % 16 == 0 && a->stride_vc_b % 16 == 0 && a->stride_vc_h % 16 == 0 &&
                        a->block_size % 16 == 0;
  if (a->head_size != 128) {  // head sizes 64 and 256: token by token, whatever the number of tokens
    const dim3 grid((unsigned)blocks), block(256);
    const bool fp8 = a->cache_dtype == PA_DTYPE_FP8_E4M3FN;
    if (a->head_size == 64)
      return fp8 ? pa_launch(kv_cache_write_kernel<true, 64>, grid, block, 0, stream, *a)
                 : pa_launch(kv_cache_write_kernel<false, 64>, grid, block, 0, stream, *a);
    return fp8 ? pa_launch(kv_cache_write_kernel<true, 256>, grid, block, 0, stream, *a)
               : pa_launch(kv_cache_write_kernel<false, 256>, grid, block, 0, stream, *a);
  }
  if (rows_16b && a->num_tokens >= 2048) {
    const int regroup = a->block_size > 16;
    const int bs_shift = (a->block_size & (a->block_size - 1)) == 0 ? __builtin_ctz((unsigned)a->block_size) : -1;
    long long windows = (a->num_tokens + 15) / 16;
    if (regroup) windows = (windows + 63) / 64 * 64;
    const bool per_token = a->cache_dtype == PA_DTYPE_FP8_E4M3FN && a->kv_quant_mode == PA_QUANT_PER_TOKEN;
    const int hpw = per_token ? 2 : 4;
    const long long head_groups = (a->num_kv_heads + hpw - 1) / hpw;
    if (windows * head_groups > 0x7fffffffLL) return PA_ERR_BAD_SHAPE;
    const dim3 grid((unsigned)(windows * head_groups));
    if (per_token) return pa_launch(kv_cache_write_tile_kernel<true, 2>, grid, dim3(256), 0, stream, *a, regroup, bs_shift);
    if (a->cache_dtype == PA_DTYPE_FP8_E4M3FN)
      return pa_launch(kv_cache_write_tile_kernel<true, 4>, grid, dim3(256), 0, stream, *a, regroup, bs_shift);
    return pa_launch(kv_cache_write_tile_kernel<false, 4>, grid, dim3(256), 0, stream, *a, regroup, bs_shift);
  }
  if (a->cache_dtype == PA_DTYPE_FP8_E4M3FN)
    return pa_launch(kv_cache_write_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, stream, *a);
  return pa_launch(kv_cache_write_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, stream, *a);
}

int pa_quantize_kv_cache(const void* key_cache_bf16, const void* value_cache_bf16, void* key_cache_fp8,
                         void* value_cache_fp8, float* key_scale, float* value_scale, int64_t num_blocks,
                         int32_t num_kv_heads, int32_t head_size, int32_t block_size, void* hip_stream) {
  if (!key_cache_bf16 || !value_cache_bf16 || !key_cache_fp8 || !value_cache_fp8 || !key_scale || !value_scale)
    return PA_ERR_NULL_POINTER;
  if (num_blocks <= 0 || num_kv_heads <= 0 || block_size <= 0) return PA_ERR_BAD_SHAPE;
  if (head_size != 128) return PA_ERR_UNSUPPORTED;
  const long long n = (long long)num_blocks * num_kv_heads * block_size;
  hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
  const bool aligned = ((reinterpret_cast<uintptr_t>(key_cache_bf16) | reinterpret_cast<uintptr_t>(value_cache_bf16) |
                         reinterpret_cast<uintptr_t>(key_cache_fp8) | reinterpret_cast<uintptr_t>(value_cache_fp8)) & 15) == 0;
  if (aligned && block_size % 16 == 0) {
    PaKvWriteArgs a = {};
    a.struct_size = sizeof(PaKvWriteArgs);
    a.key = key_cache_bf16;
    a.value = value_cache_bf16;
    a.key_cache = key_cache_fp8;
    a.value_cache = value_cache_fp8;
    a.key_scale = key_scale;
    a.value_scale = value_scale;
    a.num_kv_heads = num_kv_heads;
    a.head_size = head_size;
    a.block_size = block_size;
    a.cache_dtype = PA_DTYPE_FP8_E4M3FN;
    a.kv_quant_mode = PA_QUANT_PER_TOKEN;
    a.stride_kc_h = a.stride_vc_h = (int64_t)head_size * block_size;
    a.stride_kc_b = a.stride_vc_b = a.stride_kc_h * num_kv_heads;
    a.stride_scale_h = block_size;
    a.stride_scale_b = (int64_t)block_size * num_kv_heads;
    const long long num_windows = n / 16;
    const int regroup = block_size > 16;
    const long long grid = regroup ? (num_windows + 63) / 64 * 64 : num_windows;
    if (grid > 0x7fffffffLL) return PA_ERR_BAD_SHAPE;
    return pa_launch(quantize_kv_cache_tile_kernel, dim3((unsigned)grid), dim3(256), 0, stream, a, num_windows, regroup);
  }
  const long long blocks = (n + 255) / 256;
  if (blocks > 0x7fffffffLL) return PA_ERR_BAD_SHAPE;
  return pa_launch(quantize_kv_cache_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (const uint16_t*)key_cache_bf16,
                   (const uint16_t*)value_cache_bf16, (uint8_t*)key_cache_fp8, (uint8_t*)value_cache_fp8, key_scale,
                   value_scale, (long long)num_blocks * num_kv_heads, (int)block_size);
}

}  // extern "C"
