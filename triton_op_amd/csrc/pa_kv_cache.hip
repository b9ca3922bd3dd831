// KV-cache write and quantisation kernels for the paged layouts the decode kernels read:
//   key_cache   [blocks, Hkv, D/x, bs, x]     x = 16 / sizeof(element)
//   value_cache [blocks, Hkv, D, bs]
//   scales      [blocks, Hkv, bs, 1] f32 (one per token and kv head) or one f32 per tensor
// FP8 is OCP e4m3fn.  Quantisation is symmetric: scale = amax / 448 (1 for an all-zero row),
// q = round_to_nearest_even(x / scale), both with IEEE division so the bytes match a float32 host
// computation of the same formula bit for bit.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/pa_decode.h"

namespace {

constexpr float kFp8Max = 448.f;

__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }

__device__ __forceinline__ uint8_t f32_to_fp8(float x) {
  x = fminf(fmaxf(x, -kFp8Max), kFp8Max);
  return (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(x, 0.f, 0, false) & 0xff);
}

// ---- append: one wave per (token, kv head); lane l owns head dims 2l, 2l+1 --------------------------------
template <bool TO_FP8>
__global__ __launch_bounds__(256) void kv_cache_write_kernel(const PaKvWriteArgs a) {
  const int lane = threadIdx.x & 63;
  const long long item = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= (long long)a.num_tokens * a.num_kv_heads) return;
  const int h = (int)(item % a.num_kv_heads);
  const long long t = item / a.num_kv_heads;
  const long long slot = a.slot_mapping[t];
  if (slot < 0) return;  // padding token
  const long long block = slot / a.block_size;
  const int off = (int)(slot - block * a.block_size);
  const int bs = a.block_size;

  const uint32_t kraw = *reinterpret_cast<const uint32_t*>((const uint16_t*)a.key + t * a.stride_k_t + h * a.stride_k_h + 2 * lane);
  const uint32_t vraw = *reinterpret_cast<const uint32_t*>((const uint16_t*)a.value + t * a.stride_v_t + h * a.stride_v_h + 2 * lane);
  const int d0 = 2 * lane;
  if constexpr (!TO_FP8) {
    // 16-bit cache: x = 8; the two dims of a lane are adjacent in a chunk
    uint16_t* kc = (uint16_t*)a.key_cache + block * a.stride_kc_b + h * a.stride_kc_h;
    *reinterpret_cast<uint32_t*>(kc + (int64_t)(d0 / 8) * bs * 8 + off * 8 + d0 % 8) = kraw;
    uint16_t* vc = (uint16_t*)a.value_cache + block * a.stride_vc_b + h * a.stride_vc_h;
    vc[(int64_t)d0 * bs + off] = (uint16_t)(vraw & 0xffffu);
    vc[(int64_t)(d0 + 1) * bs + off] = (uint16_t)(vraw >> 16);
    return;
  } else {
    const float k0 = bf16_to_f32(kraw & 0xffffu), k1 = bf16_to_f32(kraw >> 16);
    const float v0 = bf16_to_f32(vraw & 0xffffu), v1 = bf16_to_f32(vraw >> 16);
    float ks, vs;
    if (a.kv_quant_mode == PA_QUANT_PER_TOKEN) {
      float ka = fmaxf(fabsf(k0), fabsf(k1)), va = fmaxf(fabsf(v0), fabsf(v1));
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
    const uint8_t qk0 = f32_to_fp8(__fdiv_rn(k0, ks)), qk1 = f32_to_fp8(__fdiv_rn(k1, ks));
    const uint8_t qv0 = f32_to_fp8(__fdiv_rn(v0, vs)), qv1 = f32_to_fp8(__fdiv_rn(v1, vs));
    uint8_t* kc = (uint8_t*)a.key_cache + block * a.stride_kc_b + h * a.stride_kc_h;
    *reinterpret_cast<uint16_t*>(kc + (int64_t)(d0 / 16) * bs * 16 + off * 16 + d0 % 16) = (uint16_t)(qk0 | (qk1 << 8));
    uint8_t* vc = (uint8_t*)a.value_cache + block * a.stride_vc_b + h * a.stride_vc_h;
    vc[(int64_t)d0 * bs + off] = qv0;
    vc[(int64_t)(d0 + 1) * bs + off] = qv1;
  }
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
  typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
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

thread_local int g_last_hip_error_kv = 0;

}  // namespace

extern "C" {

int pa_kv_cache_write(const PaKvWriteArgs* a, void* hip_stream) {
  if (!a) return PA_ERR_NULL_POINTER;
  if (a->struct_size != sizeof(PaKvWriteArgs)) return PA_ERR_BAD_STRUCT;
  if (!a->key || !a->value || !a->slot_mapping || !a->key_cache || !a->value_cache) return PA_ERR_NULL_POINTER;
  if (a->num_tokens < 0 || a->num_kv_heads <= 0 || a->block_size <= 0) return PA_ERR_BAD_SHAPE;
  if (a->head_size != 128) return PA_ERR_UNSUPPORTED;
  if (a->cache_dtype != PA_DTYPE_BF16 && a->cache_dtype != PA_DTYPE_FP8_E4M3FN) return PA_ERR_UNSUPPORTED;
  if (a->cache_dtype == PA_DTYPE_FP8_E4M3FN && a->kv_quant_mode != PA_QUANT_NONE && (!a->key_scale || !a->value_scale))
    return PA_ERR_NULL_POINTER;
  if (a->cache_dtype == PA_DTYPE_BF16 && a->kv_quant_mode != PA_QUANT_NONE) return PA_ERR_UNSUPPORTED;
  if (a->stride_k_t % 2 || a->stride_k_h % 2 || a->stride_v_t % 2 || a->stride_v_h % 2) return PA_ERR_BAD_SHAPE;
  if (a->num_tokens == 0) return PA_OK;
  const long long items = (long long)a->num_tokens * a->num_kv_heads;
  const long long blocks = (items + 3) / 4;
  if (blocks > 0x7fffffffLL) return PA_ERR_BAD_SHAPE;
  hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
  if (a->cache_dtype == PA_DTYPE_FP8_E4M3FN)
    hipLaunchKernelGGL(kv_cache_write_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, stream, *a);
  else
    hipLaunchKernelGGL(kv_cache_write_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, stream, *a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    g_last_hip_error_kv = (int)e;
    return PA_ERR_LAUNCH;
  }
  return PA_OK;
}

int pa_quantize_kv_cache(const void* key_cache_bf16, const void* value_cache_bf16, void* key_cache_fp8,
                         void* value_cache_fp8, float* key_scale, float* value_scale, int64_t num_blocks,
                         int32_t num_kv_heads, int32_t head_size, int32_t block_size, void* hip_stream) {
  if (!key_cache_bf16 || !value_cache_bf16 || !key_cache_fp8 || !value_cache_fp8 || !key_scale || !value_scale)
    return PA_ERR_NULL_POINTER;
  if (num_blocks <= 0 || num_kv_heads <= 0 || block_size <= 0) return PA_ERR_BAD_SHAPE;
  if (head_size != 128) return PA_ERR_UNSUPPORTED;
  const long long n = (long long)num_blocks * num_kv_heads * block_size;
  const long long blocks = (n + 255) / 256;
  if (blocks > 0x7fffffffLL) return PA_ERR_BAD_SHAPE;
  hipLaunchKernelGGL(quantize_kv_cache_kernel, dim3((unsigned)blocks), dim3(256), 0, reinterpret_cast<hipStream_t>(hip_stream),
                     (const uint16_t*)key_cache_bf16, (const uint16_t*)value_cache_bf16, (uint8_t*)key_cache_fp8,
                     (uint8_t*)value_cache_fp8, key_scale, value_scale, (long long)num_blocks * num_kv_heads, block_size);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    g_last_hip_error_kv = (int)e;
    return PA_ERR_LAUNCH;
  }
  return PA_OK;
}

}  // extern "C"
