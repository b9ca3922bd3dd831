// A caller of the C ABI with no Python and no torch: plain hipMalloc'ed buffers, an FP8 cache written by
// pa_kv_cache_write, one pa_decode call, and the result checked against a double-precision attention over the
// bytes the cache actually holds.  Exit code 0 and a line "abi_smoke ok" on success.
//   hipcc -O2 tests/native/abi_smoke.cpp -Iinclude -Ltriton_op_amd -lpa_decode -o tests/native/abi_smoke
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <vector>

#include "pa_decode.h"

#define HIP_OK(x)                                                              \
  do {                                                                         \
    hipError_t e_ = (x);                                                       \
    if (e_ != hipSuccess) {                                                    \
      printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);    \
      return 2;                                                                \
    }                                                                          \
  } while (0)

static uint16_t f32_to_bf16(float f) {  // round to nearest even
  uint32_t u;
  memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
static float bf16_to_f32(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static float e4m3fn_to_f32(uint8_t c) {  // OCP e4m3fn: bias 7, no infinities, 0x7f / 0xff are NaN
  const int e = (c >> 3) & 15, m = c & 7;
  float v = e == 0 ? ldexpf((float)m, -9) : ldexpf((float)(8 + m), e - 10);
  if (e == 15 && m == 7) v = NAN;
  return (c & 0x80) ? -v : v;
}
static uint32_t rng_state = 12345u;
static float rnd() {  // uniform in (-1, 1)
  rng_state = rng_state * 1664525u + 1013904223u;
  return (float)((rng_state >> 8) & 0xffff) / 32768.f - 1.f;
}

int main() {
  const int B = 3, Hkv = 2, G = 8, D = 128, bs = 16, q = 1;
  const int ctx[B] = {40, 300, 1};
  const int max_ctx = 300, blocks_per_seq = (max_ctx + bs - 1) / bs, num_blocks = B * blocks_per_seq + 3;
  const int Hq = Hkv * G;
  if (pa_decode_abi_version() != PA_DECODE_ABI_VERSION || pa_decode_args_size() != sizeof(PaDecodeArgs)) {
    printf("ABI mismatch\n");
    return 1;
  }
  // block tables: sequence b, logical block i -> physical block (a fixed scramble)
  std::vector<int32_t> bt(B * blocks_per_seq);
  for (int i = 0; i < B * blocks_per_seq; ++i) bt[i] = (i * 7 + 2) % (B * blocks_per_seq) + 3;
  // new tokens: all tokens of all sequences, appended in one pa_kv_cache_write call
  int ntok = 0;
  for (int b = 0; b < B; ++b) ntok += ctx[b];
  std::vector<uint16_t> key((size_t)ntok * Hkv * D), value((size_t)ntok * Hkv * D);
  std::vector<int64_t> slots(ntok);
  {
    int t = 0;
    for (int b = 0; b < B; ++b)
      for (int i = 0; i < ctx[b]; ++i, ++t) slots[t] = (int64_t)bt[b * blocks_per_seq + i / bs] * bs + i % bs;
    for (auto& v : key) v = f32_to_bf16(rnd());
    for (auto& v : value) v = f32_to_bf16(rnd());
  }
  std::vector<uint16_t> query((size_t)B * Hq * D);
  for (auto& v : query) v = f32_to_bf16(rnd());

  const size_t cache_bytes = (size_t)num_blocks * Hkv * D * bs, scale_elems = (size_t)num_blocks * Hkv * bs;
  void *d_key, *d_value, *d_slots, *d_kc, *d_vc, *d_q, *d_out, *d_tmp;
  float *d_ks, *d_vs, *d_es, *d_ml;
  int32_t *d_ctx, *d_bt, *d_ws;
  HIP_OK(hipMalloc(&d_key, key.size() * 2));
  HIP_OK(hipMalloc(&d_value, value.size() * 2));
  HIP_OK(hipMalloc(&d_slots, slots.size() * 8));
  HIP_OK(hipMalloc(&d_kc, cache_bytes));
  HIP_OK(hipMalloc(&d_vc, cache_bytes));
  HIP_OK(hipMalloc((void**)&d_ks, scale_elems * 4));
  HIP_OK(hipMalloc((void**)&d_vs, scale_elems * 4));
  HIP_OK(hipMalloc(&d_q, query.size() * 2));
  HIP_OK(hipMalloc(&d_out, query.size() * 2));
  HIP_OK(hipMalloc((void**)&d_ctx, B * 4));
  HIP_OK(hipMalloc((void**)&d_bt, bt.size() * 4));
  HIP_OK(hipMemcpy(d_key, key.data(), key.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_value, value.data(), value.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_slots, slots.data(), slots.size() * 8, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_q, query.data(), query.size() * 2, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_ctx, ctx, B * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_bt, bt.data(), bt.size() * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemset(d_kc, 0, cache_bytes));
  HIP_OK(hipMemset(d_vc, 0, cache_bytes));
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));

  // ---- the step before the path: quantise the new rows into the paged FP8 cache --------------------------------
  PaKvWriteArgs w;
  memset(&w, 0, sizeof(w));
  w.struct_size = sizeof(w);
  w.key = d_key;
  w.value = d_value;
  w.slot_mapping = (const int64_t*)d_slots;
  w.key_cache = d_kc;
  w.value_cache = d_vc;
  w.key_scale = d_ks;
  w.value_scale = d_vs;
  w.num_tokens = ntok;
  w.num_kv_heads = Hkv;
  w.head_size = D;
  w.block_size = bs;
  w.cache_dtype = PA_DTYPE_FP8_E4M3FN;
  w.kv_quant_mode = PA_QUANT_PER_TOKEN;
  w.stride_k_t = w.stride_v_t = (int64_t)Hkv * D;
  w.stride_k_h = w.stride_v_h = D;
  w.stride_kc_b = w.stride_vc_b = (int64_t)Hkv * D * bs;
  w.stride_kc_h = w.stride_vc_h = (int64_t)D * bs;
  w.stride_scale_b = (int64_t)Hkv * bs;
  w.stride_scale_h = bs;
  int rc = pa_kv_cache_write(&w, stream);
  if (rc) {
    printf("pa_kv_cache_write: %s\n", pa_decode_error_string(rc));
    return 1;
  }

  // ---- the decode call ------------------------------------------------------------------------------------------
  const int ps = pa_decode_select_partition_size(B, Hkv, q * G, max_ctx, bs, 0);
  if (ps <= 0 || ps % 256) {
    printf("bad partition size %d\n", ps);
    return 1;
  }
  const int P = (max_ctx + ps - 1) / ps;
  const int64_t ws_bytes = pa_decode_workspace_bytes(B, P);
  const size_t n = (size_t)B * Hkv * P * q * G;
  HIP_OK(hipMalloc((void**)&d_es, n * 4));
  HIP_OK(hipMalloc((void**)&d_ml, n * 4));
  HIP_OK(hipMalloc(&d_tmp, n * D * 2));
  HIP_OK(hipMalloc((void**)&d_ws, ws_bytes));
  HIP_OK(hipMemsetAsync(d_ws, 0, ws_bytes, stream));
  PaDecodeArgs a;
  memset(&a, 0, sizeof(a));
  a.struct_size = sizeof(a);
  a.output = d_out;
  a.query = d_q;
  a.key_cache = d_kc;
  a.value_cache = d_vc;
  a.context_lens = d_ctx;
  a.block_tables = d_bt;
  a.key_scale = d_ks;
  a.value_scale = d_vs;
  a.exp_sums = d_es;
  a.max_logits = d_ml;
  a.tmp_output = d_tmp;
  a.workspace = d_ws;
  a.workspace_bytes = ws_bytes;
  a.num_seqs = B;
  a.num_kv_heads = Hkv;
  a.group_size = G;
  a.q_len = q;
  a.head_size = D;
  a.block_size = bs;
  a.max_num_partitions = P;
  a.partition_size = ps;
  a.query_dtype = PA_DTYPE_BF16;
  a.kv_dtype = PA_DTYPE_FP8_E4M3FN;
  a.query_quant_mode = PA_QUANT_NONE;
  a.kv_quant_mode = PA_QUANT_PER_TOKEN;
  a.softmax_scale = 1.f / sqrtf((float)D);
  a.stride_out_s = a.stride_q_s = (int64_t)Hq * D;
  a.stride_out_h = a.stride_q_h = D;
  a.stride_k_b = a.stride_v_b = (int64_t)Hkv * D * bs;
  a.stride_k_h = a.stride_v_h = (int64_t)D * bs;
  a.stride_k_c = (int64_t)bs * 16;
  a.stride_v_2 = bs;
  a.stride_bt_s = blocks_per_seq;
  a.stride_es_s = (int64_t)Hkv * P * q * G;
  a.stride_es_h = (int64_t)P * q * G;
  a.stride_es_p = q * G;
  a.stride_tmp_s = a.stride_es_s * D;
  a.stride_tmp_h = a.stride_es_h * D;
  a.stride_tmp_p = a.stride_es_p * D;
  a.stride_tmp_g = D;
  a.stride_kvscale_b = (int64_t)Hkv * bs;
  a.stride_kvscale_h = bs;
  rc = pa_decode(&a, stream);
  if (rc) {
    printf("pa_decode: %s (hip error %d)\n", pa_decode_error_string(rc), pa_decode_last_hip_error());
    return 1;
  }
  HIP_OK(hipStreamSynchronize(stream));

  // ---- check against a double-precision attention over the cache as written -----------------------------------
  std::vector<uint8_t> kc(cache_bytes), vc(cache_bytes);
  std::vector<float> ks(scale_elems), vs(scale_elems);
  std::vector<uint16_t> out(query.size());
  HIP_OK(hipMemcpy(kc.data(), d_kc, cache_bytes, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(vc.data(), d_vc, cache_bytes, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(ks.data(), d_ks, scale_elems * 4, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(vs.data(), d_vs, scale_elems * 4, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(out.data(), d_out, out.size() * 2, hipMemcpyDeviceToHost));
  double worst = 0.0;
  for (int b = 0; b < B; ++b)
    for (int hq = 0; hq < Hq; ++hq) {
      const int h = hq / G;
      std::vector<double> logit(ctx[b]), o(D, 0.0);
      double mx = -1e300;
      for (int i = 0; i < ctx[b]; ++i) {
        const size_t page = (size_t)bt[b * blocks_per_seq + i / bs], off = i % bs;
        const size_t base = (page * Hkv + h) * D * bs;
        double s = 0.0;
        for (int d = 0; d < D; ++d)  // K element (token off, dim d) at [d/16][off][d%16]
          s += (double)bf16_to_f32(query[((size_t)b * Hq + hq) * D + d]) *
               e4m3fn_to_f32(kc[base + (size_t)(d / 16) * bs * 16 + off * 16 + d % 16]);
        logit[i] = s * ks[(page * Hkv + h) * bs + off] * a.softmax_scale;
        mx = logit[i] > mx ? logit[i] : mx;
      }
      double l = 0.0;
      for (int i = 0; i < ctx[b]; ++i) {
        const size_t page = (size_t)bt[b * blocks_per_seq + i / bs], off = i % bs;
        const size_t base = (page * Hkv + h) * D * bs;
        const double p = exp(logit[i] - mx);
        l += p;
        for (int d = 0; d < D; ++d)  // V element (dim d, token off) at [d][off]
          o[d] += p * e4m3fn_to_f32(vc[base + (size_t)d * bs + off]) * vs[(page * Hkv + h) * bs + off];
      }
      for (int d = 0; d < D; ++d) {
        const double ref = o[d] / l, got = bf16_to_f32(out[((size_t)b * Hq + hq) * D + d]);
        const double err = fabs(got - ref) / (2e-2 + 2e-2 * fabs(ref));  // atol 2e-2, rtol 2e-2
        worst = err > worst ? err : worst;
      }
    }
  if (!(worst <= 1.0)) {
    printf("abi_smoke FAILED: worst |diff| / (atol + rtol |ref|) = %.3f\n", worst);
    return 1;
  }
  printf("abi_smoke ok: partition_size %d, worst |diff| / (atol + rtol |ref|) = %.4f\n", ps, worst);
  return 0;
}
