// libpa_probe.so: the two measuring kernels behind bench.py's probe workloads (declared in pa_probe.h).  Built
// from the decode library's own headers, so the probe reads the cache with the same loads as the partition kernel.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "pa_probe.h"
#include "pa_probe_kernel.h"

namespace {

template <typename K, typename... Args>
int launch(K kernel, dim3 grid, dim3 block, hipStream_t stream, Args... args) {
  void* ptrs[] = {static_cast<void*>(&args)...};
  return hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, ptrs, 0, stream) == hipSuccess ? PA_OK
                                                                                                           : PA_ERR_LAUNCH;
}

}  // namespace

extern "C" {

int pa_probe_gather(const PaDecodeArgs* a, int32_t* sink, void* hip_stream) {
  if (!a || !sink) return PA_ERR_NULL_POINTER;
  if (a->struct_size != sizeof(PaDecodeArgs)) return PA_ERR_BAD_STRUCT;
  if (!a->key_cache || !a->value_cache || !a->context_lens || !a->block_tables) return PA_ERR_NULL_POINTER;
  if (a->num_seqs <= 0 || a->num_kv_heads <= 0 || a->max_num_partitions <= 0 || a->partition_size <= 0 ||
      a->partition_size % 256)
    return PA_ERR_BAD_SHAPE;
  if (a->kv_dtype != PA_DTYPE_FP8_E4M3FN || a->block_size < 16 || (a->block_size & (a->block_size - 1)) ||
      a->v_transposed || a->head_size != kHeadSize)
    return PA_ERR_UNSUPPORTED;
  const long long blocks = (long long)a->num_seqs * a->num_kv_heads * a->max_num_partitions;
  if (blocks > 0x7fffffffLL) return PA_ERR_BAD_SHAPE;
  const bool bs16 = a->block_size == 16 && a->stride_k_c == 256 && a->stride_v_2 == 16;
  if (bs16)
    return launch(pa_gather_probe_kernel<true>, dim3((unsigned)blocks), dim3(256), reinterpret_cast<hipStream_t>(hip_stream),
                  *a, reinterpret_cast<int*>(sink));
  return launch(pa_gather_probe_kernel<false>, dim3((unsigned)blocks), dim3(256), reinterpret_cast<hipStream_t>(hip_stream),
                *a, reinterpret_cast<int*>(sink));
}

int pa_probe_stream(const PaDecodeArgs* a, int32_t depth, int32_t workgroups_per_cu, int32_t variant, int32_t* sink,
                    void* hip_stream) {
  if (!a || !sink) return PA_ERR_NULL_POINTER;
  if (a->struct_size != sizeof(PaDecodeArgs)) return PA_ERR_BAD_STRUCT;
  if (!a->key_cache || !a->value_cache || !a->context_lens || !a->block_tables) return PA_ERR_NULL_POINTER;
  if (a->num_seqs <= 0 || a->num_kv_heads <= 0 || a->max_num_partitions <= 0 || a->partition_size <= 0 ||
      a->partition_size % 256)
    return PA_ERR_BAD_SHAPE;
  if (a->kv_dtype != PA_DTYPE_FP8_E4M3FN || a->block_size != 16 || a->stride_k_c != 256 || a->stride_v_2 != 16 ||
      a->v_transposed || a->head_size != kHeadSize)
    return PA_ERR_UNSUPPORTED;
  if (a->kv_quant_mode == PA_QUANT_PER_TOKEN && (!a->key_scale || !a->value_scale)) return PA_ERR_NULL_POINTER;
  const long long blocks = (long long)a->num_seqs * a->num_kv_heads * a->max_num_partitions;
  if (blocks > 0x7fffffffLL) return PA_ERR_BAD_SHAPE;
  hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
  const dim3 grid((unsigned)blocks), block(256);
  int* s = reinterpret_cast<int*>(sink);
  const int v = variant;
  switch (depth * 10 + workgroups_per_cu) {
    case 22: return launch(pa_stream_probe_kernel<2, 2>, grid, block, stream, *a, s, v);
    case 42: return launch(pa_stream_probe_kernel<4, 2>, grid, block, stream, *a, s, v);
    case 62: return launch(pa_stream_probe_kernel<6, 2>, grid, block, stream, *a, s, v);
    case 23: return launch(pa_stream_probe_kernel<2, 3>, grid, block, stream, *a, s, v);
    case 43: return launch(pa_stream_probe_kernel<4, 3>, grid, block, stream, *a, s, v);
    case 24: return launch(pa_stream_probe_kernel<2, 4>, grid, block, stream, *a, s, v);
    case 44: return launch(pa_stream_probe_kernel<4, 4>, grid, block, stream, *a, s, v);
    default: return PA_ERR_UNSUPPORTED;
  }
}

int pa_probe_issue(int32_t mode, int32_t iterations, int32_t workgroups, int32_t* sink, void* hip_stream) {
  if (!sink) return PA_ERR_NULL_POINTER;
  if (iterations <= 0 || workgroups <= 0) return PA_ERR_BAD_SHAPE;
  hipStream_t stream = reinterpret_cast<hipStream_t>(hip_stream);
  const dim3 grid((unsigned)workgroups), block(256);
  int* s = reinterpret_cast<int*>(sink);
  const int it = iterations;
  switch (mode) {
    case 0: return launch(pa_issue_probe_kernel<0>, grid, block, stream, s, it);
    case 1: return launch(pa_issue_probe_kernel<1>, grid, block, stream, s, it);
    case 2: return launch(pa_issue_probe_kernel<2>, grid, block, stream, s, it);
    case 3: return launch(pa_issue_probe_kernel<3>, grid, block, stream, s, it);
    case 4: return launch(pa_issue_probe_kernel<4>, grid, block, stream, s, it);
    case 5: return launch(pa_issue_probe_kernel<5>, grid, block, stream, s, it);
    default: return PA_ERR_UNSUPPORTED;
  }
}

}  // extern "C"
