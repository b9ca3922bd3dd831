// Kernel launches of the library: every launch goes through pa_launch(), which takes the launch's own return code.
// The HIP runtime also keeps a sticky "last error" per thread; an error that the caller's earlier work left there
// is the caller's, and is neither read nor cleared here.
#ifndef PA_LAUNCH_H_
#define PA_LAUNCH_H_

#include <hip/hip_runtime.h>

#include <type_traits>

#include "../../include/pa_decode.h"

// hipError_t of the calling thread's last failed launch (pa_decode_last_hip_error); defined in pa_decode.hip
extern thread_local int pa_last_hip_error __attribute__((visibility("hidden")));

// Launches kernel<<<grid, block, lds_bytes, stream>>>(args...) and returns PA_OK or PA_ERR_LAUNCH.
template <typename... KArgs>
inline int pa_launch(void (*kernel)(KArgs...), dim3 grid, dim3 block, unsigned lds_bytes, hipStream_t stream,
                     std::type_identity_t<KArgs>... args) {
  void* ptrs[] = {const_cast<void*>(static_cast<const void*>(&args))...};
  const hipError_t e = hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, ptrs, lds_bytes, stream);
  if (e == hipSuccess) return PA_OK;
  pa_last_hip_error = (int)e;
  return PA_ERR_LAUNCH;
}

#endif  // PA_LAUNCH_H_
