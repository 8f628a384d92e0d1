// Shared host/device helpers of the gfx950 GPTQ library.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hip/hip_bf16.h>
#include <stdint.h>
#include <stddef.h>

#include "../../include/gptq_hip.h"

#define GPTQ_CHECK_LAUNCH()                                   \
  do {                                                        \
    if (hipGetLastError() != hipSuccess) return GPTQ_HIP_ELAUNCH; \
  } while (0)

// Raises the dynamic-LDS limit of a kernel (hipFuncAttributeMaxDynamicSharedMemorySize) the first time
// the kernel is used on a device with that size and remembers it: later calls are a table lookup and
// make no HIP call.  Returns false if the runtime refuses.  (api.hip)
bool gptq_raise_lds_limit(const void *kernel, int bytes);

static inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

static inline int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline int64_t round_up64(int64_t a, int64_t b) { return ceil_div64(a, b) * b; }

// element conversion to float for the three supported input types
__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(__half v) { return __half2float(v); }
__device__ __forceinline__ float to_f32(__hip_bfloat16 v) { return __bfloat162float(v); }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ __half from_f32<__half>(float v) { return __float2half_rn(v); }
template <> __device__ __forceinline__ __hip_bfloat16 from_f32<__hip_bfloat16>(float v) {
  return __float2bfloat16(v);
}

static inline size_t dtype_size(int dt) {
  return dt == GPTQ_HIP_F64 ? 8 : (dt == GPTQ_HIP_F32 ? 4 : 2);
}
