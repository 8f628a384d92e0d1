// Vectorised tile loads shared by the fp32 MFMA kernels: four consecutive elements of a row
// of fp32 / fp16 / bf16 data, converted to fp32.
#pragma once
#include "common.h"

typedef float floatx16 __attribute__((ext_vector_type(16)));

template <typename T> struct Vec4;
template <> struct Vec4<float> {
  static __device__ __forceinline__ void load(const float *p, float (&v)[4]) {
    const float4 r = *reinterpret_cast<const float4 *>(p);
    v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w;
  }
};
template <> struct Vec4<__half> {
  static __device__ __forceinline__ void load(const __half *p, float (&v)[4]) {
    const uint2 r = *reinterpret_cast<const uint2 *>(p);
    const __half2 a = *reinterpret_cast<const __half2 *>(&r.x);
    const __half2 b = *reinterpret_cast<const __half2 *>(&r.y);
    const float2 fa = __half22float2(a), fb = __half22float2(b);
    v[0] = fa.x; v[1] = fa.y; v[2] = fb.x; v[3] = fb.y;
  }
};
template <> struct Vec4<__hip_bfloat16> {
  static __device__ __forceinline__ void load(const __hip_bfloat16 *p, float (&v)[4]) {
    const uint2 r = *reinterpret_cast<const uint2 *>(p);
    v[0] = __uint_as_float(r.x << 16); v[1] = __uint_as_float(r.x & 0xffff0000u);
    v[2] = __uint_as_float(r.y << 16); v[3] = __uint_as_float(r.y & 0xffff0000u);
  }
};

// 4 consecutive elements of a row; `nvalid` of them exist (0..4), the rest read as 0.
template <typename T>
__device__ __forceinline__ void load_row4(const T *p, bool fast, int nvalid, float (&v)[4]) {
  if (fast) {
    Vec4<T>::load(p, v);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = (e < nvalid) ? to_f32(p[e]) : 0.f;
  }
}

