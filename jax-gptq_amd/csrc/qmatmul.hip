// Packed-int4 matmul: out = x @ dequant(Wpacked)  (and the transposed form).
#include "common.h"

namespace {

constexpr int TPB = 256;

// ---------------------------------------------------------------------------- baseline
// One thread per output element; used for shapes the tuned kernels do not cover.
template <typename TX, typename TZ>
__global__ __launch_bounds__(TPB) void qmm_fwd_simple(const TX *x, int64_t M, const uint8_t *pk,
                                                      int64_t R, int64_t C, const TZ *zero,
                                                      const TZ *scale, TX *out) {
  const int64_t n = (int64_t)blockIdx.x * TPB + threadIdx.x;
  const int64_t m = blockIdx.y;
  if (n >= C) return;
  const TX *xr = x + m * (2 * R);
  float acc = 0.f, xs = 0.f;
  for (int64_t j = 0; j < R; ++j) {
    const uint8_t b = pk[j * C + n];
    const float x0 = to_f32(xr[2 * j]), x1 = to_f32(xr[2 * j + 1]);
    acc += x0 * (float)(b & 0xF) + x1 * (float)(b >> 4);
    xs += x0 + x1;
  }
  const float v = to_f32(scale[n]) * (acc - to_f32(zero[n]) * xs);
  out[m * C + n] = from_f32<TX>(__half2float(__float2half_rn(v)));
}

// transposed: out[m, 2r+p] = sum_c x[m,c] * (nibble_p(pk[r,c]) - zero[c]) * scale[c]
template <typename TX, typename TZ>
__global__ __launch_bounds__(TPB) void qmm_bwd_simple(const TX *x, int64_t M, const uint8_t *pk,
                                                      int64_t R, int64_t C, const TZ *zero,
                                                      const TZ *scale, TX *out) {
  // one wavefront per (m, r): lanes stride over c, then reduce
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * (TPB / 64) + (threadIdx.x >> 6);
  const int64_t m = blockIdx.y;
  if (r >= R) return;
  const TX *xr = x + m * C;
  float a0 = 0.f, a1 = 0.f;
  for (int64_t c = lane; c < C; c += 64) {
    const uint8_t b = pk[r * C + c];
    const float xv = to_f32(xr[c]) * to_f32(scale[c]);
    const float z = to_f32(zero[c]);
    a0 += xv * ((float)(b & 0xF) - z);
    a1 += xv * ((float)(b >> 4) - z);
  }
  for (int off = 32; off > 0; off >>= 1) {
    a0 += __shfl_xor(a0, off);
    a1 += __shfl_xor(a1, off);
  }
  if (lane == 0) {
    out[m * (2 * R) + 2 * r] = from_f32<TX>(__half2float(__float2half_rn(a0)));
    out[m * (2 * R) + 2 * r + 1] = from_f32<TX>(__half2float(__float2half_rn(a1)));
  }
}

template <typename TX, typename TZ>
int launch_simple(hipStream_t st, const void *x, int64_t M, const uint8_t *pk, int64_t R, int64_t C,
                  const void *zero, const void *scale, int transpose_b, void *out) {
  if (M > 65535) return GPTQ_HIP_EINVAL;
  if (!transpose_b) {
    hipLaunchKernelGGL((qmm_fwd_simple<TX, TZ>), dim3((unsigned)ceil_div64(C, TPB), (unsigned)M),
                       dim3(TPB), 0, st, (const TX *)x, M, pk, R, C, (const TZ *)zero,
                       (const TZ *)scale, (TX *)out);
  } else {
    hipLaunchKernelGGL((qmm_bwd_simple<TX, TZ>),
                       dim3((unsigned)ceil_div64(R, TPB / 64), (unsigned)M), dim3(TPB), 0, st,
                       (const TX *)x, M, pk, R, C, (const TZ *)zero, (const TZ *)scale, (TX *)out);
  }
  GPTQ_CHECK_LAUNCH();
  return GPTQ_HIP_OK;
}

template <typename TX>
int dispatch_z(hipStream_t st, const void *x, int64_t M, const uint8_t *pk, int64_t R, int64_t C,
               const void *zero, const void *scale, int zs_dtype, int transpose_b, void *out) {
  switch (zs_dtype) {
    case GPTQ_HIP_F32:
      return launch_simple<TX, float>(st, x, M, pk, R, C, zero, scale, transpose_b, out);
    case GPTQ_HIP_F16:
      return launch_simple<TX, __half>(st, x, M, pk, R, C, zero, scale, transpose_b, out);
    case GPTQ_HIP_BF16:
      return launch_simple<TX, __hip_bfloat16>(st, x, M, pk, R, C, zero, scale, transpose_b, out);
    default:
      return GPTQ_HIP_EDTYPE;
  }
}

}  // namespace

extern "C" {

size_t gptq_hip_qmatmul_workspace_bytes(int64_t M, int64_t R, int64_t C, int transpose_b) {
  (void)M; (void)R; (void)C; (void)transpose_b;
  return 0;
}

int gptq_hip_qmatmul(void *stream, const void *x, int x_dtype, int64_t M, const uint8_t *packed,
                     int64_t R, int64_t C, const void *zero, const void *scale, int zs_dtype,
                     int transpose_b, void *out, void *ws, size_t ws_bytes) {
  (void)ws; (void)ws_bytes;
  if (M < 0 || R <= 0 || C <= 0) return GPTQ_HIP_EINVAL;
  if (M == 0) return GPTQ_HIP_OK;
  if (!x || !packed || !zero || !scale || !out) return GPTQ_HIP_EINVAL;
  hipStream_t st = as_stream(stream);
  switch (x_dtype) {
    case GPTQ_HIP_F32:
      return dispatch_z<float>(st, x, M, packed, R, C, zero, scale, zs_dtype, transpose_b, out);
    case GPTQ_HIP_F16:
      return dispatch_z<__half>(st, x, M, packed, R, C, zero, scale, zs_dtype, transpose_b, out);
    case GPTQ_HIP_BF16:
      return dispatch_z<__hip_bfloat16>(st, x, M, packed, R, C, zero, scale, zs_dtype, transpose_b,
                                        out);
    default:
      return GPTQ_HIP_EDTYPE;
  }
}

}  // extern "C"
