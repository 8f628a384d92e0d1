// Hessian accumulation H += sum_b X_b^T X_b (upper 128x128 tiles) and its finalisation.
#include "common.h"
#include "gemm_f32.h"

namespace {

constexpr int TS = 32;

// Scale the upper tiles by 1/n and mirror them below the diagonal.  One workgroup
// per 32x32 tile pair (ti <= tj); the transposed copy goes through LDS so that both
// the read and the mirrored write are coalesced.
__global__ __launch_bounds__(TS * 8) void finalize_kernel(float *H, int64_t K, float n) {
  __shared__ float tile[TS][TS + 1];
  const int t = blockIdx.x;
  int j = (int)((sqrtf(8.f * (float)t + 1.f) - 1.f) * 0.5f);
  while ((j + 1) * (j + 2) / 2 <= t) ++j;
  while (j * (j + 1) / 2 > t) --j;
  const int i = t - j * (j + 1) / 2;  // i <= j : tile row i, tile column j (upper)
  const int tx = threadIdx.x % TS, ty = threadIdx.x / TS;
  for (int r = ty; r < TS; r += 8) {
    const int64_t row = (int64_t)i * TS + r, col = (int64_t)j * TS + tx;
    float v = 0.f;
    if (row < K && col < K) {
      v = H[row * K + col] / n;
      // inside a diagonal tile only the upper part is authoritative
      if (i != j || col >= row) H[row * K + col] = v;
    }
    tile[r][tx] = v;
  }
  __syncthreads();
  for (int r = ty; r < TS; r += 8) {
    // element (row', col') of the mirrored tile (j, i) = tile[tx][r] transposed
    const int64_t row = (int64_t)j * TS + r, col = (int64_t)i * TS + tx;
    if (row < K && col < K && (i != j || col < row)) H[row * K + col] = tile[tx][r];
  }
}

}  // namespace

extern "C" {

int gptq_hip_hessian_accumulate(void *stream, const void *const *x_ptrs, const int64_t *x_rows,
                                int n_batches, int x_dtype, int64_t K, float *H) {
  if (n_batches < 0 || K <= 0 || K > 2147483647LL / 2 || !H) return GPTQ_HIP_EINVAL;
  if (x_dtype != GPTQ_HIP_F32 && x_dtype != GPTQ_HIP_F16 && x_dtype != GPTQ_HIP_BF16)
    return GPTQ_HIP_EDTYPE;
  if (n_batches > 0 && (!x_ptrs || !x_rows)) return GPTQ_HIP_EINVAL;
  for (int b = 0; b < n_batches; ++b) {
    if (x_rows[b] < 0 || x_rows[b] > 2147483647LL) return GPTQ_HIP_EINVAL;
    if (x_rows[b] == 0) continue;
    if (!x_ptrs[b]) return GPTQ_HIP_EINVAL;
    GemmArgs g;
    g.A = x_ptrs[b];
    g.B = x_ptrs[b];
    g.C = H;
    g.lda = g.ldb = g.ldc = K;
    g.m = g.n = (int)K;
    g.k = (int)x_rows[b];
    g.alpha = 1.f;
    g.beta = 1.f;
    g.a_kmajor = 1;
    g.in_dtype = x_dtype;
    g.tri = 1;
    const int rc = gptq_gemm_f32(as_stream(stream), g);
    if (rc) return rc;
  }
  return GPTQ_HIP_OK;
}

int gptq_hip_hessian_finalize(void *stream, float *H, int64_t K, double n_samples) {
  if (!H || K <= 0 || !(n_samples > 0)) return GPTQ_HIP_EINVAL;
  const int64_t T = ceil_div64(K, TS);
  hipLaunchKernelGGL(finalize_kernel, dim3((unsigned)(T * (T + 1) / 2)), dim3(TS * 8), 0,
                     as_stream(stream), H, K, (float)n_samples);
  GPTQ_CHECK_LAUNCH();
  return GPTQ_HIP_OK;
}

}  // extern "C"
