// MFMA GEMMs used by the Hessian, the Cholesky/inverse and the lazy block update: an fp32
// one (v_mfma_f32_32x32x2_f32) and an fp64 one (v_mfma_f64_16x16x4_f64) behind one argument block.
#pragma once
#include "common.h"

// C[m, n] = alpha * op(A) * B + beta * C.
//   a_kmajor = 1: A is stored [k][m] (op(A) = A^T, the X^T X form); 0: A is stored [m][k].
//   B is always stored [k][n].
struct GemmArgs {
  const void *A = nullptr;
  const void *B = nullptr;
  void *C = nullptr;   // float for gptq_gemm_f32, double for gptq_gemm_f64
  int64_t lda = 0, ldb = 0, ldc = 0;
  int m = 0, n = 0, k = 0;
  float alpha = 1.f, beta = 0.f;
  int a_kmajor = 0;
  int in_dtype = GPTQ_HIP_F32;  // element type of A and B (GPTQ_HIP_F64 only for gptq_gemm_f64)
  // tile filter for symmetric results: 0 all tiles, 1 upper (tile_n >= tile_m), 2 lower.
  int tri = 0;
  // structural zeros: bit0: B[k][n] == 0 for k < n-tile start (B lower triangular);
  //                   bit1: A[m][k] == 0 for k >= m-tile end (A lower triangular).
  int kskip = 0;
  // batching over blockIdx.z with constant element strides
  int batch = 1;
  int64_t strideA = 0, strideB = 0, strideC = 0;
  // ragged last batch entry: m_eff = min(m, m_total - z*m_step), same for k (0 = off)
  int m_total = 0, m_step = 0;
  int k_total = 0, k_step = 0;
};

int gptq_gemm_f32(hipStream_t stream, const GemmArgs &args);
int gptq_gemm_f64(hipStream_t stream, const GemmArgs &args);

// the GEMM whose accumulator and result type is R
inline int gptq_gemm(hipStream_t stream, const GemmArgs &args, float *) { return gptq_gemm_f32(stream, args); }
inline int gptq_gemm(hipStream_t stream, const GemmArgs &args, double *) { return gptq_gemm_f64(stream, args); }
