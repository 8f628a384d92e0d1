// fp64 MFMA GEMM for gfx950: C = alpha * op(A) * B + beta * C with C and the accumulation
// in double; A and B may be fp16, bf16, fp32 (all converted exactly) or fp64.
//
// Same tiling as the fp32 kernel: a workgroup of 4 wavefronts owns a 128x128 tile of C and
// each wavefront a 64x64 quadrant, here as 4x4 tiles of v_mfma_f64_16x16x4_f64 (64
// accumulator doubles per lane).  The instruction occupies the matrix pipe for 64 cycles
// and needs one double of A and one of B per lane, so the LDS traffic (8 ds_read_b64 per
// 16 MFMAs) and the global loads hide behind it; both operands are kept k-major in LDS
// ([k][idx], row stride 144 doubles: the two k rows a half-wave reads are 32 banks apart).
// A stored [m][k] is transposed on its way into LDS.
//
// Operand layout of the instruction (lane l): A[i = l % 16][k = l / 16],
// B[k = l / 16][j = l % 16]; result register r of lane l is D[i = 4 * r + l / 16][j = l % 16].
#include "gemm_f32.h"

namespace {

constexpr int BM = 128, BN = 128, BK = 8, NTHREADS = 256;
constexpr int LDD = 144;
typedef double doublex4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ double to_f64(double v) { return v; }
__device__ __forceinline__ double to_f64(float v) { return (double)v; }
__device__ __forceinline__ double to_f64(__half v) { return (double)__half2float(v); }
__device__ __forceinline__ double to_f64(__hip_bfloat16 v) { return (double)__bfloat162float(v); }

// four consecutive elements; nv (0..4) of them exist, the rest read as zero
template <typename T>
__device__ __forceinline__ void load4_f64(const T *src, bool fast, int nv, double out[4]) {
  if (fast) {
    if constexpr (sizeof(T) == 8) {
      const double2 a = *reinterpret_cast<const double2 *>(src);
      const double2 b = *reinterpret_cast<const double2 *>(src + 2);
      out[0] = a.x; out[1] = a.y; out[2] = b.x; out[3] = b.y;
    } else if constexpr (sizeof(T) == 4) {
      const float4 a = *reinterpret_cast<const float4 *>(src);
      out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w;
    } else {
      struct alignas(8) Q { T v[4]; };
      const Q q = *reinterpret_cast<const Q *>(src);
#pragma unroll
      for (int e = 0; e < 4; ++e) out[e] = to_f64(q.v[e]);
    }
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) out[e] = (e < nv) ? to_f64(src[e]) : 0.0;
  }
}

// FAST: every tile is full and every 4-element group aligned (checked on the host), so the
// loads carry no guards: a load inside a branch would make the compiler wait for it at the
// join, in front of the MFMAs it is meant to overlap with.
template <typename T, bool AK, bool FAST>
__global__ __launch_bounds__(NTHREADS) void gemm_f64_kernel(GemmArgs p) {
  __shared__ __attribute__((aligned(16))) double As[2][BK * LDD];
  __shared__ __attribute__((aligned(16))) double Bs[2][BK * LDD];

  int tm, tn;
  if (p.tri) {
    const int t = blockIdx.x;
    int i = (int)((sqrtf(8.f * (float)t + 1.f) - 1.f) * 0.5f);
    while ((i + 1) * (i + 2) / 2 <= t) ++i;
    while (i * (i + 1) / 2 > t) --i;
    const int j = t - i * (i + 1) / 2;  // j <= i
    if (p.tri == 2) { tm = i; tn = j; } else { tm = j; tn = i; }
  } else {
    tn = blockIdx.x;
    tm = blockIdx.y;
  }
  const int z = blockIdx.z;
  int m_eff = p.m, k_eff = p.k;
  if (p.m_step) m_eff = min(p.m, p.m_total - z * p.m_step);
  if (p.k_step) k_eff = min(p.k, p.k_total - z * p.k_step);
  const int m0 = tm * BM, n0 = tn * BN;
  if (m0 >= m_eff || n0 >= p.n || k_eff <= 0) return;

  int kb = 0, ke = k_eff;
  if (p.kskip & 1) kb = min(n0, ke) & ~(BK - 1);
  if (p.kskip & 2) ke = min(ke, m0 + BM);

  const T *A = reinterpret_cast<const T *>(p.A) + (int64_t)z * p.strideA;
  const T *B = reinterpret_cast<const T *>(p.B) + (int64_t)z * p.strideB;
  double *C = reinterpret_cast<double *>(p.C) + (int64_t)z * p.strideC;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int l16 = lane & 15, lk = lane >> 4;

  constexpr int VB = 4 * sizeof(T) < 16 ? 4 * sizeof(T) : 16;   // alignment the fast path needs
  const bool a_al = (p.lda % 4 == 0) && ((reinterpret_cast<uintptr_t>(A) % VB) == 0);
  const bool b_al = (p.ldb % 4 == 0) && ((reinterpret_cast<uintptr_t>(B) % VB) == 0);
  const bool m_full = (m0 + BM <= m_eff);
  const bool n_full = (n0 + BN <= p.n);

  double ra[4], rb[4];

  auto load_tiles = [&](int kt) {
    const bool k_full = (kt + BK <= ke);
    if (AK) {   // A stored [k][m]: 8 k rows x 128 m, four consecutive m per thread
      const int r = tid >> 5, c4 = (tid & 31) * 4;
      const int kk = kt + r;
      const int nv = (kk < ke) ? min(4, m_eff - (m0 + c4)) : 0;
      load4_f64<T>(A + (int64_t)kk * p.lda + m0 + c4, FAST || (a_al && m_full && k_full), nv, ra);
    } else {    // A stored [m][k]: 128 m rows x 8 k, four consecutive k per thread
      const int row = tid >> 1, k4 = (tid & 1) * 4;
      const int mm = m0 + row;
      const int nv = (mm < m_eff) ? min(4, ke - (kt + k4)) : 0;
      load4_f64<T>(A + (int64_t)mm * p.lda + kt + k4, FAST || (a_al && m_full && k_full), nv, ra);
    }
    {
      const int r = tid >> 5, c4 = (tid & 31) * 4;
      const int kk = kt + r;
      const int nv = (kk < ke) ? min(4, p.n - (n0 + c4)) : 0;
      load4_f64<T>(B + (int64_t)kk * p.ldb + n0 + c4, FAST || (b_al && n_full && k_full), nv, rb);
    }
  };

  auto store_tiles = [&](int buf) {
    if (AK) {
      const int r = tid >> 5, c4 = (tid & 31) * 4;
#pragma unroll
      for (int e = 0; e < 4; ++e) As[buf][r * LDD + c4 + e] = ra[e];
    } else {
      const int row = tid >> 1, k4 = (tid & 1) * 4;
#pragma unroll
      for (int e = 0; e < 4; ++e) As[buf][(k4 + e) * LDD + row] = ra[e];
    }
    {
      const int r = tid >> 5, c4 = (tid & 31) * 4;
#pragma unroll
      for (int e = 0; e < 4; ++e) Bs[buf][r * LDD + c4 + e] = rb[e];
    }
  };

  doublex4 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0;

  int buf = 0;
  if (kb < ke) {
    load_tiles(kb);
    store_tiles(0);
  }
  __syncthreads();
  for (int kt = kb; kt < ke; kt += BK) {
    const bool more = (kt + BK < ke);
    if (more) load_tiles(kt + BK);
    const double *as = As[buf];
    const double *bs = Bs[buf];
#pragma unroll
    for (int kk = 0; kk < BK; kk += 4) {
      const int krow = kk + lk;
      double a[4], b[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        a[t] = as[krow * LDD + wm * 64 + t * 16 + l16];
        b[t] = bs[krow * LDD + wn * 64 + t * 16 + l16];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    if (more) store_tiles(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }

  const double alpha = (double)p.alpha, beta = (double)p.beta;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = n0 + wn * 64 + j * 16 + l16;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = m0 + wm * 64 + i * 16 + lk + 4 * r;
        if (row < m_eff && col < p.n) {
          double *dst = C + (int64_t)row * p.ldc + col;
          double v = alpha * acc[i][j][r];
          if (beta != 0.0) v += beta * (*dst);
          *dst = v;
        }
      }
    }
}

template <typename T>
void launch(hipStream_t stream, dim3 grid, const GemmArgs &a) {
  const uintptr_t vb = 4 * sizeof(T) < 16 ? 4 * sizeof(T) : 16;
  const bool fast = a.m % BM == 0 && a.n % BN == 0 && a.k % BK == 0 && a.m_step == 0 &&
                    a.k_step == 0 && a.lda % 4 == 0 && a.ldb % 4 == 0 &&
                    reinterpret_cast<uintptr_t>(a.A) % vb == 0 &&
                    reinterpret_cast<uintptr_t>(a.B) % vb == 0 &&
                    (a.batch == 1 || (a.strideA % 4 == 0 && a.strideB % 4 == 0));
  const dim3 block(NTHREADS);
  if (a.a_kmajor) {
    if (fast) hipLaunchKernelGGL((gemm_f64_kernel<T, true, true>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((gemm_f64_kernel<T, true, false>), grid, block, 0, stream, a);
  } else {
    if (fast) hipLaunchKernelGGL((gemm_f64_kernel<T, false, true>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((gemm_f64_kernel<T, false, false>), grid, block, 0, stream, a);
  }
}

}  // namespace

int gptq_gemm_f64(hipStream_t stream, const GemmArgs &a) {
  if (a.m <= 0 || a.n <= 0 || a.batch <= 0) return GPTQ_HIP_OK;
  if (!a.A || !a.B || !a.C) return GPTQ_HIP_EINVAL;
  dim3 grid;
  const int tm = (a.m + BM - 1) / BM, tn = (a.n + BN - 1) / BN;
  if (a.tri) {
    const int t = tm > tn ? tm : tn;
    grid = dim3((unsigned)((int64_t)t * (t + 1) / 2), 1, (unsigned)a.batch);
  } else {
    grid = dim3((unsigned)tn, (unsigned)tm, (unsigned)a.batch);
  }
  if (grid.y > 65535u || grid.z > 65535u) return GPTQ_HIP_EINVAL;
  switch (a.in_dtype) {
    case GPTQ_HIP_F64: launch<double>(stream, grid, a); break;
    case GPTQ_HIP_F32: launch<float>(stream, grid, a); break;
    case GPTQ_HIP_F16: launch<__half>(stream, grid, a); break;
    case GPTQ_HIP_BF16: launch<__hip_bfloat16>(stream, grid, a); break;
    default: return GPTQ_HIP_EDTYPE;
  }
  GPTQ_CHECK_LAUNCH();
  return GPTQ_HIP_OK;
}
