// Hessian accumulation H += sum_b X_b^T X_b (upper 128x128 tiles) and its finalisation.
//
// X^T X kernel (fp32 MFMA, v_mfma_f32_32x32x2_f32).  One workgroup owns one upper 128x128
// tile of H and one of RS row slices of EVERY batch of the launch: it walks the batches in
// order, stages 16-row slabs of the two 128-feature panels of X through LDS (double
// buffered, natural [row][feature] layout, which is already the k-major layout the MFMA
// operand fetch wants for both operands) and keeps the tile in 64 accumulator VGPRs per
// lane for the whole launch.  Consequences:
//   * T * RS workgroups (thousands) are scheduled dynamically over the 256 CUs, so the tile
//     count no longer has to be a multiple of the number of CUs;
//   * workgroups that run together read the same few rows of the same batch: the slice of
//     one batch (rows/RS x K) stays L2 resident and X is read from HBM once;
//   * H is touched once per launch instead of once per batch.
// With RS > 1 the RS partial tiles go to a caller-provided workspace and a second kernel
// adds them to H in slice order, so the result does not depend on scheduling.
#include "common.h"
#include "gemm_f32.h"
#include "tile_io.h"

namespace {

constexpr int HB = 128;        // tile edge
constexpr int HBK = 16;        // rows per LDS slab
constexpr int HLD = 160;       // LDS row stride (floats): half-waves land 32 banks apart
constexpr int H_NBMAX = 128;   // batches per launch (pointer table lives in the kernel arguments)
constexpr int H_RSMAX = 16;

struct SyrkArgs {
  const void *ptr[H_NBMAX];
  int rows[H_NBMAX];
  int nb;
  int K;
  int T;       // tiles per side
  int RS;      // row slices
  float *H;
  float *ws;   // [RS][tiles][128][128] when RS > 1
};

__device__ __forceinline__ void tile_decode(int t, int &ti, int &tj) {
  int j = (int)((sqrtf(8.f * (float)t + 1.f) - 1.f) * 0.5f);
  while ((j + 1) * (j + 2) / 2 <= t) ++j;
  while (j * (j + 1) / 2 > t) --j;
  ti = t - j * (j + 1) / 2;  // ti <= tj : upper triangle
  tj = j;
}

// FAST: K % 128 == 0, every batch 16-byte aligned with a multiple of 16 rows.  All slabs are
// then full and aligned, the loads carry no predicates or branches, and the compiler keeps
// the prefetch of slab s+1 in flight across the MFMAs of slab s.
template <typename T, bool FAST>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) void syrk_kernel(SyrkArgs p) {
  __shared__ __attribute__((aligned(16))) float As[2][HBK * HLD];
  __shared__ __attribute__((aligned(16))) float Bs[2][HBK * HLD];
  const int ntiles = p.T * (p.T + 1) / 2;
  // Workgroup ids are dealt round-robin to the 8 XCDs (each with its own L2).  With a
  // multiple of 8 row slices, give every XCD its own slices: all tiles of one slice then
  // run on one XCD and that L2 sees only 1/RS of the rows of X.
  int rs, t;
  if ((p.RS & 7) == 0) {
    const int xcd = blockIdx.x & 7, q = blockIdx.x >> 3;
    rs = xcd + 8 * (q / ntiles);
    t = q % ntiles;
  } else {
    rs = blockIdx.x / ntiles;
    t = blockIdx.x - rs * ntiles;
  }
  int ti, tj;
  tile_decode(t, ti, tj);
  const int m0 = ti * HB, n0 = tj * HB, K = p.K;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, lhi = lane >> 5;
  const bool m_full = (m0 + HB <= K), n_full = (n0 + HB <= K);
  const bool k_al = (K % 4 == 0);
  const int lr = tid >> 5, c4 = (tid & 31) * 4;   // this thread's slab row (and +8) / column

  // row range [r0, r1) of slice rs in batch b
  auto range = [&](int b, int &r0, int &r1) {
    const int rows = p.rows[b];
    const int chunk = (((rows + p.RS - 1) / p.RS) + HBK - 1) & ~(HBK - 1);
    r0 = min(rows, rs * chunk);
    r1 = min(rows, r0 + chunk);
  };
  int b = 0, kt = 0, r1 = 0;
  auto seek = [&]() {   // skip batches whose slice is empty
    while (b < p.nb) {
      int r0;
      range(b, r0, r1);
      if (r0 < r1) { kt = r0; return; }
      ++b;
    }
  };
  seek();

  float ra[2][4], rb[2][4];
  auto load_slab = [&](int bb, int kk0, int kend) {
    const T *X = reinterpret_cast<const T *>(p.ptr[bb]);
    const bool al = k_al && ((reinterpret_cast<uintptr_t>(X) % (4 * sizeof(T))) == 0);
    const bool k_full = (kk0 + HBK <= kend);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int kk = kk0 + lr + 8 * i;
      const T *row = X + (int64_t)kk * K;
      if (FAST) {
        Vec4<T>::load(row + m0 + c4, ra[i]);
        Vec4<T>::load(row + n0 + c4, rb[i]);
      } else {
        const int nva = (kk < kend) ? min(4, K - (m0 + c4)) : 0;
        const int nvb = (kk < kend) ? min(4, K - (n0 + c4)) : 0;
        load_row4<T>(row + m0 + c4, al && m_full && k_full, nva, ra[i]);
        load_row4<T>(row + n0 + c4, al && n_full && k_full, nvb, rb[i]);
      }
    }
  };
  auto store_slab = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      *reinterpret_cast<float4 *>(&As[buf][(lr + 8 * i) * HLD + c4]) =
          make_float4(ra[i][0], ra[i][1], ra[i][2], ra[i][3]);
      *reinterpret_cast<float4 *>(&Bs[buf][(lr + 8 * i) * HLD + c4]) =
          make_float4(rb[i][0], rb[i][1], rb[i][2], rb[i][3]);
    }
  };

  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  if (b < p.nb) {
    int buf = 0;
    load_slab(b, kt, r1);
    store_slab(0);
    __syncthreads();
    while (true) {
      // position of the next slab (possibly in a later batch)
      int nb_ = b, nkt = kt + HBK, nr1 = r1;
      if (nkt >= r1) {
        ++b;
        seek();
        nb_ = b; nkt = kt; nr1 = r1;
      } else {
        kt = nkt;
      }
      const bool more = (nb_ < p.nb);
      if (more) load_slab(nb_, nkt, nr1);
      const float *as = As[buf];
      const float *bs = Bs[buf];
#pragma unroll
      for (int kk = 0; kk < HBK; kk += 2) {
        const int krow = kk + lhi;
        float a[2], bq[2];
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          a[q] = as[krow * HLD + wm * 64 + q * 32 + l32];
          bq[q] = bs[krow * HLD + wn * 64 + q * 32 + l32];
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], bq[j], acc[i][j], 0, 0, 0);
      }
      if (more) store_slab(buf ^ 1);
      __syncthreads();
      buf ^= 1;
      if (!more) break;
    }
  }

  if (p.RS == 1) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int col = n0 + wn * 64 + j * 32 + l32;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3);
          if (row < K && col < K) p.H[(int64_t)row * K + col] += acc[i][j][r];
        }
      }
  } else {
    float *dst = p.ws + ((int64_t)rs * ntiles + t) * (HB * HB);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int col = wn * 64 + j * 32 + l32;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = wm * 64 + i * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3);
          dst[row * HB + col] = acc[i][j][r];
        }
      }
  }
}

// H tile += sum over the row slices, in slice order
__global__ __launch_bounds__(256) void syrk_reduce_kernel(float *H, const float *ws, int K, int T,
                                                          int RS) {
  const int ntiles = T * (T + 1) / 2;
  const int t = blockIdx.x;
  int ti, tj;
  tile_decode(t, ti, tj);
  const int m0 = ti * HB, n0 = tj * HB;
  for (int e = threadIdx.x; e < HB * HB / 4; e += 256) {
    const int row = e >> 5, c4 = (e & 31) * 4;
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int rs = 0; rs < RS; ++rs) {
      const float4 v = *reinterpret_cast<const float4 *>(
          ws + ((int64_t)rs * ntiles + t) * (HB * HB) + row * HB + c4);
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    const int gr = m0 + row, gc = n0 + c4;
    if (gr >= K) continue;
    float *dst = H + (int64_t)gr * K + gc;
    if (gc + 0 < K) dst[0] += s.x;
    if (gc + 1 < K) dst[1] += s.y;
    if (gc + 2 < K) dst[2] += s.z;
    if (gc + 3 < K) dst[3] += s.w;
  }
}

int pick_rs(int64_t K) {
  const int64_t T = ceil_div64(K, HB), ntiles = T * (T + 1) / 2;
  int64_t rs = ceil_div64(6144, ntiles);   // about eight waves of workgroups over 768 slots
  if (rs < 1) rs = 1;
  if (rs > 4) rs = (rs <= 8) ? 8 : H_RSMAX;   // multiples of 8 get the per-XCD slice mapping
  return (int)rs;
}

constexpr int TS = 32;

// Scale the upper tiles by 1/n and mirror them below the diagonal.  One workgroup
// per 32x32 tile pair (ti <= tj); the transposed copy goes through LDS so that both
// the read and the mirrored write are coalesced.
template <typename R>
__global__ __launch_bounds__(TS * 8) void finalize_kernel(R *H, int64_t K, R n) {
  __shared__ R tile[TS][TS + 1];
  const int t = blockIdx.x;
  int j = (int)((sqrtf(8.f * (float)t + 1.f) - 1.f) * 0.5f);
  while ((j + 1) * (j + 2) / 2 <= t) ++j;
  while (j * (j + 1) / 2 > t) --j;
  const int i = t - j * (j + 1) / 2;  // i <= j : tile row i, tile column j (upper)
  const int tx = threadIdx.x % TS, ty = threadIdx.x / TS;
  for (int r = ty; r < TS; r += 8) {
    const int64_t row = (int64_t)i * TS + r, col = (int64_t)j * TS + tx;
    R v = 0;
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

size_t gptq_hip_hessian_accumulate_workspace_bytes(int64_t K, int h_dtype) {
  if (K <= 0 || h_dtype != GPTQ_HIP_F32) return 0;
  const int rs = pick_rs(K);
  if (rs == 1) return 0;
  const int64_t T = ceil_div64(K, HB), ntiles = T * (T + 1) / 2;
  return (size_t)rs * ntiles * HB * HB * sizeof(float);
}

int gptq_hip_hessian_accumulate(void *stream, const void *const *x_ptrs, const int64_t *x_rows,
                                int n_batches, int x_dtype, int64_t K, void *Hv, int h_dtype,
                                void *ws, size_t ws_bytes) {
  if (n_batches < 0 || K <= 0 || K > 46000 || !Hv) return GPTQ_HIP_EINVAL;
  if (h_dtype != GPTQ_HIP_F32 && h_dtype != GPTQ_HIP_F64) return GPTQ_HIP_EDTYPE;
  if (x_dtype != GPTQ_HIP_F32 && x_dtype != GPTQ_HIP_F16 && x_dtype != GPTQ_HIP_BF16 &&
      !(x_dtype == GPTQ_HIP_F64 && h_dtype == GPTQ_HIP_F64))
    return GPTQ_HIP_EDTYPE;
  if (n_batches > 0 && (!x_ptrs || !x_rows)) return GPTQ_HIP_EINVAL;
  hipStream_t st = as_stream(stream);
  if (h_dtype == GPTQ_HIP_F64) {
    // fp64 accumulation: one X_b^T X_b product per batch on the fp64 MFMA GEMM, upper tiles
    for (int b = 0; b < n_batches; ++b) {
      const int64_t rows = x_rows[b];
      if (rows < 0 || rows > 2147483647LL) return GPTQ_HIP_EINVAL;
      if (rows == 0) continue;
      if (!x_ptrs[b]) return GPTQ_HIP_EINVAL;
      GemmArgs g;
      g.A = x_ptrs[b];
      g.B = x_ptrs[b];
      g.C = Hv;
      g.lda = g.ldb = g.ldc = K;
      g.m = g.n = (int)K;
      g.k = (int)rows;
      g.alpha = 1.f;
      g.beta = 1.f;
      g.a_kmajor = 1;
      g.in_dtype = x_dtype;
      g.tri = 1;
      const int rc = gptq_gemm_f64(st, g);
      if (rc) return rc;
    }
    return GPTQ_HIP_OK;
  }
  float *H = reinterpret_cast<float *>(Hv);
  const size_t need = gptq_hip_hessian_accumulate_workspace_bytes(K, h_dtype);
  if (need && (!ws || ws_bytes < need)) return GPTQ_HIP_EWORKSPACE;
  const int T = (int)ceil_div64(K, HB);
  const int ntiles = T * (T + 1) / 2;
  int b0 = 0;
  while (b0 < n_batches) {
    SyrkArgs a;
    a.nb = 0;
    int64_t max_rows = 0;
    while (b0 < n_batches && a.nb < H_NBMAX) {
      const int64_t rows = x_rows[b0];
      if (rows < 0 || rows > 2147483647LL) return GPTQ_HIP_EINVAL;
      if (rows > 0) {
        if (!x_ptrs[b0]) return GPTQ_HIP_EINVAL;
        a.ptr[a.nb] = x_ptrs[b0];
        a.rows[a.nb] = (int)rows;
        ++a.nb;
        if (rows > max_rows) max_rows = rows;
      }
      ++b0;
    }
    if (a.nb == 0) continue;
    a.K = (int)K;
    a.T = T;
    a.RS = pick_rs(K);
    // never more slices than 16-row slabs in the largest batch
    const int64_t slabs = ceil_div64(max_rows, HBK);
    while (a.RS > 1 && a.RS > slabs) a.RS = (a.RS > 8) ? 8 : ((a.RS > 4) ? 4 : a.RS - 1);
    a.H = H;
    a.ws = reinterpret_cast<float *>(ws);
    const dim3 grid((unsigned)((int64_t)ntiles * a.RS)), block(256);
    bool fast = (K % HB == 0);
    for (int i = 0; i < a.nb && fast; ++i)
      fast = (a.rows[i] % HBK == 0) && ((reinterpret_cast<uintptr_t>(a.ptr[i]) & 15) == 0);
#define GPTQ_SYRK_LAUNCH(T)                                                       \
  do {                                                                            \
    if (fast) hipLaunchKernelGGL((syrk_kernel<T, true>), grid, block, 0, st, a);  \
    else hipLaunchKernelGGL((syrk_kernel<T, false>), grid, block, 0, st, a);      \
  } while (0)
    switch (x_dtype) {
      case GPTQ_HIP_F32: GPTQ_SYRK_LAUNCH(float); break;
      case GPTQ_HIP_F16: GPTQ_SYRK_LAUNCH(__half); break;
      default: GPTQ_SYRK_LAUNCH(__hip_bfloat16); break;
    }
#undef GPTQ_SYRK_LAUNCH
    GPTQ_CHECK_LAUNCH();
    if (a.RS > 1) {
      hipLaunchKernelGGL(syrk_reduce_kernel, dim3((unsigned)ntiles), dim3(256), 0, st, H, a.ws,
                         (int)K, T, a.RS);
      GPTQ_CHECK_LAUNCH();
    }
  }
  return GPTQ_HIP_OK;
}

int gptq_hip_hessian_finalize(void *stream, void *H, int h_dtype, int64_t K, double n_samples) {
  if (!H || K <= 0 || !(n_samples > 0)) return GPTQ_HIP_EINVAL;
  const int64_t T = ceil_div64(K, TS);
  const dim3 grid((unsigned)(T * (T + 1) / 2)), block(TS * 8);
  if (h_dtype == GPTQ_HIP_F32)
    hipLaunchKernelGGL(finalize_kernel<float>, grid, block, 0, as_stream(stream),
                       reinterpret_cast<float *>(H), K, (float)n_samples);
  else if (h_dtype == GPTQ_HIP_F64)
    hipLaunchKernelGGL(finalize_kernel<double>, grid, block, 0, as_stream(stream),
                       reinterpret_cast<double *>(H), K, n_samples);
  else
    return GPTQ_HIP_EDTYPE;
  GPTQ_CHECK_LAUNCH();
  return GPTQ_HIP_OK;
}

}  // extern "C"
