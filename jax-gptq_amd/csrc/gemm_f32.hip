// fp32 MFMA GEMM for gfx950: C = alpha * op(A) * B + beta * C.
//
// One workgroup (4 wavefronts of 64) owns a 128x128 tile of C; each wavefront owns a
// 64x64 quadrant as 2x2 tiles of v_mfma_f32_32x32x2_f32 (64 accumulator VGPRs).  A and B
// are staged through LDS in slabs of 16 along k, double buffered: the global loads of
// slab s+1 are issued before the MFMAs of slab s and written to the other LDS buffer
// afterwards, so one barrier per slab is enough.
//
// LDS layouts are chosen for the MFMA operand fetch (lane l supplies element
// [l % 32][l / 32] of a 32x2 operand):
//   k-major operands ([k][idx], row stride 160 floats): the two half-waves read two
//     consecutive k rows, 32 consecutive floats each, 32 banks apart;
//   idx-major A ([m][k], row stride 17 floats): consecutive lanes are 17 banks apart.
#include "gemm_f32.h"
#include "tile_io.h"

namespace {

constexpr int BM = 128, BN = 128, BK = 16, NTHREADS = 256;
constexpr int LDT = 160;   // k-major LDS row stride (floats)
constexpr int LDI = 17;    // idx-major LDS row stride (floats)
constexpr int TILE_FLOATS = BK * LDT;  // 2560 >= BM * LDI (2176)

// FAST: every tile is full and every 4-element group aligned (checked on the host), so the
// loads carry no guards: a load inside a branch makes the compiler wait for it at the join,
// in front of the MFMAs it is meant to overlap with.
template <typename T, bool AK, bool FAST>
__global__ __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(4, 4))) void gemm_f32_kernel(GemmArgs p) {
  __shared__ __attribute__((aligned(16))) float As[2][TILE_FLOATS];
  __shared__ __attribute__((aligned(16))) float Bs[2][TILE_FLOATS];

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
  float *C = reinterpret_cast<float *>(p.C) + (int64_t)z * p.strideC;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, lhi = lane >> 5;

  const bool a_al = (p.lda % 4 == 0) && ((reinterpret_cast<uintptr_t>(A) % (4 * sizeof(T))) == 0);
  const bool b_al = (p.ldb % 4 == 0) && ((reinterpret_cast<uintptr_t>(B) % (4 * sizeof(T))) == 0);
  const bool m_full = (m0 + BM <= m_eff);
  const bool n_full = (n0 + BN <= p.n);

  float ra[2][4], rb[2][4];

  auto load_tiles = [&](int kt) {
    const bool k_full = (kt + BK <= ke);
    if (AK) {
      const int r = tid >> 5, c4 = (tid & 31) * 4;
      const bool fast = FAST || (a_al && m_full && k_full);
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int kk = kt + r + 8 * i;
        int nv = (kk < ke) ? min(4, m_eff - (m0 + c4)) : 0;
        const T *src = A + (int64_t)kk * p.lda + m0 + c4;
        load_row4<T>(src, fast, nv, ra[i]);
      }
    } else {
      const int row = tid >> 2, k4 = (tid & 3) * 4;
      const bool fast = FAST || (a_al && m_full && k_full);
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int mm = m0 + row + 64 * i;
        int nv = (mm < m_eff) ? min(4, ke - (kt + k4)) : 0;
        const T *src = A + (int64_t)mm * p.lda + kt + k4;
        load_row4<T>(src, fast, nv, ra[i]);
      }
    }
    {
      const int r = tid >> 5, c4 = (tid & 31) * 4;
      const bool fast = FAST || (b_al && n_full && k_full);
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int kk = kt + r + 8 * i;
        int nv = (kk < ke) ? min(4, p.n - (n0 + c4)) : 0;
        const T *src = B + (int64_t)kk * p.ldb + n0 + c4;
        load_row4<T>(src, fast, nv, rb[i]);
      }
    }
  };

  auto store_tiles = [&](int buf) {
    if (AK) {
      const int r = tid >> 5, c4 = (tid & 31) * 4;
#pragma unroll
      for (int i = 0; i < 2; ++i)
        *reinterpret_cast<float4 *>(&As[buf][(r + 8 * i) * LDT + c4]) =
            make_float4(ra[i][0], ra[i][1], ra[i][2], ra[i][3]);
    } else {
      const int row = tid >> 2, k4 = (tid & 3) * 4;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) As[buf][(row + 64 * i) * LDI + k4 + e] = ra[i][e];
    }
    {
      const int r = tid >> 5, c4 = (tid & 31) * 4;
#pragma unroll
      for (int i = 0; i < 2; ++i)
        *reinterpret_cast<float4 *>(&Bs[buf][(r + 8 * i) * LDT + c4]) =
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

  int buf = 0;
  if (kb < ke) {
    load_tiles(kb);
    store_tiles(0);
  }
  __syncthreads();
  for (int kt = kb; kt < ke; kt += BK) {
    const bool more = (kt + BK < ke);
    if (more) load_tiles(kt + BK);
    const float *as = As[buf];
    const float *bs = Bs[buf];
#pragma unroll
    for (int kk = 0; kk < BK; kk += 2) {
      const int krow = kk + lhi;
      float a[2], b[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        a[t] = AK ? as[krow * LDT + wm * 64 + t * 32 + l32]
                  : as[(wm * 64 + t * 32 + l32) * LDI + krow];
        b[t] = bs[krow * LDT + wn * 64 + t * 32 + l32];
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    if (more) store_tiles(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }

  const float alpha = p.alpha, beta = p.beta;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = n0 + wn * 64 + j * 32 + l32;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3);
        if (row < m_eff && col < p.n) {
          float *dst = C + (int64_t)row * p.ldc + col;
          float v = alpha * acc[i][j][r];
          if (beta != 0.f) v += beta * (*dst);
          *dst = v;
        }
      }
    }
}

// ---------------------------------------------------------------------------- k = 64, A stored [k][m]
// The panel products and trailing updates of the blocked factorisation have k = 64: with the
// pipeline above (16 rows per stage, one stage ahead) such a launch is four exposed memory
// latencies long, whatever its size.  Here a workgroup issues all the loads of its two
// 64 x 128 operand tiles at once (16 loads of 16 bytes per thread), stores them to LDS, and
// multiplies: one latency, one barrier.  fp32 operands, rows 16-byte aligned, m and n
// multiples of 4; tiles at the edge load clamped (valid) columns and do not store them.
// In-place use (C == B with m <= 128, or C == A / B tiles that only this workgroup reads) is
// safe because every load of a tile completes before its first store.
constexpr int K64 = 64;
constexpr int k64_lds_bytes(int tb) { return 2 * K64 * (tb + 4) * 4; }

// TB = 128: the tile of the kernel above; TB = 64 (32 x 32 per wavefront, a quarter of the MFMA
// chain) for launches with few tiles, where the length of one workgroup is what counts.
template <int TB>
__global__ __launch_bounds__(NTHREADS) void gemm_f32_tn_k64_kernel(GemmArgs p) {
  constexpr int LD = TB + 4;                    // LDS row stride (floats): rows stay 16-byte aligned
  constexpr int TPR = TB / 4;                   // threads per operand row
  constexpr int RPP = NTHREADS / TPR;           // rows per pass
  constexpr int NP = K64 / RPP;                 // passes (float4 loads per thread and operand)
  constexpr int WT = TB / 2;                    // wavefront tile edge
  constexpr int NT = WT / 32;                   // 32 x 32 MFMA tiles per wavefront and dimension
  extern __shared__ __attribute__((aligned(16))) float k64_lds[];
  float *As = k64_lds, *Bs = k64_lds + K64 * LD;
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
  const int m0 = tm * TB, n0 = tn * TB;
  if (m0 >= p.m || n0 >= p.n) return;
  const float *A = reinterpret_cast<const float *>(p.A);
  const float *B = reinterpret_cast<const float *>(p.B);
  float *C = reinterpret_cast<float *>(p.C);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, lhi = lane >> 5;

  // thread -> rows r, r + RPP, ... of both operands, columns c4 .. c4 + 3 of the tile
  const int r = tid / TPR, c4 = (tid % TPR) * 4;
  const int ca = min(m0 + c4, p.m - 4), cb = min(n0 + c4, p.n - 4);
  float4 ra[NP], rb[NP];
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    ra[i] = *reinterpret_cast<const float4 *>(A + (int64_t)(r + RPP * i) * p.lda + ca);
    rb[i] = *reinterpret_cast<const float4 *>(B + (int64_t)(r + RPP * i) * p.ldb + cb);
  }
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    *reinterpret_cast<float4 *>(&As[(r + RPP * i) * LD + c4]) = ra[i];
    *reinterpret_cast<float4 *>(&Bs[(r + RPP * i) * LD + c4]) = rb[i];
  }
  __syncthreads();

  floatx16 acc[NT][NT];
#pragma unroll
  for (int i = 0; i < NT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;
#pragma unroll 8
  for (int kk = 0; kk < K64; kk += 2) {
    const int krow = kk + lhi;
    float a[NT], b[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      a[t] = As[krow * LD + wm * WT + t * 32 + l32];
      b[t] = Bs[krow * LD + wn * WT + t * 32 + l32];
    }
#pragma unroll
    for (int i = 0; i < NT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
  }

  const float alpha = p.alpha, beta = p.beta;
#pragma unroll
  for (int i = 0; i < NT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int col = n0 + wn * WT + j * 32 + l32;
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        const int row = m0 + wm * WT + i * 32 + 8 * (q >> 2) + 4 * lhi + (q & 3);
        if (row < p.m && col < p.n) {
          float *dst = C + (int64_t)row * p.ldc + col;
          float v = alpha * acc[i][j][q];
          if (beta != 0.f) v += beta * (*dst);
          *dst = v;
        }
      }
    }
}

// ---------------------------------------------------------------------------- k <= 128, A stored [m][k]
// The same idea for the products of the column loop inside a 512-row group,
// W[end:ge] -= L[end:ge, start:end] @ Err with k = block size <= 128: 64 x 64 tiles, all loads of
// both operand tiles in flight at once.  A is kept [row][k] in LDS with an odd stride (129), which
// makes the MFMA operand reads (32 consecutive rows at one k) conflict free.  fp32, k = 128, 64 or
// 32, n a multiple of 4, rows 16-byte aligned.
constexpr int WK_LDB = 64 + 4;
constexpr int wk_lds_bytes(int k) { return (64 * (k + 1) + k * WK_LDB) * 4; }

template <int KK>   // k, a power of two from 32 to 128: every count below is a compile-time constant
__global__ __launch_bounds__(NTHREADS) void gemm_f32_nn_wk_kernel(GemmArgs p) {
  constexpr int LDA = KK + 1;
  constexpr int KQ = KK / 4;                   // float4 per row of A
  constexpr int NP = 64 * KQ / NTHREADS;       // float4 per thread and operand (A: 64 x KK, B: KK x 64)
  extern __shared__ __attribute__((aligned(16))) float wk_lds[];
  float *As = wk_lds, *Bs = wk_lds + 64 * LDA;
  const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  const float *A = reinterpret_cast<const float *>(p.A);
  const float *B = reinterpret_cast<const float *>(p.B);
  float *C = reinterpret_cast<float *>(p.C);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, lhi = lane >> 5;

  float4 ra[NP], rb[NP];
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const int ia = tid + NTHREADS * i;
    const int row = min(m0 + ia / KQ, p.m - 1);
    ra[i] = *reinterpret_cast<const float4 *>(A + (int64_t)row * p.lda + (ia % KQ) * 4);
    const int col = min(n0 + (ia & 15) * 4, p.n - 4);
    rb[i] = *reinterpret_cast<const float4 *>(B + (int64_t)(ia >> 4) * p.ldb + col);
  }
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const int ia = tid + NTHREADS * i;
    float *dst = &As[(ia / KQ) * LDA + (ia % KQ) * 4];
    dst[0] = ra[i].x;
    dst[1] = ra[i].y;
    dst[2] = ra[i].z;
    dst[3] = ra[i].w;
    *reinterpret_cast<float4 *>(&Bs[(ia >> 4) * WK_LDB + (ia & 15) * 4]) = rb[i];
  }
  __syncthreads();

  floatx16 acc;
#pragma unroll
  for (int q = 0; q < 16; ++q) acc[q] = 0.f;
  const float *as = As + (wm * 32 + l32) * LDA + lhi;
  const float *bs = Bs + lhi * WK_LDB + wn * 32 + l32;
#pragma unroll 16
  for (int kk = 0; kk < KK; kk += 2)
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(as[kk], bs[kk * WK_LDB], acc, 0, 0, 0);

  const float alpha = p.alpha, beta = p.beta;
  const int col = n0 + wn * 32 + l32;
#pragma unroll
  for (int q = 0; q < 16; ++q) {
    const int row = m0 + wm * 32 + 8 * (q >> 2) + 4 * lhi + (q & 3);
    if (row < p.m && col < p.n) {
      float *dst = C + (int64_t)row * p.ldc + col;
      float v = alpha * acc[q];
      if (beta != 0.f) v += beta * (*dst);
      *dst = v;
    }
  }
}

template <int KK>
int launch_nn_wk(hipStream_t stream, const GemmArgs &a) {
  const dim3 g64((unsigned)((a.n + 63) / 64), (unsigned)((a.m + 63) / 64), 1);
  if (g64.y > 65535u) return GPTQ_HIP_EINVAL;
  if (wk_lds_bytes(KK) > 48 * 1024 &&
      !gptq_raise_lds_limit(reinterpret_cast<const void *>(gemm_f32_nn_wk_kernel<KK>), wk_lds_bytes(KK)))
    return GPTQ_HIP_ELAUNCH;
  hipLaunchKernelGGL(gemm_f32_nn_wk_kernel<KK>, g64, dim3(NTHREADS), wk_lds_bytes(KK), stream, a);
  GPTQ_CHECK_LAUNCH();
  return GPTQ_HIP_OK;
}

// ---------------------------------------------------------------------------- long k, few tiles, A stored [m][k]
// The triangular-inverse merges are products with k up to K/2 on a handful of tiles (K = 4096:
// 256 tiles of 128 x 128 at every level): one workgroup per CU walks a long k loop, and with a
// single slab of prefetch every slab pays most of a memory latency (50 TFLOP/s at best).  This
// kernel trades operand reuse for parallelism and depth: 64 x 64 tiles (four times the
// workgroups), and a register ring that keeps three slabs of 16 in flight per thread (one
// 16-byte load per operand and slab).  Guard-free: m, n multiples of 64, k of 16, rows 16-byte
// aligned; structural zeros (kskip) and batching as in the general kernel.
constexpr int N64_LDA = 17;
constexpr int N64_LDB = 64 + 4;

__global__ __launch_bounds__(NTHREADS) void gemm_f32_nn64_kernel(GemmArgs p) {
  __shared__ __attribute__((aligned(16))) float As[2][64 * N64_LDA];
  __shared__ __attribute__((aligned(16))) float Bs[2][BK * N64_LDB];
  const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64, z = blockIdx.z;
  int kb = 0, ke = p.k;
  if (p.kskip & 1) kb = min(n0, ke) & ~(BK - 1);
  if (p.kskip & 2) ke = min(ke, m0 + 64);
  const float *A = reinterpret_cast<const float *>(p.A) + (int64_t)z * p.strideA;
  const float *B = reinterpret_cast<const float *>(p.B) + (int64_t)z * p.strideB;
  float *C = reinterpret_cast<float *>(p.C) + (int64_t)z * p.strideC;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, lhi = lane >> 5;
  const int a_row = tid >> 2, a_k = (tid & 3) * 4;       // A: 64 rows x 16 k per slab
  const int b_row = tid >> 4, b_c = (tid & 15) * 4;      // B: 16 k x 64 columns per slab
  const float *a_src = A + (int64_t)(m0 + a_row) * p.lda + a_k;
  const float *b_src = B + (int64_t)b_row * p.ldb + n0 + b_c;
  const int k_last = max(ke - BK, 0);                    // clamp for the loads past the end (never used)

  struct Slab { float4 a, b; };
  auto load_slab = [&](int kt, Slab &sl) __attribute__((always_inline)) {
    const int kc = min(kt, k_last);
    sl.a = *reinterpret_cast<const float4 *>(a_src + kc);
    sl.b = *reinterpret_cast<const float4 *>(b_src + (int64_t)kc * p.ldb);
  };
  auto store_slab = [&](int buf, const Slab &sl) __attribute__((always_inline)) {
    float *da = &As[buf][a_row * N64_LDA + a_k];
    da[0] = sl.a.x;
    da[1] = sl.a.y;
    da[2] = sl.a.z;
    da[3] = sl.a.w;
    *reinterpret_cast<float4 *>(&Bs[buf][b_row * N64_LDB + b_c]) = sl.b;
  };
  floatx16 acc;
#pragma unroll
  for (int q = 0; q < 16; ++q) acc[q] = 0.f;

  const int nst = (ke - kb + BK - 1) / BK;
  if (nst > 0) {
    Slab s0, s1, s2, s3;
    load_slab(kb, s0);
    load_slab(kb + BK, s1);
    load_slab(kb + 2 * BK, s2);
    load_slab(kb + 3 * BK, s3);
    int buf = 0;
    store_slab(0, s0);
    __syncthreads();
    auto step = [&](int kt, Slab &refill, const Slab &next, bool do_load, bool has_next)
                    __attribute__((always_inline)) {
      if (do_load) load_slab(kt + 4 * BK, refill);
      const float *as = &As[buf][(wm * 32 + l32) * N64_LDA + lhi];
      const float *bs = &Bs[buf][lhi * N64_LDB + wn * 32 + l32];
#pragma unroll
      for (int kk = 0; kk < BK; kk += 2)
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(as[kk], bs[kk * N64_LDB], acc, 0, 0, 0);
      if (has_next) store_slab(buf ^ 1, next);
      __syncthreads();
      buf ^= 1;
    };
    // full groups of four without exits (the ring stays in flight across the loop head), then a
    // tail that issues no loads
    int si = 0, kt = kb;
    for (; si + 4 < nst; si += 4, kt += 4 * BK) {
      step(kt, s0, s1, true, true);
      step(kt + BK, s1, s2, true, true);
      step(kt + 2 * BK, s2, s3, true, true);
      step(kt + 3 * BK, s3, s0, true, true);
    }
    for (; si < nst; ++si, kt += BK) {      // at most four slabs, all of them loaded
      step(kt, s0, s1, false, si + 1 < nst);
      s1 = s2;
      s2 = s3;
    }
  }

  const float alpha = p.alpha, beta = p.beta;
  const int col = n0 + wn * 32 + l32;
#pragma unroll
  for (int q = 0; q < 16; ++q) {
    const int row = m0 + wm * 32 + 8 * (q >> 2) + 4 * lhi + (q & 3);
    float *dst = C + (int64_t)row * p.ldc + col;
    float v = alpha * acc[q];
    if (beta != 0.f) v += beta * (*dst);
    *dst = v;
  }
}

}  // namespace

int gptq_gemm_f32(hipStream_t stream, const GemmArgs &a) {
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
  const dim3 block(NTHREADS);
  if (a.k == K64 && a.a_kmajor && a.in_dtype == GPTQ_HIP_F32 && a.kskip == 0 && a.batch == 1 &&
      a.m_step == 0 && a.k_step == 0 && a.m >= 4 && a.n >= 4 && a.m % 4 == 0 && a.n % 4 == 0 &&
      a.lda % 4 == 0 && a.ldb % 4 == 0 && reinterpret_cast<uintptr_t>(a.A) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(a.B) % 16 == 0) {
    // 64 x 64 tiles up to 512 tiles of 128 x 128 (measured: faster up to there, equal beyond), and
    // when m is a single 64-row block
    const int64_t t128 = a.tri ? (int64_t)(tm > tn ? tm : tn) * ((tm > tn ? tm : tn) + 1) / 2 : (int64_t)tm * tn;
    const bool small = a.m <= 64 || t128 < 512;
    if (small) {
      const int sm = (a.m + 63) / 64, sn = (a.n + 63) / 64;
      dim3 g64;
      if (a.tri) {
        const int t = sm > sn ? sm : sn;
        g64 = dim3((unsigned)((int64_t)t * (t + 1) / 2), 1, 1);
      } else {
        g64 = dim3((unsigned)sn, (unsigned)sm, 1);
      }
      if (g64.y > 65535u) return GPTQ_HIP_EINVAL;
      hipLaunchKernelGGL(gemm_f32_tn_k64_kernel<64>, g64, block, k64_lds_bytes(64), stream, a);
    } else {
      if (!gptq_raise_lds_limit(reinterpret_cast<const void *>(gemm_f32_tn_k64_kernel<128>), k64_lds_bytes(128)))
        return GPTQ_HIP_ELAUNCH;
      hipLaunchKernelGGL(gemm_f32_tn_k64_kernel<128>, grid, block, k64_lds_bytes(128), stream, a);
    }
    GPTQ_CHECK_LAUNCH();
    return GPTQ_HIP_OK;
  }
  if (!a.a_kmajor && a.in_dtype == GPTQ_HIP_F32 && (a.k == 128 || a.k == 64 || a.k == 32) &&
      a.kskip == 0 && a.tri == 0 && a.batch == 1 && a.m_step == 0 && a.k_step == 0 && a.n >= 4 &&
      a.n % 4 == 0 && a.lda % 4 == 0 && a.ldb % 4 == 0 && reinterpret_cast<uintptr_t>(a.A) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(a.B) % 16 == 0) {
    if (a.k == 128) return launch_nn_wk<128>(stream, a);
    if (a.k == 64) return launch_nn_wk<64>(stream, a);
    return launch_nn_wk<32>(stream, a);
  }
  // up to 4096 tiles of 128 x 128 (measured: faster up to ~2600, slower from ~11000): 64 x 64 tiles
  // with a deep register ring
  if (!a.a_kmajor && a.in_dtype == GPTQ_HIP_F32 && a.tri == 0 && a.m_step == 0 && a.k_step == 0 &&
      a.m % 64 == 0 && a.n % 64 == 0 && a.k % BK == 0 && a.k >= 4 * BK &&
      (int64_t)tm * tn * a.batch <= 4096 && a.lda % 4 == 0 && a.ldb % 4 == 0 &&
      reinterpret_cast<uintptr_t>(a.A) % 16 == 0 && reinterpret_cast<uintptr_t>(a.B) % 16 == 0 &&
      (a.batch == 1 || (a.strideA % 4 == 0 && a.strideB % 4 == 0))) {
    const dim3 g64((unsigned)(a.n / 64), (unsigned)(a.m / 64), (unsigned)a.batch);
    if (g64.y > 65535u || g64.z > 65535u) return GPTQ_HIP_EINVAL;
    hipLaunchKernelGGL(gemm_f32_nn64_kernel, g64, block, 0, stream, a);
    GPTQ_CHECK_LAUNCH();
    return GPTQ_HIP_OK;
  }
  const size_t es = a.in_dtype == GPTQ_HIP_F32 ? 4 : 2;
  const bool fast = a.m % BM == 0 && a.n % BN == 0 && a.k % BK == 0 && a.m_step == 0 &&
                    a.k_step == 0 && a.lda % 4 == 0 && a.ldb % 4 == 0 &&
                    reinterpret_cast<uintptr_t>(a.A) % (4 * es) == 0 &&
                    reinterpret_cast<uintptr_t>(a.B) % (4 * es) == 0 &&
                    (a.batch == 1 || (a.strideA % 4 == 0 && a.strideB % 4 == 0));
#define GPTQ_GEMM_LAUNCH(T, AK)                                                              \
  do {                                                                                      \
    if (fast) hipLaunchKernelGGL((gemm_f32_kernel<T, AK, true>), grid, block, 0, stream, a); \
    else hipLaunchKernelGGL((gemm_f32_kernel<T, AK, false>), grid, block, 0, stream, a);     \
  } while (0)
  if (a.in_dtype == GPTQ_HIP_F32) {
    if (a.a_kmajor) GPTQ_GEMM_LAUNCH(float, true);
    else GPTQ_GEMM_LAUNCH(float, false);
  } else if (a.in_dtype == GPTQ_HIP_F16 && a.a_kmajor) {
    GPTQ_GEMM_LAUNCH(__half, true);
  } else if (a.in_dtype == GPTQ_HIP_BF16 && a.a_kmajor) {
    GPTQ_GEMM_LAUNCH(__hip_bfloat16, true);
  } else {
    return GPTQ_HIP_EDTYPE;
  }
#undef GPTQ_GEMM_LAUNCH
  GPTQ_CHECK_LAUNCH();
  return GPTQ_HIP_OK;
}
