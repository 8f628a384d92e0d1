// Dead-feature fix, damping and the lower Cholesky factor L of the inverse Hessian,
// L L^T = H^-1, on one device.
//
// The reference obtains L in three LAPACK steps (factor, solve against I, factor again,
// about 8/3 K^3 flop).  Here L is obtained in two (about 2/3 K^3 flop):
//   1. H = M^T M with M lower triangular ("reverse" Cholesky, processed from the last
//      diagonal block upwards so that every trailing update is an X^T X form);
//   2. L = M^-1, by pairwise merging of inverted diagonal blocks:
//      inv([[A,0],[C,B]]) = [[A^-1,0],[-B^-1 C A^-1, B^-1]].
// H^-1 = M^-1 M^-T = L L^T with L lower triangular and a positive diagonal, which is the
// unique Cholesky factor the reference computes.
//
// All O(K^3) work runs on MFMAs; only the NB x NB diagonal blocks are factorised and
// inverted with vector instructions, by five wavefronts.  Everything is templated on the
// scalar type R: float is the default path, double the reference's use_fp64 option
// (gptq.py:182-197).  In fp32 a step of the factorisation (solve the block's panel, update
// what lies above and left of it, factorise the next diagonal block) is one launch
// (chol_step_kernel), or two where the panel is long; fp64 keeps three launches per step.
#include "common.h"
#include "gemm_f32.h"
#include "tile_io.h"

namespace {

constexpr int NB = 64;

// ---------------------------------------------------------------- diag / damping prep
// One workgroup.  dead_i = (H_ii == 0) -> H_ii = 1; mean over the fixed diagonal;
// H_ii += damping * mean.  Writes dead flags and status[1] = number of dead features.
template <typename R>
__global__ __launch_bounds__(1024) void damp_diag_kernel(R *H, int64_t K, R damping,
                                                         int fix_dead, uint8_t *dead,
                                                         int32_t *status) {
#pragma clang fp contract(off)
  __shared__ R ssum[1024];
  __shared__ int scnt[1024];
  const int tid = threadIdx.x;
  R sum = 0;
  int cnt = 0;
  for (int64_t i = tid; i < K; i += 1024) {
    R d = H[i * K + i];
    const bool is_dead = fix_dead && (d == R(0));
    if (is_dead) { d = 1; ++cnt; }
    dead[i] = is_dead ? 1 : 0;
    sum += d;
  }
  ssum[tid] = sum;
  scnt[tid] = cnt;
  __syncthreads();
  for (int s = 512; s > 0; s >>= 1) {
    if (tid < s) { ssum[tid] += ssum[tid + s]; scnt[tid] += scnt[tid + s]; }
    __syncthreads();
  }
  const R add = (ssum[0] / (R)K) * damping;
  for (int64_t i = tid; i < K; i += 1024) {
    R d = H[i * K + i];
    if (dead[i]) d = 1;
    H[i * K + i] = d + add;
  }
  if (tid == 0) { status[0] = 0; status[1] = scnt[0]; }
}

__global__ __launch_bounds__(256) void zero_dead_rows_kernel(float *W, int64_t N, int64_t ldw,
                                                             const uint8_t *dead) {
  const int64_t row = blockIdx.y;
  if (!dead[row]) return;
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < N; c += (int64_t)gridDim.x * 256)
    W[row * ldw + c] = 0.f;
}

// The same, with the flags taken from the diagonal of an untouched H (H_ii == 0)
template <typename R>
__global__ __launch_bounds__(256) void zero_rows_of_dead_features_kernel(const R *H, int64_t K, float *W,
                                                                         int64_t N, int64_t ldw) {
  const int64_t row = blockIdx.y;
  if (H[row * (K + 1)] != R(0)) return;
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < N; c += (int64_t)gridDim.x * 256)
    W[row * ldw + c] = 0.f;
}

// A (Kp x Kp, padded with the identity) <- H ; Minv <- 0
template <typename R>
__global__ __launch_bounds__(256) void pad_copy_kernel(const R *H, int64_t K, R *A, R *Minv,
                                                       int64_t Kp) {
  const int64_t row = blockIdx.y;
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < Kp; c += (int64_t)gridDim.x * 256) {
    R v;
    if (row < K && c < K) v = H[row * K + c];
    else v = (row == c) ? 1 : 0;
    A[row * Kp + c] = v;
    Minv[row * Kp + c] = 0;
  }
}

// L (K x K, ld K) <- lower(Minv[0:K, 0:K]), upper part zero; L32, if given, gets the fp32 cast
template <typename R>
__global__ __launch_bounds__(256) void copy_out_kernel(const R *Minv, int64_t Kp, R *L,
                                                       float *L32, int64_t K) {
  const int64_t row = blockIdx.y;
  for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < K; c += (int64_t)gridDim.x * 256) {
    const R v = (c <= row) ? Minv[row * Kp + c] : R(0);
    L[row * K + c] = v;
    if (L32) L32[row * K + c] = (float)v;
  }
}

// ---------------------------------------------------------------- NB x NB diagonal block
// D = A[b,b] (its lower triangle is read).  Finds M_bb lower with M_bb^T M_bb = D by a
// standard Cholesky of the index-reversed block: G G^T = J D J, M_bb = J G^T J.  Writes
// M_bb over A[b,b] (upper part zeroed) and M_bb^-1 = J G^-T J into Minv[b,b].
//
// Five wavefronts.  Four factorise: lane r of each keeps row r of G for 16 columns, dealt in panels of four
// adjacent columns (panel p belongs to wavefront p mod 4).  What bounds the kernel is the chain from one
// synchronisation to the next, so there is one per panel, not one per column: the owner of a panel factorises
// its four columns by itself (pivot by v_readlane, reciprocal square root, the later columns of the panel
// updated at once) and publishes them through LDS; after the barrier every factorising wavefront holds the four
// columns in four VGPRs, from which lane c's entries become scalar operands (v_readlane) of the updates of its
// column c: two instructions per column and pivot, in the order of the pivots.  The owner of the next panel
// updates that panel first and factorises and publishes it before it turns to its other columns.  The fifth
// wavefront follows one panel behind and computes four rows of X = G^-1 (lane j keeps column j of X) from the
// rows of G, which it reads from LDS with broadcast reads.  The block is on the critical path of the blocked
// factorisation (nothing else can run while it does), so latency is what counts here.  Entries above the
// diagonal of G hold garbage while the factorisation runs (masking them would cost a third instruction per
// element) and are written out as zeros.
static_assert(NB == 64, "the diagonal kernel maps one matrix row to one lane of a wavefront");
constexpr int GSTR = NB + 4;   // LDS row stride of G: rows stay 16-byte aligned

__device__ __forceinline__ float lane_bcast(float v, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
__device__ __forceinline__ double lane_bcast(double v, int lane) {
  const int2 w = __builtin_bit_cast(int2, v);
  int2 o;
  o.x = __builtin_amdgcn_readlane(w.x, lane);
  o.y = __builtin_amdgcn_readlane(w.y, lane);
  return __builtin_bit_cast(double, o);
}
// square root of a pivot and its reciprocal
__device__ __forceinline__ void root_and_inverse(float piv, float &root, float &rinv) {
  // hardware reciprocal square root (1 ulp) plus one Newton step instead of the long
  // correctly-rounded sqrt and division sequences: this sits on the per-step latency chain
  const float y = __builtin_amdgcn_rsqf(piv);
  rinv = y * fmaf(-0.5f * piv * y, y, 1.5f);
  root = piv * rinv;
}
__device__ __forceinline__ void root_and_inverse(double piv, double &root, double &rinv) {
  root = sqrt(piv);
  rinv = 1.0 / root;
}

constexpr int DIAG_FW = 4;                       // factorising wavefronts
constexpr int PW = 4;                            // columns per panel
constexpr int DIAG_THREADS = (DIAG_FW + 1) * 64;

// The block's work.  src (row stride lds): the block D, in global memory or (ALIAS) in the LDS array that Gs
// overwrites once every lane holds its part; Mout (may be null) / Dinv: where M_bb and its inverse go, row stride
// ld.  dinv [NB], Gs [NB * GSTR], Xs [NB * (NB + 1)], Lcol [2 * PW * NB]: LDS.  All five wavefronts call it.
template <typename R, bool ALIAS>
__device__ __forceinline__ void chol_diag_block(const R *src, int64_t lds, R *Mout, R *Dinv, int64_t ld, int b,
                                                int32_t *status, R *dinv, R *Gs, R *Xs, R *Lcol) {
  constexpr int XSTR = NB + 1;
  constexpr int CW = NB / DIAG_FW;                           // columns per factorising wavefront
  const int r = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  typedef R colvec __attribute__((ext_vector_type(CW)));    // vector values, never an alloca
  typedef R rowvec __attribute__((ext_vector_type(NB)));
  auto lcol = [&](int par, int q) __attribute__((always_inline)) -> R * { return Lcol + (par * PW + q) * NB; };

  if (wave < DIAG_FW) {
    // slot j of wavefront w holds column col_of(j) = 16 (j / 4) + 4 w + j % 4
    auto col_of = [&](int j) __attribute__((always_inline)) { return (PW * DIAG_FW) * (j / PW) + PW * wave + (j % PW); };
    // G[r][c] (c <= r) = D[63-c][63-r]: for fixed c the lanes read one row of D (coalesced)
    colvec g;
#pragma unroll
    for (int j = 0; j < CW; ++j) {
      const int c = col_of(j);
      g[j] = src[(int64_t)(NB - 1 - c) * lds + (NB - 1 - r)];   // c > r: finite garbage, never used
    }
    if (ALIAS) __syncthreads();               // every lane has its part of the block: Gs may overwrite it
    bool bad = false;
    // G[r][c] -= l[r] l[c] for the column in slot j; pinned to its place: left free, the compiler may defer
    // every update until the element is needed and keep the operands of all steps alive
    auto update = [&](int j, R l) __attribute__((always_inline)) {
      R t = g[j] - l * lane_bcast(l, col_of(j));
      asm volatile("" : "+v"(t));
      g[j] = t;
    };
    // factorises panel p (held by this wavefront in slots 4 (p / 4) ...) and publishes it
    auto factor_panel = [&](int p) __attribute__((always_inline)) {
      const int j0 = PW * (p / DIAG_FW);
#pragma unroll
      for (int q = 0; q < PW; ++q) {
        const int k = PW * p + q;
        const R piv = lane_bcast(g[j0 + q], k);
        bad = bad || !(piv > R(0));
        R root, rinv;
        root_and_inverse(piv, root, rinv);
        const R l = (r == k) ? root : g[j0 + q] * rinv;
        g[j0 + q] = l;
        lcol(p & 1, q)[r] = l;
        Gs[r * GSTR + k] = (k <= r) ? l : R(0);
        if (r == k) dinv[k] = rinv;
#pragma unroll
        for (int q2 = q + 1; q2 < PW; ++q2) update(j0 + q2, l);
      }
    };
    if (wave == 0) factor_panel(0);
#pragma unroll
    for (int p = 0; p < NB / PW; ++p) {
      __syncthreads();                        // panel p is in LDS
      R l[PW];
#pragma unroll
      for (int q = 0; q < PW; ++q) l[q] = lcol(p & 1, q)[r];
      auto apply = [&](int j) __attribute__((always_inline)) {
#pragma unroll
        for (int q = 0; q < PW; ++q) update(j, l[q]);
      };
      if (p + 1 < NB / PW) {
        // the next panel first, by its owner, which then factorises and publishes it
        const int nown = (p + 1) % DIAG_FW, jn0 = PW * ((p + 1) / DIAG_FW);
        if (wave == nown) {
#pragma unroll
          for (int q = 0; q < PW; ++q) apply(jn0 + q);
          factor_panel(p + 1);
        }
        // the other columns right of the panel
#pragma unroll
        for (int j = 0; j < CW; ++j) {
          const int jp = j / PW;                       // the slot's panel is 4 jp + wave
          const bool next = (jp == (p + 1) / DIAG_FW);  // ... the next panel, if this wavefront owns it
          if (jp > p / DIAG_FW) {
            if (!next || wave != nown) apply(j);
          } else if (jp == p / DIAG_FW) {
            if (wave > p % DIAG_FW && !(next && wave == nown)) apply(j);
          }
        }
      }
    }
    if (__any(bad) && r == 0) atomicMax(status, b + 1);
  } else {
    if (ALIAS) __syncthreads();
    // ---- X = G^-1, lane j computes column j: x[i] = (delta_ij - sum_{k<i} G[i][k] x[k]) / G[i][i]
    rowvec x;
#pragma unroll
    for (int p = 0; p < NB / PW; ++p) {
      __syncthreads();                       // rows 4 p .. 4 p + 3 of G are complete
#pragma unroll
      for (int q = 0; q < PW; ++q) {
        const int i = PW * p + q;
        R acc = (i == r) ? R(1) : R(0);
#pragma unroll
        for (int k = 0; k < i; ++k) acc -= Gs[i * GSTR + k] * x[k];
        R xi = acc * dinv[i];                // stays 0 for i < j: every term is 0
        asm volatile("" : "+v"(xi));         // keeps the row reads of later steps from being hoisted
        x[i] = xi;
      }
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) Xs[i * XSTR + r] = x[i];
  }
  __syncthreads();
  // M_bb[i][j] = G[63-j][63-i], Minv_bb[i][j] = X[63-j][63-i]  (i >= j), zero above; wavefronts 0-1
  // write M_bb (half of the rows each), 2-3 the inverse (all four the inverse where M_bb is not wanted)
  if (wave < 4) {
    if (Mout == nullptr) {
      for (int i = wave * (NB / 4); i < (wave + 1) * (NB / 4); ++i)
        Dinv[(int64_t)i * ld + r] = (i >= r) ? Xs[(NB - 1 - r) * XSTR + (NB - 1 - i)] : R(0);
    } else {
      const int half = wave & 1;
      if (wave < 2) {
        for (int i = half * (NB / 2); i < (half + 1) * (NB / 2); ++i)
          Mout[(int64_t)i * ld + r] = (i >= r) ? Gs[(NB - 1 - r) * GSTR + (NB - 1 - i)] : R(0);
      } else {
        for (int i = half * (NB / 2); i < (half + 1) * (NB / 2); ++i)
          Dinv[(int64_t)i * ld + r] = (i >= r) ? Xs[(NB - 1 - r) * XSTR + (NB - 1 - i)] : R(0);
      }
    }
  }
}

template <typename R>
__global__ __launch_bounds__(DIAG_THREADS) void chol_diag_kernel(R *A, R *Minv, int64_t ld, int b,
                                                                 int32_t *status) {
  __shared__ __attribute__((aligned(16))) R dinv[NB];        // 1 / G[k][k]
  __shared__ __attribute__((aligned(16))) R Gs[NB * GSTR];   // G, row major
  __shared__ __attribute__((aligned(16))) R Xs[NB * (NB + 1)];   // X = G^-1, row major
  __shared__ __attribute__((aligned(16))) R Lcol[2 * PW * NB];   // the columns of a panel of G, by panel parity
  R *D = A + (int64_t)b * NB * ld + (int64_t)b * NB;
  R *Dinv = Minv + (int64_t)b * NB * ld + (int64_t)b * NB;
  chol_diag_block<R, false>(D, ld, D, Dinv, ld, b, status, dinv, Gs, Xs, Lcol);
}

// ---------------------------------------------------------------- one launch per step of the factorisation (fp32)
// Block b is factorised and its inverse is in Minv[b, b].  What the chain of three launches did per step (solve the
// block's panel, update everything above and to the left of it, factorise block b - 1) is one launch here: a
// workgroup owns the 64 x 64 tile (i, j), j <= i < b, of the trailing matrix, and
//   * solves the panel pieces it needs itself, P_i = Minv_bb^T H[b, i], P_j = Minv_bb^T H[b, j] (each piece is
//     solved by every workgroup of its tile row and column: 2.1 Mflop, against a launch and its latency); the
//     unsolved panel stays where it is in A, the tiles on the diagonal write their piece to Minv[b, i], which is
//     where the merging step reads it;
//   * updates its tile, A[i, j] -= P_i^T P_j;
//   * the workgroup of tile (b - 1, b - 1), the first to be dispatched, keeps the updated tile in LDS and
//     factorises it on the spot (chol_diag_block).
// Every product is the MFMA sequence of gemm_f32_tn_k64_kernel on the same operands, so the factor is bit for
// bit the one of the three-launch chain.  52 KB of LDS: three workgroups per CU.
constexpr int STEP_LD = GSTR;
constexpr int STEP_MAT = NB * STEP_LD;
constexpr int STEP_LDS_BYTES = 3 * STEP_MAT * (int)sizeof(float);
static_assert(NB * (NB + 1) <= STEP_MAT && 2 * PW * NB + NB <= STEP_MAT, "the block's arrays fit the operand buffers");

// SOLVED: the panel has been solved by a launch of its own and lies in Minv[b, :]; the workgroups only update and
// factorise (late steps have up to 2016 tiles, whose redundant solves take longer than that launch).
template <bool SOLVED>
__global__ __launch_bounds__(DIAG_THREADS) void chol_step_kernel(float *A, float *Minv, int64_t ld, int b,
                                                                 int32_t *status) {
  extern __shared__ __attribute__((aligned(16))) float step_lds[];
  float *Dv = step_lds, *Hm = step_lds + STEP_MAT, *Hn = step_lds + 2 * STEP_MAT;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // tile (i, j), j <= i, the last one first
  const int t = b * (b + 1) / 2 - 1 - (int)blockIdx.x;
  int i = (int)((sqrtf(8.f * (float)t + 1.f) - 1.f) * 0.5f);
  while ((i + 1) * (i + 2) / 2 <= t) ++i;
  while (i * (i + 1) / 2 > t) --i;
  const int j = t - i * (i + 1) / 2;
  const bool on_diag = i == j;
  const bool factor = blockIdx.x == 0;            // tile (b - 1, b - 1)
  const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, lhi = lane >> 5;
  float *C = A + (int64_t)i * NB * ld + (int64_t)j * NB;
  float cv[16];
  if (wave < 4) {
    const float *Dsrc = Minv + (int64_t)b * NB * ld + (int64_t)b * NB;
    const float *Hrow = (SOLVED ? Minv : A) + (int64_t)b * NB * ld;
    const int r = tid >> 4, c4 = (tid & 15) * 4;
    float4 rd[4], rm[4], rn[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (!SOLVED) rd[q] = *reinterpret_cast<const float4 *>(Dsrc + (int64_t)(r + 16 * q) * ld + c4);
      rm[q] = *reinterpret_cast<const float4 *>(Hrow + (int64_t)(r + 16 * q) * ld + i * NB + c4);
      rn[q] = *reinterpret_cast<const float4 *>(Hrow + (int64_t)(r + 16 * q) * ld + j * NB + c4);
    }
#pragma unroll
    for (int q = 0; q < 16; ++q)
      cv[q] = C[(int64_t)(wm * 32 + 8 * (q >> 2) + 4 * lhi + (q & 3)) * ld + wn * 32 + l32];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (!SOLVED) *reinterpret_cast<float4 *>(&Dv[(r + 16 * q) * STEP_LD + c4]) = rd[q];
      *reinterpret_cast<float4 *>(&Hm[(r + 16 * q) * STEP_LD + c4]) = rm[q];
      *reinterpret_cast<float4 *>(&Hn[(r + 16 * q) * STEP_LD + c4]) = rn[q];
    }
  }
  __syncthreads();
  floatx16 pm, pn;
#pragma unroll
  for (int q = 0; q < 16; ++q) pm[q] = pn[q] = 0.f;
  if (!SOLVED && wave < 4) {
#pragma unroll 8
    for (int kk = 0; kk < NB; kk += 2) {
      const int krow = kk + lhi;
      const float a = Dv[krow * STEP_LD + wm * 32 + l32];
      pm = __builtin_amdgcn_mfma_f32_32x32x2f32(a, Hm[krow * STEP_LD + wn * 32 + l32], pm, 0, 0, 0);
      if (!on_diag) pn = __builtin_amdgcn_mfma_f32_32x32x2f32(a, Hn[krow * STEP_LD + wn * 32 + l32], pn, 0, 0, 0);
    }
  }
  if (!SOLVED) __syncthreads();                   // the unsolved pieces have been read
  if (!SOLVED && wave < 4) {
    float *Pout = Minv + (int64_t)b * NB * ld + (int64_t)i * NB;
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const int row = wm * 32 + 8 * (q >> 2) + 4 * lhi + (q & 3), col = wn * 32 + l32;
      Hm[row * STEP_LD + col] = pm[q];
      if (on_diag) Pout[(int64_t)row * ld + col] = pm[q];
      else Hn[row * STEP_LD + col] = pn[q];
    }
  }
  if (!SOLVED) __syncthreads();
  if (wave < 4) {
    const float *Pn = on_diag ? Hm : Hn;
    floatx16 acc;
#pragma unroll
    for (int q = 0; q < 16; ++q) acc[q] = 0.f;
#pragma unroll 8
    for (int kk = 0; kk < NB; kk += 2) {
      const int krow = kk + lhi;
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(Hm[krow * STEP_LD + wm * 32 + l32], Pn[krow * STEP_LD + wn * 32 + l32],
                                                 acc, 0, 0, 0);
    }
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const int row = wm * 32 + 8 * (q >> 2) + 4 * lhi + (q & 3), col = wn * 32 + l32;
      const float v = cv[q] - acc[q];
      if (factor) Dv[row * STEP_LD + col] = v;
      else C[(int64_t)row * ld + col] = v;
    }
  }
  if (!factor) return;
  __syncthreads();                                // the updated block is in Dv; the solved pieces have been read
  __builtin_amdgcn_s_setprio(3);
  float *Dinv = Minv + (int64_t)(b - 1) * NB * ld + (int64_t)(b - 1) * NB;
  chol_diag_block<float, true>(Dv, STEP_LD, nullptr, Dinv, ld, b - 1, status, Hn + 2 * PW * NB, Dv, Hm, Hn);
}

template <typename R>
struct Plan {
  int64_t K, Kp;
  R *A, *Minv, *T;
  uint8_t *dead;
  size_t bytes;
};

template <typename R>
Plan<R> make_plan(int64_t K, void *ws) {
  Plan<R> p;
  p.K = K;
  p.Kp = round_up64(K, NB);
  const size_t mat = (size_t)p.Kp * (size_t)p.Kp * sizeof(R);
  char *base = reinterpret_cast<char *>(ws);
  p.A = reinterpret_cast<R *>(base);
  p.Minv = reinterpret_cast<R *>(base + mat);
  p.T = reinterpret_cast<R *>(base + 2 * mat);
  p.dead = reinterpret_cast<uint8_t *>(base + 3 * mat);
  p.bytes = 3 * mat + (size_t)round_up64(K, 256);
  return p;
}

template <typename R>
int damp_invert(hipStream_t st, R *H, float *W, int64_t K, int64_t N, int64_t ldw, double damping,
                int fix_dead, R *L, float *L32, int32_t *status, void *ws) {
  const Plan<R> p = make_plan<R>(K, ws);
  const int64_t Kp = p.Kp;
  const int nblk = (int)(Kp / NB);
  constexpr int DT = sizeof(R) == 8 ? GPTQ_HIP_F64 : GPTQ_HIP_F32;

  hipLaunchKernelGGL(damp_diag_kernel<R>, dim3(1), dim3(1024), 0, st, H, K, (R)damping, fix_dead,
                     p.dead, status);
  GPTQ_CHECK_LAUNCH();
  if (N > 0) {
    unsigned gx = (unsigned)ceil_div64(N, 256);
    if (gx > 32) gx = 32;
    hipLaunchKernelGGL(zero_dead_rows_kernel, dim3(gx, (unsigned)K), dim3(256), 0, st, W, N, ldw,
                       p.dead);
    GPTQ_CHECK_LAUNCH();
  }
  {
    unsigned gx = (unsigned)ceil_div64(Kp, 256);
    if (gx > 32) gx = 32;
    hipLaunchKernelGGL(pad_copy_kernel<R>, dim3(gx, (unsigned)Kp), dim3(256), 0, st, H, K, p.A,
                       p.Minv, Kp);
    GPTQ_CHECK_LAUNCH();
  }

  // ---- step 1: H = M^T M, last block first.  Two blocking levels: inside an outer block of
  // OUTER diagonal blocks a finished panel updates only the rows of that outer block (a few
  // hundred rows, all columns to their left); everything above the outer block receives one
  // update with k = OUTER * NB when the outer block is complete.  A single level would read and
  // write the whole trailing matrix once per NB rows, which is what bounds it from K ~ 8192 on
  // (K = 28672: 352 ms with one level, 194 ms with two); below K = 6144 the trailing matrix stays
  // in the caches and one level (OUTER = 1) has fewer, larger launches.
  const int OUTER = Kp >= 6144 ? 8 : 1;
  // fp32: one launch per step, or two; the solved panels go to Minv, where the outer updates and the merging step
  // find them
  const bool fused = sizeof(R) == 4;
  auto solve_panel = [&](int b) -> int {
    // Minv[b, 0:b] <- Minv_bb^T A[b, 0:b]
    GemmArgs g;
    g.A = p.Minv + (int64_t)b * NB * Kp + (int64_t)b * NB;
    g.B = p.A + (int64_t)b * NB * Kp;
    g.C = p.Minv + (int64_t)b * NB * Kp;
    g.lda = g.ldb = g.ldc = Kp;
    g.m = NB;
    g.n = b * NB;
    g.k = NB;
    g.alpha = 1.f;
    g.beta = 0.f;
    g.a_kmajor = 1;
    g.in_dtype = DT;
    return gptq_gemm(st, g, (R *)nullptr);
  };
  if constexpr (sizeof(R) == 4) {
    if (fused && OUTER == 1) {
      if (!gptq_raise_lds_limit(reinterpret_cast<const void *>(chol_step_kernel<false>), STEP_LDS_BYTES) ||
          !gptq_raise_lds_limit(reinterpret_cast<const void *>(chol_step_kernel<true>), STEP_LDS_BYTES))
        return GPTQ_HIP_ELAUNCH;
      // from 32 blocks on (528 tiles) the panel is solved by a launch of its own (5 us): the tiles' redundant solves
      // would take longer
      constexpr int bsplit = 32;
      hipLaunchKernelGGL(chol_diag_kernel<R>, dim3(1), dim3(DIAG_THREADS), 0, st, p.A, p.Minv, Kp, nblk - 1, status);
      GPTQ_CHECK_LAUNCH();
      for (int b = nblk - 1; b > 0; --b) {
        const dim3 grid((unsigned)(b * (b + 1) / 2));
        if (b >= bsplit) {
          const int rc = solve_panel(b);
          if (rc) return rc;
          hipLaunchKernelGGL(chol_step_kernel<true>, grid, dim3(DIAG_THREADS), STEP_LDS_BYTES, st,
                             reinterpret_cast<float *>(p.A), reinterpret_cast<float *>(p.Minv), Kp, b, status);
        } else {
          hipLaunchKernelGGL(chol_step_kernel<false>, grid, dim3(DIAG_THREADS), STEP_LDS_BYTES, st,
                             reinterpret_cast<float *>(p.A), reinterpret_cast<float *>(p.Minv), Kp, b, status);
        }
        GPTQ_CHECK_LAUNCH();
      }
    } else if (fused) {
      // two levels: inside an outer block the workgroups update the tiles of its rows only (tiles (i, j), b0 <= i < b,
      // j <= i: the last b (b + 1) / 2 - b0 (b0 + 1) / 2 of the enumeration); the outer block's first diagonal block
      // stands alone, behind the update with k = OUTER * NB
      if (!gptq_raise_lds_limit(reinterpret_cast<const void *>(chol_step_kernel<true>), STEP_LDS_BYTES))
        return GPTQ_HIP_ELAUNCH;
      for (int b1 = nblk; b1 > 0;) {
        const int b0 = ((b1 - 1) / OUTER) * OUTER;
        hipLaunchKernelGGL(chol_diag_kernel<R>, dim3(1), dim3(DIAG_THREADS), 0, st, p.A, p.Minv, Kp, b1 - 1, status);
        GPTQ_CHECK_LAUNCH();
        for (int b = b1 - 1; b >= b0 && b > 0; --b) {
          int rc = solve_panel(b);
          if (rc) return rc;
          if (b == b0) break;
          const dim3 grid((unsigned)(b * (b + 1) / 2 - b0 * (b0 + 1) / 2));
          hipLaunchKernelGGL(chol_step_kernel<true>, grid, dim3(DIAG_THREADS), STEP_LDS_BYTES, st,
                             reinterpret_cast<float *>(p.A), reinterpret_cast<float *>(p.Minv), Kp, b, status);
          GPTQ_CHECK_LAUNCH();
        }
        if (b0 > 0) {
          // A[0:b0, 0:b0] -= P^T P, P = the outer block's solved rows, columns 0 .. b0*NB  (lower tiles)
          const R *outer = p.Minv + (int64_t)b0 * NB * Kp;
          GemmArgs s;
          s.A = outer;
          s.B = outer;
          s.C = p.A;
          s.lda = s.ldb = s.ldc = Kp;
          s.m = s.n = b0 * NB;
          s.k = (b1 - b0) * NB;
          s.alpha = -1.f;
          s.beta = 1.f;
          s.a_kmajor = 1;
          s.in_dtype = DT;
          s.tri = 2;
          const int rc = gptq_gemm(st, s, (R *)nullptr);
          if (rc) return rc;
        }
        b1 = b0;
      }
    }
  }
  for (int b1 = fused ? 0 : nblk; b1 > 0;) {
    const int b0 = ((b1 - 1) / OUTER) * OUTER;      // outer block = diagonal blocks [b0, b1)
    for (int b = b1 - 1; b >= b0; --b) {
      hipLaunchKernelGGL(chol_diag_kernel<R>, dim3(1), dim3(DIAG_THREADS), 0, st, p.A, p.Minv, Kp, b, status);
      GPTQ_CHECK_LAUNCH();
      if (b == 0) break;
      R *panel = p.A + (int64_t)b * NB * Kp;  // rows of block b, columns 0 .. b*NB
      // panel <- Minv_bb^T * panel   (in place: every workgroup reads only its own columns)
      GemmArgs g;
      g.A = p.Minv + (int64_t)b * NB * Kp + (int64_t)b * NB;
      g.B = panel;
      g.C = panel;
      g.lda = g.ldb = g.ldc = Kp;
      g.m = NB;
      g.n = b * NB;
      g.k = NB;
      g.alpha = 1.f;
      g.beta = 0.f;
      g.a_kmajor = 1;
      g.in_dtype = DT;
      int rc = gptq_gemm(st, g, (R *)nullptr);
      if (rc) return rc;
      if (b == b0) break;
      // A[b0:b, 0:b] -= panel[:, b0:b]^T panel[:, 0:b]   (the blocks right of the diagonal that
      // this touches are never read)
      GemmArgs s;
      s.A = panel + (int64_t)b0 * NB;
      s.B = panel;
      s.C = p.A + (int64_t)b0 * NB * Kp;
      s.lda = s.ldb = s.ldc = Kp;
      s.m = (b - b0) * NB;
      s.n = b * NB;
      s.k = NB;
      s.alpha = -1.f;
      s.beta = 1.f;
      s.a_kmajor = 1;
      s.in_dtype = DT;
      if (s.m == s.n) s.tri = 2;         // single level: a square, of which only the lower tiles are read
      rc = gptq_gemm(st, s, (R *)nullptr);
      if (rc) return rc;
    }
    if (b0 > 0) {
      // A[0:b0, 0:b0] -= P^T P, P = rows of the outer block, columns 0 .. b0*NB  (lower tiles)
      R *outer = p.A + (int64_t)b0 * NB * Kp;
      GemmArgs s;
      s.A = outer;
      s.B = outer;
      s.C = p.A;
      s.lda = s.ldb = s.ldc = Kp;
      s.m = s.n = b0 * NB;
      s.k = (b1 - b0) * NB;
      s.alpha = -1.f;
      s.beta = 1.f;
      s.a_kmajor = 1;
      s.in_dtype = DT;
      s.tri = 2;
      const int rc = gptq_gemm(st, s, (R *)nullptr);
      if (rc) return rc;
    }
    b1 = b0;
  }

  // ---- step 2: L = M^-1 by pairwise merging
  for (int64_t s = NB; s < Kp; s *= 2) {
    const int npairs = (int)ceil_div64(Kp, 2 * s);
    const int64_t pair_stride = 2 * s * (Kp + 1);
    // The complete pairs go in one batched launch without the ragged-size logic (which would
    // keep every tile on the guarded load path), the incomplete last pair, if any, in its own.
    const int nfull = (int)(Kp / (2 * s));
    auto merge_gemm = [&](const GemmArgs &a) -> int {
      if (nfull > 0) {
        GemmArgs f = a;
        f.batch = nfull;
        f.m_total = f.m_step = f.k_total = f.k_step = 0;
        const int rc = gptq_gemm(st, f, (R *)nullptr);
        if (rc) return rc;
      }
      if (nfull < npairs && Kp - s - (int64_t)nfull * 2 * s > 0) {
        GemmArgs r = a;
        r.batch = 1;
        r.A = reinterpret_cast<const R *>(a.A) + (int64_t)nfull * pair_stride;
        r.B = reinterpret_cast<const R *>(a.B) + (int64_t)nfull * pair_stride;
        r.C = reinterpret_cast<R *>(a.C) + (int64_t)nfull * pair_stride;
        r.m_total = a.m_total - nfull * a.m_step;
        if (a.k_step) r.k_total = a.k_total - nfull * a.k_step;
        return gptq_gemm(st, r, (R *)nullptr);
      }
      return GPTQ_HIP_OK;
    };
    // T = C * Ainv
    GemmArgs g;
    g.A = (fused ? p.Minv : p.A) + s * Kp;   // C of pair 0: rows [s, 2s), cols [0, s)
    g.B = p.Minv;                   // Ainv of pair 0
    g.C = p.T + s * Kp;
    g.lda = g.ldb = g.ldc = Kp;
    g.m = (int)s;
    g.n = (int)s;
    g.k = (int)s;
    g.alpha = 1.f;
    g.beta = 0.f;
    g.a_kmajor = 0;
    g.in_dtype = DT;
    g.kskip = 1;
    g.batch = npairs;
    g.strideA = g.strideB = g.strideC = pair_stride;
    g.m_total = (int)(Kp - s);
    g.m_step = (int)(2 * s);
    int rc = merge_gemm(g);
    if (rc) return rc;
    // Minv[B rows, A cols] = -Binv * T
    GemmArgs h;
    h.A = p.Minv + s * (Kp + 1);    // Binv of pair 0
    h.B = p.T + s * Kp;
    h.C = p.Minv + s * Kp;
    h.lda = h.ldb = h.ldc = Kp;
    h.m = (int)s;
    h.n = (int)s;
    h.k = (int)s;
    h.alpha = -1.f;
    h.beta = 0.f;
    h.a_kmajor = 0;
    h.in_dtype = DT;
    h.kskip = 2;
    h.batch = npairs;
    h.strideA = h.strideB = h.strideC = pair_stride;
    h.m_total = (int)(Kp - s);
    h.m_step = (int)(2 * s);
    h.k_total = (int)(Kp - s);
    h.k_step = (int)(2 * s);
    rc = merge_gemm(h);
    if (rc) return rc;
  }

  {
    unsigned gx = (unsigned)ceil_div64(K, 256);
    if (gx > 32) gx = 32;
    hipLaunchKernelGGL(copy_out_kernel<R>, dim3(gx, (unsigned)K), dim3(256), 0, st, p.Minv, Kp, L,
                       L32, K);
    GPTQ_CHECK_LAUNCH();
  }
  return GPTQ_HIP_OK;
}

}  // namespace

extern "C" {

int gptq_hip_zero_dead_rows(void *stream, const void *H, int h_dtype, int64_t K, float *W, int64_t N,
                            int64_t ldw) {
  if (K < 0 || N < 0 || ldw < N) return GPTQ_HIP_EINVAL;
  if (K == 0 || N == 0) return GPTQ_HIP_OK;
  if (!H || !W) return GPTQ_HIP_EINVAL;
  if (h_dtype != GPTQ_HIP_F32 && h_dtype != GPTQ_HIP_F64) return GPTQ_HIP_EDTYPE;
  if (K > 65535) return GPTQ_HIP_EINVAL;          // one grid row per feature, as in damp_invert
  hipStream_t st = as_stream(stream);
  unsigned gx = (unsigned)ceil_div64(N, 256);
  if (gx > 32) gx = 32;
  const dim3 grid(gx, (unsigned)K);
  if (h_dtype == GPTQ_HIP_F64)
    hipLaunchKernelGGL(zero_rows_of_dead_features_kernel<double>, grid, dim3(256), 0, st,
                       reinterpret_cast<const double *>(H), K, W, N, ldw);
  else
    hipLaunchKernelGGL(zero_rows_of_dead_features_kernel<float>, grid, dim3(256), 0, st,
                       reinterpret_cast<const float *>(H), K, W, N, ldw);
  GPTQ_CHECK_LAUNCH();
  return GPTQ_HIP_OK;
}

size_t gptq_hip_damp_invert_workspace_bytes(int64_t K, int h_dtype) {
  if (K <= 0) return 0;
  return h_dtype == GPTQ_HIP_F64 ? make_plan<double>(K, nullptr).bytes
                                 : make_plan<float>(K, nullptr).bytes;
}

int gptq_hip_damp_invert(void *stream, void *H, int h_dtype, float *W, int64_t K, int64_t N,
                         int64_t ldw, double damping, int fix_dead, void *L, float *L32,
                         int32_t *status, void *ws, size_t ws_bytes) {
  if (!H || !L || !status || K <= 0 || K > 65535 || N < 0 || (N > 0 && (!W || ldw < N)))
    return GPTQ_HIP_EINVAL;
  if (h_dtype != GPTQ_HIP_F32 && h_dtype != GPTQ_HIP_F64) return GPTQ_HIP_EDTYPE;
  if (!ws || ws_bytes < gptq_hip_damp_invert_workspace_bytes(K, h_dtype)) return GPTQ_HIP_EWORKSPACE;
  if ((reinterpret_cast<uintptr_t>(ws) & 15) != 0) return GPTQ_HIP_EINVAL;
  hipStream_t st = as_stream(stream);
  if (h_dtype == GPTQ_HIP_F64)
    return damp_invert<double>(st, reinterpret_cast<double *>(H), W, K, N, ldw, damping, fix_dead,
                               reinterpret_cast<double *>(L), L32, status, ws);
  return damp_invert<float>(st, reinterpret_cast<float *>(H), W, K, N, ldw, damping, fix_dead,
                            reinterpret_cast<float *>(L), L32, status, ws);
}

}  // extern "C"
