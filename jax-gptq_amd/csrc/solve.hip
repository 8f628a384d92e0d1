// Blocked GPTQ column loop: quantise block_size rows with error feedback, then push the
// accumulated error into the remaining rows with fp32 MFMAs: inside a 512-row group every
// block first receives what the group's earlier blocks owe it (in the prologue of its own kernel,
// or, for irregular shapes, in a product launch in front of it), and after every group everything
// below it receives the group's errors in one product.
//
// In-block kernel: the N output channels are independent, so one lane owns one channel and a
// workgroup of eight wavefronts owns 64 channels.  It works out of LDS: its channels of the
// block's rows, the block's corner of L, the refined reciprocals of L's diagonal.  The block is
// walked in sub-blocks of SB rows:
//   * the first wavefront evaluates the sub-block's sequential chain (row t needs the error of
//     row t - 1) with the sub-block's triangle of L and its rows in VGPRs;
//   * meanwhile the other wavefronts apply the previous sub-block's errors to the rows below
//     (rows dealt round-robin) and write that sub-block's results to memory;
//   * then all wavefronts put the new errors into the rows of the next sub-block.
// Each lane touches only its own column of the tile (no bank conflicts); L is read with
// broadcast reads (every lane the same address).  W itself is not written.
//
// Every floating-point result is that of the IEEE operation the reference writes (true
// division, round-half-even, separate multiply and subtract) and every element receives
// its updates in the reference's order, so given the same L and W the block result is
// bit-identical to a CPU evaluation of gptq.py:136-147.
#include "common.h"
#include "gemm_f32.h"
#include "tile_io.h"
#include <type_traits>
#include <utility>

namespace {

constexpr int SOLVE_CH = 64;               // channels per workgroup (one per lane)
constexpr int SOLVE_NW = 8;                // wavefronts per workgroup: one runs the chains, seven update and store
constexpr int SOLVE_TPB = SOLVE_CH * SOLVE_NW;
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <int I> using ic = std::integral_constant<int, I>;
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>) {
  (f(ic<I>{}), ...);
}
// f(ic<0>), f(ic<1>), ..., f(ic<N - 1>): a loop whose index is a constant expression in the body
template <int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

template <int SB, typename TQ>
__global__ __launch_bounds__(SOLVE_TPB) void block_quant_kernel(
    const float *Wb, int64_t N, const float *Lb, int64_t ldl, int bs, const float *scale,
    const float *zero, float maxq, TQ *Qb, uint8_t *cb, float *Err, const float *Lprev, const float *Eprev, int kprev) {
  // Wb, Qb, cb: first row of the block in W, Q, codes; Lb: the block's diagonal corner of L
  // kprev > 0 (bs = 128, whole 64-channel tiles, 16-byte aligned rows; kprev a multiple of 64): the block's rows
  // first receive what the kprev rows in front of them in their update group owe them,
  //   W[block] - Lprev[128, kprev] @ Eprev[kprev, N]   (Lprev = L[block rows, group start ..], Eprev: those rows' errors),
  // which a product launch of its own did before (14 - 24 us each, three per group of four blocks): here every
  // workgroup forms its 128 x 64 tile of it with fp32 MFMAs, k ascending in one accumulator and the difference
  // taken once, so the bits are those of that product.
#pragma clang fp contract(off)
  extern __shared__ __attribute__((aligned(16))) float smem[];
  float *Ln = smem;                         // Ln[j * bs + i] = Lb[j][i] for i <= j (nothing right of the diagonal is read)
  float *Wl = Ln + bs * bs;                 // Wl[j * SOLVE_CH + lane] = W[block row j][channel]
  float *Es = Wl + bs * SOLVE_CH;           // [2][SB][SOLVE_CH] errors of a sub-block (two sub-blocks alternate)
  float *Qs = Es + 2 * SB * SOLVE_CH;       // the same for the codes
  float *QHs = Qs + 2 * SB * SOLVE_CH;      // and for the dequantised values
  float *R1s = QHs + 2 * SB * SOLVE_CH;     // [bs] refined reciprocals of L's diagonal (NaN: outside the fast form's range)
  const int tid = threadIdx.x;
  const int lane = tid & (SOLVE_CH - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / SOLVE_CH);   // wave-uniform: scalar branches on it
  const int64_t n0 = (int64_t)blockIdx.x * SOLVE_CH;
  const int64_t n = n0 + lane;
  const bool live = n < N;
  const int64_t nl = live ? n : N - 1;   // lanes past the edge shadow the last channel, store nothing

  // ---- staging of rows [row_lo, row_hi) of L's corner and of the W tile by threads t = 0 .. nthr - 1.  Loads are
  //      unconditional (clamped) and go out in batches before the first wait; 16-byte loads where the shapes allow.
  const bool vec = (bs & 3) == 0 && (ldl & 3) == 0 && (reinterpret_cast<uintptr_t>(Lb) & 15) == 0 && (N & 3) == 0 &&
                   n0 + SOLVE_CH <= N && (reinterpret_cast<uintptr_t>(Wb) & 15) == 0;
  // d -> the reciprocal as the compiler's division sequence refines it; NaN where the fast form of the chain
  // may not be used for the row
  auto diag_recip = [](float d) __attribute__((always_inline)) -> float {
    const float r0c = __builtin_amdgcn_rcpf(d);
    const float e0 = __builtin_fmaf(-d, r0c, 1.0f);
    const float r1 = __builtin_fmaf(e0, r0c, r0c);
    return (fabsf(d) >= 0x1p-40f && fabsf(d) <= 0x1p40f) ? r1 : __builtin_nanf("");
  };
  auto stage = [&](int row_lo, int row_hi, int t, int nthr) __attribute__((always_inline)) {
    const int rows = row_hi - row_lo;
    if (t < 0 || rows <= 0) return;
    if (vec) {
      // the first batch of the W tile goes out before the loads of L and is stored after them
      // (kprev > 0: the tile is in LDS already)
      const int totalw = kprev > 0 ? 0 : rows * (SOLVE_CH / 4);
      f32x4 wv[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int idx = max(min(u * nthr + t, totalw - 1), 0);
        const int j = idx / (SOLVE_CH / 4), c4 = idx - j * (SOLVE_CH / 4);
        wv[u] = *reinterpret_cast<const f32x4 *>(Wb + (int64_t)(row_lo + j) * N + n0 + 4 * c4);
      }
      const int q4 = bs >> 2, total4 = rows * q4;
      if (nthr % q4 == 0) {
        // a thread keeps its group of four columns and walks down the rows (no division per load)
        const int j0 = t / q4, i4 = t - j0 * q4, jstep = nthr / q4;
        for (int jb = j0; jb < rows; jb += jstep * 8) {
          f32x4 v[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            // (right of the diagonal nothing is needed: those threads re-read the diagonal's group)
            const int j = min(jb + u * jstep, rows - 1);
            v[u] = *reinterpret_cast<const f32x4 *>(Lb + (int64_t)(row_lo + j) * ldl + 4 * min(i4, (row_lo + j) >> 2));
          }
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            const int row = row_lo + jb + u * jstep;
            if (row < row_hi && i4 <= (row >> 2)) {
              *reinterpret_cast<f32x4 *>(Ln + row * bs + 4 * i4) = v[u];
              if ((row >> 2) == i4) {
                const int r = row & 3;
                R1s[row] = diag_recip(r == 0 ? v[u][0] : (r == 1 ? v[u][1] : (r == 2 ? v[u][2] : v[u][3])));
              }
            }
          }
        }
      } else {
        for (int base = 0; base < total4; base += nthr * 8) {
          f32x4 v[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            const int idx = min(base + u * nthr + t, total4 - 1);
            const int j = idx / q4, i4 = idx - j * q4;
            v[u] = *reinterpret_cast<const f32x4 *>(Lb + (int64_t)(row_lo + j) * ldl + 4 * i4);
          }
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            const int idx = base + u * nthr + t;
            if (idx < total4) {
              *reinterpret_cast<f32x4 *>(Ln + row_lo * bs + 4 * idx) = v[u];
              const int j = idx / q4, i4 = idx - j * q4, row = row_lo + j;
              if ((row >> 2) == i4) {
                const int r = row & 3;
                R1s[row] = diag_recip(r == 0 ? v[u][0] : (r == 1 ? v[u][1] : (r == 2 ? v[u][2] : v[u][3])));
              }
            }
          }
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int idx = u * nthr + t;
        if (idx < totalw) *reinterpret_cast<f32x4 *>(Wl + row_lo * SOLVE_CH + 4 * idx) = wv[u];
      }
      for (int base = nthr * 4; base < totalw; base += nthr * 4) {
        f32x4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int idx = min(base + u * nthr + t, totalw - 1);
          const int j = idx / (SOLVE_CH / 4), c4 = idx - j * (SOLVE_CH / 4);
          v[u] = *reinterpret_cast<const f32x4 *>(Wb + (int64_t)(row_lo + j) * N + n0 + 4 * c4);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int idx = base + u * nthr + t;
          if (idx < totalw) *reinterpret_cast<f32x4 *>(Wl + row_lo * SOLVE_CH + 4 * idx) = v[u];
        }
      }
    } else {
      const int total = rows * bs;
      for (int base = 0; base < total; base += nthr * 16) {
        float v[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) {
          const int idx = min(base + u * nthr + t, total - 1);
          const int j = idx / bs, i = idx - j * bs;
          v[u] = Lb[(int64_t)(row_lo + j) * ldl + i];
        }
#pragma unroll
        for (int u = 0; u < 16; ++u) {
          const int idx = base + u * nthr + t;
          if (idx < total) {
            Ln[row_lo * bs + idx] = v[u];
            const int j = idx / bs, i = idx - j * bs;
            if (i == row_lo + j) R1s[i] = diag_recip(v[u]);
          }
        }
      }
      const int totalw = kprev > 0 ? 0 : rows * SOLVE_CH;
      for (int base = 0; base < totalw; base += nthr * 16) {
        float v[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) {
          const int idx = min(base + u * nthr + t, totalw - 1);
          const int j = idx / SOLVE_CH, c = idx - j * SOLVE_CH;
          const int64_t nc = n0 + c < N ? n0 + c : N - 1;
          v[u] = Wb[(int64_t)(row_lo + j) * N + nc];
        }
#pragma unroll
        for (int u = 0; u < 16; ++u) {
          const int idx = base + u * nthr + t;
          if (idx < totalw) Wl[row_lo * SOLVE_CH + idx] = v[u];
        }
      }
    }
  };
  // rows [row_lo, row_hi) of the tile receive the errors e of the sub-block whose first row (= first column
  // of L) is lcol; the rows are dealt round-robin to UW wavefronts, NB rows at a time (a row is a chain of SB
  // dependent subtractions)
  float *wcol = Wl + lane;
  auto update_rows = [&](int row_lo, int row_hi, const float (&e)[SB], int lcol, int widx, auto nbc, auto nwc)
                         __attribute__((always_inline)) {
    constexpr int NB = decltype(nbc)::value, UW = decltype(nwc)::value;
    for (int j = row_lo + widx; j < row_hi; j += UW * NB) {
      float x[NB], l[NB][SB];
#pragma unroll
      for (int v = 0; v < NB; ++v) {
        const int jj = min(j + UW * v, row_hi - 1);
        x[v] = wcol[jj * SOLVE_CH];
        const float *lr = Ln + jj * bs + lcol;
        if constexpr (SB % 4 == 0) {
#pragma unroll
          for (int c = 0; c < SB / 4; ++c) {
            const f32x4 q = *reinterpret_cast<const f32x4 *>(lr + 4 * c);
#pragma unroll
            for (int i = 0; i < 4; ++i) l[v][4 * c + i] = q[i];
          }
        } else {
#pragma unroll
          for (int u = 0; u < SB; ++u) l[v][u] = lr[u];
        }
      }
#pragma unroll
      for (int u = 0; u < SB; ++u) {
#pragma unroll
        for (int v = 0; v < NB; ++v) {
          const float upd = l[v][u] * e[u];
          x[v] = x[v] - upd;
        }
      }
#pragma unroll
      for (int v = 0; v < NB; ++v)
        if (j + UW * v < row_hi) wcol[(j + UW * v) * SOLVE_CH] = x[v];
    }
  };
  // results of sub-block sb (in its LDS buffers) to memory, rows dealt over NWV wavefronts
  auto store_sub = [&](int sb, int widx, auto nwc) __attribute__((always_inline)) {
    constexpr int NWV = decltype(nwc)::value;
    if (!live) return;
    const int off = (sb & 1) * SB * SOLVE_CH + lane;
#pragma unroll
    for (int t = 0; t < SB; ++t) {
      if ((t % NWV) == widx) {
        const int64_t o = (int64_t)(sb * SB + t) * N + n;
        if (Qb) Qb[o] = from_f32<TQ>(QHs[off + t * SOLVE_CH]);
        if (cb) cb[o] = (uint8_t)Qs[off + t * SOLVE_CH];
        Err[o] = Es[off + t * SOLVE_CH];
      }
    }
  };

  if (kprev > 0) {
    // ---- the tile W[block] - Lprev @ Eprev into Wl.  Wavefront w: rows 32 (w >> 1) .. + 31, channels 32 (w & 1) .. + 31
    // of the tile, as one 32 x 32 MFMA tile.  k in chunks of 64 through LDS (the regions of L's corner, of the tile
    // and of the sub-block buffers, all filled afterwards): Lprev's chunk [128][64] with row stride 65, Eprev's
    // [64][64] with row stride 68, two buffers, one barrier per chunk.
    constexpr int KC = 64, LDA = KC + 1, LDB = SOLVE_CH + 4, BUF = 128 * LDA + KC * LDB;
    constexpr int TPR = KC / 4, RPP = SOLVE_TPB / TPR, NPA = 128 / RPP;      // threads per row of Lprev's chunk, rows per pass, passes
    constexpr int NPB = KC / (SOLVE_TPB / 16);                              // passes over Eprev's chunk (16 threads per row)
    static_assert(2 * BUF * 4 <= (128 * 128 + 128 * SOLVE_CH + 6 * 16 * SOLVE_CH) * 4, "the chunk buffers fit in front of R1s");
    const int rblk = wave >> 1, cblk = wave & 1, l32 = lane & 31, lhi = lane >> 5;
    float cv[16];
#pragma unroll
    for (int q = 0; q < 16; ++q)
      cv[q] = Wb[(int64_t)(32 * rblk + 8 * (q >> 2) + 4 * lhi + (q & 3)) * N + n0 + 32 * cblk + l32];
    // this thread's pieces of a chunk: Lprev rows (tid / TPR) + RPP i, columns 4 (tid % TPR) .. + 3; Eprev rows
    // (tid >> 4) + 32 i, channels 4 (tid & 15) .. + 3
    const float *ap = Lprev + (int64_t)(tid / TPR) * ldl + 4 * (tid % TPR);
    const float *bp = Eprev + (int64_t)(tid >> 4) * N + n0 + 4 * (tid & 15);
    f32x4 ra[NPA], rb[NPB];
    auto load_chunk = [&](int k0) __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < NPA; ++i) ra[i] = *reinterpret_cast<const f32x4 *>(ap + (int64_t)(RPP * i) * ldl + k0);
#pragma unroll
      for (int i = 0; i < NPB; ++i) rb[i] = *reinterpret_cast<const f32x4 *>(bp + (int64_t)(k0 + 32 * i) * N);
    };
    auto store_chunk = [&](float *buf) __attribute__((always_inline)) {
      float *as = buf + (tid / TPR) * LDA + 4 * (tid % TPR);
#pragma unroll
      for (int i = 0; i < NPA; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) as[RPP * i * LDA + e] = ra[i][e];
#pragma unroll
      for (int i = 0; i < NPB; ++i)
        *reinterpret_cast<f32x4 *>(buf + 128 * LDA + ((tid >> 4) + 32 * i) * LDB + 4 * (tid & 15)) = rb[i];
    };
    floatx16 acc;
#pragma unroll
    for (int q = 0; q < 16; ++q) acc[q] = 0.f;
    load_chunk(0);
    store_chunk(smem);
    __syncthreads();
    int b = 0;
    for (int k0 = 0; k0 < kprev; k0 += KC) {
      const bool more = k0 + KC < kprev;
      if (more) load_chunk(k0 + KC);
      const float *as = smem + b * BUF + (32 * rblk + l32) * LDA + lhi;
      const float *bs_ = smem + b * BUF + 128 * LDA + lhi * LDB + 32 * cblk + l32;
#pragma unroll
      for (int kk = 0; kk < KC; kk += 2) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(as[kk], bs_[kk * LDB], acc, 0, 0, 0);
      if (more) store_chunk(smem + (b ^ 1) * BUF);
      __syncthreads();
      b ^= 1;
    }
#pragma unroll
    for (int q = 0; q < 16; ++q)
      Wl[(32 * rblk + 8 * (q >> 2) + 4 * lhi + (q & 3)) * SOLVE_CH + 32 * cblk + l32] = cv[q] - acc[q];
    // (the loop's last barrier: every wavefront is done with the chunk buffers, which the staging below overwrites;
    //  the tile itself is read after the barrier that follows the staging)
  }
  stage(0, SB, tid, SOLVE_TPB);
  const float sc = scale[nl], z = zero[nl];
  const float rs = 1.0f / sc;
  // the clamp of the code, moved to the integer before the zero point is added: exact for an integral zero point
  const float klo = -z, khi = maxq - z;
  const bool z_plain = !(z == rintf(z) && fabsf(z) <= 0x1p22f);
  __syncthreads();

  // ---- The chain of a sub-block (first wavefront): row t needs the error of row t - 1, and one wavefront issues
  // an instruction every five to six cycles, so what counts is the number of instructions.  The fast form has
  // 12 dependent ones per row (the two IEEE divisions of the plain form alone have 20):
  //  * rint(x / sc) is taken from x * (1 / sc).  The product lies within 2^-22 |x / sc| of the rounded
  //    quotient, so both round to the same integer unless the product is that close to a half-integer;
  //  * the code is clamped as an integer before the zero point is added (see klo, khi);
  //  * (x - qh) / d is the sequence the compiler emits for a division (reciprocal refined once, quotient
  //    refined twice with exact remainders), with the part that depends only on d taken out of the chain.
  //    The emitted form first rescales operands whose exponents are extreme (v_div_scale) and patches
  //    special values afterwards (v_div_fixup); with 2^-40 <= |a|, |d| <= 2^40 neither does anything, and
  //    the results are the same bit for bit.
  // A lane that leaves these ranges anywhere in the sub-block (or meets a NaN, which reaches the last error)
  // makes the wavefront evaluate the sub-block again with the plain divisions.
  // What does not depend on the errors is out of the chain: the refined reciprocals of L's diagonal are computed
  // by the threads that stage it, and the sub-block's triangle of L is read into registers between two chains.  The chain is
  // right-looking (an error goes into all later rows of the sub-block as soon as it exists; every element still
  // receives its updates in the order u = 0, 1, ...), and the source fixes the instruction order: between two
  // dependent instructions of row t stand the updates that the error of row t - 1 owes to rows t + 1 ..., and
  // that row's bookkeeping.
  constexpr int TRI = SB * (SB + 1) / 2;
  float lt[TRI], r1[SB];
  auto prologue = [&](int r0) __attribute__((always_inline)) {
    const float *ld = Ln + r0 * bs + r0;  // diagonal sub-block
    if constexpr (SB % 4 == 0) {
#pragma unroll
      for (int t = 0; t < SB; ++t)
#pragma unroll
        for (int c = 0; c <= t / 4; ++c) {
          const f32x4 v = *reinterpret_cast<const f32x4 *>(ld + t * bs + 4 * c);
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (4 * c + i <= t) lt[t * (t + 1) / 2 + 4 * c + i] = v[i];
        }
    } else {
#pragma unroll
      for (int t = 0; t < SB; ++t)
#pragma unroll
        for (int u = 0; u <= t; ++u) lt[t * (t + 1) / 2 + u] = ld[t * bs + u];
    }
#pragma unroll
    for (int t = 0; t < SB; ++t) r1[t] = R1s[r0 + t];
  };
  auto chain_fast = [&](int r0, int boff) __attribute__((always_inline)) -> bool {
    float xs[SB], e[SB], tmp[SB];
    float qa_s[SB], k_s[SB], kc_s[SB], qh_s[SB], a_s[SB];
    int ex_s[SB];
    float fmax_acc = 0.f, qmax_acc = 0.f, amax_acc = 1.0f;
    int emin_acc = 0;                  // smallest binary exponent of the non-zero a (frexp's: a = m 2^e, 0.5 <= m < 1)
#pragma unroll
    for (int t = 0; t < SB; ++t) xs[t] = wcol[(r0 + t) * SOLVE_CH];
    // the i-th instruction that the error of row te owes to the rows te + 2, ... (multiply, then subtract)
    auto upd_op = [&](int te, int i) __attribute__((always_inline)) {
      const int t2 = te + 2 + (i >> 1);
      if ((i & 1) == 0) tmp[i >> 1] = lt[t2 * (t2 + 1) / 2 + te] * e[te];
      else xs[t2] = xs[t2] - tmp[i >> 1];
    };
    constexpr int NBK = 8;
    auto bk_op = [&](int te, int j) __attribute__((always_inline)) {
      if (j == 0) fmax_acc = fmaxf(fmax_acc, fabsf(qa_s[te] - k_s[te]));
      if (j == 1) qmax_acc = fmaxf(qmax_acc, fabsf(qa_s[te]));
      // (an exact zero has exponent 0 here: it needs none of what the plain division adds, the fast form gives
      // the same zero; rows of dead features and weights that sit on the grid produce them)
      if (j == 2) ex_s[te] = __builtin_amdgcn_frexp_expf(a_s[te]);
      if (j == 3) emin_acc = min(emin_acc, ex_s[te]);
      if (j == 4) amax_acc = fmaxf(amax_acc, fabsf(a_s[te]));
      if (j == 5) Es[boff + te * SOLVE_CH] = e[te];
      if (j == 6) Qs[boff + te * SOLVE_CH] = kc_s[te] + z;
      if (j == 7) QHs[boff + te * SOLVE_CH] = qh_s[te];
    };
    static_for<SB>([&](auto tc) __attribute__((always_inline)) {
      constexpr int t = decltype(tc)::value;
      constexpr int te = t - 1;
      constexpr int P = t >= 1 ? 2 * (SB - 1 - t) : 0;
      constexpr int B = t >= 1 ? NBK : 0;
      constexpr int G = 12;
      constexpr int per = (P + B + G - 1) / G;
      // gap g of the row: the next `per` owed instructions, then a fence for the scheduler
      auto fill = [&](auto gc) __attribute__((always_inline)) {
        static_for<per>([&](auto cc) __attribute__((always_inline)) {
          constexpr int done = decltype(gc)::value * per + decltype(cc)::value;
          if constexpr (done < P) upd_op(te, done);
          else if constexpr (done < P + B) bk_op(te, done - P);
        });
        __builtin_amdgcn_sched_barrier(0);
      };
      const float d = lt[t * (t + 1) / 2 + t];
      float x = xs[t];
      if constexpr (t >= 1) {
        const float upd = lt[t * (t + 1) / 2 + te] * e[te];
        fill(ic<0>{});
        x = x - upd;
        fill(ic<1>{});
      }
      const float qa = x * rs;
      fill(ic<2>{});
      const float k = rintf(qa);
      fill(ic<3>{});
      const float kc = __builtin_amdgcn_fmed3f(k, klo, khi);
      fill(ic<4>{});
      const float qh = sc * kc;
      fill(ic<5>{});
      const float a = x - qh;
      fill(ic<6>{});
      const float q0 = a * r1[t];
      fill(ic<7>{});
      const float rem0 = __builtin_fmaf(-d, q0, a);
      fill(ic<8>{});
      const float q1 = __builtin_fmaf(rem0, r1[t], q0);
      fill(ic<9>{});
      const float rem1 = __builtin_fmaf(-d, q1, a);
      fill(ic<10>{});
      e[t] = __builtin_fmaf(rem1, r1[t], q1);
      fill(ic<11>{});
      qa_s[t] = qa;
      k_s[t] = k;
      kc_s[t] = kc;
      qh_s[t] = qh;
      a_s[t] = a;
    });
#pragma unroll
    for (int j = 0; j < NBK; ++j) bk_op(SB - 1, j);
    bool redo = z_plain;
    redo |= !(fmax_acc <= 0.5f - 0x1p-21f * fmaxf(qmax_acc, 1.0f));
    redo |= !(emin_acc >= -39 && amax_acc <= 0x1p40f);
    redo |= !(e[SB - 1] == e[SB - 1]);
    return redo;
  };
  // the plain form (gptq.py:136-147 as written)
  auto chain_plain = [&](int r0, int boff) __attribute__((always_inline)) {
    const float *ld = Ln + r0 * bs + r0;
    float e[SB];
#pragma unroll
    for (int t = 0; t < SB; ++t) {
      float x = wcol[(r0 + t) * SOLVE_CH];
#pragma unroll
      for (int u = 0; u < t; ++u) {
        const float upd = ld[t * bs + u] * e[u];
        x = x - upd;
      }
      float q = rintf(x / sc) + z;
      q = fminf(fmaxf(q, 0.f), maxq);
      const float qh = sc * (q - z);
      e[t] = (x - qh) / ld[t * bs + t];
      Es[boff + t * SOLVE_CH] = e[t];
      Qs[boff + t * SOLVE_CH] = q;
      QHs[boff + t * SOLVE_CH] = qh;
    }
  };

  // The block is walked in sub-blocks of SB rows.  The first wavefront evaluates the sub-block's chain;
  // meanwhile the others bring the rows below the sub-block up to date with the errors of the previous
  // sub-block and write that sub-block's results out (first sub-block: they stage the rest of the tile).  Then
  // all put the new errors into the rows of the next sub-block, and the first wavefront reads that sub-block's
  // triangle.  Two barriers per sub-block.
  // (The first wavefront runs a loop of its own, with the same barriers: the triangle's 150 registers are then
  // live in that loop only.)
  const int nsb = bs / SB;
  constexpr int NBA = (SB + SOLVE_NW - 1) / SOLVE_NW;      // rows per wavefront between two chains
  if (wave == 0) {
    prologue(0);
    for (int s = 0; s < nsb; ++s) {
      const int r0 = s * SB;
      const int boff = (s & 1) * SB * SOLVE_CH + lane;
      if (__builtin_amdgcn_ballot_w64(chain_fast(r0, boff)) != 0ull) chain_plain(r0, boff);
      __syncthreads();
      if (s + 1 < nsb) {
        float e[SB];
#pragma unroll
        for (int t = 0; t < SB; ++t) e[t] = Es[boff + t * SOLVE_CH];
        update_rows(r0 + SB, r0 + 2 * SB, e, r0, 0, ic<NBA>{}, ic<SOLVE_NW>{});
        prologue(r0 + SB);
        __syncthreads();
      }
    }
  } else {
    for (int s = 0; s < nsb; ++s) {
      const int r0 = s * SB;
      const int boff = (s & 1) * SB * SOLVE_CH + lane;
      if (s == 0) {
        stage(SB, bs, tid - SOLVE_CH, SOLVE_TPB - SOLVE_CH);
      } else {
        float e[SB];
        const int poff = ((s - 1) & 1) * SB * SOLVE_CH + lane;
#pragma unroll
        for (int t = 0; t < SB; ++t) e[t] = Es[poff + t * SOLVE_CH];
        update_rows(r0 + SB, bs, e, r0 - SB, wave - 1, ic<4>{}, ic<SOLVE_NW - 1>{});
        store_sub(s - 1, wave - 1, std::integral_constant<int, SOLVE_NW - 1>{});
      }
      __syncthreads();
      if (s + 1 < nsb) {
        float e[SB];
#pragma unroll
        for (int t = 0; t < SB; ++t) e[t] = Es[boff + t * SOLVE_CH];
        update_rows(r0 + SB, r0 + 2 * SB, e, r0, wave, ic<NBA>{}, ic<SOLVE_NW>{});
        __syncthreads();
      }
    }
  }
  store_sub(nsb - 1, wave, std::integral_constant<int, SOLVE_NW>{});
}

// Lprev / Eprev / kprev: see the kernel (kprev = 0: none)
bool fused_update_ok(const float *W, int64_t N, const float *L, int64_t ldl, int bs, int64_t kprev) {
  return bs == 128 && kprev > 0 && kprev % 64 == 0 && N % SOLVE_CH == 0 && (ldl & 3) == 0 &&
         (reinterpret_cast<uintptr_t>(L) & 15) == 0 && (reinterpret_cast<uintptr_t>(W) & 15) == 0;
}

template <int SB>
int launch_block(hipStream_t st, const float *W, int64_t N, const float *L, int64_t ldl, int bs,
                 const float *scale, const float *zero, float maxq, void *Q, int q_dtype,
                 uint8_t *codes, float *Err, const float *Lprev = nullptr, const float *Eprev = nullptr, int kprev = 0) {
  const dim3 grid((unsigned)ceil_div64(N, SOLVE_CH)), block(SOLVE_TPB);
  const size_t lds = ((size_t)bs * bs + (size_t)bs * SOLVE_CH + (size_t)6 * SB * SOLVE_CH + (size_t)bs) * sizeof(float);
  if (lds > 64 * 1024) {
    // up to 120 KB of the 160 KB LDS of a CU; the limit has to be raised per kernel
    const void *fn = q_dtype == GPTQ_HIP_F32
                         ? reinterpret_cast<const void *>(block_quant_kernel<SB, float>)
                         : (q_dtype == GPTQ_HIP_F16
                                ? reinterpret_cast<const void *>(block_quant_kernel<SB, __half>)
                                : reinterpret_cast<const void *>(block_quant_kernel<SB, __hip_bfloat16>));
    if (!gptq_raise_lds_limit(fn, (int)lds)) return GPTQ_HIP_ELAUNCH;
  }
  switch (q_dtype) {
    case GPTQ_HIP_F32:
      hipLaunchKernelGGL((block_quant_kernel<SB, float>), grid, block, lds, st, W, N, L, ldl,
                         bs, scale, zero, maxq, (float *)Q, codes, Err, Lprev, Eprev, kprev);
      break;
    case GPTQ_HIP_F16:
      hipLaunchKernelGGL((block_quant_kernel<SB, __half>), grid, block, lds, st, W, N, L, ldl,
                         bs, scale, zero, maxq, (__half *)Q, codes, Err, Lprev, Eprev, kprev);
      break;
    case GPTQ_HIP_BF16:
      hipLaunchKernelGGL((block_quant_kernel<SB, __hip_bfloat16>), grid, block, lds, st, W, N, L,
                         ldl, bs, scale, zero, maxq, (__hip_bfloat16 *)Q, codes, Err, Lprev, Eprev, kprev);
      break;
    default:
      return GPTQ_HIP_EDTYPE;
  }
  GPTQ_CHECK_LAUNCH();
  return GPTQ_HIP_OK;
}

bool block_size_ok(int bs) { return bs >= 1 && bs <= 128; }

// Rows whose error rows are kept together for one trailing update (a whole number of blocks).
// The rows below a group receive the updates of all its blocks in one product with k up to
// 512 instead of one product per block: every product reads and writes the rows it updates,
// so this cuts the traffic over the trailing part of W by the number of blocks in a group.
constexpr int GROUP_ROWS = 512;
int group_rows(int bs) { return (GROUP_ROWS / bs > 0 ? GROUP_ROWS / bs : 1) * bs; }

// C[m, n] -= A[m, k] @ B[k, n]
int trailing_update(hipStream_t st, const float *A, int64_t lda, const float *B, float *C,
                    int64_t N, int64_t m, int64_t k) {
  GemmArgs g;
  g.A = A;
  g.B = B;
  g.C = C;
  g.lda = lda;
  g.ldb = N;
  g.ldc = N;
  g.m = (int)m;
  g.n = (int)N;
  g.k = (int)k;
  g.alpha = -1.f;
  g.beta = 1.f;
  g.a_kmajor = 0;
  return gptq_gemm_f32(st, g);
}

int process_block(hipStream_t st, const float *Wb, int64_t N, const float *Lb, int64_t ldl, int bs,
                  const float *scale, const float *zero, int maxq, void *Qb, int q_dtype,
                  uint8_t *cb, float *Err, const float *Lprev = nullptr, const float *Eprev = nullptr, int kprev = 0) {
#define GPTQ_SB_CASE(SB) \
  return launch_block<SB>(st, Wb, N, Lb, ldl, bs, scale, zero, (float)maxq, Qb, q_dtype, cb, Err, Lprev, Eprev, kprev)
  if (bs % 16 == 0) GPTQ_SB_CASE(16);
  if (bs % 8 == 0) GPTQ_SB_CASE(8);
  if (bs % 4 == 0) GPTQ_SB_CASE(4);
  if (bs % 2 == 0) GPTQ_SB_CASE(2);
  GPTQ_SB_CASE(1);
#undef GPTQ_SB_CASE
}

}  // namespace

extern "C" {

size_t gptq_hip_solve_workspace_bytes(int64_t K, int64_t N, int block_size) {
  if (K <= 0 || N <= 0 || !block_size_ok(block_size)) return 0;
  return (size_t)group_rows(block_size) * (size_t)N * sizeof(float);
}

int gptq_hip_process_block(void *stream, const float *Wblock, int64_t N, const float *Lblock,
                           int64_t ldl, int block_size, const float *scale, const float *zero,
                           int maxq, void *Qblock, int q_dtype, uint8_t *codes_block,
                           float *errors) {
  if (!Wblock || !Lblock || !scale || !zero || !errors || N <= 0 || ldl < block_size)
    return GPTQ_HIP_EINVAL;
  if (!block_size_ok(block_size) || maxq < 1 || maxq > 255) return GPTQ_HIP_EINVAL;
  return process_block(as_stream(stream), Wblock, N, Lblock, ldl, block_size, scale, zero, maxq,
                       Qblock, q_dtype, codes_block, errors);
}

int gptq_hip_lazy_update(void *stream, float *Wbelow, int64_t N, const float *Lpanel, int64_t ldl, const float *errors,
                         int64_t rows, int64_t k) {
  if (rows < 0 || k < 0 || N <= 0 || rows > 2147483647LL || k > 2147483647LL || N > 2147483647LL)
    return GPTQ_HIP_EINVAL;
  if (rows == 0 || k == 0) return GPTQ_HIP_OK;
  if (!Wbelow || !Lpanel || !errors || ldl < k) return GPTQ_HIP_EINVAL;
  return trailing_update(as_stream(stream), Lpanel, ldl, errors, Wbelow, N, rows, k);
}

}  // extern "C"

namespace {

// The column loop.  group_size = 0: one scale / zero per channel for the whole column (the reference).
// group_size > 0: the parameters of rows [r0, r0 + group_size) are taken, when the loop reaches r0, from the
// column minima and maxima of those rows as they then stand (all corrections of the rows above applied), and
// written to row r0 / group_size of scale_g / zero_g [K / group_size, N].
int solve_impl(hipStream_t st, float *W, int64_t K, int64_t N, const float *L, const float *scale, const float *zero,
               float *scale_g, float *zero_g, int group_size, int bits, int maxq, int block_size, void *Q,
               int q_dtype, uint8_t *codes, float *Err, void *cp_ws, size_t cp_ws_bytes) {
  const size_t qsz = dtype_size(q_dtype);
  const int64_t grp = group_rows(block_size);
  for (int64_t gs = 0; gs < K; gs += grp) {
    const int64_t ge = gs + grp < K ? gs + grp : K;
    for (int64_t start = gs; start < ge; start += block_size) {
      const float *sc = scale, *zr = zero;
      if (group_size > 0) {
        const int64_t gi = start / group_size;
        if (start % group_size == 0) {
          // the group's rows lie inside the current update group (group_size divides its height), so they are current
          const int rc = gptq_hip_col_params(st, W + start * N, GPTQ_HIP_F32, group_size, N, N, bits,
                                             scale_g + gi * N, zero_g + gi * N, cp_ws, cp_ws_bytes);
          if (rc) return rc;
        }
        sc = scale_g + gi * N;
        zr = zero_g + gi * N;
      }
      // the block's rows receive what the earlier blocks of this update group owe them, in one product
      // with k = start - gs (per-channel parameters: nothing reads the rows below the block before their
      // own turn, so each row of the group is read and written once per group, not once per block above it):
      // inside the block's own kernel where the shapes allow, else in a launch of its own
      const bool fuse = group_size == 0 && start > gs && fused_update_ok(W + start * N, N, L, K, block_size, start - gs);
      if (group_size == 0 && start > gs && !fuse) {
        const int rc = trailing_update(st, L + start * K + gs, K, Err, W + start * N, N, block_size, start - gs);
        if (rc) return rc;
      }
      void *Qb = Q ? (void *)((char *)Q + (size_t)start * N * qsz) : nullptr;
      uint8_t *cb = codes ? codes + start * N : nullptr;
      float *Eb = Err + (start - gs) * N;
      int rc = process_block(st, W + start * N, N, L + start * K + start, K, block_size, sc, zr, maxq, Qb,
                             q_dtype, cb, Eb, fuse ? L + start * K + gs : nullptr, fuse ? Err : nullptr,
                             fuse ? (int)(start - gs) : 0);
      if (rc) return rc;
      const int64_t end = start + block_size;
      if (group_size > 0 && end < ge) {
        // grouped parameters are taken from rows that must be current when their group begins, so here every
        // block updates all rows of the update group below it: W[end:ge] -= L[end:ge, start:end] @ Err_block
        rc = trailing_update(st, L + end * K + start, K, Eb, W + end * N, N, ge - end, block_size);
        if (rc) return rc;
      }
    }
    if (ge < K) {
      // everything below the group: W[ge:] -= L[ge:, gs:ge] @ Err_group  (gptq.py:204-205, summed
      // over the blocks of the group)
      const int rc = trailing_update(st, L + ge * K + gs, K, Err, W + ge * N, N, K - ge, ge - gs);
      if (rc) return rc;
    }
  }
  return GPTQ_HIP_OK;
}

}  // namespace

extern "C" {

int gptq_hip_solve(void *stream, float *W, int64_t K, int64_t N, const float *L,
                   const float *scale, const float *zero, int maxq, int block_size, void *Q,
                   int q_dtype, uint8_t *codes, void *ws, size_t ws_bytes) {
  if (!W || !L || !scale || !zero || K <= 0 || N <= 0 || K > 2147483647LL || N > 2147483647LL)
    return GPTQ_HIP_EINVAL;
  if (!block_size_ok(block_size) || K % block_size != 0 || maxq < 1 || maxq > 255)
    return GPTQ_HIP_EINVAL;
  if (q_dtype != GPTQ_HIP_F32 && q_dtype != GPTQ_HIP_F16 && q_dtype != GPTQ_HIP_BF16)
    return GPTQ_HIP_EDTYPE;
  if (!ws || ws_bytes < gptq_hip_solve_workspace_bytes(K, N, block_size)) return GPTQ_HIP_EWORKSPACE;
  return solve_impl(as_stream(stream), W, K, N, L, scale, zero, nullptr, nullptr, 0, 0, maxq, block_size, Q, q_dtype,
                    codes, reinterpret_cast<float *>(ws), nullptr, 0);
}

size_t gptq_hip_solve_grouped_workspace_bytes(int64_t K, int64_t N, int block_size, int group_size) {
  if (K <= 0 || N <= 0 || !block_size_ok(block_size) || group_size <= 0) return 0;
  const size_t a = (gptq_hip_solve_workspace_bytes(K, N, block_size) + 255) & ~(size_t)255;
  return a + gptq_hip_col_params_workspace_bytes(group_size, N);
}

int gptq_hip_solve_grouped(void *stream, float *W, int64_t K, int64_t N, const float *L, int group_size, int bits,
                           int block_size, void *Q, int q_dtype, uint8_t *codes, float *scale_g, float *zero_g,
                           void *ws, size_t ws_bytes) {
  if (!W || !L || !scale_g || !zero_g || K <= 0 || N <= 0 || K > 2147483647LL || N > 2147483647LL)
    return GPTQ_HIP_EINVAL;
  if (!block_size_ok(block_size) || K % block_size != 0 || bits < 1 || bits > 8) return GPTQ_HIP_EINVAL;
  // a group is a whole number of blocks, lies inside one update group of the loop, and groups tile K
  if (group_size <= 0 || group_size % block_size != 0 || group_rows(block_size) % group_size != 0 ||
      K % group_size != 0)
    return GPTQ_HIP_EINVAL;
  if (q_dtype != GPTQ_HIP_F32 && q_dtype != GPTQ_HIP_F16 && q_dtype != GPTQ_HIP_BF16)
    return GPTQ_HIP_EDTYPE;
  if (!ws || ws_bytes < gptq_hip_solve_grouped_workspace_bytes(K, N, block_size, group_size)) return GPTQ_HIP_EWORKSPACE;
  const size_t a = (gptq_hip_solve_workspace_bytes(K, N, block_size) + 255) & ~(size_t)255;
  return solve_impl(as_stream(stream), W, K, N, L, nullptr, nullptr, scale_g, zero_g, group_size, bits, (1 << bits) - 1,
                    block_size, Q, q_dtype, codes, reinterpret_cast<float *>(ws), reinterpret_cast<char *>(ws) + a,
                    ws_bytes - a);
}

}  // extern "C"
