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
  static constexpr bool DUAL = false;
  const void *ptr[H_NBMAX];
  int rows[H_NBMAX];
  int nb;
  int K;
  int T;       // tiles per side
  int RS;      // row slices
  int chunk;   // 16-bit kernel: rows of the concatenated batches per slice (multiple of 64)
  float *H;
  float *ws;   // [RS][tiles][128][128] when RS > 1
};

// Two-matrix form of the 16-bit kernel: sum_b A_b^T B_b for batch pairs whose sum is symmetric
// (operand A of a tile comes from ptr[b], operand B from ptrB[b]).
struct SyrkArgsDual : SyrkArgs {
  static constexpr bool DUAL = true;
  const void *ptrB[H_NBMAX];
  const float *factor;   // device scalar: the sums are in units of 1 / factor
  int accum;             // partial tiles: add to what the workspace holds instead of overwriting
};

// upper-triangular pair number t -> (i <= j), column by column
__device__ __forceinline__ void tri_decode(int t, int &i, int &j) {
  int c = (int)((sqrtf(8.f * (float)t + 1.f) - 1.f) * 0.5f);
  while ((c + 1) * (c + 2) / 2 <= t) ++c;
  while (c * (c + 1) / 2 > t) --c;
  i = t - c * (c + 1) / 2;
  j = c;
}

// Tile number -> upper tile (ti <= tj) of a T x T tile grid, in blocks of 8 x 8 tiles:
// workgroups that run at the same time have neighbouring numbers, so the ~64 of them that
// share an XCD's L2 work on one block and read 8 + 8 feature panels of X between them instead
// of nearly all T (consecutive tiles of a plain column order span whole tile columns).
constexpr int TBLK = 8;
__device__ __forceinline__ void tile_decode(int t, int T, int &ti, int &tj) {
  const int nblk = (T + TBLK - 1) / TBLK;
  for (int bj = 0; bj < nblk; ++bj) {
    const int wj = min(TBLK, T - TBLK * bj);        // tile columns in this block column
    const int off = bj * TBLK * wj;                 // tiles in its bj full-height blocks
    const int cnt = off + wj * (wj + 1) / 2;        // ... plus the diagonal block
    if (t < cnt) {
      if (t < off) {
        const int bi = t / (TBLK * wj), r = t - bi * (TBLK * wj);
        ti = TBLK * bi + (r % TBLK);
        tj = TBLK * bj + (r / TBLK);
      } else {
        int a, b;
        tri_decode(t - off, a, b);
        ti = TBLK * bj + a;
        tj = TBLK * bj + b;
      }
      return;
    }
    t -= cnt;
  }
  ti = tj = 0;   // not reached for t < T (T + 1) / 2
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
  tile_decode(t, p.T, ti, tj);
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

// ---------------------------------------------------------------------------- 16-bit inputs
// X^T X for fp16 / bf16 batches on v_mfma_f32_32x32x16_{f16,bf16}.  The product of two fp16
// (or two bf16) numbers is exact in fp32 and the instruction accumulates in fp32, so this
// computes what the fp32 kernel computes from the widened inputs, up to summation order, at
// the 16-bit matrix rate.  Same ownership as above (upper tile x row slice, accumulators in
// registers for the whole launch, partial tiles reduced in slice order).
//
// Both MFMA operands want, per lane, 8 consecutive rows (k) of ONE feature, while X is stored
// with the features contiguous.  The transpose happens in registers on the way into LDS: a
// thread loads an 8-row x 8-feature block (8 loads of 16 bytes), turns it with 32 byte
// permutes and writes 8 feature rows of 16 bytes.  LDS
// holds [feature][k] with a pitch of 72 halves, which makes the operand fetch (16 bytes per
// lane, 32 consecutive features) conflict free.  Slabs are 64 rows, double buffered (72 KiB).
constexpr int S16_BK = 64;
constexpr int S16_PITCH = S16_BK + 8;
constexpr int S16_OP = HB * S16_PITCH;            // halves per operand buffer
constexpr int S16_LDS_BYTES = 2 * 2 * S16_OP * 2;

typedef uint32_t hu32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Mfma16;
template <> struct Mfma16<__half> {
  typedef _Float16 v8 __attribute__((ext_vector_type(8)));
  static __device__ __forceinline__ floatx16 mma(v8 a, v8 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma16<__hip_bfloat16> {
  typedef __bf16 v8 __attribute__((ext_vector_type(8)));
  static __device__ __forceinline__ floatx16 mma(v8 a, v8 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};

// Requires K % 8 == 0 and 16-byte aligned batches (checked on the host).
template <typename T>
__global__ __launch_bounds__(256) void syrk16_kernel(SyrkArgs p) {
  extern __shared__ __attribute__((aligned(16))) uint16_t lds16[];   // [buffer][A, B][feature][k]
  typedef typename Mfma16<T>::v8 v8;
  const int ntiles = p.T * (p.T + 1) / 2;
  // Slices are taken out of the concatenation of all batches and handed out slice-major: the
  // workgroups in flight then work on one or two slices (134 MB each for K = 4096 and 16384
  // rows), which the 256 MB Infinity Cache keeps while the tiles re-read them.
  // Workgroup ids are dealt round-robin to the 8 XCDs, each with an L2 of its own, and ~64
  // workgroups run on an XCD at a time.  Renumber so that those 64 are consecutive work items
  // (one 8 x 8 block of tiles of one slice, 16 feature panels between them) instead of every
  // eighth one: item = ((q / 64) * 8 + xcd) * 64 + q % 64 for id = 8 q + xcd.
  unsigned item = blockIdx.x;
  {
    const unsigned full = gridDim.x & ~511u;
    if (item < full) {
      const unsigned xcd = item & 7u, q = item >> 3;
      item = ((q >> 6) * 8u + xcd) * 64u + (q & 63u);
    }
  }
  const int rs = (int)item / ntiles, t = (int)item - rs * ntiles;
  int ti, tj;
  tile_decode(t, p.T, ti, tj);
  const int m0 = ti * HB, n0 = tj * HB, K = p.K;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, lhi = lane >> 5;

  // staging role: wavefronts 0-1 bring in the ti panel (operand A), 2-3 the tj panel (B).
  // Block assignment: 16 neighbouring lanes hold the 16 feature groups of one row block, so a
  // load instruction reads four 256-byte row segments (the vector memory pipe was measured to
  // cost about as much per contiguous segment as per instruction: eight 128-byte segments took
  // 8.3 ms for the loads alone, four 256-byte ones 5.6 ms).  The transposed 16-byte stores of
  // those 16 lanes would all fall on two groups of four banks (feature groups are 8 x 36 words
  // = 32 banks apart), so the 8-row blocks of a feature row are stored in a swizzled order:
  // block kb of feature group fg goes to position kb ^ (fg >> 1).  Bank = 32 (fg & 1) +
  // 4 (kb ^ (fg >> 1)) + const: 16 distinct groups of four banks.  A reader's 16 neighbouring
  // lanes (16 consecutive features, i.e. two feature groups 2h, 2h + 1) share the swizzle h.
  const int op = tid >> 7, t7 = tid & 127, fg = t7 & 15, kb = t7 >> 4;
  const int kb_sw = kb ^ (fg >> 1);
  const int f0 = (op ? n0 : m0) + fg * 8;
  const bool f_ok = f0 + 8 <= K;
  const int f0c = f_ok ? f0 : 0;
  const bool edge_tile = (n0 + HB > K);   // tj >= ti: the only panels that can run past K

  // this slice: global rows [g0, g0 + left); find the batch and row it starts at and count
  // its slabs (a slab never crosses a batch boundary)
  int b = 0, kt = 0, left = 0, nslabs = 0;
  {
    const int64_t g0 = (int64_t)rs * p.chunk;
    int64_t base = 0;
    bool started = false;
    int rem = 0;
    for (int bb = 0; bb < p.nb; ++bb) {
      const int rows = p.rows[bb];
      if (!started && g0 < base + rows) {
        started = true;
        b = bb;
        kt = (int)(g0 - base);
        rem = p.chunk;
      }
      if (started && rem > 0) {
        const int from = (bb == b) ? kt : 0;
        const int take = min(rows - from, rem);
        nslabs += (take + S16_BK - 1) / S16_BK;
        left += take;
        rem -= take;
      }
      base += rows;
    }
  }

  // A slab in flight: this thread's 8 x 8 block, the number of its rows that exist and whether
  // the whole slab is full.  Three slabs are kept in flight (a slab is only ~0.2 us of matrix
  // work, far less than a trip to memory).  Loads are unconditional, from clamped addresses (a
  // load inside a branch would be waited for at the join); what does not exist is zeroed
  // before the store to LDS.
  struct Slab { hu32x4 r[8]; int nvalid; bool full; };
  auto load_next = [&](Slab &sl) __attribute__((always_inline)) {
    const bool live = left > 0;
    const int bb = live ? b : 0;
    const int rows = p.rows[bb];
    const uint16_t *X = reinterpret_cast<const uint16_t *>(p.ptr[bb]);
    const int k0 = live ? kt : 0;
    const int avail = live ? min(min(S16_BK, rows - k0), left) : 1;
    const int row0 = k0 + kb * 8, kend = k0 + avail;
    sl.nvalid = (live && f_ok) ? kend - row0 : 0;
    sl.full = live && avail == S16_BK && !edge_tile;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const int row = min(row0 + r, kend - 1);
      sl.r[r] = *reinterpret_cast<const hu32x4 *>(X + (int64_t)row * K + f0c);
    }
    // advance (scalar selects only)
    const int nkt = k0 + avail;
    const bool wrap = nkt >= rows;
    left = live ? left - avail : 0;
    kt = live ? (wrap ? 0 : nkt) : kt;
    b = (live && wrap) ? b + 1 : b;
  };
  auto store_slab = [&](Slab &sl, int buf) __attribute__((always_inline)) {
    if (!sl.full) {     // ragged end of a batch or slice, or features past K (uniform branch)
      const hu32x4 zero4 = {0u, 0u, 0u, 0u};
#pragma unroll
      for (int r = 0; r < 8; ++r) sl.r[r] = (r < sl.nvalid) ? sl.r[r] : zero4;
    }
    uint16_t *dst = lds16 + (buf * 2 + op) * S16_OP + (fg * 8) * S16_PITCH + kb_sw * 8;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;   // high / low halves of two words
      hu32x4 o;
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const uint32_t w0 = sl.r[2 * m][c >> 1], w1 = sl.r[2 * m + 1][c >> 1];
        o[m] = __builtin_amdgcn_perm(w1, w0, sel);                // {X[2m][f], X[2m+1][f]}
      }
      *reinterpret_cast<hu32x4 *>(dst + c * S16_PITCH) = o;
    }
  };

  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  Slab s0, s1, s2;
  load_next(s0);
  load_next(s1);
  load_next(s2);
  int buf = 0;
  if (nslabs > 0) store_slab(s0, 0);
  __syncthreads();
  int sw_a[2], sw_b[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    sw_a[q] = ((wm * 64 + q * 32 + l32) >> 4) & 7;
    sw_b[q] = ((wn * 64 + q * 32 + l32) >> 4) & 7;
  }
  // one step: refill the ring slot whose slab is already in LDS, multiply the slab in LDS,
  // stage the next one.  The main loop runs whole triples with no conditions inside (every
  // early exit would be another path into the loop head on which the compiler has to assume
  // the worst about loads still in flight); the last one to three slabs follow it.
  auto step = [&](Slab &refill, Slab &next, bool do_load, bool has_next) __attribute__((always_inline)) {
    if (do_load) load_next(refill);
    const uint16_t *as = lds16 + (buf * 2) * S16_OP + (wm * 64 + l32) * S16_PITCH;
    const uint16_t *bs = lds16 + (buf * 2 + 1) * S16_OP + (wn * 64 + l32) * S16_PITCH;
#pragma unroll
    for (int ks = 0; ks < S16_BK; ks += 16) {
      v8 a[2], bq[2];
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        // 8-row block (ks / 8 + lhi) of feature 32 q + l32 (+ 64 wm / wn): swizzle (feature >> 4) & 7
        const int blk = ks / 8 + lhi;
        a[q] = *reinterpret_cast<const v8 *>(as + q * 32 * S16_PITCH + ((blk ^ sw_a[q]) * 8));
        bq[q] = *reinterpret_cast<const v8 *>(bs + q * 32 * S16_PITCH + ((blk ^ sw_b[q]) * 8));
      }
#pragma unroll
      for (int ii = 0; ii < 2; ++ii)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[ii][j] = Mfma16<T>::mma(a[ii], bq[j], acc[ii][j]);
    }
    if (has_next) store_slab(next, buf ^ 1);
    __syncthreads();
    buf ^= 1;
  };
  int i = 0;
  for (; i + 3 < nslabs; i += 3) {
    step(s0, s1, true, true);
    step(s1, s2, true, true);
    step(s2, s0, true, true);
  }
  if (i < nslabs) step(s0, s1, false, i + 1 < nslabs);
  if (i + 1 < nslabs) step(s1, s2, false, i + 2 < nslabs);
  if (i + 2 < nslabs) step(s2, s0, false, false);

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

// ---------------------------------------------------------------------------- 16-bit inputs, wide tiles
// Same product as syrk16_kernel with a 256 x 256 tile per workgroup (128 x 128 per wavefront:
// 4 x 4 MFMA tiles, 256 accumulator registers).  Two things bound the 128 x 128 version and both
// scale with the tile edge: the vector-memory pipe costs about as much per contiguous row segment
// as per instruction (here a load instruction covers two 512-byte segments instead of four
// 256-byte ones, and feeds four times the MFMA work), and every 16-byte operand fetch from LDS
// now feeds four 32-cycle MFMAs instead of two.  Slabs are 32 rows (80 KiB of LDS double
// buffered, one workgroup per CU, one wavefront per SIMD), pitch 40 halves.
constexpr int W16_TB = 256;
constexpr int W16_BK = 32;
constexpr int W16_PITCH = W16_BK + 8;
constexpr int W16_OP = W16_TB * W16_PITCH;          // halves per operand buffer
constexpr int W16_LDS_BYTES = 2 * 2 * W16_OP * 2;

template <typename T>
__global__ __launch_bounds__(256) void syrk16w_kernel(SyrkArgs p) {
  extern __shared__ __attribute__((aligned(16))) uint16_t lds16w[];   // [buffer][A, B][feature][k]
  typedef typename Mfma16<T>::v8 v8;
  const int ntiles = p.T * (p.T + 1) / 2;
  // 32 workgroups (one per CU) run on an XCD at a time: make them consecutive work items
  unsigned item = blockIdx.x;
  {
    const unsigned full = gridDim.x & ~255u;
    if (item < full) {
      const unsigned xcd = item & 7u, q = item >> 3;
      item = ((q >> 5) * 8u + xcd) * 32u + (q & 31u);
    }
  }
  const int rs = (int)item / ntiles, t = (int)item - rs * ntiles;
  int ti, tj;
  tile_decode(t, p.T, ti, tj);
  const int m0 = ti * W16_TB, n0 = tj * W16_TB, K = p.K;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, lhi = lane >> 5;

  // staging: wavefronts 0-1 bring in the ti panel (operand A), 2-3 the tj panel (B); 32
  // neighbouring lanes hold the 32 feature groups of one 8-row block (512 contiguous bytes)
  const int op = tid >> 7, t7 = tid & 127, fg = t7 & 31, kb = t7 >> 5;
  const int kb_sw = kb ^ ((fg >> 1) & 3);
  const int f0 = (op ? n0 : m0) + fg * 8;
  const bool f_ok = f0 + 8 <= K;
  const int f0c = f_ok ? f0 : 0;
  const bool edge_tile = (n0 + W16_TB > K);

  int b = 0, kt = 0, left = 0, nslabs = 0;
  {
    const int64_t g0 = (int64_t)rs * p.chunk;
    int64_t base = 0;
    bool started = false;
    int rem = 0;
    for (int bb = 0; bb < p.nb; ++bb) {
      const int rows = p.rows[bb];
      if (!started && g0 < base + rows) {
        started = true;
        b = bb;
        kt = (int)(g0 - base);
        rem = p.chunk;
      }
      if (started && rem > 0) {
        const int from = (bb == b) ? kt : 0;
        const int take = min(rows - from, rem);
        nslabs += (take + W16_BK - 1) / W16_BK;
        left += take;
        rem -= take;
      }
      base += rows;
    }
  }

  struct Slab { hu32x4 r[8]; int nvalid; bool full; };
  auto load_next = [&](Slab &sl) __attribute__((always_inline)) {
    const bool live = left > 0;
    const int bb = live ? b : 0;
    const int rows = p.rows[bb];
    const uint16_t *X = reinterpret_cast<const uint16_t *>(p.ptr[bb]);
    const int k0 = live ? kt : 0;
    const int avail = live ? min(min(W16_BK, rows - k0), left) : 1;
    const int row0 = k0 + kb * 8, kend = k0 + avail;
    sl.nvalid = (live && f_ok) ? kend - row0 : 0;
    sl.full = live && avail == W16_BK && !edge_tile;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const int row = min(row0 + r, kend - 1);
      sl.r[r] = *reinterpret_cast<const hu32x4 *>(X + (int64_t)row * K + f0c);
    }
    const int nkt = k0 + avail;
    const bool wrap = nkt >= rows;
    left = live ? left - avail : 0;
    kt = live ? (wrap ? 0 : nkt) : kt;
    b = (live && wrap) ? b + 1 : b;
  };
  auto store_slab = [&](Slab &sl, int buf) __attribute__((always_inline)) {
    // rows past the end of a batch / slice and features past K become zeros; done with selects
    // for every slab (full ones have nvalid >= 8): a branch here would cut the step into short
    // scheduling regions and keep this work from being interleaved with the MFMAs
    {
      const hu32x4 zero4 = {0u, 0u, 0u, 0u};
#pragma unroll
      for (int r = 0; r < 8; ++r) sl.r[r] = (r < sl.nvalid) ? sl.r[r] : zero4;
    }
    uint16_t *dst = lds16w + (buf * 2 + op) * W16_OP + (fg * 8) * W16_PITCH + kb_sw * 8;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;
      hu32x4 o;
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const uint32_t w0 = sl.r[2 * m][c >> 1], w1 = sl.r[2 * m + 1][c >> 1];
        o[m] = __builtin_amdgcn_perm(w1, w0, sel);
      }
      *reinterpret_cast<hu32x4 *>(dst + c * W16_PITCH) = o;
    }
  };

  floatx16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  Slab s0, s1, s2;
  load_next(s0);
  load_next(s1);
  load_next(s2);
  int buf = 0;
  if (nslabs > 0) store_slab(s0, 0);
  __syncthreads();
  int sw_a[4], sw_b[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    sw_a[q] = ((wm * 128 + q * 32 + l32) >> 4) & 3;
    sw_b[q] = ((wn * 128 + q * 32 + l32) >> 4) & 3;
  }
  // operands of one 16-row half of a slab: a[q] / b[q] = rows 32 q + l32 of this wavefront's
  // 128 features, eight consecutive k of block 2 * half + lhi
  struct Ops { v8 a[4], b[4]; };
  auto read_ops = [&](Ops &o, int bufi, int half) __attribute__((always_inline)) {
    const uint16_t *as = lds16w + (bufi * 2) * W16_OP + (wm * 128 + l32) * W16_PITCH;
    const uint16_t *bs = lds16w + (bufi * 2 + 1) * W16_OP + (wn * 128 + l32) * W16_PITCH;
    const int blk = 2 * half + lhi;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      o.a[q] = *reinterpret_cast<const v8 *>(as + q * 32 * W16_PITCH + ((blk ^ sw_a[q]) * 8));
      o.b[q] = *reinterpret_cast<const v8 *>(bs + q * 32 * W16_PITCH + ((blk ^ sw_b[q]) * 8));
    }
  };
  auto mfma_all = [&](const Ops &o) __attribute__((always_inline)) {
#pragma unroll
    for (int ii = 0; ii < 4; ++ii)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[ii][j] = Mfma16<T>::mma(o.a[ii], o.b[j], acc[ii][j]);
  };
  // One barrier per slab, and no LDS latency in front of the matrix pipe: the operands of the
  // first half of slab s+1 are fetched (after the barrier that publishes slab s+1) while the
  // MFMAs of the second half of slab s run, those of the second half while the first half runs.
  // Slab s+2 goes into the buffer of slab s during step s+1, i.e. after the barrier of step s,
  // which every wavefront reaches with its reads of slab s complete.
  Ops o0, o1;
  if (nslabs > 0) read_ops(o0, 0, 0);
  // A wavefront issues in order and is alone on its SIMD, so whatever is not placed between two
  // MFMAs in program order runs while the matrix pipe idles.  Each half of a step is one
  // scheduling region (no branches) with 16 MFMAs of 32 cycles; the group barriers spread the
  // other work of the half over the gaps: operand reads, transposing permutes and LDS writes
  // in the first half, address arithmetic, global loads and operand reads in the second.
  auto step = [&](Slab &refill, Slab &next, bool do_load, bool has_next) __attribute__((always_inline)) {
    read_ops(o1, buf, 1);
    mfma_all(o0);
    if (has_next) store_slab(next, buf ^ 1);
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // MFMA
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // LDS read
      __builtin_amdgcn_sched_group_barrier(0x002, 5, 0);   // VALU
      __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);   // LDS write
    }
    __syncthreads();
    if (do_load) load_next(refill);
    if (has_next) read_ops(o0, buf ^ 1, 0);
    mfma_all(o1);
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // MFMA
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // LDS read
      __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);   // VALU
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);   // global load
    }
    buf ^= 1;
  };
  int i = 0;
  for (; i + 3 < nslabs; i += 3) {
    step(s0, s1, true, true);
    step(s1, s2, true, true);
    step(s2, s0, true, true);
  }
  if (i < nslabs) step(s0, s1, false, i + 1 < nslabs);
  if (i + 1 < nslabs) step(s1, s2, false, i + 2 < nslabs);
  if (i + 2 < nslabs) step(s2, s0, false, false);

  if (p.RS == 1) {
#pragma unroll
    for (int ii = 0; ii < 4; ++ii)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int col = n0 + wn * 128 + j * 32 + l32;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = m0 + wm * 128 + ii * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3);
          if (row < K && col < K) p.H[(int64_t)row * K + col] += acc[ii][j][r];
        }
      }
  } else {
    float *dst = p.ws + ((int64_t)rs * ntiles + t) * (W16_TB * W16_TB);
#pragma unroll
    for (int ii = 0; ii < 4; ++ii)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int col = wn * 128 + j * 32 + l32;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = wm * 128 + ii * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3);
          dst[row * W16_TB + col] = acc[ii][j][r];
        }
      }
  }
}

// ---------------------------------------------------------------------------- 16-bit inputs, loads straight into LDS
// Same tiles, slices and accumulators as syrk16w_kernel, for the regular case: K a multiple of
// 256 and every batch a multiple of 32 rows (all slabs full, no feature past K).  There the rows
// travel from global memory to LDS without touching a register (global_load_lds_dwordx4: a
// wavefront instruction moves 64 x 16 bytes to 1 KB of consecutive LDS, i.e. two rows of a
// 256-feature panel), LDS keeps them as they are in memory, [k][feature], and the MFMA operands
// (eight k of one feature per lane) come from the transposing read ds_read_b64_tr_b16: within
// 16 lanes, lanes 4r .. 4r+3 address four features each of row r, and lane i receives feature i
// of the four rows.  Against the register-staged kernel this takes the 96 ring VGPRs, the byte
// permutes, the LDS writes and the trip of every row through the vector-memory return path out
// of the loop.
//
// LDS: 4 slab buffers of 32 rows; a slab holds, per operand, 16 row pairs of 1024 + 64 bytes.
// The padding puts the four rows that a 16-lane group reads (the even or the odd rows of four
// pairs) and the two feature halves of a 32-lane group on eight different 32-byte bank ranges.
// The k slots of a lane are the even rows of its four pairs, then the odd rows; both operands
// use the same assignment, so the products pair up.
//
// The loads are issued through inline assembly: the compiler then does not know that they
// write LDS and inserts no waits of its own between them and the LDS reads (with the builtin it
// waits for every outstanding load before any read, which serialises the pipeline).  The waits
// that are needed are explicit: before the barrier of step s a wavefront waits for its own
// loads of slab s (vmcnt leaves the two later slabs in flight) and for its LDS reads of slab
// s-1, whose buffer is the target of the loads issued right after the barrier.
constexpr int D16_BK = 32;
constexpr int D16_NBUF = 4;
constexpr int D16_PAIR = 1024 + 64;
constexpr int D16_OP = (D16_BK / 2) * D16_PAIR;
constexpr int D16_SLAB = 2 * D16_OP;
constexpr int D16_LDS_BYTES = D16_NBUF * D16_SLAB;

// 16 bytes per lane from global memory to LDS byte address dst (wave-uniform) + 16 * lane
__device__ __forceinline__ void load_to_lds_16(const void *src, uint32_t dst) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
               :
               : "s"(dst), "v"(src)
               : "memory", "m0");
}

template <typename T, typename ARGS, bool PIECES = false>
__global__ __launch_bounds__(256) void syrk16d_kernel(ARGS p) {
  extern __shared__ __attribute__((aligned(16))) char lds16d[];
  typedef typename Mfma16<T>::v8 v8;
  typedef short s4 __attribute__((ext_vector_type(4)));
  typedef short s8 __attribute__((ext_vector_type(8)));
  typedef __attribute__((address_space(3))) char lds_char;
  const int ntiles = p.T * (p.T + 1) / 2;
  unsigned item = blockIdx.x;
  {
    const unsigned full = gridDim.x & ~255u;
    if (item < full) {
      const unsigned xcd = item & 7u, q = item >> 3;
      item = ((q >> 5) * 8u + xcd) * 32u + (q & 31u);
    }
  }
  static_assert(!(PIECES && ARGS::DUAL), "runs of (tile, slab) pairs: plain batches only");
  const int K = p.K;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, lhi = lane >> 5;
  // PIECES: this workgroup's run [u0, u1) of the tile-major (tile, slab) pairs (see syrk32d_kernel); p.chunk
  // holds the slabs per tile (rows of the call / 32)
  int64_t u0 = 0, u1 = 0;
  if (PIECES) {
    const int64_t U = (int64_t)ntiles * p.chunk;
    u0 = (int64_t)item * U / gridDim.x;
    u1 = (int64_t)(item + 1) * U / gridDim.x;
    if (u0 >= u1) return;
  }
  bool first_piece = true;
  do {
  int rs = 0, t, piece_rows = p.chunk;
  int64_t g0;
  bool whole = false;
  if (PIECES) {
    t = (int)(u0 / p.chunk);
    const int s0 = (int)(u0 - (int64_t)t * p.chunk);
    const int n = (int)min((int64_t)(p.chunk - s0), u1 - u0);
    g0 = (int64_t)s0 * D16_BK;
    piece_rows = n * D16_BK;
    whole = n == p.chunk;
    u0 += n;
  } else {
    rs = (int)item / ntiles;
    t = (int)item - rs * ntiles;
    g0 = (int64_t)rs * p.chunk;
  }
  int ti, tj;
  tile_decode(t, p.T, ti, tj);
  const int m0 = ti * W16_TB, n0 = tj * W16_TB;

  // rows [g0, g0 + piece_rows) of the concatenated batches: first slab (b, kt), number of slabs
  int b = 0, kt = 0, nslabs = 0;
  {
    int64_t base = 0;
    bool started = false;
    int rem = 0;
    for (int bb = 0; bb < p.nb; ++bb) {
      const int rows = p.rows[bb];
      if (!started && g0 < base + rows) {
        started = true;
        b = bb;
        kt = (int)(g0 - base);
        rem = piece_rows;
      }
      if (started && rem > 0) {
        const int from = (bb == b) ? kt : 0;
        const int take = min(rows - from, rem);
        nslabs += take / D16_BK;          // rows, chunk and kt are multiples of D16_BK here
        rem -= take;
      }
      base += rows;
    }
  }

  const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_char *)lds16d;
  // loads: wavefronts 0-1 bring in the ti panel (operand A), 2-3 the tj panel (B); a wavefront
  // owns 8 row pairs of its operand; lanes 0-31 the even row of a pair, 32-63 the odd one
  const int ld_op = wave >> 1, ld_pair0 = (wave & 1) * 8;
  const int ld_feat = (ld_op ? n0 : m0) + l32 * 8;
  const uint32_t ld_dst0 = lds0 + ld_op * D16_OP + ld_pair0 * D16_PAIR;
  // position of the next slab to load: batch b (base pointer Xb, rows_b rows), row kt
  // (the choice of the table is made on a scalar: left to a per-lane select, the batch pointer
  //  would live in vector registers, of which this kernel has none to spare)
  const bool from_b = ARGS::DUAL && __builtin_amdgcn_readfirstlane(ld_op) != 0;
  auto batch_ptr = [&](int bb) __attribute__((always_inline)) -> const uint16_t * {
    if constexpr (ARGS::DUAL) {
      const void *const *tab = from_b ? p.ptrB : p.ptr;
      return reinterpret_cast<const uint16_t *>(tab[bb]);
    } else {
      return reinterpret_cast<const uint16_t *>(p.ptr[bb]);
    }
  };
  const uint16_t *Xb = batch_ptr(b);
  int rows_b = p.rows[b];
  int issued = 0;
  // source of this lane for the 8 loads of the next slab, LDS target of the first of them; then advance
  auto next_slab = [&](const uint16_t *&src, uint32_t &dst) __attribute__((always_inline)) {
    src = Xb + (int64_t)(kt + 2 * ld_pair0 + lhi) * K + ld_feat;
    dst = __builtin_amdgcn_readfirstlane(ld_dst0 + (uint32_t)(issued & (D16_NBUF - 1)) * D16_SLAB);
    ++issued;
    kt += D16_BK;
    if (kt >= rows_b && issued < nslabs) {      // rare: next batch
      ++b;
      kt = 0;
      Xb = batch_ptr(b);
      rows_b = p.rows[b];
    }
  };
  auto load_pair = [&](const uint16_t *src, uint32_t dst, int j) __attribute__((always_inline)) {
    load_to_lds_16(src + (int64_t)(2 * j) * K, dst + j * D16_PAIR);
  };

  // operand reads: 16-lane group g16 = lane / 16 covers features (g16 & 1) * 16 .. + 15 of a
  // 32-feature MFMA row block and the k half lhi = g16 / 2; within it lane i addresses row pair
  // 4 * lhi + i / 4 (+ 8 for the second 16 rows of the slab) at features 4 * (i % 4) .. + 3
  const int rd_i = lane & 15;
  const uint32_t rd_lane = (uint32_t)((4 * lhi + (rd_i >> 2)) * D16_PAIR + ((((lane >> 4) & 1) * 16 + (rd_i & 3) * 4) * 2));
  const uint32_t rd_a = rd_lane + (uint32_t)(wm * 128 * 2);
  const uint32_t rd_b = rd_lane + (uint32_t)(D16_OP + wn * 128 * 2);
  auto tr8 = [&](uint32_t addr) __attribute__((always_inline)) -> v8 {
    lds_char *q = (lds_char *)lds16d + addr;
    const s4 even = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s4 __attribute__((address_space(3))) *)q);
    const s4 odd = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s4 __attribute__((address_space(3))) *)(q + 512));
    const s8 w = __builtin_shufflevector(even, odd, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(v8, w);
  };

  floatx16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // One slab: 8 groups of 4 MFMAs (one row block of A against the four of B), in two halves
  // of 16 rows.  A wavefront issues in order and is alone on its SIMD, and the four wavefronts
  // leave the barrier together: eight loads each, issued at once, queue up in the vector-memory
  // unit and stall the MFMA issue behind them (measured: a third of the kernel).  So the order
  // is fixed by hand: one load and the operand reads of a later group between two groups of
  // MFMAs.  The loop is skewed by half a slab: a step runs the second half of slab s-1 from
  // registers, then the first half of slab s, so that the first reads after a barrier have
  // four groups of MFMAs in front of their first use.
  struct Half { v8 a[4], b[4]; };
  auto group = [&](const v8 &a, const v8 (&bq)[4], int ii) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[ii][j] = Mfma16<T>::mma(a, bq[j], acc[ii][j]);
  };
  // second half of the previous slab (operands in `prev`), then the first half of the slab in
  // `buf`; leaves the operands of its second half in `prev`
  auto step = [&](Half &prev, int buf, bool dma, const uint16_t *src, uint32_t dst) __attribute__((always_inline)) {
    const uint32_t h0 = (uint32_t)(buf * D16_SLAB), h1 = h0 + 8 * D16_PAIR;
    Half cur, nxt;
#pragma unroll
    for (int q = 0; q < 4; ++q) cur.b[q] = tr8(rd_b + h0 + q * 64);
    cur.a[0] = tr8(rd_a + h0);
    if (dma) load_pair(src, dst, 0);
    __builtin_amdgcn_sched_barrier(0);
    group(prev.a[0], prev.b, 0);
    cur.a[1] = tr8(rd_a + h0 + 64);
    if (dma) load_pair(src, dst, 1);
    __builtin_amdgcn_sched_barrier(0);
    group(prev.a[1], prev.b, 1);
    cur.a[2] = tr8(rd_a + h0 + 128);
    if (dma) load_pair(src, dst, 2);
    __builtin_amdgcn_sched_barrier(0);
    group(prev.a[2], prev.b, 2);
    cur.a[3] = tr8(rd_a + h0 + 192);
    if (dma) load_pair(src, dst, 3);
    __builtin_amdgcn_sched_barrier(0);
    group(prev.a[3], prev.b, 3);
    nxt.b[0] = tr8(rd_b + h1);
    nxt.b[1] = tr8(rd_b + h1 + 64);
    if (dma) load_pair(src, dst, 4);
    __builtin_amdgcn_sched_barrier(0);
    group(cur.a[0], cur.b, 0);
    nxt.b[2] = tr8(rd_b + h1 + 128);
    nxt.b[3] = tr8(rd_b + h1 + 192);
    nxt.a[0] = tr8(rd_a + h1);
    if (dma) load_pair(src, dst, 5);
    __builtin_amdgcn_sched_barrier(0);
    group(cur.a[1], cur.b, 1);
    nxt.a[1] = tr8(rd_a + h1 + 64);
    if (dma) load_pair(src, dst, 6);
    __builtin_amdgcn_sched_barrier(0);
    group(cur.a[2], cur.b, 2);
    nxt.a[2] = tr8(rd_a + h1 + 128);
    if (dma) load_pair(src, dst, 7);
    __builtin_amdgcn_sched_barrier(0);
    group(cur.a[3], cur.b, 3);
    nxt.a[3] = tr8(rd_a + h1 + 192);
    __builtin_amdgcn_sched_barrier(0);
    prev = nxt;
  };
  // own loads of slab s done (`later` slabs of 8 loads each may stay in flight), own LDS reads
  // done, then the workgroup barrier: slab s is visible, nobody reads the buffer of slab s-1 any more
  auto publish = [&](int later) __attribute__((always_inline)) {
    asm volatile("" ::: "memory");
    if (later >= 2) __builtin_amdgcn_s_waitcnt(0x4070);        // vmcnt(16) lgkmcnt(0)
    else if (later == 1) __builtin_amdgcn_s_waitcnt(0x0078);   // vmcnt(8) lgkmcnt(0)
    else __builtin_amdgcn_s_waitcnt(0x0070);                   // vmcnt(0) lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };

  if (nslabs > 0) {
    for (int s = 0; s < D16_NBUF - 1 && s < nslabs; ++s) {
      const uint16_t *src;
      uint32_t dst;
      next_slab(src, dst);
#pragma unroll
      for (int j = 0; j < 8; ++j) load_pair(src, dst, j);
    }
    Half prev;
#pragma unroll
    for (int q = 0; q < 4; ++q) prev.a[q] = prev.b[q] = v8{0, 0, 0, 0, 0, 0, 0, 0};   // "slab -1": adds zeros
    int s = 0;
    // steady state: slab s + 3 is loaded during step s, two later slabs (16 loads) stay in flight
    for (; s + D16_NBUF - 1 < nslabs; ++s) {
      const uint16_t *src;
      uint32_t dst;
      next_slab(src, dst);
      publish(2);
      step(prev, s & (D16_NBUF - 1), true, src, dst);
    }
    for (; s < nslabs; ++s) {
      publish(nslabs - 1 - s);
      step(prev, s & (D16_NBUF - 1), false, nullptr, 0u);
    }
    // second half of the last slab
#pragma unroll
    for (int ii = 0; ii < 4; ++ii) group(prev.a[ii], prev.b, ii);
  }

  float unit = 1.f;
  bool accum = false;
  if constexpr (ARGS::DUAL) {
    unit = *p.factor;
    accum = p.accum != 0;
  }
  // (PIECES: offsets that do not change from piece to piece are hidden from the compiler, which would otherwise
  // compute all 512 of them in front of the loop and park them in scratch memory)
  int e_col = wn * 128 + l32, e_row = wm * 128 + 4 * lhi;
  if (PIECES) asm volatile("" : "+v"(e_col), "+v"(e_row));
  if (PIECES ? whole : p.RS == 1) {
#pragma unroll
    for (int ii = 0; ii < 4; ++ii)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int col = n0 + e_col + j * 32;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = m0 + e_row + ii * 32 + 8 * (r >> 2) + (r & 3);
          p.H[(int64_t)row * K + col] += ARGS::DUAL ? acc[ii][j][r] * unit : acc[ii][j][r];
        }
      }
  } else if (PIECES) {
    // partial tile in register order, slot 2 w (the run's first piece) or 2 w + 1 (its last), as syrk32d_kernel
    // stores it and syrk_reduce_pieces_kernel sums it
    float4 *dst = reinterpret_cast<float4 *>(p.ws + (int64_t)(2 * item + (first_piece ? 0 : 1)) * (W16_TB * W16_TB)) +
                  wave * 4096 + lane;
#pragma unroll
    for (int ii = 0; ii < 4; ++ii)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int rq = 0; rq < 4; ++rq)
          dst[((ii * 4 + j) * 4 + rq) * 64] =
              make_float4(acc[ii][j][4 * rq], acc[ii][j][4 * rq + 1], acc[ii][j][4 * rq + 2], acc[ii][j][4 * rq + 3]);
  } else {
    float *dst = p.ws + ((int64_t)rs * ntiles + t) * (W16_TB * W16_TB);
#pragma unroll
    for (int ii = 0; ii < 4; ++ii)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int col = wn * 128 + j * 32 + l32;
        // (accumulating: the sixteen loads of a block first, so that they are in flight together)
        float old[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = wm * 128 + ii * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3);
          old[r] = (ARGS::DUAL && accum) ? dst[row * W16_TB + col] : 0.f;
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = wm * 128 + ii * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3);
          dst[row * W16_TB + col] = ARGS::DUAL ? acc[ii][j][r] + old[r] : acc[ii][j][r];
        }
      }
  }
  if (!PIECES) break;
  first_piece = false;
  __syncthreads();           // the next piece's loads reuse the slab buffers
  } while (u0 < u1);
}

// ---------------------------------------------------------------------------- fp32 inputs, loads straight into LDS
// The fp32 counterpart of syrk16d_kernel for the regular case (K a multiple of 256, every batch a
// multiple of 16 rows, 16-byte aligned): 256 x 256 tiles, four wavefronts with 128 x 128 each (16
// accumulator tiles of v_mfma_f32_32x32x2_f32 = 256 registers), slabs of 16 rows, four slab
// buffers.  A row of a 256-feature panel is 1 KB, i.e. exactly one global_load_lds_dwordx4 of a
// wavefront; LDS keeps the rows as they are in memory ([k][feature], 1 KB + 128 B apart so that
// the two rows of an MFMA's k pair fall on different banks), which is the operand order of this
// MFMA: lane l reads row 2 kp + l / 32, and - the four MFMA blocks of an operand being the features
// 4 i + q rather than 32 q + i - its features 4 (l % 32) .. + 3 with one ds_read_b128, the operands of
// all four blocks.  Against the 128 x 128-tile kernel at the top of this file: a quarter of the
// barriers and an eighth of the LDS operand reads per MFMA, no staging registers, no LDS writes.
//
// Per slab and wavefront: 8 k pairs x 16 MFMAs (64 cycles each), 8 loads, 16 operand reads; the
// order is fixed by hand as in syrk16d_kernel: before the MFMAs of k pair kp one load of a later
// slab and the operand reads of k pair kp + 1 are issued.  The loop is skewed by one k pair: a
// step starts with the last k pair of the previous slab out of registers, so that the first
// reads after a barrier have 16 MFMAs in front of their first use.
constexpr int D32_BK = 16;
constexpr int D32_NBUF = 4;
constexpr int D32_ROW = 1024 + 128;
constexpr int D32_OP = D32_BK * D32_ROW;
constexpr int D32_SLAB = 2 * D32_OP;
constexpr int D32_LDS_BYTES = D32_NBUF * D32_SLAB;

//
// PIECES: the short call (one batch per call, the reference's streaming use, gptq.py:97-98).  With row slices
// the 136 tiles of K = 4096 times RS never come close to a multiple of the 256 CUs unless RS is large, and every
// workgroup pays its pipeline fill and 256 KB of partial tile.  Here the (tile, slab) pairs of the call, tile
// major, are cut into gridDim.x equal runs, one per workgroup: a workgroup works through the end of one tile,
// whole tiles (added to H directly) and the beginning of another, so it writes at most two partial tiles
// (slots 2 w and 2 w + 1 of the workspace), which syrk_reduce_pieces_kernel sums in workgroup order.
// p.chunk holds the slabs per tile (rows of the call / 16).
template <bool PIECES>
__global__ __launch_bounds__(256) void syrk32d_kernel(SyrkArgs p) {
  extern __shared__ __attribute__((aligned(16))) char lds32d[];
  typedef __attribute__((address_space(3))) char lds_char;
  const int ntiles = p.T * (p.T + 1) / 2;
  unsigned item = blockIdx.x;
  {
    const unsigned full = gridDim.x & ~255u;
    if (item < full) {
      const unsigned xcd = item & 7u, q = item >> 3;
      item = ((q >> 5) * 8u + xcd) * 32u + (q & 31u);
    }
  }
  const int K = p.K;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, lhi = lane >> 5;
  // PIECES: this workgroup's run [u0, u1) of the tile-major (tile, slab) pairs
  int64_t u0 = 0, u1 = 0;
  if (PIECES) {
    const int64_t U = (int64_t)ntiles * p.chunk;
    u0 = (int64_t)item * U / gridDim.x;
    u1 = (int64_t)(item + 1) * U / gridDim.x;
    if (u0 >= u1) return;
  }
  bool first_piece = true;
  do {
  int rs = 0, t, piece_rows = p.chunk;
  int64_t g0;
  bool whole = false;
  if (PIECES) {
    t = (int)(u0 / p.chunk);
    const int s0 = (int)(u0 - (int64_t)t * p.chunk);
    const int n = (int)min((int64_t)(p.chunk - s0), u1 - u0);
    g0 = (int64_t)s0 * D32_BK;
    piece_rows = n * D32_BK;
    whole = n == p.chunk;
    u0 += n;
  } else {
    rs = (int)item / ntiles;
    t = (int)item - rs * ntiles;
    g0 = (int64_t)rs * p.chunk;
  }
  int ti, tj;
  tile_decode(t, p.T, ti, tj);
  const int m0 = ti * W16_TB, n0 = tj * W16_TB;

  // rows [g0, g0 + piece_rows) of the concatenated batches: first slab (b, kt), number of slabs
  int b = 0, kt = 0, nslabs = 0;
  {
    int64_t base = 0;
    bool started = false;
    int rem = 0;
    for (int bb = 0; bb < p.nb; ++bb) {
      const int rows = p.rows[bb];
      if (!started && g0 < base + rows) {
        started = true;
        b = bb;
        kt = (int)(g0 - base);
        rem = piece_rows;
      }
      if (started && rem > 0) {
        const int from = (bb == b) ? kt : 0;
        const int take = min(rows - from, rem);
        nslabs += take / D32_BK;          // rows, chunk and kt are multiples of D32_BK here
        rem -= take;
      }
      base += rows;
    }
  }

  const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_char *)lds32d;
  // loads: wavefronts 0-1 bring in the ti panel (operand A), 2-3 the tj panel (B); a wavefront
  // owns 8 rows of its operand, one load each (lane l: features 4 l .. 4 l + 3 of the panel)
  const int ld_op = wave >> 1, ld_row0 = (wave & 1) * 8;
  const int ld_feat = (ld_op ? n0 : m0) + lane * 4;
  const uint32_t ld_dst0 = lds0 + ld_op * D32_OP + ld_row0 * D32_ROW;
  const float *Xb = reinterpret_cast<const float *>(p.ptr[b]);
  int rows_b = p.rows[b];
  int issued = 0;
  auto next_slab = [&](const float *&src, uint32_t &dst) __attribute__((always_inline)) {
    src = Xb + (int64_t)(kt + ld_row0) * K + ld_feat;
    dst = __builtin_amdgcn_readfirstlane(ld_dst0 + (uint32_t)(issued & (D32_NBUF - 1)) * D32_SLAB);
    ++issued;
    kt += D32_BK;
    if (kt >= rows_b && issued < nslabs) {      // rare: next batch
      ++b;
      kt = 0;
      Xb = reinterpret_cast<const float *>(p.ptr[b]);
      rows_b = p.rows[b];
    }
  };
  auto load_row = [&](const float *src, uint32_t dst, int j) __attribute__((always_inline)) {
    load_to_lds_16(src + (int64_t)j * K, dst + j * D32_ROW);
  };

  // operand reads of k pair kp: row 2 kp + lhi, features 4 l32 .. 4 l32 + 3 of the wavefront's 128 in ONE 16-byte
  // read per operand: MFMA block q of an operand is the features 4 i + q (i = 0 .. 31: the MFMA's row / column i),
  // not 32 q + i - which rows of the tile an accumulator holds is free, and this choice takes 2 LDS reads per
  // 16 MFMAs instead of 8
  const uint32_t rd_a = (uint32_t)(lhi * D32_ROW + (wm * 128 + 4 * l32) * 4);
  const uint32_t rd_b = (uint32_t)(D32_OP + lhi * D32_ROW + (wn * 128 + 4 * l32) * 4);
  struct Ops { float a[4], b[4]; };
  auto read_ops = [&](int buf, int kp, Ops &o) __attribute__((always_inline)) {
    const lds_char *base = (const lds_char *)lds32d + buf * D32_SLAB + kp * 2 * D32_ROW;
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    const f32x4 va = *reinterpret_cast<const __attribute__((address_space(3))) f32x4 *>(base + rd_a);
    const f32x4 vb = *reinterpret_cast<const __attribute__((address_space(3))) f32x4 *>(base + rd_b);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      o.a[q] = va[q];
      o.b[q] = vb[q];
    }
  };

  floatx16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  auto mfma_all = [&](const Ops &o) __attribute__((always_inline)) {
#pragma unroll
    for (int ii = 0; ii < 4; ++ii)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[ii][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(o.a[ii], o.b[j], acc[ii][j], 0, 0, 0);
  };
  // the last k pair of the previous slab (operands in `prev`), then k pairs 0 .. 6 of the slab in
  // `buf`; leaves the operands of its k pair 7 in `prev`
  auto step = [&](Ops &prev, int buf, bool dma, const float *src, uint32_t dst) __attribute__((always_inline)) {
    Ops cur;
    read_ops(buf, 0, cur);
    if (dma) load_row(src, dst, 0);
    __builtin_amdgcn_sched_barrier(0);
    mfma_all(prev);
#pragma unroll
    for (int kp = 0; kp < 7; ++kp) {
      Ops nxt;
      read_ops(buf, kp + 1, nxt);
      if (dma) load_row(src, dst, kp + 1);
      __builtin_amdgcn_sched_barrier(0);
      mfma_all(cur);
      __builtin_amdgcn_sched_barrier(0);
      cur = nxt;
    }
    prev = cur;
  };
  // own loads of slab s done (`later` slabs of 8 loads each may stay in flight), own LDS reads
  // done, then the workgroup barrier: slab s is visible, nobody reads the buffer of slab s-1 any more
  auto publish = [&](int later) __attribute__((always_inline)) {
    asm volatile("" ::: "memory");
    if (later >= 2) __builtin_amdgcn_s_waitcnt(0x4070);        // vmcnt(16) lgkmcnt(0)
    else if (later == 1) __builtin_amdgcn_s_waitcnt(0x0078);   // vmcnt(8) lgkmcnt(0)
    else __builtin_amdgcn_s_waitcnt(0x0070);                   // vmcnt(0) lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };

  if (nslabs > 0) {
    for (int s = 0; s < D32_NBUF - 1 && s < nslabs; ++s) {
      const float *src;
      uint32_t dst;
      next_slab(src, dst);
#pragma unroll
      for (int j = 0; j < 8; ++j) load_row(src, dst, j);
    }
    Ops prev;
#pragma unroll
    for (int q = 0; q < 4; ++q) prev.a[q] = prev.b[q] = 0.f;   // "slab -1": adds zeros
    int s = 0;
    // steady state: slab s + 3 is loaded during step s, two later slabs (16 loads) stay in flight
    for (; s + D32_NBUF - 1 < nslabs; ++s) {
      const float *src;
      uint32_t dst;
      next_slab(src, dst);
      publish(2);
      step(prev, s & (D32_NBUF - 1), true, src, dst);
    }
    for (; s < nslabs; ++s) {
      publish(nslabs - 1 - s);
      step(prev, s & (D32_NBUF - 1), false, nullptr, 0u);
    }
    mfma_all(prev);          // last k pair of the last slab
  }

  // accumulator acc[ii][j][r] is row 4 i + ii, column 4 l32 + j of the wavefront's 128 x 128, i = 8 (r / 4) + 4 lhi
  // + r % 4: the four j of a lane are adjacent columns, 16 bytes of a row
  // (PIECES: the element offsets below do not change from piece to piece; left visible, the compiler computes
  // them all in front of the loop and parks them in scratch memory, and a kernel with that much scratch
  // pays for its allocation at every launch)
  int e_col = wn * 128 + 4 * l32, e_row = wm * 128 + 16 * lhi;
  if (PIECES) asm volatile("" : "+v"(e_col), "+v"(e_row));
  if (PIECES ? whole : p.RS == 1) {
#pragma unroll
    for (int ii = 0; ii < 4; ++ii)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + e_row + 32 * (r >> 2) + 4 * (r & 3) + ii;
        float4 *hp = reinterpret_cast<float4 *>(p.H + (int64_t)row * K + n0 + e_col);
        float4 h = *hp;
        h.x += acc[ii][0][r]; h.y += acc[ii][1][r]; h.z += acc[ii][2][r]; h.w += acc[ii][3][r];
        *hp = h;
      }
  } else if (PIECES) {
    // a partial tile is the workgroup's first piece (slot 2 w) or, whole tiles in between, its last.  It is
    // stored in register order (16 bytes per lane, 1 KB per store instruction: float4 number
    // ((wave * 16 + ii * 4 + j) * 4 + r / 4) * 64 + lane), which is the order syrk_reduce_pieces_kernel sums in.
    float4 *dst = reinterpret_cast<float4 *>(p.ws + (int64_t)(2 * item + (first_piece ? 0 : 1)) * (W16_TB * W16_TB)) +
                  wave * 4096 + lane;
#pragma unroll
    for (int ii = 0; ii < 4; ++ii)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int rq = 0; rq < 4; ++rq)
          dst[((ii * 4 + j) * 4 + rq) * 64] =
              make_float4(acc[ii][j][4 * rq], acc[ii][j][4 * rq + 1], acc[ii][j][4 * rq + 2], acc[ii][j][4 * rq + 3]);
  } else {
    float *dst = p.ws + ((int64_t)rs * ntiles + t) * (W16_TB * W16_TB);
#pragma unroll
    for (int ii = 0; ii < 4; ++ii)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = e_row + 32 * (r >> 2) + 4 * (r & 3) + ii;
        *reinterpret_cast<float4 *>(dst + row * W16_TB + e_col) =
            make_float4(acc[ii][0][r], acc[ii][1][r], acc[ii][2][r], acc[ii][3][r]);
      }
  }
  if (!PIECES) break;
  first_piece = false;
  __syncthreads();           // the next piece's loads reuse the slab buffers
  } while (u0 < u1);
}

// PIECES form of the reduction: the partial tiles of tile t lie in the slots of the workgroups whose runs cut it
// (see syrk32d_kernel); H tile += their sum in workgroup order.  A tile that one workgroup covered alone has
// been added already.  G workgroups, S slabs per tile.  PERM: the accumulators' rows and columns as
// syrk32d_kernel deals them (a lane's four column blocks are adjacent columns, its rows four apart).
template <bool PERM>
__global__ __launch_bounds__(256) void syrk_reduce_pieces_kernel(float *H, const float *ws, int K, int T, int S, int G) {
  constexpr int TB = W16_TB, RED_PARTS = TB * TB / 4096;
  const int ntiles = T * (T + 1) / 2;
  const int t = blockIdx.x / RED_PARTS, part = blockIdx.x % RED_PARTS;
  const int64_t U = (int64_t)ntiles * S, lo = (int64_t)t * S, hi = lo + S;
  // first workgroup whose run [w U / G, (w + 1) U / G) reaches into [lo, hi)
  int w = (int)(lo * G / U);
  while (w > 0 && (int64_t)w * U / G > lo) --w;
  while ((int64_t)(w + 1) * U / G <= lo) ++w;
  if ((int64_t)w * U / G <= lo && (int64_t)(w + 1) * U / G >= hi) return;     // whole tile, one workgroup
  int ti, tj;
  tile_decode(t, T, ti, tj);
  const int m0 = ti * TB, n0 = tj * TB;
  // float4 number e of a partial tile holds the accumulator's registers r .. r + 3 of one lane (the kernel's
  // register order): e = (((wave * 4 + ii) * 4 + j) * 4 + r / 4) * 64 + lane; a thread's four numbers are j = 0 .. 3.
  // Plain order: rows row .. row + 3 of column block j.  PERM: column j of the lane's four adjacent columns, rows
  // row, row + 4, row + 8, row + 12 - the thread reads and writes H in rows of 16 bytes.
  float4 s[4], h[4];
  int e[4];
  float *hp[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    e[u] = part * 1024 + u * 256 + threadIdx.x;
    s[u] = make_float4(0.f, 0.f, 0.f, 0.f);
    const int lane = e[u] & 63, rq = (e[u] >> 6) & 3, j = (e[u] >> 8) & 3, ii = (e[u] >> 10) & 3, wv = e[u] >> 12;
    if (PERM) {
      // u-th of the thread's four rows, its four columns
      const int row = (wv >> 1) * 128 + 32 * rq + 16 * (lane >> 5) + 4 * u + ii, col = (wv & 1) * 128 + 4 * (lane & 31);
      hp[u] = H + (int64_t)(m0 + row) * K + n0 + col;
      h[u] = *reinterpret_cast<const float4 *>(hp[u]);
    } else {
      const int row = (wv >> 1) * 128 + ii * 32 + 8 * rq + 4 * (lane >> 5), col = (wv & 1) * 128 + j * 32 + (lane & 31);
      hp[u] = H + (int64_t)(m0 + row) * K + n0 + col;
      h[u] = make_float4(hp[u][0], hp[u][K], hp[u][2 * (int64_t)K], hp[u][3 * (int64_t)K]);
    }
  }
  for (; w < G && (int64_t)w * U / G < hi; ++w) {
    const int64_t a = (int64_t)w * U / G;
    if ((int64_t)(w + 1) * U / G <= a) continue;      // an empty run wrote nothing
    const bool first = a >= lo;                       // the run starts inside this tile: its first piece
    const float4 *src = reinterpret_cast<const float4 *>(ws) + (int64_t)(2 * w + (first ? 0 : 1)) * (TB * TB / 4);
    float4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = src[e[u]];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      s[u].x += v[u].x; s[u].y += v[u].y; s[u].z += v[u].z; s[u].w += v[u].w;
    }
  }
  if (PERM) {
    // s[j] holds column j of rows 0 .. 3 (of the thread's four): transposed on the way out
    *reinterpret_cast<float4 *>(hp[0]) = make_float4(h[0].x + s[0].x, h[0].y + s[1].x, h[0].z + s[2].x, h[0].w + s[3].x);
    *reinterpret_cast<float4 *>(hp[1]) = make_float4(h[1].x + s[0].y, h[1].y + s[1].y, h[1].z + s[2].y, h[1].w + s[3].y);
    *reinterpret_cast<float4 *>(hp[2]) = make_float4(h[2].x + s[0].z, h[2].y + s[1].z, h[2].z + s[2].z, h[2].w + s[3].z);
    *reinterpret_cast<float4 *>(hp[3]) = make_float4(h[3].x + s[0].w, h[3].y + s[1].w, h[3].z + s[2].w, h[3].w + s[3].w);
    return;
  }
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    hp[u][0] = h[u].x + s[u].x;
    hp[u][K] = h[u].y + s[u].y;
    hp[u][2 * (int64_t)K] = h[u].z + s[u].z;
    hp[u][3 * (int64_t)K] = h[u].w + s[u].w;
  }
}

// H tile += unit * sum over the row slices, in slice order (unit: device scalar, 1 if null).
// A tile is cut into RED_PARTS pieces, one workgroup each, and a thread keeps the loads of all its
// elements of four slices in flight: the reduction reads RS partial copies of the upper triangle,
// which is HBM traffic worth the bandwidth (one workgroup per tile with one load in flight per
// thread took 0.47 ms for 13 slices at K = 4096; the bytes need 0.1 ms).
template <int TB>
__global__ __launch_bounds__(256) void syrk_reduce_kernel(float *H, const float *ws, int K, int T,
                                                          int RS, const float *unit_ptr) {
  constexpr int RED_PARTS = TB * TB / 4096;          // 4096 elements = 4 float4 per thread
  const float unit = unit_ptr ? *unit_ptr : 1.f;
  const int ntiles = T * (T + 1) / 2;
  const int t = blockIdx.x / RED_PARTS, part = blockIdx.x % RED_PARTS;
  int ti, tj;
  tile_decode(t, T, ti, tj);
  const int m0 = ti * TB, n0 = tj * TB;
  float4 s[4];
  int e[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    e[u] = part * 1024 + u * 256 + threadIdx.x;      // float4 index inside the tile
    s[u] = make_float4(0.f, 0.f, 0.f, 0.f);
  }
  const float4 *base = reinterpret_cast<const float4 *>(ws) + (int64_t)t * (TB * TB / 4);
  const int64_t slice_stride = (int64_t)ntiles * (TB * TB / 4);
  for (int rs0 = 0; rs0 < RS; rs0 += 4) {
    float4 v[4][4];
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int u = 0; u < 4; ++u)
        v[q][u] = (rs0 + q < RS) ? base[(int64_t)(rs0 + q) * slice_stride + e[u]] : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        s[u].x += v[q][u].x; s[u].y += v[q][u].y; s[u].z += v[q][u].z; s[u].w += v[q][u].w;
      }
  }
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int row = e[u] / (TB / 4), c4 = (e[u] % (TB / 4)) * 4;
    const int gr = m0 + row, gc = n0 + c4;
    if (gr >= K) continue;
    float *dst = H + (int64_t)gr * K + gc;
    if (gc + 3 < K && (K & 3) == 0) {
      float4 h = *reinterpret_cast<float4 *>(dst);
      h.x += s[u].x * unit; h.y += s[u].y * unit; h.z += s[u].z * unit; h.w += s[u].w * unit;
      *reinterpret_cast<float4 *>(dst) = h;
    } else {
      if (gc + 0 < K) dst[0] += s[u].x * unit;
      if (gc + 1 < K) dst[1] += s[u].y * unit;
      if (gc + 2 < K) dst[2] += s[u].z * unit;
      if (gc + 3 < K) dst[3] += s[u].w * unit;
    }
  }
}

// rows per row slice and launch (a multiple of 64, so that a cut batch keeps full slabs)
constexpr int64_t H_CHAIN_ROWS = 32768;

int pick_rs(int64_t K) {
  const int64_t T = ceil_div64(K, HB), ntiles = T * (T + 1) / 2;
  int64_t rs = ceil_div64(6144, ntiles);   // about eight waves of workgroups over 768 slots
  if (rs < 1) rs = 1;
  if (rs > 4) rs = (rs <= 8) ? 8 : H_RSMAX;   // multiples of 8 get the per-XCD slice mapping
  return (int)rs;
}

// Row slices of the wide 16-bit kernel: one workgroup per CU, so the number of work items should
// be close below a multiple of 256, with at least six rounds.
int pick_rs_wide(int64_t K, bool fp32_rows = false) {
  const int64_t T = ceil_div64(K, W16_TB), ntiles = T * (T + 1) / 2;
  int best = 1;
  double best_eff = 0.0;
  for (int rs = 1; rs <= 32; ++rs) {
    const double rounds = (double)(ntiles * rs) / 256.0;
    if (rounds < 6.0 && rs < 32) continue;
    const double eff = rounds / (double)ceil_div64(ntiles * rs, 256);
    if (eff > best_eff + 1e-9) { best_eff = eff; best = rs; }
    // (fp32 rows, up to 256 tiles: a fuller last round is worth more slices - K = 4096 with 15 instead of 13
    // slices, 7.97 instead of 6.91 rounds, measured 0.9 % faster; the workspace grows with the slices, so not
    // beyond, and the 16-bit kernels, whose partial tiles weigh more against their products, measured no gain)
    if (eff >= (fp32_rows && ntiles <= 256 ? 0.99 : 0.97)) break;
  }
  return best;
}
bool use_wide16(int64_t K) { return K >= 1024; }

// Row slices of one launch of a 256 x 256-tile kernel over `total_rows` rows.  pick_rs_wide(K) suits a
// long calibration set and sizes the workspace; a short call (one batch per call, the reference's
// streaming use, gptq.py:97-98) pays a fixed cost per round of workgroups (pipeline fill, 64 MB of
// partial tiles written and read again), so fewer, longer slices win there.  Model fitted to
// measurements at K = 4096 (2048 rows per call, 1 .. 13 slices, within 5 %):
//   time = rounds * (us_per_row * rows_per_slice + 30 us),  rounds = ceil(tiles * slices / 256 CUs).
int pick_rs_call(int64_t K, int64_t total_rows, int slab_rows, double us_per_row, bool fp32_rows) {
  const int rs_max = pick_rs_wide(K, fp32_rows);
  const int64_t T = ceil_div64(K, W16_TB), ntiles = T * (T + 1) / 2;
  int best = rs_max;
  double best_cost = 0.0;
  for (int rs = rs_max; rs >= 1; --rs) {
    // fewer workgroups than CUs: each is bound by the latency of its own loads (measured slower
    // than the model at one slice of 136 tiles)
    if (ntiles * rs < 256 && rs < rs_max) break;
    const int64_t rows = round_up64(ceil_div64(total_rows, rs), slab_rows);
    const double cost = (double)ceil_div64(ntiles * rs, 256) * (us_per_row * (double)rows + 30.0);
    if (rs == rs_max || cost < 0.97 * best_cost) { best = rs; best_cost = cost; }
  }
  return best;
}
constexpr double H_US_PER_ROW_F32 = 0.228, H_US_PER_ROW_16 = 0.0305;

// The (tile, slab) runs of syrk32d_kernel<true> and of syrk16d_kernel<.., true> (slabs of slab_rows rows): G
// workgroups (one round), two partial-tile slots each.  A run is one chain of MFMA accumulations, so the call may
// not be longer than H_CHAIN_ROWS rows (see gptq_hip_hessian_accumulate); runs shorter than eight slabs are not
// worth their pipeline fill.
struct PiecesPlan { bool use; int G; size_t ws_bytes; };
PiecesPlan pieces_plan(int64_t K, int64_t total_rows, int slab_rows) {
  PiecesPlan pp{false, 0, 0};
  if (!use_wide16(K) || K % W16_TB != 0 || total_rows <= 0 || total_rows % slab_rows != 0 || total_rows > H_CHAIN_ROWS)
    return pp;
  const int64_t T = K / W16_TB, nt = T * (T + 1) / 2, U = nt * (total_rows / slab_rows);
  int64_t G = U / 8;
  if (G > 256) G = 256;
  if (G < 1) return pp;
  pp.use = true;
  pp.G = (int)G;
  pp.ws_bytes = (size_t)(2 * G) * W16_TB * W16_TB * sizeof(float);
  return pp;
}

// ---------------------------------------------------------------------------- fp32 rows on the 16-bit matrix cores
// Opt-in path for fp32 calibration rows: x = (hi + lo) * 2^e with hi = fp16(x 2^-e), lo =
// fp16(x 2^-e - hi), e chosen so that the largest magnitude of the call lands in [2^14, 2^15).
// hi + lo carries 22 mantissa bits of x (fewer only for entries more than 2^18 below the largest),
// all products of two fp16 numbers are exact in the fp32 accumulators, and
//   X^T X = 4^e (hi^T hi + hi^T lo + lo^T hi)  up to lo^T lo (relative 2^-22 per product).
// The three products are one launch of the two-matrix 16-bit kernel over the batch pairs
// (hi, hi), (hi, lo), (lo, hi): three times the 16-bit work instead of fp32 MFMAs at a
// sixteenth of the rate (K = 4096, 262144 rows: 15.7 ms against 35.4 ms).  Steps: largest magnitude of all batches (one read of X), then per
// group of batches split into two fp16 planes (workspace), multiply, and at the end one reduction
// that applies 4^e.  No host synchronisation: e lives in device memory.
struct SplitScalars { uint32_t amax_bits; float down, unit; };

__global__ void split_reset_kernel(SplitScalars *sc) {
  sc->amax_bits = 0u;
  sc->down = 1.f;
  sc->unit = 1.f;
}

// largest finite |x| over the batches of the table (grid: blocks x batches)
__global__ __launch_bounds__(256) void split_absmax_kernel(SyrkArgs p, SplitScalars *sc) {
  const int b = blockIdx.y;
  const float4 *x = reinterpret_cast<const float4 *>(p.ptr[b]);
  const int64_t n4 = (int64_t)p.rows[b] * p.K / 4;
  float m = 0.f;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (int64_t)gridDim.x * 256) {
    const float4 v = x[i];
    const float a = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    // fmaxf drops NaN operands; infinities are left out, too (they reach H through the planes)
    m = (a <= 3.4028235e38f) ? fmaxf(m, a) : m;
  }
  for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
  if ((threadIdx.x & 63) == 0 && m > 0.f) atomicMax(&sc->amax_bits, __float_as_uint(m));
}

__global__ void split_scale_kernel(SplitScalars *sc) {
  const float amax = __uint_as_float(sc->amax_bits);
  int ex = 0;
  (void)frexpf(amax, &ex);                       // 2^(ex-1) <= amax < 2^ex
  int e = amax > 0.f ? ex - 15 : 0;
  e = e < -60 ? -60 : (e > 60 ? 60 : e);         // 2^-e and 4^e stay normal fp32 numbers
  sc->down = ldexpf(1.f, -e);
  sc->unit = ldexpf(1.f, 2 * e);
}

// planes: rows of the table's batches one after the other, [row][K] fp16 each
__global__ __launch_bounds__(256) void split_planes_kernel(SyrkArgs p, const SplitScalars *sc, __half *hi,
                                                           __half *lo) {
  const int b = blockIdx.y;
  int64_t row0 = 0;
  for (int i = 0; i < b; ++i) row0 += p.rows[i];
  const float down = sc->down;
  const float4 *x = reinterpret_cast<const float4 *>(p.ptr[b]);
  const int64_t n4 = (int64_t)p.rows[b] * p.K / 4, o4 = row0 * p.K / 4;
  typedef _Float16 h4 __attribute__((ext_vector_type(4)));
  h4 *dh = reinterpret_cast<h4 *>(hi) + o4, *dl = reinterpret_cast<h4 *>(lo) + o4;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (int64_t)gridDim.x * 256) {
    const float4 v = x[i];
    const float s[4] = {v.x * down, v.y * down, v.z * down, v.w * down};
    h4 h, l;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      h[c] = (_Float16)s[c];
      l[c] = (_Float16)(s[c] - (float)h[c]);     // the difference is exact in fp32
    }
    dh[i] = h;
    dl[i] = l;
  }
}

constexpr int SPLIT_BATCHES = H_NBMAX / 3;        // real batches per launch (three table entries each)

struct SplitPlan {
  int64_t cap_rows;            // rows of a batch group (one launch)
  int rs, T;
  size_t part_bytes, sc_off, hi_off, lo_off, total_bytes;
};

SplitPlan split_plan(int64_t K, int64_t max_batch_rows) {
  SplitPlan p{};
  p.T = (int)ceil_div64(K, W16_TB);
  const int64_t nt = (int64_t)p.T * (p.T + 1) / 2;
  p.rs = pick_rs_wide(K);
  p.part_bytes = p.rs == 1 ? 0 : (size_t)p.rs * nt * W16_TB * W16_TB * sizeof(float);
  int64_t cap = ((int64_t)1 << 29) / K / D16_BK * D16_BK;     // planes of about 1 GB each
  if (cap < max_batch_rows) cap = max_batch_rows;
  p.cap_rows = cap;
  p.sc_off = (p.part_bytes + 255) & ~(size_t)255;
  p.hi_off = p.sc_off + 256;
  const size_t plane = (((size_t)cap * K * sizeof(__half)) + 255) & ~(size_t)255;
  p.lo_off = p.hi_off + plane;
  p.total_bytes = p.lo_off + plane;
  return p;
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
  // enough for either kernel (which one runs depends on the element type of the batches)
  const int rs = pick_rs(K);
  const int64_t T = ceil_div64(K, HB), ntiles = T * (T + 1) / 2;
  size_t need = rs == 1 ? 0 : (size_t)rs * ntiles * HB * HB * sizeof(float);
  if (use_wide16(K)) {
    const int rw = pick_rs_wide(K, true);      // fp32 rows take at least as many slices as 16-bit rows
    const int64_t Tw = ceil_div64(K, W16_TB), nw = Tw * (Tw + 1) / 2;
    const size_t wide = rw == 1 ? 0 : (size_t)rw * nw * W16_TB * W16_TB * sizeof(float);
    if (wide > need) need = wide;
    const size_t pieces = (size_t)512 * W16_TB * W16_TB * sizeof(float);     // pieces_plan: two slots x 256 workgroups
    if (pieces > need) need = pieces;
  }
  return need;
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
  // One launch sums its rows in registers, one chain of MFMA accumulations per row slice.  The
  // matrix instructions align their addends to the running sum with a few guard bits and drop
  // what falls below them, which biases a long sum of squares (the diagonal of H) low: measured
  // 5.5e-5 relative after 262144 rows in one chain, 4e-6 after 20000.  So a launch gets at most
  // H_CHAIN_ROWS rows per slice; longer calibration sets (and longer single batches) are cut
  // into several launches that add into H, as the reference adds batch by batch (gptq.py:97-98).
  const int rs_k = (use_wide16(K) && x_dtype != GPTQ_HIP_F64) ? pick_rs_wide(K, x_dtype == GPTQ_HIP_F32) : pick_rs(K);
  const int64_t launch_rows = (int64_t)H_CHAIN_ROWS * rs_k;
  int b0 = 0;
  int64_t off = 0;                 // rows of batch b0 already handed to a launch
  const size_t x_elem = dtype_size(x_dtype);
  while (b0 < n_batches) {
    SyrkArgs a;
    a.nb = 0;
    int64_t max_rows = 0, sum_rows = 0;
    while (b0 < n_batches && a.nb < H_NBMAX && sum_rows < launch_rows) {
      const int64_t rows = x_rows[b0];
      if (rows < 0 || rows > 2147483647LL) return GPTQ_HIP_EINVAL;
      if (rows - off > 0) {
        if (!x_ptrs[b0]) return GPTQ_HIP_EINVAL;
        int64_t take = rows - off;
        if (take > launch_rows - sum_rows) take = launch_rows - sum_rows;     // a multiple of 64 rows
        a.ptr[a.nb] = reinterpret_cast<const char *>(x_ptrs[b0]) + (size_t)off * (size_t)K * x_elem;
        a.rows[a.nb] = (int)take;
        ++a.nb;
        sum_rows += take;
        if (take > max_rows) max_rows = take;
        off += take;
      }
      if (off >= rows) {
        ++b0;
        off = 0;
      }
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
    // fp16 / bf16 batches: the 16-bit MFMA kernel, if every batch is 16-byte aligned
    bool mfma16 = (x_dtype == GPTQ_HIP_F16 || x_dtype == GPTQ_HIP_BF16) && K % 8 == 0;
    for (int i = 0; i < a.nb && mfma16; ++i)
      mfma16 = (reinterpret_cast<uintptr_t>(a.ptr[i]) & 15) == 0;
    if (mfma16 && use_wide16(K)) {
      int64_t total_rows = 0;
      for (int i = 0; i < a.nb; ++i) total_rows += a.rows[i];
      SyrkArgs w = a;
      w.T = (int)ceil_div64(K, W16_TB);
      const int64_t nt = (int64_t)w.T * (w.T + 1) / 2;
      w.RS = pick_rs_call(K, total_rows, W16_BK, H_US_PER_ROW_16, false);
      const int64_t slabs = ceil_div64(total_rows, W16_BK);
      if (w.RS > slabs) w.RS = (int)(slabs > 0 ? slabs : 1);
      const int64_t chunk = round_up64(ceil_div64(total_rows, w.RS), W16_BK);
      if (chunk > 2147483647LL) return GPTQ_HIP_EINVAL;
      w.chunk = (int)chunk;
      // all slabs full and no feature past K: loads go straight into LDS
      bool regular = (K % W16_TB == 0);
      for (int i = 0; i < w.nb; ++i) regular = regular && (w.rows[i] % D16_BK == 0);
      const bool f16 = x_dtype == GPTQ_HIP_F16;
      // a short call: equal runs of (tile, slab) pairs over one round of workgroups, as for fp32 batches below.
      // Measured against the row slices (512 .. 4096 rows per call): 10 - 50 % faster up to K = 4608 (171 tiles,
      // where no number of slices fills the rounds), slower from K = 5120 on: no two workgroups of a run
      // partition are at the same rows at the same time, every one streams its own pair of panels, and at the
      // rate of these matrix instructions the reads of X then bound the kernel.  (Fewer runs than tiles: a very
      // short call, one workgroup per tile is better.)
      const PiecesPlan pp = (regular && nt <= 171) ? pieces_plan(K, total_rows, D16_BK) : PiecesPlan{false, 0, 0};
      if (pp.use && pp.G >= nt && ws && ws_bytes >= pp.ws_bytes) {
        const void *pfn = f16 ? reinterpret_cast<const void *>(syrk16d_kernel<__half, SyrkArgs, true>)
                              : reinterpret_cast<const void *>(syrk16d_kernel<__hip_bfloat16, SyrkArgs, true>);
        if (!gptq_raise_lds_limit(pfn, D16_LDS_BYTES)) return GPTQ_HIP_ELAUNCH;
        const int64_t s32 = total_rows / D16_BK;
        w.chunk = (int)s32;
        if (f16)
          hipLaunchKernelGGL((syrk16d_kernel<__half, SyrkArgs, true>), dim3((unsigned)pp.G), block, D16_LDS_BYTES, st, w);
        else
          hipLaunchKernelGGL((syrk16d_kernel<__hip_bfloat16, SyrkArgs, true>), dim3((unsigned)pp.G), block, D16_LDS_BYTES,
                             st, w);
        GPTQ_CHECK_LAUNCH();
        hipLaunchKernelGGL(syrk_reduce_pieces_kernel<false>, dim3((unsigned)(nt * (W16_TB * W16_TB / 4096))), dim3(256), 0,
                           st, H, w.ws, (int)K, w.T, (int)s32, pp.G);
        GPTQ_CHECK_LAUNCH();
        continue;
      }
      const void *fn = regular ? (f16 ? reinterpret_cast<const void *>(syrk16d_kernel<__half, SyrkArgs>)
                                      : reinterpret_cast<const void *>(syrk16d_kernel<__hip_bfloat16, SyrkArgs>))
                               : (f16 ? reinterpret_cast<const void *>(syrk16w_kernel<__half>)
                                      : reinterpret_cast<const void *>(syrk16w_kernel<__hip_bfloat16>));
      const int lds_bytes = regular ? D16_LDS_BYTES : W16_LDS_BYTES;
      if (!gptq_raise_lds_limit(fn, lds_bytes)) return GPTQ_HIP_ELAUNCH;
      const dim3 wgrid((unsigned)(nt * w.RS));
      if (regular && f16)
        hipLaunchKernelGGL((syrk16d_kernel<__half, SyrkArgs>), wgrid, block, lds_bytes, st, w);
      else if (regular)
        hipLaunchKernelGGL((syrk16d_kernel<__hip_bfloat16, SyrkArgs>), wgrid, block, lds_bytes, st, w);
      else if (f16)
        hipLaunchKernelGGL(syrk16w_kernel<__half>, wgrid, block, lds_bytes, st, w);
      else
        hipLaunchKernelGGL(syrk16w_kernel<__hip_bfloat16>, wgrid, block, lds_bytes, st, w);
      GPTQ_CHECK_LAUNCH();
      if (w.RS > 1) {
        hipLaunchKernelGGL(syrk_reduce_kernel<W16_TB>, dim3((unsigned)(nt * (W16_TB * W16_TB / 4096))), dim3(256), 0, st, H, w.ws,
                           (int)K, w.T, w.RS, (const float *)nullptr);
        GPTQ_CHECK_LAUNCH();
      }
      continue;
    }
    if (mfma16) {
      int64_t total_rows = 0;
      for (int i = 0; i < a.nb; ++i) total_rows += a.rows[i];
      const int64_t chunk = round_up64(ceil_div64(total_rows, a.RS), S16_BK);
      if (chunk > 2147483647LL) return GPTQ_HIP_EINVAL;
      a.chunk = (int)chunk;
      const void *fn = x_dtype == GPTQ_HIP_F16
                           ? reinterpret_cast<const void *>(syrk16_kernel<__half>)
                           : reinterpret_cast<const void *>(syrk16_kernel<__hip_bfloat16>);
      if (!gptq_raise_lds_limit(fn, S16_LDS_BYTES)) return GPTQ_HIP_ELAUNCH;
      if (x_dtype == GPTQ_HIP_F16)
        hipLaunchKernelGGL(syrk16_kernel<__half>, grid, block, S16_LDS_BYTES, st, a);
      else
        hipLaunchKernelGGL(syrk16_kernel<__hip_bfloat16>, grid, block, S16_LDS_BYTES, st, a);
      GPTQ_CHECK_LAUNCH();
      if (a.RS > 1) {
        hipLaunchKernelGGL(syrk_reduce_kernel<HB>, dim3((unsigned)(ntiles * (HB * HB / 4096))), dim3(256), 0, st, H, a.ws,
                           (int)K, T, a.RS, (const float *)nullptr);
        GPTQ_CHECK_LAUNCH();
      }
      continue;
    }
    // fp32 batches, regular shapes from K = 1024 on: 256 x 256 tiles, loads straight into LDS
    bool wide32 = x_dtype == GPTQ_HIP_F32 && use_wide16(K) && K % W16_TB == 0 &&
                  ((reinterpret_cast<uintptr_t>(H) | reinterpret_cast<uintptr_t>(ws)) & 15) == 0;   // 16-byte accesses
    for (int i = 0; i < a.nb && wide32; ++i)
      wide32 = (a.rows[i] % D32_BK == 0) && ((reinterpret_cast<uintptr_t>(a.ptr[i]) & 15) == 0);
    if (wide32) {
      int64_t total_rows = 0;
      for (int i = 0; i < a.nb; ++i) total_rows += a.rows[i];
      SyrkArgs w = a;
      w.T = (int)(K / W16_TB);
      const int64_t nt = (int64_t)w.T * (w.T + 1) / 2;
      w.RS = pick_rs_call(K, total_rows, D32_BK, H_US_PER_ROW_F32, true);
      const int64_t slabs = total_rows / D32_BK;
      if (w.RS > slabs) w.RS = (int)(slabs > 0 ? slabs : 1);
      const int64_t chunk = round_up64(ceil_div64(total_rows, w.RS), D32_BK);
      if (chunk > 2147483647LL) return GPTQ_HIP_EINVAL;
      w.chunk = (int)chunk;
      // a short call: equal runs of (tile, slab) pairs over one round of workgroups instead of row slices,
      // where the model says so (time of a run + what the two partial tiles per workgroup cost)
      const PiecesPlan pp = pieces_plan(K, total_rows, D32_BK);
      if (pp.use && ws && ws_bytes >= pp.ws_bytes) {
        const double sliced = (double)ceil_div64(nt * w.RS, 256) * (H_US_PER_ROW_F32 * (double)chunk + 30.0);
        const double pieces = H_US_PER_ROW_F32 * (double)total_rows * (double)nt / (double)pp.G + 50.0;
        if (pieces < 0.9 * sliced) {
          if (!gptq_raise_lds_limit(reinterpret_cast<const void *>(syrk32d_kernel<true>), D32_LDS_BYTES))
            return GPTQ_HIP_ELAUNCH;
          w.chunk = (int)slabs;
          hipLaunchKernelGGL(syrk32d_kernel<true>, dim3((unsigned)pp.G), block, D32_LDS_BYTES, st, w);
          GPTQ_CHECK_LAUNCH();
          hipLaunchKernelGGL(syrk_reduce_pieces_kernel<true>, dim3((unsigned)(nt * (W16_TB * W16_TB / 4096))), dim3(256), 0,
                             st, H, w.ws, (int)K, w.T, (int)slabs, pp.G);
          GPTQ_CHECK_LAUNCH();
          continue;
        }
      }
      if (!gptq_raise_lds_limit(reinterpret_cast<const void *>(syrk32d_kernel<false>), D32_LDS_BYTES))
        return GPTQ_HIP_ELAUNCH;
      hipLaunchKernelGGL(syrk32d_kernel<false>, dim3((unsigned)(nt * w.RS)), block, D32_LDS_BYTES, st, w);
      GPTQ_CHECK_LAUNCH();
      if (w.RS > 1) {
        hipLaunchKernelGGL(syrk_reduce_kernel<W16_TB>, dim3((unsigned)(nt * (W16_TB * W16_TB / 4096))), dim3(256), 0, st, H, w.ws,
                           (int)K, w.T, w.RS, (const float *)nullptr);
        GPTQ_CHECK_LAUNCH();
      }
      continue;
    }
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
      hipLaunchKernelGGL(syrk_reduce_kernel<HB>, dim3((unsigned)(ntiles * (HB * HB / 4096))), dim3(256), 0, st, H, a.ws,
                         (int)K, T, a.RS, (const float *)nullptr);
      GPTQ_CHECK_LAUNCH();
    }
  }
  return GPTQ_HIP_OK;
}

size_t gptq_hip_hessian_accumulate_split16_workspace_bytes(int64_t K, int64_t max_batch_rows) {
  if (K <= 0 || K % W16_TB != 0 || max_batch_rows <= 0 || max_batch_rows % D16_BK != 0) return 0;
  return split_plan(K, max_batch_rows).total_bytes;
}

int gptq_hip_hessian_accumulate_split16(void *stream, const void *const *x_ptrs, const int64_t *x_rows,
                                        int n_batches, int64_t K, float *H, void *ws, size_t ws_bytes) {
  if (n_batches < 0 || K <= 0 || K > 46000 || !H) return GPTQ_HIP_EINVAL;
  if (n_batches > 0 && (!x_ptrs || !x_rows)) return GPTQ_HIP_EINVAL;
  if (K % W16_TB != 0) return GPTQ_HIP_EINVAL;
  int64_t max_rows = 0;
  for (int b = 0; b < n_batches; ++b) {
    const int64_t rows = x_rows[b];
    if (rows < 0 || rows > 2147483647LL || rows % D16_BK != 0) return GPTQ_HIP_EINVAL;
    if (rows > 0 && (!x_ptrs[b] || (reinterpret_cast<uintptr_t>(x_ptrs[b]) & 15))) return GPTQ_HIP_EINVAL;
    if (rows > max_rows) max_rows = rows;
  }
  if (max_rows == 0) return GPTQ_HIP_OK;
  const SplitPlan sp = split_plan(K, max_rows);
  if (!ws || ws_bytes < sp.total_bytes || (reinterpret_cast<uintptr_t>(ws) & 15)) return GPTQ_HIP_EWORKSPACE;
  hipStream_t st = as_stream(stream);
  char *base = reinterpret_cast<char *>(ws);
  SplitScalars *sc = reinterpret_cast<SplitScalars *>(base + sp.sc_off);
  __half *hi = reinterpret_cast<__half *>(base + sp.hi_off), *lo = reinterpret_cast<__half *>(base + sp.lo_off);

  // ---- largest magnitude over all batches -> e
  hipLaunchKernelGGL(split_reset_kernel, dim3(1), dim3(1), 0, st, sc);
  GPTQ_CHECK_LAUNCH();
  for (int b0 = 0; b0 < n_batches;) {
    SyrkArgs a;
    a.nb = 0;
    a.K = (int)K;
    while (b0 < n_batches && a.nb < H_NBMAX) {
      if (x_rows[b0] > 0) {
        a.ptr[a.nb] = x_ptrs[b0];
        a.rows[a.nb] = (int)x_rows[b0];
        ++a.nb;
      }
      ++b0;
    }
    if (a.nb == 0) continue;
    hipLaunchKernelGGL(split_absmax_kernel, dim3(64, (unsigned)a.nb), dim3(256), 0, st, a, sc);
    GPTQ_CHECK_LAUNCH();
  }
  hipLaunchKernelGGL(split_scale_kernel, dim3(1), dim3(1), 0, st, sc);
  GPTQ_CHECK_LAUNCH();

  // ---- groups of batches: split, multiply into the partial tiles (or into H when there is one slice)
  const void *fn = reinterpret_cast<const void *>(syrk16d_kernel<__half, SyrkArgsDual>);
  if (!gptq_raise_lds_limit(fn, D16_LDS_BYTES)) return GPTQ_HIP_ELAUNCH;
  const int64_t nt = (int64_t)sp.T * (sp.T + 1) / 2;
  // batches per launch: as even as the table allows (a short last launch costs as much per
  // workgroup as a long one)
  int n_real = 0;
  for (int b = 0; b < n_batches; ++b) n_real += x_rows[b] > 0 ? 1 : 0;
  const int n_groups = (n_real + SPLIT_BATCHES - 1) / SPLIT_BATCHES;
  const int per_group = (n_real + n_groups - 1) / n_groups;
  bool first = true;
  for (int b0 = 0; b0 < n_batches;) {
    SyrkArgs src;
    src.nb = 0;
    src.K = (int)K;
    int64_t rows_total = 0;
    while (b0 < n_batches && src.nb < per_group) {
      const int64_t rows = x_rows[b0];
      if (rows > 0) {
        if (rows_total + rows > sp.cap_rows) break;      // (a single batch always fits)
        src.ptr[src.nb] = x_ptrs[b0];
        src.rows[src.nb] = (int)rows;
        ++src.nb;
        rows_total += rows;
      }
      ++b0;
    }
    if (src.nb == 0) continue;
    hipLaunchKernelGGL(split_planes_kernel, dim3(256, (unsigned)src.nb), dim3(256), 0, st, src, sc, hi, lo);
    GPTQ_CHECK_LAUNCH();
    SyrkArgsDual w;
    w.nb = 3 * src.nb;
    w.K = (int)K;
    w.T = sp.T;
    w.RS = sp.rs;
    w.H = H;
    w.ws = reinterpret_cast<float *>(base);
    w.factor = &sc->unit;
    w.accum = first ? 0 : 1;
    int64_t row0 = 0;
    for (int i = 0; i < src.nb; ++i) {
      const __half *h = hi + row0 * K, *l = lo + row0 * K;
      w.ptr[3 * i] = h;      w.ptrB[3 * i] = h;
      w.ptr[3 * i + 1] = h;  w.ptrB[3 * i + 1] = l;
      w.ptr[3 * i + 2] = l;  w.ptrB[3 * i + 2] = h;
      w.rows[3 * i] = w.rows[3 * i + 1] = w.rows[3 * i + 2] = src.rows[i];
      row0 += src.rows[i];
    }
    const int64_t total_rows = 3 * rows_total;
    // (slices past the end of a short group get no slab and contribute zeros)
    const int64_t chunk = round_up64(ceil_div64(total_rows, w.RS), W16_BK);
    if (chunk > 2147483647LL) return GPTQ_HIP_EINVAL;
    w.chunk = (int)chunk;
    hipLaunchKernelGGL((syrk16d_kernel<__half, SyrkArgsDual>), dim3((unsigned)(nt * w.RS)), dim3(256),
                       D16_LDS_BYTES, st, w);
    GPTQ_CHECK_LAUNCH();
    first = false;
  }
  if (!first && sp.rs > 1) {
    hipLaunchKernelGGL(syrk_reduce_kernel<W16_TB>, dim3((unsigned)(nt * (W16_TB * W16_TB / 4096))), dim3(256), 0, st, H,
                       reinterpret_cast<const float *>(base), (int)K, sp.T, sp.rs, &sc->unit);
    GPTQ_CHECK_LAUNCH();
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
