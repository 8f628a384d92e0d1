// Packed-weight matmul, forward, 4-bit codes, 17 to a few hundred rows:
//   out[M, C] = x[M, K] @ ((code - zero) * scale)
// on tall, narrow output tiles whose eight wavefronts split the contraction.
//
// With a few dozen rows the product is neither a decode (the activations are no longer negligible) nor a GEMM (the
// output has too few tiles for 256 CUs).  A workgroup owns all rows of a row tile (16 RB rows, RB = 2 or 4) and 64
// channels over all of K or one of S ranges of k-steps:
//   * a weight operand register is dequantised once per workgroup and feeds RB MFMAs;
//   * eight wavefronts, two per SIMD; wavefront w takes k-step 8 j + w of stage j, and the eight accumulator sets
//     are summed through LDS at the end;
//   * the activations of a stage (16 RB rows x 256 k) are shared: fetched with 512-byte row segments (a direct load
//     of an operand fragment touches sixteen rows with 64 bytes each, which costs the address unit four times as
//     much) into registers and laid into LDS, rows 528 bytes apart so that the sixteen rows of an operand read fall
//     on different banks.  KS stages lie between two workgroup barriers (two buffers of KS stages; as many as
//     the LDS holds: the barrier and the latencies around it cost as much as a stage of a 32-row tile);
//   * B: a k-step's 16 packed rows x 64 bytes are fetched with ONE 16-byte load per lane (the address unit takes
//     as long over a 4-byte load as over a 16-byte one), lane L taking chunk L % 4 of row L / 4, and turned into
//     the operand layout (a lane's four rows of four channels each) through 1 KB of LDS that only this wavefront
//     touches: four 4-byte stores and one 16-byte load per lane, no barrier (a wavefront's LDS operations
//     execute in order).  Lane l16 then owns the channels c0 + 4 l16 .. + 3.  The low and the high nibbles of a
//     row's four channels are masked in place (two instructions per row), a byte permute puts a channel's pair
//     into the two halves of a register as fp16 subnormals {lo 2^-24, 16 hi 2^-24}, and one packed fma turns
//     that into (code - zero) 2^-9, both codes exact (the zero point with fp16's relative precision): 2.5
//     instructions per operand register, no row sums; the epilogue multiplies by 512 scale.
// Loads return to a wavefront in the order of their issue, so whoever waits for a stage of activations also waits
// for every weight load issued before it: within a stage the weights go out first and the activations last.
// S > 1: partial tiles through the workspace and an arrival ticket, summed in split order by the last
// workgroup, as in the register-operand kernels.
//
// What bounds it: every workgroup reads all of its rows' activations from L2 (C / 64 workgroups x 2 M K bytes:
// 44 MB at M = 32 on 4096 x 11008, twice the weights), which is why the dispatcher takes it up to 64 rows
// (128 on small matrices) and leaves more rows to the 64 x 128 and 128 x 128 tiles.
//
// bf16 activations: the operand registers are 128 + code (a byte permute and an or under 0x4300: exact in bf16),
// the term (128 + zero) sum_k x[m][k] leaves in the epilogue; the row sums come from one more MFMA per row block and
// k-step against a vector of ones (the matrix pipe is mostly idle here) and are summed over the wavefronts with
// the tiles.  A split applies the term to its own partial sums before it hands them over (it is linear in them).
//
// Shapes: K % 256 == 0 (whole stages), C % 16 == 0, operands 16-byte aligned, per-channel parameters, fp16 or bf16
// activations (fp32 rows through the fp16 staging of the dispatcher: out32 / rowexp).
#include "qmatmul_reg.h"
#include "qmm_reg_common.h"
#include <type_traits>

namespace {

using namespace qmm;

constexpr int MID_WAVES = 8;
constexpr int MID_TPB = 64 * MID_WAVES;
constexpr int MID_PITCH = 528;            // bytes between two rows of a stage in LDS (512 of data)
constexpr int MID_STAGE_K = 32 * MID_WAVES;

// Elements first .. first + NB - 1 (indices clamped to n - 1) of a zero / scale vector as raw bits (16-bit types
// zero-extended): the element type is switched on once around independent loads, and nothing waits for them here.
template <int NB>
__device__ __forceinline__ void mid_params_raw(const void *p, int dtype, int first, int n, uint32_t (&out)[NB]) {
  int idx[NB];
#pragma unroll
  for (int i = 0; i < NB; ++i) idx[i] = min(first + i, n - 1);
  if (dtype == GPTQ_HIP_F32) {
    const uint32_t *q = reinterpret_cast<const uint32_t *>(p);
#pragma unroll
    for (int i = 0; i < NB; ++i) out[i] = q[idx[i]];
  } else {
    const uint16_t *q = reinterpret_cast<const uint16_t *>(p);
#pragma unroll
    for (int i = 0; i < NB; ++i) out[i] = q[idx[i]];
  }
}

// Row blocks per pass of the final reduction: the eight wavefronts' tiles of a pass fit 128 KB of LDS
constexpr int mid_rbt(int nb, int rb) {
  int r = rb;
  while (r > 1 && r * nb > 16) r /= 2;
  return r;
}

template <typename TX, int RB, int WR, int KS>
__global__ __launch_bounds__(MID_TPB) void qmm_fwd_mid_kernel(const TX *x, int M, int K, const uint8_t *pk, int R,
                                                             int C, const void *zero, const void *scale, int zs_dtype,
                                                             TX *out, float *part, int32_t *counters, int S,
                                                             int steps_per_split, int tiles_x, int tiles_y, float *out32,
                                                             const int32_t *rowexp) {
  constexpr bool BF = Act<TX>::BF;
  constexpr int NB = 4;                          // 16-channel blocks per tile
  constexpr int ROWS = 16 * RB;
  constexpr int BUF = ROWS * MID_PITCH;          // one stage
  constexpr int BUFK = KS * BUF;                 // one buffer: the KS stages between two barriers
  constexpr int RBT = mid_rbt(NB, RB);           // row blocks per pass of the final reduction
  constexpr int NP = RB / RBT;
  extern __shared__ __attribute__((aligned(16))) unsigned char mid_lds[];
  __shared__ int s_flag;
  asm volatile("" ::"s"(x), "s"(pk), "s"(zero), "s"(scale), "s"(out), "s"(part), "s"(counters), "s"(M), "s"(K), "s"(R),
               "s"(C), "s"(zs_dtype), "s"(S), "s"(steps_per_split));
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int g = lane >> 4, l16 = lane & 15;
  // Workgroups are dealt to the 8 XCDs round-robin in dispatch order, and each XCD has its own L2.  A tile's
  // weight rows are 64 bytes long, half a cache line, so XCD j (workgroup ids j, j + 8, ...) takes a contiguous
  // range of work items, in which column tiles are adjacent: the lines that neighbouring tiles share are then
  // fetched into one L2, not into two.
  int tx, ty, split;
  {
    const int total = gridDim.x, j = blockIdx.x & 7, k = blockIdx.x >> 3, q = total >> 3, rem = total & 7;
    const int item = j * q + min(j, rem) + k;
    tx = item % tiles_x;
    ty = (item / tiles_x) % tiles_y;
    split = item / (tiles_x * tiles_y);
  }
  const int m0 = ty * ROWS, c0 = tx * (16 * NB);
  const int T = K >> 5;
  const int t_begin = split * steps_per_split, t_end = min(T, t_begin + steps_per_split);
  const int nst = (max(t_end - t_begin, 0) + MID_WAVES - 1) / MID_WAVES;       // stages (the plan keeps them whole)

  // ---- weights: row and 16-byte chunk of this lane's load, and where its four words go in the wavefront's LDS
  // region: word d of (row r, chunk q) belongs to lane 4 q + d of lane group r / 4 as its word r % 4; the position
  // within the group is rotated by four per group
  const int cr = lane >> 2, cq = lane & 3;
  const uint8_t *cp = pk + (int64_t)cr * C + min(c0 + 16 * cq, C - 16);
  unsigned char *const wl = mid_lds + 2 * BUFK + w * 1024;
  const int cwoff = ((cr >> 2) * 16 + ((4 * cq + 4 * (cr >> 2)) & 15)) * 16 + (cr & 3) * 4;
  const int croff = (g * 16 + ((l16 + 4 * g) & 15)) * 16;
  u32x4_t ring[WR];
  // (nothing in the loop is conditional: a stage past the last one re-reads the last one, valid memory that is
  // never multiplied.  With branches between the loads the compiler's wait counts fall back to "everything
  // outstanding", which turns the rings into one exposed memory latency per stage.)
  auto load_w = [&](int slot, int j) __attribute__((always_inline)) {
    const int t = t_begin + MID_WAVES * min(j, nst - 1) + w;
    ring[slot] = *reinterpret_cast<const u32x4_t *>(cp + (int64_t)(16 * t) * C);
  };
  // ---- activations: RB pieces of 16 bytes per thread and stage; piece i is row 16 i + tid / 32, chunk tid % 32
  const int chunk = tid & 31;
  int xoff[RB];
#pragma unroll
  for (int i = 0; i < RB; ++i) xoff[i] = min(m0 + 16 * i + (tid >> 5), M - 1) * K + 8 * chunk;      // M K < 2^31
  u32x4_t xr[KS][RB];
  auto load_x = [&](int q, int j) __attribute__((always_inline)) {
    const int k = 32 * (t_begin + MID_WAVES * min(j, nst - 1));
#pragma unroll
    for (int i = 0; i < RB; ++i) xr[q][i] = *reinterpret_cast<const u32x4_t *>(x + xoff[i] + k);
  };
  unsigned char *const xw = mid_lds + (tid >> 5) * MID_PITCH + 16 * chunk;
  auto store_x = [&](int q, int off) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < RB; ++i) *reinterpret_cast<u32x4_t *>(xw + off + i * (16 * MID_PITCH)) = xr[q][i];
  };
  const unsigned char *const xa = mid_lds + l16 * MID_PITCH + 64 * w + 16 * g;

  // zero points first (the first k-step's dequantisation needs them), then the first stages' loads
  const int col = c0 + 4 * l16;                  // this lane's channels col .. col + 3
  uint32_t zraw[NB], sraw[NB];
  mid_params_raw<NB>(zero, zs_dtype, col, C, zraw);
  mid_params_raw<NB>(scale, zs_dtype, col, C, sraw);
  __builtin_amdgcn_sched_barrier(0);
  load_x(0, 0);
#pragma unroll
  for (int u = 0; u < WR; ++u) load_w(u, u);
  __builtin_amdgcn_sched_barrier(0);
  uint32_t zneg[NB];
#pragma unroll
  for (int t = 0; t < NB; ++t) {
    const _Float16 h = (_Float16)(-rg_raw_to_f32(zraw[t], zs_dtype) * 0x1p-9f);
    zneg[t] = __builtin_bit_cast(uint32_t, half2_t{h, h});
  }
  const half2_t mul = half2_t{(_Float16)32768.f, (_Float16)2048.f};
  uint32_t c43 = 0x43004300u, one2 = 0x3F803F80u;
  asm volatile("" : "+v"(c43), "+v"(one2));
  floatx4 rsacc[RB];                             // bf16: sum_k x[m][k] of this wavefront's k-steps (every column alike)
#pragma unroll
  for (int i = 0; i < RB; ++i) rsacc[i] = floatx4{0.f, 0.f, 0.f, 0.f};

  floatx4 acc[RB][NB];
#pragma unroll
  for (int i = 0; i < RB; ++i)
#pragma unroll
    for (int t = 0; t < NB; ++t) acc[i][t] = floatx4{0.f, 0.f, 0.f, 0.f};

  // Register set q holds the stages s with s % KS == q; during stage j the rows of stage j + KS go to the other
  // buffer and those of stage j + 2 KS are fetched.  The operands of a stage are read from LDS while the stage
  // before it is multiplied, except across a barrier.
  uint4 a[KS > 1 ? 2 : 1][RB];
#pragma unroll
  for (int q = 1; q < KS; ++q) load_x(q, q);
#pragma unroll
  for (int q = 0; q < KS; ++q) {
    store_x(q, q * BUF);
    load_x(q, KS + q);
  }
  __syncthreads();

  auto stage = [&](int j, int u) __attribute__((always_inline)) {
    const int sub = u % KS, buf = (u / KS) & 1;                       // (the loop is unrolled by a multiple of 2 KS)
    constexpr int AS = KS > 1 ? 2 : 1;
    if (sub == 0) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
        a[0][rb] = *reinterpret_cast<const uint4 *>(xa + buf * BUFK + rb * (16 * MID_PITCH));
    }
    if (sub + 1 < KS) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
        a[(sub + 1) % AS][rb] =
            *reinterpret_cast<const uint4 *>(xa + buf * BUFK + (sub + 1) * BUF + rb * (16 * MID_PITCH));
    }
#pragma unroll
    for (int d = 0; d < 4; ++d) *reinterpret_cast<uint32_t *>(wl + cwoff + 16 * d) = ring[u % WR][d];
    const u32x4_t wv = *reinterpret_cast<const u32x4_t *>(wl + croff);
    __builtin_amdgcn_sched_barrier(0);
    load_w(u % WR, j + WR);
    __builtin_amdgcn_sched_barrier(0);
    uint32_t mlo[4], mhi[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      mlo[i] = wv[i] & 0x0F0F0F0Fu;
      mhi[i] = BF ? (wv[i] >> 4) & 0x0F0F0F0Fu : wv[i] & 0xF0F0F0F0u;
    }
#pragma unroll
    for (int t = 0; t < NB; ++t) {
      const uint32_t sel = 0x0c000c00u | ((uint32_t)(4 + t) << 16) | (uint32_t)t;
      uint32_t b4[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t pb = __builtin_amdgcn_perm(mhi[i], mlo[i], sel);     // fp16: {lo, 16 hi} as subnormals
        if constexpr (BF) {
          b4[i] = pb | c43;                                                   // {128 + lo, 128 + hi}
        } else {
          const half2_t d = __builtin_elementwise_fma(__builtin_bit_cast(half2_t, pb), mul,
                                                      __builtin_bit_cast(half2_t, zneg[t]));
          b4[i] = __builtin_bit_cast(uint32_t, d);
        }
      }
      const uint4 b = make_uint4(b4[0], b4[1], b4[2], b4[3]);
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) acc[rb][t] = Act<TX>::mma(a[sub % AS][rb], b, acc[rb][t]);
    }
    if constexpr (BF) {
      const uint4 ones = make_uint4(one2, one2, one2, one2);
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) rsacc[rb] = Act<TX>::mma(a[sub % AS][rb], ones, rsacc[rb]);
    }
    __builtin_amdgcn_sched_barrier(0);
    store_x(sub, (buf ^ 1) * BUFK + sub * BUF);
    load_x(sub, j + 2 * KS);
    if (sub == KS - 1) __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
  };
  // UN stages per trip (a multiple of 2 KS and of WR, so that buffer, register set and ring slot are
  // compile-time), then the remaining ones
  constexpr int UN = (2 * KS) % WR == 0 ? 2 * KS : WR;
  static_assert(UN % (2 * KS) == 0 && UN % WR == 0, "unroll count");
  int j0 = 0;
  for (; j0 + UN <= nst; j0 += UN) {
#pragma unroll
    for (int u = 0; u < UN; ++u) stage(j0 + u, u);
  }
#pragma unroll
  for (int u = 0; u < UN - 1; ++u)
    if (j0 + u < nst) stage(j0 + u, u);

  __syncthreads();                       // (the last stages may have ended without one)
  // ---- sum over the eight wavefronts (and the S workgroups of a split tile); wavefront q < RBT finishes row
  // block q of the pass
  float sc[NB], zoff[NB];
#pragma unroll
  for (int t = 0; t < NB; ++t) {
    sc[t] = rg_raw_to_f32(sraw[t], zs_dtype) * (BF ? 1.f : 512.f);
    zoff[t] = 128.f + rg_raw_to_f32(zraw[t], zs_dtype);
  }
  float *red = reinterpret_cast<float *>(mid_lds);      // [wavefront][row block of the pass][tile][lane][4]
  auto finish = [&](auto pc) __attribute__((always_inline)) {
    constexpr int P = decltype(pc)::value;
    const bool owner = w < RBT;
    const int rbo = owner ? w : 0;
    floatx4 rs = floatx4{0.f, 0.f, 0.f, 0.f};
    if constexpr (BF) {
      // the row sums first, through the same buffer
#pragma unroll
      for (int rb = 0; rb < RBT; ++rb)
        *reinterpret_cast<floatx4 *>(red + ((w * RBT + rb) * 64 + lane) * 4) = rsacc[P * RBT + rb];
      __syncthreads();
      if (owner) {
#pragma unroll
        for (int q = 0; q < MID_WAVES; ++q)
          rs += *reinterpret_cast<const floatx4 *>(red + ((q * RBT + rbo) * 64 + lane) * 4);
      }
      __syncthreads();
    }
#pragma unroll
    for (int rb = 0; rb < RBT; ++rb)
#pragma unroll
      for (int t = 0; t < NB; ++t)
        *reinterpret_cast<floatx4 *>(red + (((w * RBT + rb) * NB + t) * 64 + lane) * 4) = acc[P * RBT + rb][t];
    __syncthreads();
    floatx4 sum[NB];
#pragma unroll
    for (int t = 0; t < NB; ++t) {
      floatx4 v = floatx4{0.f, 0.f, 0.f, 0.f};
      if (owner) {
#pragma unroll
        for (int q = 0; q < MID_WAVES; ++q)
          v += *reinterpret_cast<const floatx4 *>(red + (((q * RBT + rbo) * NB + t) * 64 + lane) * 4);
      }
      sum[t] = v;
    }
    if constexpr (BF) {
      // sum_k x (128 + code) - (128 + zero) sum_k x, on this workgroup's range of k
#pragma unroll
      for (int t = 0; t < NB; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) sum[t][r] -= zoff[t] * rs[r];
    }
    if (S > 1) {
      const int tile = ((ty * NP + P) * tiles_x + tx);
      float *mine = part + ((((int64_t)tile * S + split) * RBT + rbo) * NB) * RG_TILE_FLOATS + lane * 4;
      if (owner) {
#pragma unroll
        for (int t = 0; t < NB; ++t) rg_store_part(mine + t * RG_TILE_FLOATS, sum[t]);
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");        // this wavefront's write-through stores have completed
      __syncthreads();
      if (tid == 0) {
        int32_t *ctr = counters + tile;
        const int ticket = __hip_atomic_fetch_add(ctr, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const int last = ticket == S - 1;
        if (last) __hip_atomic_store(ctr, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_flag = last;
      }
      __syncthreads();
      const bool last = s_flag != 0;
      if (P + 1 < NP) __syncthreads();                         // s_flag and red are free for the next pass
      if (!last || !owner) return;
      const float *src = part + (((int64_t)tile * S * RBT + rbo) * NB) * RG_TILE_FLOATS + lane * 4;
#pragma unroll
      for (int t = 0; t < NB; ++t) sum[t] = floatx4{0.f, 0.f, 0.f, 0.f};
      for (int sp = 0; sp < S; sp += 2) {
        floatx4 pv[2][NB];
#pragma unroll
        for (int f = 0; f < 2; ++f) {
          const int sq = min(sp + f, S - 1);
#pragma unroll
          for (int t = 0; t < NB; ++t)
            pv[f][t] = rg_load_part_issue(src + (int64_t)sq * (RBT * NB * RG_TILE_FLOATS) + t * RG_TILE_FLOATS);
        }
#pragma unroll
        for (int f = 0; f < 2; ++f)
#pragma unroll
          for (int t = 0; t < NB; ++t) asm volatile("s_waitcnt vmcnt(0)" : "+v"(pv[f][t]) : : "memory");
#pragma unroll
        for (int f = 0; f < 2; ++f)
          if (sp + f < S) {
#pragma unroll
            for (int t = 0; t < NB; ++t) sum[t] += pv[f][t];
          }
      }
    } else {
      if (P + 1 < NP) __syncthreads();                         // red is free for the next pass
      if (!owner) return;
    }
    // sum[t][r] = (fp16: 2^-9) sum_k x[m][k] (code - zero)[k][col + t], m = m0 + 16 (P RBT + rbo) + 4 g + r
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = m0 + 16 * (P * RBT + rbo) + 4 * g + r;
      if (m >= M) continue;
      const bool whole = c0 + 16 * NB <= C;                    // (uniform) every channel of the tile exists
      if constexpr (BF) {
        TX ob[NB];
#pragma unroll
        for (int t = 0; t < NB; ++t) ob[t] = Act<TX>::out(sc[t] * sum[t][r]);
        TX *dstb = out + (int64_t)m * C + col;
        if (whole) {
          *reinterpret_cast<uint2 *>(dstb) = *reinterpret_cast<const uint2 *>(ob);
        } else {
#pragma unroll
          for (int t = 0; t < NB; ++t)
            if (col + t < C) dstb[t] = ob[t];
        }
        continue;
      }
      _Float16 o[NB];
#pragma unroll
      for (int t = 0; t < NB; ++t) o[t] = (_Float16)(sc[t] * sum[t][r]);
      if (out32 != nullptr) {
        // fp32 rows: the fp16 result widened and scaled back by the row's power of two (exact)
        const int e = rowexp[m];
        float *d32 = out32 + (int64_t)m * C + col;
        if (whole) {
          *reinterpret_cast<float4 *>(d32) =
              make_float4(ldexpf((float)o[0], e), ldexpf((float)o[1], e), ldexpf((float)o[2], e), ldexpf((float)o[3], e));
        } else {
#pragma unroll
          for (int t = 0; t < NB; ++t)
            if (col + t < C) d32[t] = ldexpf((float)o[t], e);
        }
        continue;
      }
      __half *dst = reinterpret_cast<__half *>(out) + (int64_t)m * C + col;
      if (whole) {
        // (col % 4 == 0, C % 16 == 0, out 16-byte aligned)
        *reinterpret_cast<uint2 *>(dst) = make_uint2(__builtin_bit_cast(uint32_t, half2_t{o[0], o[1]}),
                                                     __builtin_bit_cast(uint32_t, half2_t{o[2], o[3]}));
      } else {
#pragma unroll
        for (int t = 0; t < NB; ++t)
          if (col + t < C) dst[t] = __builtin_bit_cast(__half, o[t]);
      }
    }
  };
  finish(std::integral_constant<int, 0>{});
  if constexpr (NP == 2) finish(std::integral_constant<int, 1>{});
}

template <typename TX, int RB>
int mid_launch_inst(hipStream_t st, const MidPlan &p, const void *x, int64_t M, const uint8_t *pk, int64_t R, int64_t C,
                    const void *zero, const void *scale, int zs_dtype, void *out, void *wsp) {
  // ring of weight k-steps (what the registers allow) and stages between two barriers (what the LDS holds twice)
  constexpr int WR = RB == 2 ? 8 : 4;
  constexpr int KS = RB == 2 ? 4 : 2;
  constexpr int RBT = mid_rbt(4, RB);
  constexpr size_t stage_bytes = (size_t)2 * KS * 16 * RB * MID_PITCH + (size_t)MID_WAVES * 1024;
  constexpr size_t red_bytes = (size_t)MID_WAVES * RBT * 4 * RG_TILE_FLOATS * sizeof(float);
  constexpr size_t lds = stage_bytes > red_bytes ? stage_bytes : red_bytes;
  auto kern = qmm_fwd_mid_kernel<TX, RB, WR, KS>;
  if (lds > 64 * 1024 && !gptq_raise_lds_limit(reinterpret_cast<const void *>(kern), (int)lds)) return GPTQ_HIP_ELAUNCH;
  int32_t *counters = reinterpret_cast<int32_t *>(wsp);
  float *part = reinterpret_cast<float *>(reinterpret_cast<char *>(wsp) + QMM_HEAD_BYTES);
  const dim3 grid((unsigned)(p.tiles_x * p.tiles_y * p.S));
  hipLaunchKernelGGL(kern, grid, dim3(MID_TPB), lds, st, (const TX *)x, (int)M, (int)(2 * R), pk, (int)R, (int)C, zero,
                     scale, zs_dtype, (TX *)out, part, counters, p.S, p.steps, (int)p.tiles_x, (int)p.tiles_y, p.out32, p.rowexp);
  GPTQ_CHECK_LAUNCH();
  return GPTQ_HIP_OK;
}

}  // namespace

namespace qmm {

MidPlan mid_fwd_plan(int64_t M, int64_t R, int64_t C, bool aligned, bool bf16) {
  MidPlan p{};
  p.bf16 = bf16;
  const int64_t K = 2 * R;
  if (!aligned || M < 17 || M > 256 || K % MID_STAGE_K != 0 || C % 16 != 0 || C < 64 || M * K >= (1LL << 31) ||
      R >= (1LL << 30) || C >= (1LL << 30))
    return p;
  // Where these tiles are the faster ones (measured against the 64 x 128 and 128 x 128 tiles of the register-operand
  // kernel: 4096 x 11008 at M = 32 19.5 -> 15.5 us, M = 64 21.6 -> 19 us, M = 128 27.8 = 27.9 us; 4096 x 4096 at
  // M = 64 17.0 -> 13.9 us, M = 128 16.3 -> 15.4 us; 768 x 3072 11 -> 7 us at any M up to 256): every workgroup pulls
  // all of its rows' activations through L2, C / 64 times 2 M K bytes in all, so the range ends where that
  // outgrows what the wider tiles spend on everything.
  const int64_t elems = K * C;
  const int64_t m_max = elems <= (4LL << 20) ? 256 : (elems <= (20LL << 20) ? 128 : (elems <= (64LL << 20) ? 64 : 32));
  if (M > m_max) return p;
  const int64_t T = K / 32;
  p.nb = 4;
  p.rb = M <= 32 ? 2 : 4;
  p.tiles_x = ceil_div64(C, 64);
  p.tiles_y = ceil_div64(M, 16 * p.rb);
  // splits of the contraction: up to one workgroup per CU; a split keeps at least 32 k-steps (four per wavefront)
  // and whole stages
  int64_t S = 256 / (p.tiles_x * p.tiles_y);
  if (S > 8) S = 8;
  if (S < 1) S = 1;
  for (; S > 1; --S) {
    const int64_t steps = round_up64(ceil_div64(T, S), MID_WAVES);
    if (steps >= 32 && ceil_div64(T, steps) == S) break;
  }
  p.S = (int)S;
  p.steps = (int)round_up64(ceil_div64(T, S), MID_WAVES);
  const int64_t np = p.rb / mid_rbt(p.nb, p.rb);
  if (p.tiles_x * p.tiles_y * np > QMM_MAX_COUNTERS || p.tiles_x * p.tiles_y * p.S > 65535 * 16) return MidPlan{};
  p.part_bytes = p.S > 1 ? (size_t)p.tiles_x * p.tiles_y * p.S * p.rb * p.nb * RG_TILE_FLOATS * sizeof(float) : 0;
  p.total_bytes = p.S > 1 ? QMM_HEAD_BYTES + p.part_bytes : 0;
  p.use = true;
  return p;
}

int mid_fwd_launch(hipStream_t st, const MidPlan &p, const void *x, int64_t M, const uint8_t *pk, int64_t R, int64_t C,
                   const void *zero, const void *scale, int zs_dtype, void *out, void *ws) {
  if (zs_dtype != GPTQ_HIP_F32 && zs_dtype != GPTQ_HIP_F16 && zs_dtype != GPTQ_HIP_BF16) return GPTQ_HIP_EDTYPE;
  if (p.nb != 4) return GPTQ_HIP_EINVAL;
  if (p.bf16) {
    if (p.out32) return GPTQ_HIP_EINVAL;
    if (p.rb == 2) return mid_launch_inst<__hip_bfloat16, 2>(st, p, x, M, pk, R, C, zero, scale, zs_dtype, out, ws);
    if (p.rb == 4) return mid_launch_inst<__hip_bfloat16, 4>(st, p, x, M, pk, R, C, zero, scale, zs_dtype, out, ws);
    return GPTQ_HIP_EINVAL;
  }
  if (p.rb == 2) return mid_launch_inst<__half, 2>(st, p, x, M, pk, R, C, zero, scale, zs_dtype, out, ws);
  if (p.rb == 4) return mid_launch_inst<__half, 4>(st, p, x, M, pk, R, C, zero, scale, zs_dtype, out, ws);
  return GPTQ_HIP_EINVAL;
}

}  // namespace qmm
