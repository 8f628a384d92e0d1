// Packed-weight matmul, forward, with both MFMA operands built in registers:
//   out[M, C] = x[M, K] @ ((code - zero) * scale),  codes packed as 4-bit pairs (K = 2 R) or bytes (K = R).
// Serves every forward product of more than 16 rows, and below that what the decode kernel of qmatmul.hip
// does not take: shapes whose rows are not 8- or 16-byte multiples (C % 8 != 0, e.g. a vocabulary-sized C;
// K % 8 != 0; unaligned operands), and of the 8-bit products those with bf16 activations or a matrix beyond
// what the decode kernel keeps in flight.
//
// A workgroup owns a (16 RB) x 128 output tile (RB = 1, 4 or 8 row blocks) over a range of k-steps (all of K
// unless the contraction is split over S workgroups) and its four wavefronts split those k-steps among them
// (k-step t of 32 k goes to wavefront t % 4): nothing is staged in LDS and the k loop has no barrier.
//   B: lane (l16, g) loads 8 bytes = 8 channels of each packed row that holds its 8 k of the k-step
//      (4-bit: rows 4g .. 4g+3, 8-bit: rows 8g .. 8g+7); the MFMA tile t8 takes byte t8 of every row.
//      4-bit, fp16: byte permute, and-or under the exponent of 1024, one packed fma that rescales the high
//      nibble and subtracts 1024 + rint(zero): exact small integers.  4-bit, bf16: 128 + code by shifts and
//      masks, the offset 128 + zero leaves in the epilogue.  8-bit, fp16: byte permute of two rows, or with
//      the exponent of 1024, one packed add of -(1024 + rint(zero)).  8-bit, bf16: byte -> fp32, minus
//      rint(zero), rounded to bf16 (exact: magnitude <= 255).
//   A: lane (l16, g) loads the 16 bytes x[m][32 t + 8 g ..+7] of row m = 16 rb + l16: the operand as it stands.
// A ninth tile per row block multiplies the activations with ones: the row sums of x that the epilogue
// needs for the part of the zero point not folded into B (its fraction; for 4-bit bf16 all of 128 + zero).
// Out-of-range rows, channels and k are handled by clamped addresses: loads never leave the operands.
#include "qmatmul_reg.h"
#include "qmm_reg_common.h"
#include <type_traits>

namespace {

using namespace qmm;

constexpr int RG_BN = 128;                       // channels per output tile

// GROUPED (an extension: the reference has one scale / zero per channel): zero / scale are [K / group, C] tables;
// the parameters of a k-step's group travel with its loads, and B = (code - zero) scale is formed in fp16
// (converted for bf16 activations), so the accumulators need no offset or scale afterwards.
template <int BITS, int RB, int RING, bool RAGGED, typename TX, bool GROUPED>
__global__ __launch_bounds__(256, (RB == 1 ? 2 : 1)) void qmm_fwd_reg_kernel(const TX *x, int M, int K, const uint8_t *pk, int R,
                                                          int C, const void *zero, const void *scale,
                                                          int zs_dtype, TX *out, float *part, int32_t *counters,
                                                          int S, int steps_per_split, int group_size,
                                                          unsigned long long *acc64, int tx0, float *out32,
                                                          const int32_t *rowexp) {
  constexpr bool BF = Act<TX>::BF && !GROUPED;      // grouped: the fp16 form of the dequantisation for both types
  // vector instructions between two MFMAs of the main loop (0: compiler's order)
  constexpr int SCHED = (RB == 4 && (GROUPED || RAGGED)) ? 4 : 0;
  // 64- and 128-row tiles: every MFMA accumulates in place (Act::mma_acc; the compiler's own form may write
  // another register than it reads, and it rotates accumulators through copies).  128-row tiles: the 256
  // accumulation registers hold the 8 x 8 product tiles, the row-sum tiles live in vector registers.
  constexpr bool TIED = RB >= 4;
  constexpr int RBT = RB > 4 ? 4 : RB;           // row blocks per pass of the final reduction (LDS: 36 KB each)
  constexpr int NH = RB / RBT;                   // passes
  constexpr int NL = BITS == 4 ? 4 : 8;          // packed rows per lane and k-step
  constexpr int PR = 4 * NL;                     // packed rows per k-step
  extern __shared__ __attribute__((aligned(16))) float rg_lds[];   // [4 wavefronts][RB][RG_NT][64 lanes][4]
  __shared__ int s_flag;
  // every kernel argument in registers before the first address is formed (left to itself the compiler
  // fetches them in groups where they are first used, and waits for each group)
  asm volatile("" ::"s"(x), "s"(pk), "s"(zero), "s"(scale), "s"(out), "s"(part), "s"(counters), "s"(M), "s"(K),
               "s"(R), "s"(C), "s"(zs_dtype), "s"(S), "s"(steps_per_split), "s"(group_size), "s"(acc64), "s"(tx0));
  const int tid = threadIdx.x, lane = tid & 63, wk = tid >> 6;
  const int g = lane >> 4, l16 = lane & 15;
  int tx, ty;
  qmm_tile_coords(tx, ty);
  // (tx0: first column tile of this launch, where the columns are dealt over two launches)
  const int m0 = ty * (16 * RB), nbase = (tx + tx0) * RG_BN, split = blockIdx.z;
  const int T = (K + 31) >> 5;
  // this workgroup's k-steps [t_begin, t_end); wavefront wk takes t_begin + wk, + 4, ...
  const int t_begin = split * steps_per_split, t_end = min(T, t_begin + steps_per_split);
  const int range = max(0, t_end - t_begin);
  const int iters = range > wk ? (range - wk + 3) >> 2 : 0;
  // a ragged last k-step (K % 32 != 0) is multiplied after the loop, with masked activations
  const bool has_tail = (K & 31) != 0 && iters > 0 && (t_begin + 4 * (iters - 1) + wk == T - 1);
  const int iters_full = iters - (has_tail ? 1 : 0);

  const int col = nbase + 8 * l16;
  const bool col_ok = col < C;
  const int colc = min(col, C - 8);                                   // C >= 8
  const int wshift = (RAGGED && col_ok) ? col - colc : 0;             // bytes to drop from a load at colc
  const uint8_t *wp = pk + colc;
  int xrow[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) xrow[rb] = min(m0 + 16 * rb + l16, M - 1) * K;      // M K < 2^31

  uint2 wr[RING][NL];
  uint4 aq[RING][RB];
  uint32_t zraw[GROUPED ? RING : 1][8], sraw[GROUPED ? RING : 1][8];
  auto load_step = [&](int slot, int s) __attribute__((always_inline)) {
    // (steps past this workgroup's range re-read its own last k-step, a cache hit, not the next split's rows)
    const int t = min(t_begin + 4 * s + wk, max(t_end - 1, 0));
#pragma unroll
    for (int i = 0; i < NL; ++i)
      wr[slot][i] = rg_load8<RAGGED>(wp + (int64_t)min(PR * t + NL * g + i, R - 1) * C);
    const int koff = min(32 * t + 8 * g, K - 8);                      // K >= 8: a chunk inside the row
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) aq[slot][rb] = rg_load16<RAGGED>(x + xrow[rb] + koff);
    if constexpr (GROUPED) {
      const int64_t row_base = (int64_t)((32 * t) / group_size) * C;
      rg_params8_raw(zero, zs_dtype, row_base, col, C, zraw[slot]);
      rg_params8_raw(scale, zs_dtype, row_base, col, C, sraw[slot]);
    }
  };

  // Loads return in the order of their issue: the zero points, which the first k-step's dequantisation needs,
  // go out first, then the first k-steps' loads, all before anything that has to wait for memory.
  uint32_t zraw0[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
  if constexpr (!GROUPED) rg_params8_raw(zero, zs_dtype, 0, col, C, zraw0);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int u = 0; u < RING; ++u) load_step(u, u);
  __builtin_amdgcn_sched_barrier(0);

  // ---- per-channel constants of the dequantisation (the integer part of the zero point)
  uint32_t zc[8];
  float zi8[(BF && BITS == 8) ? 8 : 1];
  if constexpr (!GROUPED) {
#pragma unroll
    for (int t8 = 0; t8 < 8; ++t8) {
    const float zi = fminf(fmaxf(rintf(rg_raw_to_f32(zraw0[t8], zs_dtype)), -512.f), 512.f);
    if constexpr (BF) {
      zc[t8] = 0u;
      if constexpr (BITS == 8) zi8[t8] = zi;
    } else if constexpr (BITS == 4) {
      zc[t8] = __builtin_bit_cast(uint32_t, half2_t{(_Float16)(-(1024.f + zi)), (_Float16)(-(64.f + zi))});
    } else {
      zc[t8] = __builtin_bit_cast(uint32_t, half2_t{(_Float16)(-(1024.f + zi)), (_Float16)(-(1024.f + zi))});
    }
    }
  }
  uint32_t mask = BF ? 0x000F000Fu : 0x00F0000Fu, cexp = BF ? 0x43004300u : 0x64006400u;
  asm volatile("" : "+s"(mask));
  asm volatile("" : "+v"(cexp));
  const half2_t unscale = half2_t{(_Float16)1.f, (_Float16)0.0625f};
  const uint32_t one2 = BF ? 0x3F803F80u : 0x3C003C00u;
  uint4 ones = make_uint4(one2, one2, one2, one2);
  asm volatile("" : "+v"(ones.x), "+v"(ones.y), "+v"(ones.z), "+v"(ones.w));      // kept in registers: not rebuilt in front of an MFMA

  floatx4 acc[RB][RG_NT];
#pragma unroll
  for (int i = 0; i < RB; ++i)
#pragma unroll
    for (int j = 0; j < RG_NT; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

  auto compute = [&](int slot, auto masked) __attribute__((always_inline)) {
    uint4 a[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      a[rb] = aq[slot][rb];
      if (decltype(masked)::value) {
        const int k0 = 32 * (T - 1) + 8 * g;
        a[rb] = rg_mask_tail(a[rb], k0, min(k0, K - 8), K);
      }
    }
    uint2 w[NL];
#pragma unroll
    for (int i = 0; i < NL; ++i) w[i] = RAGGED ? rg_shr_bytes(wr[slot][i], wshift) : wr[slot][i];
    uint32_t s2[GROUPED ? 8 : 1], nzf2[GROUPED ? 8 : 1];
    if constexpr (GROUPED) {
#pragma unroll
      for (int t8 = 0; t8 < 8; ++t8) {
        const float z = rg_raw_to_f32(zraw[slot][t8], zs_dtype), sc = rg_raw_to_f32(sraw[slot][t8], zs_dtype);
        const float zi = fminf(fmaxf(rintf(z), -512.f), 512.f);
        const _Float16 hs = (_Float16)sc, hz = (_Float16)(-(z - zi) * sc);
        s2[t8] = __builtin_bit_cast(uint32_t, half2_t{hs, hs});
        nzf2[t8] = __builtin_bit_cast(uint32_t, half2_t{hz, hz});
        zc[t8] = BITS == 4
                     ? __builtin_bit_cast(uint32_t, half2_t{(_Float16)(-(1024.f + zi)), (_Float16)(-(64.f + zi))})
                     : __builtin_bit_cast(uint32_t, half2_t{(_Float16)(-(1024.f + zi)), (_Float16)(-(1024.f + zi))});
      }
    }
    // grouped: (code - zi) * scale - (zero - zi) * scale in fp16, as bf16 for bf16 activations
    auto finish_b = [&](half2_t d, int t8) __attribute__((always_inline)) -> uint32_t {
      if constexpr (GROUPED) {
        const half2_t e = d * __builtin_bit_cast(half2_t, s2[t8]) + __builtin_bit_cast(half2_t, nzf2[t8]);
        if constexpr (Act<TX>::BF) {
          typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));
          typedef float f2_t __attribute__((ext_vector_type(2)));
          return __builtin_bit_cast(uint32_t, __builtin_convertvector(f2_t{(float)e[0], (float)e[1]}, bf2_t));
        }
        return __builtin_bit_cast(uint32_t, e);
      } else {
        return __builtin_bit_cast(uint32_t, d);
      }
    };
#pragma unroll
    for (int t8 = 0; t8 < 8; ++t8) {
      const uint32_t tb = (uint32_t)(t8 & 3);
      uint32_t r4[4];
      if constexpr (BITS == 4) {
        // fp16: the byte in both halves; bf16: in the low half only
        const uint32_t sel = BF ? (0x0c0c0c00u | tb) : (0x0c000c00u | tb | (tb << 16));
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t pb = __builtin_amdgcn_perm(0u, t8 < 4 ? w[i].x : w[i].y, sel);
          if (BF) {
            r4[i] = (((pb << 12) | pb) & mask) | cexp;                   // {128 + lo, 128 + hi}
          } else {
            const uint32_t v = (pb & mask) | cexp;                       // {1024 + lo, 1024 + 16 hi}
            const half2_t d = __builtin_bit_cast(half2_t, v) * unscale + __builtin_bit_cast(half2_t, zc[t8]);
            r4[i] = finish_b(d, t8);
          }
        }
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t wa = t8 < 4 ? w[2 * i].x : w[2 * i].y, wb = t8 < 4 ? w[2 * i + 1].x : w[2 * i + 1].y;
          if constexpr (BF) {
            typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));
            typedef float f2_t __attribute__((ext_vector_type(2)));
            const float fa = (float)((wa >> (8 * tb)) & 0xFFu) - zi8[t8];
            const float fb = (float)((wb >> (8 * tb)) & 0xFFu) - zi8[t8];
            r4[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f2_t{fa, fb}, bf2_t));
          } else {
            const uint32_t pb = __builtin_amdgcn_perm(wb, wa, 0x0c000c00u | ((4u + tb) << 16) | tb);
            const half2_t d = __builtin_bit_cast(half2_t, pb | cexp) + __builtin_bit_cast(half2_t, zc[t8]);
            r4[i] = finish_b(d, t8);
          }
        }
      }
      const uint4 b = make_uint4(r4[0], r4[1], r4[2], r4[3]);
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        if constexpr (TIED) Act<TX>::mma_acc(acc[rb][t8], a[rb], b);
        else acc[rb][t8] = Act<TX>::mma(a[rb], b, acc[rb][t8]);
      }
    }
    if constexpr (!GROUPED) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        if constexpr (TIED) Act<TX>::mma_accv(acc[rb][8], a[rb], ones);
        else acc[rb][8] = Act<TX>::mma(a[rb], ones, acc[rb][8]);
      }
    }
  };
  // ---- 64- and 128-row tiles, per-channel parameters: the k-step in software-pipelined form.  The in-place MFMAs
  // are inline asm, which the scheduler does not move; so the source order is the issue order: after every MFMA
  // (128-row tiles: every second one) of a tile the three vector instructions that build one operand register of
  // the NEXT tile, and under the row-sum tile's MFMAs the first tile of the next k-step, whose weights are in
  // the next ring slot.
  auto dq_reg = [&](const uint2 (&w)[NL], int t8, int i) __attribute__((always_inline)) -> uint32_t {
    const uint32_t tb = (uint32_t)(t8 & 3);
    if constexpr (BITS == 4) {
      const uint32_t sel = BF ? (0x0c0c0c00u | tb) : (0x0c000c00u | tb | (tb << 16));
      const uint32_t pb = __builtin_amdgcn_perm(0u, t8 < 4 ? w[i].x : w[i].y, sel);
      if (BF) return (((pb << 12) | pb) & mask) | cexp;
      const uint32_t v = (pb & mask) | cexp;
      const half2_t d = __builtin_bit_cast(half2_t, v) * unscale + __builtin_bit_cast(half2_t, zc[t8]);
      return __builtin_bit_cast(uint32_t, d);
    } else {
      const uint32_t wa = t8 < 4 ? w[2 * i].x : w[2 * i].y, wb = t8 < 4 ? w[2 * i + 1].x : w[2 * i + 1].y;
      if constexpr (BF) {
        typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));
        typedef float f2_t __attribute__((ext_vector_type(2)));
        const float fa = (float)((wa >> (8 * tb)) & 0xFFu) - zi8[t8];
        const float fb = (float)((wb >> (8 * tb)) & 0xFFu) - zi8[t8];
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f2_t{fa, fb}, bf2_t));
      } else {
        const uint32_t pb = __builtin_amdgcn_perm(wb, wa, 0x0c000c00u | ((4u + tb) << 16) | tb);
        const half2_t d = __builtin_bit_cast(half2_t, pb | cexp) + __builtin_bit_cast(half2_t, zc[t8]);
        return __builtin_bit_cast(uint32_t, d);
      }
    }
  };
  constexpr bool PIPE = TIED && !GROUPED && !RAGGED;     // (the ragged form has no registers left for it)
  uint32_t bcarry[4] = {0u, 0u, 0u, 0u};         // tile 0 of the k-step about to be multiplied
  auto shifted = [&](int slot, uint2 (&w)[NL]) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < NL; ++i) w[i] = RAGGED ? rg_shr_bytes(wr[slot][i], wshift) : wr[slot][i];
  };
  // 128-row tiles: the vector instructions stand after the MFMAs of the even row blocks, so an MFMA that reads a
  // freshly built operand always has another MFMA between itself and the instruction that wrote it (the odd row
  // blocks' MFMAs count as a use of what was just built, which keeps the compiler from sinking it further), and
  // the MFMAs go without wait states.  Where that use cannot be expressed (the first tile of the next k-step, built
  // under the row-sum MFMAs) and at the head of the k-step the wait states stay.
  auto pipe_mma = [&](floatx4 &c, const uint4 &a, const uint4 &b) __attribute__((always_inline)) {
    if constexpr (RB == 8) Act<TX>::mma_acc_nw(c, a, b);
    else Act<TX>::mma_acc(c, a, b);
  };
  auto pipe_mmav = [&](floatx4 &c, const uint4 &a, const uint4 &b) __attribute__((always_inline)) {
    if constexpr (RB == 8) Act<TX>::mma_accv_nw(c, a, b);
    else Act<TX>::mma_accv(c, a, b);
  };
  auto step_pipe = [&](int slot, int next_slot) __attribute__((always_inline)) {
    uint2 w[NL];
    shifted(slot, w);
    uint32_t bc[4] = {bcarry[0], bcarry[1], bcarry[2], bcarry[3]};
    if constexpr (RB == 8) asm volatile("s_nop 1");
#pragma unroll
    for (int t8 = 0; t8 < 8; ++t8) {
      const uint4 b = make_uint4(bc[0], bc[1], bc[2], bc[3]);
      uint32_t nx[4] = {0u, 0u, 0u, 0u};
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        if (RB == 8 && (rb & 1) && t8 < 7) Act<TX>::mma_acc_nw_after(acc[rb][t8], aq[slot][rb], b, nx[rb >> 1]);
        else pipe_mma(acc[rb][t8], aq[slot][rb], b);
        if (t8 < 7 && (RB == 4 || !(rb & 1))) nx[RB == 4 ? rb : rb >> 1] = dq_reg(w, t8 + 1, RB == 4 ? rb : rb >> 1);
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) bc[i] = nx[i];
    }
    uint2 wn[NL];
    shifted(next_slot, wn);
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      if (RB == 8 && (rb & 1)) Act<TX>::mma_accv(acc[rb][8], aq[slot][rb], ones);      // (with wait states: see bcarry)
      else pipe_mmav(acc[rb][8], aq[slot][rb], ones);
      if (RB == 4 || !(rb & 1)) bcarry[RB == 4 ? rb : rb >> 1] = dq_reg(wn, 0, RB == 4 ? rb : rb >> 1);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  const std::integral_constant<bool, false> plain{};
  const std::integral_constant<bool, true> tail{};
  int s0 = 0;
  if constexpr (PIPE) {
    uint2 w0[NL];
    shifted(0, w0);
#pragma unroll
    for (int i = 0; i < 4; ++i) bcarry[i] = dq_reg(w0, 0, i);
  }
  for (; s0 + RING <= iters_full; s0 += RING) {
#pragma unroll
    for (int u = 0; u < RING; ++u) {
      if constexpr (PIPE) step_pipe(u, (u + 1) % RING);
      else compute(u, plain);
      // (16-row tiles: nothing is fetched for k-steps past this wavefront's last; wave-uniform.  64-row tiles keep
      // one basic block per k-step for the instruction order below, and re-read their last k-step instead)
      if (SCHED != 0 || PIPE || s0 + u + RING < iters) load_step(u, s0 + u + RING);
      // One wavefront per SIMD issues in order: an MFMA occupies the matrix pipe for four passes, during
      // which the wavefront can issue only what stands behind it in program order and does not depend on it.
      // So the dequantisation of the next tile goes between the MFMAs of this one: one MFMA, then a few
      // vector instructions, and the k-step's loads spread over its first groups.
      if (SCHED) {
#pragma unroll
        for (int i = 0; i < RB * RG_NT; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if (i < NL + RB) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, SCHED, 0);
        }
      }
    }
  }
  // at most RING - 1 full k-steps left, all of them loaded; then the ragged one
#pragma unroll
  for (int u = 0; u < RING - 1; ++u)
    if (s0 + u < iters_full) {
      if constexpr (PIPE) step_pipe(u, u + 1);
      else compute(u, plain);
    }
  if (has_tail) {
    const int slot = iters_full - s0;            // 0 .. RING - 1
#pragma unroll
    for (int u = 0; u < RING; ++u)
      if (u == slot) compute(u, tail);
  }

  if constexpr (TIED) mma_drain();
  // scale and zero point of this lane's channels, in flight while the tiles are summed
  float sc[8], zf[8];
  if constexpr (!GROUPED) {
    rg_params8(scale, zs_dtype, col, C, sc);
    rg_params8(zero, zs_dtype, col, C, zf);
  }
  // acc64 (16-row tiles only): every split finishes its own outputs and adds them to the cells
  const bool atom = RB == 1 && acc64 != nullptr && S > 1;
  // One pass of the reduction per four row blocks (a 128-row tile: two passes, each with its own arrival
  // counter and partial tiles, as if it were two 64-row tiles).
  auto finish = [&](auto hc) __attribute__((always_inline)) {
    constexpr int H = decltype(hc)::value;
    floatx4 sum[RG_NT];
    const int tile = (ty * NH + H) * gridDim.x + tx;
    if (!rg_reduce<RBT, RB, H * RBT>(acc, sum, rg_lds, &s_flag, part, counters, tile, split, atom ? 1 : S)) return;
    // sum[t8][r] = sum_k x[m][k] (code - zi)[k][col + t8] (bf16, 4-bit: code + 128), sum[8][r] = sum_k x[m][k],
    // m = m0 + 16 (H RBT + rb) + 4 g + r
    if (!col_ok && !atom) return;
    const int rb = H * RBT + wk;                   // rg_reduce returned true: wk < RBT
    // (first use of the parameters: after the reduction's waits)
    float sca[8], zfa[8];
#pragma unroll
    for (int t8 = 0; t8 < 8; ++t8) {
      sca[t8] = GROUPED ? 1.f : sc[t8];
      zfa[t8] = GROUPED ? 0.f
                        : ((BF && BITS == 4) ? 128.f + zf[t8] : zf[t8] - fminf(fmaxf(rintf(zf[t8]), -512.f), 512.f));
    }
    if constexpr (RB == 1) {
      if (atom) {
        // This wavefront's finished values go through the LDS (the other wavefronts are done with it) so that
        // consecutive lanes hold consecutive channels: the memory side takes an atomic per 64-byte segment,
        // not per lane.  Then two passes per eight rows, so that a lane's atomics are in flight together.  The
        // word that comes back tells the last of the S contributions that it is the last, and gives it the
        // complete sum: it rounds, stores the output and zeroes the cell.  Integer addition is exact and
        // commutative: the result does not depend on the order of arrival.
        float *tr = rg_lds;                                  // [16 rows][128 channels]
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float rs = sum[8][r];
          float pv[8];
#pragma unroll
          for (int t8 = 0; t8 < 8; ++t8) pv[t8] = sca[t8] * (sum[t8][r] - zfa[t8] * rs);
          float *dst = tr + (4 * g + r) * RG_BN + 8 * l16;
          *reinterpret_cast<float4 *>(dst) = make_float4(pv[0], pv[1], pv[2], pv[3]);
          *reinterpret_cast<float4 *>(dst + 4) = make_float4(pv[4], pv[5], pv[6], pv[7]);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // one wavefront: its LDS accesses complete in order
#pragma unroll
        for (int mh = 0; mh < 2; ++mh) {
          if (8 * mh >= M - m0) break;
          unsigned long long old[16], word[16];
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int mr = 8 * mh + (i >> 1), c = 64 * (i & 1) + lane;
            old[i] = word[i] = 0ull;
            if (m0 + mr >= M || nbase + c >= C) continue;
            const float pv = tr[mr * RG_BN + c];
            const bool ok = fabsf(pv) <= 65536.f;                       // false for NaN, too
            const long long fx = ok ? __float2ll_rn(pv * (float)(1 << QD_FRAC)) : QD_POISON;
            word[i] = ((unsigned long long)fx << 8) + 1ull;
            old[i] = atomicAdd(acc64 + (int64_t)(m0 + mr) * C + nbase + c, word[i]);
          }
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int mr = 8 * mh + (i >> 1), c = 64 * (i & 1) + lane;
            const unsigned long long total = old[i] + word[i];
            if ((int)(total & 255ull) != S) continue;                   // (also the lanes that added nothing: 0 != S)
            const long long fsum = (long long)total >> 8;
            const bool fine = fsum <= (1LL << 49) && fsum >= -(1LL << 49);
            const float res = fine ? (float)fsum * (1.f / (float)(1 << QD_FRAC)) : __builtin_nanf("");
            out[(int64_t)(m0 + mr) * C + nbase + c] = Act<TX>::out(res);
            __hip_atomic_store(acc64 + (int64_t)(m0 + mr) * C + nbase + c, 0ull, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
          }
        }
        return;
      }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = m0 + 16 * rb + 4 * g + r;
      if (m >= M) continue;
      const float rs = sum[8][r];
      TX o[8];
#pragma unroll
      for (int t8 = 0; t8 < 8; ++t8) o[t8] = Act<TX>::out(sca[t8] * (sum[t8][r] - zfa[t8] * rs));
      if (out32 != nullptr) {
        // fp32 rows: the fp16 result widened and scaled back by the row's power of two (exact)
        const int e = rowexp[m];
        float *d32 = out32 + (int64_t)m * C + col;
        float f[8];
#pragma unroll
        for (int t8 = 0; t8 < 8; ++t8) f[t8] = ldexpf((float)o[t8], e);
        if (RAGGED) {
#pragma unroll
          for (int t8 = 0; t8 < 8; ++t8)
            if (col + t8 < C) d32[t8] = f[t8];
        } else {
          *reinterpret_cast<float4 *>(d32) = make_float4(f[0], f[1], f[2], f[3]);
          *reinterpret_cast<float4 *>(d32 + 4) = make_float4(f[4], f[5], f[6], f[7]);
        }
        continue;
      }
      TX *dst = out + (int64_t)m * C + col;
      if (RAGGED) {
#pragma unroll
        for (int t8 = 0; t8 < 8; ++t8)
          if (col + t8 < C) dst[t8] = o[t8];
      } else {
        *reinterpret_cast<uint4 *>(dst) = *reinterpret_cast<const uint4 *>(o);
      }
    }
  };
  finish(std::integral_constant<int, 0>{});
  if constexpr (NH == 2) {
    __syncthreads();                                 // the first pass's sums have been read
    finish(std::integral_constant<int, 1>{});
  }
}

template <int BITS, int RB, int RING, bool RAGGED, typename TX, bool GROUPED>
int launch_inst(hipStream_t st, const RegPlan &p, const void *x, int64_t M, const uint8_t *pk, int64_t R,
                int64_t C, const void *zero, const void *scale, int zs_dtype, void *out, void *wsp, int group_size,
                int64_t tx0 = 0, int64_t ntx = -1) {
  constexpr size_t lds = (size_t)4 * (RB > 4 ? 4 : RB) * RG_NT * RG_TILE_FLOATS * sizeof(float);
  auto kern = qmm_fwd_reg_kernel<BITS, RB, RING, RAGGED, TX, GROUPED>;
  if (lds > 64 * 1024 && !gptq_raise_lds_limit(reinterpret_cast<const void *>(kern), (int)lds)) return GPTQ_HIP_ELAUNCH;
  const int64_t K = BITS == 4 ? 2 * R : R;
  int32_t *counters = reinterpret_cast<int32_t *>(wsp);
  float *part = reinterpret_cast<float *>(reinterpret_cast<char *>(wsp) + QMM_HEAD_BYTES);
  unsigned long long *acc64 =
      p.atom ? reinterpret_cast<unsigned long long *>(reinterpret_cast<char *>(wsp) + QMM_COUNTER_BYTES) : nullptr;
  // column tiles [tx0, tx0 + ntx) (all of them unless the plan deals the columns over two launches)
  const int64_t tiles_all = ceil_div64(C, RG_BN);
  const int64_t tiles_x = ntx < 0 ? tiles_all : ntx;
  // rows per launch: 32-bit element offsets into x, grid.y, one arrival counter per tile, the partial region
  int64_t rows_max = ((1LL << 31) - 1) / K;
  if (rows_max > 65535LL * 16 * RB) rows_max = 65535LL * 16 * RB;
  const int64_t tiles_y_max = p.tiles / tiles_all;                     // what the plan sized the workspace for
  if (p.S > 1 && rows_max > tiles_y_max * 16 * RB) rows_max = tiles_y_max * 16 * RB;
  rows_max -= rows_max % (16 * RB);
  if (rows_max < 16 * RB) return GPTQ_HIP_EINVAL;
  for (int64_t r0 = 0; r0 < M; r0 += rows_max) {
    const int64_t rows = M - r0 < rows_max ? M - r0 : rows_max;
    const dim3 grid((unsigned)tiles_x, (unsigned)ceil_div64(rows, 16 * RB), (unsigned)p.S);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, st, (const TX *)x + r0 * K, (int)rows, (int)K, pk, (int)R,
                       (int)C, zero, scale, zs_dtype, (TX *)out + r0 * C, part, counters, p.S, p.steps, group_size, acc64,
                       (int)tx0, (RB > 1 && p.out32) ? p.out32 + r0 * C : nullptr, p.rowexp ? p.rowexp + r0 : nullptr);
    GPTQ_CHECK_LAUNCH();
  }
  return GPTQ_HIP_OK;
}

// 128-row tiles whose last round of workgroups would be at most half full (one workgroup per CU): this many
// trailing column tiles go to 64-row tiles in a launch of their own, one partial round of half-sized tiles, and
// the columns in front of them fill whole rounds.  Rounds have to be long (T k-steps) for the second launch to pay.
int64_t deal_tail(int64_t tiles_x, int64_t tiles_y, int64_t T) {
  if (T < 64) return 0;
  const int64_t all = tiles_x * tiles_y, full = all / 256, rem = all % 256;
  if (full < 1 || rem == 0 || rem > 128) return 0;
  const int64_t main_x = full * 256 / tiles_y, tail = tiles_x - main_x;
  return (main_x >= 1 && tail >= 1 && tail * tiles_y * 2 <= 256) ? tail : 0;
}

template <int BITS, typename TX>
int launch_bx(hipStream_t st, const RegPlan &p, const void *x, int64_t M, const uint8_t *pk, int64_t R, int64_t C,
              const void *zero, const void *scale, int zs_dtype, void *out, void *ws, int group_size) {
#define GPTQ_REG(RB, RING, RAGGED, GROUPED) \
  return launch_inst<BITS, RB, RING, RAGGED, TX, GROUPED>(st, p, x, M, pk, R, C, zero, scale, zs_dtype, out, ws, group_size)
  if (group_size > 0) {
    // the group's parameters ride in the ring: shorter rings
    if (p.rb == 8) {
      if (p.ragged) GPTQ_REG(8, 2, true, true);
      GPTQ_REG(8, 2, false, true);
    }
    if (p.rb == 4) {
      if (p.ragged) GPTQ_REG(4, 2, true, true);
      GPTQ_REG(4, 2, false, true);
    }
    if (p.ragged) GPTQ_REG(1, 3, true, true);
    GPTQ_REG(1, 3, false, true);
  }
  // a ring of two k-steps for 128-row tiles, of three for 64-row tiles (registers), of six for the 16-row tiles
  // of the decode case
  if (p.rb == 8) {
    const RegParts q = reg_fwd_parts(p, M, R, C, Act<TX>::BF, group_size);
    if (q.wide_x > 0) {
      const int rc = wide_fwd_launch(st, x, Act<TX>::BF ? GPTQ_HIP_BF16 : GPTQ_HIP_F16, M, pk, R, C, zero, scale,
                                     zs_dtype, out, q.wide_x, q.half, p.out32, p.rowexp, BITS);
      if (rc) return rc;
    }
    if (q.wide2_x > 0) {
      const int rc = wide_fwd_launch(st, x, Act<TX>::BF ? GPTQ_HIP_BF16 : GPTQ_HIP_F16, M, pk, R, C, zero, scale, zs_dtype,
                                     out, q.wide2_x, true, p.out32, p.rowexp, BITS, 512 * q.wide_x);
      if (rc) return rc;
    }
    if (q.main_x > 0) {
      const int rc = p.ragged ? launch_inst<BITS, 8, 2, true, TX, false>(st, p, x, M, pk, R, C, zero, scale, zs_dtype,
                                                                           out, ws, group_size, q.first, q.main_x)
                              : launch_inst<BITS, 8, 3, false, TX, false>(st, p, x, M, pk, R, C, zero, scale, zs_dtype,
                                                                            out, ws, group_size, q.first, q.main_x);
      if (rc) return rc;
    }
    if (q.tail == 0) return GPTQ_HIP_OK;
    if (p.ragged)
      return launch_inst<BITS, 4, 3, true, TX, false>(st, p, x, M, pk, R, C, zero, scale, zs_dtype, out, ws,
                                                      group_size, q.first + q.main_x, q.tail);
    return launch_inst<BITS, 4, 3, false, TX, false>(st, p, x, M, pk, R, C, zero, scale, zs_dtype, out, ws,
                                                     group_size, q.first + q.main_x, q.tail);
  }
  if (p.rb == 4) {
    if (p.ragged) GPTQ_REG(4, 3, true, false);
    GPTQ_REG(4, 3, false, false);
  }
  if (p.ragged) GPTQ_REG(1, 6, true, false);
  GPTQ_REG(1, 6, false, false);
#undef GPTQ_REG
}

}  // namespace

namespace qmm {

RegParts reg_fwd_parts(const RegPlan &p, int64_t M, int64_t R, int64_t C, bool bf16, int group_size) {
  RegParts q{};
  const int64_t tiles_all = ceil_div64(C, RG_BN);
  if (p.rb != 8 || group_size > 0) {
    q.main_x = tiles_all;
    return q;
  }
  const int64_t tiles_y = ceil_div64(M, 128), K = p.bits == 4 ? 2 * R : R;
  // 128 x 512 tiles (qmatmul_wide.hip) on the leading columns that fill whole rounds of workgroups
  if ((p.bits == 4 || !bf16) && !p.ragged && p.S == 1) {
    q.wide_x = wide_fwd_tiles(M, R, C, true, &q.half, p.bits);
    if (q.wide_x > 0) q.first = (q.half ? 2 : 4) * q.wide_x;
    // the 128-row tiles run at 50 - 60 % of the wide tiles' rate, so what is left behind whole rounds of 512-channel
    // tiles goes to 256-channel tiles if those fill half a round or more (M = 2048 on 4096 x 11008: 198 -> 186 us)
    if (q.wide_x > 0 && !q.half) {
      const int64_t n2 = (C - 512 * q.wide_x) / 256;
      if (n2 * tiles_y >= 128 && n2 * tiles_y <= 256) {
        q.wide2_x = n2;
        q.first += 2 * n2;
      }
    }
  }
  const int64_t rest = tiles_all - q.first;
  if (rest == 0) return q;
  // of the rest: 128-row tiles on the columns that fill whole rounds, 64-row tiles on the remaining ones
  q.tail = q.first == 0 ? p.tail_x : deal_tail(rest, tiles_y, ceil_div64(K, 32));
  if (q.first > 0 && rest * tiles_y <= 128) q.tail = rest;
  q.main_x = rest - q.tail;
  return q;
}

RegPlan reg_fwd_plan(int64_t M, int64_t R, int64_t C, int bits, bool aligned) {
  RegPlan p{};
  const int64_t K = bits == 4 ? 2 * R : R;
  if ((bits != 4 && bits != 8) || M < 1 || C < 8 || K < 8 || R >= (1LL << 30) || C >= (1LL << 30)) return p;
  p.bits = bits;
  // 128-row tiles (a weight tile is dequantised once for twice the rows; their reduction takes two passes) where
  // they alone fill most of the chip, 64-row tiles otherwise
  p.rb = M <= 16 ? 1 : ((M > 64 && ceil_div64(C, RG_BN) * ceil_div64(M, 128) >= 160) ? 8 : 4);
  p.ragged = !aligned || C % 8 != 0 || K % 8 != 0;
  const int64_t tiles_x = ceil_div64(C, RG_BN);
  const int64_t nh = p.rb == 8 ? 2 : 1;          // arrival counters per tile (a 128-row tile is reduced in two passes)
  if (tiles_x * nh > QMM_MAX_COUNTERS) return p;
  int64_t tiles_y = ceil_div64(M, 16 * p.rb);
  if (tiles_y > QMM_MAX_COUNTERS / (tiles_x * nh)) tiles_y = QMM_MAX_COUNTERS / (tiles_x * nh);    // further rows: further launches
  p.tiles = tiles_x * tiles_y;
  const int64_t T = ceil_div64(K, 32);
  // workgroups wanted: one per CU for 64- and 128-row tiles (their registers allow no more), two for 16-row
  // tiles; every wavefront of a split keeps at least four k-steps
  const int64_t want = p.rb == 1 ? 512 : 256;
  int64_t S = 1;
  if (p.tiles < want) {
    S = want / p.tiles;
    if (S > 32) S = 32;
    while (S > 1 && T / S < 16) --S;
  }
  p.steps = (int)ceil_div64(T, S);
  p.S = (int)ceil_div64(T, p.steps);
  // 128-row tiles whose last round of workgroups would be at most half full (one workgroup per CU): the
  // columns that fill whole rounds keep them, the remaining column tiles run on 64-row tiles in a second
  // launch, one partial round of half-sized tiles (M = 2048 on 4096 x 11008: 80 + 6 column tiles, 5 rounds +
  // 192 workgroups instead of 5.4 -> 6 rounds).  Rounds have to be long for the second launch to pay.
  p.tail_x = (p.rb == 8 && p.S == 1) ? (int)deal_tail(tiles_x, tiles_y, T) : 0;
  // 16-row tiles (one launch, M <= 16): the atomic sum where the cells hold the output and the atomics are few
  // (the memory side retires them at a limited rate: 900000 of them cost what the ticket path costs on
  // 4096 x 11008 and 4 us more on 7168 x 28672)
  p.atom = p.rb == 1 && p.S > 1 && M * C * 8 <= QMM_ACC_BYTES && M * C * p.S <= 500000;
  p.part_bytes = (p.S > 1 && !p.atom) ? (size_t)p.tiles * p.S * p.rb * RG_NT * RG_TILE_FLOATS * sizeof(float) : 0;
  p.total_bytes = p.S > 1 ? QMM_HEAD_BYTES + p.part_bytes : 0;
  p.use = true;
  return p;
}

int reg_fwd_launch(hipStream_t st, const RegPlan &p, const void *x, int x_dtype, int64_t M, const uint8_t *pk,
                   int64_t R, int64_t C, const void *zero, const void *scale, int zs_dtype, void *out, void *ws,
                   int group_size) {
  if (group_size < 0 || group_size % 32 != 0) return GPTQ_HIP_EINVAL;
  if (zs_dtype != GPTQ_HIP_F32 && zs_dtype != GPTQ_HIP_F16 && zs_dtype != GPTQ_HIP_BF16) return GPTQ_HIP_EDTYPE;
  if (x_dtype == GPTQ_HIP_BF16) {
    if (p.bits == 4) return launch_bx<4, __hip_bfloat16>(st, p, x, M, pk, R, C, zero, scale, zs_dtype, out, ws, group_size);
    return launch_bx<8, __hip_bfloat16>(st, p, x, M, pk, R, C, zero, scale, zs_dtype, out, ws, group_size);
  }
  if (x_dtype != GPTQ_HIP_F16) return GPTQ_HIP_EDTYPE;
  if (p.bits == 4) return launch_bx<4, __half>(st, p, x, M, pk, R, C, zero, scale, zs_dtype, out, ws, group_size);
  return launch_bx<8, __half>(st, p, x, M, pk, R, C, zero, scale, zs_dtype, out, ws, group_size);
}

}  // namespace qmm
