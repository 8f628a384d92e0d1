// Packed-weight matmul, forward, 4-bit codes, many rows: out[M, C] = x[M, K] @ ((code - zero) * scale) on
// 128 x 512 output tiles whose four wavefronts stand side by side.
//
// Each wavefront owns a 128 x 128 output tile over ALL of K (8 x 8 product tiles in the 256 accumulation
// registers) and builds its weight operands in registers from its own 128 channels (lane (l16, g): 8 bytes = 8
// channels of each packed row that holds its 8 k of the k-step; product tile t8 takes byte t8 of every row).
//
// fp16 rows: the weight operand is the RAW codes read as fp16 subnormals, which the MFMA multiplies exactly: a
// byte permute puts byte t8 into both halves of a register and one mask leaves {lo, hi << 4} = {lo 2^-24,
// 16 hi 2^-24}: two vector instructions per operand register, no conversion.  The 16 goes to the other operand
// (the activations of odd k are divided by 16 on their way into LDS, the row sums' operand holds 16 for them);
// 2^24, the scale and the zero point (- zero sum_k x[m][k], the row sums from a ninth tile) wait for the epilogue.
// bf16 rows: 128 + code (three instructions), the term (128 + zero) sum_k x leaves in the epilogue likewise.
//
// The activations: the four wavefronts need the same 128 rows, so a
// stage of 64 k (16 KB) is fetched once per workgroup, 16 bytes per thread and piece, and laid into LDS in
// operand order ([k-step][row block][lane]: a wavefront's operand register quad is one conflict-free 16-byte
// read).  Per k-step a CU takes in 8 KB of activations + 4 x 2 KB of packed weights for 4 x 72 MFMAs, where
// the K-split tiles take 4 x 10 KB; the wavefronts' tiles are complete when the loop ends, so there is no
// reduction over wavefronts either.
//
// One barrier per stage, two LDS slots.  Stage s, first k-step: the operand quads of the second k-step are
// read from LDS while the first is multiplied; then stage s + 1's pieces (fetched two stages earlier into
// registers) are written to the other slot and stage s + 3's fetched; barrier; second k-step, under which the
// first operand quads of stage s + 1 are read.  Weights are fetched two stages (less one k-step) ahead.
//
// Shapes: K % 64 == 0, C % 8 == 0, 16-byte aligned operands, per-channel parameters; the launch covers whole
// 512-channel tiles only (the dispatcher gives the remaining columns to the other kernels).  Rows past M are
// read from row M - 1 and not stored.
#include "qmatmul_reg.h"
#include "qmm_reg_common.h"
#include <type_traits>

namespace {

using namespace qmm;

// HALF: a 128 x 256 tile (for shapes whose 128 x 512 tiles are under one round of workgroups), the four wavefronts
// side by side with all 128 rows and 64 channels each (a lane loads 4 bytes = 4 channels of each of its rows): the
// operand instructions per MFMA stay those of the 128 x 512 tile, the activation reads from LDS double.  (As two
// row halves x two column halves of 64 x 128 each, every operand was built twice: M = 2048 on 11008 x 4096 took
// 205 us against 186, with bf16 rows 192 against 175, with 8-bit codes 202 against 188.)
//
// BITS = 8 (one code per byte, K = R, fp16 rows): a lane loads 8 bytes of each of its eight rows of a k-step; the
// bytes of two rows that a byte permute pairs ARE the operand, fp16 subnormals {a 2^-24, b 2^-24}: one vector
// instruction per operand register.
template <int NWV, typename TX, bool HALF = false, int BITS = 4>
__global__ __launch_bounds__(64 * NWV, 1) void qmm_fwd_wide_kernel(const TX *x, int M, int K, const uint8_t *pk, int C,
                                                                   const void *zero, const void *scale,
                                                                   int zs_dtype, TX *out, int c0, float *out32,
                                                                   const int32_t *rowexp) {
  constexpr bool BF = Act<TX>::BF;
  static_assert(NWV == 4, "the row sums are dealt to four wavefronts");
  static_assert(BITS == 4 || (BITS == 8 && !BF), "8-bit codes: fp16 rows");
  constexpr int NRW = BITS == 8 ? 8 : 4;         // packed rows of a lane per k-step
  constexpr int NT = 64 * NWV;
  constexpr int CH = 1024 / NT;                  // 16-byte pieces of a stage per thread
  constexpr int RB = 8;                          // row blocks of a wavefront
  constexpr int NTL = HALF ? 4 : 8;              // product tiles (16 channels) of a wavefront's row block
  constexpr int CPL = HALF ? 4 : 8;              // channels of a lane
  constexpr int TB = 8;                          // row blocks of the workgroup's tile
  __shared__ u32x4_t a_lds[2 * 2 * TB * 64];       // [slot][k-step of the stage][row block][lane]
  asm volatile("" ::"s"(x), "s"(pk), "s"(zero), "s"(scale), "s"(out), "s"(M), "s"(K), "s"(C), "s"(zs_dtype),
               "s"(c0), "s"(out32), "s"(rowexp));
  const int tid = threadIdx.x, lane = tid & 63, wk = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 4, l16 = lane & 15;
  int tx, ty;
  qmm_tile_coords(tx, ty);
  constexpr int rb0 = 0;                         // first row block of this wavefront
  const int m0 = ty * 128;
  const int nbase = c0 + (tx * NWV + wk) * (16 * NTL);
  const int NS = K >> 6;
  const int col = nbase + CPL * l16;

  // this thread's pieces of a stage: row (tid >> 3) + (NT / 8) i of the tile, k 8 (tid & 7) .. + 7 of the stage
  const int kc = tid & 7;
  int xoff[CH];
#pragma unroll
  for (int i = 0; i < CH; ++i) xoff[i] = min(m0 + (tid >> 3) + (NT / 8) * i, M - 1) * K + 8 * kc;      // M K < 2^31
  // piece i lands at [kc >> 2][(tid >> 7) + (NT / 128) i][16 (kc & 3) + ((tid >> 3) & 15)]
  // (the lane index within a block is XORed with 4 g ^ 2 h: the eight lanes that write one row's 128 bytes would
  //  otherwise hit the same banks; the reads, which XOR the same value, stay conflict free)
  const int dst0 = ((kc >> 2) * TB + (tid >> 7)) * 64 + 16 * (kc & 3) + (((tid >> 3) & 15) ^ (4 * (kc & 3)) ^ (2 * (kc >> 2)));
  const uint8_t *wp = pk + (int64_t)(NRW * g) * C + col;

  u32x4_t stg[2][CH];
  uint2 wr[2][2][NRW];
  u32x4_t aq[2][RB];
  u32x4_t aqr[2][2];                             // row blocks 2 wk, 2 wk + 1 once more, for the row sums
  auto load_a = [&](int p, int s) __attribute__((always_inline)) {
    const int so = 64 * min(s, NS - 1);
#pragma unroll
    for (int i = 0; i < CH; ++i) stg[p][i] = *reinterpret_cast<const u32x4_t *>(x + xoff[i] + so);
  };
  auto write_a = [&](int p, int slot) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      if constexpr (!BF && BITS == 4) {
        // fp16 rows, 4-bit codes: the high nibbles enter the MFMA as 16 code 2^-24, so the activations of odd k
        // enter divided by 16 (exact down to 2^-10; below that to 2^-25 absolute)
        // (written as the instruction: the compiler's own packed multiply of the four words by this constant came
        //  out as one multiply of the second word copied into all four)
        const uint32_t odd16 = 0x2C003C00u;      // {1, 1/16}
        const u32x4_t v = stg[p][i];
        uint32_t e0, e1, e2, e3;
        asm("v_pk_mul_f16 %0, %1, %2" : "=v"(e0) : "v"(v.x), "s"(odd16));
        asm("v_pk_mul_f16 %0, %1, %2" : "=v"(e1) : "v"(v.y), "s"(odd16));
        asm("v_pk_mul_f16 %0, %1, %2" : "=v"(e2) : "v"(v.z), "s"(odd16));
        asm("v_pk_mul_f16 %0, %1, %2" : "=v"(e3) : "v"(v.w), "s"(odd16));
        a_lds[slot * (2 * TB * 64) + dst0 + (NT / 128) * 64 * i] = u32x4_t{e0, e1, e2, e3};
        continue;
      }
      a_lds[slot * (2 * TB * 64) + dst0 + (NT / 128) * 64 * i] = stg[p][i];
    }
  };
  auto load_w = [&](int p, int h, int s) __attribute__((always_inline)) {
    const uint8_t *q = wp + (int64_t)(8 * NRW * min(s, NS - 1) + 4 * NRW * h) * C;
#pragma unroll
    for (int i = 0; i < NRW; ++i) {
      if constexpr (HALF) wr[p][h][i] = make_uint2(*reinterpret_cast<const uint32_t *>(q + (int64_t)i * C), 0u);
      else wr[p][h][i] = *reinterpret_cast<const uint2 *>(q + (int64_t)i * C);
    }
  };
  auto read_a = [&](int q, int slot, int h) __attribute__((always_inline)) {
    const int sl = lane ^ (4 * g) ^ (2 * h);
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) aq[q][rb] = a_lds[((slot * 2 + h) * TB + rb0 + rb) * 64 + sl];
#pragma unroll
    for (int j = 0; j < 2; ++j) aqr[q][j] = a_lds[((slot * 2 + h) * TB + 2 * wk + j) * 64 + sl];
  };

  load_a(1, 0);
  load_w(0, 0, 0);
  load_w(0, 1, 0);
  load_a(0, 1);
  load_w(1, 0, 1);
  load_w(1, 1, 1);
  __builtin_amdgcn_sched_barrier(0);

  uint32_t mask = BF ? 0x000F000Fu : 0x00F0000Fu, cexp = 0x43004300u;
  asm volatile("" : "+s"(mask));
  asm volatile("" : "+v"(cexp));
  // the row sums' operand: ones (fp16 rows with 4-bit codes: 16 for the odd k, whose activations enter divided by 16)
  const uint32_t one2 = BF ? 0x3F803F80u : (BITS == 4 ? 0x4C003C00u : 0x3C003C00u);
  uint4 ones = make_uint4(one2, one2, one2, one2);
  asm volatile("" : "+v"(ones.x), "+v"(ones.y), "+v"(ones.z), "+v"(ones.w));      // kept in registers: not rebuilt in front of an MFMA

  floatx4 acc[RB][8];
#pragma unroll
  for (int i = 0; i < RB; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

  // operand register i of tile t8 (channel 8 l16 + t8): codes of packed row i of the lane's four, see qmatmul_reg.hip
  auto dq_reg = [&](const uint2 (&w)[NRW], int t8, int i) __attribute__((always_inline)) -> uint32_t {
    const uint32_t tb = (uint32_t)(t8 & 3);
    if constexpr (BITS == 8) {
      // byte t8 of rows 2 i (even k, low half) and 2 i + 1 (odd k): the operand as it stands, {a 2^-24, b 2^-24}
      const uint32_t sel8 = 0x0c000c00u | tb | ((4u + tb) << 16);
      return t8 < 4 ? __builtin_amdgcn_perm(w[2 * i + 1].x, w[2 * i].x, sel8)
                    : __builtin_amdgcn_perm(w[2 * i + 1].y, w[2 * i].y, sel8);
    }
    const uint32_t sel = BF ? (0x0c0c0c00u | tb) : (0x0c000c00u | tb | (tb << 16));
    const uint32_t pb = __builtin_amdgcn_perm(0u, t8 < 4 ? w[i].x : w[i].y, sel);
    if (BF) return (((pb << 12) | pb) & mask) | cexp;                  // {128 + lo, 128 + hi}
    return pb & mask;                                                  // {lo 2^-24, 16 hi 2^-24}
  };
  // One k-step: the in-place MFMAs are inline asm, which the scheduler does not move, so the source order is the
  // issue order: after every second MFMA of a tile the three vector instructions of one operand register of the
  // next tile (under the last tile: of the first tile of the next k-step).  The vector instructions stand after
  // the even row blocks' MFMAs and the odd ones count as a use of what was just built, so every MFMA that reads a
  // freshly built operand has at least one other MFMA between itself and the instruction that wrote it: the
  // MFMAs need no wait states in front of them.
  // Row sums (the ninth tile): wavefront wk accumulates those of row blocks 2 wk and 2 wk + 1 only (operand quads
  // ar, read from LDS a second time so that no register is indexed with wk); the wavefronts exchange them through
  // LDS when the loop is done.
  uint32_t bcarry[4];
  floatx4 rsum[2] = {floatx4{0.f, 0.f, 0.f, 0.f}, floatx4{0.f, 0.f, 0.f, 0.f}};
  auto step_pipe = [&](const u32x4_t (&a)[RB], const u32x4_t (&ar)[2], const uint2 (&w)[NRW], const uint2 (&wn)[NRW]) __attribute__((always_inline)) {
    uint32_t bc[4] = {bcarry[0], bcarry[1], bcarry[2], bcarry[3]};
#pragma unroll
    for (int t8 = 0; t8 < NTL; ++t8) {
      const uint4 b = make_uint4(bc[0], bc[1], bc[2], bc[3]);
      uint32_t nx[4] = {0u, 0u, 0u, 0u};
      auto dq_next = [&](int i) __attribute__((always_inline)) { nx[i] = t8 < NTL - 1 ? dq_reg(w, t8 + 1, i) : dq_reg(wn, 0, i); };
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        if (rb & 1) Act<TX>::mma_acc_nw_after(acc[rb][t8], __builtin_bit_cast(uint4, a[rb]), b, nx[rb >> 1]);
        else Act<TX>::mma_acc_nw(acc[rb][t8], __builtin_bit_cast(uint4, a[rb]), b);
        if (!(rb & 1)) dq_next(rb >> 1);
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) bc[i] = nx[i];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) bcarry[i] = bc[i];
    Act<TX>::mma_accv_nw(rsum[0], __builtin_bit_cast(uint4, ar[0]), ones);
    Act<TX>::mma_accv_nw(rsum[1], __builtin_bit_cast(uint4, ar[1]), ones);
    __builtin_amdgcn_sched_barrier(0);
  };

  write_a(1, 0);
  load_a(1, 2);
  __syncthreads();
  read_a(0, 0, 0);
#pragma unroll
  for (int i = 0; i < 4; ++i) bcarry[i] = dq_reg(wr[0][0], 0, i);
  __builtin_amdgcn_sched_barrier(0);

  // stage s with ring position cur = s & 1 (a compile-time constant: registers are indexed with it)
  auto stage = [&](auto curc, int s) __attribute__((always_inline)) {
    constexpr int cur = decltype(curc)::value;
    read_a(1, cur, 1);
    __builtin_amdgcn_sched_barrier(0);
    step_pipe(aq[0], aqr[0], wr[cur][0], wr[cur][1]);
    load_w(cur, 0, s + 2);
    write_a(cur, cur ^ 1);
    load_a(cur, s + 3);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    read_a(0, cur ^ 1, 0);
    __builtin_amdgcn_sched_barrier(0);
    step_pipe(aq[1], aqr[1], wr[cur][1], wr[cur ^ 1][0]);
    load_w(cur, 1, s + 2);
    __builtin_amdgcn_sched_barrier(0);
  };
  int s = 0;
  for (; s + 2 <= NS; s += 2) {
    stage(std::integral_constant<int, 0>{}, s);
    stage(std::integral_constant<int, 1>{}, s + 1);
  }
  if (s < NS) stage(std::integral_constant<int, 0>{}, s);

  mma_drain();
  float sc[8], zf[8];
  rg_params8(scale, zs_dtype, col, C, sc);
  rg_params8(zero, zs_dtype, col, C, zf);
  // the row sums change hands through the LDS of the activations, once every wavefront has left the loop
  floatx4 *rs_lds = reinterpret_cast<floatx4 *>(a_lds);                 // [row block][lane]
  __syncthreads();
  rs_lds[(2 * wk) * 64 + lane] = rsum[0];
  rs_lds[(2 * wk + 1) * 64 + lane] = rsum[1];
  __syncthreads();
  float zfa[8];
#pragma unroll
  for (int t8 = 0; t8 < 8; ++t8) zfa[t8] = BF ? 128.f + zf[t8] : zf[t8];
  // acc[rb][t8][r] = sum_k x[m][k] code[k][col + t8] 2^-24 (bf16: code + 128, unscaled), rs_lds[rb][lane][r] =
  // sum_k x[m][k], m = m0 + 16 rb + 4 g + r
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const floatx4 rs4 = rs_lds[(rb0 + rb) * 64 + lane];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = m0 + 16 * (rb0 + rb) + 4 * g + r;
      if (m >= M) continue;
      const float rs = rs4[r];
      TX o[8];
#pragma unroll
      for (int t8 = 0; t8 < NTL; ++t8)
        o[t8] = Act<TX>::out(sc[t8] * ((BF ? acc[rb][t8][r] : 0x1p24f * acc[rb][t8][r]) - zfa[t8] * rs));
      if (out32 != nullptr) {
        // fp32 rows: the fp16 result widened and scaled back by the row's power of two (exact)
        const int e = rowexp[m];
        float *d32 = out32 + (int64_t)m * C + col;
        float f[8];
#pragma unroll
        for (int t8 = 0; t8 < NTL; ++t8) f[t8] = ldexpf((float)o[t8], e);
        *reinterpret_cast<float4 *>(d32) = make_float4(f[0], f[1], f[2], f[3]);
        if constexpr (!HALF) *reinterpret_cast<float4 *>(d32 + 4) = make_float4(f[4], f[5], f[6], f[7]);
        continue;
      }
      if constexpr (HALF) *reinterpret_cast<uint2 *>(out + (int64_t)m * C + col) = *reinterpret_cast<const uint2 *>(o);
      else *reinterpret_cast<uint4 *>(out + (int64_t)m * C + col) = *reinterpret_cast<const uint4 *>(o);
    }
  }
}

// The transposed product on the same tiling: out[M, K] = x[M, C] @ ((code - zero) * scale)^T, fp16 rows.  A
// wavefront owns 128 rows x 128 output columns (64 packed rows) over all channels; the contraction runs along the
// channels, in stages of 64, whose activations the four wavefronts share through LDS as above; the weight operand
// is built as in qmatmul_reg_bwd.hip (lane (l16, g): 8 channels of packed row j0 + 16 jg + l16; scale and
// -zero * scale of all channels converted once into LDS).  C % 64 == 0, whole 512-column tiles only.
//
// bf16 rows: (code - zero) * scale rounded to bf16 would lose precision, so, as in qmatmul_reg_bwd.hip, the scale
// goes to the other operand, once per workgroup on the way into LDS: A = bf16(x * scale), B = 128 + code (a byte
// permute under 0x43: 1.75 vector instructions per operand register against fp16's four), and the term
// t[m] = sum_c A (128 + zero) comes from a ninth MFMA tile whose B operand holds 128 + rint(zero) in its first eight
// columns and zero - rint(zero) in the others; wavefront wk accumulates it for row blocks 2 wk and 2 wk + 1 only
// and the four exchange it through LDS at the end, as the forward kernel's row sums.  Tables: scale in fp32 and
// the offset pair, 8 C bytes (C <= 16384).
//
// BITS = 8 (one code per byte, fp16 rows): a packed row is one output column, a wavefront's 128 columns are eight
// groups of 16 rows with one product tile each; the bytes of two channels that a permute pairs are fp16 subnormals
// {a 2^-24, b 2^-24}, and one packed fma with the channels' scale 2^15 and -zero scale 2^-9 (the tables hold
// them in that form) yields (code - zero) scale 2^-9: two vector instructions per operand register; the epilogue
// multiplies by 512.
template <typename TX, int HALFM = 0, int BITS = 4>
__global__ __launch_bounds__(256, 1) void qmm_bwd_wide_kernel(const TX *x, int M, const uint8_t *pk, int R, int C,
                                                               const void *zero, const void *scale, int zs_dtype,
                                                               TX *out, float *out32, const int32_t *rowexp, int jbase) {
  // jbase: first packed row of this launch's tiles (where the output columns are dealt over two launches)
  constexpr bool BF = Act<TX>::BF;
  // (HALFM != 0: 128 rows x 256 output columns.  1: the four wavefronts as two row halves x two column halves, as
  //  forward.  2 (SIDE): the four wavefronts side by side with all 128 rows and 64 columns each: half the groups of
  //  packed rows per wavefront and everything else as in the full tile, so the operand instructions per MFMA stay
  //  what they are there, while the activation reads from LDS double.  M = 2048 on 4096 x 11008: 8-bit codes
  //  239 -> 204 us, 4-bit codes with fp16 rows 221 -> 211 us, with bf16 rows 223 -> 228 us, which therefore keep
  //  form 1)
  static_assert(BITS == 4 || (BITS == 8 && !BF), "8-bit codes: fp16 rows");
  constexpr bool HALF = HALFM != 0, SIDE = HALFM == 2;
  constexpr int RB = (HALF && !SIDE) ? 4 : 8, TB = 8, NG = (BITS == 8 ? 8 : 4) / (SIDE ? 2 : 1);
  // fp16: halves sc[C], halves nzs[C]; bf16: floats sf[C], words {128 + rint z | z - rint z}[C]; then the stages
  extern __shared__ __attribute__((aligned(16))) float wide_lds[];
  _Float16 *tab_s = reinterpret_cast<_Float16 *>(wide_lds);
  _Float16 *tab_nz = tab_s + C;
  float *tab_sf = wide_lds;
  uint32_t *tab_zt = reinterpret_cast<uint32_t *>(wide_lds + C);
  u32x4_t *a_lds = reinterpret_cast<u32x4_t *>(wide_lds + (BF ? 2 : 1) * C);   // [slot][k-step of the stage][row block][lane]
  typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));
  typedef float f2_t __attribute__((ext_vector_type(2)));
  const int tid = threadIdx.x, lane = tid & 63, wk = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 4, l16 = lane & 15;
  int tx, ty;
  qmm_tile_coords(tx, ty);
  const int rb0 = (HALF && !SIDE) ? 4 * (wk >> 1) : 0;
  const int m0 = ty * 128, j0 = jbase + ((HALF && !SIDE) ? tx * 2 + (wk & 1) : tx * 4 + wk) * (16 * NG);
  const int NS = C >> 6;

  const int kc = tid & 7;
  int xoff[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) xoff[i] = min(m0 + (tid >> 3) + 32 * i, M - 1) * C + 8 * kc;            // M C < 2^31
  // Which eight channels of a stage lane group g multiplies in k-step h is free as long as both operands agree:
  // here they are 16 g + 8 h .. + 7, so that a lane's weights of BOTH k-steps are 16 contiguous bytes of a packed row,
  // one load per row and stage (the address unit's cost is per instruction, and these loads touch sixteen rows
  // each).  Chunk kc of the activations (channels 8 kc .. + 7) therefore belongs to k-step kc & 1, lane group kc >> 1.
  const int kg = kc >> 1, kh = kc & 1;
  const int dst0 = (kh * TB + (tid >> 7)) * 64 + 16 * kg + (((tid >> 3) & 15) ^ (4 * kg) ^ (2 * kh));
  const uint8_t *wpj[NG];
#pragma unroll
  for (int jg = 0; jg < NG; ++jg) wpj[jg] = pk + (int64_t)(j0 + 16 * jg + l16) * C + 16 * g;

  u32x4_t stg[2][4];
  uint4 wr[2][NG];
  u32x4_t aq[2][RB];
  u32x4_t aqr[2][2];                             // bf16: row blocks 2 wk, 2 wk + 1 once more, for the ninth tile
  auto load_a = [&](int p, int s) __attribute__((always_inline)) {
    const int so = 64 * min(s, NS - 1);
#pragma unroll
    for (int i = 0; i < 4; ++i) stg[p][i] = *reinterpret_cast<const u32x4_t *>(x + xoff[i] + so);
  };
  auto write_a = [&](int p, int slot) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 4; ++i) a_lds[slot * (2 * TB * 64) + dst0 + 2 * 64 * i] = stg[p][i];
  };
  // bf16 rows: the pieces of stage s in stg[p] times their channels' scale, rounded to bf16 (register e of piece i
  // is unit 4 i + e; the units of a stage are spread over the MFMAs of the k-step in front of its write_a)
  auto scales_of = [&](int s, float (&sf)[8]) __attribute__((always_inline)) {
    const float *sp = tab_sf + 64 * min(s, NS - 1) + 8 * kc;
    const float4 f0 = *reinterpret_cast<const float4 *>(sp), f1 = *reinterpret_cast<const float4 *>(sp + 4);
    sf[0] = f0.x; sf[1] = f0.y; sf[2] = f0.z; sf[3] = f0.w; sf[4] = f1.x; sf[5] = f1.y; sf[6] = f1.z; sf[7] = f1.w;
  };
  auto scale_unit = [&](int p, int u, const float (&sf)[8]) __attribute__((always_inline)) {
    const int i = u >> 2, e = u & 3;
    stg[p][i][e] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f2_t{Act<TX>::lo(stg[p][i][e]) * sf[2 * e],
                                                                             Act<TX>::hi(stg[p][i][e]) * sf[2 * e + 1]}, bf2_t));
  };
  auto load_w = [&](int p, int s) __attribute__((always_inline)) {
    const int c = 64 * min(s, NS - 1);
#pragma unroll
    for (int jg = 0; jg < NG; ++jg) wr[p][jg] = *reinterpret_cast<const uint4 *>(wpj[jg] + c);
  };
  // the weights of k-step h of the stage in slot p
  auto half_w = [&](int p, int h, uint2 (&w)[NG]) __attribute__((always_inline)) {
#pragma unroll
    for (int jg = 0; jg < NG; ++jg) w[jg] = h ? make_uint2(wr[p][jg].z, wr[p][jg].w) : make_uint2(wr[p][jg].x, wr[p][jg].y);
  };
  auto read_a = [&](int q, int slot, int h) __attribute__((always_inline)) {
    const int sl = lane ^ (4 * g) ^ (2 * h);                         // (bank swizzle, as in the forward kernel)
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) aq[q][rb] = a_lds[((slot * 2 + h) * TB + rb0 + rb) * 64 + sl];
    if constexpr (BF) {
#pragma unroll
      for (int j = 0; j < 2; ++j) aqr[q][j] = a_lds[((slot * 2 + h) * TB + 2 * wk + j) * 64 + sl];
    }
  };

  load_a(1, 0);
  load_w(0, 0);
  load_a(0, 1);
  load_w(1, 1);
  __builtin_amdgcn_sched_barrier(0);
  // per-channel constants of all channels
  for (int c = tid; c < C; c += 256) {
    const float z = rg_param(zero, zs_dtype, c), sc = rg_param(scale, zs_dtype, c);
    if constexpr (BF) {
      const float zi = fminf(fmaxf(rintf(z), -128.f), 128.f);       // 128 + zi: an integer bf16 holds exactly
      tab_sf[c] = sc;
      tab_zt[c] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f2_t{128.f + zi, z - zi}, bf2_t));
    } else if constexpr (BITS == 8) {
      tab_s[c] = (_Float16)(sc * 32768.f);
      tab_nz[c] = (_Float16)(-z * sc * 0x1p-9f);
    } else {
      tab_s[c] = (_Float16)sc;
      tab_nz[c] = (_Float16)(-z * sc);
    }
  }

  floatx4 acc[RB][8];
#pragma unroll
  for (int i = 0; i < RB; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};
  const half2_t k1024 = half2_t{(_Float16)1024.f, (_Float16)1024.f};
  const half2_t k16th = half2_t{(_Float16)0.0625f, (_Float16)0.0625f}, k64 = half2_t{(_Float16)64.f, (_Float16)64.f};
  uint32_t c64 = 0x64646464u, c43 = 0x43434343u;
  asm volatile("" : "+v"(c64), "+v"(c43));
  floatx4 rsum[2] = {floatx4{0.f, 0.f, 0.f, 0.f}, floatx4{0.f, 0.f, 0.f, 0.f}};

  // operand registers of a pair of output columns (low / high nibbles) from word `word` of a packed row: codes of the
  // two channels that `sel` picks, times their scale, minus zero * scale
  auto build_lo = [&](uint32_t word, uint32_t sel, uint32_t scw, uint32_t nzw) __attribute__((always_inline)) -> uint32_t {
    if constexpr (BF) return __builtin_amdgcn_perm(c43, word & 0x0F0F0F0Fu, sel);      // {128 + code, 128 + code}
    if constexpr (BITS == 8) {
      // sel pairs bytes (2 e, 2 e + 1) under zero bytes: {a 2^-24, b 2^-24} as fp16 subnormals
      const half2_t v = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0u, word, sel | 0x0c000c00u));
      return __builtin_bit_cast(uint32_t, v * __builtin_bit_cast(half2_t, scw) + __builtin_bit_cast(half2_t, nzw));
    }
    const half2_t cl = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(c64, word & 0x0F0F0F0Fu, sel)) - k1024;
    return __builtin_bit_cast(uint32_t, cl * __builtin_bit_cast(half2_t, scw) + __builtin_bit_cast(half2_t, nzw));
  };
  auto build_hi = [&](uint32_t word, uint32_t sel, uint32_t scw, uint32_t nzw) __attribute__((always_inline)) -> uint32_t {
    if constexpr (BF) return __builtin_amdgcn_perm(c43, (word >> 4) & 0x0F0F0F0Fu, sel);
    const half2_t ch = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(c64, word & 0xF0F0F0F0u, sel)) * k16th - k64;
    return __builtin_bit_cast(uint32_t, ch * __builtin_bit_cast(half2_t, scw) + __builtin_bit_cast(half2_t, nzw));
  };
  // One k-step of 32 channels starting at channel c0 (of which this lane's operand registers hold 8 g .. 8 g + 7),
  // software-pipelined: under the 16 MFMAs of a group of 16 packed rows the operand registers of the next group are
  // built (of the next k-step's first group under the last), four vector instructions behind every second MFMA,
  // and the MFMA after them counts as a use of the fresh register; so the MFMAs go without wait states, as in the
  // forward kernel.  carry_l / carry_h: the operand registers of the group about to be multiplied.
  uint32_t carry_l[4], carry_h[4];
  // scp: (bf16 rows) -1, or the stg slot whose pieces, those of stage sst, are scaled under this k-step's MFMAs
  auto compute = [&](const u32x4_t (&a)[RB], const u32x4_t (&ar)[2], const uint2 (&w)[NG], const uint2 &wnext, int c0,
                     int c0n, auto scp, int sst) __attribute__((always_inline)) {
    constexpr int SCP = BF ? decltype(scp)::value : -1;
    float sf[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if constexpr (SCP >= 0) scales_of(sst, sf);
    const int ti = c0 + 16 * g, tin = c0n + 16 * g;
    uint32_t sw[4] = {0u, 0u, 0u, 0u}, nw[4] = {0u, 0u, 0u, 0u}, swn[4] = {0u, 0u, 0u, 0u}, nwn[4] = {0u, 0u, 0u, 0u};
    uint4 bz = make_uint4(0u, 0u, 0u, 0u);
    if constexpr (BF) {
      // the ninth tile's B operand of this k-step: columns < 8 the integer parts, the others the fractions
      const uint4 z0 = *reinterpret_cast<const uint4 *>(tab_zt + ti), z1 = *reinterpret_cast<const uint4 *>(tab_zt + ti + 4);
      const uint32_t zsel = l16 < 8 ? 0x05040100u : 0x07060302u;
      bz = make_uint4(__builtin_amdgcn_perm(z0.y, z0.x, zsel), __builtin_amdgcn_perm(z0.w, z0.z, zsel),
                      __builtin_amdgcn_perm(z1.y, z1.x, zsel), __builtin_amdgcn_perm(z1.w, z1.z, zsel));
      // a use here, in front of the k-step's MFMAs: left to the compiler the four permutes sink down to their
      // first use, the ninth tile's MFMA at the end, which must not follow them directly
      asm volatile("" ::"v"(bz.x), "v"(bz.y), "v"(bz.z), "v"(bz.w));
    } else {
      const uint4 s4 = *reinterpret_cast<const uint4 *>(tab_s + ti), n4 = *reinterpret_cast<const uint4 *>(tab_nz + ti);
      const uint4 s4n = *reinterpret_cast<const uint4 *>(tab_s + tin), n4n = *reinterpret_cast<const uint4 *>(tab_nz + tin);
      sw[0] = s4.x; sw[1] = s4.y; sw[2] = s4.z; sw[3] = s4.w;
      nw[0] = n4.x; nw[1] = n4.y; nw[2] = n4.z; nw[3] = n4.w;
      swn[0] = s4n.x; swn[1] = s4n.y; swn[2] = s4n.z; swn[3] = s4n.w;
      nwn[0] = n4n.x; nwn[1] = n4n.y; nwn[2] = n4n.z; nwn[3] = n4n.w;
    }
    uint32_t bl[4] = {carry_l[0], carry_l[1], carry_l[2], carry_l[3]};
    uint32_t bh[4] = {carry_h[0], carry_h[1], carry_h[2], carry_h[3]};
#pragma unroll
    for (int jg = 0; jg < NG; ++jg) {
      const uint4 Bl = make_uint4(bl[0], bl[1], bl[2], bl[3]), Bh = make_uint4(bh[0], bh[1], bh[2], bh[3]);
      const uint2 wsrc = jg + 1 < NG ? w[jg + 1 < NG ? jg + 1 : 0] : wnext;
      uint32_t nl[4] = {0u, 0u, 0u, 0u}, nh[4] = {0u, 0u, 0u, 0u};
      auto piece = [&](int pc) __attribute__((always_inline)) {      // piece pc = 2 i + (0: low, 1: high nibbles)
        const int i = pc >> 1;
        const uint32_t word = i < 2 ? wsrc.x : wsrc.y;
        const uint32_t sel = (i & 1) ? 0x04030402u : 0x04010400u;            // bytes (2e, 2e+1) under 0x64
        const uint32_t scw = jg + 1 < NG ? sw[i] : swn[i], nzw = jg + 1 < NG ? nw[i] : nwn[i];
        if (pc & 1) nh[i] = build_hi(word, sel, scw, nzw);
        else nl[i] = build_lo(word, sel, scw, nzw);
      };
      if constexpr (BITS == 8) {
        // one product tile per group of 16 packed rows: RB MFMAs, the four operand registers of the next group
        // behind them (as the forward kernel's k-step)
        auto piece8 = [&](int i) __attribute__((always_inline)) {
          const uint32_t word = i < 2 ? wsrc.x : wsrc.y;
          const uint32_t sel = (i & 1) ? 0x04030402u : 0x04010400u;
          nl[i] = build_lo(word, sel, jg + 1 < NG ? sw[i] : swn[i], jg + 1 < NG ? nw[i] : nwn[i]);
        };
        if constexpr (!HALF || SIDE) {
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) {
            if (rb & 1) Act<TX>::mma_acc_nw_after(acc[rb][jg], __builtin_bit_cast(uint4, a[rb]), Bl, nl[rb >> 1]);
            else Act<TX>::mma_acc_nw(acc[rb][jg], __builtin_bit_cast(uint4, a[rb]), Bl);
            if (!(rb & 1)) piece8(rb >> 1);
            __builtin_amdgcn_sched_barrier(0);
          }
        } else {
          Act<TX>::mma_acc_nw(acc[0][jg], __builtin_bit_cast(uint4, a[0]), Bl);
          piece8(0);
          piece8(1);
          __builtin_amdgcn_sched_barrier(0);
          Act<TX>::mma_acc_nw_after2(acc[1][jg], __builtin_bit_cast(uint4, a[1]), Bl, nl[0], nl[1]);
          piece8(2);
          __builtin_amdgcn_sched_barrier(0);
          Act<TX>::mma_acc_nw_after(acc[2][jg], __builtin_bit_cast(uint4, a[2]), Bl, nl[2]);
          piece8(3);
          __builtin_amdgcn_sched_barrier(0);
          Act<TX>::mma_acc_nw_after(acc[3][jg], __builtin_bit_cast(uint4, a[3]), Bl, nl[3]);
          __builtin_amdgcn_sched_barrier(0);
        }
      } else if constexpr (!HALF || SIDE) {
#pragma unroll
        for (int n = 0; n < 16; ++n) {
          const int rb = n >> 1, i = n >> 2;
          const bool hi_piece = (n >> 1) & 1;
          if (!(n & 1)) {
            Act<TX>::mma_acc_nw(acc[rb][2 * jg], __builtin_bit_cast(uint4, a[rb]), Bl);
            piece(n >> 1);
          } else {
            Act<TX>::mma_acc_nw_after(acc[rb][2 * jg + 1], __builtin_bit_cast(uint4, a[rb]), Bh, hi_piece ? nh[i] : nl[i]);
            // the sixteen units of the stage being scaled, spread over the k-step's groups
            if constexpr (SCP >= 0) {
              if constexpr (NG == 4) {
                if ((n & 3) == 1) scale_unit(SCP, 4 * jg + (n >> 2), sf);
              } else {
                scale_unit(SCP, 8 * jg + (n >> 1), sf);
              }
            }
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
        // eight MFMAs per group: two pieces behind the first, one behind each of the next six, none behind the last
        Act<TX>::mma_acc_nw(acc[0][2 * jg], __builtin_bit_cast(uint4, a[0]), Bl);
        piece(0);
        piece(1);
        __builtin_amdgcn_sched_barrier(0);
        Act<TX>::mma_acc_nw_after2(acc[0][2 * jg + 1], __builtin_bit_cast(uint4, a[0]), Bh, nl[0], nh[0]);
        piece(2);
        if constexpr (SCP >= 0) scale_unit(SCP, 4 * jg, sf);
        __builtin_amdgcn_sched_barrier(0);
        Act<TX>::mma_acc_nw_after(acc[1][2 * jg], __builtin_bit_cast(uint4, a[1]), Bl, nl[1]);
        piece(3);
        __builtin_amdgcn_sched_barrier(0);
        Act<TX>::mma_acc_nw_after(acc[1][2 * jg + 1], __builtin_bit_cast(uint4, a[1]), Bh, nh[1]);
        piece(4);
        if constexpr (SCP >= 0) scale_unit(SCP, 4 * jg + 1, sf);
        __builtin_amdgcn_sched_barrier(0);
        Act<TX>::mma_acc_nw_after(acc[2][2 * jg], __builtin_bit_cast(uint4, a[2]), Bl, nl[2]);
        piece(5);
        __builtin_amdgcn_sched_barrier(0);
        Act<TX>::mma_acc_nw_after(acc[2][2 * jg + 1], __builtin_bit_cast(uint4, a[2]), Bh, nh[2]);
        piece(6);
        if constexpr (SCP >= 0) scale_unit(SCP, 4 * jg + 2, sf);
        __builtin_amdgcn_sched_barrier(0);
        Act<TX>::mma_acc_nw_after(acc[3][2 * jg], __builtin_bit_cast(uint4, a[3]), Bl, nl[3]);
        piece(7);
        __builtin_amdgcn_sched_barrier(0);
        Act<TX>::mma_acc_nw_after(acc[3][2 * jg + 1], __builtin_bit_cast(uint4, a[3]), Bh, nh[3]);
        if constexpr (SCP >= 0) scale_unit(SCP, 4 * jg + 3, sf);
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        bl[i] = nl[i];
        bh[i] = nh[i];
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      carry_l[i] = bl[i];
      carry_h[i] = bh[i];
    }
    if constexpr (BF) {
      Act<TX>::mma_accv_nw(rsum[0], __builtin_bit_cast(uint4, ar[0]), bz);
      Act<TX>::mma_accv_nw(rsum[1], __builtin_bit_cast(uint4, ar[1]), bz);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  if constexpr (BF) {
    __syncthreads();                                                 // the scales are in LDS
    float sf[8];
    scales_of(0, sf);
#pragma unroll
    for (int u = 0; u < 16; ++u) scale_unit(1, u, sf);
  }
  write_a(1, 0);
  load_a(1, 2);
  __syncthreads();                                                   // stage 0 and the tables are in LDS
  {
    uint32_t sw[4] = {0u, 0u, 0u, 0u}, nw[4] = {0u, 0u, 0u, 0u};
    if constexpr (!BF) {
      const uint4 s4 = *reinterpret_cast<const uint4 *>(tab_s + 16 * g), n4 = *reinterpret_cast<const uint4 *>(tab_nz + 16 * g);
      sw[0] = s4.x; sw[1] = s4.y; sw[2] = s4.z; sw[3] = s4.w;
      nw[0] = n4.x; nw[1] = n4.y; nw[2] = n4.z; nw[3] = n4.w;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t word = i < 2 ? wr[0][0].x : wr[0][0].y, sel = (i & 1) ? 0x04030402u : 0x04010400u;
      carry_l[i] = build_lo(word, sel, sw[i], nw[i]);
      carry_h[i] = BITS == 8 ? 0u : build_hi(word, sel, sw[i], nw[i]);
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  read_a(0, 0, 0);                                                   // (LDS reads between the build and the first MFMA)
  __builtin_amdgcn_sched_barrier(0);

  auto stage = [&](auto curc, int s) __attribute__((always_inline)) {
    constexpr int cur = decltype(curc)::value;
    read_a(1, cur, 1);
    __builtin_amdgcn_sched_barrier(0);
    uint2 w0[NG], w1[NG];
    half_w(cur, 0, w0);
    half_w(cur, 1, w1);
    compute(aq[0], aqr[0], w0, w1[0], 64 * s, 64 * s + 8, std::integral_constant<int, cur>{}, s + 1);
    __builtin_amdgcn_sched_barrier(0);
    write_a(cur, cur ^ 1);
    load_a(cur, s + 3);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    read_a(0, cur ^ 1, 0);
    __builtin_amdgcn_sched_barrier(0);
    compute(aq[1], aqr[1], w1, make_uint2(wr[cur ^ 1][0].x, wr[cur ^ 1][0].y), 64 * s + 8, min(64 * s + 64, C - 64),
            std::integral_constant<int, -1>{}, 0);
    __builtin_amdgcn_sched_barrier(0);
    load_w(cur, s + 2);
    __builtin_amdgcn_sched_barrier(0);
  };
  int s = 0;
  for (; s + 2 <= NS; s += 2) {
    stage(std::integral_constant<int, 0>{}, s);
    stage(std::integral_constant<int, 1>{}, s + 1);
  }
  if (s < NS) stage(std::integral_constant<int, 0>{}, s);

  mma_drain();
  // acc[rb][2 jg + e][r] = out[m0 + 16 rb + 4 g + r][2 (j0 + 16 jg + l16) + e]  (bf16: plus t[m], see above)
  const int64_t KO = BITS == 8 ? (int64_t)R : 2 * (int64_t)R;
  floatx4 *rs_lds = reinterpret_cast<floatx4 *>(a_lds);                 // [row block][lane]
  if constexpr (BF) {
    __syncthreads();                                                   // every wavefront has left the loop
    rs_lds[(2 * wk) * 64 + lane] = rsum[0];
    rs_lds[(2 * wk + 1) * 64 + lane] = rsum[1];
    __syncthreads();
  }
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    floatx4 t4 = floatx4{0.f, 0.f, 0.f, 0.f};
    if constexpr (BF) {
      t4 = rs_lds[(rb0 + rb) * 64 + lane];
#pragma unroll
      for (int r = 0; r < 4; ++r) t4[r] += __shfl_xor(t4[r], 8);      // integer parts' term + fractions' term
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = m0 + 16 * (rb0 + rb) + 4 * g + r;
      if (m >= M) continue;
      if (out32 != nullptr) {
        const int e = rowexp[m];
        float *orow32 = out32 + (int64_t)m * KO;
        if constexpr (BITS == 8) {
#pragma unroll
          for (int jg = 0; jg < NG; ++jg)
            orow32[j0 + 16 * jg + l16] = ldexpf((float)Act<TX>::out(512.f * acc[rb][jg][r]), e);
          continue;
        }
#pragma unroll
        for (int jg = 0; jg < NG; ++jg) {
          const int j = j0 + 16 * jg + l16;
          *reinterpret_cast<float2 *>(orow32 + 2 * j) = make_float2(ldexpf((float)Act<TX>::out(acc[rb][2 * jg][r]), e),
                                                                    ldexpf((float)Act<TX>::out(acc[rb][2 * jg + 1][r]), e));
        }
        continue;
      }
      TX *orow = out + (int64_t)m * KO;
      if constexpr (BITS == 8) {
#pragma unroll
        for (int jg = 0; jg < NG; ++jg) orow[j0 + 16 * jg + l16] = Act<TX>::out(512.f * acc[rb][jg][r]);
        continue;
      }
#pragma unroll
      for (int jg = 0; jg < NG; ++jg) {
        const int j = j0 + 16 * jg + l16;
        TX o2[2] = {Act<TX>::out(acc[rb][2 * jg][r] - t4[r]), Act<TX>::out(acc[rb][2 * jg + 1][r] - t4[r])};
        *reinterpret_cast<uint32_t *>(orow + 2 * j) = *reinterpret_cast<const uint32_t *>(o2);
      }
    }
  }
}

template <typename TX, int BITS = 4>
int launch_wide(hipStream_t st, const void *x, int64_t M, const uint8_t *pk, int64_t R, int64_t C, const void *zero,
                const void *scale, int zs_dtype, void *out, int64_t wide_x, float *out32, const int32_t *rowexp,
                bool half, int64_t c0) {
  const int64_t K = BITS == 8 ? R : 2 * R;
  int64_t rows_max = ((1LL << 31) - 1) / K;
  if (rows_max > 65535LL * 128) rows_max = 65535LL * 128;
  rows_max -= rows_max % 128;
  if (rows_max < 128) return GPTQ_HIP_EINVAL;
  for (int64_t r0 = 0; r0 < M; r0 += rows_max) {
    const int64_t rows = M - r0 < rows_max ? M - r0 : rows_max;
    const dim3 grid((unsigned)wide_x, (unsigned)ceil_div64(rows, 128), 1);
    if (half)
      hipLaunchKernelGGL((qmm_fwd_wide_kernel<4, TX, true, BITS>), grid, dim3(256), 0, st, (const TX *)x + r0 * K, (int)rows,
                         (int)K, pk, (int)C, zero, scale, zs_dtype, (TX *)out + r0 * C, (int)c0,
                         out32 ? out32 + r0 * C : nullptr, rowexp ? rowexp + r0 : nullptr);
    else
      hipLaunchKernelGGL((qmm_fwd_wide_kernel<4, TX, false, BITS>), grid, dim3(256), 0, st, (const TX *)x + r0 * K, (int)rows,
                         (int)K, pk, (int)C, zero, scale, zs_dtype, (TX *)out + r0 * C, (int)c0,
                         out32 ? out32 + r0 * C : nullptr, rowexp ? rowexp + r0 : nullptr);
    GPTQ_CHECK_LAUNCH();
  }
  return GPTQ_HIP_OK;
}

template <typename TX, int BITS = 4>
int launch_bwd_wide(hipStream_t st, const void *x, int64_t M, const uint8_t *pk, int64_t R, int64_t C, const void *zero,
                    const void *scale, int zs_dtype, void *out, int64_t wide_x, float *out32, const int32_t *rowexp,
                    bool half, int64_t jbase) {
  // 128 x 256 tiles: four wavefronts side by side, except for bf16 rows (two by two)
  auto kern = half ? qmm_bwd_wide_kernel<TX, Act<TX>::BF ? 1 : 2, BITS> : qmm_bwd_wide_kernel<TX, 0, BITS>;
  const int lds = (int)((Act<TX>::BF ? 8 : 4) * C + 2 * 2 * 8 * 64 * 16);
  if (!gptq_raise_lds_limit(reinterpret_cast<const void *>(kern), lds)) return GPTQ_HIP_ELAUNCH;
  const int64_t KO = BITS == 8 ? R : 2 * R;
  int64_t rows_max = ((1LL << 31) - 1) / C;
  if (rows_max > 65535LL * 128) rows_max = 65535LL * 128;
  rows_max -= rows_max % 128;
  if (rows_max < 128) return GPTQ_HIP_EINVAL;
  for (int64_t r0 = 0; r0 < M; r0 += rows_max) {
    const int64_t rows = M - r0 < rows_max ? M - r0 : rows_max;
    const dim3 grid((unsigned)wide_x, (unsigned)ceil_div64(rows, 128), 1);
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, st, (const TX *)x + r0 * C, (int)rows, pk, (int)R, (int)C, zero,
                       scale, zs_dtype, (TX *)out + r0 * KO, out32 ? out32 + r0 * KO : nullptr,
                       rowexp ? rowexp + r0 : nullptr, (int)jbase);
    GPTQ_CHECK_LAUNCH();
  }
  return GPTQ_HIP_OK;
}

}  // namespace

namespace qmm {

// whole rounds of 256 workgroups (one per CU); a single round that is at least 7/8 full is taken as it is
static int64_t wide_rounds(int64_t full_x, int64_t tiles_y) {
  const int64_t wgs = full_x * tiles_y;
  if (wgs >= 256) return (wgs / 256) * 256 / tiles_y;
  return wgs >= 224 ? full_x : 0;
}

int64_t wide_fwd_tiles(int64_t M, int64_t R, int64_t C, bool aligned, bool *half, int bits) {
  const int64_t K = bits == 8 ? R : 2 * R;
  *half = false;
  if (!aligned || K % 64 != 0 || K < 512 || C % 8 != 0 || M < 256) return 0;
  const int64_t tiles_y = ceil_div64(M, 128);
  const int64_t n = wide_rounds(C / 512, tiles_y);
  if (n > 0) return n;
  // 128 x 256 tiles of four 64 x 128 wavefronts where the 512-channel tiles are under a round
  *half = true;
  return wide_rounds(C / 256, tiles_y);
}

int wide_fwd_launch(hipStream_t st, const void *x, int x_dtype, int64_t M, const uint8_t *pk, int64_t R, int64_t C,
                    const void *zero, const void *scale, int zs_dtype, void *out, int64_t wide_x, bool half, float *out32,
                    const int32_t *rowexp, int bits, int64_t c0) {
  if (zs_dtype != GPTQ_HIP_F32 && zs_dtype != GPTQ_HIP_F16 && zs_dtype != GPTQ_HIP_BF16) return GPTQ_HIP_EDTYPE;
  if (wide_x < 1 || c0 < 0 || c0 % 128 != 0 || c0 + wide_x * (half ? 256 : 512) > C) return GPTQ_HIP_EINVAL;
  if (bits == 8) {
    if (x_dtype != GPTQ_HIP_F16) return GPTQ_HIP_EDTYPE;
    return launch_wide<__half, 8>(st, x, M, pk, R, C, zero, scale, zs_dtype, out, wide_x, out32, rowexp, half, c0);
  }
  if (x_dtype == GPTQ_HIP_BF16)
    return launch_wide<__hip_bfloat16>(st, x, M, pk, R, C, zero, scale, zs_dtype, out, wide_x, out32, rowexp, half, c0);
  if (x_dtype != GPTQ_HIP_F16) return GPTQ_HIP_EDTYPE;
  return launch_wide<__half>(st, x, M, pk, R, C, zero, scale, zs_dtype, out, wide_x, out32, rowexp, half, c0);
}

int64_t wide_bwd_tiles(int64_t M, int64_t R, int64_t C, bool aligned, bool *half, bool bf16, int bits) {
  *half = false;
  const int64_t rows512 = bits == 8 ? 512 : 256;       // packed rows of 512 output columns
  // (the constants of all channels and the stages share the LDS: 4 C + 32 KB; bf16 rows: 8 C + 32 KB)
  if (!aligned || C % 64 != 0 || C < 512 || C > (bf16 ? 16384 : 30720) || M < 256) return 0;
  const int64_t tiles_y = ceil_div64(M, 128);
  if (bits == 8 && bf16) return 0;
  const int64_t n = wide_rounds(R / rows512, tiles_y);
  if (n > 0) return n;
  *half = true;
  return wide_rounds(R / (rows512 / 2), tiles_y);
}

int wide_bwd_launch(hipStream_t st, const void *x, int64_t M, const uint8_t *pk, int64_t R, int64_t C, const void *zero,
                    const void *scale, int zs_dtype, void *out, int64_t wide_x, bool half, float *out32,
                    const int32_t *rowexp, bool bf16, int bits, int64_t jbase) {
  if (zs_dtype != GPTQ_HIP_F32 && zs_dtype != GPTQ_HIP_F16 && zs_dtype != GPTQ_HIP_BF16) return GPTQ_HIP_EDTYPE;
  if (wide_x < 1 || jbase < 0 || jbase % 64 != 0 || jbase + wide_x * (half ? 128 : 256) * (bits == 8 ? 2 : 1) > R)
    return GPTQ_HIP_EINVAL;
  if (bits == 8) {
    if (bf16) return GPTQ_HIP_EDTYPE;
    return launch_bwd_wide<__half, 8>(st, x, M, pk, R, C, zero, scale, zs_dtype, out, wide_x, out32, rowexp, half, jbase);
  }
  if (bf16) {
    if (out32 || C > 16384) return GPTQ_HIP_EINVAL;
    return launch_bwd_wide<__hip_bfloat16>(st, x, M, pk, R, C, zero, scale, zs_dtype, out, wide_x, nullptr, nullptr, half,
                                           jbase);
  }
  return launch_bwd_wide<__half>(st, x, M, pk, R, C, zero, scale, zs_dtype, out, wide_x, out32, rowexp, half, jbase);
}

}  // namespace qmm
