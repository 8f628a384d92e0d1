// Packed-weight matmul, transposed form (the VJP of the forward product), both MFMA operands built in registers:
//   out[M, K] = x[M, C] @ ((code - zero) * scale)^T,  codes packed as 4-bit pairs (K = 2 R) or bytes (K = R).
// Serves fp16 activations of more than 64 rows (128-row tiles), and what qmm_bwd_gemm_kernel does not: 8-bit
// codes, shapes whose rows are not multiples of 16 channels or that are not 16-byte aligned, and products whose
// output tiles are too few to fill the chip without a split over the contraction.
//
// The contraction runs along the channels, the contiguous axis of the packed matrix.  A workgroup owns a
// 64 x 128 or 128 x 128 output tile (128 output columns = 64 packed rows of nibble pairs or 128 rows of bytes) over a range
// of k-steps of 32 channels; its four wavefronts take the k-steps t % 4 == wavefront; no staging of the
// operands in LDS, no barrier in the k loop.
//   B: lane (l16, g) loads the 8 bytes = channels 32 t + 8 g .. + 7 of packed row j0 + 16 jg + l16 for every
//      group jg of 16 packed rows.  fp16: a byte permute against 0x64 gives 1024 + code pairs, one packed
//      add (or, for high nibbles, one packed fma with 1/16) makes them exact small integers, one packed fma
//      applies scale and -zero * scale of the two channels.  bf16: (code - zero) * scale rounded to bf16 would
//      lose precision, so the scale goes to the other operand: A = bf16(x * scale), B = 128 + code (4-bit)
//      or code (8-bit), exact in bf16, and the term sum_c A (offset + zero) comes from a ninth MFMA tile whose
//      B operand holds offset + rint(zero) in its first eight columns and zero - rint(zero) in the others.
//   A: lane (l16, g) loads the 16 bytes x[m][32 t + 8 g .. + 7] of row m = 16 rb + l16.
// The per-channel constants (fp16: scale and -zero * scale; bf16: scale in fp32 and the offset pair) of the
// workgroup's channel range are converted once into LDS, which the final reduction reuses.
#include "qmatmul_reg.h"
#include "qmm_reg_common.h"
#include <type_traits>

namespace {

using namespace qmm;

constexpr int RGB_RB = 4;                      // row blocks per pass of the final reduction (and per 64-row tile)
constexpr int RGB_RING = 3;
constexpr int RGB_LDS_BYTES = 4 * RGB_RB * RG_NT * RG_TILE_FLOATS * 4;     // 144 KB: the reduction buffer
constexpr int RGB_MAX_STEPS = RGB_LDS_BYTES / 8 / 32;                      // k-steps whose constants fit (8 B / channel)

// RB = 4: 64-row tiles.  RB = 8: 128-row tiles, a dequantised operand serves twice the rows;
// the 8 x 8 product tiles fill the 256 accumulation registers and every MFMA accumulates in place
// (Act::mma_acc, read only after mma_drain; bf16's ninth tiles in vector registers), the reduction runs in two
// passes of four row blocks.
template <int BITS, bool RAGGED, typename TX, int RB = RGB_RB>
__global__ __launch_bounds__(256) void qmm_bwd_reg_kernel(const TX *x, int M, const uint8_t *pk, int R, int C,
                                                          const void *zero, const void *scale, int zs_dtype,
                                                          TX *out, float *part, int32_t *counters, int S,
                                                          int steps_per_split, int group_size, int tx0, float *out32,
                                                          const int32_t *rowexp) {
  constexpr bool BF = Act<TX>::BF;
  constexpr int RING = RB == 8 ? 2 : RGB_RING;
  constexpr bool TIED = RB == 8;
  constexpr int RBT = RGB_RB, NH = RB / RBT;      // row blocks per pass of the final reduction, passes
  static_assert(RB == 4 || RB == 8, "64- or 128-row tiles");
  constexpr int NG = BITS == 4 ? 4 : 8;          // groups of 16 packed rows: 8 MFMA tiles either way
  constexpr int NJ = 16 * NG;
  extern __shared__ __attribute__((aligned(16))) float rg_lds[];
  __shared__ int s_flag;
  const int tid = threadIdx.x, lane = tid & 63, wk = tid >> 6;
  const int g = lane >> 4, l16 = lane & 15;
  int tx, ty;
  qmm_tile_coords(tx, ty);
  // (tx0: first column tile of this launch, where the columns are dealt over two launches)
  const int j0 = (tx + tx0) * NJ, m0 = ty * (16 * RB), split = blockIdx.z;
  const int T = (C + 31) >> 5;
  const int t_begin = split * steps_per_split, t_end = min(T, t_begin + steps_per_split);
  const int range = max(0, t_end - t_begin);
  const int iters = range > wk ? (range - wk + 3) >> 2 : 0;
  const bool has_tail = (C & 31) != 0 && iters > 0 && (t_begin + 4 * (iters - 1) + wk == T - 1);
  const int iters_full = iters - (has_tail ? 1 : 0);

  // ---- constants of the channels [32 t_begin, 32 t_end) into LDS (zero beyond C)
  //   fp16: halves sc[n], then halves nzs[n] = -zero scale;  bf16: floats sf[n], then words {off + rint z | z - rint z}
  const int c_begin = 32 * t_begin, nch = 32 * range;
  _Float16 *tab_s = reinterpret_cast<_Float16 *>(rg_lds);
  _Float16 *tab_nz = tab_s + nch;
  float *tab_sf = rg_lds;
  uint32_t *tab_zt = reinterpret_cast<uint32_t *>(rg_lds + nch);
  auto put = [&](int i, float s, float z) __attribute__((always_inline)) {
    const int c = c_begin + i;
    if (BF) {
      typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));
      typedef float f2_t __attribute__((ext_vector_type(2)));
      // off + zi must be an integer bf16 holds exactly (magnitude <= 256)
      const float lim = BITS == 4 ? 128.f : 256.f, off = BITS == 4 ? 128.f : 0.f;
      const float zi = fminf(fmaxf(rintf(z), -lim), lim);
      tab_sf[i] = c < C ? s : 0.f;
      tab_zt[i] = c < C ? __builtin_bit_cast(uint32_t, __builtin_convertvector(f2_t{off + zi, z - zi}, bf2_t)) : 0u;
    } else {
      tab_s[i] = (_Float16)(c < C ? s : 0.f);
      tab_nz[i] = (_Float16)(c < C ? -z * s : 0.f);
    }
  };
  // the element type is switched on outside the loops, and a thread's loads of a round are independent:
  // four channels' zero and scale in flight per thread instead of one load at a time
  // grouped parameters ([K / group, C] tables): the tile's 128 output columns lie in one group
  const int64_t prow = group_size > 0 ? (int64_t)(((int64_t)j0 * (BITS == 4 ? 2 : 1)) / group_size) * C : 0;
  auto fill = [&](auto *zp0, auto *sp0) __attribute__((always_inline)) {
    auto *zp = zp0 + prow;
    auto *sp = sp0 + prow;
    for (int i0 = tid; i0 < nch; i0 += 4 * 256) {
      float zv[4], sv[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int c = min(c_begin + i0 + u * 256, C - 1);
        zv[u] = to_f32(zp[c]);
        sv[u] = to_f32(sp[c]);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (i0 + u * 256 < nch) put(i0 + u * 256, sv[u], zv[u]);
    }
  };
  if (zs_dtype == GPTQ_HIP_F32) fill(reinterpret_cast<const float *>(zero), reinterpret_cast<const float *>(scale));
  else if (zs_dtype == GPTQ_HIP_F16) fill(reinterpret_cast<const __half *>(zero), reinterpret_cast<const __half *>(scale));
  else fill(reinterpret_cast<const __hip_bfloat16 *>(zero), reinterpret_cast<const __hip_bfloat16 *>(scale));

  const uint8_t *wpj[NG];
#pragma unroll
  for (int jg = 0; jg < NG; ++jg) wpj[jg] = pk + (int64_t)min(j0 + 16 * jg + l16, R - 1) * C;
  int xrow[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) xrow[rb] = min(m0 + 16 * rb + l16, M - 1) * C;      // M C < 2^31

  uint2 wr[RING][NG];
  uint4 aq[RING][RB];
  auto load_step = [&](int slot, int s) __attribute__((always_inline)) {
    // (steps past this workgroup's range re-read its own last k-step, a cache hit, not the next split's rows)
    const int t = min(t_begin + 4 * s + wk, max(t_end - 1, 0));
    const int c = min(32 * t + 8 * g, C - 8);                        // C >= 8
#pragma unroll
    for (int jg = 0; jg < NG; ++jg) wr[slot][jg] = rg_load8<RAGGED>(wpj[jg] + c);
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) aq[slot][rb] = rg_load16<RAGGED>(x + xrow[rb] + c);
  };

  floatx4 acc[RB][RG_NT];
#pragma unroll
  for (int i = 0; i < RB; ++i)
#pragma unroll
    for (int j = 0; j < RG_NT; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

#pragma unroll
  for (int u = 0; u < RING; ++u) load_step(u, u);
  __syncthreads();                                                   // the tables are complete

  const half2_t k1024 = half2_t{(_Float16)1024.f, (_Float16)1024.f};
  const half2_t k16th = half2_t{(_Float16)0.0625f, (_Float16)0.0625f}, k64 = half2_t{(_Float16)64.f, (_Float16)64.f};
  uint32_t c64 = 0x64646464u, c43 = 0x43434343u;
  asm volatile("" : "+v"(c64), "+v"(c43));

  auto compute = [&](int slot, int s, auto masked) __attribute__((always_inline)) {
    constexpr bool MASKED = decltype(masked)::value;
    const int t = t_begin + 4 * s + wk;
    const int k0 = 32 * t + 8 * g;                                   // first channel of this lane's chunk
    const int ti = k0 - c_begin;                                     // its place in the tables
    uint4 a[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      a[rb] = aq[slot][rb];
      if (MASKED) a[rb] = rg_mask_tail(a[rb], k0, min(k0, C - 8), C);
    }
    uint2 w[NG];
#pragma unroll
    for (int jg = 0; jg < NG; ++jg)
      w[jg] = MASKED ? rg_shr_bytes(wr[slot][jg], min(max(k0 - (C - 8), 0), 8)) : wr[slot][jg];

    if constexpr (!BF) {
      const uint4 s4 = *reinterpret_cast<const uint4 *>(tab_s + ti);
      const uint4 n4 = *reinterpret_cast<const uint4 *>(tab_nz + ti);
      const uint32_t sw[4] = {s4.x, s4.y, s4.z, s4.w}, nw[4] = {n4.x, n4.y, n4.z, n4.w};
#pragma unroll
      for (int jg = 0; jg < NG; ++jg) {
        uint32_t lo4[4], hi4[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t word = i < 2 ? w[jg].x : w[jg].y;
          const uint32_t sel = (i & 1) ? 0x04030402u : 0x04010400u;          // bytes (2e, 2e+1) under 0x64
          const half2_t sc = __builtin_bit_cast(half2_t, sw[i]), nz = __builtin_bit_cast(half2_t, nw[i]);
          if constexpr (BITS == 4) {
            const half2_t cl = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(c64, word & 0x0F0F0F0Fu, sel)) - k1024;
            const half2_t ch = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(c64, word & 0xF0F0F0F0u, sel)) * k16th - k64;
            lo4[i] = __builtin_bit_cast(uint32_t, cl * sc + nz);
            hi4[i] = __builtin_bit_cast(uint32_t, ch * sc + nz);
          } else {
            const half2_t cl = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(c64, word, sel)) - k1024;
            lo4[i] = __builtin_bit_cast(uint32_t, cl * sc + nz);
          }
        }
        const uint4 bl = make_uint4(lo4[0], lo4[1], lo4[2], lo4[3]);
        if constexpr (BITS == 4) {
          const uint4 bh = make_uint4(hi4[0], hi4[1], hi4[2], hi4[3]);
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) {
            if constexpr (TIED) {
              Act<TX>::mma_acc(acc[rb][2 * jg], a[rb], bl);
              Act<TX>::mma_acc(acc[rb][2 * jg + 1], a[rb], bh);
            } else {
              acc[rb][2 * jg] = Act<TX>::mma(a[rb], bl, acc[rb][2 * jg]);
              acc[rb][2 * jg + 1] = Act<TX>::mma(a[rb], bh, acc[rb][2 * jg + 1]);
            }
          }
        } else {
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) {
            if constexpr (TIED) Act<TX>::mma_acc(acc[rb][jg], a[rb], bl);
            else acc[rb][jg] = Act<TX>::mma(a[rb], bl, acc[rb][jg]);
          }
        }
      }
    } else {
      typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));
      typedef float f2_t __attribute__((ext_vector_type(2)));
      // A = bf16(x * scale); the ninth tile's B operand from the offset pairs
      float sf[8];
      uint32_t zt[8];
      {
        const float4 f0 = *reinterpret_cast<const float4 *>(tab_sf + ti), f1 = *reinterpret_cast<const float4 *>(tab_sf + ti + 4);
        const uint4 z0 = *reinterpret_cast<const uint4 *>(tab_zt + ti), z1 = *reinterpret_cast<const uint4 *>(tab_zt + ti + 4);
        sf[0] = f0.x; sf[1] = f0.y; sf[2] = f0.z; sf[3] = f0.w; sf[4] = f1.x; sf[5] = f1.y; sf[6] = f1.z; sf[7] = f1.w;
        zt[0] = z0.x; zt[1] = z0.y; zt[2] = z0.z; zt[3] = z0.w; zt[4] = z1.x; zt[5] = z1.y; zt[6] = z1.z; zt[7] = z1.w;
      }
      const uint32_t zsel = l16 < 8 ? 0x05040100u : 0x07060302u;
      const uint4 bz = make_uint4(__builtin_amdgcn_perm(zt[1], zt[0], zsel), __builtin_amdgcn_perm(zt[3], zt[2], zsel),
                                  __builtin_amdgcn_perm(zt[5], zt[4], zsel), __builtin_amdgcn_perm(zt[7], zt[6], zsel));
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const uint32_t aw[4] = {a[rb].x, a[rb].y, a[rb].z, a[rb].w};
        uint32_t o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
          o[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f2_t{Act<TX>::lo(aw[i]) * sf[2 * i],
                                                                           Act<TX>::hi(aw[i]) * sf[2 * i + 1]}, bf2_t));
        a[rb] = make_uint4(o[0], o[1], o[2], o[3]);
        if constexpr (TIED) Act<TX>::mma_accv(acc[rb][8], a[rb], bz);      // (the ninth tiles live in vector registers)
        else acc[rb][8] = Act<TX>::mma(a[rb], bz, acc[rb][8]);
      }
#pragma unroll
      for (int jg = 0; jg < NG; ++jg) {
        uint32_t lo4[4], hi4[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t word = i < 2 ? w[jg].x : w[jg].y;
          if constexpr (BITS == 4) {
            const uint32_t sel = (i & 1) ? 0x04030402u : 0x04010400u;        // bytes (2e, 2e+1) under 0x43: 128 + code
            lo4[i] = __builtin_amdgcn_perm(c43, word & 0x0F0F0F0Fu, sel);
            hi4[i] = __builtin_amdgcn_perm(c43, (word >> 4) & 0x0F0F0F0Fu, sel);
          } else {
            const uint32_t sh = 16u * (uint32_t)(i & 1);
            const float fa = (float)((word >> sh) & 0xFFu), fb = (float)((word >> (sh + 8u)) & 0xFFu);
            lo4[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f2_t{fa, fb}, bf2_t));
          }
        }
        const uint4 bl = make_uint4(lo4[0], lo4[1], lo4[2], lo4[3]);
        if constexpr (BITS == 4) {
          const uint4 bh = make_uint4(hi4[0], hi4[1], hi4[2], hi4[3]);
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) {
            if constexpr (TIED) {
              Act<TX>::mma_acc(acc[rb][2 * jg], a[rb], bl);
              Act<TX>::mma_acc(acc[rb][2 * jg + 1], a[rb], bh);
            } else {
              acc[rb][2 * jg] = Act<TX>::mma(a[rb], bl, acc[rb][2 * jg]);
              acc[rb][2 * jg + 1] = Act<TX>::mma(a[rb], bh, acc[rb][2 * jg + 1]);
            }
          }
        } else {
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) {
            if constexpr (TIED) Act<TX>::mma_acc(acc[rb][jg], a[rb], bl);
            else acc[rb][jg] = Act<TX>::mma(a[rb], bl, acc[rb][jg]);
          }
        }
      }
    }
  };
  const std::integral_constant<bool, false> plain{};
  const std::integral_constant<bool, true> tail{};
  int s0 = 0;
  for (; s0 + RING <= iters_full; s0 += RING) {
#pragma unroll
    for (int u = 0; u < RING; ++u) {
      compute(u, s0 + u, plain);
      load_step(u, s0 + u + RING);
    }
  }
#pragma unroll
  for (int u = 0; u < RING - 1; ++u)
    if (s0 + u < iters_full) compute(u, s0 + u, plain);
  if (has_tail) {
    const int slot = iters_full - s0;
#pragma unroll
    for (int u = 0; u < RING; ++u)
      if (u == slot) compute(u, iters_full, tail);
  }

  if constexpr (TIED) mma_drain();
  __syncthreads();                                                   // every wavefront is done with the tables
  const int64_t KO = BITS == 4 ? 2 * (int64_t)R : R;
  // one pass of the reduction per four row blocks (a 128-row tile: two passes, each with its own arrival counter
  // and partial tiles, as if it were two 64-row tiles)
  auto finish = [&](auto hc) __attribute__((always_inline)) {
    constexpr int H = decltype(hc)::value;
    floatx4 sum[RG_NT];
    const int tile = (ty * NH + H) * gridDim.x + tx;
    if (!rg_reduce<RBT, RB, H * RBT>(acc, sum, rg_lds, &s_flag, part, counters, tile, split, S)) return;
    const int rb = H * RBT + wk;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = m0 + 16 * rb + 4 * g + r;
      float t = 0.f;
      if (BF) {
        t = sum[8][r];
        t += __shfl_xor(t, 8);                  // columns < 8: the integer part's term, the others: the fraction's
      }
      if (m >= M) continue;
      if (out32 != nullptr) {
        // fp32 rows: the fp16 result widened and scaled back by the row's power of two (exact)
        const int e = rowexp[m];
        float *orow32 = out32 + (int64_t)m * KO;
#pragma unroll
        for (int jg = 0; jg < NG; ++jg) {
          const int j = j0 + 16 * jg + l16;
          if (j >= R) continue;
          if constexpr (BITS == 4) {
            const float2 o2 = make_float2(ldexpf((float)Act<TX>::out(sum[2 * jg][r] - t), e),
                                          ldexpf((float)Act<TX>::out(sum[2 * jg + 1][r] - t), e));
            *reinterpret_cast<float2 *>(orow32 + 2 * j) = o2;
          } else {
            orow32[j] = ldexpf((float)Act<TX>::out(sum[jg][r] - t), e);
          }
        }
        continue;
      }
      TX *orow = out + (int64_t)m * KO;
#pragma unroll
      for (int jg = 0; jg < NG; ++jg) {
        const int j = j0 + 16 * jg + l16;
        if (j >= R) continue;
        if constexpr (BITS == 4) {
          TX o2[2] = {Act<TX>::out(sum[2 * jg][r] - t), Act<TX>::out(sum[2 * jg + 1][r] - t)};
          *reinterpret_cast<uint32_t *>(orow + 2 * j) = *reinterpret_cast<const uint32_t *>(o2);
        } else {
          orow[j] = Act<TX>::out(sum[jg][r] - t);
        }
      }
    }
  };
  finish(std::integral_constant<int, 0>{});
  if constexpr (NH == 2) {
    __syncthreads();                                                 // the first pass's sums have been read
    finish(std::integral_constant<int, 1>{});
  }
}

template <int BITS, bool RAGGED, typename TX, int RB = RGB_RB>
int launch_inst(hipStream_t st, const RegBwdPlan &p, const void *x, int64_t M, const uint8_t *pk, int64_t R,
                int64_t C, const void *zero, const void *scale, int zs_dtype, void *out, void *wsp, int group_size,
                int64_t tx0 = 0, int64_t ntx = -1) {
  constexpr int NJ = BITS == 4 ? 64 : 128;
  auto kern = qmm_bwd_reg_kernel<BITS, RAGGED, TX, RB>;
  if (!gptq_raise_lds_limit(reinterpret_cast<const void *>(kern), RGB_LDS_BYTES)) return GPTQ_HIP_ELAUNCH;
  const int64_t KO = BITS == 4 ? 2 * R : R;
  int32_t *counters = reinterpret_cast<int32_t *>(wsp);
  float *part = reinterpret_cast<float *>(reinterpret_cast<char *>(wsp) + QMM_HEAD_BYTES);
  // column tiles [tx0, tx0 + ntx) (all of them unless the plan deals the columns over two launches)
  const int64_t tiles_all = ceil_div64(R, NJ);
  const int64_t tiles_x = ntx < 0 ? tiles_all : ntx;
  constexpr int TR = 16 * RB;                    // rows of a tile
  int64_t rows_max = ((1LL << 31) - 1) / C;
  if (rows_max > 65535LL * TR) rows_max = 65535LL * TR;
  const int64_t tiles_y_max = p.tiles / tiles_all;
  if (p.S > 1 && rows_max > tiles_y_max * TR) rows_max = tiles_y_max * TR;
  rows_max -= rows_max % TR;
  if (rows_max < TR) return GPTQ_HIP_EINVAL;
  for (int64_t r0 = 0; r0 < M; r0 += rows_max) {
    const int64_t rows = M - r0 < rows_max ? M - r0 : rows_max;
    const dim3 grid((unsigned)tiles_x, (unsigned)ceil_div64(rows, TR), (unsigned)p.S);
    hipLaunchKernelGGL(kern, grid, dim3(256), RGB_LDS_BYTES, st, (const TX *)x + r0 * C, (int)rows, pk, (int)R,
                       (int)C, zero, scale, zs_dtype, (TX *)out + r0 * KO, part, counters, p.S, p.steps, group_size,
                       (int)tx0, p.out32 ? p.out32 + r0 * KO : nullptr, p.rowexp ? p.rowexp + r0 : nullptr);
    GPTQ_CHECK_LAUNCH();
  }
  return GPTQ_HIP_OK;
}

// 128-row tiles whose last round of workgroups would be at most half full: this many trailing column tiles run on
// 64-row tiles in a second launch (as in the forward kernel's plan)
int64_t bwd_deal_tail(int64_t tiles_x, int64_t tiles_y, int64_t T) {
  if (T < 64) return 0;
  const int64_t all = tiles_x * tiles_y, full = all / 256, rem = all % 256;
  if (full < 1 || rem == 0 || rem > 128) return 0;
  const int64_t main_x = full * 256 / tiles_y, tail = tiles_x - main_x;
  return (main_x >= 1 && tail >= 1 && tail * tiles_y * 2 <= 256) ? tail : 0;
}

template <int BITS, typename TX>
int launch_bx(hipStream_t st, const RegBwdPlan &p, const void *x, int64_t M, const uint8_t *pk, int64_t R,
              int64_t C, const void *zero, const void *scale, int zs_dtype, void *out, void *ws, int group_size) {
  if (p.rb == 8) {
    const RegParts q = reg_bwd_parts(p, M, R, C, Act<TX>::BF, group_size);
    if (q.wide_x > 0) {
      const int rc = wide_bwd_launch(st, x, M, pk, R, C, zero, scale, zs_dtype, out, q.wide_x, q.half, p.out32, p.rowexp,
                                     Act<TX>::BF, BITS);
      if (rc) return rc;
    }
    if (q.wide2_x > 0) {
      const int rc = wide_bwd_launch(st, x, M, pk, R, C, zero, scale, zs_dtype, out, q.wide2_x, true, p.out32, p.rowexp,
                                     Act<TX>::BF, BITS, (BITS == 8 ? 512 : 256) * q.wide_x);
      if (rc) return rc;
    }
    if (q.main_x > 0) {
      const int rc = p.ragged ? launch_inst<BITS, true, TX, 8>(st, p, x, M, pk, R, C, zero, scale, zs_dtype, out, ws,
                                                               group_size, q.first, q.main_x)
                              : launch_inst<BITS, false, TX, 8>(st, p, x, M, pk, R, C, zero, scale, zs_dtype, out, ws,
                                                                group_size, q.first, q.main_x);
      if (rc) return rc;
    }
    if (q.tail == 0) return GPTQ_HIP_OK;
    if (p.ragged)
      return launch_inst<BITS, true, TX>(st, p, x, M, pk, R, C, zero, scale, zs_dtype, out, ws, group_size,
                                         q.first + q.main_x, q.tail);
    return launch_inst<BITS, false, TX>(st, p, x, M, pk, R, C, zero, scale, zs_dtype, out, ws, group_size,
                                        q.first + q.main_x, q.tail);
  }
  if (p.ragged) return launch_inst<BITS, true, TX>(st, p, x, M, pk, R, C, zero, scale, zs_dtype, out, ws, group_size);
  return launch_inst<BITS, false, TX>(st, p, x, M, pk, R, C, zero, scale, zs_dtype, out, ws, group_size);
}

}  // namespace

namespace qmm {

RegParts reg_bwd_parts(const RegBwdPlan &p, int64_t M, int64_t R, int64_t C, bool bf16, int group_size) {
  RegParts q{};
  const int64_t tiles_all = ceil_div64(R, p.bits == 4 ? 64 : 128);
  if (p.rb != 8) {
    q.main_x = tiles_all;
    return q;
  }
  const int64_t tiles_y = ceil_div64(M, 128);
  // 128 x 512 tiles (qmatmul_wide.hip) on the leading output columns that fill whole rounds of workgroups
  // (also where this kernel's own tiles need a split because the constants of all channels do not fit its LDS)
  if ((p.bits == 4 || !bf16) && !p.ragged && !p.no_wide && group_size == 0) {
    q.wide_x = wide_bwd_tiles(M, R, C, true, &q.half, bf16, p.bits);
    if (q.wide_x > 0) q.first = (q.half ? 2 : 4) * q.wide_x;
    // what is left behind whole rounds of 512-column tiles goes to 256-column tiles if those fill half a round or more
    if (q.wide_x > 0 && !q.half) {
      const int64_t rows512 = p.bits == 8 ? 512 : 256;
      const int64_t n2 = (R - rows512 * q.wide_x) / (rows512 / 2);
      if (n2 * tiles_y >= 128 && n2 * tiles_y <= 256) {
        q.wide2_x = n2;
        q.first += 2 * n2;
      }
    }
  }
  const int64_t rest = tiles_all - q.first;
  if (rest == 0) return q;
  // of the rest: 128-row tiles on the columns that fill whole rounds of workgroups, 64-row tiles on the others
  q.tail = q.first == 0 ? p.tail_x : (p.S == 1 ? bwd_deal_tail(rest, tiles_y, ceil_div64(C, 32)) : 0);
  if (q.first > 0 && p.S == 1 && rest * tiles_y <= 128) q.tail = rest;
  q.main_x = rest - q.tail;
  return q;
}

RegBwdPlan reg_bwd_plan(int64_t M, int64_t R, int64_t C, int bits, bool aligned, int rb) {
  RegBwdPlan p{};
  if ((bits != 4 && bits != 8) || M < 1 || C < 8 || R < 1 || R >= (1LL << 30) || C >= (1LL << 30)) return p;
  p.bits = bits;
  p.ragged = !aligned || C % 8 != 0;
  const int64_t tiles_x = ceil_div64(R, bits == 4 ? 64 : 128);
  if (tiles_x > QMM_MAX_COUNTERS) return p;
  if (rb != 4 && rb != 8) return p;
  p.rb = rb;
  const int64_t nh = p.rb / 4;                   // arrival counters per tile
  int64_t tiles_y = ceil_div64(M, 16 * p.rb);
  if (tiles_y > QMM_MAX_COUNTERS / (tiles_x * nh)) tiles_y = QMM_MAX_COUNTERS / (tiles_x * nh);
  p.tiles = tiles_x * tiles_y;
  const int64_t T = ceil_div64(C, 32);
  int64_t S = 1;
  if (p.tiles < 256) {
    S = 256 / p.tiles;
    if (S > 32) S = 32;
    while (S > 1 && T / S < 16) --S;
  }
  const int64_t s_min = ceil_div64(T, RGB_MAX_STEPS);               // the constants of a split must fit in LDS
  if (S < s_min) S = s_min;
  p.steps = (int)ceil_div64(T, S);
  p.S = (int)ceil_div64(T, p.steps);
  p.tail_x = (p.rb == 8 && p.S == 1) ? (int)bwd_deal_tail(tiles_x, tiles_y, T) : 0;
  p.part_bytes = p.S > 1 ? (size_t)p.tiles * p.S * p.rb * RG_NT * RG_TILE_FLOATS * sizeof(float) : 0;
  p.total_bytes = p.S > 1 ? QMM_HEAD_BYTES + p.part_bytes : 0;
  p.use = true;
  return p;
}

int reg_bwd_launch(hipStream_t st, const RegBwdPlan &p, const void *x, int x_dtype, int64_t M, const uint8_t *pk,
                   int64_t R, int64_t C, const void *zero, const void *scale, int zs_dtype, void *out, void *ws,
                   int group_size) {
  if (group_size < 0 || group_size % 128 != 0) return GPTQ_HIP_EINVAL;
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
