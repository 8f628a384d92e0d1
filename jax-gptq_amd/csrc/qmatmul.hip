// Packed-int4 matmul: out = x @ dequant(Wpacked)  (and the transposed form).
#include "common.h"
#include "qmm_common.h"
#include "qmatmul_reg.h"
#include <mutex>
#include <type_traits>

namespace {

using namespace qmm;

constexpr int TPB = 256;

// ---------------------------------------------------------------------------- baseline
// One thread per output element; used for shapes the tuned kernels do not cover.
template <typename TX, typename TZ, int BITS>
__global__ __launch_bounds__(TPB) void qmm_fwd_simple(const TX *x, int64_t M, const uint8_t *pk,
                                                      int64_t R, int64_t C, const TZ *zero,
                                                      const TZ *scale, TX *out, int64_t group) {
  const int64_t n = (int64_t)blockIdx.x * TPB + threadIdx.x;
  const int64_t m = blockIdx.y;
  if (n >= C) return;
  const TX *xr = x + m * (BITS == 4 ? 2 * R : R);
  float acc = 0.f, xs = 0.f;
  if (group > 0) {
    // zero / scale [K / group, C]: applied term by term
    for (int64_t j = 0; j < R; ++j) {
      const uint8_t b = pk[j * C + n];
      const int64_t gi = (BITS == 4 ? 2 * j : j) / group;
      const float z = to_f32(zero[gi * C + n]), sc = to_f32(scale[gi * C + n]);
      if (BITS == 4)
        acc += to_f32(xr[2 * j]) * (((float)(b & 0xF) - z) * sc) + to_f32(xr[2 * j + 1]) * (((float)(b >> 4) - z) * sc);
      else
        acc += to_f32(xr[j]) * (((float)b - z) * sc);
    }
    out[m * C + n] = from_f32<TX>(__half2float(__float2half_rn(acc)));
    return;
  }
  for (int64_t j = 0; j < R; ++j) {
    const uint8_t b = pk[j * C + n];
    if (BITS == 4) {
      const float x0 = to_f32(xr[2 * j]), x1 = to_f32(xr[2 * j + 1]);
      acc += x0 * (float)(b & 0xF) + x1 * (float)(b >> 4);
      xs += x0 + x1;
    } else {
      const float x0 = to_f32(xr[j]);
      acc += x0 * (float)b;
      xs += x0;
    }
  }
  const float v = to_f32(scale[n]) * (acc - to_f32(zero[n]) * xs);
  out[m * C + n] = from_f32<TX>(__half2float(__float2half_rn(v)));
}

// transposed: out[m, 2r+p] = sum_c x[m,c] * (nibble_p(pk[r,c]) - zero[c]) * scale[c]
template <typename TX, typename TZ, int BITS>
__global__ __launch_bounds__(TPB) void qmm_bwd_simple(const TX *x, int64_t M, const uint8_t *pk,
                                                      int64_t R, int64_t C, const TZ *zero0,
                                                      const TZ *scale0, TX *out, int64_t group) {
  // one wavefront per (m, r): lanes stride over c, then reduce
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * (TPB / 64) + (threadIdx.x >> 6);
  const int64_t m = blockIdx.y;
  if (r >= R) return;
  const TX *xr = x + m * C;
  // grouped parameters: the row's group (both nibbles of a packed row lie in one group: group is even)
  const int64_t prow = group > 0 ? ((BITS == 4 ? 2 * r : r) / group) * C : 0;
  const TZ *zero = zero0 + prow, *scale = scale0 + prow;
  float a0 = 0.f, a1 = 0.f;
  for (int64_t c = lane; c < C; c += 64) {
    const uint8_t b = pk[r * C + c];
    const float xv = to_f32(xr[c]) * to_f32(scale[c]);
    const float z = to_f32(zero[c]);
    a0 += xv * ((float)(BITS == 4 ? (b & 0xF) : b) - z);
    a1 += xv * ((float)(b >> 4) - z);
  }
  for (int off = 32; off > 0; off >>= 1) {
    a0 += __shfl_xor(a0, off);
    a1 += __shfl_xor(a1, off);
  }
  if (lane == 0) {
    if (BITS == 4) {
      out[m * (2 * R) + 2 * r] = from_f32<TX>(__half2float(__float2half_rn(a0)));
      out[m * (2 * R) + 2 * r + 1] = from_f32<TX>(__half2float(__float2half_rn(a1)));
    } else {
      out[m * R + r] = from_f32<TX>(__half2float(__float2half_rn(a0)));
    }
  }
}

// ---------------------------------------------------------------------------- MFMA path
// Forward, fp16 or bf16 activations, C % 16 == 0 (described for fp16; bf16 differs only in the
// dequantisation constants, see dequant_pair and the epilogue).  One workgroup owns a strip of 256 output
// channels and a slice of NW * SPW * 16 packed rows (NW wavefronts, SPW MFMA k-steps of 16
// packed rows each).  A wavefront first issues its (small, L2-resident) activation loads,
// then ALL its weight loads in one burst (SPW * 4 loads of 16 B per lane), so that the
// whole matrix is in flight at once; it dequantises in registers as the rows arrive and
// feeds v_mfma_f32_16x16x32_f16:
//   A = activations  (lane: row m = l % 16, eight k slots of lane group g = l / 16)
//   B = weights      (lane: channel 16*(l % 16) + t for t = 0..15, same eight k slots)
// Lane group g owns the packed rows 16*s + 4*g + i (i = 0..3) of k-step s (eight consecutive k,
// so its activations are 16 contiguous bytes), as the k slots
// [2r0, 2r1, 2r0+1, 2r1+1, 2r2, 2r3, 2r2+1, 2r3+1]; both operands are built in that order.
// Nibbles become fp16 with three VALU operations per four codes: one byte permute and two
// and-or with 0x6400 (fp16 1024), giving 1024 + code for even k and 1024 + 16*code for odd
// k.  Odd-k activations enter the MFMA divided by 16 (exact in fp16 but for subnormals), so
//   acc = sum_k x*code + 1024 * (sum_even x + sum_odd x/16)
// and with the two activation sums (kept per lane in fp32) the epilogue computes
//   out = scale * (acc - 1024*(se + so) - zero * (se + 16*so)),  se = sum_even x, so = sum_odd x/16.
// No LDS or barrier is used before the final cross-wavefront reduction.
constexpr int QSTRIP = 256;    // channels per workgroup

// LDS layout of one row of a wavefront's partial tile (256 floats): a lane holds the 16 channels
// 16 l16 + 4 q + j (q, j = 0..3) and stores them as four 16-byte chunks.  Chunk q of lane l16 sits at
// float offset 64 q + ((4 l16) ^ (16 q)): the sixteen lanes of a lane group then write 256
// consecutive bytes per chunk (in channel order they would be 64 bytes apart: 4 of 16 banks), and the
// XOR keeps the reading side, where consecutive threads take consecutive channels, on distinct banks.
__device__ __forceinline__ int qtile_chunk(int l16, int q) { return 64 * q + ((4 * l16) ^ (16 * q)); }
__device__ __forceinline__ int qtile_pos(int c) {      // c = channel within the strip
  const int q = (c >> 2) & 3;
  return 64 * q + ((((c >> 4) << 2) | (c & 3)) ^ (16 * q));
}

__device__ __forceinline__ uint32_t u4_comp(const uint4 &v, int w) {
  return w == 0 ? v.x : (w == 1 ? v.y : (w == 2 ? v.z : v.w));
}

// The masks live in scalar registers and the 16-bit constant in a vector register, all three opaque
// to the compiler: (p & mask) | c is then one v_and_or_b32 (a VOP3 instruction takes no literal
// and one scalar operand; from literals the compiler forms v_and_b32 + v_or_b32, ten instead of
// six vector instructions per MFMA, and the dequantisation is what bounds these kernels' tail).
struct DqConst { uint32_t mlo, mhi, c; };
template <bool BF>
__device__ __forceinline__ DqConst dq_const() {
  DqConst k{0x000F000Fu, BF ? 0x000F000Fu : 0x00F000F0u, BF ? 0x43004300u : 0x64006400u};
  asm volatile("" : "+s"(k.mlo), "+s"(k.mhi));
  asm volatile("" : "+v"(k.c));
  return k;
}

template <bool BF>
__device__ __forceinline__ void dequant_pair(const DqConst &k, uint32_t da, uint32_t db, uint32_t sel,
                                             uint32_t &lo, uint32_t &hi) {
  // bytes of p: [7:0] = row a, [23:16] = row b.
  const uint32_t p = __builtin_amdgcn_perm(db, da, sel);
  if (BF) {
    // bf16 pairs 128 + code for both nibbles (0x4300 = 128.0; its 7 mantissa bits hold the code)
    lo = (p & k.mlo) | k.c;
    hi = ((p >> 4) & k.mhi) | k.c;
  } else {
    // fp16 pairs: lo = 1024 + code (even k), hi = 1024 + 16*code (odd k); the offsets and the
    // factor 16 are undone outside the MFMA.
    lo = (p & k.mlo) | k.c;
    hi = (p & k.mhi) | k.c;
  }
}

// Cross-wavefront reduction and output of one (m-chunk, strip, split) workgroup.  On entry every
// wavefront has written its partial tile to red[wave][mrows][QSTRIP]; se / so are this lane's
// activation sums (already reduced over the four lane groups).  IT * blockDim.x >= 16 * QSTRIP.
template <int IT, typename TZ, typename TX>
__device__ __forceinline__ void qmm_reduce_and_store(float *red, int *s_last_p, int nw, int mrows,
                                                     int mvalid, int strip, int split, int m0, int M,
                                                     int C, int S, const TZ *zero, const TZ *scale,
                                                     TX *out, const QmmWs &ws, float se, float so) {
  constexpr bool BF = Act<TX>::BF;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 4, l16 = lane & 15;
  float *xs = red + (size_t)nw * mrows * QSTRIP;   // [wave][2][16]
  if (g == 0) { xs[wave * 32 + l16] = se; xs[wave * 32 + 16 + l16] = so; }
  __syncthreads();

  // epilogue value of one output from the accumulated tile sum v and the activation sums
  // (bf16: both nibbles carry 128 + code and o is the plain odd-k sum)
  auto finish = [&](float v, float e, float o, float z, float sc) -> TX {
    const float r = BF ? (v - 128.f * (e + o)) - z * (e + o)
                       : (v - 1024.f * (e + o)) - z * (e + 16.f * o);
    return Act<TX>::out(sc * r);
  };
  const int n_items = mvalid * QSTRIP;
  // x sums of this workgroup: [split][2][16] per (m-chunk, strip)
  const int64_t x1base = (((int64_t)blockIdx.z * gridDim.x + strip) * S) * 32;
  if (S == 1) {
    for (int idx = tid; idx < n_items; idx += blockDim.x) {
      const int m = idx >> 8, c = idx & 255, n = strip * QSTRIP + c;
      if (n >= C) continue;
      const float z = to_f32(zero[n]), sc = to_f32(scale[n]);
      float v = 0.f, e = 0.f, o = 0.f;
      for (int w = 0; w < nw; ++w) {
        v += red[(w * mrows + m) * QSTRIP + qtile_pos(c)];
        e += xs[w * 32 + m];
        o += xs[w * 32 + 16 + m];
      }
      out[(int64_t)(m0 + m) * C + n] = finish(v, e, o, z, sc);
    }
    return;
  }
  for (int idx = tid; idx < n_items; idx += blockDim.x) {
    const int m = idx >> 8, c = idx & 255, n = strip * QSTRIP + c;
    if (n >= C) continue;
    float v = 0.f;
    for (int w = 0; w < nw; ++w) v += red[(w * mrows + m) * QSTRIP + qtile_pos(c)];
    // agent-scope write-through store: visible to every XCD once it has completed
    __hip_atomic_store(&ws.part[((int64_t)split * M + m0 + m) * C + n], v, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
  }
  if (tid < 32 && (tid & 15) < mvalid) {
    float x1 = 0.f;
    for (int w = 0; w < nw; ++w) x1 += xs[w * 32 + tid];
    __hip_atomic_store(&ws.x1part[x1base + (int64_t)split * 32 + tid], x1, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
  }
  // Each thread waits for its own write-through stores, then the barrier orders all of them
  // before the ticket.  (A device-wide fence here would write back / invalidate the whole
  // L2 of the XCD, which costs tens of microseconds.)
  __syncthreads();
  if (tid == 0) {
    int32_t *ctr = ws.counters + blockIdx.z * gridDim.x + strip;
    const int ticket = atomicAdd(ctr, 1);
    *s_last_p = (ticket == S - 1);
    if (ticket == S - 1)               // every other workgroup of this strip has arrived
      __hip_atomic_store(ctr, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (!*s_last_p) return;
  // Last workgroup of the strip: sum the S partials in split order.  Loads are agent-scope
  // (never served from a stale line of this XCD's L2).  Every thread keeps all its outputs
  // in registers and walks the splits in order, so that the loads of one split (and, through
  // unrolling, of the next) are in flight together instead of one latency per output.
  if (tid < 32) {
    float a = 0.f;
    for (int sp0 = 0; sp0 < S; sp0 += 8) {
      float px[8];
#pragma unroll
      for (int u = 0; u < 8; ++u)
        px[u] = __hip_atomic_load(&ws.x1part[x1base + (int64_t)min(sp0 + u, S - 1) * 32 + tid],
                                  __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (sp0 + u < S) a += px[u];
    }
    xs[tid] = a;     // [0..15] even-k sums, [16..31] odd-k sums, per row m
  }
  // n_items <= 4096 = IT * blockDim.x.  The column parameters are fetched together with the
  // partials (one memory latency less at the end of the chain).
  float v[IT], zc[IT], scl[IT];
#pragma unroll
  for (int it = 0; it < IT; ++it) {
    const int idx = tid + it * blockDim.x;
    const int n = min(strip * QSTRIP + (idx & 255), C - 1);
    v[it] = 0.f;
    zc[it] = to_f32(zero[n]);
    scl[it] = to_f32(scale[n]);
  }
  constexpr int SPLITS_IN_FLIGHT = IT <= 8 ? 4 : 2;     // IT * this many loads per thread at a time
#pragma unroll SPLITS_IN_FLIGHT
  for (int sp = 0; sp < S; ++sp) {
    float pv[IT];
#pragma unroll
    for (int it = 0; it < IT; ++it) {
      const int idx = tid + it * blockDim.x;
      const int m = idx >> 8, n = strip * QSTRIP + (idx & 255);
      pv[it] = (idx < n_items && n < C)
                   ? __hip_atomic_load(&ws.part[((int64_t)sp * M + m0 + m) * C + n],
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                   : 0.f;
    }
#pragma unroll
    for (int it = 0; it < IT; ++it) v[it] += pv[it];
  }
  __syncthreads();
#pragma unroll
  for (int it = 0; it < IT; ++it) {
    const int idx = tid + it * blockDim.x;
    const int m = idx >> 8, n = strip * QSTRIP + (idx & 255);
    if (idx < n_items && n < C)
      out[(int64_t)(m0 + m) * C + n] = finish(v[it], xs[m], xs[16 + m], zc[it], scl[it]);
  }
}

// X16: the activations are 16-byte aligned and R % 4 == 0, so the four (k, k+1) pairs of a lane group
// (packed rows 4g .. 4g+3) are one 16-byte load instead of four 4-byte ones.
template <int SPW, typename TZ, typename TX, bool X16>
__global__ __launch_bounds__(SPW == 2 ? 1024 : 512) void qmm_fwd_mfma_kernel(
    const TX *x, int M, int K, const uint8_t *pk, int R, int C, const TZ *zero,
    const TZ *scale, TX *out, QmmWs ws, int S) {
  constexpr bool BF = Act<TX>::BF;
  extern __shared__ float red[];   // [wave][mrows][256] partial tiles, then [wave][2][16] x sums
  __shared__ int s_last;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int nw = blockDim.x >> 6;
  const int strip = blockIdx.x, split = blockIdx.y, m0 = blockIdx.z * 16;
  const int mvalid = min(16, M - m0);
  const int mrows = mvalid <= 4 ? 4 : 16;
  const int r_wave = (split * nw + wave) * SPW * 16;
  const int g = lane >> 4, l16 = lane & 15;

  // ---- activation loads (k pairs 2r, 2r+1 of this lane's rows): small, L2 resident
  uint32_t pr[SPW][4];
  {
    const TX *xr = x + (int64_t)(m0 + l16) * K;
#pragma unroll
    for (int s = 0; s < SPW; ++s) {
      if (X16) {
        const int row = r_wave + s * 16 + 4 * g;          // R % 4 == 0: the four rows are in or out together
        const uint4 v = (l16 < mvalid && row < R) ? *reinterpret_cast<const uint4 *>(xr + 2 * row)
                                                  : make_uint4(0u, 0u, 0u, 0u);
        pr[s][0] = v.x;
        pr[s][1] = v.y;
        pr[s][2] = v.z;
        pr[s][3] = v.w;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int row = r_wave + s * 16 + 4 * g + i;
          pr[s][i] = (l16 < mvalid && row < R) ? *reinterpret_cast<const uint32_t *>(xr + 2 * row) : 0u;
        }
      }
    }
  }
  // ---- weight loads of this wavefront, all in flight
  uint4 d[SPW][4];
  const int col0 = strip * QSTRIP + 16 * l16;
#pragma unroll
  for (int s = 0; s < SPW; ++s)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = r_wave + s * 16 + 4 * g + i;
      d[s][i] = (row < R && col0 < C)
                    ? *reinterpret_cast<const uint4 *>(pk + (int64_t)row * C + col0)
                    : make_uint4(0, 0, 0, 0);
    }

  // A operands: even-k slots hold x, odd-k slots hold x/16 (see above); per-lane fp32 sums of
  // exactly the fp16 values the MFMA sees, then summed over the four lane groups
  uint4 av[SPW];
  float se = 0.f, so = 0.f;
  const half2_t sixteenth = half2_t{(_Float16)0.0625f, (_Float16)0.0625f};
#pragma unroll
  for (int s = 0; s < SPW; ++s) {
    av[s].x = __builtin_amdgcn_perm(pr[s][1], pr[s][0], 0x05040100u);  // {x[2r0],   x[2r1]}
    av[s].z = __builtin_amdgcn_perm(pr[s][3], pr[s][2], 0x05040100u);
    uint32_t o0 = __builtin_amdgcn_perm(pr[s][1], pr[s][0], 0x07060302u);   // {x[2r0+1], x[2r1+1]}
    uint32_t o1 = __builtin_amdgcn_perm(pr[s][3], pr[s][2], 0x07060302u);
    if (!BF) {      // fp16: odd-k activations enter divided by 16 (bf16: both nibbles are 128 + code)
      o0 = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, o0) * sixteenth);
      o1 = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, o1) * sixteenth);
    }
    av[s].y = o0;
    av[s].w = o1;
    se += (Act<TX>::lo(av[s].x) + Act<TX>::hi(av[s].x)) + (Act<TX>::lo(av[s].z) + Act<TX>::hi(av[s].z));
    so += (Act<TX>::lo(o0) + Act<TX>::hi(o0)) + (Act<TX>::lo(o1) + Act<TX>::hi(o1));
  }
  se += __shfl_xor(se, 16);
  se += __shfl_xor(se, 32);
  so += __shfl_xor(so, 16);
  so += __shfl_xor(so, 32);

  float *slot = red + (size_t)wave * mrows * QSTRIP;
  const DqConst dqk = dq_const<BF>();
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    floatx4 acc[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < SPW; ++s) {
#pragma unroll
      for (int tt = 0; tt < 8; ++tt) {
        const int t = half * 8 + tt;
        const int w = t >> 2, tb = t & 3;
        const uint32_t sel = 0x0c000c00u | ((uint32_t)(4 + tb) << 16) | (uint32_t)tb;
        uint4 bv;
        dequant_pair<BF>(dqk, u4_comp(d[s][0], w), u4_comp(d[s][1], w), sel, bv.x, bv.y);
        dequant_pair<BF>(dqk, u4_comp(d[s][2], w), u4_comp(d[s][3], w), sel, bv.z, bv.w);
        acc[tt] = Act<TX>::mma(av[s], bv, acc[tt]);
      }
    }
    // acc[tt][r] = tile[m = 4g + r][channel 16*l16 + half*8 + tt]
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = 4 * g + r;
      if (m < mrows) {
        float *dst = slot + m * QSTRIP;
        *reinterpret_cast<float4 *>(dst + qtile_chunk(l16, 2 * half)) =
            make_float4(acc[0][r], acc[1][r], acc[2][r], acc[3][r]);
        *reinterpret_cast<float4 *>(dst + qtile_chunk(l16, 2 * half + 1)) =
            make_float4(acc[4][r], acc[5][r], acc[6][r], acc[7][r]);
      }
    }
  }
  qmm_reduce_and_store<(SPW == 2) ? 4 : 8>(red, &s_last, nw, mrows, mvalid, strip, split, m0, M, C, S,
                                           zero, scale, out, ws, se, so);
}

// 16 bytes from an address of any alignment
struct __attribute__((packed, aligned(1))) QdU4 { uint32_t x, y, z, w; };
template <bool UNALIGNED>
__device__ __forceinline__ uint4 qd_load16(const void *p) {
  if (UNALIGNED) {
    QdU4 v;
    __builtin_memcpy(&v, p, 16);
    return make_uint4(v.x, v.y, v.z, v.w);
  }
  return *reinterpret_cast<const uint4 *>(p);
}
// the 16 bytes of v moved down by `bytes` (0 .. 15) places, zeros from above
__device__ __forceinline__ uint4 qd_shr_bytes16(uint4 v, int bytes) {
  const int ws = bytes >> 2;
  const uint32_t bs = (uint32_t)(bytes & 3);
  const uint32_t w0 = ws == 0 ? v.x : (ws == 1 ? v.y : (ws == 2 ? v.z : v.w));
  const uint32_t w1 = ws == 0 ? v.y : (ws == 1 ? v.z : (ws == 2 ? v.w : 0u));
  const uint32_t w2 = ws == 0 ? v.z : (ws == 1 ? v.w : 0u);
  const uint32_t w3 = ws == 0 ? v.w : 0u;
  return make_uint4(__builtin_amdgcn_alignbyte(w1, w0, bs), __builtin_amdgcn_alignbyte(w2, w1, bs),
                    __builtin_amdgcn_alignbyte(w3, w2, bs), __builtin_amdgcn_alignbyte(0u, w3, bs));
}

// ---------------------------------------------------------------------------- MFMA path, decode
// M <= 16 on matrices that the chip holds in flight (up to ~50 MB packed).  Same operands and
// arithmetic as qmm_fwd_mfma_kernel; what differs is everything around the MFMAs, which is where
// the time of a 22 MB product goes once the loads run at the memory's pace:
//  * a workgroup of NW wavefronts owns a strip and `rows_per_split` packed rows; k-step t of
//    wavefront w is the 16 rows (t NW + w) 16 .. + 15 of that range, KS k-steps per wavefront, all
//    loads issued before anything else; k-steps past the range are skipped (wave-uniform branch);
//  * the column parameters of the outputs a thread will finish are fetched under the weight loads;
//  * ATOM (M <= 8, and larger M while the atomics stay few; MR = 1, 4 or 16 rows of the tile kept): the workgroups of a strip add their partial results to 64-bit
//    accumulators with ONE returning atomic per output: the word is value * 2^28 (fixed point,
//    a partial beyond +-65536 or not finite adds the poison 3 * 2^49 instead) << 8 | 1, so the
//    returned old word tells the caller whether it was the last of the S contributions, and the
//    last one has the complete sum in hand: it rounds, stores the output and zeroes the word.
//    Integer addition is exact and commutative: the result does not depend on the arrival order.
//    One round trip to the memory side instead of three (partial stores -> ticket -> partial
//    loads).  A poisoned sum yields NaN.  S <= 32.
//    A thread issues the atomics of all its outputs before it looks at any returned word: one round
//    trip per thread, not per output (M = 16 on 4096 x 11008: 14.2 -> 12.8 us).
//  * M > 8: the memory side retires the atomics at a limited rate (700000 of them add about 3 us);
//    where there would be more than ~760000 in at most three splits, the workgroups keep
//    qmm_reduce_and_store (ATOM = false).
constexpr int QD_MAX_SPLITS = 32;

//  * X32 (fp16 arithmetic, ATOM only): activations and result are fp32 in memory.  What the separate
//    conversion kernels do around the other paths happens in here: the power of two that brings a row's
//    largest finite magnitude into [2, 4) is either found by every workgroup itself (rowexp_in == nullptr:
//    it reads the whole row, 16 KB of L2-resident data per row at K = 4096, which pays for one or two
//    rows) or comes from x32_rowexp_kernel; the scaled activations of the workgroup's k range are rounded
//    to fp16 as they are consumed, and the workgroup that completes an output rounds it to fp16, widens it
//    and scales it back: the same arithmetic, bit for bit, without staging buffers and with one launch
//    (M = 1: 16.8 -> 9.8 us) or two (more rows) instead of three.
//  * BITS = 8 (fp16 activations): a k-step is 32 rows of one code per byte, eight 16-byte rows per lane; two
//    rows' bytes become {1024 + a, 1024 + b} with a byte permute and an or, the activations enter as they
//    are, and all offsets leave through one activation sum (the odd-k sum stays zero).
//  * RAGC (ATOM only): rows of any length C >= 16, so rows that start anywhere: unaligned 16-byte loads, and in the
//    last strip a lane whose 16 channels would reach past the row loads the row's last 16 bytes instead and
//    shifts them into place (a wave-uniform branch; the other strips run the code of the aligned form).
template <int NW, int KS, int MR, bool ATOM, bool LOOP, typename TZ, typename TX, bool X32 = false, int BITS = 4,
          bool RAGC = false>
__global__ __launch_bounds__(NW * 64) void qmm_fwd_dec_kernel(
    const std::conditional_t<X32, float, TX> *x, int M, int K, const uint8_t *pk, int R, int C, const TZ *zero,
    const TZ *scale, std::conditional_t<X32, float, TX> *out, QmmWs ws, int S, int rows_per_split,
    const int32_t *rowexp_in) {
  constexpr bool BF = Act<TX>::BF;
  static_assert(!X32 || (ATOM && !BF), "fp32 rows: fp16 arithmetic and the atomic sum only");
  static_assert(BITS == 4 || (BITS == 8 && !BF && !X32), "8-bit codes: fp16 activations");
  static_assert(!RAGC || (ATOM && !X32 && BITS == 4), "ragged rows: 4-bit codes, the atomic sum");
  constexpr int NR = BITS == 4 ? 4 : 8;          // rows per lane and k-step
  constexpr int RPS = 4 * NR;                    // rows per k-step of a wavefront
  constexpr int XK = BITS == 4 ? 2 : 1;          // k per row
  typedef std::conditional_t<X32, float, TX> XT;
  extern __shared__ float red[];   // [NW][MR][256] partial tiles, then [NW][2][16] x sums
  __shared__ int s_last;
  __shared__ float s_rowmax[X32 ? NW : 1][16];
  __shared__ int s_rowexp[16];
  // every kernel argument in registers before the first address is formed (left to itself the compiler
  // fetches them one by one where they are first used, and waits for each)
  asm volatile("" ::"s"(x), "s"(pk), "s"(zero), "s"(scale), "s"(out), "s"(ws.acc64), "s"(ws.counters), "s"(ws.part),
               "s"(ws.x1part), "s"(M), "s"(K), "s"(R), "s"(C), "s"(S), "s"(rows_per_split));
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int strip = blockIdx.x, split = blockIdx.y, m0 = blockIdx.z * 16;
  const int mvalid = min(16, M - m0);
  const int g = lane >> 4, l16 = lane & 15;
  const int r_begin = split * rows_per_split, r_end = min(R, r_begin + rows_per_split);
  // k-step t of this wavefront: packed rows r_begin + (t NW + wave) RPS + [0, RPS)
  const int groups = (r_end - r_begin + RPS - 1) / RPS;
  const int nsteps = groups > wave ? (groups - wave + NW - 1) / NW : 0;

  // One k-step of loads: the activations of the lane group's four packed rows (16 bytes = 8 k; range
  // boundaries are multiples of 4 rows, so the four rows are inside the range or outside together)
  // and the four weight rows.  Nothing is predicated per lane (a predicated load is a branch, and its
  // zero fill a register move per word: they delayed the last load of a workgroup by several hundred
  // cycles): loads past the range or past the last column read clamped, valid addresses, and such a
  // k-step enters with zero activations.  LOOP: a ring of KS k-steps that is refilled as it is consumed,
  // for matrices beyond what the chip holds in flight; otherwise all KS k-steps of the range are issued
  // at once, and a wavefront skips the k-steps that lie past its range altogether.
  struct Step { uint4 d[NR]; uint4 pr; uint4 pr2; };     // pr2: the second half of an fp32 chunk (X32)
  const bool m_ok = l16 < mvalid;
  const XT *xr = x + (int64_t)(m0 + (m_ok ? l16 : 0)) * K;
  const int col0 = min(strip * QSTRIP + 16 * l16, C - 16);
  const uint8_t *wp = pk + col0;
  // RAGC: bytes by which this lane's loads start before its first channel (its channels past the row's end, if
  // any, are never stored); only the last strip has such lanes
  const int rag_shift = RAGC ? max(0, min(strip * QSTRIP + 16 * l16, C - 1) - col0) : 0;
  const bool rag_strip = RAGC && strip * QSTRIP + QSTRIP > C;
  auto issue = [&](Step &st, int t) __attribute__((always_inline)) {
    const int rbase = r_begin + (t * NW + wave) * RPS + NR * g;
    st.pr = *reinterpret_cast<const uint4 *>(xr + XK * min(rbase, R - NR));
    if (X32) st.pr2 = *reinterpret_cast<const uint4 *>(xr + XK * min(rbase, R - NR) + 4);
    const uint8_t *row = wp + (int64_t)min(rbase, R - NR) * C;      // R % NR == 0: the rows are inside the matrix
#pragma unroll
    for (int i = 0; i < NR; ++i) st.d[i] = qd_load16<RAGC>(row + (int64_t)i * C);
  };

  const DqConst dqk = dq_const<BF>();
  const half2_t sixteenth = half2_t{(_Float16)0.0625f, (_Float16)0.0625f};
  floatx4 acc[16];
#pragma unroll
  for (int t = 0; t < 16; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
  float se = 0.f, so = 0.f;
  int xe = 0;                                     // X32: exponent of this lane's row scale
  auto consume = [&](Step &st, int t) __attribute__((always_inline)) {
    uint4 pr = st.pr;
    if constexpr (RAGC) {
      if (rag_strip) {
#pragma unroll
        for (int i = 0; i < NR; ++i) st.d[i] = qd_shr_bytes16(st.d[i], rag_shift);
      }
    }
    if constexpr (X32) {
      // eight fp32 activations -> fp16 of the scaled row, round to nearest even
      const uint32_t f[8] = {st.pr.x, st.pr.y, st.pr.z, st.pr.w, st.pr2.x, st.pr2.y, st.pr2.z, st.pr2.w};
      uint32_t h[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const __half a = __float2half_rn(ldexpf(__builtin_bit_cast(float, f[2 * i]), -xe));
        const __half b = __float2half_rn(ldexpf(__builtin_bit_cast(float, f[2 * i + 1]), -xe));
        h[i] = (uint32_t)__builtin_bit_cast(uint16_t, a) | ((uint32_t)__builtin_bit_cast(uint16_t, b) << 16);
      }
      pr = make_uint4(h[0], h[1], h[2], h[3]);
    }
    {
      const bool ok = m_ok && t < nsteps && r_begin + (t * NW + wave) * RPS + NR * g < r_end;
      pr.x = ok ? pr.x : 0u;
      pr.y = ok ? pr.y : 0u;
      pr.z = ok ? pr.z : 0u;
      pr.w = ok ? pr.w : 0u;
    }
    if constexpr (BITS == 8) {
      // the lane's eight k are its eight rows, in order: A as loaded, B register i = rows 2 i, 2 i + 1
      se += (Act<TX>::lo(pr.x) + Act<TX>::hi(pr.x)) + (Act<TX>::lo(pr.y) + Act<TX>::hi(pr.y));
      se += (Act<TX>::lo(pr.z) + Act<TX>::hi(pr.z)) + (Act<TX>::lo(pr.w) + Act<TX>::hi(pr.w));
#pragma unroll
      for (int tl = 0; tl < 16; ++tl) {
        const int w = tl >> 2, tb = tl & 3;
        const uint32_t sel = 0x0c000c00u | ((uint32_t)(4 + tb) << 16) | (uint32_t)tb;
        uint4 bv;
        bv.x = __builtin_amdgcn_perm(u4_comp(st.d[1], w), u4_comp(st.d[0], w), sel) | 0x64006400u;
        bv.y = __builtin_amdgcn_perm(u4_comp(st.d[3], w), u4_comp(st.d[2], w), sel) | 0x64006400u;
        bv.z = __builtin_amdgcn_perm(u4_comp(st.d[5 % NR], w), u4_comp(st.d[4 % NR], w), sel) | 0x64006400u;
        bv.w = __builtin_amdgcn_perm(u4_comp(st.d[7 % NR], w), u4_comp(st.d[6 % NR], w), sel) | 0x64006400u;
        acc[tl] = Act<TX>::mma(pr, bv, acc[tl]);
      }
      return;
    }
    uint4 av;
    av.x = __builtin_amdgcn_perm(pr.y, pr.x, 0x05040100u);  // {x[2r0],   x[2r1]}
    av.z = __builtin_amdgcn_perm(pr.w, pr.z, 0x05040100u);
    uint32_t o0 = __builtin_amdgcn_perm(pr.y, pr.x, 0x07060302u);   // {x[2r0+1], x[2r1+1]}
    uint32_t o1 = __builtin_amdgcn_perm(pr.w, pr.z, 0x07060302u);
    if (!BF) {      // fp16: odd-k activations enter divided by 16 (bf16: both nibbles are 128 + code)
      o0 = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, o0) * sixteenth);
      o1 = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, o1) * sixteenth);
    }
    av.y = o0;
    av.w = o1;
    se += (Act<TX>::lo(av.x) + Act<TX>::hi(av.x)) + (Act<TX>::lo(av.z) + Act<TX>::hi(av.z));
    so += (Act<TX>::lo(o0) + Act<TX>::hi(o0)) + (Act<TX>::lo(o1) + Act<TX>::hi(o1));
#pragma unroll
    for (int tl = 0; tl < 16; ++tl) {
      const int w = tl >> 2, tb = tl & 3;
      const uint32_t sel = 0x0c000c00u | ((uint32_t)(4 + tb) << 16) | (uint32_t)tb;
      uint4 bv;
      dequant_pair<BF>(dqk, u4_comp(st.d[0], w), u4_comp(st.d[1], w), sel, bv.x, bv.y);
      dequant_pair<BF>(dqk, u4_comp(st.d[2], w), u4_comp(st.d[3], w), sel, bv.z, bv.w);
      acc[tl] = Act<TX>::mma(av, bv, acc[tl]);
    }
  };

  Step ring[KS];
#pragma unroll
  for (int u = 0; u < KS; ++u)
    if (LOOP || u == 0 || u < nsteps) issue(ring[u], u);      // (wave-uniform)
  // ---- column parameters of the outputs this thread finishes, fetched under the weight loads
  constexpr int NT = NW * 64;
  constexpr int ITEMS = MR * QSTRIP;
  constexpr int IT = (ITEMS + NT - 1) / NT;
  float pz[ATOM ? IT : 1], psc[ATOM ? IT : 1];
  if (ATOM) {
#pragma unroll
    for (int it = 0; it < IT; ++it) {
      const int n = min(strip * QSTRIP + ((tid + it * NT) & 255), C - 1);
      pz[it] = to_f32(zero[n]);
      psc[it] = to_f32(scale[n]);
    }
  }
  if constexpr (X32) {
    // the scale of every row of this workgroup: largest finite magnitude over all of K (K % 8 == 0, rows 32-byte
    // aligned), under the weight loads
    if (rowexp_in == nullptr) {
      for (int m = 0; m < mvalid; ++m) {
        const float *row = x + (int64_t)(m0 + m) * K;
        float amax = 0.f;
        for (int k = tid * 4; k < K; k += NT * 4) {
          const float4 v = *reinterpret_cast<const float4 *>(row + k);
          const float a4[4] = {fabsf(v.x), fabsf(v.y), fabsf(v.z), fabsf(v.w)};
#pragma unroll
          for (int i = 0; i < 4; ++i) amax = (a4[i] <= 3.4028235e38f && a4[i] > amax) ? a4[i] : amax;   // not NaN, not infinity
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
        if (lane == 0) s_rowmax[wave][m] = amax;
      }
    }
    __syncthreads();
    if (tid < 16) {
      if (rowexp_in != nullptr) {
        s_rowexp[tid] = tid < mvalid ? rowexp_in[m0 + tid] : 0;
      } else {
        float a = 0.f;
        if (tid < mvalid) {
#pragma unroll
          for (int w = 0; w < NW; ++w) a = fmaxf(a, s_rowmax[w][tid]);
        }
        int ex = 0;
        (void)frexpf(a, &ex);                      // 2^(ex-1) <= a < 2^ex
        s_rowexp[tid] = a > 0.f ? ex - 2 : 0;      // largest magnitude of the scaled row in [2, 4)
      }
    }
    __syncthreads();
    xe = s_rowexp[l16];
  }
  // rounds a finished output to the 16-bit type; fp32 rows: widened again and scaled back (exact)
  auto store_out = [&](int m, int n, float v) __attribute__((always_inline)) {
    if constexpr (X32) out[(int64_t)(m0 + m) * C + n] = ldexpf(__half2float(__float2half_rn(v)), s_rowexp[m]);
    else out[(int64_t)(m0 + m) * C + n] = Act<TX>::out(v);
  };
  // (without this the scheduler sinks the parameter loads below the wait for the weights, and their latency
  // is paid after the last k-step instead of under it)
  __builtin_amdgcn_sched_barrier(0);
  if (LOOP) {
    int t0 = 0;
    for (; t0 + KS <= nsteps; t0 += KS) {
#pragma unroll
      for (int u = 0; u < KS; ++u) {
        consume(ring[u], t0 + u);
        issue(ring[u], t0 + u + KS);
      }
    }
    // at most KS - 1 k-steps left, all of them loaded
#pragma unroll
    for (int u = 0; u < KS - 1; ++u)
      if (t0 + u < nsteps) consume(ring[u], t0 + u);
  } else {
#pragma unroll
    for (int u = 0; u < KS; ++u) {
      if (u > 0 && u >= nsteps) break;        // wave-uniform: nothing was loaded for this k-step
      consume(ring[u], u);
    }
  }
  se += __shfl_xor(se, 16);
  se += __shfl_xor(se, 32);
  so += __shfl_xor(so, 16);
  so += __shfl_xor(so, 32);

  // acc[t][r] = tile[m = 4g + r][channel 16 * l16 + t]
  float *slot = red + (size_t)wave * MR * QSTRIP;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int m = 4 * g + r;
    if (m < MR) {
      float *dst = slot + m * QSTRIP;
#pragma unroll
      for (int q = 0; q < 4; ++q)
        *reinterpret_cast<float4 *>(dst + qtile_chunk(l16, q)) =
            make_float4(acc[4 * q][r], acc[4 * q + 1][r], acc[4 * q + 2][r], acc[4 * q + 3][r]);
    }
  }
  if constexpr (!ATOM) {
    qmm_reduce_and_store<IT>(red, &s_last, NW, MR, mvalid, strip, split, m0, M, C, S, zero, scale, out, ws,
                             se, so);
    return;
  }
  float *xs = red + (size_t)NW * MR * QSTRIP;   // [wave][2][16]
  if (g == 0) { xs[wave * 32 + l16] = se; xs[wave * 32 + 16 + l16] = so; }
  __syncthreads();
  // the activation sums over the wavefronts, once per workgroup (read per output they were 2 NW broadcast
  // reads for each of a thread's outputs: most of the LDS instructions of this phase)
  float *xt = xs + NW * 32;                     // [2][16]
  if (tid < 32) {
    float a = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) a += xs[w * 32 + tid];
    xt[tid] = a;
  }
  __syncthreads();
  // Two passes over this thread's outputs, so that its atomics are in flight together: a pass that used each
  // returned word at once would pay one round trip to the memory side per output.
  unsigned long long old[IT], word[IT];
  bool live[IT];
#pragma unroll
  for (int it = 0; it < IT; ++it) {
    const int idx = tid + it * NT;
    const int m = idx >> 8, c = idx & 255, n = strip * QSTRIP + c;
    live[it] = idx < ITEMS && m < mvalid && n < C;
    old[it] = word[it] = 0ull;
    if (!live[it]) continue;
    float v = 0.f;
    const float e = xt[m], o = xt[16 + m];
#pragma unroll
    for (int w = 0; w < NW; ++w) v += red[(w * MR + m) * QSTRIP + qtile_pos(c)];
    const float r = BF ? (v - 128.f * (e + o)) - pz[it] * (e + o)
                       : (v - 1024.f * (e + o)) - pz[it] * (e + 16.f * o);
    const float pv = psc[it] * r;
    if (S == 1) {
      store_out(m, n, pv);
      live[it] = false;
      continue;
    }
    const bool ok = fabsf(pv) <= 65536.f;                       // false for NaN, too
    const long long fx = ok ? __float2ll_rn(pv * (float)(1 << QD_FRAC)) : QD_POISON;
    word[it] = ((unsigned long long)fx << 8) + 1ull;
    old[it] = atomicAdd(ws.acc64 + (int64_t)(m0 + m) * C + n, word[it]);     // (used in the second pass only)
  }
#pragma unroll
  for (int it = 0; it < IT; ++it) {
    const unsigned long long total = old[it] + word[it];
    if (!live[it] || (int)(total & 255ull) != S) continue;      // not the last of the S contributions
    const int idx = tid + it * NT;
    const int m = idx >> 8, n = strip * QSTRIP + (idx & 255);
    const long long sum = (long long)total >> 8;
    const bool fine = sum <= (1LL << 49) && sum >= -(1LL << 49);
    const float res = fine ? (float)sum * (1.f / (float)(1 << QD_FRAC)) : __builtin_nanf("");
    store_out(m, n, res);
    __hip_atomic_store(ws.acc64 + (int64_t)(m0 + m) * C + n, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

struct FwdPlan {
  int nw, spw, S, strips, mch;
  size_t lds_bytes, counter_bytes, x1_bytes, part_bytes, total_bytes;
};

FwdPlan fwd_plan(int64_t M, int64_t R, int64_t C) {
  FwdPlan p;
  p.strips = (int)ceil_div64(C, QSTRIP);
  p.mch = (int)ceil_div64(M, 16);
  // 512 packed rows per workgroup either way: 16 wavefronts x 8 KB (all resident, small
  // tiles) for M <= 4, 8 wavefronts x 16 KB otherwise
  if (M <= 4) { p.nw = 16; p.spw = 2; }
  else { p.nw = 8; p.spw = 4; }
  p.S = (int)ceil_div64(R, (int64_t)p.nw * p.spw * 16);
  const int mrows = (M <= 4) ? 4 : 16;
  p.lds_bytes = ((size_t)p.nw * mrows * QSTRIP + (size_t)p.nw * 32) * sizeof(float);
  p.counter_bytes = QMM_HEAD_BYTES;
  p.x1_bytes = (size_t)round_up64((int64_t)p.strips * p.mch * p.S * 32 * sizeof(float), 256);
  p.part_bytes = (size_t)p.S * M * C * sizeof(float);
  p.total_bytes = p.S > 1 ? p.counter_bytes + p.x1_bytes + p.part_bytes : 0;
  return p;
}

template <int SPW, typename TZ, typename TX, bool X16>
int launch_fwd_mfma(hipStream_t st, const FwdPlan &p, const void *x, int64_t M, const uint8_t *pk,
                    int64_t R, int64_t C, const void *zero, const void *scale, void *out, void *wsp) {
  const QmmWs ws = qmm_ws(wsp, p.x1_bytes);
  auto kern = qmm_fwd_mfma_kernel<SPW, TZ, TX, X16>;
  if (p.lds_bytes > 48 * 1024 && !gptq_raise_lds_limit(reinterpret_cast<const void *>(kern), (int)p.lds_bytes))
    return GPTQ_HIP_ELAUNCH;
  // at most QMM_MAX_COUNTERS (m-chunk, strip) pairs per launch
  const int mch_per = QMM_MAX_COUNTERS / p.strips;
  if (mch_per < 1) return GPTQ_HIP_EINVAL;
  for (int c0 = 0; c0 < p.mch; c0 += mch_per) {
    const int nch = min(mch_per, p.mch - c0);
    const int64_t row0 = (int64_t)c0 * 16;
    const int64_t rows = min((int64_t)nch * 16, M - row0);
    const dim3 grid((unsigned)p.strips, (unsigned)p.S, (unsigned)nch);
    // the kernel sees the sub-problem rows [row0, row0 + rows); launches are stream ordered,
    // so they can share the workspace
    hipLaunchKernelGGL(kern, grid, dim3(p.nw * 64), p.lds_bytes, st,
                       (const TX *)x + row0 * 2 * R, (int)rows, (int)(2 * R), pk, (int)R,
                       (int)C, (const TZ *)zero, (const TZ *)scale, (TX *)out + row0 * C, ws,
                       p.S);
    GPTQ_CHECK_LAUNCH();
  }
  return GPTQ_HIP_OK;
}

// Which instantiation of qmm_fwd_dec_kernel serves M rows of a [2R, C] matrix, if any.
struct DecPlan {
  bool use, atom, loop;
  int nw, ks, mr, S, rows, strips;
  size_t lds_bytes, x1_bytes, part_bytes, total_bytes;
};

DecPlan dec_plan(int64_t M, int64_t R8, int64_t C, int bits = 4, bool ragged_c = false) {
  DecPlan p{};
  // 8-bit codes: planned in k-steps like a 4-bit matrix of half the rows (a k-step carries twice the bytes)
  if (bits == 8 && R8 % 8 != 0) return p;
  const int64_t R = bits == 8 ? R8 / 2 : R8;
  if (M < 1 || M > 16 || R % 4 != 0 || (C % 16 != 0 && !(ragged_c && bits == 4)) || C < 16 || R >= (1LL << 30) || C >= (1LL << 30)) return p;
  p.strips = (int)ceil_div64(C, QSTRIP);
  if (p.strips > QMM_MAX_COUNTERS) return p;
  p.mr = M == 1 ? 1 : (M <= 4 ? 4 : 16);
  p.atom = M * C * 8 <= QMM_ACC_BYTES;
  if (p.mr <= 4) {
    if (!p.atom) return p;
    // eight wavefronts, two workgroups per CU: as many splits as 512 slots allow, at least 128 rows each
    int64_t S = 512 / p.strips;
    if (S > QD_MAX_SPLITS) S = QD_MAX_SPLITS;
    if (S > R / 128) S = R / 128;
    if (S < 1) S = 1;
    int64_t rows = round_up64(ceil_div64(R, S), 4);
    if (rows <= 256) {
      p.nw = 8;
      p.ks = rows <= 128 ? 1 : 2;
    } else {
      // sixteen wavefronts, one workgroup per CU
      S = 256 / p.strips;
      if (S > QD_MAX_SPLITS) S = QD_MAX_SPLITS;
      if (S < 1) S = 1;
      rows = round_up64(ceil_div64(R, S), 4);
      p.nw = 16;
      p.ks = 2;
      p.loop = rows > 512;                      // beyond two k-steps per wavefront: a ring of two
    }
    p.S = (int)ceil_div64(R, rows);
    p.rows = (int)rows;
    p.x1_bytes = p.part_bytes = 0;
    p.total_bytes = p.S > 1 ? QMM_HEAD_BYTES : 0;
  } else {
    // 16 rows kept: eight wavefronts of four k-steps, one workgroup per CU (132 KB of LDS)
    p.nw = 8;
    p.ks = 4;
    p.rows = 512;
    p.S = (int)ceil_div64(R, 512);
    if ((int64_t)p.strips * p.S > 256) {
      // more than one workgroup per CU that way: as many splits as 256 slots allow, a ring of four k-steps
      int64_t S = 256 / p.strips;
      if (S > QD_MAX_SPLITS) S = QD_MAX_SPLITS;
      if (S < 1) S = 1;
      const int64_t rows = round_up64(ceil_div64(R, S), 4);
      p.S = (int)ceil_div64(R, rows);
      p.rows = (int)rows;
      p.loop = true;
    }
    if (p.S > QD_MAX_SPLITS) p.atom = false;
    // Beyond 8 rows the memory side's rate of atomics shows (700000 of them add about 3 us), and so does what the
    // other path costs, whose last workgroup reads S partial tiles: with many atomics and at most three splits
    // the workgroups keep qmm_reduce_and_store (7168 x 28672 at M = 16, S = 2, 920000 atomics: 27.3 us against
    // 28.1), otherwise the atomic sum wins (28672 x 7168, S = 9: 30.3 -> 28.9 us; 8192 x 8192, S = 8: 18.1 -> 16.6).
    if (M > 8 && M * C * p.S > 760000 && p.S < 4) p.atom = false;
    if (p.atom) {
      p.x1_bytes = p.part_bytes = 0;
      p.total_bytes = p.S > 1 ? QMM_HEAD_BYTES : 0;
    } else {
      p.x1_bytes = (size_t)round_up64((int64_t)p.strips * p.S * 32 * sizeof(float), 256);
      p.part_bytes = (size_t)p.S * M * C * sizeof(float);
      p.total_bytes = p.S > 1 ? QMM_HEAD_BYTES + p.x1_bytes + p.part_bytes : 0;
    }
  }
  p.lds_bytes = ((size_t)p.nw * p.mr * QSTRIP + (size_t)p.nw * 32 + 32) * sizeof(float);
  if (C % 16 != 0 && !p.atom) return DecPlan{};      // ragged rows: instantiated for the atomic sum only
  if (bits == 8) {
    // (the ring-loop forms of the 8-bit instantiation do not fit their register budgets: those matrices stay
    // with the register-operand kernel)
    if (p.loop) return DecPlan{};
    p.rows *= 2;
  }
  p.use = true;
  return p;
}

template <int NW, int KS, int MR, bool ATOM, bool LOOP, typename TZ, typename TX, bool X32 = false, int BITS = 4,
          bool RAGC = false>
int launch_dec_inst(hipStream_t st, const DecPlan &p, const void *x, int64_t M, const uint8_t *pk, int64_t R,
                    int64_t C, const void *zero, const void *scale, void *out, void *wsp,
                    const int32_t *rowexp = nullptr) {
  typedef std::conditional_t<X32, float, TX> XT;
  auto kern = qmm_fwd_dec_kernel<NW, KS, MR, ATOM, LOOP, TZ, TX, X32, BITS, RAGC>;
  if (p.lds_bytes > 48 * 1024 && !gptq_raise_lds_limit(reinterpret_cast<const void *>(kern), (int)p.lds_bytes))
    return GPTQ_HIP_ELAUNCH;
  const QmmWs ws = qmm_ws(wsp, p.x1_bytes);
  hipLaunchKernelGGL(kern, dim3((unsigned)p.strips, (unsigned)p.S, 1), dim3(NW * 64), p.lds_bytes, st,
                     (const XT *)x, (int)M, (int)(BITS == 4 ? 2 * R : R), pk, (int)R, (int)C, (const TZ *)zero,
                     (const TZ *)scale, (XT *)out, ws, p.S, p.rows, rowexp);
  GPTQ_CHECK_LAUNCH();
  return GPTQ_HIP_OK;
}

// fp32 rows in, fp32 rows out, fp16 arithmetic (plans with the atomic sum only); rowexp: the rows' scale
// exponents from x32_rowexp_kernel, or nullptr (the kernel finds them itself: one or two rows)
template <typename TZ>
int launch_dec_x32(hipStream_t st, const DecPlan &p, const void *x, int64_t M, const uint8_t *pk, int64_t R,
                   int64_t C, const void *zero, const void *scale, void *out, void *wsp, const int32_t *rowexp) {
#define GPTQ_DEC32(NW, KS, MR, LOOP) \
  return launch_dec_inst<NW, KS, MR, true, LOOP, TZ, __half, true>(st, p, x, M, pk, R, C, zero, scale, out, wsp, \
                                                                   rowexp)
  if (!p.atom) return GPTQ_HIP_EINVAL;
  if (p.mr == 16) {
    if (p.loop) GPTQ_DEC32(8, 4, 16, true);
    GPTQ_DEC32(8, 4, 16, false);
  }
  if (p.mr == 1) {
    if (p.loop) GPTQ_DEC32(16, 2, 1, true);
    if (p.nw == 16) GPTQ_DEC32(16, 2, 1, false);
    if (p.ks == 1) GPTQ_DEC32(8, 1, 1, false);
    GPTQ_DEC32(8, 2, 1, false);
  }
  if (p.loop) GPTQ_DEC32(16, 2, 4, true);
  if (p.nw == 16) GPTQ_DEC32(16, 2, 4, false);
  if (p.ks == 1) GPTQ_DEC32(8, 1, 4, false);
  GPTQ_DEC32(8, 2, 4, false);
#undef GPTQ_DEC32
}

template <typename TZ, typename TX>
int launch_dec_zx(hipStream_t st, const DecPlan &p, const void *x, int64_t M, const uint8_t *pk, int64_t R,
                  int64_t C, const void *zero, const void *scale, void *out, void *wsp) {
#define GPTQ_DEC(NW, KS, MR, ATOM, LOOP) \
  return launch_dec_inst<NW, KS, MR, ATOM, LOOP, TZ, TX>(st, p, x, M, pk, R, C, zero, scale, out, wsp)
  if (p.mr == 16) {
    if (p.loop && p.atom) GPTQ_DEC(8, 4, 16, true, true);
    if (p.loop) GPTQ_DEC(8, 4, 16, false, true);
    if (p.atom) GPTQ_DEC(8, 4, 16, true, false);
    GPTQ_DEC(8, 4, 16, false, false);
  }
  if (p.mr == 1) {
    if (p.loop) GPTQ_DEC(16, 2, 1, true, true);
    if (p.nw == 16) GPTQ_DEC(16, 2, 1, true, false);
    if (p.ks == 1) GPTQ_DEC(8, 1, 1, true, false);
    GPTQ_DEC(8, 2, 1, true, false);
  }
  if (p.loop) GPTQ_DEC(16, 2, 4, true, true);
  if (p.nw == 16) GPTQ_DEC(16, 2, 4, true, false);
  if (p.ks == 1) GPTQ_DEC(8, 1, 4, true, false);
  GPTQ_DEC(8, 2, 4, true, false);
#undef GPTQ_DEC
}

// 4-bit codes, rows of any length (plans with the atomic sum)
template <typename TZ, typename TX>
int launch_dec_zx_rag(hipStream_t st, const DecPlan &p, const void *x, int64_t M, const uint8_t *pk, int64_t R,
                      int64_t C, const void *zero, const void *scale, void *out, void *wsp) {
#define GPTQ_DECR(NW, KS, MR, LOOP) \
  return launch_dec_inst<NW, KS, MR, true, LOOP, TZ, TX, false, 4, true>(st, p, x, M, pk, R, C, zero, scale, out, wsp)
  if (!p.atom) return GPTQ_HIP_EINVAL;
  if (p.mr == 16) {
    if (p.loop) GPTQ_DECR(8, 4, 16, true);
    GPTQ_DECR(8, 4, 16, false);
  }
  if (p.mr == 1) {
    if (p.loop) GPTQ_DECR(16, 2, 1, true);
    if (p.nw == 16) GPTQ_DECR(16, 2, 1, false);
    if (p.ks == 1) GPTQ_DECR(8, 1, 1, false);
    GPTQ_DECR(8, 2, 1, false);
  }
  if (p.loop) GPTQ_DECR(16, 2, 4, true);
  if (p.nw == 16) GPTQ_DECR(16, 2, 4, false);
  if (p.ks == 1) GPTQ_DECR(8, 1, 4, false);
  GPTQ_DECR(8, 2, 4, false);
#undef GPTQ_DECR
}
template <typename TZ>
int launch_dec_z_rag(hipStream_t st, const DecPlan &p, const void *x, int x_dtype, int64_t M, const uint8_t *pk,
                     int64_t R, int64_t C, const void *zero, const void *scale, void *out, void *wsp) {
  if (x_dtype == GPTQ_HIP_BF16)
    return launch_dec_zx_rag<TZ, __hip_bfloat16>(st, p, x, M, pk, R, C, zero, scale, out, wsp);
  return launch_dec_zx_rag<TZ, __half>(st, p, x, M, pk, R, C, zero, scale, out, wsp);
}

// 8-bit codes, fp16 activations
template <typename TZ>
int launch_dec_z8(hipStream_t st, const DecPlan &p, const void *x, int64_t M, const uint8_t *pk, int64_t R,
                  int64_t C, const void *zero, const void *scale, void *out, void *wsp) {
#define GPTQ_DEC8(NW, KS, MR, ATOM, LOOP) \
  return launch_dec_inst<NW, KS, MR, ATOM, LOOP, TZ, __half, false, 8>(st, p, x, M, pk, R, C, zero, scale, out, wsp)
  if (p.loop) return GPTQ_HIP_EINVAL;
  if (p.mr == 16) {
    if (p.atom) GPTQ_DEC8(8, 4, 16, true, false);
    GPTQ_DEC8(8, 4, 16, false, false);
  }
  if (p.mr == 1) {
    if (p.nw == 16) GPTQ_DEC8(16, 2, 1, true, false);
    if (p.ks == 1) GPTQ_DEC8(8, 1, 1, true, false);
    GPTQ_DEC8(8, 2, 1, true, false);
  }
  if (p.nw == 16) GPTQ_DEC8(16, 2, 4, true, false);
  if (p.ks == 1) GPTQ_DEC8(8, 1, 4, true, false);
  GPTQ_DEC8(8, 2, 4, true, false);
#undef GPTQ_DEC8
}

template <typename TZ>
int launch_dec_z(hipStream_t st, const DecPlan &p, const void *x, int x_dtype, int64_t M, const uint8_t *pk,
                 int64_t R, int64_t C, const void *zero, const void *scale, void *out, void *wsp) {
  if (x_dtype == GPTQ_HIP_BF16)
    return launch_dec_zx<TZ, __hip_bfloat16>(st, p, x, M, pk, R, C, zero, scale, out, wsp);
  return launch_dec_zx<TZ, __half>(st, p, x, M, pk, R, C, zero, scale, out, wsp);
}

template <typename TZ, typename TX>
int launch_fwd_mfma_zx(hipStream_t st, const FwdPlan &p, const void *x, int64_t M, const uint8_t *pk,
                       int64_t R, int64_t C, const void *zero, const void *scale, void *out,
                       void *wsp) {
  if (p.spw == 2) return launch_fwd_mfma<2, TZ, TX, false>(st, p, x, M, pk, R, C, zero, scale, out, wsp);
  // the m-chunks of one call start 16 rows (32 R bytes) apart: aligned together with x when R % 4 == 0
  if ((reinterpret_cast<uintptr_t>(x) & 15) == 0 && R % 4 == 0)
    return launch_fwd_mfma<4, TZ, TX, true>(st, p, x, M, pk, R, C, zero, scale, out, wsp);
  return launch_fwd_mfma<4, TZ, TX, false>(st, p, x, M, pk, R, C, zero, scale, out, wsp);
}

template <typename TZ>
int launch_fwd_mfma_z(hipStream_t st, const FwdPlan &p, const void *x, int x_dtype, int64_t M,
                      const uint8_t *pk, int64_t R, int64_t C, const void *zero, const void *scale,
                      void *out, void *wsp) {
  if (x_dtype == GPTQ_HIP_BF16)
    return launch_fwd_mfma_zx<TZ, __hip_bfloat16>(st, p, x, M, pk, R, C, zero, scale, out, wsp);
  return launch_fwd_mfma_zx<TZ, __half>(st, p, x, M, pk, R, C, zero, scale, out, wsp);
}

// ---------------------------------------------------------------------------- tiled kernel, LDS layout
// 64 x 128 x 64 tiles of the transposed kernel below: row pitch 72 halves and a skew of 8 words per 16-channel group
// keep both the transposing stores and the operand reads free of bank conflicts.
constexpr int GBM = 64, GBK = 64;
constexpr int GPITCH = GBK + 8;                 // halves per LDS row
constexpr int GGROUP = 16 * GPITCH + 16;        // halves per 16-row group (16 = the 8-word skew)

__device__ __forceinline__ int g_off(int row, int k) {   // LDS offset (halves) of element [row][k]
  return (row >> 4) * GGROUP + (row & 15) * GPITCH + k;
}

// ---------------------------------------------------------------------------- transposed
// out[m, 2j + h] = sum_n x[m, n] * scale[n] * (nibble_h(pk[j, n]) - zero[n]): the VJP of the
// forward product (op.py:71-81, kernel.py:141-253).  The contraction runs along the packed
// rows, which is the contiguous axis of the packed matrix, so the weights need no transpose
// on their way into LDS: a thread loads 16 bytes of one packed row (16 consecutive n), turns
// them into the 16 + 16 fp16 values (code - zero[n]) * scale[n] of output columns 2j and
// 2j + 1 (byte permute against 0x64 gives 1024 + code, the subtraction of 1024 is exact, one
// packed fma applies zero and scale) and stores them k-contiguous, which is the operand
// order.  Same 64 x 128 x 64 tiles, LDS layout, register ring and MFMA loop as the forward
// kernel; zero and scale of a stage's 64 channels travel in the ring with the weights.
//
// bf16 activations: (code - zero) * scale rounded to bf16 would lose five of fp16's mantissa bits,
// so the scale goes to the other operand.  A = bf16(x[m, n] * scale[n]) (rounded once, on the
// way into LDS), B = 128 + code (one byte permute against 0x43, exact), and
//   out[m, 2j + h] = sum_n A[m, n] * (128 + code) - t[m],  t[m] = sum_n A[m, n] * (128 + zero[n]),
// with t[m] summed in fp32 by the staging threads from the rounded values the MFMA sees.
template <typename TZ> struct ZsRaw;          // 16 consecutive zero / scale values as loaded
template <> struct ZsRaw<__half> { static constexpr int NV = 2; };
template <> struct ZsRaw<__hip_bfloat16> { static constexpr int NV = 2; };
template <> struct ZsRaw<float> { static constexpr int NV = 4; };

typedef uint32_t qu32x4 __attribute__((ext_vector_type(4)));

// the 16 values of v[] as 8 fp16 pairs, negated if NEG
template <typename TZ, bool NEG>
__device__ __forceinline__ void zs_to_half2(const qu32x4 *v, half2_t out[8]) {
  if constexpr (sizeof(TZ) == 4) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      // (the element is copied out first: a bit cast applied directly to a vector element
      //  reads element 0 whatever the index)
      const uint32_t wa = v[i >> 1][(2 * i) & 3], wb = v[i >> 1][(2 * i + 1) & 3];
      const float a = __builtin_bit_cast(float, wa);
      const float b = __builtin_bit_cast(float, wb);
      out[i] = NEG ? half2_t{(_Float16)-a, (_Float16)-b} : half2_t{(_Float16)a, (_Float16)b};
    }
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t w = v[i >> 2][i & 3];
      if constexpr (std::is_same<TZ, __half>::value) {
        const half2_t h = __builtin_bit_cast(half2_t, w);
        out[i] = NEG ? -h : h;
      } else {   // bf16 pair -> fp32 -> fp16
        const float a = __builtin_bit_cast(float, w << 16);
        const float b = __builtin_bit_cast(float, w & 0xFFFF0000u);
        out[i] = NEG ? half2_t{(_Float16)-a, (_Float16)-b} : half2_t{(_Float16)a, (_Float16)b};
      }
    }
  }
}

// PV consecutive zero / scale values, loaded as PW words, as fp32
template <typename TZ> struct ParamQuad { static constexpr int PW = sizeof(TZ) == 4 ? 4 : 2; };
template <typename TZ>
__device__ __forceinline__ void quad_to_f32(const uint32_t *w, float out[4]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if constexpr (sizeof(TZ) == 4) out[i] = __builtin_bit_cast(float, w[i]);
    else if constexpr (std::is_same<TZ, __half>::value) out[i] = (float)__builtin_bit_cast(half2_t, w[i >> 1])[i & 1];
    else out[i] = (i & 1) ? __builtin_bit_cast(float, w[i >> 1] & 0xFFFF0000u) : __builtin_bit_cast(float, w[i >> 1] << 16);
  }
}

template <typename TZ, typename TX>
__global__ __launch_bounds__(256, 2) void qmm_bwd_gemm_kernel(const TX *x, int M, const uint8_t *pk,
                                                           int R, int C, const TZ *zero,
                                                           const TZ *scale, TX *out) {
  constexpr bool BF = Act<TX>::BF;
  constexpr int BN = 128;                       // output columns per tile = 64 packed rows
  constexpr int A_HALVES = (GBM / 16) * GGROUP;
  constexpr int B_HALVES = (BN / 16) * GGROUP;
  constexpr int TN = BN / 32;
  constexpr int NV = ZsRaw<TZ>::NV;
  constexpr int PW = ParamQuad<TZ>::PW;
  __shared__ __attribute__((aligned(16))) _Float16 As[2][A_HALVES];
  __shared__ __attribute__((aligned(16))) _Float16 Bs[2][B_HALVES];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, g = lane >> 4, l16 = lane & 15;
  int tx, ty;
  qmm_tile_coords(tx, ty);
  const int j0 = tx * (BN / 2), m0 = ty * GBM;

  // B staging: thread -> packed row j0 + tid/4, 16 channels at (tid%4)*16 of the stage
  // A staging, fp16: thread -> row tid/4, the same 16 channels (whose zero and scale the thread
  //   needs for the weights anyway)
  // A staging, bf16: thread -> rows 4*(tid/16) .. +3, 4 channels at (tid%16)*4: the scale and the
  //   zero point go with the activations here, and this way a thread needs 4 + 4 of them per
  //   stage instead of 16 + 16 (fp32 parameters: 8 registers per ring slot instead of 32)
  const int s_row = tid >> 2, s_k = (tid & 3) * 16;
  const int q_row = (tid >> 4) * 4, q_k = (tid & 15) * 4;
  const bool a_ok = (m0 + s_row) < M;
  const bool b_ok = (j0 + s_row) < R;
  const TX *a_src = x + (int64_t)(m0 + (BF ? q_row : s_row)) * C + (BF ? q_k : s_k);
  const uint8_t *b_src = pk + (int64_t)(j0 + s_row) * C + s_k;
  float tsum[4] = {0.f, 0.f, 0.f, 0.f};     // bf16: this thread's share of t[m0 + q_row + i]

  // Activations and weights come from HBM and travel in a ring of four stages; zero and scale
  // of a stage's channels are cache hits (a few tens of KB, read by every workgroup) and need
  // only two stages of lead, which keeps fp32 parameters affordable.
  struct Stage { qu32x4 a0, a1, b; };          // bf16: a0 = rows 0, 1 (2 words each), a1 = rows 2, 3
  struct Params16 { qu32x4 z[NV], s[NV]; };
  struct Params4 { uint32_t z[PW], s[PW]; };
  typedef typename std::conditional<BF, Params4, Params16>::type Params;
  typedef uint32_t qu32x2 __attribute__((ext_vector_type(2)));
  // unconditional, clamped loads (see the forward kernel); C % 16 == 0 is guaranteed
  auto load_stage = [&](int k0, Stage &st) __attribute__((always_inline)) {
    const bool in = (k0 + s_k + 16 <= C);
    if constexpr (BF) {
      const bool ina = (k0 + q_k + 4 <= C);
      qu32x2 r[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        r[i] = *reinterpret_cast<const qu32x2 *>((m0 + q_row + i < M) && ina ? a_src + (int64_t)i * C + k0 : x);
      st.a0 = qu32x4{r[0][0], r[0][1], r[1][0], r[1][1]};
      st.a1 = qu32x4{r[2][0], r[2][1], r[3][0], r[3][1]};
    } else {
      st.a0 = *reinterpret_cast<const qu32x4 *>(a_ok && in ? a_src + k0 : x);
      st.a1 = *reinterpret_cast<const qu32x4 *>(a_ok && in ? a_src + k0 + 8 : x);
    }
    st.b = *reinterpret_cast<const qu32x4 *>(b_ok && in ? b_src + k0 : pk);
  };
  auto load_params = [&](int k0, Params &zs) __attribute__((always_inline)) {
    if constexpr (BF) {
      const int n = (k0 + q_k + 4 <= C) ? k0 + q_k : 0;
      typedef uint32_t vec __attribute__((ext_vector_type(PW)));
      const vec vz = *reinterpret_cast<const vec *>(zero + n), vs = *reinterpret_cast<const vec *>(scale + n);
#pragma unroll
      for (int v = 0; v < PW; ++v) {
        zs.z[v] = vz[v];
        zs.s[v] = vs[v];
      }
    } else {
      const int n = (k0 + s_k + 16 <= C) ? k0 + s_k : 0;
#pragma unroll
      for (int v = 0; v < NV; ++v) {
        zs.z[v] = reinterpret_cast<const qu32x4 *>(zero + n)[v];
        zs.s[v] = reinterpret_cast<const qu32x4 *>(scale + n)[v];
      }
    }
  };
  auto store_stage = [&](int buf, int k0, const Stage &st, const Params &zs) __attribute__((always_inline)) {
    const qu32x4 zero4 = {0u, 0u, 0u, 0u};
    const bool in = (k0 + s_k + 16 <= C);
    if constexpr (BF) {
      typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));
      float sc[4], zz[4];
      quad_to_f32<TZ>(zs.s, sc);
      quad_to_f32<TZ>(zs.z, zz);
      const bool ina = (k0 + q_k + 4 <= C);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bool ok = (m0 + q_row + i < M) && ina;
        const qu32x4 src = i < 2 ? st.a0 : st.a1;
        const uint32_t w0 = ok ? src[2 * (i & 1)] : 0u, w1 = ok ? src[2 * (i & 1) + 1] : 0u;
        const bf2_t p0 = bf2_t{(__bf16)(Act<TX>::lo(w0) * sc[0]), (__bf16)(Act<TX>::hi(w0) * sc[1])};
        const bf2_t p1 = bf2_t{(__bf16)(Act<TX>::lo(w1) * sc[2]), (__bf16)(Act<TX>::hi(w1) * sc[3])};
        const uint32_t u0 = __builtin_bit_cast(uint32_t, p0), u1 = __builtin_bit_cast(uint32_t, p1);
        tsum[i] += (Act<TX>::lo(u0) * (128.f + zz[0]) + Act<TX>::hi(u0) * (128.f + zz[1])) +
                   (Act<TX>::lo(u1) * (128.f + zz[2]) + Act<TX>::hi(u1) * (128.f + zz[3]));
        *reinterpret_cast<qu32x2 *>(&As[buf][g_off(q_row + i, q_k)]) = qu32x2{u0, u1};
      }
      // rows past R produce columns that are never stored, channels past C meet A = 0: any
      // finite weight value will do there
      qu32x4 lo[2], hi[2];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const uint32_t w = st.b[q];
        const uint32_t l = w & 0x0F0F0F0Fu, h = (w >> 4) & 0x0F0F0F0Fu;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          const uint32_t sel = e ? 0x04030402u : 0x04010400u;      // bytes (2e, 2e+1) -> 0x43xx pairs
          const int i = 2 * q + e;
          lo[i >> 2][i & 3] = __builtin_amdgcn_perm(0x43434343u, l, sel);
          hi[i >> 2][i & 3] = __builtin_amdgcn_perm(0x43434343u, h, sel);
        }
      }
      *reinterpret_cast<qu32x4 *>(&Bs[buf][g_off(2 * s_row, s_k)]) = lo[0];
      *reinterpret_cast<qu32x4 *>(&Bs[buf][g_off(2 * s_row, s_k + 8)]) = lo[1];
      *reinterpret_cast<qu32x4 *>(&Bs[buf][g_off(2 * s_row + 1, s_k)]) = hi[0];
      *reinterpret_cast<qu32x4 *>(&Bs[buf][g_off(2 * s_row + 1, s_k + 8)]) = hi[1];
    } else {
      *reinterpret_cast<qu32x4 *>(&As[buf][g_off(s_row, s_k)]) = (a_ok && in) ? st.a0 : zero4;
      *reinterpret_cast<qu32x4 *>(&As[buf][g_off(s_row, s_k + 8)]) = (a_ok && in) ? st.a1 : zero4;
      half2_t sc[8], nzs[8];
      zs_to_half2<TZ, false>(zs.s, sc);
      zs_to_half2<TZ, true>(zs.z, nzs);
#pragma unroll
      for (int i = 0; i < 8; ++i) nzs[i] = nzs[i] * sc[i];        // -zero * scale
      const bool okb = b_ok && in;
      const half2_t k1024 = half2_t{(_Float16)1024.f, (_Float16)1024.f};
      qu32x4 lo[2], hi[2];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const uint32_t w = okb ? st.b[q] : 0u;
        const uint32_t l = w & 0x0F0F0F0Fu, h = (w >> 4) & 0x0F0F0F0Fu;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          const uint32_t sel = e ? 0x04030402u : 0x04010400u;      // bytes (2e, 2e+1) -> 0x64xx pairs
          const half2_t cl = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, l, sel)) - k1024;
          const half2_t ch = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0x64646464u, h, sel)) - k1024;
          const int i = 2 * q + e;                                   // pair index: n = s_k + 2i, 2i+1
          const half2_t dl = okb ? cl * sc[i] + nzs[i] : half2_t{(_Float16)0.f, (_Float16)0.f};
          const half2_t dh = okb ? ch * sc[i] + nzs[i] : half2_t{(_Float16)0.f, (_Float16)0.f};
          lo[i >> 2][i & 3] = __builtin_bit_cast(uint32_t, dl);
          hi[i >> 2][i & 3] = __builtin_bit_cast(uint32_t, dh);
        }
      }
      *reinterpret_cast<qu32x4 *>(&Bs[buf][g_off(2 * s_row, s_k)]) = lo[0];
      *reinterpret_cast<qu32x4 *>(&Bs[buf][g_off(2 * s_row, s_k + 8)]) = lo[1];
      *reinterpret_cast<qu32x4 *>(&Bs[buf][g_off(2 * s_row + 1, s_k)]) = hi[0];
      *reinterpret_cast<qu32x4 *>(&Bs[buf][g_off(2 * s_row + 1, s_k + 8)]) = hi[1];
    }
  };

  floatx4 acc[2][TN];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

  Stage s0, s1, s2, s3;
  Params q0, q1;
  load_params(0, q0);
  load_params(GBK, q1);
  load_stage(0, s0);
  load_stage(GBK, s1);
  load_stage(2 * GBK, s2);
  load_stage(3 * GBK, s3);
  int buf = 0;
  store_stage(0, 0, s0, q0);
  load_params(2 * GBK, q0);
  __syncthreads();
  // multiplies the stage at k0 out of LDS, writes the next one (whose parameters are in zs) and
  // reloads zs for the stage that is written two steps from now
  auto step = [&](int k0, Stage &refill, const Stage &next, Params &zs, bool do_load, bool has_next)
                  __attribute__((always_inline)) {
    if (do_load) load_stage(k0 + 4 * GBK, refill);
#pragma unroll
    for (int ks = 0; ks < GBK; ks += 32) {
      uint4 a[2], b[TN];
#pragma unroll
      for (int i = 0; i < 2; ++i)
        a[i] = *reinterpret_cast<const uint4 *>(&As[buf][g_off(wm * 32 + i * 16 + l16, ks + 8 * g)]);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        b[j] = *reinterpret_cast<const uint4 *>(
            &Bs[buf][g_off(wn * (BN / 2) + j * 16 + l16, ks + 8 * g)]);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = Act<TX>::mma(a[i], b[j], acc[i][j]);
    }
    if (has_next) store_stage(buf ^ 1, k0 + GBK, next, zs);
    if (do_load) load_params(k0 + 3 * GBK, zs);
    __syncthreads();
    buf ^= 1;
  };
  // (the exit-free form of the forward kernel was measured 4 % slower here)
  auto stepx = [&](int k0, Stage &refill, const Stage &next, Params &zs) __attribute__((always_inline)) {
    if (k0 >= C) return;
    step(k0, refill, next, zs, true, k0 + GBK < C);
  };
  for (int kb = 0; kb < C; kb += 4 * GBK) {
    stepx(kb, s0, s1, q1);
    stepx(kb + GBK, s1, s2, q0);
    stepx(kb + 2 * GBK, s2, s3, q1);
    stepx(kb + 3 * GBK, s3, s0, q0);
  }

  __shared__ float trow[GBM];
  if constexpr (BF) {     // t[m]: the sixteen staging threads of a row are neighbouring lanes
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float v = tsum[i];
#pragma unroll
      for (int off = 1; off < 16; off <<= 1) v += __shfl_xor(v, off);
      if ((tid & 15) == 0) trow[q_row + i] = v;
    }
    __syncthreads();
  }
  // acc[i][j][r] = out[m0 + wm*32 + i*16 + 4g + r][2*j0 + wn*64 + j*16 + l16]
  const int KO = 2 * R;
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int c = 2 * j0 + wn * (BN / 2) + j * 16 + l16;
    if (c >= KO) continue;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int ml = wm * 32 + i * 16 + 4 * g + r;
        const float v = BF ? acc[i][j][r] - trow[ml] : acc[i][j][r];
        if (m0 + ml < M) out[(int64_t)(m0 + ml) * KO + c] = Act<TX>::out(v);
      }
  }
}

template <typename TZ>
int launch_bwd_gemm(hipStream_t st, const void *x, int x_dtype, int64_t M, const uint8_t *pk, int64_t R,
                    int64_t C, const void *zero, const void *scale, void *out) {
  const int64_t mt = ceil_div64(M, GBM);
  if (mt > 65535) return GPTQ_HIP_EINVAL;
  const dim3 grid((unsigned)ceil_div64(R, 64), (unsigned)mt);
  if (x_dtype == GPTQ_HIP_BF16)
    hipLaunchKernelGGL((qmm_bwd_gemm_kernel<TZ, __hip_bfloat16>), grid, dim3(256), 0, st,
                       (const __hip_bfloat16 *)x, (int)M, pk, (int)R, (int)C, (const TZ *)zero,
                       (const TZ *)scale, (__hip_bfloat16 *)out);
  else
    hipLaunchKernelGGL((qmm_bwd_gemm_kernel<TZ, __half>), grid, dim3(256), 0, st, (const __half *)x,
                       (int)M, pk, (int)R, (int)C, (const TZ *)zero, (const TZ *)scale, (__half *)out);
  GPTQ_CHECK_LAUNCH();
  return GPTQ_HIP_OK;
}

bool bwd_fast_ok(int x_dtype, int64_t M, int64_t R, int64_t C, const void *x, const uint8_t *pk,
                 const void *zero, const void *scale) {
  return (x_dtype == GPTQ_HIP_F16 || x_dtype == GPTQ_HIP_BF16) && C % 16 == 0 && M >= 1 &&
         R < (1LL << 30) && C < (1LL << 30) &&
         ((reinterpret_cast<uintptr_t>(pk) | reinterpret_cast<uintptr_t>(x) |
           reinterpret_cast<uintptr_t>(zero) | reinterpret_cast<uintptr_t>(scale)) & 15) == 0;
}

bool fwd_fast_ok(int x_dtype, int64_t M, int64_t R, int64_t C, const void *x, const uint8_t *pk) {
  return (x_dtype == GPTQ_HIP_F16 || x_dtype == GPTQ_HIP_BF16) && C % 16 == 0 && M >= 1 && M <= 65535 * 16LL &&
         (reinterpret_cast<uintptr_t>(pk) & 15) == 0 && (reinterpret_cast<uintptr_t>(x) & 3) == 0 &&
         R < (1LL << 30) && C < (1LL << 30);
}

template <typename TX, typename TZ, int BITS>
int launch_simple(hipStream_t st, const void *x, int64_t M, const uint8_t *pk, int64_t R, int64_t C,
                  const void *zero, const void *scale, int transpose_b, void *out, int64_t group) {
  const int64_t kin = transpose_b ? C : (BITS == 4 ? 2 * R : R), nout = transpose_b ? (BITS == 4 ? 2 * R : R) : C;
  // the rows are the grid's y dimension: 65535 of them per launch
  for (int64_t r0 = 0; r0 < M; r0 += 65535) {
    const int64_t rows = M - r0 < 65535 ? M - r0 : 65535;
    const TX *xs = (const TX *)x + r0 * kin;
    TX *os = (TX *)out + r0 * nout;
    if (!transpose_b) {
      hipLaunchKernelGGL((qmm_fwd_simple<TX, TZ, BITS>), dim3((unsigned)ceil_div64(C, TPB), (unsigned)rows),
                         dim3(TPB), 0, st, xs, rows, pk, R, C, (const TZ *)zero, (const TZ *)scale, os, group);
    } else {
      hipLaunchKernelGGL((qmm_bwd_simple<TX, TZ, BITS>),
                         dim3((unsigned)ceil_div64(R, TPB / 64), (unsigned)rows), dim3(TPB), 0, st, xs, rows, pk,
                         R, C, (const TZ *)zero, (const TZ *)scale, os, group);
    }
    GPTQ_CHECK_LAUNCH();
  }
  return GPTQ_HIP_OK;
}

template <typename TX, int BITS>
int dispatch_z(hipStream_t st, const void *x, int64_t M, const uint8_t *pk, int64_t R, int64_t C,
               const void *zero, const void *scale, int zs_dtype, int transpose_b, void *out, int64_t group) {
  switch (zs_dtype) {
    case GPTQ_HIP_F32:
      return launch_simple<TX, float, BITS>(st, x, M, pk, R, C, zero, scale, transpose_b, out, group);
    case GPTQ_HIP_F16:
      return launch_simple<TX, __half, BITS>(st, x, M, pk, R, C, zero, scale, transpose_b, out, group);
    case GPTQ_HIP_BF16:
      return launch_simple<TX, __hip_bfloat16, BITS>(st, x, M, pk, R, C, zero, scale, transpose_b, out, group);
    default:
      return GPTQ_HIP_EDTYPE;
  }
}

template <int BITS>
int dispatch_simple(hipStream_t st, const void *x, int x_dtype, int64_t M, const uint8_t *pk, int64_t R, int64_t C,
                    const void *zero, const void *scale, int zs_dtype, int transpose_b, void *out, int64_t group) {
  switch (x_dtype) {
    case GPTQ_HIP_F32: return dispatch_z<float, BITS>(st, x, M, pk, R, C, zero, scale, zs_dtype, transpose_b, out, group);
    case GPTQ_HIP_F16: return dispatch_z<__half, BITS>(st, x, M, pk, R, C, zero, scale, zs_dtype, transpose_b, out, group);
    case GPTQ_HIP_BF16:
      return dispatch_z<__hip_bfloat16, BITS>(st, x, M, pk, R, C, zero, scale, zs_dtype, transpose_b, out, group);
    default: return GPTQ_HIP_EDTYPE;
  }
}

// ---------------------------------------------------------------------------- fp32 activations
// The 16-bit MFMA kernels serve fp32 activations through two small passes around them: every row
// of x is scaled by the power of two that brings its largest finite magnitude into [2, 4) and
// rounded to fp16, the product runs on the fp16 kernels, and the fp16 result is widened and scaled
// back (powers of two: exact), so rows of any fp32 magnitude keep fp16's relative precision in
// operand and result.  The reference's dot rounds fp32 operands to TF32 (tl.dot at kernel.py:106
// with Triton's default), which has fp16's mantissa width, and its result is rounded to fp16 as
// well (op.py:43).  Rows are processed in chunks so that the staging buffers stay bounded for any M.
constexpr int64_t F32_CHUNK_ROWS = 8192;

__global__ __launch_bounds__(256) void x32_to_f16_rows_kernel(const float *x, int64_t kin, __half *x16,
                                                              int32_t *rowexp) {
  const int64_t m = blockIdx.x;
  const float *xr = x + m * kin;
  __half *dst = x16 + m * kin;
  __shared__ float smax[4];
  constexpr int VR = 16;                       // 16-byte loads per thread that the one-pass form keeps in registers
  // rows of up to 16384 elements, 16-byte aligned: read once, all loads in flight together
  const bool one_pass = (kin & 3) == 0 && kin <= 256 * 4 * VR && (reinterpret_cast<uintptr_t>(x) & 15) == 0;
  float4 v[VR];
  float amax = 0.f;
  auto see = [&](float f) __attribute__((always_inline)) {
    const float a = fabsf(f);
    amax = (a <= 3.4028235e38f && a > amax) ? a : amax;   // NaN and infinity do not set the scale
  };
  if (one_pass) {
    const int64_t last = kin - 4;
#pragma unroll
    for (int i = 0; i < VR; ++i) {
      const int64_t k = (int64_t)(i * 256 + threadIdx.x) * 4;
      v[i] = *reinterpret_cast<const float4 *>(xr + (k < kin ? k : last));
    }
#pragma unroll
    for (int i = 0; i < VR; ++i) {
      see(v[i].x);
      see(v[i].y);
      see(v[i].z);
      see(v[i].w);
    }
  } else {
    for (int64_t k = threadIdx.x; k < kin; k += 256) see(xr[k]);
  }
  for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
  if ((threadIdx.x & 63) == 0) smax[threadIdx.x >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(smax[0], smax[1]), fmaxf(smax[2], smax[3]));
  int ex = 0;
  (void)frexpf(amax, &ex);                    // 2^(ex-1) <= amax < 2^ex
  const int e = amax > 0.f ? ex - 2 : 0;      // largest magnitude of the scaled row in [2, 4)
  if (one_pass) {
#pragma unroll
    for (int i = 0; i < VR; ++i) {
      const int64_t k = (int64_t)(i * 256 + threadIdx.x) * 4;
      if (k < kin) {
        const __half h[4] = {__float2half_rn(ldexpf(v[i].x, -e)), __float2half_rn(ldexpf(v[i].y, -e)),
                             __float2half_rn(ldexpf(v[i].z, -e)), __float2half_rn(ldexpf(v[i].w, -e))};
        *reinterpret_cast<uint2 *>(dst + k) = *reinterpret_cast<const uint2 *>(h);
      }
    }
  } else {
    for (int64_t k = threadIdx.x; k < kin; k += 256) dst[k] = __float2half_rn(ldexpf(xr[k], -e));
  }
  if (threadIdx.x == 0) rowexp[m] = e;
}

// only the exponent of a row's scale (for the decode kernel that converts in place)
__global__ __launch_bounds__(256) void x32_rowexp_kernel(const float *x, int64_t kin, int32_t *rowexp) {
  const float *xr = x + (int64_t)blockIdx.x * kin;
  __shared__ float smax[4];
  float amax = 0.f;
  auto see = [&](float f) __attribute__((always_inline)) {
    const float a = fabsf(f);
    amax = (a <= 3.4028235e38f && a > amax) ? a : amax;   // NaN and infinity do not set the scale
  };
  if ((kin & 3) == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0) {
    // 16-byte loads, four of a thread in flight together
    for (int64_t k0 = (int64_t)threadIdx.x * 4; k0 < kin; k0 += 4 * 1024) {
      float4 v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int64_t k = k0 + i * 1024;
        v[i] = *reinterpret_cast<const float4 *>(xr + (k < kin ? k : kin - 4));
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        see(v[i].x);
        see(v[i].y);
        see(v[i].z);
        see(v[i].w);
      }
    }
  } else {
    for (int64_t k = threadIdx.x; k < kin; k += 256) see(xr[k]);
  }
  for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
  if ((threadIdx.x & 63) == 0) smax[threadIdx.x >> 6] = amax;
  __syncthreads();
  if (threadIdx.x == 0) {
    amax = fmaxf(fmaxf(smax[0], smax[1]), fmaxf(smax[2], smax[3]));
    int ex = 0;
    (void)frexpf(amax, &ex);
    rowexp[blockIdx.x] = amax > 0.f ? ex - 2 : 0;
  }
}

__global__ __launch_bounds__(256) void f16_rows_to_f32_kernel(const __half *o16, int64_t nout,
                                                              const int32_t *rowexp, float *out) {
  const int64_t m = blockIdx.y;
  const int e = rowexp[m];
  for (int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x; n < nout; n += (int64_t)gridDim.x * 256)
    out[m * nout + n] = ldexpf(__half2float(o16[m * nout + n]), e);
}

struct F32Plan {
  bool use;
  int64_t mc;                 // rows per chunk
  size_t inner;               // workspace of the fp16 product of one chunk (at offset 0: its counters)
  size_t x16_off, o16_off, exp_off, total_bytes;
};

size_t round_up_256(size_t v) { return (v + 255) & ~(size_t)255; }

}  // namespace

namespace {

// workspace of a product whose activations are fp16 or bf16
size_t ws16_bytes(int64_t M, int64_t R, int64_t C, int transpose_b, int bits) {
  if (M <= 0 || R <= 0 || C <= 0) return 0;
  if (transpose_b) {
    const RegBwdPlan bp = reg_bwd_plan(M, R, C, bits, true), bp8 = reg_bwd_plan(M, R, C, bits, true, 8);
    const size_t a = bp.use ? bp.total_bytes : 0, b = bp8.use ? bp8.total_bytes : 0;
    return a > b ? a : b;
  }
  const RegPlan rp = reg_fwd_plan(M, R, C, bits, true);
  size_t need = rp.use ? rp.total_bytes : 0;
  if (bits != 4) {
    const DecPlan d8 = dec_plan(M, R, C, 8);
    if (d8.use && d8.total_bytes > need) need = d8.total_bytes;
    return need;
  }
  // which kernel runs also depends on pointer alignment: enough for any of them
  const size_t chunked = fwd_plan(M, R, C).total_bytes;
  need = chunked > need ? chunked : need;
  const DecPlan dp = dec_plan(M, R, C);
  if (dp.use && dp.total_bytes > need) need = dp.total_bytes;
  const MidPlan mp = mid_fwd_plan(M, R, C, true);
  if (mp.use && mp.total_bytes > need) need = mp.total_bytes;
  const DecPlan dr = dec_plan(M, R, C, 4, true);
  if (dr.use && dr.total_bytes > need) need = dr.total_bytes;
  return need;
}

// whether a matrix-core kernel serves this shape for 16-bit activations
bool has_fast16(int64_t M, int64_t R, int64_t C, int transpose_b, int bits) {
  if (M < 1 || R >= (1LL << 30) || C >= (1LL << 30)) return false;
  if (bits == 4 && C % 16 == 0) return true;
  return transpose_b ? reg_bwd_plan(M, R, C, bits, true).use : reg_fwd_plan(M, R, C, bits, true).use;
}

F32Plan f32_plan(int64_t M, int64_t R, int64_t C, int transpose_b, int bits) {
  F32Plan p{};
  p.use = has_fast16(M, R, C, transpose_b, bits);
  if (!p.use) return p;
  p.mc = M < F32_CHUNK_ROWS ? M : F32_CHUNK_ROWS;
  const int64_t tail = M % p.mc;
  size_t inner = ws16_bytes(p.mc, R, C, transpose_b, bits);
  if (tail) {
    const size_t t = ws16_bytes(tail, R, C, transpose_b, bits);
    inner = t > inner ? t : inner;
  }
  const int64_t Kl = bits == 4 ? 2 * R : R;
  const int64_t kin = transpose_b ? C : Kl, nout = transpose_b ? Kl : C;
  p.inner = inner;
  // the counter region stays out of reach of the staging buffers whatever this call's own product
  // needs: a later call on the same workspace expects its counters to be zero
  p.x16_off = round_up_256(inner > (size_t)QMM_HEAD_BYTES ? inner : (size_t)QMM_HEAD_BYTES);
  p.o16_off = p.x16_off + round_up_256((size_t)p.mc * kin * sizeof(__half));
  p.exp_off = p.o16_off + round_up_256((size_t)p.mc * nout * sizeof(__half));
  p.total_bytes = p.exp_off + round_up_256((size_t)p.mc * sizeof(int32_t));
  return p;
}

bool aligned16(const void *a, const void *b) {
  return ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15) == 0;
}

// group_size = 0: zero / scale [C]; group_size > 0: zero / scale [K / group_size, C] (register-operand kernels,
// whose k-steps of 32 and tiles of 128 output columns must not straddle a group, or the plain kernels)
// out32 / rowexp / wrote32 (the recursive call for fp32 rows): where the product runs on register-operand tiles of
// more than 16 rows it stores the fp32 result itself (RegPlan::out32) and sets *wrote32
int qmatmul_impl(void *stream, const void *x, int x_dtype, int64_t M, const uint8_t *packed, int64_t R, int64_t C,
                 const void *zero, const void *scale, int zs_dtype, int bits, int64_t group_size, int transpose_b,
                 void *out, void *ws, size_t ws_bytes, float *out32 = nullptr, const int32_t *rowexp = nullptr,
                 bool *wrote32 = nullptr, gptq_hip_qmatmul_plan *plan = nullptr) {
  // plan != nullptr: nothing is launched; the pointers are only looked at for their alignment, and *plan says
  // which kernel the same call would run (`planned` in front of every launch).
  auto planned = [&](int kernel, int rest, int64_t splits, int64_t workgroups) -> bool {
    if (!plan) return false;
    plan->kernel = kernel;
    plan->kernel_rest = rest;
    plan->splits = (int)splits;
    plan->workgroups = workgroups;
    return true;
  };
  if (M < 0 || R <= 0 || C <= 0 || (bits != 4 && bits != 8)) return GPTQ_HIP_EINVAL;
  if (group_size < 0 || group_size % 2 != 0 || (group_size > 0 && (bits == 4 ? 2 * R : R) % group_size != 0) ||
      group_size > (1LL << 30))
    return GPTQ_HIP_EINVAL;
  const bool reg_groups_ok = group_size == 0 || group_size % (transpose_b ? 128 : 32) == 0;
  if (M == 0) return GPTQ_HIP_OK;
  if (!x || !packed || !zero || !scale || !out) return GPTQ_HIP_EINVAL;
  hipStream_t st = as_stream(stream);
  if (x_dtype == GPTQ_HIP_F32) {
    // through the 16-bit kernels, if the shape suits them and the caller sized the workspace for
    // it (gptq_hip_qmatmul_workspace_bytes_x); else the plain fp32 kernels below
    const F32Plan fp = f32_plan(M, R, C, transpose_b, bits);
    if (fp.use && reg_groups_ok && ws && ws_bytes >= fp.total_bytes && (reinterpret_cast<uintptr_t>(ws) & 15) == 0) {
      char *base = reinterpret_cast<char *>(ws);
      __half *x16 = reinterpret_cast<__half *>(base + fp.x16_off);
      __half *o16 = reinterpret_cast<__half *>(base + fp.o16_off);
      int32_t *rowexp = reinterpret_cast<int32_t *>(base + fp.exp_off);
      const int64_t Kl = bits == 4 ? 2 * R : R;
      const int64_t kin = transpose_b ? C : Kl, nout = transpose_b ? Kl : C;
      // up to 16 rows on the decode kernel's shapes: converted inside that kernel (no staging, one launch)
      if (bits == 4 && !transpose_b && group_size == 0 && M <= 16 && R % 4 == 0 && C % 16 == 0 &&
          ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(packed)) & 15) == 0 &&
          (reinterpret_cast<uintptr_t>(out) & 3) == 0) {
        const DecPlan dp = dec_plan(M, R, C);
        if (dp.use && dp.atom && (dp.total_bytes == 0 || (ws && ws_bytes >= dp.total_bytes))) {
          if (planned(GPTQ_HIP_QMM_DECODE, 0, dp.S, (int64_t)dp.strips * dp.S)) {
            plan->fp32_rows = 2;
            return GPTQ_HIP_OK;
          }
          const int32_t *re = nullptr;
          if (M > 2) {            // beyond two rows every workgroup's own pass over the rows costs more than a launch
            hipLaunchKernelGGL(x32_rowexp_kernel, dim3((unsigned)M), dim3(256), 0, st,
                               reinterpret_cast<const float *>(x), kin, rowexp);
            GPTQ_CHECK_LAUNCH();
            re = rowexp;
          }
          switch (zs_dtype) {
            case GPTQ_HIP_F32: return launch_dec_x32<float>(st, dp, x, M, packed, R, C, zero, scale, out, ws, re);
            case GPTQ_HIP_F16: return launch_dec_x32<__half>(st, dp, x, M, packed, R, C, zero, scale, out, ws, re);
            case GPTQ_HIP_BF16:
              return launch_dec_x32<__hip_bfloat16>(st, dp, x, M, packed, R, C, zero, scale, out, ws, re);
            default: return GPTQ_HIP_EDTYPE;
          }
        }
      }
      if (plan) {
        // the kernel of the (first) chunk of rows, on the aligned staging buffers
        const int64_t mm = M < fp.mc ? M : fp.mc;
        const int rc = qmatmul_impl(stream, x16, GPTQ_HIP_F16, mm, packed, R, C, zero, scale, zs_dtype, bits, group_size,
                                    transpose_b, o16, ws, fp.inner, nullptr, nullptr, nullptr, plan);
        plan->fp32_rows = 1;
        return rc;
      }
      for (int64_t r0 = 0; r0 < M; r0 += fp.mc) {
        const int64_t mm = M - r0 < fp.mc ? M - r0 : fp.mc;
        hipLaunchKernelGGL(x32_to_f16_rows_kernel, dim3((unsigned)mm), dim3(256), 0, st,
                           reinterpret_cast<const float *>(x) + r0 * kin, kin, x16, rowexp);
        GPTQ_CHECK_LAUNCH();
        bool wrote = false;
        const int rc = qmatmul_impl(stream, x16, GPTQ_HIP_F16, mm, packed, R, C, zero, scale, zs_dtype, bits,
                                    group_size, transpose_b, o16, ws, fp.inner,
                                    (reinterpret_cast<uintptr_t>(out) & 15) != 0
                                        ? nullptr
                                        : reinterpret_cast<float *>(out) + r0 * nout,
                                    rowexp, &wrote);
        if (rc) return rc;
        if (wrote) continue;                  // the product's tiles stored the fp32 rows themselves
        unsigned gx = (unsigned)ceil_div64(nout, 1024);
        if (gx > 64) gx = 64;
        hipLaunchKernelGGL(f16_rows_to_f32_kernel, dim3(gx, (unsigned)mm), dim3(256), 0, st, o16, nout,
                           rowexp, reinterpret_cast<float *>(out) + r0 * nout);
        GPTQ_CHECK_LAUNCH();
      }
      return GPTQ_HIP_OK;
    }
    if (planned(transpose_b ? GPTQ_HIP_QMM_BWD_SIMPLE : GPTQ_HIP_QMM_SIMPLE, 0, 1, 0)) return GPTQ_HIP_OK;
    return bits == 4
               ? dispatch_simple<4>(st, x, x_dtype, M, packed, R, C, zero, scale, zs_dtype, transpose_b, out, group_size)
               : dispatch_simple<8>(st, x, x_dtype, M, packed, R, C, zero, scale, zs_dtype, transpose_b, out, group_size);
  }
  if (x_dtype != GPTQ_HIP_F16 && x_dtype != GPTQ_HIP_BF16) return GPTQ_HIP_EDTYPE;
  if (zs_dtype != GPTQ_HIP_F32 && zs_dtype != GPTQ_HIP_F16 && zs_dtype != GPTQ_HIP_BF16) return GPTQ_HIP_EDTYPE;
  const bool al = aligned16(x, out) && (reinterpret_cast<uintptr_t>(packed) & 7) == 0;
  const RegPlan rp = (transpose_b || !reg_groups_ok) ? RegPlan{} : reg_fwd_plan(M, R, C, bits, al);
  auto run_reg_fwd = [&]() -> int {
    if (rp.total_bytes && (!ws || ws_bytes < rp.total_bytes)) return GPTQ_HIP_EWORKSPACE;
    if (plan) {
      const RegParts parts = reg_fwd_parts(rp, M, R, C, x_dtype == GPTQ_HIP_BF16, (int)group_size);
      const int own = rp.rb == 8 ? GPTQ_HIP_QMM_REG128 : (rp.rb == 4 ? GPTQ_HIP_QMM_REG64 : GPTQ_HIP_QMM_REG16);
      const int64_t ty = ceil_div64(M, 16 * rp.rb);
      if (parts.wide_x > 0)
        planned(parts.half ? GPTQ_HIP_QMM_WIDE_HALF : GPTQ_HIP_QMM_WIDE,
                parts.wide2_x > 0 ? GPTQ_HIP_QMM_WIDE_HALF
                                  : (parts.main_x > 0 ? GPTQ_HIP_QMM_REG128 : (parts.tail > 0 ? GPTQ_HIP_QMM_REG64 : 0)), 1,
                parts.wide_x * ceil_div64(M, 128));
      else
        planned(parts.main_x > 0 ? own : GPTQ_HIP_QMM_REG64, (parts.main_x > 0 && parts.tail > 0) ? GPTQ_HIP_QMM_REG64 : 0,
                rp.S, (parts.main_x > 0 ? parts.main_x : parts.tail) * ty * rp.S);
      return GPTQ_HIP_OK;
    }
    RegPlan q = rp;
    if (out32 && rowexp && wrote32 && rp.rb > 1 && x_dtype == GPTQ_HIP_F16) {
      q.out32 = out32;
      q.rowexp = rowexp;
      *wrote32 = true;
    }
    return reg_fwd_launch(st, q, x, x_dtype, M, packed, R, C, zero, scale, zs_dtype, out, ws, (int)group_size);
  };
  if (bits == 8 && !transpose_b && group_size == 0 && x_dtype == GPTQ_HIP_F16 && M <= 16 &&
      fwd_fast_ok(x_dtype, M, R, C, x, packed) && (reinterpret_cast<uintptr_t>(x) & 15) == 0) {
    // up to 16 fp16 rows against 8-bit codes: the decode kernel
    const DecPlan dp = dec_plan(M, R, C, 8);
    if (dp.use) {
      if (dp.total_bytes && (!ws || ws_bytes < dp.total_bytes)) return GPTQ_HIP_EWORKSPACE;
      if (planned(GPTQ_HIP_QMM_DECODE, 0, dp.S, (int64_t)dp.strips * dp.S)) return GPTQ_HIP_OK;
      switch (zs_dtype) {
        case GPTQ_HIP_F32: return launch_dec_z8<float>(st, dp, x, M, packed, R, C, zero, scale, out, ws);
        case GPTQ_HIP_F16: return launch_dec_z8<__half>(st, dp, x, M, packed, R, C, zero, scale, out, ws);
        default: return launch_dec_z8<__hip_bfloat16>(st, dp, x, M, packed, R, C, zero, scale, out, ws);
      }
    }
  }
  if (bits == 4 && !transpose_b && group_size == 0 && M <= 16 && C % 16 != 0 && R % 4 == 0 &&
      (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 1) == 0) {
    // up to 16 rows against rows that are no multiple of 16 channels (a vocabulary-sized C): the decode kernel's
    // form for rows of any length and alignment
    const DecPlan dp = dec_plan(M, R, C, 4, true);
    if (dp.use) {
      if (dp.total_bytes && (!ws || ws_bytes < dp.total_bytes)) return GPTQ_HIP_EWORKSPACE;
      if (planned(GPTQ_HIP_QMM_DECODE_RAGGED, 0, dp.S, (int64_t)dp.strips * dp.S)) return GPTQ_HIP_OK;
      switch (zs_dtype) {
        case GPTQ_HIP_F32: return launch_dec_z_rag<float>(st, dp, x, x_dtype, M, packed, R, C, zero, scale, out, ws);
        case GPTQ_HIP_F16: return launch_dec_z_rag<__half>(st, dp, x, x_dtype, M, packed, R, C, zero, scale, out, ws);
        default:
          return launch_dec_z_rag<__hip_bfloat16>(st, dp, x, x_dtype, M, packed, R, C, zero, scale, out, ws);
      }
    }
  }
  if (bits == 4 && !transpose_b && group_size == 0) {
    // 17 .. 256 rows: tall, narrow tiles whose eight wavefronts split the contraction (qmatmul_mid.hip)
    MidPlan mp = mid_fwd_plan(M, R, C, al && (reinterpret_cast<uintptr_t>(packed) & 15) == 0, x_dtype == GPTQ_HIP_BF16);
    if (mp.use) {
      if (mp.total_bytes && (!ws || ws_bytes < mp.total_bytes)) return GPTQ_HIP_EWORKSPACE;
      if (planned(GPTQ_HIP_QMM_MID, 0, mp.S, mp.tiles_x * mp.tiles_y * mp.S)) return GPTQ_HIP_OK;
      if (out32 && rowexp && wrote32 && x_dtype == GPTQ_HIP_F16) {
        mp.out32 = out32;
        mp.rowexp = rowexp;
        *wrote32 = true;
      }
      return mid_fwd_launch(st, mp, x, M, packed, R, C, zero, scale, zs_dtype, out, ws);
    }
  }
  if (bits == 4 && !transpose_b && group_size == 0) {
    // more than 16 rows: the register-operand kernel, unless its tiles are too few to fill a quarter of the chip
    // even when split (small matrices: the chunked kernel below, 16 rows at a time)
    if (rp.use && !rp.ragged && M > 16 && rp.tiles * rp.S >= 64) return run_reg_fwd();
    if (fwd_fast_ok(x_dtype, M, R, C, x, packed) && (reinterpret_cast<uintptr_t>(x) & 15) == 0) {
      const DecPlan dp = dec_plan(M, R, C);
      if (dp.use) {
        if (dp.total_bytes && (!ws || ws_bytes < dp.total_bytes)) return GPTQ_HIP_EWORKSPACE;
        if (planned(GPTQ_HIP_QMM_DECODE, 0, dp.S, (int64_t)dp.strips * dp.S)) return GPTQ_HIP_OK;
        switch (zs_dtype) {
          case GPTQ_HIP_F32: return launch_dec_z<float>(st, dp, x, x_dtype, M, packed, R, C, zero, scale, out, ws);
          case GPTQ_HIP_F16: return launch_dec_z<__half>(st, dp, x, x_dtype, M, packed, R, C, zero, scale, out, ws);
          default:
            return launch_dec_z<__hip_bfloat16>(st, dp, x, x_dtype, M, packed, R, C, zero, scale, out, ws);
        }
      }
    }
    if (fwd_fast_ok(x_dtype, M, R, C, x, packed)) {
      const FwdPlan p = fwd_plan(M, R, C);
      if (p.total_bytes && (!ws || ws_bytes < p.total_bytes)) return GPTQ_HIP_EWORKSPACE;
      if (planned(GPTQ_HIP_QMM_CHUNKED, 0, p.S, (int64_t)p.strips * p.S * p.mch)) return GPTQ_HIP_OK;
      switch (zs_dtype) {
        case GPTQ_HIP_F32:
          return launch_fwd_mfma_z<float>(st, p, x, x_dtype, M, packed, R, C, zero, scale, out, ws);
        case GPTQ_HIP_F16:
          return launch_fwd_mfma_z<__half>(st, p, x, x_dtype, M, packed, R, C, zero, scale, out, ws);
        default:
          return launch_fwd_mfma_z<__hip_bfloat16>(st, p, x, x_dtype, M, packed, R, C, zero, scale, out, ws);
      }
    }
  }
  // Transposed, 4-bit: the tiled kernel has no split over the contraction, so while its 64 x 128 output tiles
  // number no more than the CUs it runs as long as a full chip's worth of tiles would (122 us for any M <= 448
  // on 4096 x 11008); there the register-operand kernel, which splits, takes over (M = 128: 124 -> 38 us,
  // M = 16: 122 -> 23 us; exactly one tile per CU, M = 512: 133 -> 103 us).
  // more than 64 rows: 128-row tiles of the register-operand kernel (a dequantised operand
  // serves twice the rows; 4096 x 11008 at M = 2048: 335 -> 268 us, 8-bit: 512 -> 347 us) unless their last round
  // of 256 workgroups would leave much of the chip idle (11008 x 4096 at M = 512: 344 tiles)
  auto plan_reg_bwd = [&](const RegBwdPlan &bp) {
    const RegParts parts = reg_bwd_parts(bp, M, R, C, x_dtype == GPTQ_HIP_BF16, (int)group_size);
    const int own = bp.rb == 8 ? GPTQ_HIP_QMM_BWD_REG128 : GPTQ_HIP_QMM_BWD_REG64;
    const int64_t ty = ceil_div64(M, 16 * bp.rb);
    if (parts.wide_x > 0)
      planned(parts.half ? GPTQ_HIP_QMM_BWD_WIDE_HALF : GPTQ_HIP_QMM_BWD_WIDE,
              parts.wide2_x > 0 ? GPTQ_HIP_QMM_BWD_WIDE_HALF
                                : (parts.main_x > 0 ? GPTQ_HIP_QMM_BWD_REG128 : (parts.tail > 0 ? GPTQ_HIP_QMM_BWD_REG64 : 0)), 1,
              parts.wide_x * ceil_div64(M, 128));
    else
      planned(parts.main_x > 0 ? own : GPTQ_HIP_QMM_BWD_REG64,
              (parts.main_x > 0 && parts.tail > 0) ? GPTQ_HIP_QMM_BWD_REG64 : 0, bp.S,
              (parts.main_x > 0 ? parts.main_x : parts.tail) * ty * bp.S);
  };
  if (transpose_b && reg_groups_ok && M > 64) {
    RegBwdPlan bp8 = reg_bwd_plan(M, R, C, bits, al, 8);
    bp8.no_wide = (reinterpret_cast<uintptr_t>(packed) & 15) != 0;
    const int64_t rounds = bp8.use ? (bp8.tiles + 255) / 256 : 0;
    if (bp8.use && (bp8.tiles <= 256 || bp8.tail_x > 0 || bp8.tiles * 5 >= rounds * 256 * 4)) {
      if (bp8.total_bytes && (!ws || ws_bytes < bp8.total_bytes)) return GPTQ_HIP_EWORKSPACE;
      if (plan) {
        plan_reg_bwd(bp8);
        return GPTQ_HIP_OK;
      }
      RegBwdPlan q = bp8;
      if (out32 && rowexp && wrote32 && x_dtype == GPTQ_HIP_F16) {
        q.out32 = out32;
        q.rowexp = rowexp;
        *wrote32 = true;
      }
      return reg_bwd_launch(st, q, x, x_dtype, M, packed, R, C, zero, scale, zs_dtype, out, ws, (int)group_size);
    }
  }
  const bool bwd_tiles_fill = ceil_div64(2 * R, 128) * ceil_div64(M, 64) > 256 ||
                              !(reg_groups_ok && reg_bwd_plan(M, R, C, bits, al).use);
  if (bits == 4 && transpose_b && group_size == 0 && bwd_tiles_fill &&
      bwd_fast_ok(x_dtype, M, R, C, x, packed, zero, scale)) {
    if (planned(GPTQ_HIP_QMM_BWD_GEMM, 0, 1, ceil_div64(2 * R, 128) * ceil_div64(M, 64))) return GPTQ_HIP_OK;
    switch (zs_dtype) {
      case GPTQ_HIP_F32: return launch_bwd_gemm<float>(st, x, x_dtype, M, packed, R, C, zero, scale, out);
      case GPTQ_HIP_F16: return launch_bwd_gemm<__half>(st, x, x_dtype, M, packed, R, C, zero, scale, out);
      default: return launch_bwd_gemm<__hip_bfloat16>(st, x, x_dtype, M, packed, R, C, zero, scale, out);
    }
  }
  // 8-bit codes, and 4-bit shapes whose rows are not multiples of 16 channels or that are not aligned
  if (!transpose_b && rp.use) return run_reg_fwd();
  if (transpose_b && reg_groups_ok) {
    const RegBwdPlan bp = reg_bwd_plan(M, R, C, bits, al);
    if (bp.use) {
      if (bp.total_bytes && (!ws || ws_bytes < bp.total_bytes)) return GPTQ_HIP_EWORKSPACE;
      if (plan) {
        plan_reg_bwd(bp);
        return GPTQ_HIP_OK;
      }
      RegBwdPlan q = bp;
      if (out32 && rowexp && wrote32 && x_dtype == GPTQ_HIP_F16) {
        q.out32 = out32;
        q.rowexp = rowexp;
        *wrote32 = true;
      }
      return reg_bwd_launch(st, q, x, x_dtype, M, packed, R, C, zero, scale, zs_dtype, out, ws, (int)group_size);
    }
  }
  if (planned(transpose_b ? GPTQ_HIP_QMM_BWD_SIMPLE : GPTQ_HIP_QMM_SIMPLE, 0, 1, 0)) return GPTQ_HIP_OK;
  return bits == 4
             ? dispatch_simple<4>(st, x, x_dtype, M, packed, R, C, zero, scale, zs_dtype, transpose_b, out, group_size)
             : dispatch_simple<8>(st, x, x_dtype, M, packed, R, C, zero, scale, zs_dtype, transpose_b, out, group_size);
}

}  // namespace

extern "C" {

int gptq_hip_qmatmul_plan_query(int64_t M, int64_t R, int64_t C, int transpose_b, int x_dtype, int zs_dtype, int bits,
                                int64_t group_size, int aligned, gptq_hip_qmatmul_plan *plan) {
  if (!plan || M < 1) return GPTQ_HIP_EINVAL;
  *plan = gptq_hip_qmatmul_plan{};
  // never dereferenced: qmatmul_impl only looks at the alignment of the pointers when it is given a plan
  const uintptr_t base = aligned ? 0x10000u : 0x10002u;
  void *fake = reinterpret_cast<void *>(base);
  void *fake_ws = reinterpret_cast<void *>((uintptr_t)0x20000u);
  return qmatmul_impl(nullptr, fake, x_dtype, M, reinterpret_cast<const uint8_t *>(aligned ? base : base - 1), R, C, fake,
                      fake, zs_dtype, bits, group_size, transpose_b, fake, fake_ws, ~(size_t)0, nullptr, nullptr, nullptr, plan);
}

const char *gptq_hip_qmatmul_kernel_name(int kernel) {
  switch (kernel) {
    case GPTQ_HIP_QMM_SIMPLE: return "qmm_fwd_simple";
    case GPTQ_HIP_QMM_DECODE: return "qmm_fwd_dec_kernel";
    case GPTQ_HIP_QMM_DECODE_RAGGED: return "qmm_fwd_dec_kernel (rows of any length)";
    case GPTQ_HIP_QMM_CHUNKED: return "qmm_fwd_mfma_kernel";
    case GPTQ_HIP_QMM_MID: return "qmm_fwd_mid_kernel";
    case GPTQ_HIP_QMM_REG16: return "qmm_fwd_reg_kernel (16-row tiles)";
    case GPTQ_HIP_QMM_REG64: return "qmm_fwd_reg_kernel (64-row tiles)";
    case GPTQ_HIP_QMM_REG128: return "qmm_fwd_reg_kernel (128-row tiles)";
    case GPTQ_HIP_QMM_WIDE: return "qmm_fwd_wide_kernel (128 x 512)";
    case GPTQ_HIP_QMM_WIDE_HALF: return "qmm_fwd_wide_kernel (128 x 256)";
    case GPTQ_HIP_QMM_BWD_SIMPLE: return "qmm_bwd_simple";
    case GPTQ_HIP_QMM_BWD_REG64: return "qmm_bwd_reg_kernel (64-row tiles)";
    case GPTQ_HIP_QMM_BWD_REG128: return "qmm_bwd_reg_kernel (128-row tiles)";
    case GPTQ_HIP_QMM_BWD_WIDE: return "qmm_bwd_wide_kernel (128 x 512)";
    case GPTQ_HIP_QMM_BWD_WIDE_HALF: return "qmm_bwd_wide_kernel (128 x 256)";
    case GPTQ_HIP_QMM_BWD_GEMM: return "qmm_bwd_gemm_kernel";
    default: return "none";
  }
}

size_t gptq_hip_qmatmul_workspace_bytes(int64_t M, int64_t R, int64_t C, int transpose_b) {
  return ws16_bytes(M, R, C, transpose_b, 4);
}

size_t gptq_hip_qmatmul_workspace_bytes_x(int64_t M, int64_t R, int64_t C, int transpose_b, int x_dtype) {
  return gptq_hip_qmatmul_bits_workspace_bytes(M, R, C, transpose_b, x_dtype, 4);
}

size_t gptq_hip_qmatmul_bits_workspace_bytes(int64_t M, int64_t R, int64_t C, int transpose_b, int x_dtype,
                                             int bits) {
  if (M <= 0 || R <= 0 || C <= 0 || (bits != 4 && bits != 8)) return 0;
  if (x_dtype == GPTQ_HIP_F32) {
    const F32Plan fp = f32_plan(M, R, C, transpose_b, bits);
    if (fp.use) return fp.total_bytes;
  }
  return ws16_bytes(M, R, C, transpose_b, bits);
}

int gptq_hip_qmatmul(void *stream, const void *x, int x_dtype, int64_t M, const uint8_t *packed,
                     int64_t R, int64_t C, const void *zero, const void *scale, int zs_dtype,
                     int transpose_b, void *out, void *ws, size_t ws_bytes) {
  return qmatmul_impl(stream, x, x_dtype, M, packed, R, C, zero, scale, zs_dtype, 4, 0, transpose_b, out, ws,
                      ws_bytes);
}

int gptq_hip_qmatmul_bits(void *stream, const void *x, int x_dtype, int64_t M, const uint8_t *packed,
                          int64_t R, int64_t C, const void *zero, const void *scale, int zs_dtype, int bits,
                          int transpose_b, void *out, void *ws, size_t ws_bytes) {
  return qmatmul_impl(stream, x, x_dtype, M, packed, R, C, zero, scale, zs_dtype, bits, 0, transpose_b, out, ws,
                      ws_bytes);
}

int gptq_hip_qmatmul_grouped(void *stream, const void *x, int x_dtype, int64_t M, const uint8_t *packed,
                             int64_t R, int64_t C, const void *zero, const void *scale, int zs_dtype,
                             int64_t group_size, int bits, int transpose_b, void *out, void *ws, size_t ws_bytes) {
  if (group_size <= 0) return GPTQ_HIP_EINVAL;
  return qmatmul_impl(stream, x, x_dtype, M, packed, R, C, zero, scale, zs_dtype, bits, group_size, transpose_b, out,
                      ws, ws_bytes);
}

}  // extern "C"

// ---------------------------------------------------------------- the call that allocates nothing
// gptq_hip_qmatmul_static is gptq_hip_qmatmul with the workspace (arrival counters, split-K
// partials, fp16 staging of fp32 activations) taken from a fixed array in device memory instead of
// a caller's buffer, for callers that cannot allocate: code under graph capture, serving loops,
// harnesses that forbid hipMalloc.  Every GPU the library runs on holds its own copy of the array
// until the process ends.  In host code the array's name is only a stand-in: the address a kernel
// may use is the one hipGetSymbolAddress returns with that device current, looked up once per
// device below and used for everything the host does with the memory.
constexpr size_t QMM_STATIC_BYTES = GPTQ_HIP_QMATMUL_STATIC_BYTES;
static __device__ __align__(256) unsigned char scratch[QMM_STATIC_BYTES];

namespace {

constexpr int QMM_STATIC_MAX_DEVICES = 64;
std::mutex g_static_mutex;
void *g_static_ptr[QMM_STATIC_MAX_DEVICES] = {};

// Address of the current device's copy of the array (looked up once per device).  Nothing has to be cleared: the
// array is zero when the library is loaded, and every product leaves the arrival counters and the 64-bit cells at
// its head as it found them.
int qmm_static_base(void **base) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= QMM_STATIC_MAX_DEVICES) return GPTQ_HIP_EINVAL;
  std::lock_guard<std::mutex> lock(g_static_mutex);
  if (!g_static_ptr[dev]) {
    void *ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) {
      (void)hipGetLastError();
      return GPTQ_HIP_ELAUNCH;
    }
    g_static_ptr[dev] = ptr;
  }
  *base = g_static_ptr[dev];
  return GPTQ_HIP_OK;
}

}  // namespace

extern "C" {

int gptq_hip_qmatmul_static(void *stream, const void *x, int x_dtype, int64_t M, const uint8_t *packed,
                            int64_t R, int64_t C, const void *zero, const void *scale, int zs_dtype,
                            int transpose_b, void *out) {
  if (M < 0 || R <= 0 || C <= 0) return GPTQ_HIP_EINVAL;
  if (M == 0) return GPTQ_HIP_OK;
  if (gptq_hip_qmatmul_workspace_bytes_x(M, R, C, transpose_b, x_dtype) > QMM_STATIC_BYTES)
    return GPTQ_HIP_ETOOBIG;
  void *base = nullptr;
  const int rc = qmm_static_base(&base);
  if (rc) return rc;
  return gptq_hip_qmatmul(stream, x, x_dtype, M, packed, R, C, zero, scale, zs_dtype, transpose_b, out,
                          base, QMM_STATIC_BYTES);
}

}  // extern "C"
