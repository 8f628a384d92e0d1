// Device helpers shared by the register-operand matmul kernels (forward and transposed).
#pragma once
#include "qmm_common.h"

namespace qmm {

constexpr int RG_NT = 9;                 // accumulator tiles per 16-row block: 8 output tiles + one tile of sums
constexpr int RG_TILE_FLOATS = 256;      // one 16 x 16 fp32 tile: 64 lanes x 4

struct __attribute__((packed)) RgU2 { uint32_t x, y; };
struct __attribute__((packed)) RgU4 { uint32_t x, y, z, w; };

// 8- and 16-byte loads from addresses of any alignment (the hardware takes them; the packed types tell
// the compiler not to assume more)
template <bool UNALIGNED>
__device__ __forceinline__ uint2 rg_load8(const void *p) {
  if (UNALIGNED) {
    RgU2 v;
    __builtin_memcpy(&v, p, 8);
    return make_uint2(v.x, v.y);
  }
  return *reinterpret_cast<const uint2 *>(p);
}
template <bool UNALIGNED>
__device__ __forceinline__ uint4 rg_load16(const void *p) {
  if (UNALIGNED) {
    RgU4 v;
    __builtin_memcpy(&v, p, 16);
    return make_uint4(v.x, v.y, v.z, v.w);
  }
  return *reinterpret_cast<const uint4 *>(p);
}

// element i of a zero / scale vector of run-time element type
__device__ __forceinline__ float rg_param(const void *p, int dtype, int i) {
  if (dtype == GPTQ_HIP_F32) return reinterpret_cast<const float *>(p)[i];
  if (dtype == GPTQ_HIP_F16) return __half2float(reinterpret_cast<const __half *>(p)[i]);
  return __bfloat162float(reinterpret_cast<const __hip_bfloat16 *>(p)[i]);
}

// Elements first .. first + 7 (indices clamped to n - 1) of a zero / scale vector as fp32.  The element
// type is switched on once, around eight independent loads: a switch per element would put every load
// behind a branch and make the wavefront wait for each in turn.
__device__ __forceinline__ void rg_params8(const void *p, int dtype, int first, int n, float (&out)[8]) {
  int idx[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) idx[i] = min(first + i, n - 1);
  if (dtype == GPTQ_HIP_F32) {
    const float *q = reinterpret_cast<const float *>(p);
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = q[idx[i]];
  } else if (dtype == GPTQ_HIP_F16) {
    const __half *q = reinterpret_cast<const __half *>(p);
    __half h[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) h[i] = q[idx[i]];
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = __half2float(h[i]);
  } else {
    const __hip_bfloat16 *q = reinterpret_cast<const __hip_bfloat16 *>(p);
    __hip_bfloat16 h[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) h[i] = q[idx[i]];
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = __bfloat162float(h[i]);
  }
}

// The same eight elements as raw bits (16-bit types zero-extended), for values that are fetched one k-step ahead
// and converted when they are used: the conversion is what would make the wavefront wait for the loads.
__device__ __forceinline__ void rg_params8_raw(const void *p, int dtype, int64_t row_base, int first, int n,
                                               uint32_t (&out)[8]) {
  int idx[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) idx[i] = min(first + i, n - 1);
  if (dtype == GPTQ_HIP_F32) {
    const uint32_t *q = reinterpret_cast<const uint32_t *>(p) + row_base;
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = q[idx[i]];
  } else {
    const uint16_t *q = reinterpret_cast<const uint16_t *>(p) + row_base;
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = q[idx[i]];
  }
}
__device__ __forceinline__ float rg_raw_to_f32(uint32_t raw, int dtype) {
  if (dtype == GPTQ_HIP_F32) return __builtin_bit_cast(float, raw);
  if (dtype == GPTQ_HIP_F16) return (float)__builtin_bit_cast(half2_t, raw)[0];
  return __builtin_bit_cast(float, raw << 16);
}

// Activations of a ragged last k-step: the lane wants the 8 elements [k0, k0 + 8) of its row, of which
// only those below K exist; `a` was loaded from [kl, kl + 8) with kl = min(k0, K - 8) <= k0.  Returns the
// wanted elements with zeros past K (element = 16 bits).
__device__ __forceinline__ uint4 rg_mask_tail(uint4 a, int k0, int kl, int K) {
  const int valid = min(max(K - k0, 0), 8);          // elements of the chunk that exist
  const int sh = k0 - kl;                            // element shift, 0 .. 8
  // 128-bit right shift by 16 sh bits
  uint32_t w[8] = {a.x, a.y, a.z, a.w, 0u, 0u, 0u, 0u};
  uint32_t o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    uint32_t lo = 0u, hi = 0u;                       // words i + sh / 2 and the next one
#pragma unroll
    for (int j = 0; j < 5; ++j) {
      lo = (sh >> 1) == j ? w[i + j] : lo;
      hi = (sh >> 1) == j ? w[i + j + 1 < 8 ? i + j + 1 : 7] : hi;
    }
    o[i] = (sh & 1) ? ((lo >> 16) | (hi << 16)) : lo;
    const int e = 2 * i;                             // first element of this word
    const uint32_t m = (e + 1 < valid) ? 0xFFFFFFFFu : (e < valid ? 0x0000FFFFu : 0u);
    o[i] &= m;
  }
  return make_uint4(o[0], o[1], o[2], o[3]);
}

__device__ __forceinline__ uint2 rg_shr_bytes(uint2 v, int bytes) {   // 0 <= bytes <= 8
  const unsigned long long w = ((unsigned long long)v.y << 32) | v.x;
  const unsigned long long s = bytes >= 8 ? 0ull : (w >> (8 * bytes));
  return make_uint2((uint32_t)s, (uint32_t)(s >> 32));
}

// agent-scope 16-byte store / load of a partial tile: written through to memory, read past the L2 of the
// reading XCD (which may hold a stale line of the same workspace address from an earlier call)
__device__ __forceinline__ void rg_store_part(float *p, floatx4 v) {
  // (the s_nop keeps the next instruction from overwriting the data registers while the store still reads
  //  them: the compiler cannot see that this statement is a wide store)
  asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ floatx4 rg_load_part_issue(const float *p) {
  floatx4 v;
  asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v) : "v"(p) : "memory");
  return v;
}

// Sum of the four wavefronts' accumulators and, when the contraction is split over S workgroups per output
// tile, of the S workgroups' partial tiles.  A workgroup is four wavefronts that each hold RB x RG_NT tiles
// over a quarter of the workgroup's k-steps.  Row block rb is finished by wavefront rb (RB <= 4); on return `sum` holds that row block's complete tiles and the return value says
// whether this wavefront is to write them out (false for the wavefronts that own nothing and for all
// workgroups but the last arrival of a split tile).
//   S > 1: the owner wavefronts write their sums to part[tile][split][rb] with agent-scope write-through
//   stores and wait for them; after a barrier one thread takes an arrival ticket (relaxed atomic at agent
//   scope, executed at the memory side); the last workgroup of the tile reads all S partials with
//   agent-scope loads and adds them in split order, so the result does not depend on the arrival order,
//   and leaves the counter at zero for the next call.
// (NRB, R0: the wavefront holds NRB row blocks, of which this call sums the RB blocks R0 .. R0 + RB - 1; a
// 128-row tile goes through as two calls of four row blocks, with a barrier between them.)
template <int RB, int NRB = RB, int R0 = 0>
__device__ __forceinline__ bool rg_reduce(floatx4 (&acc)[NRB][RG_NT], floatx4 (&sum)[RG_NT], float *lds,
                                          int *s_flag, float *part, int32_t *counters, int tile, int split,
                                          int S) {
  const int tid = threadIdx.x, lane = tid & 63, wk = tid >> 6;
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int t = 0; t < RG_NT; ++t)
      *reinterpret_cast<floatx4 *>(lds + (((wk * RB + rb) * RG_NT + t) * 64 + lane) * 4) = acc[R0 + rb][t];
  __syncthreads();
  const bool owner = wk < RB;
  const int rb_own = owner ? wk : 0;
#pragma unroll
  for (int t = 0; t < RG_NT; ++t) {
    floatx4 v = floatx4{0.f, 0.f, 0.f, 0.f};
    if (owner) {
#pragma unroll
      for (int w = 0; w < 4; ++w)
        v += *reinterpret_cast<const floatx4 *>(lds + (((w * RB + rb_own) * RG_NT + t) * 64 + lane) * 4);
    }
    sum[t] = v;
  }
  if (S == 1) return owner;
  float *mine = part + (((int64_t)tile * S + split) * RB + rb_own) * (RG_NT * RG_TILE_FLOATS) + lane * 4;
  if (owner) {
#pragma unroll
    for (int t = 0; t < RG_NT; ++t) rg_store_part(mine + t * RG_TILE_FLOATS, sum[t]);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");        // this wavefront's write-through stores have completed
  __syncthreads();
  if (tid == 0) {
    int32_t *ctr = counters + tile;
#ifdef GPTQ_TICKET_RELACQ
    const int ticket = __hip_atomic_fetch_add(ctr, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
#else
    const int ticket = __hip_atomic_fetch_add(ctr, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#endif
    const int last = ticket == S - 1;
    if (last) __hip_atomic_store(ctr, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *s_flag = last;
  }
  __syncthreads();
  if (!*s_flag || !owner) return false;
#pragma unroll
  for (int t = 0; t < RG_NT; ++t) sum[t] = floatx4{0.f, 0.f, 0.f, 0.f};
  const float *src = part + (((int64_t)tile * S) * RB + rb_own) * (RG_NT * RG_TILE_FLOATS) + lane * 4;
  // NF splits' partials in flight at a time (a 16-row workgroup has the registers for four)
  constexpr int NF = RB == 1 ? 4 : 2;
  for (int sp = 0; sp < S; sp += NF) {
    floatx4 pv[NF][RG_NT];
#pragma unroll
    for (int f = 0; f < NF; ++f) {
      const int sq = min(sp + f, S - 1);
#pragma unroll
      for (int t = 0; t < RG_NT; ++t)
        pv[f][t] = rg_load_part_issue(src + (int64_t)sq * RB * (RG_NT * RG_TILE_FLOATS) + t * RG_TILE_FLOATS);
    }
    // the loads above are invisible to the compiler's wait counting: wait here, and make every use of
    // the values depend on this statement
#pragma unroll
    for (int f = 0; f < NF; ++f)
      asm volatile("s_waitcnt vmcnt(0)"
                   : "+v"(pv[f][0]), "+v"(pv[f][1]), "+v"(pv[f][2]), "+v"(pv[f][3]), "+v"(pv[f][4]), "+v"(pv[f][5]),
                     "+v"(pv[f][6]), "+v"(pv[f][7]), "+v"(pv[f][8])
                   :
                   : "memory");
#pragma unroll
    for (int f = 0; f < NF; ++f) {
      if (sp + f < S) {
#pragma unroll
        for (int t = 0; t < RG_NT; ++t) sum[t] += pv[f][t];
      }
    }
  }
  return true;
}

}  // namespace qmm
