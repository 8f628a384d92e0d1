// Types, activation traits and the workspace layout shared by the packed-weight matmul kernels.
#pragma once
#include "common.h"

namespace qmm {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// 16-bit activation types of the MFMA kernels
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
template <typename TX> struct Act;
template <> struct Act<__half> {
  static constexpr bool BF = false;
  static __device__ __forceinline__ float lo(uint32_t w) { return (float)__builtin_bit_cast(half2_t, w)[0]; }
  static __device__ __forceinline__ float hi(uint32_t w) { return (float)__builtin_bit_cast(half2_t, w)[1]; }
  static __device__ __forceinline__ floatx4 mma(const uint4 &a, const uint4 &b, floatx4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a),
                                                  __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
  }
  // The same MFMA with the accumulator tied in place: `acc` in accumulation registers, `accv` in vector
  // registers.  For kernels whose accumulators fill the accumulation file: the compiler's own form of the
  // instruction may write a different register than it reads, which then costs a copy per tile and k-step.
  // (Inline asm is outside the compiler's hazard handling.  An MFMA must not read an operand register within two
  // wait states of the vector instruction that wrote it, hence the s_nop in front; callers keep the reads of
  // the result away from the last MFMA, see mma_drain.)
  static __device__ __forceinline__ void mma_acc(floatx4 &c, const uint4 &a, const uint4 &b) {
    asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, %0"
                 : "+a"(c) : "v"(__builtin_bit_cast(u32x4_t, a)), "v"(__builtin_bit_cast(u32x4_t, b)));
  }
  static __device__ __forceinline__ void mma_accv(floatx4 &c, const uint4 &a, const uint4 &b) {
    asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, %0"
                 : "+v"(c) : "v"(__builtin_bit_cast(u32x4_t, a)), "v"(__builtin_bit_cast(u32x4_t, b)));
  }
  // The same two without the wait states: for a caller whose source order guarantees that the instruction in
  // front of the MFMA is not a vector instruction that writes one of its operands (e.g. another MFMA).
  static __device__ __forceinline__ void mma_acc_nw(floatx4 &c, const uint4 &a, const uint4 &b) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0"
                 : "+a"(c) : "v"(__builtin_bit_cast(u32x4_t, a)), "v"(__builtin_bit_cast(u32x4_t, b)));
  }
  static __device__ __forceinline__ void mma_accv_nw(floatx4 &c, const uint4 &a, const uint4 &b) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0"
                 : "+v"(c) : "v"(__builtin_bit_cast(u32x4_t, a)), "v"(__builtin_bit_cast(u32x4_t, b)));
  }
  // mma_acc_nw that also counts as a use of `dep` (which the instruction does not read): whatever computes
  // `dep` is thereby placed in front of this MFMA, so the MFMA that really reads it, further down, has this one
  // between itself and the write.  (The compiler is otherwise free to sink a computation down to its first use.)
  static __device__ __forceinline__ void mma_acc_nw_after(floatx4 &c, const uint4 &a, const uint4 &b, uint32_t dep) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0"
                 : "+a"(c) : "v"(__builtin_bit_cast(u32x4_t, a)), "v"(__builtin_bit_cast(u32x4_t, b)), "v"(dep));
  }
  static __device__ __forceinline__ void mma_acc_nw_after2(floatx4 &c, const uint4 &a, const uint4 &b, uint32_t dep0,
                                                           uint32_t dep1) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0"
                 : "+a"(c)
                 : "v"(__builtin_bit_cast(u32x4_t, a)), "v"(__builtin_bit_cast(u32x4_t, b)), "v"(dep0), "v"(dep1));
  }
  static __device__ __forceinline__ __half out(float v) { return __float2half_rn(v); }
};
template <> struct Act<__hip_bfloat16> {
  static constexpr bool BF = true;
  typedef __bf16 bf8_t __attribute__((ext_vector_type(8)));
  static __device__ __forceinline__ float lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
  static __device__ __forceinline__ float hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xFFFF0000u); }
  static __device__ __forceinline__ floatx4 mma(const uint4 &a, const uint4 &b, floatx4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8_t, a),
                                                   __builtin_bit_cast(bf8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ void mma_acc(floatx4 &c, const uint4 &a, const uint4 &b) {
    asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %2, %0"
                 : "+a"(c) : "v"(__builtin_bit_cast(u32x4_t, a)), "v"(__builtin_bit_cast(u32x4_t, b)));
  }
  static __device__ __forceinline__ void mma_accv(floatx4 &c, const uint4 &a, const uint4 &b) {
    asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %2, %0"
                 : "+v"(c) : "v"(__builtin_bit_cast(u32x4_t, a)), "v"(__builtin_bit_cast(u32x4_t, b)));
  }
  // The same two without the wait states: for a caller whose source order guarantees that the instruction in
  // front of the MFMA is not a vector instruction that writes one of its operands (e.g. another MFMA).
  static __device__ __forceinline__ void mma_acc_nw(floatx4 &c, const uint4 &a, const uint4 &b) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0"
                 : "+a"(c) : "v"(__builtin_bit_cast(u32x4_t, a)), "v"(__builtin_bit_cast(u32x4_t, b)));
  }
  static __device__ __forceinline__ void mma_accv_nw(floatx4 &c, const uint4 &a, const uint4 &b) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0"
                 : "+v"(c) : "v"(__builtin_bit_cast(u32x4_t, a)), "v"(__builtin_bit_cast(u32x4_t, b)));
  }
  // mma_acc_nw that also counts as a use of `dep` (which the instruction does not read): whatever computes
  // `dep` is thereby placed in front of this MFMA, so the MFMA that really reads it, further down, has this one
  // between itself and the write.  (The compiler is otherwise free to sink a computation down to its first use.)
  static __device__ __forceinline__ void mma_acc_nw_after(floatx4 &c, const uint4 &a, const uint4 &b, uint32_t dep) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0"
                 : "+a"(c) : "v"(__builtin_bit_cast(u32x4_t, a)), "v"(__builtin_bit_cast(u32x4_t, b)), "v"(dep));
  }
  static __device__ __forceinline__ void mma_acc_nw_after2(floatx4 &c, const uint4 &a, const uint4 &b, uint32_t dep0,
                                                           uint32_t dep1) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0"
                 : "+a"(c)
                 : "v"(__builtin_bit_cast(u32x4_t, a)), "v"(__builtin_bit_cast(u32x4_t, b)), "v"(dep0), "v"(dep1));
  }
  static __device__ __forceinline__ __hip_bfloat16 out(float v) { return __float2bfloat16(v); }
};
// After the last mma_acc / mma_accv and before anything reads their accumulators: an MFMA's result is
// written several passes after its issue, and nothing but wait states keeps a read from overtaking it.
__device__ __forceinline__ void mma_drain() { asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); }

// Workspace layout (only touched when the K range is split over S > 1 workgroups):
//   [counters: QMM_COUNTER_BYTES, one int32 per (m-chunk, strip), zero between calls; the
//    size is fixed so that no other region of an earlier call can alias a counter]
//   [acc64: QMM_ACC_BYTES, see below]
//   [x1part:  (m-chunk, strip, split, 2, 16) fp32]   [part: (split, M, C) fp32]
// The last workgroup to finish a strip (atomic ticket) sums the S partials in split order,
// so the result does not depend on the arrival order, and resets the counter.
constexpr int QMM_COUNTER_BYTES = 65536;
constexpr int QMM_MAX_COUNTERS = QMM_COUNTER_BYTES / 4;
// After the counters: 64-bit accumulators of the decode kernel's split-K sum (M <= 4), one per output,
// zero between calls like the counters.  Counters and accumulators form the head of every workspace
// at fixed offsets, whatever the shape, so that calls of different shapes can share one buffer.
constexpr int QMM_ACC_BYTES = 4 << 20;
constexpr int QMM_HEAD_BYTES = QMM_COUNTER_BYTES + QMM_ACC_BYTES;
// Split-K sums through acc64: a contribution is value * 2^QD_FRAC in fixed point (a value beyond +-65536 or
// not finite adds QD_POISON instead) << 8 | 1; the low byte of the word counts the contributions.
constexpr int QD_FRAC = 28;
constexpr long long QD_POISON = 3LL << 49;

struct QmmWs {
  int32_t *counters;
  unsigned long long *acc64;
  float *x1part;
  float *part;
};

__host__ __device__ inline QmmWs qmm_ws(void *base_v, size_t x1_bytes) {
  char *base = reinterpret_cast<char *>(base_v);
  QmmWs ws;
  ws.counters = reinterpret_cast<int32_t *>(base);
  ws.acc64 = reinterpret_cast<unsigned long long *>(base + QMM_COUNTER_BYTES);
  ws.x1part = reinterpret_cast<float *>(base + QMM_HEAD_BYTES);
  ws.part = reinterpret_cast<float *>(base + QMM_HEAD_BYTES + x1_bytes);
  return ws;
}

// Output tile of this workgroup.  Workgroups are dealt to the 8 XCDs round-robin in dispatch order (x fastest),
// and each XCD has its own L2.  Column tile tx belongs to XCD tx % 8, which walks its column tiles in blocks of
// up to 8 row tiles: the workgroups running on an XCD at one time form a block of a few column tiles x a few row
// tiles, so a weight tile is fetched once per block of row tiles (not once per row tile and XCD) and a row tile's
// activations once per group of column tiles.  The last gx % 8 column tiles keep the plain order.
__device__ __forceinline__ void qmm_tile_coords(int &tx, int &ty) {
  const int gx = gridDim.x, gy = gridDim.y;
  if (gy == 1) {
    // One row of tiles: XCD j (workgroup ids j, j + 8, ...) takes a contiguous range of column tiles, so that a
    // cache line that two neighbouring tiles share (rows that do not start on line boundaries) is fetched into
    // one L2, not two.
    const int j = blockIdx.x & 7, k = blockIdx.x >> 3, q = gx >> 3, rem = gx & 7;
    tx = j * q + min(j, rem) + k;
    ty = 0;
    return;
  }
  const int id = blockIdx.x + gx * blockIdx.y;
  const int full = (gx >> 3) << 3;
  if (id < full * gy) {
    constexpr int BY = 8;
    const int c = id & 7, sl = id >> 3, nq = full >> 3;
    const int yb = min(sl / (BY * nq), (gy - 1) / BY);
    const int r = sl - yb * BY * nq, by = min(BY, gy - yb * BY);
    tx = (r / by) * 8 + c;
    ty = yb * BY + r % by;
  } else {
    const int r = id - full * gy, rem = gx - full;
    tx = full + r % rem;
    ty = r / rem;
  }
}

}  // namespace qmm
