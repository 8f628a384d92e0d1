// Register-operand packed-weight matmul kernels (qmatmul_reg.hip), as the dispatcher in qmatmul.hip sees them.
#pragma once
#include "common.h"

namespace qmm {

// Plan of one forward product out[M, C] = x[M, K] @ dequant(packed[R, C]); bits = 4 (K = 2 R, two codes
// per byte along the rows) or 8 (K = R, one code per byte).
struct RegPlan {
  bool use;
  int bits, rb;            // rb: 16-row blocks per output tile (1 for M <= 16, else 4)
  bool ragged;             // C % 8 != 0, K % 8 != 0 or operands not 16-byte aligned: unaligned loads, element stores
  int S, steps;            // split of the contraction over S workgroups per tile, k-steps (32 k) per split
  bool atom;               // 16-row tiles: the splits add their results to 64-bit fixed-point cells (one returning
                           // atomic per output) instead of writing partial tiles and taking a ticket
  int64_t tiles;           // output tiles of one launch
  int tail_x;              // 128-row tiles: this many trailing column tiles run on 64-row tiles in a second launch
  // Not part of the plan proper; set by the caller for a product whose activations were fp32 rows scaled by
  // 2^-rowexp[m] and rounded to fp16: tiles of more than 16 rows then store ldexp(fp16(result), rowexp[m]) as
  // fp32 into out32 [M, C] instead of fp16 into `out`.
  float *out32;
  const int32_t *rowexp;
  size_t part_bytes, total_bytes;
};

RegPlan reg_fwd_plan(int64_t M, int64_t R, int64_t C, int bits, bool aligned);
// How a product on 128-row tiles (rb = 8) is dealt over launches: the leading wide_x tiles of 512 (half: 256)
// channels or output columns on the 128 x 512 tiles of qmatmul_wide.hip = `first` column tiles of 128, then main_x
// column tiles on 128-row tiles, then `tail` column tiles on 64-row tiles.  The launch functions and the plan
// query both go by this.
struct RegParts {
  int64_t wide_x;
  bool half;
  int64_t wide2_x;         // 256-channel (transposed: 256-column) tiles behind the whole rounds of 512-wide ones (part of `first`)
  int64_t first, main_x, tail;
};
RegParts reg_fwd_parts(const RegPlan &p, int64_t M, int64_t R, int64_t C, bool bf16, int group_size);
// x / out element type x_dtype (F16 or BF16), zero / scale element type zs_dtype (F32, F16, BF16).
// group_size = 0: zero / scale [C]; group_size > 0 (a multiple of 32): zero / scale [K / group_size, C].
int reg_fwd_launch(hipStream_t st, const RegPlan &p, const void *x, int x_dtype, int64_t M, const uint8_t *pk,
                   int64_t R, int64_t C, const void *zero, const void *scale, int zs_dtype, void *out, void *ws,
                   int group_size);

// Tall, narrow tiles for a few dozen rows (qmatmul_mid.hip; 4-bit codes, per-channel parameters, 16-byte aligned
// operands, fp16 activations, K % 256 == 0, C % 16 == 0; `use` is false where the other tiles are faster): a workgroup
// of eight wavefronts owns 16 rb rows x 16 nb channels over one of S ranges of `steps` k-steps.  out32 / rowexp as in
// RegPlan.
struct MidPlan {
  bool use, bf16;
  int rb, nb, S, steps;
  int64_t tiles_x, tiles_y;
  float *out32;
  const int32_t *rowexp;
  size_t part_bytes, total_bytes;
};
MidPlan mid_fwd_plan(int64_t M, int64_t R, int64_t C, bool aligned, bool bf16 = false);
int mid_fwd_launch(hipStream_t st, const MidPlan &p, const void *x, int64_t M, const uint8_t *pk, int64_t R, int64_t C,
                   const void *zero, const void *scale, int zs_dtype, void *out, void *ws);

// 128 x 512 tiles for many rows (qmatmul_wide.hip; 4-bit codes, or 8-bit codes with fp16 rows; per-channel
// parameters, aligned operands):
// number of leading 512-channel tiles they take (0: none; *half: tiles of 256 channels, four wavefronts of 64 x 128,
// for shapes whose 512-channel tiles are under one round), and the launch over those tiles.  out32 / rowexp as in
// RegPlan.
int64_t wide_fwd_tiles(int64_t M, int64_t R, int64_t C, bool aligned, bool *half, int bits = 4);
int wide_fwd_launch(hipStream_t st, const void *x, int x_dtype, int64_t M, const uint8_t *pk, int64_t R, int64_t C,
                    const void *zero, const void *scale, int zs_dtype, void *out, int64_t wide_x, bool half, float *out32,
                    const int32_t *rowexp, int bits = 4, int64_t c0 = 0);

// The same for the transposed product (fp16 rows; bf16 rows up to 16384 channels; 8-bit codes with fp16 rows:
// tiles of 512 / 256 output columns = as many packed rows): leading tiles of 512 output columns = 256 packed rows (*half: of 256
// output columns = 128 packed rows).
int64_t wide_bwd_tiles(int64_t M, int64_t R, int64_t C, bool aligned, bool *half, bool bf16 = false, int bits = 4);
int wide_bwd_launch(hipStream_t st, const void *x, int64_t M, const uint8_t *pk, int64_t R, int64_t C, const void *zero,
                    const void *scale, int zs_dtype, void *out, int64_t wide_x, bool half, float *out32,
                    const int32_t *rowexp, bool bf16 = false, int bits = 4, int64_t jbase = 0);

// Transposed product out[M, K] = x[M, C] @ dequant(packed[R, C])^T.
struct RegBwdPlan {
  bool use;
  int bits, rb;            // rb: 16-row blocks per output tile (4, or 8: 128-row tiles)
  int tail_x;              // 128-row tiles: this many trailing column tiles run on 64-row tiles in a second launch
  // set by the caller for fp32 rows (see RegPlan): the tiles store ldexp(fp16(result), rowexp[m]) as fp32
  float *out32;
  const int32_t *rowexp;
  bool ragged;
  bool no_wide;            // set by the caller when the packed matrix is not 16-byte aligned (the 128 x 512 tiles load 16 bytes)
  int S, steps;
  int64_t tiles;
  size_t part_bytes, total_bytes;
};
// rb = 8: 128-row tiles
RegBwdPlan reg_bwd_plan(int64_t M, int64_t R, int64_t C, int bits, bool aligned, int rb = 4);
RegParts reg_bwd_parts(const RegBwdPlan &p, int64_t M, int64_t R, int64_t C, bool bf16, int group_size);
// group_size > 0: a multiple of 128 (the 128 output columns of a tile share one group)
int reg_bwd_launch(hipStream_t st, const RegBwdPlan &p, const void *x, int x_dtype, int64_t M, const uint8_t *pk,
                   int64_t R, int64_t C, const void *zero, const void *scale, int zs_dtype, void *out, void *ws,
                   int group_size);

}  // namespace qmm
