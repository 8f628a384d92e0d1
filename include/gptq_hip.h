/*
 * gptq_hip.h -- C ABI of the MI355X (gfx950) GPTQ solve and packed-int4 matmul.
 *
 * This is the drop-in boundary: the entry points below are what a binding of the
 * reference's per-layer solve (jax_gptq/gptq.py) and of its quantized-matmul
 * custom call (jax_gptq/op.py:46-63, jt.triton_call) would bind.  Each entry
 * names the reference code it replaces (paths relative to the reference).
 *
 * Conventions (all entry points):
 *   - `stream` is a hipStream_t passed as void*; NULL means the default stream.
 *   - every pointer except the host tables named below is a DEVICE pointer;
 *   - matrices are row-major; W is [K, N] with K = input features (contraction
 *     axis 0) and N = output channels, exactly as in gptq.py:118,136-147;
 *   - calls only enqueue work on `stream`: no host synchronisation, no device
 *     allocation.  Scratch memory is passed in by the caller (`ws`, `ws_bytes`);
 *     the matching `*_workspace_bytes` query gives the required size;
 *   - return value 0 means success, otherwise a GPTQ_HIP_E* code; nothing throws.
 *   - thread-safe; no mutable global state (gptq_hip_qmatmul_static, at the end of this
 *     file, is the one exception: its calls share a fixed array per GPU).
 */
#ifndef GPTQ_HIP_H_
#define GPTQ_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GPTQ_HIP_ABI_VERSION 1

/* element types of float operands */
enum { GPTQ_HIP_F32 = 0, GPTQ_HIP_F16 = 1, GPTQ_HIP_BF16 = 2, GPTQ_HIP_F64 = 3 };

/* status codes */
enum {
  GPTQ_HIP_OK = 0,
  GPTQ_HIP_EINVAL = 1,      /* bad shape / null pointer / unsupported block size */
  GPTQ_HIP_EDTYPE = 2,      /* unsupported element type */
  GPTQ_HIP_EWORKSPACE = 3,  /* workspace too small */
  GPTQ_HIP_ELAUNCH = 4,     /* the HIP runtime refused a launch */
  GPTQ_HIP_ETOOBIG = 5      /* the problem needs more than the fixed scratch of gptq_hip_qmatmul_static */
};

int gptq_hip_abi_version(void);
const char *gptq_hip_error_string(int code);

/* ---- buffer helpers of the solve's driver --------------------------------------------------------
 * What the reference gets from XLA around its kernels: the zero-filled H and mean (gptq.py:90-95),
 * the fp32 working copy of W (gptq.py:184) and the copy of a matrix that a later step still needs.
 * fill_zero / copy: device pointers, 16-byte aligned, any byte count.  to_f32: n elements of type
 * in_dtype (F32, F16, BF16) widened to fp32.  Fill kernels rather than memsets, so that the calls can
 * be recorded into a captured graph. */
int gptq_hip_fill_zero(void *stream, void *ptr, size_t bytes);
int gptq_hip_copy(void *stream, void *dst, const void *src, size_t bytes);
int gptq_hip_to_f32(void *stream, const void *in, int in_dtype, int64_t n, float *out);

/* Measurement aid, not part of the path: reads `bytes` bytes (16-byte aligned) linearly with `workgroups`
 * workgroups of 256 threads, eight 16-byte loads in flight per thread, and does nothing else.  Its duration
 * is what the memory system delivers to a pure read of that size on this device: the yardstick bench.py
 * reports next to the HBM-bound matmul.  `sink` is a device word that is (practically) never written. */
int gptq_hip_read_probe(void *stream, const void *ptr, size_t bytes, int workgroups, uint32_t *sink);

/* ---- per-column quantisation parameters -------------------------------------
 * Replaces get_quantize_params / get_col_quantize_params (gptq.py:105-118).
 * W [K, N] (element type w_dtype, row stride ldw) -> scale[N], zero[N] (fp32).
 * maxq = 2^bits - 1.  ws: gptq_hip_col_params_workspace_bytes(K, N). */
size_t gptq_hip_col_params_workspace_bytes(int64_t K, int64_t N);
int gptq_hip_col_params(void *stream, const void *W, int w_dtype, int64_t K, int64_t N,
                        int64_t ldw, int bits, float *scale, float *zero, void *ws,
                        size_t ws_bytes);

/* fp32 rows on the 16-bit matrix cores (opt-in; the reference has no counterpart: its
 * gptq.py:65-72 multiplies in fp32).  Every element is split as x = (hi + lo) 2^e, hi and lo
 * fp16, e one exponent for the whole call, and X^T X = 4^e (hi^T hi + hi^T lo + lo^T hi) is
 * accumulated in fp32 from exact fp16 products; the dropped lo^T lo term is below 2^-22 of each
 * product.  2.2 times faster than gptq_hip_hessian_accumulate on fp32 rows (K = 4096).  Requires
 * K % 256 == 0 and every batch a multiple of 32 rows and 16-byte aligned; returns
 * GPTQ_HIP_EINVAL otherwise (use gptq_hip_hessian_accumulate then).
 * H += sum_b X_b^T X_b (upper tiles), fp32; ws: ..._split16_workspace_bytes(K, largest batch). */
size_t gptq_hip_hessian_accumulate_split16_workspace_bytes(int64_t K, int64_t max_batch_rows);
int gptq_hip_hessian_accumulate_split16(void *stream, const void *const *x_ptrs, const int64_t *x_rows,
                                        int n_batches, int64_t K, float *H, void *ws, size_t ws_bytes);

/* ---- Hessian ------------------------------------------------------------------
 * Replaces _accumulate_H_step / accumulate_H (gptq.py:57-103).
 * gptq_hip_hessian_accumulate adds sum_b X_b^T X_b to the UPPER triangle (128x128
 * tile granularity) of H [K, K], whose element type h_dtype is GPTQ_HIP_F32 or, for the
 * reference's use_fp64 option (gptq.py:88, 182-187), GPTQ_HIP_F64 (products and sums in
 * double; the batches may then be fp64 too).  x_ptrs / x_rows are HOST arrays of
 * n_batches device pointers / row counts; batch b is [x_rows[b], K] row-major,
 * contiguous.  All batches of one call are reduced in one launch (in registers), so
 * passing the whole calibration set at once is the fast path; one batch per call
 * reproduces the reference's streaming use.  The running mean of the reference cancels
 * algebraically (H = sum X^T X / n), so none is kept.
 * ws: gptq_hip_hessian_accumulate_workspace_bytes(K, h_dtype) bytes (0 for fp64; partial tiles of the row slices
 * of a long call or of the equal runs of (tile, row slab) pairs that a call of up to 32768 fp32 rows is cut into).
 * gptq_hip_hessian_finalize multiplies by 1/n_samples and mirrors the upper
 * triangle into the lower one, giving the full symmetric H the reference returns.
 * Limits: K <= 46000 (one launch's table of tiles), a call's batches at most 2^31 rows in all;
 * GPTQ_HIP_EINVAL beyond them. */
size_t gptq_hip_hessian_accumulate_workspace_bytes(int64_t K, int h_dtype);
int gptq_hip_hessian_accumulate(void *stream, const void *const *x_ptrs, const int64_t *x_rows,
                                int n_batches, int x_dtype, int64_t K, void *H, int h_dtype,
                                void *ws, size_t ws_bytes);
int gptq_hip_hessian_finalize(void *stream, void *H, int h_dtype, int64_t K, double n_samples);

/* ---- dead features, damping, Cholesky factor of the inverse -----------------------
 * Replaces _damp_and_invert + _cholesky_inv (gptq.py:155-168, 44-48).
 * H [K, K] full symmetric, element type h_dtype = GPTQ_HIP_F32 or GPTQ_HIP_F64 (read; its
 * diagonal is rewritten with the dead-feature fix and the damping, as the reference's
 * donated buffer is); W [K, N] fp32 (rows of dead features zeroed in place; may be NULL
 * with N = 0); L [K, K] out, same element type as H: lower triangular,
 * L L^T = (H + damping*mean(diag H) I)^-1, upper part zero.  L32 (may be NULL) also
 * receives L rounded to fp32, the cast of gptq.py:197 that feeds the column loop.
 * status (device int32[2]): status[0] = 0, or 1 + index of the first 64-block whose
 * pivot was not positive (L then holds NaN, as the reference's does, gptq.py:166);
 * status[1] = number of dead features.  fix_dead = 0 skips the dead-feature fix (with
 * damping = 0 the call is then exactly _cholesky_inv, gptq.py:44-48).
 * Limit: K <= 65535 (rows are a grid dimension), also for gptq_hip_zero_dead_rows and the
 * gathers below; GPTQ_HIP_EINVAL beyond it. */
size_t gptq_hip_damp_invert_workspace_bytes(int64_t K, int h_dtype);
int gptq_hip_damp_invert(void *stream, void *H, int h_dtype, float *W, int64_t K, int64_t N,
                         int64_t ldw, double damping, int fix_dead, void *L, float *L32,
                         int32_t *status, void *ws, size_t ws_bytes);

/* Only the dead-feature part of _damp_and_invert (gptq.py:157-159) for a caller that solves
 * several matrices against one Hessian and keeps the factor L of the first call: rows i of
 * W [K, N] (fp32, row pitch ldw) with H_ii == 0 are zeroed; H [K, K] (h_dtype F32 or F64) is
 * the Hessian as accumulated (before damp_invert rewrote its diagonal) and is only read. */
int gptq_hip_zero_dead_rows(void *stream, const void *H, int h_dtype, int64_t K, float *W, int64_t N,
                            int64_t ldw);

/* ---- blocked column loop ------------------------------------------------------------
 * Replaces the loop of gptq() with _process_block and the lazy update
 * (gptq.py:199-208, 130-153).  W [K, N] fp32 is consumed (overwritten).  L [K, K]
 * lower factor from gptq_hip_damp_invert.  Outputs (either may be NULL):
 *   Q      [K, N] dequantised values scale*(q - zero) in element type q_dtype
 *          (what gptq() returns, gptq.py:208,212);
 *   codes  [K, N] uint8 integer codes q.
 * block_size must divide K and be <= 128 (the reference's default is 128).
 * ws: gptq_hip_solve_workspace_bytes(K, N, block_size). */
size_t gptq_hip_solve_workspace_bytes(int64_t K, int64_t N, int block_size);
int gptq_hip_solve(void *stream, float *W, int64_t K, int64_t N, const float *L,
                   const float *scale, const float *zero, int maxq, int block_size, void *Q,
                   int q_dtype, uint8_t *codes, void *ws, size_t ws_bytes);

/* One block of the loop: replaces _process_block (gptq.py:130-153).  Wblock points at
 * the first of the block's block_size rows of W [*, N] (read only); Lblock points at
 * L[start][start] (row stride ldl).  Outputs:
 * Qblock / codes_block [block_size, N] (either may be NULL) and errors [block_size, N]
 * fp32, the (w - q) / L_ii rows that the lazy update consumes. */
int gptq_hip_process_block(void *stream, const float *Wblock, int64_t N, const float *Lblock,
                           int64_t ldl, int block_size, const float *scale, const float *zero,
                           int maxq, void *Qblock, int q_dtype, uint8_t *codes_block,
                           float *errors);

/* The lazy batch update that follows a block (or a group of blocks): replaces
 *   W = W.at[end:, :].add(-(Hinv[end:, start:end] @ errors))        (gptq.py:204-205).
 * Wbelow points at W[end][0] ([rows, N], updated in place), Lpanel at L[end][start] (row stride ldl),
 * errors is [k, N] fp32 as gptq_hip_process_block writes them (k = end - start rows, or the rows of several
 * consecutive blocks).  fp32 MFMA product, k summed in ascending order within a workgroup's tile. */
int gptq_hip_lazy_update(void *stream, float *Wbelow, int64_t N, const float *Lpanel, int64_t ldl, const float *errors,
                         int64_t rows, int64_t k);

/* ---- activation order ---------------------------------------------------------------
 * Replaces the gathers of _permute / _unpermute (gptq.py:170-180); the argsort itself
 * stays with the caller.  out[i, :] = in[perm[i], :] for rows; the symmetric form
 * gathers rows and columns: out[i, j] = in[perm[i], perm[j]].  perm is device int64[K];
 * elem_bytes is 1, 2, 4 or 8 for rows and 4 or 8 for the symmetric form. */
int gptq_hip_gather_rows(void *stream, const void *in, void *out, int elem_bytes, int64_t K,
                         int64_t N, const int64_t *perm);
int gptq_hip_gather_sym(void *stream, const void *in, void *out, int elem_bytes, int64_t K,
                        const int64_t *perm);

/* ---- int4 codec -----------------------------------------------------------------------
 * A tensor is viewed as [outer, axis_len, inner] and packed along the middle axis:
 * byte[o, j, i] = c[o, 2j, i] | c[o, 2j+1, i] << 4   (gptq.py:237-249, 265-292).
 * axis_len must be even for pack.  unpack is the inverse (gptq.py:251-263).
 * codes are taken modulo 256 from elements of code_bytes bytes (1 = uint8, 4 = int32,
 * 8 = int64). */
int gptq_hip_pack_int4(void *stream, const void *codes, int code_bytes, int64_t outer,
                       int64_t axis_len, int64_t inner, uint8_t *packed);
int gptq_hip_unpack_int4(void *stream, const uint8_t *packed, int64_t outer,
                         int64_t packed_axis_len, int64_t inner, uint8_t *codes);
/* pack_matrix (gptq.py:214-228): c = uint8(rint(Q/scale + zero)) then pack along the
 * middle axis; scale/zero are fp32 and indexed [o, i] (the contraction axis removed). */
int gptq_hip_quantize_pack(void *stream, const void *Q, int q_dtype, int64_t outer,
                           int64_t axis_len, int64_t inner, const float *scale,
                           const float *zero, uint8_t *packed);
/* unpack_matrix (gptq.py:230-235): out = (code - zero) * scale in element type
 * zs_dtype (that of zero/scale, which is also the output type, gptq.py:20-22). */
int gptq_hip_dequant(void *stream, const uint8_t *packed, int64_t outer,
                     int64_t packed_axis_len, int64_t inner, const void *zero,
                     const void *scale, int zs_dtype, void *out);

/* The same two for 8-bit codes (no counterpart in the reference, which packs 4-bit codes only,
 * gptq.py:241,253): bits = 4 is exactly the call above; bits = 8 stores / reads one code per byte,
 * c = uint8(rint(Q/scale + zero)) clipped to [0, 255], so `packed` has axis_len (quantize) resp.
 * packed_axis_len (dequant) bytes along the middle axis and the dense tensor has as many elements. */
int gptq_hip_quantize_pack_bits(void *stream, const void *Q, int q_dtype, int64_t outer, int64_t axis_len,
                                int64_t inner, const float *scale, const float *zero, int bits,
                                uint8_t *packed);
int gptq_hip_dequant_bits(void *stream, const uint8_t *packed, int64_t outer, int64_t packed_axis_len,
                          int64_t inner, const void *zero, const void *scale, int zs_dtype, int bits, void *out);

/* ---- packed-int4 matmul ------------------------------------------------------------------
 * Replaces the jt.triton_call custom call of _quantized_matmul (op.py:19-69) and the two
 * Triton kernels behind it (kernel.py:17-127, 141-253).
 * packed [R, C] uint8 holds W [2R, C] (contraction axis 0).  zero/scale [C] of type
 * zs_dtype.  x [M, Kx] and out of type x_dtype.
 *   transpose_b = 0: Kx = 2R, out [M, C]  = x @ ((code - zero) * scale)
 *   transpose_b = 1: Kx = C,  out [M, 2R] = x @ ((code - zero) * scale)^T
 * fp32 accumulation; the result is rounded to fp16 and then converted to x_dtype, as
 * op.py:43,66-68 does.  ws: gptq_hip_qmatmul_workspace_bytes(M, R, C, transpose_b) bytes.
 * fp32 activations (the reference's dot rounds them to TF32, kernel.py:106): with a workspace of
 * gptq_hip_qmatmul_workspace_bytes_x(..., GPTQ_HIP_F32) bytes and C % 16 == 0 they are rounded
 * to fp16 precision (after a per-row power-of-two scaling that keeps any fp32 magnitude in
 * range; the result is scaled back after its rounding to fp16) and run on the same matrix-core kernels as fp16 ones; with the smaller workspace, or
 * other shapes, they run unrounded on plain kernels that are an order of magnitude slower.
 * Any M, R, C below 2^30: shapes with C % 16 == 0 and 16-byte aligned operands run on the tuned
 * kernels, other shapes with C >= 8 and 2R >= 8 (rows that are not multiples of 16 channels, e.g. a
 * vocabulary-sized C; unaligned views) on matrix-core kernels that take unaligned loads, the rest on
 * plain kernels (several launches where M exceeds a grid dimension).
 * The workspace begins with arrival counters of the split-K reduction: it must be
 * ZERO-FILLED before its first use; every call leaves the counters zero again, so one
 * buffer can serve any sequence of calls that do not overlap in time.
 * Range of the split sums: where up to 16 rows (forward) are summed over S > 1 workgroups through the workspace's
 * 64-bit cells, a workgroup's PARTIAL result enters as a fixed-point number (2^-28 steps): a partial that is
 * not finite or beyond +-65536 poisons its cell, and that output is NaN.  The reference accumulates in fp32 and
 * casts to fp16 (kernel.py:111, op.py:43), so it yields +-inf for a result beyond the fp16 range and a finite value
 * where partial sums of that size cancel; here both cases give NaN.  Results within the fp16 range whose partial sums
 * stay within +-65536 (every product of fp16-range activations with 4-bit weights of sensible scale) are summed
 * exactly, in an order-independent way. */
size_t gptq_hip_qmatmul_workspace_bytes(int64_t M, int64_t R, int64_t C, int transpose_b);
size_t gptq_hip_qmatmul_workspace_bytes_x(int64_t M, int64_t R, int64_t C, int transpose_b, int x_dtype);
int gptq_hip_qmatmul(void *stream, const void *x, int x_dtype, int64_t M, const uint8_t *packed,
                     int64_t R, int64_t C, const void *zero, const void *scale, int zs_dtype,
                     int transpose_b, void *out, void *ws, size_t ws_bytes);

/* ---- which kernel a product runs on (host only: nothing is launched, no device is touched) ----------
 * No counterpart in the reference, whose Triton kernel picks its tiles by autotuning at run time
 * (kernel.py:4-16).  gptq_hip_qmatmul_plan_query fills *plan with what gptq_hip_qmatmul /
 * gptq_hip_qmatmul_bits / gptq_hip_qmatmul_grouped would run for these arguments when they are given the
 * workspace their size query names: `kernel` takes the product or its leading columns, `kernel_rest` (0 if none) the
 * remaining columns, `splits` workgroups share one output tile's contraction, `workgroups` is the first kernel's
 * grid (0 where it is not planned ahead), `fp32_rows` says how fp32 activations travel (0: as they are, 1: scaled
 * and rounded to fp16 rows in the workspace by a kernel of their own, 2: inside the product's kernel).  `aligned`:
 * all operands 16-byte aligned (1) or only to their element size (0).  For tests that keep every kernel family
 * reachable, benchmarks that name the kernel they time, and callers that want to know. */
enum {
  GPTQ_HIP_QMM_SIMPLE = 1,        /* one thread per output */
  GPTQ_HIP_QMM_DECODE = 2,        /* up to 16 rows: 256-channel strips, all loads in flight at once */
  GPTQ_HIP_QMM_DECODE_RAGGED = 3, /* the same for rows of any length */
  GPTQ_HIP_QMM_CHUNKED = 4,       /* up to 16 rows per chunk, activations only 4-byte aligned */
  GPTQ_HIP_QMM_MID = 6,           /* 17 to a few dozen rows: tall, narrow tiles */
  GPTQ_HIP_QMM_REG16 = 7,         /* register-operand tiles of 16, 64, 128 rows x 128 channels */
  GPTQ_HIP_QMM_REG64 = 8,
  GPTQ_HIP_QMM_REG128 = 9,
  GPTQ_HIP_QMM_WIDE = 10,         /* 128 x 512 tiles, activations shared through LDS */
  GPTQ_HIP_QMM_WIDE_HALF = 11,    /* 128 x 256 */
  GPTQ_HIP_QMM_BWD_SIMPLE = 21,   /* transposed product */
  GPTQ_HIP_QMM_BWD_REG64 = 22,
  GPTQ_HIP_QMM_BWD_REG128 = 23,
  GPTQ_HIP_QMM_BWD_WIDE = 24,
  GPTQ_HIP_QMM_BWD_WIDE_HALF = 25,
  GPTQ_HIP_QMM_BWD_GEMM = 26      /* weights dequantised into LDS */
};
typedef struct gptq_hip_qmatmul_plan {
  int kernel, kernel_rest, splits, fp32_rows;
  int64_t workgroups;
} gptq_hip_qmatmul_plan;
int gptq_hip_qmatmul_plan_query(int64_t M, int64_t R, int64_t C, int transpose_b, int x_dtype, int zs_dtype, int bits,
                                int64_t group_size, int aligned, gptq_hip_qmatmul_plan *plan);
const char *gptq_hip_qmatmul_kernel_name(int kernel);

/* ---- the same product for 8-bit codes -----------------------------------------------------------
 * No counterpart in the reference, whose packing and kernels are fixed at 4 bits (gptq.py:241,253,
 * kernel.py:92-104); for the 8-bit codes gptq() can produce here (bits = 8).  bits = 4: exactly
 * gptq_hip_qmatmul.  bits = 8: packed [R, C] uint8 holds one code per byte, W is [R, C] (Kx = R for
 * transpose_b = 0, out [M, R] for transpose_b = 1); everything else as above.
 * ws: gptq_hip_qmatmul_bits_workspace_bytes(M, R, C, transpose_b, x_dtype, bits) bytes, zero-filled before
 * its first use like the workspace of gptq_hip_qmatmul (one buffer can serve both). */
size_t gptq_hip_qmatmul_bits_workspace_bytes(int64_t M, int64_t R, int64_t C, int transpose_b, int x_dtype,
                                             int bits);
int gptq_hip_qmatmul_bits(void *stream, const void *x, int x_dtype, int64_t M, const uint8_t *packed,
                          int64_t R, int64_t C, const void *zero, const void *scale, int zs_dtype, int bits,
                          int transpose_b, void *out, void *ws, size_t ws_bytes);

/* ---- grouped parameters ------------------------------------------------------------------------
 * No counterpart in the reference, which has one scale / zero per output channel (gptq.py:105-118):
 * here every group of group_size consecutive input features (rows of W) has its own scale / zero per
 * channel, tables [K / group_size, N] (fp32 from the solve).
 * gptq_hip_solve_grouped is gptq_hip_solve with the parameters of rows [r0, r0 + group_size) taken, when
 * the column loop reaches r0, from the column minima / maxima of those rows as they then stand (every
 * correction of the rows above applied), by the rule of get_col_quantize_params (gptq.py:105-118) with
 * maxq = 2^bits - 1, and written to row r0 / group_size of scale_g / zero_g.  group_size must be a multiple
 * of block_size, divide K and divide the loop's update group (512 rows for block_size 128): 128, 256, 512.
 * ws: gptq_hip_solve_grouped_workspace_bytes.
 * quantize_pack_grouped / dequant_grouped: pack_matrix / unpack_matrix (gptq.py:214-235) for a 2-D W [K, N]
 * packed along the rows with such tables (group_size even, dividing K; bits 4 or 8).
 * gptq_hip_qmatmul_grouped: the product of gptq_hip_qmatmul_bits with zero / scale [K / group_size, C];
 * matrix-core kernels for group_size % 32 == 0 (transpose_b = 1: % 128 == 0), plain kernels otherwise;
 * ws as for gptq_hip_qmatmul_bits (gptq_hip_qmatmul_bits_workspace_bytes). */
size_t gptq_hip_solve_grouped_workspace_bytes(int64_t K, int64_t N, int block_size, int group_size);
int gptq_hip_solve_grouped(void *stream, float *W, int64_t K, int64_t N, const float *L, int group_size, int bits,
                           int block_size, void *Q, int q_dtype, uint8_t *codes, float *scale_g, float *zero_g,
                           void *ws, size_t ws_bytes);
int gptq_hip_quantize_pack_grouped(void *stream, const void *Q, int q_dtype, int64_t K, int64_t N, const float *scale,
                                   const float *zero, int64_t group_size, int bits, uint8_t *packed);
int gptq_hip_dequant_grouped(void *stream, const uint8_t *packed, int64_t R, int64_t C, const void *zero,
                             const void *scale, int zs_dtype, int64_t group_size, int bits, void *out);
int gptq_hip_qmatmul_grouped(void *stream, const void *x, int x_dtype, int64_t M, const uint8_t *packed,
                             int64_t R, int64_t C, const void *zero, const void *scale, int zs_dtype,
                             int64_t group_size, int bits, int transpose_b, void *out, void *ws, size_t ws_bytes);

/* ---- packed-int4 matmul that allocates nothing and takes no workspace ----------------------
 * No counterpart in the reference.  For callers that cannot allocate device memory: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  Same operation,
 * arguments and results as gptq_hip_qmatmul; the workspace is a fixed array of
 * GPTQ_HIP_QMATMUL_STATIC_BYTES bytes of device memory inside the library (one copy per GPU,
 * held until the process ends), so the call makes no hipMalloc / hipFree and calls no allocating
 * routine.  A problem whose gptq_hip_qmatmul_workspace_bytes_x(M, R, C, transpose_b, x_dtype)
 * exceeds GPTQ_HIP_QMATMUL_STATIC_BYTES is refused with GPTQ_HIP_ETOOBIG and nothing is enqueued.
 * All calls on one GPU share the one array: calls that may overlap in time on a GPU (different
 * streams, different threads) race on it; serialise them or use gptq_hip_qmatmul with a workspace
 * per stream.  Nothing is cleared at run time (the array is zero when the library is loaded and every
 * product leaves its counters at zero), so a call enqueues the product's kernels and nothing else.  The FIRST
 * call on a device for a given kind of product makes host-side runtime calls that do not belong under stream
 * capture (it looks up the array's address; kernels that need more than 64 KB of LDS have their limit raised
 * once): make one eager call of the same shape before capturing, as a warm-up. */
#define GPTQ_HIP_QMATMUL_STATIC_BYTES ((size_t)32 << 20)
int gptq_hip_qmatmul_static(void *stream, const void *x, int x_dtype, int64_t M, const uint8_t *packed,
                            int64_t R, int64_t C, const void *zero, const void *scale, int zs_dtype,
                            int transpose_b, void *out);

#ifdef __cplusplus
}
#endif
#endif /* GPTQ_HIP_H_ */
