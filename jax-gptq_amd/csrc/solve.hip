// Blocked GPTQ column loop: quantise block_size rows with error feedback, then push the
// accumulated error into the remaining rows with fp32 MFMA GEMMs: after every block into the
// rest of its 512-row group, after every group into everything below it.
//
// In-block kernel: the N output channels are independent, so one lane owns one channel and a
// workgroup of eight wavefronts owns 64 channels.  The workgroup first copies its channels of
// the block's rows and the block's corner of L into LDS (all loads of a wavefront in flight
// at once), then works out of LDS only.  The block is walked in sub-blocks of SB rows:
//   * the SB rows of a sub-block and their SB errors live in VGPRs (statically indexed,
//     fully unrolled triangle).  This part is a sequential chain per channel; all
//     wavefronts evaluate it redundantly (same instructions, same values), which saves a
//     broadcast of the errors and costs nothing: the chain is bound by latency, not by issue;
//   * the rows of the block below the sub-block are then updated in the LDS tile, the rows
//     dealt round-robin to the wavefronts; one barrier per sub-block.
// Each lane touches only its own column of the tile (no bank conflicts); L is read with
// broadcast reads (every lane the same address), the SB factors of one row are consecutive.
// W itself is not written.
//
// Every floating-point operation is the IEEE operation the reference writes (true
// division, round-half-even, separate multiply and subtract) and every element receives
// its updates in the reference's order, so given the same L and W the block result is
// bit-identical to a CPU evaluation of gptq.py:136-147.
#include "common.h"
#include "gemm_f32.h"

namespace {

constexpr int SOLVE_CH = 64;               // channels per workgroup (one per lane)
constexpr int SOLVE_NW = 8;                // wavefronts per workgroup (4: 45 us per block, 8: 40, 16: 52)
constexpr int SOLVE_TPB = SOLVE_CH * SOLVE_NW;

template <int SB, typename TQ>
__global__ __launch_bounds__(SOLVE_TPB) void block_quant_kernel(
    const float *Wb, int64_t N, const float *Lb, int64_t ldl, int bs, const float *scale,
    const float *zero, float maxq, TQ *Qb, uint8_t *cb, float *Err) {
  // Wb, Qb, cb: first row of the block in W, Q, codes; Lb: the block's diagonal corner of L
#pragma clang fp contract(off)
  extern __shared__ float smem[];
  float *Ln = smem;                 // Ln[j * bs + i] = Lb[j][i]
  float *Wl = smem + bs * bs;       // Wl[j * SOLVE_CH + lane] = W[block row j][channel]
  const int tid = threadIdx.x;
  const int lane = tid & (SOLVE_CH - 1);
  const int wave = tid / SOLVE_CH;
  const int64_t n = (int64_t)blockIdx.x * SOLVE_CH + lane;
  const bool live = n < N;
  const int64_t nl = live ? n : N - 1;   // lanes past the edge shadow the last channel, store nothing

  // ---- stage L's corner and the W tile; loads are unconditional (clamped) and batched so
  //      that a wavefront has 16 of them in flight before it waits
  {
    const int total = bs * bs;
    for (int base = 0; base < total; base += SOLVE_TPB * 16) {
      float v[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int idx = min(base + u * SOLVE_TPB + tid, total - 1);
        const int j = idx / bs, i = idx - j * bs;
        v[u] = Lb[(int64_t)j * ldl + i];
      }
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int idx = base + u * SOLVE_TPB + tid;
        if (idx < total) Ln[idx] = v[u];
      }
    }
    const float *src = Wb + nl;
    for (int j0 = wave; j0 < bs; j0 += SOLVE_NW * 16) {
      float v[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) v[u] = src[(int64_t)min(j0 + SOLVE_NW * u, bs - 1) * N];
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int j = j0 + SOLVE_NW * u;
        if (j < bs) Wl[j * SOLVE_CH + lane] = v[u];
      }
    }
  }
  const float sc = scale[nl], z = zero[nl];
  float *wcol = Wl + lane;
  __syncthreads();

  for (int r0 = 0; r0 < bs; r0 += SB) {
    float w[SB], e[SB];
#pragma unroll
    for (int t = 0; t < SB; ++t) w[t] = wcol[(r0 + t) * SOLVE_CH];
    const float *ld = Ln + r0 * bs + r0;  // diagonal sub-block
#pragma unroll
    for (int t = 0; t < SB; ++t) {
      float x = w[t];
#pragma unroll
      for (int u = 0; u < t; ++u) {
        const float upd = ld[t * bs + u] * e[u];
        x = x - upd;
      }
      float q = rintf(x / sc) + z;
      q = fminf(fmaxf(q, 0.f), maxq);
      const float qh = sc * (q - z);
      e[t] = (x - qh) / ld[t * bs + t];
      if (live && (t % SOLVE_NW) == wave) {   // the stores of a sub-block are dealt over the wavefronts
        const int64_t o = (int64_t)(r0 + t) * N + n;
        if (Qb) Qb[o] = from_f32<TQ>(qh);
        if (cb) cb[o] = (uint8_t)q;
        Err[o] = e[t];
      }
    }
    // rows of this block below the sub-block, round-robin over the wavefronts
#pragma unroll 2
    for (int j = r0 + SB + wave; j < bs; j += SOLVE_NW) {
      float x = wcol[j * SOLVE_CH];
      const float *lr = Ln + j * bs + r0;
#pragma unroll
      for (int u = 0; u < SB; ++u) {
        const float upd = lr[u] * e[u];
        x = x - upd;
      }
      wcol[j * SOLVE_CH] = x;
    }
    __syncthreads();
  }
}

template <int SB>
int launch_block(hipStream_t st, const float *W, int64_t N, const float *L, int64_t ldl, int bs,
                 const float *scale, const float *zero, float maxq, void *Q, int q_dtype,
                 uint8_t *codes, float *Err) {
  const dim3 grid((unsigned)ceil_div64(N, SOLVE_CH)), block(SOLVE_TPB);
  const size_t lds = ((size_t)bs * bs + (size_t)bs * SOLVE_CH) * sizeof(float);
  if (lds > 64 * 1024) {
    // up to 96 KB of the 160 KB LDS of a CU; the limit has to be raised per kernel
    const void *fn = q_dtype == GPTQ_HIP_F32
                         ? reinterpret_cast<const void *>(block_quant_kernel<SB, float>)
                         : (q_dtype == GPTQ_HIP_F16
                                ? reinterpret_cast<const void *>(block_quant_kernel<SB, __half>)
                                : reinterpret_cast<const void *>(block_quant_kernel<SB, __hip_bfloat16>));
    if (!gptq_raise_lds_limit(fn, (int)lds)) return GPTQ_HIP_ELAUNCH;
  }
  switch (q_dtype) {
    case GPTQ_HIP_F32:
      hipLaunchKernelGGL((block_quant_kernel<SB, float>), grid, block, lds, st, W, N, L, ldl,
                         bs, scale, zero, maxq, (float *)Q, codes, Err);
      break;
    case GPTQ_HIP_F16:
      hipLaunchKernelGGL((block_quant_kernel<SB, __half>), grid, block, lds, st, W, N, L, ldl,
                         bs, scale, zero, maxq, (__half *)Q, codes, Err);
      break;
    case GPTQ_HIP_BF16:
      hipLaunchKernelGGL((block_quant_kernel<SB, __hip_bfloat16>), grid, block, lds, st, W, N, L,
                         ldl, bs, scale, zero, maxq, (__hip_bfloat16 *)Q, codes, Err);
      break;
    default:
      return GPTQ_HIP_EDTYPE;
  }
  GPTQ_CHECK_LAUNCH();
  return GPTQ_HIP_OK;
}

bool block_size_ok(int bs) { return bs >= 1 && bs <= 128; }

// Rows whose error rows are kept together for one trailing update (a whole number of blocks).
// The rows below a group receive the updates of all its blocks in one product with k up to
// 512 instead of one product per block: every product reads and writes the rows it updates,
// so this cuts the traffic over the trailing part of W by the number of blocks in a group.
constexpr int GROUP_ROWS = 512;
int group_rows(int bs) { return (GROUP_ROWS / bs > 0 ? GROUP_ROWS / bs : 1) * bs; }

// C[m, n] -= A[m, k] @ B[k, n]
int trailing_update(hipStream_t st, const float *A, int64_t lda, const float *B, float *C,
                    int64_t N, int64_t m, int64_t k) {
  GemmArgs g;
  g.A = A;
  g.B = B;
  g.C = C;
  g.lda = lda;
  g.ldb = N;
  g.ldc = N;
  g.m = (int)m;
  g.n = (int)N;
  g.k = (int)k;
  g.alpha = -1.f;
  g.beta = 1.f;
  g.a_kmajor = 0;
  return gptq_gemm_f32(st, g);
}

int process_block(hipStream_t st, const float *Wb, int64_t N, const float *Lb, int64_t ldl, int bs,
                  const float *scale, const float *zero, int maxq, void *Qb, int q_dtype,
                  uint8_t *cb, float *Err) {
#define GPTQ_SB_CASE(SB) \
  return launch_block<SB>(st, Wb, N, Lb, ldl, bs, scale, zero, (float)maxq, Qb, q_dtype, cb, Err)
  if (bs % 16 == 0) GPTQ_SB_CASE(16);
  if (bs % 8 == 0) GPTQ_SB_CASE(8);
  if (bs % 4 == 0) GPTQ_SB_CASE(4);
  if (bs % 2 == 0) GPTQ_SB_CASE(2);
  GPTQ_SB_CASE(1);
#undef GPTQ_SB_CASE
}

}  // namespace

extern "C" {

size_t gptq_hip_solve_workspace_bytes(int64_t K, int64_t N, int block_size) {
  if (K <= 0 || N <= 0 || !block_size_ok(block_size)) return 0;
  return (size_t)group_rows(block_size) * (size_t)N * sizeof(float);
}

int gptq_hip_process_block(void *stream, const float *Wblock, int64_t N, const float *Lblock,
                           int64_t ldl, int block_size, const float *scale, const float *zero,
                           int maxq, void *Qblock, int q_dtype, uint8_t *codes_block,
                           float *errors) {
  if (!Wblock || !Lblock || !scale || !zero || !errors || N <= 0 || ldl < block_size)
    return GPTQ_HIP_EINVAL;
  if (!block_size_ok(block_size) || maxq < 1 || maxq > 255) return GPTQ_HIP_EINVAL;
  return process_block(as_stream(stream), Wblock, N, Lblock, ldl, block_size, scale, zero, maxq,
                       Qblock, q_dtype, codes_block, errors);
}

}  // extern "C"

namespace {

// The column loop.  group_size = 0: one scale / zero per channel for the whole column (the reference).
// group_size > 0: the parameters of rows [r0, r0 + group_size) are taken, when the loop reaches r0, from the
// column minima and maxima of those rows as they then stand (all corrections of the rows above applied), and
// written to row r0 / group_size of scale_g / zero_g [K / group_size, N].
int solve_impl(hipStream_t st, float *W, int64_t K, int64_t N, const float *L, const float *scale, const float *zero,
               float *scale_g, float *zero_g, int group_size, int bits, int maxq, int block_size, void *Q,
               int q_dtype, uint8_t *codes, float *Err, void *cp_ws, size_t cp_ws_bytes) {
  const size_t qsz = dtype_size(q_dtype);
  const int64_t grp = group_rows(block_size);
  for (int64_t gs = 0; gs < K; gs += grp) {
    const int64_t ge = gs + grp < K ? gs + grp : K;
    for (int64_t start = gs; start < ge; start += block_size) {
      const float *sc = scale, *zr = zero;
      if (group_size > 0) {
        const int64_t gi = start / group_size;
        if (start % group_size == 0) {
          // the group's rows lie inside the current update group (group_size divides its height), so they are current
          const int rc = gptq_hip_col_params(st, W + start * N, GPTQ_HIP_F32, group_size, N, N, bits,
                                             scale_g + gi * N, zero_g + gi * N, cp_ws, cp_ws_bytes);
          if (rc) return rc;
        }
        sc = scale_g + gi * N;
        zr = zero_g + gi * N;
      }
      void *Qb = Q ? (void *)((char *)Q + (size_t)start * N * qsz) : nullptr;
      uint8_t *cb = codes ? codes + start * N : nullptr;
      float *Eb = Err + (start - gs) * N;
      int rc = process_block(st, W + start * N, N, L + start * K + start, K, block_size, sc, zr, maxq, Qb,
                             q_dtype, cb, Eb);
      if (rc) return rc;
      const int64_t end = start + block_size;
      if (end < ge) {
        // rows of this group below the block: W[end:ge] -= L[end:ge, start:end] @ Err_block
        rc = trailing_update(st, L + end * K + start, K, Eb, W + end * N, N, ge - end, block_size);
        if (rc) return rc;
      }
    }
    if (ge < K) {
      // everything below the group: W[ge:] -= L[ge:, gs:ge] @ Err_group  (gptq.py:204-205, summed
      // over the blocks of the group)
      const int rc = trailing_update(st, L + ge * K + gs, K, Err, W + ge * N, N, K - ge, ge - gs);
      if (rc) return rc;
    }
  }
  return GPTQ_HIP_OK;
}

}  // namespace

extern "C" {

int gptq_hip_solve(void *stream, float *W, int64_t K, int64_t N, const float *L,
                   const float *scale, const float *zero, int maxq, int block_size, void *Q,
                   int q_dtype, uint8_t *codes, void *ws, size_t ws_bytes) {
  if (!W || !L || !scale || !zero || K <= 0 || N <= 0 || K > 2147483647LL || N > 2147483647LL)
    return GPTQ_HIP_EINVAL;
  if (!block_size_ok(block_size) || K % block_size != 0 || maxq < 1 || maxq > 255)
    return GPTQ_HIP_EINVAL;
  if (q_dtype != GPTQ_HIP_F32 && q_dtype != GPTQ_HIP_F16 && q_dtype != GPTQ_HIP_BF16)
    return GPTQ_HIP_EDTYPE;
  if (!ws || ws_bytes < gptq_hip_solve_workspace_bytes(K, N, block_size)) return GPTQ_HIP_EWORKSPACE;
  return solve_impl(as_stream(stream), W, K, N, L, scale, zero, nullptr, nullptr, 0, 0, maxq, block_size, Q, q_dtype,
                    codes, reinterpret_cast<float *>(ws), nullptr, 0);
}

size_t gptq_hip_solve_grouped_workspace_bytes(int64_t K, int64_t N, int block_size, int group_size) {
  if (K <= 0 || N <= 0 || !block_size_ok(block_size) || group_size <= 0) return 0;
  const size_t a = (gptq_hip_solve_workspace_bytes(K, N, block_size) + 255) & ~(size_t)255;
  return a + gptq_hip_col_params_workspace_bytes(group_size, N);
}

int gptq_hip_solve_grouped(void *stream, float *W, int64_t K, int64_t N, const float *L, int group_size, int bits,
                           int block_size, void *Q, int q_dtype, uint8_t *codes, float *scale_g, float *zero_g,
                           void *ws, size_t ws_bytes) {
  if (!W || !L || !scale_g || !zero_g || K <= 0 || N <= 0 || K > 2147483647LL || N > 2147483647LL)
    return GPTQ_HIP_EINVAL;
  if (!block_size_ok(block_size) || K % block_size != 0 || bits < 1 || bits > 8) return GPTQ_HIP_EINVAL;
  // a group is a whole number of blocks, lies inside one update group of the loop, and groups tile K
  if (group_size <= 0 || group_size % block_size != 0 || group_rows(block_size) % group_size != 0 ||
      K % group_size != 0)
    return GPTQ_HIP_EINVAL;
  if (q_dtype != GPTQ_HIP_F32 && q_dtype != GPTQ_HIP_F16 && q_dtype != GPTQ_HIP_BF16)
    return GPTQ_HIP_EDTYPE;
  if (!ws || ws_bytes < gptq_hip_solve_grouped_workspace_bytes(K, N, block_size, group_size)) return GPTQ_HIP_EWORKSPACE;
  const size_t a = (gptq_hip_solve_workspace_bytes(K, N, block_size) + 255) & ~(size_t)255;
  return solve_impl(as_stream(stream), W, K, N, L, nullptr, nullptr, scale_g, zero_g, group_size, bits, (1 << bits) - 1,
                    block_size, Q, q_dtype, codes, reinterpret_cast<float *>(ws), reinterpret_cast<char *>(ws) + a,
                    ws_bytes - a);
}

}  // extern "C"
