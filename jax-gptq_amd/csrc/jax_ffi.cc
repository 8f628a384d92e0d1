// XLA FFI handlers over the C ABI of libgptq_hip.so: one typed custom call per entry point of
// include/gptq_hip.h, for a JAX front-end that keeps the reference's Python API
// (jax_gptq/gptq.py, op.py) and replaces its jt.triton_call (op.py:46-63) and its jitted XLA graphs
// (gptq.py:57,130,155,170,177) by these calls.
//
// Compiled only where the XLA FFI headers exist (build.py: jax.ffi.include_dir()); this translation unit
// contains no kernels, it unpacks buffers and attributes and forwards to the C ABI.  Conventions:
//   * every handler runs on the stream XLA hands it (ffi::PlatformStream<hipStream_t>) and only enqueues;
//   * buffers the C ABI updates in place (H, W, the matmul workspace) are operands that the Python side
//     aliases to a result (input_output_aliases), so XLA sees a functional update;
//   * scratch memory without content requirements comes from ffi::ScratchAllocator; the matmul workspace,
//     whose arrival counters must be zero between calls, is an operand the front-end keeps (zero-filled
//     once) and threads through the calls;
//   * a non-zero status of the C ABI becomes an ffi::Error with the library's message.
//
// Registration (Python): jax.ffi.register_ffi_target(name, jax.ffi.pycapsule(lib.<name>), platform="ROCM")
// for every XLA_FFI_DEFINE_HANDLER_SYMBOL below (jax_gptq_amd/jax_frontend.py does this).
#include <cstdint>
#include <optional>
#include <string>
#include <vector>

#include <hip/hip_runtime.h>

#include "xla/ffi/api/ffi.h"

#include "../../include/gptq_hip.h"

namespace ffi = xla::ffi;

namespace {

// element type of a float buffer in the C ABI's numbering, or -1
int float_type(ffi::DataType t) {
  switch (t) {
    case ffi::DataType::F32: return GPTQ_HIP_F32;
    case ffi::DataType::F16: return GPTQ_HIP_F16;
    case ffi::DataType::BF16: return GPTQ_HIP_BF16;
    case ffi::DataType::F64: return GPTQ_HIP_F64;
    default: return -1;
  }
}

ffi::Error status(int code, const char *what) {
  if (code == GPTQ_HIP_OK) return ffi::Error::Success();
  std::string msg = std::string(what) + ": " + gptq_hip_error_string(code);
  return ffi::Error(code == GPTQ_HIP_EINVAL || code == GPTQ_HIP_EDTYPE ? ffi::ErrorCode::kInvalidArgument
                                                                       : ffi::ErrorCode::kInternal,
                    msg);
}

ffi::Error bad(const char *msg) { return ffi::Error(ffi::ErrorCode::kInvalidArgument, msg); }

// scratch of `bytes` bytes (nullptr for 0); false if XLA cannot provide it
bool scratch(ffi::ScratchAllocator &alloc, size_t bytes, void **out) {
  *out = nullptr;
  if (bytes == 0) return true;
  std::optional<void *> p = alloc.Allocate(bytes, 256);
  if (!p.has_value()) return false;
  *out = *p;
  return true;
}

// ---- get_col_quantize_params (gptq.py:105-118): W [K, N] -> scale [N], zero [N]
ffi::Error ColParams(hipStream_t stream, ffi::ScratchAllocator alloc, ffi::AnyBuffer W,
                     ffi::Result<ffi::Buffer<ffi::DataType::F32>> scale,
                     ffi::Result<ffi::Buffer<ffi::DataType::F32>> zero, int64_t bits) {
  const auto d = W.dimensions();
  if (d.size() != 2 || float_type(W.element_type()) < 0) return bad("col_params: W must be a 2-D float matrix");
  void *ws = nullptr;
  const size_t need = gptq_hip_col_params_workspace_bytes(d[0], d[1]);
  if (!scratch(alloc, need, &ws)) return ffi::Error(ffi::ErrorCode::kResourceExhausted, "col_params: scratch");
  return status(gptq_hip_col_params(stream, W.untyped_data(), float_type(W.element_type()), d[0], d[1], d[1],
                                    (int)bits, scale->typed_data(), zero->typed_data(), ws, need),
                "col_params");
}

// ---- _accumulate_H_step / accumulate_H (gptq.py:57-103): H += sum_b X_b^T X_b over the remaining
// operands (one batch per call reproduces the reference's one jit call per batch, gptq.py:97-98; all
// batches of a layer in one call is the fast path).  Operand 0 is H, aliased to the result.
ffi::Error HessianAccumulate(hipStream_t stream, ffi::ScratchAllocator alloc, ffi::AnyBuffer H,
                             ffi::RemainingArgs batches, ffi::Result<ffi::AnyBuffer> H_out) {
  const auto hd = H.dimensions();
  const int hdt = float_type(H.element_type());
  if (hd.size() != 2 || hd[0] != hd[1] || (hdt != GPTQ_HIP_F32 && hdt != GPTQ_HIP_F64))
    return bad("hessian_accumulate: H must be a square fp32 or fp64 matrix");
  if (H_out->untyped_data() != H.untyped_data()) return bad("hessian_accumulate: H must be aliased to the result");
  const int64_t K = hd[0];
  std::vector<const void *> ptrs;
  std::vector<int64_t> rows;
  int xdt = -1;
  for (size_t i = 0; i < batches.size(); ++i) {
    auto b = batches.get<ffi::AnyBuffer>(i);
    if (!b.has_value()) return bad("hessian_accumulate: a batch is not a buffer");
    const auto bd = b->dimensions();
    if (bd.empty() || bd.back() != K) return bad("hessian_accumulate: a batch's last dimension is not K");
    const int t = float_type(b->element_type());
    if (t < 0 || (xdt >= 0 && t != xdt)) return bad("hessian_accumulate: batches must share one float type");
    xdt = t;
    ptrs.push_back(b->untyped_data());
    rows.push_back(K ? (int64_t)b->element_count() / K : 0);
  }
  if (ptrs.empty()) return ffi::Error::Success();
  void *ws = nullptr;
  const size_t need = gptq_hip_hessian_accumulate_workspace_bytes(K, hdt);
  if (!scratch(alloc, need, &ws)) return ffi::Error(ffi::ErrorCode::kResourceExhausted, "hessian_accumulate: scratch");
  return status(gptq_hip_hessian_accumulate(stream, ptrs.data(), rows.data(), (int)ptrs.size(), xdt, K,
                                            H.untyped_data(), hdt, ws, need),
                "hessian_accumulate");
}

// ---- the closing lines of accumulate_H (gptq.py:100-101): H / n, mirrored into the lower triangle
ffi::Error HessianFinalize(hipStream_t stream, ffi::AnyBuffer H, ffi::Result<ffi::AnyBuffer> H_out,
                           double n_samples) {
  const auto hd = H.dimensions();
  if (hd.size() != 2 || hd[0] != hd[1]) return bad("hessian_finalize: H must be square");
  if (H_out->untyped_data() != H.untyped_data()) return bad("hessian_finalize: H must be aliased to the result");
  return status(gptq_hip_hessian_finalize(stream, H.untyped_data(), float_type(H.element_type()), hd[0], n_samples),
                "hessian_finalize");
}

// ---- _damp_and_invert + _cholesky_inv (gptq.py:155-168, 44-48).  Operands H [K, K] (fp32 / fp64) and
// W [K, N] fp32, both aliased to results 0 and 1; results 2: L (H's type), 3: L32 (fp32 copy of an fp64 L,
// gptq.py:197; a zero-sized buffer when H is fp32), 4: status int32[2].
ffi::Error DampInvert(hipStream_t stream, ffi::ScratchAllocator alloc, ffi::AnyBuffer H, ffi::AnyBuffer W,
                      ffi::Result<ffi::AnyBuffer> H_out, ffi::Result<ffi::AnyBuffer> W_out,
                      ffi::Result<ffi::AnyBuffer> L, ffi::Result<ffi::AnyBuffer> L32,
                      ffi::Result<ffi::Buffer<ffi::DataType::S32>> st, double damping, bool fix_dead) {
  const auto hd = H.dimensions();
  const auto wd = W.dimensions();
  const int hdt = float_type(H.element_type());
  if (hd.size() != 2 || hd[0] != hd[1]) return bad("damp_invert: H must be square");
  const int64_t K = hd[0];
  int64_t N = 0;
  float *Wp = nullptr;
  if (W.element_count() > 0) {
    if (wd.size() != 2 || wd[0] != K || W.element_type() != ffi::DataType::F32)
      return bad("damp_invert: W must be [K, N] fp32");
    N = wd[1];
    Wp = reinterpret_cast<float *>(W.untyped_data());
    if (W_out->untyped_data() != W.untyped_data()) return bad("damp_invert: W must be aliased to result 1");
  }
  if (H_out->untyped_data() != H.untyped_data()) return bad("damp_invert: H must be aliased to result 0");
  void *ws = nullptr;
  const size_t need = gptq_hip_damp_invert_workspace_bytes(K, hdt);
  if (!scratch(alloc, need, &ws)) return ffi::Error(ffi::ErrorCode::kResourceExhausted, "damp_invert: scratch");
  float *l32 = L32->element_count() > 0 ? reinterpret_cast<float *>(L32->untyped_data()) : nullptr;
  return status(gptq_hip_damp_invert(stream, H.untyped_data(), hdt, Wp, K, N, N, damping, fix_dead ? 1 : 0,
                                     L->untyped_data(), l32, st->typed_data(), ws, need),
                "damp_invert");
}

// ---- the dead-feature rows of _damp_and_invert alone (gptq.py:157-159); W aliased to the result
ffi::Error ZeroDeadRows(hipStream_t stream, ffi::AnyBuffer H, ffi::AnyBuffer W, ffi::Result<ffi::AnyBuffer> W_out) {
  const auto wd = W.dimensions();
  if (wd.size() != 2 || W.element_type() != ffi::DataType::F32) return bad("zero_dead_rows: W must be [K, N] fp32");
  if (W_out->untyped_data() != W.untyped_data()) return bad("zero_dead_rows: W must be aliased to the result");
  return status(gptq_hip_zero_dead_rows(stream, H.untyped_data(), float_type(H.element_type()), wd[0],
                                        reinterpret_cast<float *>(W.untyped_data()), wd[1], wd[1]),
                "zero_dead_rows");
}

// ---- the column loop of gptq() (gptq.py:199-208, 130-153).  Operand W [K, N] fp32 is consumed (aliased to
// result 2); results 0: Q [K, N] in the caller's float type, 1: codes [K, N] uint8.
ffi::Error Solve(hipStream_t stream, ffi::ScratchAllocator alloc, ffi::AnyBuffer W,
                 ffi::Buffer<ffi::DataType::F32> L, ffi::Buffer<ffi::DataType::F32> scale,
                 ffi::Buffer<ffi::DataType::F32> zero, ffi::Result<ffi::AnyBuffer> Q,
                 ffi::Result<ffi::Buffer<ffi::DataType::U8>> codes, ffi::Result<ffi::AnyBuffer> W_out, int64_t maxq,
                 int64_t block_size) {
  const auto wd = W.dimensions();
  if (wd.size() != 2 || W.element_type() != ffi::DataType::F32) return bad("solve: W must be [K, N] fp32");
  if (W_out->untyped_data() != W.untyped_data()) return bad("solve: W must be aliased to result 2");
  const int qdt = float_type(Q->element_type());
  if (qdt < 0 || qdt == GPTQ_HIP_F64) return bad("solve: Q must be fp32, fp16 or bf16");
  void *ws = nullptr;
  const size_t need = gptq_hip_solve_workspace_bytes(wd[0], wd[1], (int)block_size);
  if (!scratch(alloc, need, &ws)) return ffi::Error(ffi::ErrorCode::kResourceExhausted, "solve: scratch");
  return status(gptq_hip_solve(stream, reinterpret_cast<float *>(W.untyped_data()), wd[0], wd[1], L.typed_data(),
                               scale.typed_data(), zero.typed_data(), (int)maxq, (int)block_size, Q->untyped_data(),
                               qdt, codes->typed_data(), ws, need),
                "solve");
}

// ---- _process_block (gptq.py:130-153): block `start` of W [K, N] against L [K, K]
ffi::Error ProcessBlock(hipStream_t stream, ffi::Buffer<ffi::DataType::F32> W, ffi::Buffer<ffi::DataType::F32> L,
                        ffi::Buffer<ffi::DataType::F32> scale, ffi::Buffer<ffi::DataType::F32> zero,
                        ffi::Result<ffi::Buffer<ffi::DataType::F32>> Qblock,
                        ffi::Result<ffi::Buffer<ffi::DataType::F32>> errors, int64_t start, int64_t block_size,
                        int64_t maxq) {
  const auto wd = W.dimensions();
  const auto ld = L.dimensions();
  if (wd.size() != 2 || ld.size() != 2 || ld[0] != wd[0] || ld[1] != wd[0] || start < 0 ||
      start + block_size > wd[0])
    return bad("process_block: shapes");
  return status(gptq_hip_process_block(stream, W.typed_data() + start * wd[1], wd[1],
                                       L.typed_data() + start * ld[1] + start, ld[1], (int)block_size,
                                       scale.typed_data(), zero.typed_data(), (int)maxq, Qblock->typed_data(),
                                       GPTQ_HIP_F32, nullptr, errors->typed_data()),
                "process_block");
}

// ---- the gathers of _permute / _unpermute (gptq.py:170-180)
ffi::Error GatherRows(hipStream_t stream, ffi::AnyBuffer in, ffi::Buffer<ffi::DataType::S64> perm,
                      ffi::Result<ffi::AnyBuffer> out) {
  const auto d = in.dimensions();
  if (d.size() != 2) return bad("gather_rows: a 2-D matrix");
  const int eb = d[0] * d[1] ? (int)(in.size_bytes() / (size_t)(d[0] * d[1])) : 4;
  return status(gptq_hip_gather_rows(stream, in.untyped_data(), out->untyped_data(), eb, d[0], d[1], perm.typed_data()),
                "gather_rows");
}

ffi::Error GatherSym(hipStream_t stream, ffi::AnyBuffer in, ffi::Buffer<ffi::DataType::S64> perm,
                     ffi::Result<ffi::AnyBuffer> out) {
  const auto d = in.dimensions();
  if (d.size() != 2 || d[0] != d[1]) return bad("gather_sym: a square matrix");
  const int eb = d[0] ? (int)(in.size_bytes() / (size_t)(d[0] * d[0])) : 4;
  return status(gptq_hip_gather_sym(stream, in.untyped_data(), out->untyped_data(), eb, d[0], perm.typed_data()),
                "gather_sym");
}

// ---- _pack / pack_along_axis and _unpack / unpack_along_axis (gptq.py:237-292) on [outer, axis, inner] views
ffi::Error PackInt4(hipStream_t stream, ffi::AnyBuffer codes, ffi::Result<ffi::Buffer<ffi::DataType::U8>> packed,
                    int64_t outer, int64_t axis_len, int64_t inner) {
  const int64_t n = outer * axis_len * inner;
  const int cb = n ? (int)(codes.size_bytes() / (size_t)n) : 1;
  return status(gptq_hip_pack_int4(stream, codes.untyped_data(), cb, outer, axis_len, inner, packed->typed_data()),
                "pack_int4");
}

ffi::Error UnpackInt4(hipStream_t stream, ffi::Buffer<ffi::DataType::U8> packed,
                      ffi::Result<ffi::Buffer<ffi::DataType::U8>> codes, int64_t outer, int64_t packed_axis_len,
                      int64_t inner) {
  return status(gptq_hip_unpack_int4(stream, packed.typed_data(), outer, packed_axis_len, inner, codes->typed_data()),
                "unpack_int4");
}

// ---- pack_matrix (gptq.py:214-228) and unpack_matrix (gptq.py:230-235); bits = 4 or 8
ffi::Error QuantizePack(hipStream_t stream, ffi::AnyBuffer Q, ffi::Buffer<ffi::DataType::F32> scale,
                        ffi::Buffer<ffi::DataType::F32> zero, ffi::Result<ffi::Buffer<ffi::DataType::U8>> packed,
                        int64_t outer, int64_t axis_len, int64_t inner, int64_t bits) {
  return status(gptq_hip_quantize_pack_bits(stream, Q.untyped_data(), float_type(Q.element_type()), outer, axis_len,
                                            inner, scale.typed_data(), zero.typed_data(), (int)bits,
                                            packed->typed_data()),
                "quantize_pack");
}

ffi::Error Dequant(hipStream_t stream, ffi::Buffer<ffi::DataType::U8> packed, ffi::AnyBuffer zero,
                   ffi::AnyBuffer scale, ffi::Result<ffi::AnyBuffer> out, int64_t outer, int64_t packed_axis_len,
                   int64_t inner, int64_t bits) {
  if (zero.element_type() != scale.element_type() || zero.element_type() != out->element_type())
    return bad("dequant: zero, scale and the result share one float type (gptq.py:20-22)");
  return status(gptq_hip_dequant_bits(stream, packed.typed_data(), outer, packed_axis_len, inner, zero.untyped_data(),
                                      scale.untyped_data(), float_type(zero.element_type()), (int)bits,
                                      out->untyped_data()),
                "dequant");
}

// ---- the custom call of _quantized_matmul (op.py:46-63) and both Triton kernels (kernel.py:17-253).
// Operands x [M, Kx], packed [R, C], zero [C], scale [C], ws (the workspace, aliased to result 1, zero-filled
// by the front-end when it is created); result 0: out [M, out_n] in x's type.
ffi::Error Qmatmul(hipStream_t stream, ffi::AnyBuffer x, ffi::Buffer<ffi::DataType::U8> packed, ffi::AnyBuffer zero,
                   ffi::AnyBuffer scale, ffi::Buffer<ffi::DataType::U8> ws, ffi::Result<ffi::AnyBuffer> out,
                   ffi::Result<ffi::Buffer<ffi::DataType::U8>> ws_out, bool transpose_b, int64_t bits) {
  const auto xd = x.dimensions();
  const auto pd = packed.dimensions();
  if (xd.size() != 2 || pd.size() != 2) return bad("qmatmul: x [M, K] and a 2-D packed matrix (op.py:27-41)");
  if (zero.element_type() != scale.element_type()) return bad("qmatmul: zero and scale share one float type");
  if (ws_out->untyped_data() != ws.untyped_data()) return bad("qmatmul: the workspace must be aliased to result 1");
  const int64_t M = xd[0], R = pd[0], C = pd[1];
  const int64_t Kw = bits == 8 ? R : 2 * R;
  if (xd[1] != (transpose_b ? C : Kw)) return bad("qmatmul: inner dimension mismatch (op.py:41)");
  const int xdt = float_type(x.element_type());
  if (ws.size_bytes() < gptq_hip_qmatmul_bits_workspace_bytes(M, R, C, transpose_b ? 1 : 0, xdt, (int)bits))
    return bad("qmatmul: workspace smaller than gptq_hip_qmatmul_bits_workspace_bytes");
  return status(gptq_hip_qmatmul_bits(stream, x.untyped_data(), xdt, M, packed.typed_data(), R, C, zero.untyped_data(),
                                      scale.untyped_data(), float_type(zero.element_type()), (int)bits,
                                      transpose_b ? 1 : 0, out->untyped_data(), ws.typed_data(), ws.size_bytes()),
                "qmatmul");
}

}  // namespace

#define GPTQ_STREAM .Ctx<ffi::PlatformStream<hipStream_t>>()

XLA_FFI_DEFINE_HANDLER_SYMBOL(gptq_ffi_col_params, ColParams,
                              ffi::Ffi::Bind() GPTQ_STREAM.Ctx<ffi::ScratchAllocator>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::Buffer<ffi::DataType::F32>>()
                                  .Ret<ffi::Buffer<ffi::DataType::F32>>()
                                  .Attr<int64_t>("bits"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(gptq_ffi_hessian_accumulate, HessianAccumulate,
                              ffi::Ffi::Bind() GPTQ_STREAM.Ctx<ffi::ScratchAllocator>()
                                  .Arg<ffi::AnyBuffer>()
                                  .RemainingArgs()
                                  .Ret<ffi::AnyBuffer>());

XLA_FFI_DEFINE_HANDLER_SYMBOL(gptq_ffi_hessian_finalize, HessianFinalize,
                              ffi::Ffi::Bind() GPTQ_STREAM.Arg<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>().Attr<double>(
                                  "n_samples"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(gptq_ffi_damp_invert, DampInvert,
                              ffi::Ffi::Bind() GPTQ_STREAM.Ctx<ffi::ScratchAllocator>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::Buffer<ffi::DataType::S32>>()
                                  .Attr<double>("damping")
                                  .Attr<bool>("fix_dead"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(gptq_ffi_zero_dead_rows, ZeroDeadRows,
                              ffi::Ffi::Bind() GPTQ_STREAM.Arg<ffi::AnyBuffer>().Arg<ffi::AnyBuffer>().Ret<ffi::AnyBuffer>());

XLA_FFI_DEFINE_HANDLER_SYMBOL(gptq_ffi_solve, Solve,
                              ffi::Ffi::Bind() GPTQ_STREAM.Ctx<ffi::ScratchAllocator>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::DataType::F32>>()
                                  .Arg<ffi::Buffer<ffi::DataType::F32>>()
                                  .Arg<ffi::Buffer<ffi::DataType::F32>>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::Buffer<ffi::DataType::U8>>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Attr<int64_t>("maxq")
                                  .Attr<int64_t>("block_size"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(gptq_ffi_process_block, ProcessBlock,
                              ffi::Ffi::Bind() GPTQ_STREAM.Arg<ffi::Buffer<ffi::DataType::F32>>()
                                  .Arg<ffi::Buffer<ffi::DataType::F32>>()
                                  .Arg<ffi::Buffer<ffi::DataType::F32>>()
                                  .Arg<ffi::Buffer<ffi::DataType::F32>>()
                                  .Ret<ffi::Buffer<ffi::DataType::F32>>()
                                  .Ret<ffi::Buffer<ffi::DataType::F32>>()
                                  .Attr<int64_t>("start")
                                  .Attr<int64_t>("block_size")
                                  .Attr<int64_t>("maxq"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(gptq_ffi_gather_rows, GatherRows,
                              ffi::Ffi::Bind() GPTQ_STREAM.Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::DataType::S64>>()
                                  .Ret<ffi::AnyBuffer>());

XLA_FFI_DEFINE_HANDLER_SYMBOL(gptq_ffi_gather_sym, GatherSym,
                              ffi::Ffi::Bind() GPTQ_STREAM.Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::DataType::S64>>()
                                  .Ret<ffi::AnyBuffer>());

XLA_FFI_DEFINE_HANDLER_SYMBOL(gptq_ffi_pack_int4, PackInt4,
                              ffi::Ffi::Bind() GPTQ_STREAM.Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::Buffer<ffi::DataType::U8>>()
                                  .Attr<int64_t>("outer")
                                  .Attr<int64_t>("axis_len")
                                  .Attr<int64_t>("inner"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(gptq_ffi_unpack_int4, UnpackInt4,
                              ffi::Ffi::Bind() GPTQ_STREAM.Arg<ffi::Buffer<ffi::DataType::U8>>()
                                  .Ret<ffi::Buffer<ffi::DataType::U8>>()
                                  .Attr<int64_t>("outer")
                                  .Attr<int64_t>("packed_axis_len")
                                  .Attr<int64_t>("inner"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(gptq_ffi_quantize_pack, QuantizePack,
                              ffi::Ffi::Bind() GPTQ_STREAM.Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::DataType::F32>>()
                                  .Arg<ffi::Buffer<ffi::DataType::F32>>()
                                  .Ret<ffi::Buffer<ffi::DataType::U8>>()
                                  .Attr<int64_t>("outer")
                                  .Attr<int64_t>("axis_len")
                                  .Attr<int64_t>("inner")
                                  .Attr<int64_t>("bits"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(gptq_ffi_dequant, Dequant,
                              ffi::Ffi::Bind() GPTQ_STREAM.Arg<ffi::Buffer<ffi::DataType::U8>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Attr<int64_t>("outer")
                                  .Attr<int64_t>("packed_axis_len")
                                  .Attr<int64_t>("inner")
                                  .Attr<int64_t>("bits"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(gptq_ffi_qmatmul, Qmatmul,
                              ffi::Ffi::Bind() GPTQ_STREAM.Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::DataType::U8>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::DataType::U8>>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::Buffer<ffi::DataType::U8>>()
                                  .Attr<bool>("transpose_b")
                                  .Attr<int64_t>("bits"));
