// XLA FFI handlers that put the C ABI of include/ragged_dot_hip.h behind jax.ffi.ffi_call: the binding a maintainer of
// the reference adds where gpu_ragged_dot.py calls pl.pallas_call (:217-226 gmm, :331-340 tgmm).
//
// Built only where jaxlib's headers exist:
//   make -C gpu_ragged_dot_amd/csrc xla_ffi XLA_FFI_INCLUDE="$(python -c 'import jax.ffi; print(jax.ffi.include_dir())')"
// It has never been compiled or run in an image without JAX; gpu_ragged_dot_amd/jax_adapter.py is its Python side.
//
// Calling convention of both targets
//   operands : x, second matrix (A for gmm, dy for tgmm), group_sizes (int32[g])
//   results  : the product; a uint8 workspace (XLA allocates it as a second result that the Python side drops)
//   attrs    : the rd_plan fields (variant, group_m, group_n, decode_nb, split_k), chunk_m (validated only), trans_rhs
//              (gmm only), compute_bf16 (float32 arrays rounded to bfloat16 for the matrix cores)
// The element type comes from the buffers themselves.  XLA owns every buffer and passes its compute stream; the
// handlers allocate nothing and never synchronise.
#include <cstdint>

#include "../../include/ragged_dot_hip.h"
#include "hip/hip_runtime.h"
#include "xla/ffi/api/ffi.h"

namespace ffi = xla::ffi;

namespace {

// RD_DTYPE_* of a call from the element type of its first operand, or -1.
int dtype_code(ffi::DataType t, bool compute_bf16) {
  if (t == ffi::DataType::BF16) return RD_DTYPE_BF16;
  if (t == ffi::DataType::F32) return compute_bf16 ? RD_DTYPE_F32_BF16 : RD_DTYPE_F32;
  if (t == ffi::DataType::F8E4M3FN) return RD_DTYPE_F8E4M3_BF16;  // the result buffer is then bfloat16
  if (t == ffi::DataType::F16) return RD_DTYPE_F16;
  return -1;
}

// Element type of the product for operands of type t: their own, except that float8 operands give bfloat16 (the
// Python side declares the result that way, jax_adapter._out_dtype).
ffi::DataType result_type(ffi::DataType t) {
  if (t == ffi::DataType::F8E4M3FN) return ffi::DataType::BF16;
  return t;
}

ffi::Error status(int rc) {
  if (rc == RD_OK) return ffi::Error::Success();
  return ffi::Error(rc == RD_ERR_HIP ? ffi::ErrorCode::kInternal : ffi::ErrorCode::kInvalidArgument, rd_last_error());
}

ffi::Error GmmImpl(hipStream_t stream, ffi::AnyBuffer x_buf, ffi::AnyBuffer A_buf, ffi::Buffer<ffi::S32> gs_buf,
                   ffi::Result<ffi::AnyBuffer> y_buf, ffi::Result<ffi::AnyBuffer> ws_buf, bool trans_rhs_attr,
                   bool compute_bf16, int32_t variant, int32_t group_m, int32_t group_n, int32_t decode_nb,
                   int32_t split_k, int32_t chunk_m) {
  if (x_buf.dimensions().size() != 2 || A_buf.dimensions().size() != 3 || gs_buf.dimensions().size() != 1)
    return ffi::Error(ffi::ErrorCode::kInvalidArgument, "rd_gmm: x is [m,k], A is [g,k,n] or [g,n,k], group_sizes is [g]");
  if (A_buf.element_type() != x_buf.element_type() || y_buf->element_type() != result_type(x_buf.element_type()))
    return ffi::Error(ffi::ErrorCode::kInvalidArgument,
                      "rd_gmm: x and A must have one element type and y that of the product (bfloat16 for float8 operands)");
  if (chunk_m < 1) return ffi::Error(ffi::ErrorCode::kInvalidArgument, "rd_gmm: chunk_m must be positive");
  const int trans_rhs = trans_rhs_attr ? 1 : 0;
  const int m = (int)x_buf.dimensions()[0], k = (int)x_buf.dimensions()[1], g = (int)A_buf.dimensions()[0];
  const int n = (int)(trans_rhs ? A_buf.dimensions()[1] : A_buf.dimensions()[2]);  // gpu_ragged_dot.py:190
  if ((int)(trans_rhs ? A_buf.dimensions()[2] : A_buf.dimensions()[1]) != k || (int)gs_buf.dimensions()[0] != g)
    return ffi::Error(ffi::ErrorCode::kInvalidArgument, "rd_gmm: contraction or group count mismatch");
  const int dtype = dtype_code(x_buf.element_type(), compute_bf16);
  if (dtype < 0) return ffi::Error(ffi::ErrorCode::kInvalidArgument, "rd_gmm: operands are bfloat16, float32 or float8_e4m3fn");
  const rd_plan plan_value = {variant, group_m, group_n, decode_nb, split_k};
  const rd_plan* plan = &plan_value;
  const void* x = x_buf.untyped_data();
  const void* A = A_buf.untyped_data();
  const int32_t* group_sizes = gs_buf.typed_data();
  void* y = y_buf->untyped_data();
  void* workspace = ws_buf->untyped_data();
  const size_t workspace_bytes = ws_buf->size_bytes();
  return status(rd_gmm(stream, x, A, group_sizes, y, m, k, n, g, trans_rhs, dtype, plan, workspace, workspace_bytes));
}

ffi::Error TgmmImpl(hipStream_t stream, ffi::AnyBuffer x_buf, ffi::AnyBuffer dy_buf, ffi::Buffer<ffi::S32> gs_buf,
                    ffi::Result<ffi::AnyBuffer> dA_buf, ffi::Result<ffi::AnyBuffer> ws_buf, bool compute_bf16,
                    int32_t variant, int32_t group_m, int32_t group_n, int32_t decode_nb, int32_t split_k,
                    int32_t chunk_m) {
  if (x_buf.dimensions().size() != 2 || dy_buf.dimensions().size() != 2 || gs_buf.dimensions().size() != 1 ||
      x_buf.dimensions()[0] != dy_buf.dimensions()[0])  // gpu_ragged_dot.py:304
    return ffi::Error(ffi::ErrorCode::kInvalidArgument, "rd_tgmm: x is [m,k], y is [m,n], group_sizes is [g]");
  if (dy_buf.element_type() != x_buf.element_type() || dA_buf->element_type() != result_type(x_buf.element_type()))
    return ffi::Error(ffi::ErrorCode::kInvalidArgument,
                      "rd_tgmm: x and y must have one element type and the result that of the product (bfloat16 for float8 operands)");
  (void)chunk_m;  // accepted and unused, as gpu_ragged_dot.py:303
  const int m = (int)x_buf.dimensions()[0], k = (int)x_buf.dimensions()[1], n = (int)dy_buf.dimensions()[1];
  const int g = (int)gs_buf.dimensions()[0];
  const int dtype = dtype_code(x_buf.element_type(), compute_bf16);
  if (dtype < 0) return ffi::Error(ffi::ErrorCode::kInvalidArgument, "rd_tgmm: operands are bfloat16, float32 or float8_e4m3fn");
  const rd_plan plan_value = {variant, group_m, group_n, decode_nb, split_k};
  const rd_plan* plan = &plan_value;
  const void* x = x_buf.untyped_data();
  const void* dy = dy_buf.untyped_data();
  const int32_t* group_sizes = gs_buf.typed_data();
  void* dA = dA_buf->untyped_data();
  void* workspace = ws_buf->untyped_data();
  const size_t workspace_bytes = ws_buf->size_bytes();
  return status(rd_tgmm(stream, x, dy, group_sizes, dA, m, k, n, g, dtype, plan, workspace, workspace_bytes));
}

}  // namespace

XLA_FFI_DEFINE_HANDLER_SYMBOL(RdGmm, GmmImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()          // x
                                  .Arg<ffi::AnyBuffer>()          // A
                                  .Arg<ffi::Buffer<ffi::S32>>()   // group_sizes
                                  .Ret<ffi::AnyBuffer>()          // y
                                  .Ret<ffi::AnyBuffer>()          // workspace
                                  .Attr<bool>("trans_rhs")
                                  .Attr<bool>("compute_bf16")
                                  .Attr<int32_t>("variant")
                                  .Attr<int32_t>("group_m")
                                  .Attr<int32_t>("group_n")
                                  .Attr<int32_t>("decode_nb")
                                  .Attr<int32_t>("split_k")
                                  .Attr<int32_t>("chunk_m"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(RdTgmm, TgmmImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()          // x
                                  .Arg<ffi::AnyBuffer>()          // dy
                                  .Arg<ffi::Buffer<ffi::S32>>()   // group_sizes
                                  .Ret<ffi::AnyBuffer>()          // dA
                                  .Ret<ffi::AnyBuffer>()          // workspace
                                  .Attr<bool>("compute_bf16")
                                  .Attr<int32_t>("variant")
                                  .Attr<int32_t>("group_m")
                                  .Attr<int32_t>("group_n")
                                  .Attr<int32_t>("decode_nb")
                                  .Attr<int32_t>("split_k")
                                  .Attr<int32_t>("chunk_m"));
