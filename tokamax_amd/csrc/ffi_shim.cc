// XLA FFI handlers over the C ABI of libtkx_ragged_dot.so: what `jax.ffi.ffi_call` reaches when
// `implementation="hip"` runs under JAX. Each handler only unpacks buffers and attributes and forwards to the entry
// point of the same name; XLA owns every buffer, the workspace included (it is declared as an extra result).
//
// The header xla/ffi/api/ffi.h ships inside jaxlib. Where it is not on the include path this file compiles to a stub
// that exports only tkx_ffi_shim_available() == 0, so that the build never depends on a JAX install:
//   make -C tokamax_amd/csrc ffi        (builds ../lib/libtkx_ragged_dot_ffi.so when the header is found)
//
// Handler symbols and the Python registration that goes with them:
//   TkxRaggedDotFwd        jax.ffi.register_ffi_target("tkx_ragged_dot_fwd", jax.ffi.pycapsule(lib.TkxRaggedDotFwd), platform="ROCM")
//   TkxRaggedDotFwdFused   ... "tkx_ragged_dot_fwd_fused"
//   TkxRaggedDotFwdFp8Out  ... "tkx_ragged_dot_fwd_fp8_out" (two results: fp8 values and their f32 scales)
//   TkxRaggedDotDrhs       ... "tkx_ragged_dot_drhs"
// They replace the kernel calls of tokamax/_src/ops/ragged_dot/pallas_mosaic_gpu.py:231-238 (forward, dlhs),
// pallas_mosaic_gpu_kernel_sm100_fp8_quant.py:797-824 (quantised output) and pallas_mosaic_gpu_kernel_sm90.py:246-285
// (drhs). Every field of TkxConfig is an attribute of the same name (TKX_CONFIG_ATTRS below).
//
// A workspace result is uninitialised memory. With `split_k` > 1 or `persistent` = 1 its counter block has to be zero
// when the kernel starts, so the handler clears it first (a fill kernel on the same stream, safe under the command
// buffers XLA captures); the workspace result must then be tkx_ragged_dot_decode_workspace_bytes /
// tkx_ragged_dot_decode_persistent_workspace_bytes long instead of tkx_ragged_dot_workspace_bytes.
#include "tkx_ragged_dot.h"

#if defined(__has_include)
#if __has_include("xla/ffi/api/ffi.h")
#define TKX_HAVE_XLA_FFI 1
#endif
#endif

#ifdef TKX_HAVE_XLA_FFI
#include <hip/hip_runtime.h>

#include "xla/ffi/api/ffi.h"

namespace ffi = xla::ffi;

namespace {

int32_t dtype_code(ffi::DataType t) {
  switch (t) {
    case ffi::DataType::F32: return TKX_F32;
    case ffi::DataType::BF16: return TKX_BF16;
    case ffi::DataType::F16: return TKX_F16;
    case ffi::DataType::F8E4M3FN: return TKX_F8E4M3FN;
    case ffi::DataType::S8: return TKX_I8;
    case ffi::DataType::U8: return TKX_I4X2;  // two int4 to a byte along k (this library's packed layout)
    default: return -1;
  }
}

// An optional operand travels as a zero-sized buffer when it is absent.
template <typename T>
const T* optional_data(const ffi::AnyBuffer& b) {
  return b.element_count() ? static_cast<const T*>(b.untyped_data()) : nullptr;
}

ffi::Error status_to_error(int32_t st) {
  if (st == TKX_OK) return ffi::Error::Success();
  // TKX_ERR_UNSUPPORTED is what the Python side turns into NotImplementedError (the dispatcher's fall-through).
  const ffi::ErrorCode code = st == TKX_ERR_UNSUPPORTED ? ffi::ErrorCode::kUnimplemented
                              : st == TKX_ERR_INVALID   ? ffi::ErrorCode::kInvalidArgument
                                                        : ffi::ErrorCode::kInternal;
  return ffi::Error(code, tkx_last_error());
}

// The attributes every handler takes, one per field of TkxConfig, in the struct's order.
#define TKX_CONFIG_PARAMS                                                                                          \
  int32_t block_m, int32_t block_n, int32_t block_k, int32_t waves_m, int32_t waves_n, int32_t grid_tile_width, \
      int32_t align_tile, int32_t num_stages, int32_t split_k, int32_t persistent
#define TKX_CONFIG_ATTRS             \
  .Attr<int32_t>("block_m")          \
      .Attr<int32_t>("block_n")      \
      .Attr<int32_t>("block_k")      \
      .Attr<int32_t>("waves_m")      \
      .Attr<int32_t>("waves_n")      \
      .Attr<int32_t>("grid_tile_width") \
      .Attr<int32_t>("align_tile")   \
      .Attr<int32_t>("num_stages")   \
      .Attr<int32_t>("split_k")      \
      .Attr<int32_t>("persistent")
#define TKX_CONFIG_INIT                                                                                            \
  TkxConfig cfg;                                                                                                   \
  cfg.block_m = block_m;                                                                                           \
  cfg.block_n = block_n;                                                                                           \
  cfg.block_k = block_k;                                                                                           \
  cfg.waves_m = waves_m;                                                                                           \
  cfg.waves_n = waves_n;                                                                                           \
  cfg.grid_tile_width = grid_tile_width;                                                                           \
  cfg.align_tile = align_tile;                                                                                     \
  cfg.num_stages = num_stages;                                                                                     \
  cfg.split_k = split_k;                                                                                           \
  cfg.persistent = persistent;

// The counter block of a split / persistent workspace is zero when the kernel starts.
ffi::Error prepare_workspace(const TkxConfig& cfg, void* workspace, hipStream_t stream) {
  if (cfg.split_k > 1 || cfg.persistent != 0) return status_to_error(tkx_ragged_dot_decode_clear_counters(workspace, stream));
  return ffi::Error::Success();
}

ffi::Error FwdImpl(hipStream_t stream, ffi::AnyBuffer lhs, ffi::AnyBuffer rhs, ffi::Buffer<ffi::DataType::S32> group_sizes,
                   ffi::AnyBuffer lhs_scale, ffi::AnyBuffer rhs_scale, ffi::Result<ffi::AnyBuffer> out,
                   ffi::Result<ffi::AnyBuffer> workspace, int32_t mode, int32_t activation, TKX_CONFIG_PARAMS) {
  const auto ld = lhs.dimensions(), rd = rhs.dimensions();
  if (ld.size() != 2 || rd.size() != 3) return ffi::Error(ffi::ErrorCode::kInvalidArgument, "expected lhs [m,k] and rhs [g,k,n]");
  const int32_t rhs_code = dtype_code(rhs.element_type());
  const int64_t m = ld[0], G = rd[0], k = rhs_code == TKX_I4X2 ? 2 * rd[1] : rd[1], n = rd[2];
  TKX_CONFIG_INIT
  if (ffi::Error e = prepare_workspace(cfg, workspace->untyped_data(), stream); e.failure()) return e;
  return status_to_error(tkx_ragged_dot_fwd(
      lhs.untyped_data(), rhs.untyped_data(), group_sizes.typed_data(), optional_data<float>(lhs_scale),
      optional_data<float>(rhs_scale), out->untyped_data(), workspace->untyped_data(), m, k, n, G,
      dtype_code(lhs.element_type()), rhs_code, dtype_code(out->element_type()), mode, activation, &cfg, stream));
}

// rhs_scale is [g, rhs_scale_blocks, n]; rhs_bias [g, n]; group_offset one S32 (zero-sized = absent), in which case
// group_sizes lists every group of the job and rhs holds those from the offset on. With gateup the result is [m, n/2].
ffi::Error FwdFusedImpl(hipStream_t stream, ffi::AnyBuffer lhs, ffi::AnyBuffer rhs, ffi::Buffer<ffi::DataType::S32> group_sizes,
                        ffi::AnyBuffer group_offset, ffi::AnyBuffer lhs_scale, ffi::AnyBuffer rhs_scale,
                        ffi::AnyBuffer rhs_bias, ffi::Result<ffi::AnyBuffer> out, ffi::Result<ffi::AnyBuffer> workspace,
                        int32_t rhs_scale_blocks, int32_t activation, int32_t gateup, TKX_CONFIG_PARAMS) {
  const auto ld = lhs.dimensions(), rd = rhs.dimensions();
  if (ld.size() != 2 || rd.size() != 3) return ffi::Error(ffi::ErrorCode::kInvalidArgument, "expected lhs [m,k] and rhs [g,k,n]");
  const int32_t rhs_code = dtype_code(rhs.element_type());
  const int64_t m = ld[0], G = rd[0], k = rhs_code == TKX_I4X2 ? 2 * rd[1] : rd[1], n = rd[2];
  TKX_CONFIG_INIT
  if (ffi::Error e = prepare_workspace(cfg, workspace->untyped_data(), stream); e.failure()) return e;
  return status_to_error(tkx_ragged_dot_fwd_fused(
      lhs.untyped_data(), rhs.untyped_data(), group_sizes.typed_data(), optional_data<int32_t>(group_offset),
      optional_data<float>(lhs_scale), optional_data<float>(rhs_scale), optional_data<float>(rhs_bias), out->untyped_data(),
      workspace->untyped_data(), m, k, n, G, (int64_t)group_sizes.element_count(), rhs_scale_blocks,
      dtype_code(lhs.element_type()), rhs_code, dtype_code(out->element_type()), activation, gateup, &cfg, stream));
}

// The result quantised in the kernel's epilogue: out fp8 (e4m3fn) [m, n] and out_scale f32 [m, n / 128].
ffi::Error FwdFp8OutImpl(hipStream_t stream, ffi::AnyBuffer lhs, ffi::AnyBuffer rhs, ffi::Buffer<ffi::DataType::S32> group_sizes,
                         ffi::AnyBuffer lhs_scale, ffi::AnyBuffer rhs_scale, ffi::Result<ffi::AnyBuffer> out,
                         ffi::Result<ffi::Buffer<ffi::DataType::F32>> out_scale, ffi::Result<ffi::AnyBuffer> workspace,
                         int32_t activation, TKX_CONFIG_PARAMS) {
  const auto ld = lhs.dimensions(), rd = rhs.dimensions();
  if (ld.size() != 2 || rd.size() != 3) return ffi::Error(ffi::ErrorCode::kInvalidArgument, "expected lhs [m,k] and rhs [g,k,n]");
  if (out->element_type() != ffi::DataType::F8E4M3FN) return ffi::Error(ffi::ErrorCode::kInvalidArgument, "the quantised result is f8e4m3fn");
  TKX_CONFIG_INIT
  return status_to_error(tkx_ragged_dot_fwd_fp8_out(
      lhs.untyped_data(), rhs.untyped_data(), group_sizes.typed_data(), optional_data<float>(lhs_scale),
      optional_data<float>(rhs_scale), out->untyped_data(), out_scale->typed_data(), workspace->untyped_data(), ld[0], rd[1],
      rd[2], rd[0], dtype_code(lhs.element_type()), dtype_code(rhs.element_type()), activation, &cfg, stream));
}

ffi::Error DrhsImpl(hipStream_t stream, ffi::AnyBuffer lhs, ffi::AnyBuffer dout, ffi::Buffer<ffi::DataType::S32> group_sizes,
                    ffi::Result<ffi::AnyBuffer> out, ffi::Result<ffi::AnyBuffer> workspace, TKX_CONFIG_PARAMS) {
  const auto ld = lhs.dimensions(), dd = dout.dimensions();
  if (ld.size() != 2 || dd.size() != 2 || ld[0] != dd[0])
    return ffi::Error(ffi::ErrorCode::kInvalidArgument, "expected lhs [m,k] and dout [m,n]");
  TKX_CONFIG_INIT
  return status_to_error(tkx_ragged_dot_drhs(lhs.untyped_data(), dout.untyped_data(), group_sizes.typed_data(),
                                             out->untyped_data(), workspace->untyped_data(), ld[0], ld[1], dd[1],
                                             (int64_t)group_sizes.element_count(), dtype_code(lhs.element_type()),
                                             dtype_code(out->element_type()), &cfg, stream));
}

}  // namespace

XLA_FFI_DEFINE_HANDLER_SYMBOL(TkxRaggedDotFwd, FwdImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::DataType::S32>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Attr<int32_t>("mode")
                                  .Attr<int32_t>("activation") TKX_CONFIG_ATTRS);

XLA_FFI_DEFINE_HANDLER_SYMBOL(TkxRaggedDotFwdFused, FwdFusedImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::DataType::S32>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Attr<int32_t>("rhs_scale_blocks")
                                  .Attr<int32_t>("activation")
                                  .Attr<int32_t>("gateup") TKX_CONFIG_ATTRS);

XLA_FFI_DEFINE_HANDLER_SYMBOL(TkxRaggedDotFwdFp8Out, FwdFp8OutImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::DataType::S32>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::Buffer<ffi::DataType::F32>>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Attr<int32_t>("activation") TKX_CONFIG_ATTRS);

XLA_FFI_DEFINE_HANDLER_SYMBOL(TkxRaggedDotDrhs, DrhsImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::DataType::S32>>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>() TKX_CONFIG_ATTRS);

extern "C" int32_t tkx_ffi_shim_available(void) { return 1; }

#else  // no xla/ffi/api/ffi.h on the include path

extern "C" int32_t tkx_ffi_shim_available(void) { return 0; }

#endif
