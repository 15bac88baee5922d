// XLA FFI handlers over the C ABI of libtkx_ragged_dot.so: what `jax.ffi.ffi_call` reaches when
// `implementation="hip"` runs under JAX. Each handler only unpacks buffers and attributes and forwards to the entry
// point of the same name; XLA owns every buffer, the workspace included (it is declared as an extra result).
//
// The header xla/ffi/api/ffi.h ships inside jaxlib. Where it is not on the include path this file compiles to a stub
// that exports only tkx_ffi_shim_available() == 0, so that the build never depends on a JAX install:
//   make -C tokamax_amd/csrc ffi        (builds ../lib/libtkx_ragged_dot_ffi.so when the header is found)
//
// Handler symbols and the Python registration that goes with them:
//   TkxRaggedDotFwd       jax.ffi.register_ffi_target("tkx_ragged_dot_fwd", jax.ffi.pycapsule(lib.TkxRaggedDotFwd), platform="ROCM")
//   TkxRaggedDotFwdFused  ... "tkx_ragged_dot_fwd_fused"
//   TkxRaggedDotDrhs      ... "tkx_ragged_dot_drhs"
// They replace the kernel calls of tokamax/_src/ops/ragged_dot/pallas_mosaic_gpu.py:231-238 (forward, dlhs) and
// pallas_mosaic_gpu_kernel_sm90.py:246-285 (drhs).
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

ffi::Error FwdImpl(hipStream_t stream, ffi::AnyBuffer lhs, ffi::AnyBuffer rhs, ffi::Buffer<ffi::DataType::S32> group_sizes,
                   ffi::AnyBuffer lhs_scale, ffi::AnyBuffer rhs_scale, ffi::Result<ffi::AnyBuffer> out,
                   ffi::Result<ffi::AnyBuffer> workspace, int32_t mode, int32_t activation, int32_t block_m,
                   int32_t block_n, int32_t block_k, int32_t waves_m, int32_t waves_n, int32_t grid_tile_width,
                   int32_t align_tile, int32_t num_stages) {
  const auto ld = lhs.dimensions(), rd = rhs.dimensions();
  if (ld.size() != 2 || rd.size() != 3) return ffi::Error(ffi::ErrorCode::kInvalidArgument, "expected lhs [m,k] and rhs [g,k,n]");
  const int64_t m = ld[0], G = rd[0], k = rd[1], n = rd[2];
  const TkxConfig cfg{block_m, block_n, block_k, waves_m, waves_n, grid_tile_width, align_tile, num_stages};
  return status_to_error(tkx_ragged_dot_fwd(
      lhs.untyped_data(), rhs.untyped_data(), group_sizes.typed_data(), optional_data<float>(lhs_scale),
      optional_data<float>(rhs_scale), out->untyped_data(), workspace->untyped_data(), m, k, n, G,
      dtype_code(lhs.element_type()), dtype_code(rhs.element_type()), dtype_code(out->element_type()), mode, activation,
      &cfg, stream));
}

// rhs_scale is [g, rhs_scale_blocks, n]; rhs_bias [g, n]; group_offset one S32 (zero-sized = absent), in which case
// group_sizes lists every group of the job and rhs holds those from the offset on. With gateup the result is [m, n/2].
ffi::Error FwdFusedImpl(hipStream_t stream, ffi::AnyBuffer lhs, ffi::AnyBuffer rhs, ffi::Buffer<ffi::DataType::S32> group_sizes,
                        ffi::AnyBuffer group_offset, ffi::AnyBuffer lhs_scale, ffi::AnyBuffer rhs_scale,
                        ffi::AnyBuffer rhs_bias, ffi::Result<ffi::AnyBuffer> out, ffi::Result<ffi::AnyBuffer> workspace,
                        int32_t rhs_scale_blocks, int32_t activation, int32_t gateup, int32_t block_m, int32_t block_n,
                        int32_t block_k, int32_t waves_m, int32_t waves_n, int32_t grid_tile_width, int32_t align_tile,
                        int32_t num_stages) {
  const auto ld = lhs.dimensions(), rd = rhs.dimensions();
  if (ld.size() != 2 || rd.size() != 3) return ffi::Error(ffi::ErrorCode::kInvalidArgument, "expected lhs [m,k] and rhs [g,k,n]");
  const int64_t m = ld[0], G = rd[0], k = rd[1], n = rd[2];
  const TkxConfig cfg{block_m, block_n, block_k, waves_m, waves_n, grid_tile_width, align_tile, num_stages};
  return status_to_error(tkx_ragged_dot_fwd_fused(
      lhs.untyped_data(), rhs.untyped_data(), group_sizes.typed_data(), optional_data<int32_t>(group_offset),
      optional_data<float>(lhs_scale), optional_data<float>(rhs_scale), optional_data<float>(rhs_bias), out->untyped_data(),
      workspace->untyped_data(), m, k, n, G, (int64_t)group_sizes.element_count(), rhs_scale_blocks,
      dtype_code(lhs.element_type()), dtype_code(rhs.element_type()), dtype_code(out->element_type()), activation, gateup,
      &cfg, stream));
}

ffi::Error DrhsImpl(hipStream_t stream, ffi::AnyBuffer lhs, ffi::AnyBuffer dout, ffi::Buffer<ffi::DataType::S32> group_sizes,
                    ffi::Result<ffi::AnyBuffer> out, ffi::Result<ffi::AnyBuffer> workspace, int32_t block_m,
                    int32_t block_n, int32_t block_k, int32_t waves_m, int32_t waves_n, int32_t align_tile,
                    int32_t num_stages) {
  const auto ld = lhs.dimensions(), dd = dout.dimensions();
  if (ld.size() != 2 || dd.size() != 2 || ld[0] != dd[0])
    return ffi::Error(ffi::ErrorCode::kInvalidArgument, "expected lhs [m,k] and dout [m,n]");
  const TkxConfig cfg{block_m, block_n, block_k, waves_m, waves_n, 1, align_tile, num_stages};
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
                                  .Attr<int32_t>("activation")
                                  .Attr<int32_t>("block_m")
                                  .Attr<int32_t>("block_n")
                                  .Attr<int32_t>("block_k")
                                  .Attr<int32_t>("waves_m")
                                  .Attr<int32_t>("waves_n")
                                  .Attr<int32_t>("grid_tile_width")
                                  .Attr<int32_t>("align_tile")
                                  .Attr<int32_t>("num_stages"));

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
                                  .Attr<int32_t>("gateup")
                                  .Attr<int32_t>("block_m")
                                  .Attr<int32_t>("block_n")
                                  .Attr<int32_t>("block_k")
                                  .Attr<int32_t>("waves_m")
                                  .Attr<int32_t>("waves_n")
                                  .Attr<int32_t>("grid_tile_width")
                                  .Attr<int32_t>("align_tile")
                                  .Attr<int32_t>("num_stages"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(TkxRaggedDotDrhs, DrhsImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::DataType::S32>>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Attr<int32_t>("block_m")
                                  .Attr<int32_t>("block_n")
                                  .Attr<int32_t>("block_k")
                                  .Attr<int32_t>("waves_m")
                                  .Attr<int32_t>("waves_n")
                                  .Attr<int32_t>("align_tile")
                                  .Attr<int32_t>("num_stages"));

extern "C" int32_t tkx_ffi_shim_available(void) { return 1; }

#else  // no xla/ffi/api/ffi.h on the include path

extern "C" int32_t tkx_ffi_shim_available(void) { return 0; }

#endif
