// Two ceilings of one MI355X that a tiled GEMM's TFLOP/s should be read against, as kernels bench.py can time on the
// box it runs on (libtkx_microbench.so; declared in include/tkx_microbench.h). They are measurement aids, not part of
// the operator library.
//
//  * tkxmb_mfma_bf16: what the matrix cores sustain on a register-resident loop of v_mfma_f32_32x32x16_bf16. The
//    published dense peak assumes the nominal shader clock; under a sustained MFMA load the clock settles lower, and
//    how much lower depends on the operand bits (the same instruction stream runs about 30 % faster on all-zero
//    operands than on random ones). A GEMM on real data is bounded by the random-data figure.
//  * tkxmb_operand_stream: the operand stream of a tiled GEMM without its arithmetic: workgroups stream HBM-resident
//    panels into LDS with global_load_lds_dwordx4, `share` workgroups of one XCD reading the same panel at a time,
//    as the tiles next to a GEMM tile share its operand panels through their XCD's L2.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "tkx_microbench.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) const void gvoid;
typedef __attribute__((address_space(3))) void lvoid;

constexpr int kThreads = 512;       // 8 waves, two per SIMD, as the GEMM kernels run
constexpr int kOperandWords = 4096; // 16-byte words of operand data (64 KB)
constexpr int kStreamGrid = 2048;   // workgroups of the stream kernel: 8 per CU, one after the other
constexpr int kStreamLds = 65536;

// One workgroup per CU; every wave cycles over 8 independent 32x32 accumulators (4 A x 2 B fragments, the shape of a
// wave's share of a 256 x 256 tile); no memory traffic inside the loop.
__global__ __launch_bounds__(kThreads) void mfma_loop(const i32x4* src, float* out, int iters) {
  constexpr int NA = 4, NB = 2;
  bf16x8 a[NA], b[NB];
  for (int i = 0; i < NA; ++i) a[i] = __builtin_bit_cast(bf16x8, src[(threadIdx.x + kThreads * i) % kOperandWords]);
  for (int i = 0; i < NB; ++i) b[i] = __builtin_bit_cast(bf16x8, src[(threadIdx.x * 7 + kThreads * i + 1234) % kOperandWords]);
  f32x16 acc[NA][NB];
  for (int i = 0; i < NA; ++i)
    for (int j = 0; j < NB; ++j)
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < NA; ++i)
#pragma unroll
      for (int j = 0; j < NB; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    if ((it & 7) == 7) {  // rotate the operands now and then so that the data path sees changing values
      const bf16x8 t = a[0];
      for (int i = 0; i + 1 < NA; ++i) a[i] = a[i + 1];
      a[NA - 1] = t;
    }
  }
  float s = 0;
  for (int i = 0; i < NA; ++i)
    for (int j = 0; j < NB; ++j)
      for (int e = 0; e < 16; ++e) s += acc[i][j][e];
  if (s == 12345.f) out[0] = s;  // keeps the loop alive
}

// The same loop on the fp8 (e4m3fn) form of the MFMA, 32x32x64 with 32-byte fragments and no block scales.
typedef int i32x8 __attribute__((ext_vector_type(8)));
__global__ __launch_bounds__(kThreads) void mfma_fp8_loop(const i32x4* src, float* out, int iters) {
  constexpr int NA = 4, NB = 2;
  i32x8 a[NA], b[NB];
  for (int i = 0; i < NA; ++i) {
    const i32x4 lo = src[(threadIdx.x + kThreads * i) % kOperandWords], hi = src[(threadIdx.x * 3 + kThreads * i + 77) % kOperandWords];
    a[i] = i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  }
  for (int i = 0; i < NB; ++i) {
    const i32x4 lo = src[(threadIdx.x * 7 + kThreads * i + 1234) % kOperandWords], hi = src[(threadIdx.x * 5 + kThreads * i + 4321) % kOperandWords];
    b[i] = i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  }
  f32x16 acc[NA][NB];
  for (int i = 0; i < NA; ++i)
    for (int j = 0; j < NB; ++j)
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < NA; ++i)
#pragma unroll
      for (int j = 0; j < NB; ++j) acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i], b[j], acc[i][j], 0, 0, 0, 0, 0, 0);
    if ((it & 7) == 7) {
      const i32x8 t = a[0];
      for (int i = 0; i + 1 < NA; ++i) a[i] = a[i + 1];
      a[NA - 1] = t;
    }
  }
  float s = 0;
  for (int i = 0; i < NA; ++i)
    for (int j = 0; j < NB; ++j)
      for (int e = 0; e < 16; ++e) s += acc[i][j][e];
  if (s == 12345.f) out[0] = s;
}

// Workgroup b runs on XCD b % 8; `share` consecutive workgroups of one XCD take the same region. A wave keeps
// INFLIGHT 1 KB loads outstanding.
template <int INFLIGHT>
__global__ __launch_bounds__(kThreads) void stream_kernel(const unsigned char* src, int64_t region_bytes, int regions, int share) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const int tid = threadIdx.x, wave = tid >> 6;
  const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
  const int per_xcd = regions / 8;
  const unsigned char* base = src + (int64_t)(xcd * per_xcd + (idx / share) % per_xcd) * region_bytes;
  const int64_t per_iter = kThreads * 16;  // one 1 KB load per wave
  const int64_t iters = region_bytes / per_iter;
  for (int64_t it = 0; it < iters; ++it) {
    __builtin_amdgcn_global_load_lds((gvoid*)(base + it * per_iter + tid * 16), (lvoid*)(smem + ((it % 8) * 8 + wave) * 1024), 16, 0, 0);
    // (vmcnt lives in bits 3:0 and 15:14 of the operand; the other counters are left alone)
    __builtin_amdgcn_s_waitcnt(0x0f70 | (INFLIGHT - 1));
  }
  __builtin_amdgcn_s_waitcnt(0);
}

}  // namespace

extern "C" {

int64_t tkxmb_mfma_bf16_flops(int32_t iters) {
  int cus = 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0) != hipSuccess) return -1;
  return (int64_t)cus * (kThreads / 64) * iters * 8 * 32768;  // 8 MFMAs of 32 x 32 x 16 x 2 FLOP per wave and iteration
}

int32_t tkxmb_mfma_bf16(const void* operands, int32_t iters, void* sink, void* stream) {
  if (operands == nullptr || sink == nullptr || iters < 1) return 1;
  int cus = 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0) != hipSuccess) return 3;
  mfma_loop<<<cus, kThreads, 0, static_cast<hipStream_t>(stream)>>>(static_cast<const i32x4*>(operands), static_cast<float*>(sink), iters);
  return hipGetLastError() == hipSuccess ? 0 : 3;
}

int64_t tkxmb_mfma_fp8_flops(int32_t iters) { return 4 * tkxmb_mfma_bf16_flops(iters); }  // 32 x 32 x 64 against 32 x 32 x 16

int32_t tkxmb_mfma_fp8(const void* operands, int32_t iters, void* sink, void* stream) {
  if (operands == nullptr || sink == nullptr || iters < 1) return 1;
  int cus = 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0) != hipSuccess) return 3;
  mfma_fp8_loop<<<cus, kThreads, 0, static_cast<hipStream_t>(stream)>>>(static_cast<const i32x4*>(operands), static_cast<float*>(sink), iters);
  return hipGetLastError() == hipSuccess ? 0 : 3;
}

int64_t tkxmb_operand_stream_bytes(int64_t region_bytes) { return (int64_t)kStreamGrid * region_bytes; }

int32_t tkxmb_operand_stream(const void* src, int64_t region_bytes, int32_t regions, int32_t share, void* stream) {
  if (src == nullptr || region_bytes < kThreads * 16 || region_bytes % (kThreads * 16) != 0 || regions < 8 || regions % 8 != 0 ||
      share < 1 || share > 32)
    return 1;
  static bool raised = false;  // (one device per process: bench.py runs on device 0)
  if (!raised) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&stream_kernel<8>), hipFuncAttributeMaxDynamicSharedMemorySize, kStreamLds) != hipSuccess)
      return 3;
    raised = true;
  }
  stream_kernel<8><<<kStreamGrid, kThreads, kStreamLds, static_cast<hipStream_t>(stream)>>>(static_cast<const unsigned char*>(src), region_bytes,
                                                                                           regions, share);
  return hipGetLastError() == hipSuccess ? 0 : 3;
}

}  // extern "C"
