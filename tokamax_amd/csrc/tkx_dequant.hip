// Dequantisation with block scales: out[r, c] = (q[r, c] - zero_point[R, C]) * scale[R, C] with
// (R, C) = (r / t_r, c / t_c), q int8 or fp8 (e4m3fn), out bf16; the zero point (f32, shaped like the scale) is optional.
//
// The tiled kernels apply one scale per lhs row and one per (group, column) in their epilogue, which
// covers scales that span the whole contraction. Operands whose scales change along the contraction
// (weights [G, k, n] with scale [G, k / t_k, n / t_n], viewed as G * k rows; an lhs [m, k] with scale
// [m, k / t]) are widened to bf16 by this streaming pass and then take the bf16 kernels; the
// reference's "xla" path does the same as a separate elementwise step (base.py:332). The pass is
// bound by HBM: it reads 1 byte and writes 2 per element.
#include "tkx_common.h"
#include "tkx_gemm.hip.h"

namespace tkx {
namespace {

constexpr int kDqThreads = 256;

// Byte B of a dword as f32: a sign-extended int8, or an OCP e4m3fn value (the hardware conversion).
template <int EQ, int B>
__device__ __forceinline__ float widen_byte(int w) {
  if constexpr (EQ == kEI8) return (float)(signed char)((w >> (8 * B)) & 0xff);
  else return __builtin_amdgcn_cvt_f32_fp8(w, B);
}

// One thread converts 16 consecutive columns of one row: a 16-byte load, the scales of those columns
// (four 16-byte loads when every column has its own, t_c == 1; one value when a scale block spans
// them, t_c % 16 == 0; L2-resident either way: a scale row serves t_r rows), two 16-byte stores.
template <int EQ, bool ZP>
__global__ __launch_bounds__(kDqThreads) void dequant_kernel(const unsigned char* __restrict__ q,
                                                            const float* __restrict__ scale,
                                                            const float* __restrict__ zero_point, __bf16* __restrict__ out,
                                                            int64_t rows, int32_t n, int32_t t_r, int32_t t_c) {
  const int chunks = n / 16;  // n % 16 == 0 (checked on the host)
  const int64_t total = rows * chunks;
  const int scale_cols = n / t_c;
  for (int64_t idx = (int64_t)blockIdx.x * kDqThreads + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * kDqThreads) {
    const int64_t row = idx / chunks;
    const int c0 = (int)(idx - row * chunks) * 16;
    const i32x4 w = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(q + row * n + c0));
    const float* srow = scale + (row / t_r) * scale_cols;
    f32x4 sc[4], zp[4];
    if (t_c == 1) {
#pragma unroll
      for (int d = 0; d < 4; ++d) sc[d] = *reinterpret_cast<const f32x4*>(srow + c0 + 4 * d);
    } else {
      const float one = srow[c0 / t_c];
#pragma unroll
      for (int d = 0; d < 4; ++d) sc[d] = (f32x4){one, one, one, one};
    }
    if constexpr (ZP) {
      const float* zrow = zero_point + (row / t_r) * scale_cols;
      if (t_c == 1) {
#pragma unroll
        for (int d = 0; d < 4; ++d) zp[d] = *reinterpret_cast<const f32x4*>(zrow + c0 + 4 * d);
      } else {
        const float one = zrow[c0 / t_c];
#pragma unroll
        for (int d = 0; d < 4; ++d) zp[d] = (f32x4){one, one, one, one};
      }
    }
    bf16x8 lo, hi;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const int word = w[d];
      float v[4] = {widen_byte<EQ, 0>(word), widen_byte<EQ, 1>(word), widen_byte<EQ, 2>(word), widen_byte<EQ, 3>(word)};
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        if constexpr (ZP) v[b] -= zp[d][b];
        v[b] *= sc[d][b];
      }
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int e = 4 * d + b;
        if (e < 8) lo[e] = (__bf16)v[b];
        else hi[e - 8] = (__bf16)v[b];
      }
    }
    __bf16* o = out + row * n + c0;
    __builtin_nontemporal_store(lo, reinterpret_cast<bf16x8*>(o));
    __builtin_nontemporal_store(hi, reinterpret_cast<bf16x8*>(o + 8));
  }
}

// Packed int4 <-> int8. A packed row holds two value rows: byte [rr, c] = value [2 rr, c] in bits 0-3 and value
// [2 rr + 1, c] in bits 4-7. One thread takes 16 columns of one packed row (16 bytes in, two rows of 16 out, or back).
__global__ __launch_bounds__(kDqThreads) void unpack_int4_kernel(const unsigned char* __restrict__ packed,
                                                                signed char* __restrict__ out, int64_t packed_rows, int32_t n) {
  const int chunks = n / 16;
  const int64_t total = packed_rows * chunks;
  for (int64_t idx = (int64_t)blockIdx.x * kDqThreads + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * kDqThreads) {
    const int64_t row = idx / chunks;
    const int c0 = (int)(idx - row * chunks) * 16;
    const i32x4 w = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(packed + row * n + c0));
    i32x4 lo, hi;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      // Per byte: sign-extend bits 0-3 (shift the nibble to the byte's top, arithmetic shift back) and bits 4-7.
      unsigned l = 0, h = 0;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        l |= ((unsigned)__builtin_amdgcn_sbfe(w[d], 8 * b, 4) & 0xffu) << (8 * b);
        h |= ((unsigned)__builtin_amdgcn_sbfe(w[d], 8 * b + 4, 4) & 0xffu) << (8 * b);
      }
      lo[d] = (int)l;
      hi[d] = (int)h;
    }
    *reinterpret_cast<i32x4*>(out + (2 * row) * n + c0) = lo;
    *reinterpret_cast<i32x4*>(out + (2 * row + 1) * n + c0) = hi;
  }
}
__global__ __launch_bounds__(kDqThreads) void pack_int4_kernel(const signed char* __restrict__ q, unsigned char* __restrict__ packed,
                                                              int64_t packed_rows, int32_t n) {
  const int chunks = n / 16;
  const int64_t total = packed_rows * chunks;
  for (int64_t idx = (int64_t)blockIdx.x * kDqThreads + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * kDqThreads) {
    const int64_t row = idx / chunks;
    const int c0 = (int)(idx - row * chunks) * 16;
    const i32x4 lo = *reinterpret_cast<const i32x4*>(q + (2 * row) * n + c0);
    const i32x4 hi = *reinterpret_cast<const i32x4*>(q + (2 * row + 1) * n + c0);
    i32x4 w;
#pragma unroll
    for (int d = 0; d < 4; ++d) w[d] = (int)(((unsigned)lo[d] & 0x0f0f0f0fu) | (((unsigned)hi[d] & 0x0f0f0f0fu) << 4));
    *reinterpret_cast<i32x4*>(packed + row * n + c0) = w;
  }
}

// Row sums of an fp8 (e4m3fn) matrix [rows, n], n % 16 == 0: one wave per row, 16 bytes per lane and step, summed in
// f32. The sums of activation rows, which the fp8 x packed-int4 kernels take their +8 weight bias off with.
// PER_128 (n % 128 == 0): one sum per run of 128 columns (8 lanes), sums[n / 128][rows].
template <bool PER_128>
__global__ __launch_bounds__(kDqThreads) void row_sums_fp8_kernel(const unsigned char* __restrict__ x, float* __restrict__ sums,
                                                                 int64_t rows, int32_t n) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * (kDqThreads / 64) + (threadIdx.x >> 6);
  if (row >= rows) return;  // (whole waves leave together)
  float s = 0.f;
  for (int c0 = lane * 16; c0 < n; c0 += 64 * 16) {
    const i32x4 w = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(x + row * n + c0));
#pragma unroll
    for (int d = 0; d < 4; ++d)
      s += (widen_byte<kEF8, 0>(w[d]) + widen_byte<kEF8, 1>(w[d])) + (widen_byte<kEF8, 2>(w[d]) + widen_byte<kEF8, 3>(w[d]));
    if constexpr (PER_128) {
      // (the lanes of a group of 8 are in the loop together: n is a multiple of 128)
#pragma unroll
      for (int o = 4; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
      if ((lane & 7) == 0) sums[(int64_t)(c0 >> 7) * rows + row] = s;
      s = 0.f;
    }
  }
  if constexpr (!PER_128) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
    if (lane == 0) sums[row] = s;
  }
}

}  // namespace

int32_t launch_row_sums_fp8(const void* x, float* sums, int64_t rows, int64_t n, bool per_128, hipStream_t stream) {
  const int64_t grid = (rows + kDqThreads / 64 - 1) / (kDqThreads / 64);
  const auto* xb = static_cast<const unsigned char*>(x);
  if (per_128) row_sums_fp8_kernel<true><<<dim3((unsigned)grid), dim3(kDqThreads), 0, stream>>>(xb, sums, rows, (int32_t)n);
  else row_sums_fp8_kernel<false><<<dim3((unsigned)grid), dim3(kDqThreads), 0, stream>>>(xb, sums, rows, (int32_t)n);
  TKX_HIP_CHECK(hipGetLastError());
  return TKX_OK;
}

int32_t launch_int4_repack(const void* in, void* out, int64_t packed_rows, int64_t n, bool unpack, hipStream_t stream) {
  const int64_t total = packed_rows * (n / 16);
  int64_t grid = (total + kDqThreads - 1) / kDqThreads;
  if (grid > 256 * 16) grid = 256 * 16;
  if (grid < 1) grid = 1;
  if (unpack)
    unpack_int4_kernel<<<dim3((unsigned)grid), dim3(kDqThreads), 0, stream>>>(static_cast<const unsigned char*>(in),
                                                                              static_cast<signed char*>(out), packed_rows, (int32_t)n);
  else
    pack_int4_kernel<<<dim3((unsigned)grid), dim3(kDqThreads), 0, stream>>>(static_cast<const signed char*>(in),
                                                                            static_cast<unsigned char*>(out), packed_rows, (int32_t)n);
  TKX_HIP_CHECK(hipGetLastError());
  return TKX_OK;
}

int32_t launch_dequant(const void* q, const float* scale, const float* zero_point, void* out, int64_t rows, int64_t n,
                       int64_t t_r, int64_t t_c, int32_t q_dtype, hipStream_t stream) {
  const int64_t total = rows * (n / 16);
  int64_t grid = (total + kDqThreads - 1) / kDqThreads;
  if (grid > 256 * 16) grid = 256 * 16;  // 16 workgroups per CU, grid-stride beyond that
  if (grid < 1) grid = 1;
  const auto* qb = static_cast<const unsigned char*>(q);
  auto* ob = static_cast<__bf16*>(out);
  const dim3 g((unsigned)grid), b(kDqThreads);
  const int32_t n32 = (int32_t)n, tr = (int32_t)t_r, tc = (int32_t)t_c;
  if (q_dtype == TKX_I8 && zero_point) dequant_kernel<kEI8, true><<<g, b, 0, stream>>>(qb, scale, zero_point, ob, rows, n32, tr, tc);
  else if (q_dtype == TKX_I8) dequant_kernel<kEI8, false><<<g, b, 0, stream>>>(qb, scale, nullptr, ob, rows, n32, tr, tc);
  else if (zero_point) dequant_kernel<kEF8, true><<<g, b, 0, stream>>>(qb, scale, zero_point, ob, rows, n32, tr, tc);
  else dequant_kernel<kEF8, false><<<g, b, 0, stream>>>(qb, scale, nullptr, ob, rows, n32, tr, tc);
  TKX_HIP_CHECK(hipGetLastError());
  return TKX_OK;
}

}  // namespace tkx
