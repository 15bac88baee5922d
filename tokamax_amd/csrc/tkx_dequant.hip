// Weight dequantisation with sub-channel scales: out[g, kk, c] = q[g, kk, c] * scale[g, kk / t_k, c].
//
// The tiled kernels apply one scale per (group, column) in their epilogue, which covers scales that
// span the whole contraction (t_k == k). Weights with several scale blocks along k (t_k < k, scale
// [G, k / t_k, n]) are widened to bf16 by this streaming pass and then take the bf16 kernels; the
// reference's "xla" path does the same as a separate elementwise step (base.py:332). The pass is
// bound by HBM: it reads 1 byte and writes 2 per weight.
#include "tkx_common.h"
#include "tkx_gemm.hip.h"

namespace tkx {
namespace {

constexpr int kDqThreads = 256;

// One thread converts 16 consecutive columns of one k-row: a 16-byte load of int8, two 16-byte
// scale loads per 8 columns (L2-resident: a scale row serves t_k weight rows), two 16-byte stores.
__global__ __launch_bounds__(kDqThreads) void dequant_i8_kernel(const signed char* __restrict__ q,
                                                               const float* __restrict__ scale, __bf16* __restrict__ out,
                                                               int64_t rows /* G * k */, int32_t k, int32_t n, int32_t t_k) {
  const int chunks = n / 16;  // n % 16 == 0 (checked on the host)
  const int64_t total = rows * chunks;
  const int kb_per_group = k / t_k;
  for (int64_t idx = (int64_t)blockIdx.x * kDqThreads + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * kDqThreads) {
    const int64_t row = idx / chunks;
    const int c0 = (int)(idx - row * chunks) * 16;
    const int64_t g = row / k;
    const int kk = (int)(row - g * k);
    const i32x4 w = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(q + row * n + c0));
    const f32x4* s = reinterpret_cast<const f32x4*>(scale + ((int64_t)g * kb_per_group + kk / t_k) * n + c0);
    bf16x8 lo, hi;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const f32x4 sc = s[d];
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const float v = (float)(signed char)((w[d] >> (8 * b)) & 0xff) * sc[b];
        const int e = 4 * d + b;
        if (e < 8) lo[e] = (__bf16)v;
        else hi[e - 8] = (__bf16)v;
      }
    }
    __bf16* o = out + row * n + c0;
    __builtin_nontemporal_store(lo, reinterpret_cast<bf16x8*>(o));
    __builtin_nontemporal_store(hi, reinterpret_cast<bf16x8*>(o + 8));
  }
}

}  // namespace

int32_t launch_dequant_i8(const void* q, const float* scale, void* out, int64_t G, int64_t k, int64_t n, int64_t t_k,
                          hipStream_t stream) {
  const int64_t total = G * k * (n / 16);
  int64_t grid = (total + kDqThreads - 1) / kDqThreads;
  if (grid > 256 * 16) grid = 256 * 16;  // 16 workgroups per CU, grid-stride beyond that
  dequant_i8_kernel<<<dim3((unsigned)grid), dim3(kDqThreads), 0, stream>>>(
      static_cast<const signed char*>(q), scale, static_cast<__bf16*>(out), G * k, (int32_t)k, (int32_t)n, (int32_t)t_k);
  TKX_HIP_CHECK(hipGetLastError());
  return TKX_OK;
}

}  // namespace tkx
