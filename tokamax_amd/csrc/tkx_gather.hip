// Row gather with optional mask, weight and reduction: the token permute / un-permute steps either
// side of the ragged dot in an MoE layer.
//
//   out[j, :] = sum over r < R of  keep(jR + r) * weight[jR + r] * x[indices[jR + r], :]
//
// R = 1 without weights is a plain gather (ragged_gather/base.py:25-32); with the row range
// [start, end) as the keep test on the index it is ragged_scatter/base.py:26-38; with weights, a
// validity mask and R > 1 it is ragged_gather_reduce/base.py:26-40 (products and sums in f32, one
// rounding to the output type). Bound by HBM: a workgroup moves one output row with 16-byte accesses.
#include "tkx_common.h"
#include "tkx_gemm.hip.h"

namespace tkx {
namespace {

constexpr int kGatherThreads = 256;

struct GatherParams {
  const unsigned char* x;
  const int32_t* indices;
  const float* weights;          // per gathered row, or null
  const unsigned char* valid;    // per gathered row (bytes, nonzero = keep), or null
  const int32_t* start;          // device scalars: keep rows with start <= index < end, or null
  const int32_t* end;
  unsigned char* out;
  int64_t in_rows, out_rows;
  int32_t hidden, reduce, dtype;  // hidden elements per row; rows reduced per output row
};

template <int ESZ>
__global__ __launch_bounds__(kGatherThreads) void gather_rows_kernel(const GatherParams p) {
  constexpr int PER = 16 / ESZ;  // elements per 16-byte access
  const int chunks = p.hidden / PER;
  const bool ranged = p.start != nullptr;
  const int lo = ranged ? p.start[0] : 0, hi = ranged ? p.end[0] : 0;
  constexpr int RMAX = 8;  // gathered rows per output row whose index, mask and weight are read once per row
  for (int64_t j = blockIdx.x; j < p.out_rows; j += gridDim.x) {
    // Source row (-1: dropped) and weight of gathered row g.
    auto source = [&](int64_t g, int64_t& row, float& w) {
      const int idx = p.indices[g];
      const bool keep = (!ranged || (idx >= lo && idx < hi)) && !(p.valid && p.valid[g] == 0);
      // x[indices] as the reference's indexing reads it: a negative index counts from the end, and what is
      // still outside the array after that is clamped to the nearest row.
      const int64_t wrapped = idx < 0 ? (int64_t)idx + p.in_rows : (int64_t)idx;
      row = !keep ? -1 : wrapped < 0 ? 0 : wrapped >= p.in_rows ? p.in_rows - 1 : wrapped;
      w = p.weights ? p.weights[g] : 1.f;
    };
    int64_t rows[RMAX];
    float wts[RMAX];
#pragma unroll
    for (int r = 0; r < RMAX; ++r) {
      rows[r] = -1;
      wts[r] = 0.f;
      if (r < p.reduce) source(j * p.reduce + r, rows[r], wts[r]);
    }
    for (int c = threadIdx.x; c < chunks; c += kGatherThreads) {
      float acc[PER];
#pragma unroll
      for (int e = 0; e < PER; ++e) acc[e] = 0.f;
      i32x4 last = {0, 0, 0, 0};
      bool any = false;
      auto add = [&](int64_t row, float w) {
        const i32x4 v = *reinterpret_cast<const i32x4*>(p.x + (row * p.hidden + (int64_t)c * PER) * ESZ);
        last = v;
        any = true;
#pragma unroll
        for (int e = 0; e < PER; ++e) {
          float f;
          // (Elements go through a scalar first: a bit cast applied straight to a vector subscript
          // was seen to read element 0 whatever the index.)
          const int word = ESZ == 4 ? v[e] : v[e >> 1];
          if constexpr (ESZ == 4) f = __builtin_bit_cast(float, word);
          else if (p.dtype == TKX_BF16) f = __builtin_bit_cast(float, (unsigned)(((unsigned)word >> (16 * (e & 1))) << 16));
          else f = (float)__builtin_bit_cast(_Float16, (unsigned short)((unsigned)word >> (16 * (e & 1))));
          acc[e] += w * f;
        }
      };
#pragma unroll
      for (int r = 0; r < RMAX; ++r)
        if (rows[r] >= 0) add(rows[r], wts[r]);
      for (int r = RMAX; r < p.reduce; ++r) {
        int64_t row;
        float w;
        source(j * p.reduce + r, row, w);
        if (row >= 0) add(row, w);
      }
      i32x4 o;
      if (p.reduce == 1 && p.weights == nullptr) {
        o = any ? last : (i32x4){0, 0, 0, 0};  // a pure copy keeps the bits
      } else if constexpr (ESZ == 4) {
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = __builtin_bit_cast(int, acc[e]);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          unsigned short h0, h1;
          if (p.dtype == TKX_BF16) {
            h0 = __builtin_bit_cast(unsigned short, (__bf16)acc[2 * e]);
            h1 = __builtin_bit_cast(unsigned short, (__bf16)acc[2 * e + 1]);
          } else {
            h0 = __builtin_bit_cast(unsigned short, (_Float16)acc[2 * e]);
            h1 = __builtin_bit_cast(unsigned short, (_Float16)acc[2 * e + 1]);
          }
          o[e] = (int)((unsigned)h0 | ((unsigned)h1 << 16));
        }
      }
      *reinterpret_cast<i32x4*>(p.out + (j * p.hidden + (int64_t)c * PER) * ESZ) = o;
    }
  }
}

}  // namespace

int32_t launch_gather_rows(const void* x, const int32_t* indices, const float* weights, const unsigned char* valid,
                           const int32_t* start, const int32_t* end, void* out, int64_t in_rows, int64_t out_rows,
                           int64_t hidden, int64_t reduce, int32_t dtype, hipStream_t stream) {
  GatherParams p;
  p.x = static_cast<const unsigned char*>(x);
  p.indices = indices;
  p.weights = weights;
  p.valid = valid;
  p.start = start;
  p.end = end;
  p.out = static_cast<unsigned char*>(out);
  p.in_rows = in_rows;
  p.out_rows = out_rows;
  p.hidden = (int32_t)hidden;
  p.reduce = (int32_t)reduce;
  p.dtype = dtype;
  int64_t grid = out_rows < 256 * 32 ? out_rows : 256 * 32;  // grid-stride beyond 32 rows per CU in flight
  if (grid < 1) return TKX_OK;
  if (dtype == TKX_F32) gather_rows_kernel<4><<<dim3((unsigned)grid), dim3(kGatherThreads), 0, stream>>>(p);
  else gather_rows_kernel<2><<<dim3((unsigned)grid), dim3(kGatherThreads), 0, stream>>>(p);
  TKX_HIP_CHECK(hipGetLastError());
  return TKX_OK;
}

}  // namespace tkx
