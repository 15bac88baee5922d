// Absmax quantisation with block scales: the inverse pass of tkx_dequant.hip.
//
//   scale[R, C] = max |x[r, c]| over the tile (R, C) / qmax      (1 where the tile is all zero)
//   q[r, c]     = convert(x[r, c] / scale[r / t_r, c / t_c])
//
// qmax is the largest finite value of the quantised type (127 for int8, 448 for OCP e4m3fn); convert rounds to
// nearest, ties to even, and saturates at +-qmax. This is the symmetric ("absmax") calibration that
// tokamax/_src/quantization.py:65-78 asks of qwix.quantize, in the form the reference states it itself for its fused
// output quantisation (pallas_mosaic_gpu_kernel_sm100_fp8_quant.py:802-822). x is f32, bf16 or f16, row-major.
//
// Three forms, all bound by HBM (the second read of a tile comes from cache where the tile is small):
//   * tiles one row tall (an lhs [m, k] with one scale per row or per (row, t_c columns)): a group of lanes owns a
//     tile, 8 elements per lane and step, and reduces with lane shuffles;
//   * tiles several rows tall (weights [g, k, n] as g * k rows with one scale per (group, column) or per
//     (t_r rows, column) or per (t_r x t_c) block): a workgroup owns t_r rows x 256 columns, 8 row slices of 32 lanes x
//     8 columns each, and reduces through LDS;
//   * any other tile several rows tall (one scale for a whole tensor, 512-column blocks, ...): the tile's maximum is
//     collected with an atomic maximum on its bit pattern, then a second pass converts.
#include "tkx_common.h"
#include "tkx_gemm.hip.h"

namespace tkx {
namespace {

constexpr int kQThreads = 256;

template <int EX> struct XVec;
template <> struct XVec<kEF32> { static constexpr int BYTES = 32; };
template <> struct XVec<kEBF16> { static constexpr int BYTES = 16; };
template <> struct XVec<kEF16> { static constexpr int BYTES = 16; };

// 8 consecutive elements of x as f32.
template <int EX>
__device__ __forceinline__ void load8(const unsigned char* p, float (&v)[8]) {
  if constexpr (EX == kEF32) {
    const f32x4 a = *reinterpret_cast<const f32x4*>(p), b = *reinterpret_cast<const f32x4*>(p + 16);
#pragma unroll
    for (int e = 0; e < 4; ++e) { v[e] = a[e]; v[4 + e] = b[e]; }
  } else if constexpr (EX == kEBF16) {
    const bf16x8 a = *reinterpret_cast<const bf16x8*>(p);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (float)a[e];
  } else {
    const f16x8 a = *reinterpret_cast<const f16x8*>(p);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (float)a[e];
  }
}

__device__ __forceinline__ float absmax8(const float (&v)[8]) {
  float m = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) m = fmaxf(m, fabsf(v[e]));
  return m;
}

__device__ __forceinline__ float scale_of(float absmax, QuantRange qr) { return absmax == 0.f ? 1.f : absmax / qr.bound; }

// 8 values / scale -> 8 quantised bytes (two dwords).
template <int EQ>
__device__ __forceinline__ i32x2 quantize8(const float (&v)[8], const float (&scale)[8], QuantRange qr) {
  i32x2 out;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    float q[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) q[e] = fminf(fmaxf(v[4 * h + e] / scale[4 * h + e], qr.lo), qr.hi);
    if constexpr (EQ == kEI8) {
      unsigned w = 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) w |= ((unsigned)(int)__builtin_rintf(q[e]) & 0xffu) << (8 * e);
      out[h] = (int)w;
    } else {
      int w = 0;
      w = __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], w, false);
      w = __builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], w, true);
      out[h] = w;
    }
  }
  return out;
}

// Tiles one row tall. L lanes (a power of two <= 64) own one tile; a wave holds 64 / L tiles of consecutive
// (row, column-tile) pairs; tiles wider than 8 L columns are walked in steps.
template <int EX, int EQ>
__global__ __launch_bounds__(kQThreads) void quantize_rows_kernel(const unsigned char* __restrict__ x,
                                                                  unsigned char* __restrict__ q, float* __restrict__ scale,
                                                                  int64_t rows, int32_t cols, int32_t t_c, int32_t L,
                                                                  QuantRange qmax) {
  constexpr int XB = XVec<EX>::BYTES;  // bytes of 8 elements of x
  const int lane = threadIdx.x & 63;
  const int tiles_per_row = cols / t_c;
  const int64_t num_tiles = rows * tiles_per_row;
  const int per_wave = 64 / L;
  const int64_t wave_id = ((int64_t)blockIdx.x * kQThreads + threadIdx.x) >> 6;
  const int64_t num_waves = ((int64_t)gridDim.x * kQThreads) >> 6;
  const int sub = lane / L, l = lane % L;
  const int chunks = t_c / 8;
  for (int64_t t0 = wave_id * per_wave; t0 < num_tiles; t0 += num_waves * per_wave) {
    const int64_t tile = t0 + sub;
    const bool live = tile < num_tiles;
    const int64_t row = live ? tile / tiles_per_row : 0;
    const int c0 = live ? (int)(tile - row * tiles_per_row) * t_c : 0;
    const unsigned char* xr = x + (row * cols + c0) * (XB / 8);
    float m = 0.f;
    if (live) {
      for (int c = l; c < chunks; c += L) {
        float v[8];
        load8<EX>(xr + (int64_t)c * XB, v);
        m = fmaxf(m, absmax8(v));
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1)
      if (off < L) m = fmaxf(m, __shfl_xor(m, off));
    const float s = scale_of(m, qmax);
    if (live) {
      if (l == 0) scale[tile] = s;
      const float sv[8] = {s, s, s, s, s, s, s, s};
      unsigned char* qr = q + row * cols + c0;
      for (int c = l; c < chunks; c += L) {
        float v[8];
        load8<EX>(xr + (int64_t)c * XB, v);
        *reinterpret_cast<i32x2*>(qr + c * 8) = quantize8<EQ>(v, sv, qmax);
      }
    }
  }
}

// Tiles t_r > 1 rows tall and t_c columns wide (t_c == 1, or a power of two in [8, 256]). A workgroup owns
// (row tile, 256 columns): thread (slice = tid / 32, lane32 = tid % 32) takes columns 8 lane32 .. + 7 of the rows
// slice, slice + 8, ...
template <int EX, int EQ>
__global__ __launch_bounds__(kQThreads) void quantize_blocks_kernel(const unsigned char* __restrict__ x,
                                                                    unsigned char* __restrict__ q, float* __restrict__ scale,
                                                                    int64_t rows, int32_t cols, int32_t t_r, int32_t t_c,
                                                                    QuantRange qmax) {
  constexpr int XB = XVec<EX>::BYTES;
  __shared__ float red[8][256];
  const int tid = threadIdx.x, slice = tid >> 5, l32 = tid & 31;
  const int col_chunks = (cols + 255) / 256;
  const int64_t row_tile = blockIdx.x / col_chunks;
  const int c0 = (int)(blockIdx.x - row_tile * col_chunks) * 256 + 8 * l32;
  const bool live = c0 < cols;  // cols % 8 == 0
  const int64_t r0 = row_tile * t_r;
  float m[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) m[e] = 0.f;
  if (live) {
    for (int r = slice; r < t_r; r += 8) {
      float v[8];
      load8<EX>(x + ((r0 + r) * cols + c0) * (XB / 8), v);
#pragma unroll
      for (int e = 0; e < 8; ++e) m[e] = fmaxf(m[e], fabsf(v[e]));
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) red[slice][8 * l32 + e] = m[e];
  __syncthreads();
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    float a = 0.f;
#pragma unroll
    for (int s_ = 0; s_ < 8; ++s_) a = fmaxf(a, red[s_][8 * l32 + e]);
    m[e] = a;
  }
  float s[8];
  if (t_c == 1) {
#pragma unroll
    for (int e = 0; e < 8; ++e) s[e] = scale_of(m[e], qmax);
    if (live && slice == 0) {
      float* so = scale + row_tile * cols + c0;
      *reinterpret_cast<f32x4*>(so) = (f32x4){s[0], s[1], s[2], s[3]};
      *reinterpret_cast<f32x4*>(so + 4) = (f32x4){s[4], s[5], s[6], s[7]};
    }
  } else {
    float a = absmax8(m);
    const int lanes = t_c / 8;  // lanes (of the 32 that share a row) whose columns lie in one scale block
#pragma unroll
    for (int off = 16; off > 0; off >>= 1)
      if (off < lanes) a = fmaxf(a, __shfl_xor(a, off));
    const float one = scale_of(a, qmax);
#pragma unroll
    for (int e = 0; e < 8; ++e) s[e] = one;
    if (live && slice == 0 && (l32 % lanes) == 0) scale[row_tile * (cols / t_c) + c0 / t_c] = one;
  }
  if (live) {
    for (int r = slice; r < t_r; r += 8) {
      float v[8];
      load8<EX>(x + ((r0 + r) * cols + c0) * (XB / 8), v);
      *reinterpret_cast<i32x2*>(q + (r0 + r) * cols + c0) = quantize8<EQ>(v, s, qmax);
    }
  }
}

// Any other tile several rows tall (wider than 256 columns, or not a power of two wide; t_c a multiple of 8): three
// passes over chunks of 8 consecutive elements, which never straddle a tile. (1) The tile's scale slot collects the bit
// pattern of max |x| with an integer atomic maximum (non-negative floats order like their bits; the result does not
// depend on the order of arrival); a wave whose chunks all lie in one tile reduces with shuffles first. (2) The slot
// becomes the scale. (3) The values are divided and converted. The slots are zeroed by the first kernel of the three.
__global__ void tile_slots_clear_kernel(float* __restrict__ scale, int64_t num_tiles) {
  for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < num_tiles; t += (int64_t)gridDim.x * blockDim.x) scale[t] = 0.f;
}

__device__ __forceinline__ int64_t tile_of_chunk(int64_t chunk, int32_t chunks_per_row, int32_t t_r, int32_t t_c, int32_t tiles_per_row,
                                                 int64_t* row, int32_t* col) {
  *row = chunk / chunks_per_row;
  *col = (int32_t)(chunk - *row * chunks_per_row) * 8;
  return (*row / t_r) * tiles_per_row + *col / t_c;
}

template <int EX>
__global__ __launch_bounds__(kQThreads) void tile_absmax_kernel(const unsigned char* __restrict__ x, float* __restrict__ scale,
                                                                int64_t rows, int32_t cols, int32_t t_r, int32_t t_c) {
  constexpr int XB = XVec<EX>::BYTES;
  const int32_t chunks_per_row = cols / 8, tiles_per_row = cols / t_c;
  const int64_t chunks = rows * chunks_per_row, stride = (int64_t)gridDim.x * kQThreads;
  // (Every lane of a wave runs the same number of rounds, so that the shuffles below see all 64 lanes.)
  for (int64_t base = (int64_t)blockIdx.x * kQThreads; base < chunks; base += stride) {
    const int64_t chunk = base + threadIdx.x;
    const bool live = chunk < chunks;
    int64_t row;
    int32_t col;
    const int64_t tile = tile_of_chunk(live ? chunk : chunks - 1, chunks_per_row, t_r, t_c, tiles_per_row, &row, &col);
    float m = 0.f;
    if (live) {
      float v[8];
      load8<EX>(x + (row * cols + col) * (XB / 8), v);
      m = absmax8(v);
    }
    const int64_t first = __shfl(tile, 0);
    if (__all(tile == first)) {
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
      if ((threadIdx.x & 63) == 0) atomicMax(reinterpret_cast<unsigned*>(scale) + tile, __builtin_bit_cast(unsigned, m));
    } else if (live) {
      atomicMax(reinterpret_cast<unsigned*>(scale) + tile, __builtin_bit_cast(unsigned, m));
    }
  }
}

__global__ void tile_scale_kernel(float* __restrict__ scale, int64_t num_tiles, QuantRange qmax) {
  for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < num_tiles; t += (int64_t)gridDim.x * blockDim.x)
    scale[t] = scale_of(scale[t], qmax);
}

template <int EX, int EQ>
__global__ __launch_bounds__(kQThreads) void quantize_tiles_kernel(const unsigned char* __restrict__ x, unsigned char* __restrict__ q,
                                                                   const float* __restrict__ scale, int64_t rows, int32_t cols,
                                                                   int32_t t_r, int32_t t_c, QuantRange qmax) {
  constexpr int XB = XVec<EX>::BYTES;
  const int32_t chunks_per_row = cols / 8, tiles_per_row = cols / t_c;
  const int64_t chunks = rows * chunks_per_row, stride = (int64_t)gridDim.x * kQThreads;
  for (int64_t chunk = (int64_t)blockIdx.x * kQThreads + threadIdx.x; chunk < chunks; chunk += stride) {
    int64_t row;
    int32_t col;
    const float s = scale[tile_of_chunk(chunk, chunks_per_row, t_r, t_c, tiles_per_row, &row, &col)];
    const float sv[8] = {s, s, s, s, s, s, s, s};
    float v[8];
    load8<EX>(x + (row * cols + col) * (XB / 8), v);
    *reinterpret_cast<i32x2*>(q + row * cols + col) = quantize8<EQ>(v, sv, qmax);
  }
}

template <int EX>
int32_t launch_for_x(const void* x, void* q, float* scale, int64_t rows, int64_t cols, int64_t t_r, int64_t t_c,
                     int32_t q_dtype, QuantRange qmax, hipStream_t stream) {
  const auto* xb = static_cast<const unsigned char*>(x);
  auto* qb = static_cast<unsigned char*>(q);
  if (t_r == 1) {
    const int chunks = (int)(t_c / 8);
    const int L = (chunks < 64 && (chunks & (chunks - 1)) == 0) ? chunks : 64;
    const int64_t tiles = rows * (cols / t_c);
    const int64_t waves = (tiles + (64 / L) - 1) / (64 / L);
    int64_t grid = (waves + 3) / 4;
    if (grid > 256 * 16) grid = 256 * 16;
    if (grid < 1) grid = 1;
    if (q_dtype == TKX_I8)
      quantize_rows_kernel<EX, kEI8><<<dim3((unsigned)grid), dim3(kQThreads), 0, stream>>>(xb, qb, scale, rows, (int32_t)cols, (int32_t)t_c, L, qmax);
    else
      quantize_rows_kernel<EX, kEF8><<<dim3((unsigned)grid), dim3(kQThreads), 0, stream>>>(xb, qb, scale, rows, (int32_t)cols, (int32_t)t_c, L, qmax);
  } else if (t_c != 1 && !((t_c & (t_c - 1)) == 0 && t_c >= 8 && t_c <= 256)) {
    const int64_t num_tiles = (rows / t_r) * (cols / t_c), chunks = rows * (cols / 8);
    int64_t grid = (chunks + kQThreads - 1) / kQThreads;
    if (grid > 256 * 32) grid = 256 * 32;
    int64_t small = (num_tiles + 255) / 256;
    if (small > 1024) small = 1024;
    tile_slots_clear_kernel<<<dim3((unsigned)small), dim3(256), 0, stream>>>(scale, num_tiles);
    tile_absmax_kernel<EX><<<dim3((unsigned)grid), dim3(kQThreads), 0, stream>>>(xb, scale, rows, (int32_t)cols, (int32_t)t_r, (int32_t)t_c);
    tile_scale_kernel<<<dim3((unsigned)small), dim3(256), 0, stream>>>(scale, num_tiles, qmax);
    if (q_dtype == TKX_I8)
      quantize_tiles_kernel<EX, kEI8><<<dim3((unsigned)grid), dim3(kQThreads), 0, stream>>>(xb, qb, scale, rows, (int32_t)cols, (int32_t)t_r, (int32_t)t_c, qmax);
    else
      quantize_tiles_kernel<EX, kEF8><<<dim3((unsigned)grid), dim3(kQThreads), 0, stream>>>(xb, qb, scale, rows, (int32_t)cols, (int32_t)t_r, (int32_t)t_c, qmax);
  } else {
    const int64_t grid = (rows / t_r) * ((cols + 255) / 256);
    if (grid > 0x7fffffffLL) return set_error(TKX_ERR_UNSUPPORTED, "too many tiles");
    if (q_dtype == TKX_I8)
      quantize_blocks_kernel<EX, kEI8><<<dim3((unsigned)grid), dim3(kQThreads), 0, stream>>>(xb, qb, scale, rows, (int32_t)cols, (int32_t)t_r, (int32_t)t_c, qmax);
    else
      quantize_blocks_kernel<EX, kEF8><<<dim3((unsigned)grid), dim3(kQThreads), 0, stream>>>(xb, qb, scale, rows, (int32_t)cols, (int32_t)t_r, (int32_t)t_c, qmax);
  }
  TKX_HIP_CHECK(hipGetLastError());
  return TKX_OK;
}

}  // namespace

int32_t launch_quantize(const void* x, void* q, float* scale, int64_t rows, int64_t cols, int64_t t_r, int64_t t_c,
                        int32_t x_dtype, int32_t q_dtype, QuantRange qmax, hipStream_t stream) {
  if (x_dtype == TKX_F32) return launch_for_x<kEF32>(x, q, scale, rows, cols, t_r, t_c, q_dtype, qmax, stream);
  if (x_dtype == TKX_BF16) return launch_for_x<kEBF16>(x, q, scale, rows, cols, t_r, t_c, q_dtype, qmax, stream);
  return launch_for_x<kEF16>(x, q, scale, rows, cols, t_r, t_c, q_dtype, qmax, stream);
}

}  // namespace tkx
