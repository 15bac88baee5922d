// Shared declarations of the gfx950 ragged-dot library (host + device).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tkx_ragged_dot.h"

namespace tkx {

// ---- workspace layout (int32 words) -----------------------------------------------------------
// [0] num_tasks  [1] total_rows (end of the last group)  [2] rows before the first group  [kWsHeader ..) group_offsets[G+1]  then eight task arrays of
// tid_size words each (group_id, block_start, actual_start, actual_end, start_within_block,
// actual_size, span_first, span_width); every array starts on a 64-word boundary. The last two
// are not part of the reference's schedule: they cut each group's tasks into spans of at most
// grid_tile_width tasks (first task and width of the span a task belongs to), which is the unit
// the GEMM launch order walks n-panel by n-panel.
constexpr int64_t kWsHeader = 64;

struct WsLayout {
  int64_t offsets;   // word offset of group_offsets
  int64_t task[8];   // word offsets of the task arrays
  int64_t split_counters;  // word offset of kSplitUnits arrival counters (tiled kernels with split_k > 1); the
                           // scheduler kernel clears them in every call
  int64_t words;     // total words (the partial tiles of a split launch lie behind them)
  int32_t tid_size;
};

// Tiled kernels with split_k > 1: the tiles of the last, partial round of workgroups are cut along the contraction
// into parts, at most this many parts in all (one per CU of a 256-CU device).
constexpr int32_t kSplitUnits = 256;

inline int64_t round_up64(int64_t x) { return (x + 63) / 64 * 64; }

inline WsLayout ws_layout(int64_t m, int64_t G, int32_t block_m) {
  WsLayout L;
  L.tid_size = (int32_t)((m + block_m - 1) / block_m + G - 1);
  if (L.tid_size < 1) L.tid_size = 1;
  int64_t w = kWsHeader;
  L.offsets = w;
  w += round_up64(G + 1);
  for (int i = 0; i < 8; ++i) {
    L.task[i] = w;
    w += round_up64(L.tid_size);
  }
  L.split_counters = w;
  w += kSplitUnits;
  L.words = w;
  return L;
}

// ---- error reporting ----------------------------------------------------------------------------
int32_t set_error(int32_t code, const char* fmt, ...);

#define TKX_HIP_CHECK(expr)                                                                      \
  do {                                                                                           \
    hipError_t _e = (expr);                                                                      \
    if (_e != hipSuccess)                                                                        \
      return ::tkx::set_error(TKX_ERR_RUNTIME, "%s failed: %s", #expr, hipGetErrorString(_e));   \
  } while (0)

// ---- schedule -------------------------------------------------------------------------------------
// `group_offset` (device, one int32; null = 0): the G groups are entries [offset, offset + G) of the
// `num_global` group sizes.
int32_t launch_schedule(const int32_t* group_sizes, int64_t G, const int32_t* group_offset, int64_t num_global, int64_t m,
                        int32_t block_m, int32_t align_tile, int32_t span_width, int32_t* ws, const WsLayout& L,
                        hipStream_t stream);
int32_t device_compute_units(int* out);

// ---- grouped GEMM -----------------------------------------------------------------------------
// kFwdGlu = forward over weights [gate | up] ([g, k, 2 n_out]) with the epilogue act(gate) * up.
// kFwdSubK = forward over int8 weights whose scales change along k ([g, k / t_k, n]): the scale row of a
// k-step's block travels into LDS with the step and the weights are scaled while they are widened.
enum KernelMode { kFwd = 0, kDlhs = 1, kDrhs = 2, kFwdGlu = 3, kFwdSubK = 4 };

// fwd/dlhs launch order: the tile list is dealt to the 8 XCDs in chunks of this many consecutive
// tiles (the number of CUs of an XCD: one chunk is what an XCD runs at a time).
constexpr int32_t kXcdChunk = 32;

struct GemmParams {
  const void* A;
  const void* B;
  void* C;
  const float* a_scale;  // per A row, or null
  const float* b_scale;  // per (group, column of B), or null
  const float* b_bias;   // per (group, column of B), added after the scales, or null
  float* c_scale;        // out_dtype fp8: f32 [m_ext, n_ext / 128], one scale per (row, 128 columns) of the result
  const int32_t* ws;
  int64_t lda, ldb, ldc;            // leading dimensions, elements
  int64_t b_group_stride;           // elements between consecutive groups of B (fwd/dlhs)
  int64_t c_group_stride;           // elements between consecutive groups of C (drhs)
  int32_t m_ext, n_ext, k_ext;      // extents of the C rows, C columns and the contraction
  int32_t nb_ext;                   // columns of B (fwd/dlhs): n_ext, or 2 * n_ext for kFwdGlu
  int32_t num_groups;
  int32_t n_tiles, m_tiles;         // tiles along C columns; along C rows (drhs only)
  int32_t real_slots;               // fwd/dlhs: workgroups that may own a task tile (multiple of 8 * kXcdChunk)
  int32_t zero_wgs;                 // fwd/dlhs: workgroups after those that clear the rows of no group
  // Split of the last round (fwd/dlhs, split_k > 1): the launch's tiles beyond the last multiple of `split_cus` are
  // cut along the contraction into floor(split_cus / their number) parts, at most split_k; part 0 belongs to the
  // tile's own workgroup, the others to workgroups behind the zeroing ones. f32 partial tiles in split_partials
  // ([unit][BM * BN]), arrival counters at ws[ws_split_counters + tile].
  int32_t split_k, split_cus, ws_split_counters;
  float* split_partials;
  int32_t tid_size;                 // fwd/dlhs: slots of the schedule's task arrays
  int32_t grid_tile_width;
  int32_t out_dtype, activation;
  int32_t scale_blocks, log2_block_rows;  // kFwdSubK: b_scale is [g, scale_blocks, n]; rows of k per block = 1 << log2
  int32_t ws_offsets, ws_gid, ws_bstart, ws_astart, ws_aend, ws_span_first, ws_span_width;  // word offsets into ws
};

struct Variant {
  int32_t mode;  // KernelMode
  int32_t a_dtype, b_dtype;
  int32_t block_m, block_n, block_k, waves_m, waves_n, num_stages;
  int32_t smem_bytes;
  const void* fn;  // __global__ void (*)(GemmParams)
  int32_t split_b; // > 0: the split pipeline (that many B stages of block_k / 2; num_stages A stages of block_k)
  const void* fn_fp8_out;  // the same kernel storing fp8 with one scale per (row, 128 columns) (GemmParams::c_scale), or null
  const void* fn_split;    // the same kernel splitting the tiles of the last round along the contraction (GemmParams::split_k), or null
};

// ---- decode (small-m streaming kernel; int8 or 16-bit weights) -----------------------------------
constexpr int32_t kDecodeBlockM = 16, kDecodeBlockN = 128, kDecodeBlockK = 32, kDecodeWaves = 4, kDecodeStages = 4;
constexpr int32_t kDecodeWideBlockN = 256;  // int8 weights with per-column scales only
// `scale_blocks`: the scale is [G, scale_blocks, n]; 1 = one scale per (group, column).
// `block_n`: output columns per workgroup, kDecodeBlockN or kDecodeWideBlockN.
// `depth`: steps of loads in flight per wave. `split_k`: workgroups that share the contraction of one
// (group, column tile); above 1, `split_workspace` holds decode_split_workspace_words words whose first
// decode_split_counter_words are zero on entry (and again on exit). `persistent` > 0: the form in which the
// workgroups of empty groups take a share of the non-empty tiles' weight bytes; `split_workspace` then holds
// decode_persistent_workspace_words words with the same zeroed counter block in front.
bool decode_supported(int32_t lhs_dtype, int32_t rhs_dtype, int64_t m, int64_t k, int64_t n, int64_t G,
                      int64_t scale_blocks, int32_t block_n, int32_t depth, int32_t split_k);
bool decode_persistent_supported(int32_t lhs_dtype, int32_t rhs_dtype, int64_t m, int64_t k, int64_t n, int64_t G,
                                 int64_t scale_blocks, int32_t block_n, int32_t depth);
int64_t decode_persistent_workspace_words();
int64_t decode_split_counter_words();
int32_t launch_clear_decode_counters(int32_t* workspace, hipStream_t stream);
int64_t decode_split_workspace_words(int64_t m, int64_t n, int32_t split_k);
int32_t launch_decode(const void* lhs, const void* rhs, const float* scale, const int32_t* group_sizes, void* out,
                      int64_t m, int64_t k, int64_t n, int64_t G, int32_t rhs_dtype, int32_t out_dtype,
                      int32_t activation, int32_t depth, int64_t scale_blocks, int32_t block_n,
                      const int32_t* group_offset, int64_t num_global, int32_t split_k, int32_t persistent,
                      int32_t* split_workspace, hipStream_t stream);

// ---- packed int4 (TKX_I4X2) <-> int8: `packed_rows` rows of n bytes against 2 * packed_rows rows of n values ----
int32_t launch_int4_repack(const void* in, void* out, int64_t packed_rows, int64_t n, bool unpack, hipStream_t stream);
int32_t launch_row_sums_fp8(const void* x, float* sums, int64_t rows, int64_t n, bool per_128, hipStream_t stream);

// ---- dequantisation of int8 weights with sub-channel scales to bf16 ------------------------------
// out[r, c] = q[r, c] * scale[r / t_r, c / t_c]; q int8 or fp8 (e4m3fn), out bf16; t_c is 1 or a multiple of 16.
// `zero_point` (f32, shaped like the scale, or null): out = (q - zero_point) * scale.
int32_t launch_dequant(const void* q, const float* scale, const float* zero_point, void* out, int64_t rows, int64_t n,
                       int64_t t_r, int64_t t_c, int32_t q_dtype, hipStream_t stream);

// ---- absmax quantisation to int8 / fp8 with block scales (the inverse pass) -------------------------
// scale[R, C] = absmax of tile (R, C) / bound (1 for an all-zero tile); q = convert(clip(x / scale)). x f32, bf16 or f16.
// `bound`: what the tile's absmax is divided by; values are clipped to [lo, hi] after the division.
struct QuantRange { float bound, lo, hi; };
int32_t launch_quantize(const void* x, void* q, float* scale, int64_t rows, int64_t cols, int64_t t_r, int64_t t_c,
                        int32_t x_dtype, int32_t q_dtype, QuantRange range, hipStream_t stream);

// ---- row gather with optional mask, weight and reduction (token permute / un-permute) -------------
int32_t launch_gather_rows(const void* x, const int32_t* indices, const float* weights, const unsigned char* valid,
                           const int32_t* start, const int32_t* end, void* out, int64_t in_rows, int64_t out_rows,
                           int64_t hidden, int64_t reduce, int32_t dtype, hipStream_t stream);

// Each dtype family registers its variants from its own translation unit.
const Variant* variants_bf16(int* count);
const Variant* variants_f16(int* count);
const Variant* variants_f32(int* count);
const Variant* variants_f8(int* count);
const Variant* variants_i8w(int* count);
const Variant* variants_i4w(int* count);

}  // namespace tkx
