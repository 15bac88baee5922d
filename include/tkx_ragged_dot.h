/* C ABI of the gfx950 (MI355X) ragged-dot library, libtkx_ragged_dot.so.
 *
 * This is the drop-in boundary for `implementation="hip"` of tokamax.ragged_dot.  Every entry point
 * takes plain device pointers, sizes and a HIP stream; none of them allocates, frees, synchronises
 * or touches any stream other than the one passed in, so they can be bound from ctypes, cgo-style
 * FFIs or an XLA FFI handler alike.  Return value: 0 on success, a TKX_ERR_* code otherwise
 * (tkx_last_error() then holds a thread-local message).  TKX_ERR_UNSUPPORTED is the C-side twin of
 * the reference's `NotImplementedError`: the caller may fall through to another implementation.
 *
 * Reference interfaces replaced (paths relative to the openxla/tokamax tree):
 *   tkx_ragged_dot_schedule     tokamax/_src/ops/ragged_dot/pallas_mosaic_gpu_common.py:87-151
 *                               (GroupInfo.create_aligned) + the offsets of :119-121
 *   tkx_ragged_dot_fwd          tokamax/_src/ops/ragged_dot/base.py:291-360 (RaggedDot._fwd) as
 *                               dispatched by pallas_mosaic_gpu.py:103-244, for
 *                               DEFAULT_RAGGED_DOT_DIM_NUMS (base.py:40-44) and
 *                               TRANS_RHS_RAGGED_DOT_DIM_NUMS (base.py:45-49, the dlhs of base.py:434-446)
 *   tkx_ragged_dot_fwd_fused    the `rhs_bias` and `fuse_gateup_activation` arguments of RaggedDot
 *                               (base.py:205-217, :242-245): ragged_dot(lhs, rhs) + rhs_bias, and
 *                               activate(tmp[:, :n]) * tmp[:, n:] with tmp = ragged_dot(lhs, [gate, up])
 *   tkx_ragged_dot_drhs         RAGGED_CONTRACTING_DOT_DIM_NUMS (base.py:50-54), the drhs of
 *                               base.py:448-461; kernel counterpart pallas_mosaic_gpu_kernel_sm90.py:184-285
 *   tkx_dequantize_weights,     quantization.py:80-83 (as_array: qvalue * scale with tile-repeat
 *   tkx_dequantize              broadcasting) for int8 / fp8 operands with sub-channel scales
 *   tkx_dequantize_zero_point   quantization.py:85-93 (operands with a zero point are dequantised first)
 *   tkx_quantize                quantization.py:65-78 (AsQArray.as_qarray: absmax quantisation on the fly)
 *   TkxConfig                   pallas_mosaic_gpu_common.py:45-73 (Config)
 */
#ifndef TKX_RAGGED_DOT_H_
#define TKX_RAGGED_DOT_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* tkx_stream_t; /* a hipStream_t */

enum TkxStatus {
  TKX_OK = 0,
  TKX_ERR_INVALID = 1,     /* bad argument (the reference raises ValueError) */
  TKX_ERR_UNSUPPORTED = 2, /* valid but not implemented here (the reference raises NotImplementedError) */
  TKX_ERR_RUNTIME = 3      /* HIP launch/runtime failure */
};

enum TkxDtype {
  TKX_F32 = 0,
  TKX_BF16 = 1,
  TKX_F16 = 2,
  TKX_F8E4M3FN = 3, /* OCP float8_e4m3fn */
  TKX_I8 = 4,
  TKX_I4X2 = 5 /* signed 4-bit integers, two to a byte along the contraction axis: byte [g, kk, c] of an rhs
                  [G, k/2, n] holds k = 2 kk in bits 0-3 and k = 2 kk + 1 in bits 4-7 (two's complement). Taken as the
                  rhs of a bf16 lhs in the default mode by the streaming small-m kernel (block_m == 16, block_n == 128)
                  and by tiled forward variants of their own (plain, gate-up fusion, scales per k-block; k % block_k
                  == 0; listed by tkx_ragged_dot_variant), and as the rhs of an fp8 lhs by the variants described
                  at tkx_row_sums_fp8 and of an int8 lhs by plain and per-k-block-scale variants (scales as for
                  int8 x int8; pallas_mosaic_gpu_kernel_sm100_i8_quant.py:114-190); tkx_unpack_int4 turns it into TKX_I8 for everything else. The reference defines no packed layout (its int4 is jnp.int4; its sm90 kernels
                  read int4 weights in pallas_mosaic_gpu_kernel_sm90_quant.py:46-387). */
};

enum TkxMode {
  TKX_MODE_DEFAULT = 0,  /* out[m,n] = lhs[m,k] . rhs[g,k,n]              (base.py:40-44) */
  TKX_MODE_TRANS_RHS = 1 /* out[m,k] = lhs[m,n] . rhs[g,k,n]^T  (dlhs)    (base.py:45-49) */
};

enum TkxActivation { TKX_ACT_NONE = 0, TKX_ACT_RELU = 1, TKX_ACT_TANH = 2, TKX_ACT_SILU = 3, TKX_ACT_GELU_TANH = 4,
                     TKX_ACT_SIGMOID = 5,
                     /* Gate-up fusion only (experimental/gmm_v2/gmm_v2.py:29-50): both clip gate from above and up
                      * from both sides at a limit first. SWIGLU_OAI (limit 7): (up + 1) * gate * sigmoid(1.702 gate);
                      * SILU_CLAMP (limit 10): silu(gate) * up. */
                     TKX_ACT_SWIGLU_OAI = 6, TKX_ACT_SILU_CLAMP = 7 };

/* Tunables; the gfx950 counterpart of the reference's Config (pallas_mosaic_gpu_common.py:45-73).
 * (block_m, block_n, block_k, waves_m, waves_n, num_stages) must name a compiled kernel variant
 * (see tkx_ragged_dot_num_variants / tkx_ragged_dot_variant). */
typedef struct TkxConfig {
  int32_t block_m;         /* rows of lhs per task (multiple of 8) */
  int32_t block_n;         /* output columns per tile */
  int32_t block_k;         /* contraction elements per LDS stage */
  int32_t waves_m;         /* wavefronts along m in a workgroup */
  int32_t waves_n;         /* wavefronts along n in a workgroup */
  int32_t grid_tile_width; /* most m-tasks (of one group) that share an n-panel in launch order (L2 reuse);
                              unused by the streaming small-m kernel (block_m == 16) */
  int32_t align_tile;      /* task starts are aligned down to this many rows (reference default 8) */
  int32_t num_stages;      /* LDS stages of block_k contraction elements kept in flight */
  int32_t split_k;         /* workgroups that share the contraction of one output tile (the reference's split_k,
                              pallas_mosaic_gpu_common.py:53, pallas_triton.py:41-48). 0 and 1: no split. Above 1, on the
                              streaming small-m kernel (block_m == 16, block_n == 128, num_stages <= 4, k a multiple of
                              128 * split_k * num_stages): every tile is split, and `workspace` then is
                              tkx_ragged_dot_decode_workspace_bytes long with its first
                              tkx_ragged_dot_decode_counter_bytes ZERO on entry; the call leaves them zero, so a caller
                              that keeps one workspace per stream clears it once. Above 1 (at most 16), on a tiled
                              kernel (plain forward and TRANS_RHS; no gate-up fusion, scales per k-block or quantised
                              result): only the tiles of the launch's last, partial round of workgroups are split, into
                              floor(CUs / their number) parts, at most split_k, so that a launch of 1.25 rounds costs
                              1.25 rounds instead of 2; `workspace` then is tkx_ragged_dot_split_workspace_bytes long and
                              needs no clearing (the schedule kernel clears the counters). Parts are added in the order
                              of their index whoever arrives last: results are reproducible run to run. */
  int32_t persistent;      /* the reference's `persistent` (pallas_mosaic_gpu_common.py:55): resident workgroups that share
                              the work out evenly instead of one workgroup per tile and nothing else. 0: off. 1 (the
                              streaming small-m kernel: block_m == 16, block_n == 128, num_stages <= 4, one scale per
                              (group, column), num_groups <= 256, at most 1024 (group, column tile) pairs, k % 32 == 0,
                              split_k <= 1): the workgroups of EMPTY groups stay and contract a share of the non-empty
                              tiles' weights, so that every workgroup streams about the same number of bytes; a tile's
                              parts meet through the workspace, which then is
                              tkx_ragged_dot_decode_persistent_workspace_bytes long with its first
                              tkx_ragged_dot_decode_counter_bytes(2) ZERO on entry (left zero on exit, like split_k).
                              Takes effect when the device holds the whole grid at once and no group has more than 16
                              rows (decided per launch; otherwise the launch runs as with 0). */
} TkxConfig;

/* Library / ABI version (major*1000 + minor). A change of the major number means that structs passed by pointer
 * changed size: 2000: TkxConfig gained `persistent` (after `split_k`, which 1001 added); a caller built against an
 * older header must be rebuilt (the library reads sizeof(TkxConfig) bytes of the config it is handed). */
int32_t tkx_version(void);

/* Thread-local message for the last non-zero status returned on this thread. */
const char* tkx_last_error(void);

/* Workspace of the streaming small-m kernel with the contraction split over split_k workgroups per output tile:
 * arrival counters (one int32 per (group, column tile); the counter bytes come first and must be zero on entry),
 * then the partial sums f32[split_k, m, n]. Both are 0 for split_k <= 1. The counters take 256 KiB whatever the
 * shapes (so calls of any shapes can share a workspace that was cleared once), which limits
 * num_groups * cdiv(n, 128) to 65536. The partial sums are added in the order of the split index whichever
 * workgroup arrives last, so results are reproducible run to run. */
int64_t tkx_ragged_dot_decode_workspace_bytes(int64_t m, int64_t n, int32_t split_k);
int64_t tkx_ragged_dot_decode_counter_bytes(int32_t split_k);

/* Workspace of the streaming small-m kernel in its persistent form (TkxConfig.persistent = 1), whatever the shapes:
 * the same 256 KiB counter block (zero on entry, zero on exit), then four partial tiles (16 x 128 f32) for each of at
 * most 1024 workgroups (32.25 MiB in all). A workspace serves split_k and persistent calls alike, one call at a time.
 * The parts of a tile are added in a fixed order whenever they arrive: results are reproducible run to run (they
 * differ in the last bits from the plain kernel's, which cuts the contraction elsewhere). */
int64_t tkx_ragged_dot_decode_persistent_workspace_bytes(void);

/* Clears the counter block (the first tkx_ragged_dot_decode_counter_bytes(2) bytes) of such a workspace with a small
 * fill kernel on `stream`: for callers whose workspace is not theirs to keep between calls (an XLA FFI handler gets a
 * fresh, uninitialised result buffer per call) and for code under graph capture. No counterpart in the reference. */
int32_t tkx_ragged_dot_decode_clear_counters(void* workspace, tkx_stream_t stream);

/* Number of task slots the schedule uses for (m, G, block_m): cdiv(m, block_m) + G - 1
 * (pallas_mosaic_gpu_kernel_sm90.py:54). */
int64_t tkx_ragged_dot_tid_size(int64_t m, int64_t num_groups, int32_t block_m);

/* Bytes of device workspace needed by schedule/fwd/drhs for these sizes (int32 arrays, 256-aligned). */
int64_t tkx_ragged_dot_workspace_bytes(int64_t m, int64_t num_groups, int32_t block_m);

/* Bytes of workspace of a tiled forward / TRANS_RHS call with config->split_k > 1: the schedule arrays, then one f32
 * partial tile (block_m x block_n) for each of at most 256 parts. */
int64_t tkx_ragged_dot_split_workspace_bytes(int64_t m, int64_t num_groups, int32_t block_m, int32_t block_n);

/* Word offsets (int32 units) inside the workspace, for callers/tests that read the schedule back:
 * which = 0 num_tasks (1 word), 1 total_rows (1 word), 2 group_offsets (G+1 words),
 * 3..8 = group_id, block_start, actual_start, actual_end, start_within_block, actual_size
 * (tid_size words each); 9, 10 = span_first, span_width (tid_size words each): the first task and
 * the number of tasks of the launch-order span a task belongs to (each group's tasks are cut into
 * spans of at most grid_tile_width tasks; tkx_ragged_dot_schedule itself uses width 1).
 * Returns -1 for an unknown `which`. */
int64_t tkx_ragged_dot_workspace_offset(int64_t m, int64_t num_groups, int32_t block_m, int32_t which);

/* Part (1): group-offset prefix sum + tile schedule, one small kernel on `stream`.
 * group_sizes: device int32[G] (negative entries count as 0). Fills `workspace`. */
int32_t tkx_ragged_dot_schedule(const int32_t* group_sizes, int64_t num_groups, int64_t m, int32_t block_m,
                                int32_t align_tile, void* workspace, tkx_stream_t stream);

/* Parts (2),(3),(4-dlhs): grouped GEMM over the rows of each group.
 *   mode DEFAULT:   lhs [m,k] row-major, rhs [G,k,n] row-major, out [m,n]
 *   mode TRANS_RHS: lhs [m,n] row-major, rhs [G,k,n] row-major, out [m,k]  (rhs read transposed in-kernel)
 * lhs_scale: f32[m] per-row scale or NULL; rhs_scale: f32[G,n] per-(group, column) scale or NULL
 * (both applied to the f32 accumulator in the epilogue; DEFAULT mode only).
 * Supported (lhs_dtype, rhs_dtype): (f32,f32) (bf16,bf16) (f16,f16) (f8e4m3fn,f8e4m3fn) (bf16,i8), and
 * (bf16,f8e4m3fn) with an rhs scale and (i8,i8) with both scales, in DEFAULT mode.
 * out_dtype: f32, bf16 or f16. Rows >= sum(group_sizes) of `out` are set to zero.
 * Runs the schedule kernel itself (workspace must hold tkx_ragged_dot_workspace_bytes bytes). */
int32_t tkx_ragged_dot_fwd(const void* lhs, const void* rhs, const int32_t* group_sizes,
                           const float* lhs_scale, const float* rhs_scale, void* out, void* workspace,
                           int64_t m, int64_t k, int64_t n, int64_t num_groups, int32_t lhs_dtype,
                           int32_t rhs_dtype, int32_t out_dtype, int32_t mode, int32_t activation,
                           const TkxConfig* config, tkx_stream_t stream);

/* tkx_ragged_dot_fwd (default mode) with the result quantised in the kernel's epilogue: out is fp8 (e4m3fn) [m, n] and
 * out_scale f32 [m, n / 128], one scale per (row, 128 columns) = absmax / 448 (1 for a run of zeros); values are
 * multiplied by the reciprocal of their scale and converted with saturation, after the operand scales and the
 * activation: the arithmetic of the fused output quantisation of pallas_mosaic_gpu_kernel_sm100_fp8_quant.py:797-824
 * (`q = acc * (1.0 / out_scale)`), with the (1, 128) tile of pallas_mosaic_gpu_common.py:63-68. The scales are those of
 * tkx_ragged_dot_fwd with an f32 result followed by tkx_quantize; the values can differ from that pass, which divides,
 * by one fp8 step where a quotient lies on a rounding boundary.
 * n % 128 == 0; bf16 x bf16 and fp8 x fp8 tile variants whose wave columns tile 128 output columns (all the 256-column
 * ones); rows of no group come out as zeros with scale 1. TKX_ERR_UNSUPPORTED otherwise. */
int32_t tkx_ragged_dot_fwd_fp8_out(const void* lhs, const void* rhs, const int32_t* group_sizes, const float* lhs_scale,
                                   const float* rhs_scale, void* out, float* out_scale, void* workspace, int64_t m,
                                   int64_t k, int64_t n, int64_t num_groups, int32_t lhs_dtype, int32_t rhs_dtype,
                                   int32_t activation, const TkxConfig* config, tkx_stream_t stream);

/* tkx_ragged_dot_fwd for callers that cannot hand over a workspace they allocated: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc. It has no counterpart in the reference (XLA owns every buffer
 * there). Same arguments and results as tkx_ragged_dot_fwd, without `workspace`: the schedule arrays live in a
 * 256 KiB device array inside the library (one copy per GPU, held until the process ends), which limits
 * tkx_ragged_dot_workspace_bytes(m, num_groups, block_m) to 262144, i.e. about cdiv(m, block_m) + num_groups <= 8100;
 * larger problems return TKX_ERR_UNSUPPORTED, and so does config->split_k > 1 (its arrival counters need a workspace
 * that was cleared). The call allocates and frees nothing. All calls on one GPU share that
 * array: two of them that overlap in time (different streams or threads) race; calls on one stream are ordered.
 * The first call on a device looks the array's address up (hipGetSymbolAddress), and the first call of a kernel on a
 * device raises that kernel's limit of dynamic LDS (hipFuncSetAttribute): both are remembered in fixed tables (no host
 * allocation either) and should happen outside capture, i.e. make one eager call per (device, config) first. */
int32_t tkx_ragged_dot_fwd_static_workspace(const void* lhs, const void* rhs, const int32_t* group_sizes,
                                            const float* lhs_scale, const float* rhs_scale, void* out, int64_t m,
                                            int64_t k, int64_t n, int64_t num_groups, int32_t lhs_dtype,
                                            int32_t rhs_dtype, int32_t out_dtype, int32_t mode, int32_t activation,
                                            const TkxConfig* config, tkx_stream_t stream);

/* Forward (mode DEFAULT) with the fused epilogue terms of base.py:205-217.
 *   rhs_bias: f32[G,n] added to the scaled accumulator, or NULL.
 *   gateup = 1: rhs is [G,k,n] with its columns [gate | up] (n/2 each) and out is [m, n/2] =
 *     act(lhs.gate + bias_gate) * (lhs.up + bias_up), `activation` naming act (NONE: the plain product); needs
 *     n % 16 == 0 (one-byte weights: n % 32 == 0, so that the up half starts on a 16-byte piece), k % block_k == 0 and a variant of mode 3 (see tkx_ragged_dot_variant; bf16 x bf16 and
 *     bf16 x int8 with one scale per (group, column)).
 *   gateup = 0: as tkx_ragged_dot_fwd plus the bias; `activation` applies to the biased result
 *   (TKX_ACT_SWIGLU_OAI and TKX_ACT_SILU_CLAMP need gateup = 1: TKX_ERR_INVALID otherwise).
 *   rhs_scale_blocks: rhs_scale is f32[G, rhs_scale_blocks, n], block b scaling the k rows
 *     [b * k/blocks, (b+1) * k/blocks) (scale tile (1, t_k, 1), pallas_mosaic_gpu_kernel_sm90_quant.py:91-97).
 *     1 = one scale per (group, column). int8 x int8 (any number of blocks; m % 4 == 0) and fp8 x fp8 with more
 *     than 1: lhs_scale is then f32[rhs_scale_blocks, m]
 *     (one scale per k-block and row), both operands' scales are folded in after every k-block (mode 4; m % 4 == 0).
 *     bf16 x fp8 weights run on the variants of mode 4 only, with any number
 *     of blocks. More than 1 (int8 or fp8 weights, k/blocks a power of two): taken by the
 *     streaming small-m kernel (k/blocks >= 32) and by the tiled variants of mode 4 (block_k divides k/blocks;
 *     256-column tiles), which multiply each k-block's scales in while they widen the weights, to the same bits
 *     as tkx_dequantize_weights followed by the bf16 kernels; for other block sizes widen the weights first.
 *   group_offset: device int32[1] or NULL (the `group_offset` argument of RaggedDot, base.py:238; semantics of
 *     experimental/gmm_v2/gmm_v2_test.py:44-101): `group_sizes` then has `num_group_sizes` entries, the
 *     `num_groups` groups of rhs are its entries [offset, offset + num_groups) (entries outside the array count
 *     as empty), and the rows of every other entry come out zero: the call of one expert-parallel shard. Read on
 *     the device, so the offset can change between replays of a captured graph. NULL: `num_group_sizes` is ignored.
 * The streaming small-m kernel (block_m == 16) takes neither a bias nor gate-up fusion. */
int32_t tkx_ragged_dot_fwd_fused(const void* lhs, const void* rhs, const int32_t* group_sizes,
                                 const int32_t* group_offset, const float* lhs_scale, const float* rhs_scale,
                                 const float* rhs_bias, void* out, void* workspace, int64_t m, int64_t k, int64_t n,
                                 int64_t num_groups, int64_t num_group_sizes, int64_t rhs_scale_blocks,
                                 int32_t lhs_dtype, int32_t rhs_dtype, int32_t out_dtype, int32_t activation,
                                 int32_t gateup, const TkxConfig* config, tkx_stream_t stream);

/* Part (4-drhs): out[G,k,n] = lhs[rows_g, k]^T . dout[rows_g, n], zeros for empty groups.
 * lhs [m,k], dout [m,n] row-major of `dtype` (f32/bf16/f16); out_dtype f32/bf16/f16.
 * Deterministic: one workgroup owns each output tile, no atomics. block_m/block_n of `config`
 * tile the (k, n) output; block_k rows of the ragged dimension are contracted per stage. */
int32_t tkx_ragged_dot_drhs(const void* lhs, const void* dout, const int32_t* group_sizes, void* out,
                            void* workspace, int64_t m, int64_t k, int64_t n, int64_t num_groups,
                            int32_t dtype, int32_t out_dtype, const TkxConfig* config, tkx_stream_t stream);

/* Weights with several scale blocks along k (the scale tile (1, t_k, 1) with t_k < k of
 * pallas_mosaic_gpu_kernel_sm90_quant.py:91-97; quantization.py:80-83 for the dequantisation):
 *   out[g, kk, c] = qvalue[g, kk, c] * scale[g, kk / scale_block_k, c]
 * qvalue int8 or fp8 (e4m3fn) [G,k,n], scale f32 [G, k / scale_block_k, n], out bf16 [G,k,n] (caller-owned);
 * the result feeds the bf16 kernels. (scale_block_k == k needs no such pass: tkx_ragged_dot_fwd applies
 * one scale per (group, column) in its epilogue.) One streaming kernel on `stream`. */
int32_t tkx_dequantize_weights(const void* qvalue, const float* scale, void* out, int64_t num_groups, int64_t k,
                               int64_t n, int64_t scale_block_k, int32_t q_dtype, int32_t out_dtype,
                               tkx_stream_t stream);

/* The same pass for any row-major quantised operand with block scales (quantization.py:80-83; the
 * k-subchannel scales xs[row, k_sub] and ws[g, k_sub, n] of pallas_mosaic_gpu_kernel_sm100_i8_quant.py:51-102):
 *   out[r, c] = qvalue[r, c] * scale[r / scale_block_rows, c / scale_block_cols]
 * qvalue int8 or fp8 (e4m3fn) [rows, cols], scale f32 [rows / scale_block_rows, cols / scale_block_cols], out bf16.
 * An lhs [m,k] with scale [m, k/t] is (rows, cols, blocks) = (m, k, 1 x t); weights [G,k,n] with scale
 * [G, k/t_k, n/t_n] are (G*k, n, t_k x t_n). cols % 16 == 0; scale_block_cols is 1 or a multiple of 16. */
int32_t tkx_dequantize(const void* qvalue, const float* scale, void* out, int64_t rows, int64_t cols,
                       int64_t scale_block_rows, int64_t scale_block_cols, int32_t q_dtype, int32_t out_dtype,
                       tkx_stream_t stream);

/* tkx_dequantize with a zero point (quantization.py:85-93 dequantises such operands before the kernels, which take
 * none): out[r, c] = (qvalue[r, c] - zero_point[R, C]) * scale[R, C], zero_point f32 shaped like the scale. */
int32_t tkx_dequantize_zero_point(const void* qvalue, const float* scale, const float* zero_point, void* out, int64_t rows,
                                  int64_t cols, int64_t scale_block_rows, int64_t scale_block_cols, int32_t q_dtype,
                                  int32_t out_dtype, tkx_stream_t stream);

/* Packed int4 (TKX_I4X2) to int8 storage and back, for [.., rows, cols] arrays viewed as 2-D: `packed` has
 * packed_rows rows of `cols` bytes, the int8 side 2 * packed_rows rows of `cols` values; value row 2 r sits in bits 0-3
 * of packed row r, value row 2 r + 1 in bits 4-7 (for an rhs [G, k, n] with even k: packed_rows = G * k / 2, cols = n).
 * tkx_pack_int4 keeps the low four bits of each value (values in [-8, 7] survive unchanged). cols % 16 == 0,
 * 16-byte aligned pointers. No counterpart in the reference, which holds int4 as jnp.int4 arrays. */
int32_t tkx_unpack_int4(const void* packed, void* out, int64_t packed_rows, int64_t cols, tkx_stream_t stream);
int32_t tkx_pack_int4(const void* values, void* packed, int64_t packed_rows, int64_t cols, tkx_stream_t stream);

/* Row sums of an fp8 (e4m3fn) matrix [rows, cols] in f32: chunk_cols == cols: sums[r] = sum_c x[r, c]; chunk_cols ==
 * 128 (cols % 128 == 0): sums[c / 128][r], one per run of 128 columns. cols % 16 == 0, x 16-byte aligned.
 * The fp8 x packed-int4 forward (lhs TKX_F8E4M3FN, rhs TKX_I4X2, plain and gate-up forward variants with block_k = 128) takes them
 * behind the row scales, lhs_scale = f32[2, m]: it feeds weight w to the fp8 MFMAs as the e4m3 denormal (w + 8) / 512
 * and computes (512 acc - 8 sums[row]) * lhs_scale[row] * rhs_scale[group, col]. The reference's kernel packs the
 * sums with the activation scales the same way (pallas_mosaic_gpu_kernel_sm100_fp8_quant.py:258-300, 436-470).
 * With rhs scales per k-block (tkx_ragged_dot_fwd_fused, rhs_scale_blocks > 1; blocks of a power of two >= 128 rows;
 * m % 4 == 0): lhs_scale = f32[blocks + k / 128, m], the lhs scales per k-block followed by the row sums per 128
 * columns, and every 128-deep k-step's products are folded in as (512 part - 8 sums[step][row]) * lhs_scale[block][row]
 * * rhs_scale[group, block, col] (the per-subchannel form of the same reference kernel, :740-790). */
int32_t tkx_row_sums_fp8(const void* x, float* sums, int64_t rows, int64_t cols, int64_t chunk_cols, tkx_stream_t stream);

/* Quantisation on the fly (AsQArray.as_qarray, quantization.py:65-78: qwix.quantize with the "absmax" calibration), the
 * inverse of tkx_dequantize:
 *   scale[R, C] = max |x[r, c]| over the tile (R, C) / bound   (1 where the tile is all zero)
 *   qvalue[r, c] = convert(x[r, c] / scale[r / scale_block_rows, c / scale_block_cols])
 * `qmax`: the largest quantised magnitude, at most 127 (int8) or 448 (fp8 e4m3fn); 0 means that maximum (7 gives int4
 * values in int8 storage). `bound`: what the tile's absmax is divided by, in [qmax, qmax + 1]; 0 means qmax, the form the
 * reference writes out for fp8 (pallas_mosaic_gpu_kernel_sm100_fp8_quant.py:802-822) and for integers in its TPU kernels
 * (pallas_mosaic_tpu_kernel.py:267-277, experimental/gmm_v2/util.py:28-50: iinfo.max). qwix, the library behind
 * `AsQArray`, is not part of the reference tree; should its integer bound be 2^(bits-1) - 0.5 (127.5, 7.5), that is
 * `bound = qmax + 0.5` here (integer types only). convert rounds to nearest even and saturates at [-qmax, qmax], or at
 * [-qmax - 1, qmax] with a bound above qmax.
 * x f32, bf16 or f16 [rows, cols] row-major; qvalue int8 or fp8 [rows, cols]; scale f32
 * [rows / scale_block_rows, cols / scale_block_cols]. Tiles: one row tall and a multiple of 8 columns wide (an lhs with
 * one scale per row, scale_block_cols = cols, or per (row, k-block)); or several rows tall and 1 column or a multiple
 * of 8 columns wide (weights [g, k, n] as g * k rows: (k, 1) is one scale per (group, column), (t_k, 1) the scale tile
 * (1, t_k, 1), (128, 128) square blocks, (rows, cols) one scale for the whole array). Tiles of 8, 16, ... 256 columns
 * are reduced inside one workgroup; wider ones, and widths that are not a power of two, take three passes that collect
 * each tile's maximum in its `scale` slot with an atomic maximum (the result does not depend on the order).
 * cols % 8 == 0. */
int32_t tkx_quantize(const void* x, void* qvalue, float* scale, int64_t rows, int64_t cols, int64_t scale_block_rows,
                     int64_t scale_block_cols, int32_t x_dtype, int32_t q_dtype, float qmax, float bound,
                     tkx_stream_t stream);

/* The token permute / un-permute steps either side of the ragged dot in an MoE layer, one kernel:
 *   out[j, :] = sum over r < reduce_group_size of keep(g) * weights[g] * x[indices[g], :],  g = j * reduce_group_size + r
 * keep(g) = (start == NULL or start[0] <= indices[g] < end[0]) and (valid == NULL or valid[g] != 0).
 *   ragged_gather         (tokamax/_src/ops/ragged_gather/base.py:25-32): weights = valid = start = end = NULL, reduce 1
 *   ragged_scatter        (ragged_scatter/base.py:26-38): start/end given (device int32 scalars), reduce 1
 *   ragged_gather_reduce  (ragged_gather_reduce/base.py:26-40): weights f32[out_rows * reduce], valid bytes, reduce = R;
 *                         products and sums in f32, one rounding to `dtype`
 * x [in_rows, hidden], out [out_rows, hidden] of `dtype` (f32/bf16/f16), rows a multiple of 16 bytes;
 * indices int32[out_rows * reduce_group_size] (negative ones count from the end; what is then still outside [0, in_rows) is clamped). */
int32_t tkx_ragged_gather_rows(const void* x, const int32_t* indices, const float* weights, const uint8_t* valid,
                               const int32_t* start, const int32_t* end, void* out, int64_t in_rows, int64_t out_rows,
                               int64_t hidden, int64_t reduce_group_size, int32_t dtype, tkx_stream_t stream);

/* Enumerates compiled kernel variants, for the autotuner's search space.
 * kind: 0 = fwd/dlhs variants, 1 = drhs variants.  Returns the count; tkx_ragged_dot_variant fills
 * `config` (tile + wave fields), the dtype pair and the mode of variant `index` (0 = fwd, 1 = dlhs,
 * 2 = drhs, 3 = fwd with gate-up fusion, 4 = fwd over int8 weights with per-k-block scales), returning 0, or
 * TKX_ERR_INVALID. */
int32_t tkx_ragged_dot_num_variants(int32_t kind);
int32_t tkx_ragged_dot_variant(int32_t kind, int32_t index, TkxConfig* config, int32_t* lhs_dtype,
                               int32_t* rhs_dtype, int32_t* mode);

#ifdef __cplusplus
}
#endif
#endif /* TKX_RAGGED_DOT_H_ */
