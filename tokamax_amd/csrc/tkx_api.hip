// extern "C" entry points of libtkx_ragged_dot.so (declared in include/tkx_ragged_dot.h).
#include <cstdarg>
#include <cstdio>
#include <mutex>

#include "tkx_common.h"

// Schedule workspace of tkx_ragged_dot_fwd_static_workspace: one copy per GPU the library runs on, held until the
// process ends. In host code this name is only a handle for hipGetSymbolAddress; the device address it yields
// (one per device) is what kernels and copies take.
constexpr int64_t kScratchWords = 64 * 1024;  // 256 KiB of int32
static __device__ __align__(256) int32_t scratch[kScratchWords];

namespace tkx {

static thread_local char g_err[512] = "";

// Compute units of the current device (fixed table: no allocation after the library is loaded).
int32_t device_compute_units(int* out) {
  constexpr int kMaxDevices = 64;
  static std::mutex mu;
  static int count[kMaxDevices] = {};
  int dev = 0;
  TKX_HIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return set_error(TKX_ERR_UNSUPPORTED, "device ordinal %d out of range", dev);
  std::lock_guard<std::mutex> lock(mu);
  if (count[dev] == 0) {
    int cus = 0;
    TKX_HIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    if (cus < 1) return set_error(TKX_ERR_RUNTIME, "device reports %d compute units", cus);
    count[dev] = cus;
  }
  *out = count[dev];
  return TKX_OK;
}

int32_t set_error(int32_t code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

namespace {

// Every compiled variant, in one fixed table (filled once; nothing here allocates).
struct Registry {
  static constexpr int kCapacity = 256;
  Variant all_[kCapacity];
  int count_ = 0;
  void add(const Variant& v) {
    if (count_ < kCapacity) all_[count_++] = v;
  }
  void add(const Variant* v, int n) {
    for (int i = 0; i < n; ++i) add(v[i]);
  }
  const Variant* begin() const { return all_; }
  const Variant* end() const { return all_ + count_; }
  Registry() {
    int n = 0;
    const Variant* v;
    v = variants_bf16(&n); add(v, n);
    v = variants_f16(&n);  add(v, n);
    v = variants_f32(&n);  add(v, n);
    v = variants_f8(&n);   add(v, n);
    v = variants_i8w(&n);  add(v, n);
    v = variants_i4w(&n);  add(v, n);
    // The streaming small-m kernel is not a tile variant of the GEMM template; it is listed here
    // (fn == nullptr, num_stages = steps of loads in flight) so that configs can name it.
    for (int depth : {2, 4, 8})
      add({kFwd, TKX_BF16, TKX_I8, kDecodeBlockM, kDecodeBlockN, kDecodeBlockK, 1, kDecodeWaves, depth, 0, nullptr});
    for (int depth : {2, 4})
      add({kFwd, TKX_BF16, TKX_I8, kDecodeBlockM, kDecodeWideBlockN, kDecodeBlockK, 1, kDecodeWaves, depth, 0, nullptr});
    for (int depth : {2, 4})
      add({kFwd, TKX_BF16, TKX_F8E4M3FN, kDecodeBlockM, kDecodeBlockN, kDecodeBlockK, 1, kDecodeWaves, depth, 0, nullptr});
    for (int dtype : {TKX_BF16, TKX_F16})
      for (int depth : {2, 4})
        add({kFwd, dtype, dtype, kDecodeBlockM, kDecodeBlockN, kDecodeBlockK, 1, kDecodeWaves, depth, 0, nullptr});
    for (int depth : {2, 4, 8})  // packed int4 weights (their tiled kernels come with variants_i4w)
      add({kFwd, TKX_BF16, TKX_I4X2, kDecodeBlockM, kDecodeBlockN, kDecodeBlockK, 1, kDecodeWaves, depth, 0, nullptr});
  }
};

const Registry& registry() {
  static Registry r;
  return r;
}

const Variant* find_variant(int mode, int a_dtype, int b_dtype, const TkxConfig& c) {
  for (const Variant& v : registry())
    if (v.mode == mode && v.a_dtype == a_dtype && v.b_dtype == b_dtype && v.block_m == c.block_m &&
        v.block_n == c.block_n && v.block_k == c.block_k && v.waves_m == c.waves_m && v.waves_n == c.waves_n &&
        v.num_stages == c.num_stages)
      return &v;
  return nullptr;
}

int dtype_bytes(int d) { return d == TKX_F32 ? 4 : (d == TKX_BF16 || d == TKX_F16) ? 2 : 1; }

// Raises the dynamic-LDS limit of a kernel once per (device, kernel); remembered in a fixed table, so that no entry
// point touches the host heap.
int32_t prepare(const void* fn, int32_t smem_bytes) {
  struct Entry { int dev; const void* fn; };
  constexpr int kSlots = 2048;
  static std::mutex mu;
  static Entry done[kSlots];
  static int used = 0;
  int dev = 0;
  TKX_HIP_CHECK(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(mu);
  for (int i = 0; i < used; ++i)
    if (done[i].dev == dev && done[i].fn == fn) return TKX_OK;
  TKX_HIP_CHECK(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, smem_bytes));
  if (used < kSlots) done[used++] = {dev, fn};  // (a full table only means the attribute is set again)
  return TKX_OK;
}

int32_t launch(const Variant* v, const GemmParams& p, int64_t grid, hipStream_t stream) {
  const void* fn = p.c_scale != nullptr ? v->fn_fp8_out : p.split_k > 1 ? v->fn_split : v->fn;
  int32_t st = prepare(fn, v->smem_bytes);
  if (st != TKX_OK) return st;
  if (grid <= 0 || grid > 0x7fffffffLL) return set_error(TKX_ERR_INVALID, "grid size %lld out of range", (long long)grid);
  GemmParams params = p;
  void* args[] = {&params};
  const int threads = v->waves_m * v->waves_n * 64;
  TKX_HIP_CHECK(hipLaunchKernel(fn, dim3((unsigned)grid), dim3(threads), args, (size_t)v->smem_bytes, stream));
  return TKX_OK;
}

bool valid_out_dtype(int d) { return d == TKX_F32 || d == TKX_BF16 || d == TKX_F16; }

// Device address of `scratch` on the current device, looked up once per device (each GPU holds its own copy of
// the array at its own address). Fixed-size table: nothing here allocates.
int32_t scratch_address(int32_t** out) {
  constexpr int kMaxDevices = 64;
  static std::mutex mu;
  static int32_t* address[kMaxDevices] = {};
  int dev = 0;
  TKX_HIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return set_error(TKX_ERR_UNSUPPORTED, "device ordinal %d out of range", dev);
  std::lock_guard<std::mutex> lock(mu);
  if (address[dev] == nullptr) {
    void* ptr = nullptr;
    TKX_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (ptr == nullptr) return set_error(TKX_ERR_RUNTIME, "hipGetSymbolAddress returned a null address");
    address[dev] = static_cast<int32_t*>(ptr);
  }
  *out = address[dev];
  return TKX_OK;
}

}  // namespace
}  // namespace tkx

using namespace tkx;

extern "C" {

int32_t tkx_version(void) { return 2000; }

const char* tkx_last_error(void) { return g_err; }

int64_t tkx_ragged_dot_decode_workspace_bytes(int64_t m, int64_t n, int32_t split_k) {
  if (m < 0 || n < 1) return -1;
  return decode_split_workspace_words(m, n, split_k) * 4;
}

int64_t tkx_ragged_dot_decode_persistent_workspace_bytes(void) { return decode_persistent_workspace_words() * 4; }

int64_t tkx_ragged_dot_decode_counter_bytes(int32_t split_k) {
  return split_k > 1 ? decode_split_counter_words() * 4 : 0;
}

int32_t tkx_ragged_dot_decode_clear_counters(void* workspace, tkx_stream_t stream) {
  if (workspace == nullptr || (uintptr_t)workspace % 4 != 0) return set_error(TKX_ERR_INVALID, "null or misaligned workspace");
  return launch_clear_decode_counters(static_cast<int32_t*>(workspace), static_cast<hipStream_t>(stream));
}

int64_t tkx_ragged_dot_tid_size(int64_t m, int64_t num_groups, int32_t block_m) {
  if (m < 0 || num_groups < 1 || block_m < 1) return -1;
  return ws_layout(m, num_groups, block_m).tid_size;
}

int64_t tkx_ragged_dot_workspace_bytes(int64_t m, int64_t num_groups, int32_t block_m) {
  if (m < 0 || num_groups < 1 || block_m < 1) return -1;
  return ws_layout(m, num_groups, block_m).words * 4;
}

int64_t tkx_ragged_dot_split_workspace_bytes(int64_t m, int64_t num_groups, int32_t block_m, int32_t block_n) {
  if (m < 0 || num_groups < 1 || block_m < 1 || block_n < 1) return -1;
  return ws_layout(m, num_groups, block_m).words * 4 + (int64_t)kSplitUnits * block_m * block_n * 4;
}

int64_t tkx_ragged_dot_workspace_offset(int64_t m, int64_t num_groups, int32_t block_m, int32_t which) {
  if (m < 0 || num_groups < 1 || block_m < 1) return -1;
  const WsLayout L = ws_layout(m, num_groups, block_m);
  if (which == 0) return 0;
  if (which == 1) return 1;
  if (which == 2) return L.offsets;
  if (which >= 3 && which <= 10) return L.task[which - 3];
  return -1;
}

int32_t tkx_ragged_dot_schedule(const int32_t* group_sizes, int64_t num_groups, int64_t m, int32_t block_m,
                                int32_t align_tile, void* workspace, tkx_stream_t stream) {
  if (group_sizes == nullptr || workspace == nullptr) return set_error(TKX_ERR_INVALID, "null pointer argument");
  if (num_groups < 1 || m < 0) return set_error(TKX_ERR_INVALID, "bad sizes m=%lld G=%lld", (long long)m, (long long)num_groups);
  if (block_m < 1 || align_tile < 1) return set_error(TKX_ERR_INVALID, "block_m and align_tile must be positive");
  const WsLayout L = ws_layout(m, num_groups, block_m);
  return launch_schedule(group_sizes, num_groups, nullptr, num_groups, m, block_m, align_tile, 1,
                         static_cast<int32_t*>(workspace), L, static_cast<hipStream_t>(stream));
}

}  // extern "C"

namespace {
// Forward / dlhs launcher behind both public forward entry points. `gateup`: rhs is [g, k, n] =
// [gate | up] and out is [m, n/2] = act(lhs.gate + bias) * (lhs.up + bias), `activation` naming act.
// `group_offset` (device, one int32, or null) and `num_group_sizes`: the num_groups groups of rhs are
// entries [offset, offset + num_groups) of the num_group_sizes group sizes.
int32_t fwd_impl(const void* lhs, const void* rhs, const int32_t* group_sizes, const int32_t* group_offset,
                 const float* lhs_scale, const float* rhs_scale, const float* rhs_bias, void* out, void* workspace,
                 int64_t m, int64_t k, int64_t n, int64_t num_groups, int64_t num_group_sizes, int32_t lhs_dtype,
                 int32_t rhs_dtype, int32_t out_dtype, int32_t mode, int32_t activation, bool gateup,
                 int64_t rhs_scale_blocks, const TkxConfig* config, tkx_stream_t stream_, float* out_scale = nullptr) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (!lhs || !rhs || !group_sizes || !out || !workspace || !config)
    return set_error(TKX_ERR_INVALID, "null pointer argument");
  if (group_offset == nullptr) num_group_sizes = num_groups;
  if (num_group_sizes < 1 || num_group_sizes > 0x7fffffffLL)
    return set_error(TKX_ERR_INVALID, "bad number of group sizes %lld", (long long)num_group_sizes);
  if (m < 1 || k < 1 || n < 1 || num_groups < 1)
    return set_error(TKX_ERR_INVALID, "bad sizes m=%lld k=%lld n=%lld G=%lld", (long long)m, (long long)k,
                     (long long)n, (long long)num_groups);
  if (mode != TKX_MODE_DEFAULT && mode != TKX_MODE_TRANS_RHS) return set_error(TKX_ERR_INVALID, "bad mode %d", mode);
  if (out_scale != nullptr) {
    // fp8 output with one scale per (row, 128 columns), written by the kernel's epilogue.
    if (out_dtype != TKX_F8E4M3FN || mode != TKX_MODE_DEFAULT || gateup || n % 128 != 0 || (uintptr_t)out_scale % 4 != 0)
      return set_error(TKX_ERR_UNSUPPORTED, "a quantised result is fp8 (e4m3fn), default mode, no gate-up fusion, n %% 128 == 0");
  } else if (!valid_out_dtype(out_dtype)) {
    return set_error(TKX_ERR_UNSUPPORTED, "out dtype %d not supported", out_dtype);
  }
  if (activation < TKX_ACT_NONE || activation > TKX_ACT_SILU_CLAMP)
    return set_error(TKX_ERR_INVALID, "bad activation %d", activation);
  if (activation > TKX_ACT_SIGMOID && !gateup)
    return set_error(TKX_ERR_INVALID, "activation %d belongs to gate-up fusion", activation);
  // Per-lane byte offsets inside a tile are 32-bit: (256 rows) x (row bytes) must stay below 2^31.
  if (m > 0x7fffffffLL / 2 || k >= (1 << 21) || n >= (1 << 21))
    return set_error(TKX_ERR_UNSUPPORTED, "dimension too large");
  const TkxConfig& c = *config;
  if (c.block_m < 8 || c.block_m % 8 != 0) return set_error(TKX_ERR_INVALID, "block_m must be a positive multiple of 8");
  if (c.grid_tile_width < 1 || c.align_tile < 1) return set_error(TKX_ERR_INVALID, "grid_tile_width/align_tile must be >= 1");
  const bool dlhs = mode == TKX_MODE_TRANS_RHS;
  if (dlhs && (lhs_scale || rhs_scale)) return set_error(TKX_ERR_UNSUPPORTED, "scales are not supported with TRANS_RHS");
  if (dlhs && (rhs_bias || gateup)) return set_error(TKX_ERR_UNSUPPORTED, "bias and gate-up fusion need the default mode");
  if (gateup && (n % 16 != 0 || k % c.block_k != 0))
    return set_error(TKX_ERR_UNSUPPORTED, "gate-up fusion needs n %% 16 == 0 and k %% block_k == 0 (k=%lld n=%lld)",
                     (long long)k, (long long)n);
  // (the up half of a weight row starts n / 2 elements in: whole 16-byte pieces of one-byte weights are 16 columns)
  if (gateup && rhs_dtype != TKX_BF16 && rhs_dtype != TKX_F16 && rhs_dtype != TKX_F32 && (n / 2) % 16 != 0)
    return set_error(TKX_ERR_UNSUPPORTED, "gate-up fusion over one-byte weights needs n %% 32 == 0 (n=%lld)", (long long)n);
  if (rhs_bias && (uintptr_t)rhs_bias % 16 != 0) return set_error(TKX_ERR_UNSUPPORTED, "pointers must be 16-byte aligned");
  // Scales that change along k: the streaming small-m kernel (block_m == 16) takes them itself; the tiled
  // kernels have variants of their own (kFwdSubK) that carry the scale rows through LDS.
  // bf16 activations x fp8 weights exist in that form only, also with a single scale block.
  const bool a16w8f = lhs_dtype == TKX_BF16 && rhs_dtype == TKX_F8E4M3FN;
  if (a16w8f && (rhs_scale == nullptr || dlhs))
    return set_error(TKX_ERR_UNSUPPORTED, "bf16 x fp8 weights: default mode with an rhs scale only");
  // int8 x int8 likewise (the int8 MFMA kernels fold both operands' scales in per k-block).
  const bool a8w8 = lhs_dtype == TKX_I8 && (rhs_dtype == TKX_I8 || rhs_dtype == TKX_I4X2);
  if (a8w8 && (rhs_scale == nullptr || lhs_scale == nullptr || dlhs))
    return set_error(TKX_ERR_UNSUPPORTED, "int8 x int8 (or packed int4): default mode with lhs and rhs scales only");
  const bool subk = rhs_scale != nullptr && (rhs_scale_blocks != 1 || a16w8f) && !dlhs && c.block_m != kDecodeBlockM;
  int32_t log2_block_rows = 0;
  if (subk && rhs_scale_blocks == 1) {
    log2_block_rows = 30;  // every k-step falls into block 0
  } else if (subk) {
    if (gateup) return set_error(TKX_ERR_UNSUPPORTED, "gate-up fusion takes one rhs scale per (group, column)");
    if (k % rhs_scale_blocks != 0) return set_error(TKX_ERR_INVALID, "k=%lld is not a multiple of the %lld scale blocks",
                                                    (long long)k, (long long)rhs_scale_blocks);
    const int64_t rows = k / rhs_scale_blocks;
    while ((1LL << log2_block_rows) < rows) ++log2_block_rows;
    if ((1LL << log2_block_rows) != rows || rows % c.block_k != 0 || k % c.block_k != 0)
      return set_error(TKX_ERR_UNSUPPORTED,
                       "the tiled kernels take scale blocks of a power-of-two number of k rows that block_k divides"
                       " (k=%lld blocks=%lld block_k=%d); widen the weights with tkx_dequantize_weights otherwise",
                       (long long)k, (long long)rhs_scale_blocks, c.block_k);
  }
  if (subk && (lhs_dtype == TKX_F8E4M3FN || lhs_dtype == TKX_I8)) {
    // fp8 x fp8, int8 x int8: the lhs scales come per k-block too, as f32[rhs_scale_blocks, m].
    if (lhs_scale == nullptr || m % 4 != 0 || c.align_tile % 4 != 0 || (uintptr_t)lhs_scale % 16 != 0)
      return set_error(TKX_ERR_UNSUPPORTED,
                       "fp8 x fp8 with scale blocks along k needs lhs scales f32[blocks, m], m %% 4 == 0 and align_tile %% 4 == 0");
  }
  // Packed int4 weights in the tiled kernels: the forward forms, whole k-steps.
  const bool packed_tiled = rhs_dtype == TKX_I4X2 && c.block_m != kDecodeBlockM;
  if (packed_tiled && (dlhs || c.block_k < 1 || k % c.block_k != 0))
    return set_error(TKX_ERR_UNSUPPORTED,
                     "packed int4 weights in a tiled kernel: default mode and k %% block_k == 0 (k=%lld block_k=%d);"
                     " tkx_unpack_int4 gives int8 storage for everything else",
                     (long long)k, c.block_k);
  // fp8 activations over packed int4 weights: the kernel feeds the weights to the fp8 MFMAs with a bias of +8 and
  // takes 8 times the row sum of the fp8 activations off in its epilogue.
  if (rhs_dtype == TKX_I4X2 && lhs_dtype == TKX_F8E4M3FN && (lhs_scale == nullptr || (subk && c.block_k != 128)))
    return set_error(TKX_ERR_UNSUPPORTED,
                     "fp8 x packed int4 weights: lhs_scale f32[2, m] (the row scales, then the row sums of the fp8 values,"
                     " tkx_row_sums_fp8), or with rhs scales per k-block f32[blocks + k / 128, m] (scales per k-block, then row"
                     " sums per 128 columns) and block_k == 128");
  const Variant* v = find_variant(dlhs ? kDlhs : gateup ? kFwdGlu : subk ? kFwdSubK : kFwd, lhs_dtype, rhs_dtype, c);
  if (v == nullptr)
    return set_error(TKX_ERR_UNSUPPORTED, "no kernel variant for mode=%d dtypes=(%d,%d) tile=%dx%dx%d waves=%dx%d stages=%d",
                     mode, lhs_dtype, rhs_dtype, c.block_m, c.block_n, c.block_k, c.waves_m, c.waves_n, c.num_stages);
  // In C terms: rows = m; cols = n (fwd) or k (dlhs); contraction = k (fwd) or n (dlhs).
  const int64_t cols = dlhs ? k : gateup ? n / 2 : n, contraction = dlhs ? n : k;

  const int lb = dtype_bytes(lhs_dtype), rb = dtype_bytes(rhs_dtype), ob = dtype_bytes(out_dtype);
  // 16-byte vector accesses: every row of every operand must start 16-byte aligned and the tile
  // loaders move whole 16-byte chunks along the contiguous axis. The contraction size itself need
  // not be a multiple of block_k: the last k-step is zero-filled.
  if ((k * lb) % 16 != 0 && !dlhs) return set_error(TKX_ERR_UNSUPPORTED, "k*sizeof(lhs) must be a multiple of 16");
  if ((n * rb) % 16 != 0 || (dlhs && (n * lb) % 16 != 0)) return set_error(TKX_ERR_UNSUPPORTED, "n*sizeof(elem) must be a multiple of 16");
  if ((cols * ob) % 16 != 0 || cols % 8 != 0) return set_error(TKX_ERR_UNSUPPORTED, "output row size must be a multiple of 8 elements");
  if (((uintptr_t)lhs | (uintptr_t)rhs | (uintptr_t)out | (uintptr_t)workspace) % 16 != 0 ||
      (rhs_scale && (uintptr_t)rhs_scale % 16 != 0))
    return set_error(TKX_ERR_UNSUPPORTED, "pointers must be 16-byte aligned");

  if (out_scale != nullptr && (v->fn == nullptr || v->fn_fp8_out == nullptr))
    return set_error(TKX_ERR_UNSUPPORTED, "this kernel variant cannot quantise its result (bf16 or fp8 forward tiles whose"
                                          " wave columns tile 128 output columns can)");
  if (v->fn != nullptr && c.split_k > 1 && v->fn_split == nullptr)
    return set_error(TKX_ERR_UNSUPPORTED, "this kernel variant cannot split its last round (plain forward and TRANS_RHS tiles of at least 128 rows can)");
  if (v->fn == nullptr) {
    // Streaming decode kernel: one launch, no schedule.
    if (lhs_scale != nullptr) return set_error(TKX_ERR_UNSUPPORTED, "the decode kernel takes no lhs scale");
    if (rhs_bias != nullptr || gateup) return set_error(TKX_ERR_UNSUPPORTED, "the decode kernel takes no bias or gate-up fusion");
    if (rhs_scale != nullptr && rhs_dtype != TKX_I8 && rhs_dtype != TKX_F8E4M3FN && rhs_dtype != TKX_I4X2)
      return set_error(TKX_ERR_UNSUPPORTED, "the decode kernel takes an rhs scale with int8, packed int4 or fp8 weights only");
    const int32_t split_k = c.split_k > 1 ? c.split_k : 1;  // (0 is 1)
    if (c.persistent != 0) {
      if (c.persistent != 1) return set_error(TKX_ERR_INVALID, "persistent must be 0 or 1, got %d", c.persistent);
      if (split_k > 1) return set_error(TKX_ERR_UNSUPPORTED, "persistent and split_k > 1 exclude each other");
      if (!decode_persistent_supported(lhs_dtype, rhs_dtype, m, k, n, num_groups, rhs_scale ? rhs_scale_blocks : 1, c.block_n,
                                       c.num_stages))
        return set_error(TKX_ERR_UNSUPPORTED,
                         "the persistent decode kernel needs block_n 128, num_stages <= 4, one scale per (group, column),"
                         " num_groups <= 256, at most 1024 tiles, k %% 32 == 0 and n %% 8 == 0 (k=%lld n=%lld G=%lld scale blocks=%lld)",
                         (long long)k, (long long)n, (long long)num_groups, (long long)rhs_scale_blocks);
      return launch_decode(lhs, rhs, rhs_scale, group_sizes, out, m, k, n, num_groups, rhs_dtype, out_dtype, activation,
                           c.num_stages, 1, c.block_n, group_offset, num_group_sizes, 1, c.persistent,
                           static_cast<int32_t*>(workspace), stream);
    }
    if (!decode_supported(lhs_dtype, rhs_dtype, m, k, n, num_groups, rhs_scale ? rhs_scale_blocks : 1, c.block_n,
                          c.num_stages, split_k))
      return set_error(TKX_ERR_UNSUPPORTED,
                       "decode kernel needs k %% 1024 == 0 (split: k %% (128 * split_k * min(num_stages, 4)) == 0, split_k <= 16,"
                       " num_stages <= 4, block_n 128), n %% 8 == 0 (n %% 16 == 0 and one scale block at block_n 256)"
                       " and scale blocks of a power-of-two multiple of 32 rows (k=%lld n=%lld G=%lld scale blocks=%lld split_k=%d)",
                       (long long)k, (long long)n, (long long)num_groups, (long long)rhs_scale_blocks, split_k);
    return launch_decode(lhs, rhs, rhs_scale, group_sizes, out, m, k, n, num_groups, rhs_dtype, out_dtype, activation,
                         c.num_stages, rhs_scale ? rhs_scale_blocks : 1, c.block_n, group_offset, num_group_sizes,
                         split_k, 0, static_cast<int32_t*>(workspace), stream);
  }

  if (c.persistent != 0) return set_error(TKX_ERR_UNSUPPORTED, "persistent belongs to the streaming small-m kernel (block_m == 16)");
  // split_k > 1 on a tiled kernel: the tiles of the last, partial round of workgroups are cut along the contraction
  // (plain forward and dlhs variants; the workspace then is tkx_ragged_dot_split_workspace_bytes long).
  const int32_t split_k = c.split_k > 1 ? c.split_k : 1;
  if (split_k > 1 && (gateup || subk || out_scale != nullptr))
    return set_error(TKX_ERR_UNSUPPORTED, "split_k > 1 on a tiled kernel: plain forward and TRANS_RHS only (no gate-up fusion, scales per k-block or quantised result)");
  if (split_k > 16) return set_error(TKX_ERR_INVALID, "split_k must lie in [1, 16], got %d", split_k);
  const WsLayout L = ws_layout(m, num_groups, c.block_m);
  int32_t st = launch_schedule(group_sizes, num_groups, group_offset, num_group_sizes, m, c.block_m, c.align_tile,
                               c.grid_tile_width, static_cast<int32_t*>(workspace), L, stream);
  if (st != TKX_OK) return st;

  GemmParams p = {};
  p.A = lhs;
  p.B = rhs;
  p.C = out;
  p.a_scale = lhs_scale;
  p.b_scale = rhs_scale;
  p.b_bias = rhs_bias;
  p.c_scale = out_scale;
  p.ws = static_cast<const int32_t*>(workspace);
  p.lda = dlhs ? n : k;
  p.ldb = n;
  p.ldc = cols;
  p.b_group_stride = rhs_dtype == TKX_I4X2 ? k / 2 * n : k * n;  // (in stored elements: packed bytes)
  p.c_group_stride = 0;
  p.m_ext = (int32_t)m;
  p.n_ext = (int32_t)cols;
  p.nb_ext = (int32_t)(gateup ? n : cols);
  p.k_ext = (int32_t)contraction;
  p.num_groups = (int32_t)num_groups;
  const int64_t out_block_n = gateup ? c.block_n / 2 : c.block_n;  // output columns of a tile
  p.n_tiles = (int32_t)((cols + out_block_n - 1) / out_block_n);
  p.m_tiles = 0;
  // Whole chunks for every XCD, so that each list entry has a workgroup (see the launch order in run()).
  const int64_t slots = ((int64_t)L.tid_size * p.n_tiles + 8 * kXcdChunk - 1) / (8 * kXcdChunk) * (8 * kXcdChunk);
  p.real_slots = (int32_t)slots;
  p.tid_size = L.tid_size;
  p.grid_tile_width = c.grid_tile_width;
  p.out_dtype = out_dtype;
  p.activation = activation;
  p.scale_blocks = subk ? (int32_t)rhs_scale_blocks : 1;
  p.log2_block_rows = log2_block_rows;
  p.ws_offsets = (int32_t)L.offsets;
  p.ws_gid = (int32_t)L.task[0];
  p.ws_bstart = (int32_t)L.task[1];
  p.ws_astart = (int32_t)L.task[2];
  p.ws_aend = (int32_t)L.task[3];
  p.ws_span_first = (int32_t)L.task[6];
  p.ws_span_width = (int32_t)L.task[7];
  if (slots > 0x7fffff00LL) return set_error(TKX_ERR_UNSUPPORTED, "too many tiles");
  // Extra workgroups zero the rows past the last group (and before the first, with a group offset);
  // they exit at once when there are none.
  int64_t zero_wgs = (m * cols * ob + (64 << 10) - 1) / (64 << 10);
  if (zero_wgs > 256) zero_wgs = 256;
  if (zero_wgs < 1) zero_wgs = 1;
  p.zero_wgs = (int32_t)zero_wgs;
  p.split_k = split_k;
  p.split_cus = 1;
  int64_t split_wgs = 0;
  if (split_k > 1) {
    int cus = 0;
    st = device_compute_units(&cus);
    if (st != TKX_OK) return st;
    p.split_cus = cus < kSplitUnits ? cus : kSplitUnits;
    p.ws_split_counters = (int32_t)L.split_counters;
    p.split_partials = reinterpret_cast<float*>(static_cast<int32_t*>(workspace) + L.words);
    split_wgs = p.split_cus;  // at most that many parts beside the tiles' own workgroups
  }
  return launch(v, p, slots + zero_wgs + split_wgs, stream);
}
}  // namespace

extern "C" {

int32_t tkx_ragged_dot_fwd(const void* lhs, const void* rhs, const int32_t* group_sizes, const float* lhs_scale,
                           const float* rhs_scale, void* out, void* workspace, int64_t m, int64_t k, int64_t n,
                           int64_t num_groups, int32_t lhs_dtype, int32_t rhs_dtype, int32_t out_dtype, int32_t mode,
                           int32_t activation, const TkxConfig* config, tkx_stream_t stream) {
  return fwd_impl(lhs, rhs, group_sizes, nullptr, lhs_scale, rhs_scale, nullptr, out, workspace, m, k, n, num_groups,
                  num_groups, lhs_dtype, rhs_dtype, out_dtype, mode, activation, false, 1, config, stream);
}

int32_t tkx_ragged_dot_fwd_fp8_out(const void* lhs, const void* rhs, const int32_t* group_sizes, const float* lhs_scale,
                                   const float* rhs_scale, void* out, float* out_scale, void* workspace, int64_t m,
                                   int64_t k, int64_t n, int64_t num_groups, int32_t lhs_dtype, int32_t rhs_dtype,
                                   int32_t activation, const TkxConfig* config, tkx_stream_t stream) {
  if (out_scale == nullptr) return set_error(TKX_ERR_INVALID, "null pointer argument");
  return fwd_impl(lhs, rhs, group_sizes, nullptr, lhs_scale, rhs_scale, nullptr, out, workspace, m, k, n, num_groups,
                  num_groups, lhs_dtype, rhs_dtype, TKX_F8E4M3FN, TKX_MODE_DEFAULT, activation, false, 1, config, stream,
                  out_scale);
}

int32_t tkx_ragged_dot_fwd_static_workspace(const void* lhs, const void* rhs, const int32_t* group_sizes,
                                            const float* lhs_scale, const float* rhs_scale, void* out, int64_t m, int64_t k,
                                            int64_t n, int64_t num_groups, int32_t lhs_dtype, int32_t rhs_dtype,
                                            int32_t out_dtype, int32_t mode, int32_t activation, const TkxConfig* config,
                                            tkx_stream_t stream) {
  if (config == nullptr) return set_error(TKX_ERR_INVALID, "null pointer argument");
  if (m < 1 || num_groups < 1 || config->block_m < 1)
    return set_error(TKX_ERR_INVALID, "bad sizes m=%lld G=%lld block_m=%d", (long long)m, (long long)num_groups, config->block_m);
  if (config->split_k > 1 || config->persistent != 0)
    return set_error(TKX_ERR_UNSUPPORTED,
                     "a split contraction (split_k > 1, persistent) keeps arrival counters in a workspace that the caller"
                     " cleared; the built-in workspace holds whatever the last call left there (use tkx_ragged_dot_fwd, or"
                     " split_k = 1 and persistent = 0)");
  const int64_t words = ws_layout(m, num_groups, config->block_m).words;
  if (words > kScratchWords)
    return set_error(TKX_ERR_UNSUPPORTED,
                     "the schedule of m=%lld, G=%lld, block_m=%d needs %lld bytes; the built-in workspace holds %lld"
                     " (use tkx_ragged_dot_fwd with a workspace of your own)",
                     (long long)m, (long long)num_groups, config->block_m, (long long)(words * 4), (long long)(kScratchWords * 4));
  int32_t* ws = nullptr;
  const int32_t st = scratch_address(&ws);
  if (st != TKX_OK) return st;
  // The scheduler kernel writes every word the GEMM kernel reads, so nothing of the last call's contents matters.
  return fwd_impl(lhs, rhs, group_sizes, nullptr, lhs_scale, rhs_scale, nullptr, out, ws, m, k, n, num_groups, num_groups,
                  lhs_dtype, rhs_dtype, out_dtype, mode, activation, false, 1, config, stream);
}

int32_t tkx_ragged_dot_fwd_fused(const void* lhs, const void* rhs, const int32_t* group_sizes, const int32_t* group_offset,
                                 const float* lhs_scale, const float* rhs_scale, const float* rhs_bias, void* out,
                                 void* workspace, int64_t m, int64_t k, int64_t n, int64_t num_groups,
                                 int64_t num_group_sizes, int64_t rhs_scale_blocks, int32_t lhs_dtype, int32_t rhs_dtype,
                                 int32_t out_dtype, int32_t activation, int32_t gateup, const TkxConfig* config,
                                 tkx_stream_t stream) {
  if (gateup != 0 && gateup != 1) return set_error(TKX_ERR_INVALID, "gateup must be 0 or 1");
  if (rhs_scale_blocks < 1) return set_error(TKX_ERR_INVALID, "rhs_scale_blocks must be >= 1");
  if (group_offset != nullptr && (uintptr_t)group_offset % 4 != 0)
    return set_error(TKX_ERR_INVALID, "group_offset must be 4-byte aligned");
  return fwd_impl(lhs, rhs, group_sizes, group_offset, lhs_scale, rhs_scale, rhs_bias, out, workspace, m, k, n, num_groups,
                  num_group_sizes, lhs_dtype, rhs_dtype, out_dtype, TKX_MODE_DEFAULT, activation, gateup == 1,
                  rhs_scale_blocks, config, stream);
}

int32_t tkx_ragged_dot_drhs(const void* lhs, const void* dout, const int32_t* group_sizes, void* out, void* workspace,
                            int64_t m, int64_t k, int64_t n, int64_t num_groups, int32_t dtype, int32_t out_dtype,
                            const TkxConfig* config, tkx_stream_t stream_) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (!lhs || !dout || !group_sizes || !out || !workspace || !config)
    return set_error(TKX_ERR_INVALID, "null pointer argument");
  if (m < 1 || k < 1 || n < 1 || num_groups < 1)
    return set_error(TKX_ERR_INVALID, "bad sizes m=%lld k=%lld n=%lld G=%lld", (long long)m, (long long)k,
                     (long long)n, (long long)num_groups);
  if (!valid_out_dtype(out_dtype)) return set_error(TKX_ERR_UNSUPPORTED, "out dtype %d not supported", out_dtype);
  if (m > 0x7fffffffLL / 2 || k >= (1 << 21) || n >= (1 << 21))
    return set_error(TKX_ERR_UNSUPPORTED, "dimension too large");
  const TkxConfig& c = *config;
  if (c.align_tile < 1) return set_error(TKX_ERR_INVALID, "align_tile must be >= 1");
  const Variant* v = find_variant(kDrhs, dtype, dtype, c);
  if (v == nullptr)
    return set_error(TKX_ERR_UNSUPPORTED, "no drhs kernel variant for dtype=%d tile=%dx%dx%d waves=%dx%d stages=%d", dtype,
                     c.block_m, c.block_n, c.block_k, c.waves_m, c.waves_n, c.num_stages);
  const int eb = dtype_bytes(dtype), ob = dtype_bytes(out_dtype);
  if ((k * eb) % 16 != 0 || (n * eb) % 16 != 0 || (n * ob) % 16 != 0 || n % 8 != 0)
    return set_error(TKX_ERR_UNSUPPORTED, "k and n row sizes must be multiples of 16 bytes (n of 8 elements)");
  if (((uintptr_t)lhs | (uintptr_t)dout | (uintptr_t)out | (uintptr_t)workspace) % 16 != 0)
    return set_error(TKX_ERR_UNSUPPORTED, "pointers must be 16-byte aligned");

  // Only the group offsets are needed; block_m of the schedule is irrelevant here, use a fixed one
  // so the workspace size depends on (m, G) alone.
  const int32_t sched_bm = 128;
  const WsLayout L = ws_layout(m, num_groups, sched_bm);
  int32_t st = launch_schedule(group_sizes, num_groups, nullptr, num_groups, m, sched_bm, c.align_tile, 1,
                               static_cast<int32_t*>(workspace), L, stream);
  if (st != TKX_OK) return st;

  GemmParams p = {};
  p.A = lhs;
  p.B = dout;
  p.C = out;
  p.ws = static_cast<const int32_t*>(workspace);
  p.lda = k;
  p.ldb = n;
  p.ldc = n;
  p.c_group_stride = k * n;
  p.m_ext = (int32_t)k;
  p.n_ext = (int32_t)n;
  p.nb_ext = (int32_t)n;
  p.k_ext = (int32_t)m;
  p.num_groups = (int32_t)num_groups;
  p.n_tiles = (int32_t)((n + c.block_n - 1) / c.block_n);
  p.m_tiles = (int32_t)((k + c.block_m - 1) / c.block_m);
  p.grid_tile_width = 1;
  p.out_dtype = out_dtype;
  p.activation = TKX_ACT_NONE;
  p.ws_offsets = (int32_t)L.offsets;
  p.split_k = 1;
  p.split_cus = 1;
  return launch(v, p, (int64_t)num_groups * p.m_tiles * p.n_tiles, stream);
}

int32_t tkx_dequantize_weights(const void* qvalue, const float* scale, void* out, int64_t num_groups, int64_t k,
                               int64_t n, int64_t scale_block_k, int32_t q_dtype, int32_t out_dtype,
                               tkx_stream_t stream) {
  if (!qvalue || !scale || !out) return set_error(TKX_ERR_INVALID, "null pointer argument");
  if (num_groups < 1 || k < 1 || n < 1 || scale_block_k < 1)
    return set_error(TKX_ERR_INVALID, "bad sizes G=%lld k=%lld n=%lld block=%lld", (long long)num_groups, (long long)k,
                     (long long)n, (long long)scale_block_k);
  if (k % scale_block_k != 0) return set_error(TKX_ERR_INVALID, "k=%lld is not a multiple of the scale block %lld",
                                               (long long)k, (long long)scale_block_k);
  // Weights [G, k, n] as G * k rows: a block of scale_block_k rows never straddles two groups.
  return tkx_dequantize(qvalue, scale, out, num_groups * k, n, scale_block_k, 1, q_dtype, out_dtype, stream);
}

int32_t tkx_dequantize(const void* qvalue, const float* scale, void* out, int64_t rows, int64_t cols,
                       int64_t scale_block_rows, int64_t scale_block_cols, int32_t q_dtype, int32_t out_dtype,
                       tkx_stream_t stream) {
  if (!qvalue || !scale || !out) return set_error(TKX_ERR_INVALID, "null pointer argument");
  if (rows < 1 || cols < 1 || scale_block_rows < 1 || scale_block_cols < 1)
    return set_error(TKX_ERR_INVALID, "bad sizes rows=%lld cols=%lld block=%lldx%lld", (long long)rows, (long long)cols,
                     (long long)scale_block_rows, (long long)scale_block_cols);
  if ((q_dtype != TKX_I8 && q_dtype != TKX_F8E4M3FN) || out_dtype != TKX_BF16)
    return set_error(TKX_ERR_UNSUPPORTED, "dequantisation is int8 or fp8 -> bf16 only (got %d -> %d)", q_dtype, out_dtype);
  if (rows % scale_block_rows != 0 || cols % scale_block_cols != 0)
    return set_error(TKX_ERR_INVALID, "scale blocks %lldx%lld do not tile %lldx%lld", (long long)scale_block_rows,
                     (long long)scale_block_cols, (long long)rows, (long long)cols);
  if (cols % 16 != 0 || cols > 0x7fffffffLL) return set_error(TKX_ERR_UNSUPPORTED, "cols must be a multiple of 16");
  if (scale_block_cols != 1 && scale_block_cols % 16 != 0)
    return set_error(TKX_ERR_UNSUPPORTED, "scale blocks along the columns must be 1 or a multiple of 16 wide");
  if (scale_block_rows > 0x7fffffffLL) return set_error(TKX_ERR_UNSUPPORTED, "scale block too tall");
  if (((uintptr_t)qvalue | (uintptr_t)out) % 16 != 0 || (uintptr_t)scale % (scale_block_cols == 1 ? 16 : 4) != 0)
    return set_error(TKX_ERR_UNSUPPORTED, "pointers must be 16-byte aligned");
  return launch_dequant(qvalue, scale, nullptr, out, rows, cols, scale_block_rows, scale_block_cols, q_dtype,
                        static_cast<hipStream_t>(stream));
}

int32_t tkx_dequantize_zero_point(const void* qvalue, const float* scale, const float* zero_point, void* out, int64_t rows,
                                  int64_t cols, int64_t scale_block_rows, int64_t scale_block_cols, int32_t q_dtype,
                                  int32_t out_dtype, tkx_stream_t stream) {
  if (!zero_point) return set_error(TKX_ERR_INVALID, "null pointer argument");
  // (the checks of tkx_dequantize, which launches nothing when one fails)
  if (!qvalue || !scale || !out) return set_error(TKX_ERR_INVALID, "null pointer argument");
  if (rows < 1 || cols < 1 || scale_block_rows < 1 || scale_block_cols < 1)
    return set_error(TKX_ERR_INVALID, "bad sizes rows=%lld cols=%lld block=%lldx%lld", (long long)rows, (long long)cols,
                     (long long)scale_block_rows, (long long)scale_block_cols);
  if ((q_dtype != TKX_I8 && q_dtype != TKX_F8E4M3FN) || out_dtype != TKX_BF16)
    return set_error(TKX_ERR_UNSUPPORTED, "dequantisation is int8 or fp8 -> bf16 only (got %d -> %d)", q_dtype, out_dtype);
  if (rows % scale_block_rows != 0 || cols % scale_block_cols != 0)
    return set_error(TKX_ERR_INVALID, "scale blocks %lldx%lld do not tile %lldx%lld", (long long)scale_block_rows,
                     (long long)scale_block_cols, (long long)rows, (long long)cols);
  if (cols % 16 != 0 || cols > 0x7fffffffLL) return set_error(TKX_ERR_UNSUPPORTED, "cols must be a multiple of 16");
  if (scale_block_cols != 1 && scale_block_cols % 16 != 0)
    return set_error(TKX_ERR_UNSUPPORTED, "scale blocks along the columns must be 1 or a multiple of 16 wide");
  if (scale_block_rows > 0x7fffffffLL) return set_error(TKX_ERR_UNSUPPORTED, "scale block too tall");
  const uintptr_t table_align = scale_block_cols == 1 ? 16 : 4;
  if (((uintptr_t)qvalue | (uintptr_t)out) % 16 != 0 || (uintptr_t)scale % table_align != 0 || (uintptr_t)zero_point % table_align != 0)
    return set_error(TKX_ERR_UNSUPPORTED, "pointers must be 16-byte aligned");
  return launch_dequant(qvalue, scale, zero_point, out, rows, cols, scale_block_rows, scale_block_cols, q_dtype,
                        static_cast<hipStream_t>(stream));
}

namespace {
int32_t int4_repack(const void* in, void* out, int64_t packed_rows, int64_t cols, bool unpack, tkx_stream_t stream) {
  if (!in || !out) return set_error(TKX_ERR_INVALID, "null pointer argument");
  if (packed_rows < 1 || cols < 1) return set_error(TKX_ERR_INVALID, "bad sizes rows=%lld cols=%lld", (long long)packed_rows, (long long)cols);
  if (cols % 16 != 0 || cols > 0x7fffffffLL) return set_error(TKX_ERR_UNSUPPORTED, "cols must be a multiple of 16");
  if (((uintptr_t)in | (uintptr_t)out) % 16 != 0) return set_error(TKX_ERR_UNSUPPORTED, "pointers must be 16-byte aligned");
  return launch_int4_repack(in, out, packed_rows, cols, unpack, static_cast<hipStream_t>(stream));
}
}  // namespace

int32_t tkx_unpack_int4(const void* packed, void* out, int64_t packed_rows, int64_t cols, tkx_stream_t stream) {
  return int4_repack(packed, out, packed_rows, cols, true, stream);
}

int32_t tkx_pack_int4(const void* values, void* packed, int64_t packed_rows, int64_t cols, tkx_stream_t stream) {
  return int4_repack(values, packed, packed_rows, cols, false, stream);
}

int32_t tkx_row_sums_fp8(const void* x, float* sums, int64_t rows, int64_t cols, int64_t chunk_cols, tkx_stream_t stream) {
  if (!x || !sums) return set_error(TKX_ERR_INVALID, "null pointer argument");
  if (rows < 1 || cols < 1 || rows > 0x7fffffffLL) return set_error(TKX_ERR_INVALID, "bad sizes rows=%lld cols=%lld", (long long)rows, (long long)cols);
  if (cols % 16 != 0 || cols > 0x7fffffffLL) return set_error(TKX_ERR_UNSUPPORTED, "cols must be a multiple of 16");
  if ((uintptr_t)x % 16 != 0 || (uintptr_t)sums % 4 != 0) return set_error(TKX_ERR_UNSUPPORTED, "x must be 16-byte aligned, sums 4-byte aligned");
  if (chunk_cols != cols && (chunk_cols != 128 || cols % 128 != 0))
    return set_error(TKX_ERR_UNSUPPORTED, "chunk_cols is cols (one sum per row) or 128 with cols %% 128 == 0 (got %lld)", (long long)chunk_cols);
  return launch_row_sums_fp8(x, sums, rows, cols, chunk_cols != cols, static_cast<hipStream_t>(stream));
}

int32_t tkx_quantize(const void* x, void* qvalue, float* scale, int64_t rows, int64_t cols, int64_t scale_block_rows,
                     int64_t scale_block_cols, int32_t x_dtype, int32_t q_dtype, float qmax, float bound,
                     tkx_stream_t stream) {
  if (!x || !qvalue || !scale) return set_error(TKX_ERR_INVALID, "null pointer argument");
  if (rows < 1 || cols < 1 || scale_block_rows < 1 || scale_block_cols < 1)
    return set_error(TKX_ERR_INVALID, "bad sizes rows=%lld cols=%lld block=%lldx%lld", (long long)rows, (long long)cols,
                     (long long)scale_block_rows, (long long)scale_block_cols);
  if (x_dtype != TKX_F32 && x_dtype != TKX_BF16 && x_dtype != TKX_F16)
    return set_error(TKX_ERR_UNSUPPORTED, "quantisation reads f32, bf16 or f16 (got %d)", x_dtype);
  if (q_dtype != TKX_I8 && q_dtype != TKX_F8E4M3FN)
    return set_error(TKX_ERR_UNSUPPORTED, "quantisation writes int8 or fp8 e4m3fn (got %d)", q_dtype);
  if (rows % scale_block_rows != 0 || cols % scale_block_cols != 0)
    return set_error(TKX_ERR_INVALID, "scale blocks %lldx%lld do not tile %lldx%lld", (long long)scale_block_rows,
                     (long long)scale_block_cols, (long long)rows, (long long)cols);
  if (cols % 8 != 0 || cols > 0x7fffffffLL) return set_error(TKX_ERR_UNSUPPORTED, "cols must be a multiple of 8");
  if (scale_block_rows == 1) {
    if (scale_block_cols % 8 != 0) return set_error(TKX_ERR_UNSUPPORTED, "tiles one row tall must be a multiple of 8 columns wide");
  } else {
    if (scale_block_rows > 0x7fffffffLL) return set_error(TKX_ERR_UNSUPPORTED, "scale block too tall");
    if (scale_block_cols != 1 && scale_block_cols % 8 != 0)
      return set_error(TKX_ERR_UNSUPPORTED, "tiles several rows tall must be 1 column or a multiple of 8 columns wide (got %lld)",
                       (long long)scale_block_cols);
    if (scale_block_cols == 1 && cols % 4 != 0) return set_error(TKX_ERR_UNSUPPORTED, "cols must be a multiple of 4");
  }
  if ((uintptr_t)x % 16 != 0 || (uintptr_t)qvalue % 8 != 0 || (uintptr_t)scale % 16 != 0)
    return set_error(TKX_ERR_UNSUPPORTED, "pointers must be 16-byte aligned");
  const float type_max = q_dtype == TKX_I8 ? 127.f : 448.f;
  if (qmax == 0.f) qmax = type_max;
  if (!(qmax > 0.f) || qmax > type_max) return set_error(TKX_ERR_INVALID, "qmax must lie in (0, %g]", (double)type_max);
  if (bound == 0.f) bound = qmax;
  if (!(bound >= qmax) || bound > qmax + 1.f)
    return set_error(TKX_ERR_INVALID, "bound must lie in [qmax, qmax + 1] (got %g for qmax %g)", (double)bound, (double)qmax);
  // A bound above qmax (integers: 2^(b-1) - 0.5) lets -qmax - 1, the type's most negative value, appear.
  QuantRange range = {bound, -qmax, qmax};
  if (bound > qmax) {
    if (q_dtype != TKX_I8) return set_error(TKX_ERR_INVALID, "a bound above qmax belongs to the integer types");
    range.lo = -qmax - 1.f;
  }
  return launch_quantize(x, qvalue, scale, rows, cols, scale_block_rows, scale_block_cols, x_dtype, q_dtype, range,
                         static_cast<hipStream_t>(stream));
}

int32_t tkx_ragged_gather_rows(const void* x, const int32_t* indices, const float* weights, const uint8_t* valid,
                               const int32_t* start, const int32_t* end, void* out, int64_t in_rows, int64_t out_rows,
                               int64_t hidden, int64_t reduce_group_size, int32_t dtype, tkx_stream_t stream) {
  if (!x || !indices || !out) return set_error(TKX_ERR_INVALID, "null pointer argument");
  if (in_rows < 1 || out_rows < 0 || hidden < 1 || reduce_group_size < 1)
    return set_error(TKX_ERR_INVALID, "bad sizes in_rows=%lld out_rows=%lld hidden=%lld reduce=%lld", (long long)in_rows,
                     (long long)out_rows, (long long)hidden, (long long)reduce_group_size);
  if ((start == nullptr) != (end == nullptr)) return set_error(TKX_ERR_INVALID, "start and end go together");
  if (dtype != TKX_F32 && dtype != TKX_BF16 && dtype != TKX_F16)
    return set_error(TKX_ERR_UNSUPPORTED, "dtype %d not supported", dtype);
  const int64_t esz = dtype_bytes(dtype);
  if ((hidden * esz) % 16 != 0 || ((uintptr_t)x | (uintptr_t)out) % 16 != 0)
    return set_error(TKX_ERR_UNSUPPORTED, "rows must be a multiple of 16 bytes and 16-byte aligned");
  if (hidden >= (1LL << 31) || reduce_group_size >= (1LL << 31)) return set_error(TKX_ERR_UNSUPPORTED, "dimension too large");
  return launch_gather_rows(x, indices, weights, valid, start, end, out, in_rows, out_rows, hidden, reduce_group_size,
                            dtype, static_cast<hipStream_t>(stream));
}

int32_t tkx_ragged_dot_num_variants(int32_t kind) {
  int32_t n = 0;
  for (const Variant& v : registry()) n += ((v.mode == kDrhs) == (kind == 1));
  return n;
}

int32_t tkx_ragged_dot_variant(int32_t kind, int32_t index, TkxConfig* config, int32_t* lhs_dtype, int32_t* rhs_dtype,
                               int32_t* mode) {
  if (!config || !lhs_dtype || !rhs_dtype || !mode) return set_error(TKX_ERR_INVALID, "null pointer argument");
  int32_t i = 0;
  for (const Variant& v : registry()) {
    if ((v.mode == kDrhs) != (kind == 1)) continue;
    if (i++ != index) continue;
    config->block_m = v.block_m;
    config->block_n = v.block_n;
    config->block_k = v.block_k;
    config->waves_m = v.waves_m;
    config->waves_n = v.waves_n;
    config->grid_tile_width = 1;
    config->align_tile = 8;
    config->num_stages = v.num_stages;
    config->split_k = 1;
    config->persistent = 0;
    *lhs_dtype = v.a_dtype;
    *rhs_dtype = v.b_dtype;
    *mode = v.mode;
    return TKX_OK;
  }
  return set_error(TKX_ERR_INVALID, "variant index %d out of range", index);
}

}  // extern "C"
