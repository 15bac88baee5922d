// Small-m ("decode") ragged dot: bf16 lhs [m,k] x int8 or fp8 (e4m3fn) rhs [G,k,n] with f32 scales [G,n],
// or x int4 rhs packed two to a byte along k ([G,k/2,n] bytes: k = 2 kk in bits 0-3, k = 2 kk + 1 in bits 4-7),
// or bf16 x bf16 / f16 x f16 without scales.
//
// This regime is bound by HBM: every touched expert's [k,n] weight panel is read once, and a group
// has a handful of rows. The kernel is built around streaming those panels:
//   * one launch, no scheduler kernel: a workgroup derives its group's row range from group_sizes
//     itself while its first weight loads are already in flight, and the workgroups of empty groups
//     exit (all but the first 2% of an empty group's weights are never read);
//   * a workgroup owns (group, 128 output columns); its 4 waves split the contraction and each
//     streams its own [k/4, 128] slice of the panel with full 128-byte rows, several steps of
//     global loads in flight in registers; no workgroup barrier and no LDS inside the loop;
//   * no transposition is needed: the contraction index of an MFMA is only a label, so lane
//     (i, q) loads 8 bytes (columns 8i..8i+7) from each of the 8 rows 8q..8q+7 of a 32-row step and
//     feeds MFMA j (j = 0..7) with byte j of those 8 loads, i.e. 8 contraction values of column
//     8i+j.  MFMA j therefore produces the output columns {8i+j}; the lhs fragment of lane (r, q) is
//     lhs[r][8q..8q+7] of the same step, one 16-byte load. (16-bit weights: 16 bytes per row and the
//     j-th half-word of each, otherwise the same; int8 weights also come with 16 columns per lane,
//     256 per workgroup: 16-byte loads and 16 MFMAs per step);
//   * int8 is widened to bf16 exactly and goes through the 16x16x32 bf16 MFMA with f32 accumulation;
//   * the four partial tiles are added in a fixed order through LDS (deterministic), scaled per
//     (group, column), and rows past the group's end are never written.
#include "tkx_common.h"
#include "tkx_gemm.hip.h"

#include <mutex>
#include <utility>
#include <vector>

namespace tkx {
namespace {

constexpr int kDecBN = 128;    // output columns per workgroup (256 for the wide int8 kernel)
constexpr int kDecWaves = 4;   // waves per workgroup; each takes k / 4 of the contraction
constexpr int kDecKS = 32;     // contraction elements per step (one 16x16x32 MFMA deep)
constexpr int kDecRows = 16;   // lhs rows per pass
constexpr int kDecThreads = kDecWaves * 64;

struct DecodeParams {
  const unsigned char* lhs;  // 16-bit elements
  const unsigned char* rhs;  // int8, or 16-bit elements of the lhs type
  const float* scale;
  const int32_t* group_sizes;
  void* out;
  int32_t m, k, n, num_groups, n_tiles, out_dtype, activation;
  const int32_t* group_offset;  // device, one int32, or null: group g is entry offset + g of group_sizes
  int32_t num_global;           // entries of group_sizes (num_groups without an offset)
  int32_t scale_blocks;     // scale blocks along k: scale is [G, scale_blocks, n]
  int32_t log2_block_rows;  // scale_blocks > 1: log2 of the contraction rows per scale block
  // Contraction split over workgroups (SK kernels): split_k workgroups per (group, column tile), each with
  // k / split_k of the contraction; f32 partial sums [split_k, m, n] and one arrival counter per tile.
  int32_t split_k;
  float* partials;
  int32_t* counters;  // [G * n_tiles], zero on entry; the last workgroup to arrive at a tile resets its counter
};

typedef float f32x4_t __attribute__((ext_vector_type(4)));

// Buffer loads: wave-uniform descriptor (base + byte count; reads past the end return zero), a
// 32-bit lane offset and a wave-uniform 32-bit step offset. No 64-bit address arithmetic in VGPRs.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t buffer_of(const void* base, uint32_t bytes) {
  const unsigned char* b = uniform_pointer(static_cast<const unsigned char*>(base));
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char*>(b), 0, __builtin_amdgcn_readfirstlane((int)bytes), 0x00020000);
}
// Weights are read exactly once: the non-temporal hint keeps them from displacing reusable lines
// in the caches, which measurably raises the streaming rate (about 8% on this kernel).
constexpr int kStreamingLoad = 2;  // cache-policy operand of the buffer load: bit 1 = nt
__device__ __forceinline__ i32x2 buffer_load_8(__amdgpu_buffer_rsrc_t r, uint32_t lane_offset, uint32_t uniform_offset) {
  return __builtin_bit_cast(i32x2, __builtin_amdgcn_raw_buffer_load_b64(r, (int)lane_offset, (int)uniform_offset, kStreamingLoad));
}
__device__ __forceinline__ i32x4 buffer_load_16(__amdgpu_buffer_rsrc_t r, uint32_t lane_offset, uint32_t uniform_offset) {
  return __builtin_bit_cast(i32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)lane_offset, (int)uniform_offset, 0));
}
__device__ __forceinline__ i32x4 buffer_load_16_streaming(__amdgpu_buffer_rsrc_t r, uint32_t lane_offset, uint32_t uniform_offset) {
  return __builtin_bit_cast(i32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)lane_offset, (int)uniform_offset, kStreamingLoad));
}

constexpr int kEI4 = TKX_I4X2;  // packed int4 weights: a stored row holds two contraction rows

// What a lane holds of one weight row of a step: its CPL columns (8, or 16 of int8).
template <int EW, int CPL> struct WeightRow { typedef i32x4 T; static constexpr int ESZ = 2; };
template <> struct WeightRow<kEI4, 8> { typedef i32x2 T; static constexpr int ESZ = 1; };
template <> struct WeightRow<kEI8, 8> { typedef i32x2 T; static constexpr int ESZ = 1; };
template <> struct WeightRow<kEF8, 8> { typedef i32x2 T; static constexpr int ESZ = 1; };
template <> struct WeightRow<kEI8, 16> { typedef i32x4 T; static constexpr int ESZ = 1; };
template <int EW, int CPL>
__device__ __forceinline__ typename WeightRow<EW, CPL>::T load_weight_row(__amdgpu_buffer_rsrc_t r, uint32_t lane_offset, uint32_t uniform_offset) {
  if constexpr ((EW == kEI8 || EW == kEF8 || EW == kEI4) && CPL == 8) return buffer_load_8(r, lane_offset, uniform_offset);
  else return buffer_load_16_streaming(r, lane_offset, uniform_offset);
}

// Sign-extended byte B of a dword -> f32, one SDWA instruction.
template <int B>
__device__ __forceinline__ unsigned i8_to_f32_bits(int w) {
  unsigned f;
  if constexpr (B == 0) asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_0" : "=v"(f) : "v"(w));
  if constexpr (B == 1) asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_1" : "=v"(f) : "v"(w));
  if constexpr (B == 2) asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_2" : "=v"(f) : "v"(w));
  if constexpr (B == 3) asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_3" : "=v"(f) : "v"(w));
  return f;
}

// Byte J of each of 8 loaded 8- or 16-byte rows -> bf16 x8 (exact: |v| <= 128 fits the significand).
// The upper halves of two f32 are the two bf16, packed with one byte permute.
template <int J, typename Row>
__device__ __forceinline__ i32x4 column_fragment_i8(const Row (&rows)[8]) {
  i32x4 out;
#pragma unroll
  for (int h = 0; h < 4; ++h) {
    const unsigned f0 = i8_to_f32_bits<(J & 3)>(rows[2 * h][J >> 2]);
    const unsigned f1 = i8_to_f32_bits<(J & 3)>(rows[2 * h + 1][J >> 2]);
    // v_perm_b32 picks bytes from {first operand: bytes 7..4, second operand: bytes 3..0}.
    out[h] = (int)__builtin_amdgcn_perm(f1, f0, 0x07060302u);
  }
  return out;
}
// Packed int4 weights: byte J of each of 4 loaded rows holds two consecutive contraction values of column J (low
// nibble first); each is sign-extended out of its bit field, converted, and the pair packed as above.
// (The bit-field builtin is declared with an unsigned result; the value is the sign-extended field.)
__device__ __forceinline__ float int4_field(int w, unsigned offset) { return (float)(int)__builtin_amdgcn_sbfe(w, offset, 4); }
template <int J>
__device__ __forceinline__ i32x4 column_fragment_i4(const i32x2 (&rows)[4]) {
  i32x4 out;
#pragma unroll
  for (int h = 0; h < 4; ++h) {
    const int w = rows[h][J >> 2];
    const float lo = int4_field(w, 8 * (J & 3)), hi = int4_field(w, 8 * (J & 3) + 4);
    out[h] = (int)__builtin_amdgcn_perm(__builtin_bit_cast(unsigned, hi), __builtin_bit_cast(unsigned, lo), 0x07060302u);
  }
  return out;
}
template <int J>
__device__ __forceinline__ i32x4 column_fragment_i4_scaled(const i32x2 (&rows)[4], float scale) {
  bf16x8 out;
#pragma unroll
  for (int h = 0; h < 4; ++h) {
    const int w = rows[h][J >> 2];
    out[2 * h] = (__bf16)(int4_field(w, 8 * (J & 3)) * scale);
    out[2 * h + 1] = (__bf16)(int4_field(w, 8 * (J & 3) + 4) * scale);
  }
  return __builtin_bit_cast(i32x4, out);
}
// fp8 (e4m3fn) weights: byte J of each row through the hardware conversion; an e4m3 value has 3
// significand bits, so the upper half of its f32 is its bf16 exactly.
template <int J>
__device__ __forceinline__ i32x4 column_fragment_f8(const i32x2 (&rows)[8]) {
  i32x4 out;
#pragma unroll
  for (int h = 0; h < 4; ++h) {
    const unsigned f0 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_f32_fp8(rows[2 * h][J >> 2], J & 3));
    const unsigned f1 = __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_f32_fp8(rows[2 * h + 1][J >> 2], J & 3));
    out[h] = (int)__builtin_amdgcn_perm(f1, f0, 0x07060302u);
  }
  return out;
}
// Sub-channel scales: the same column, each value multiplied by the column's scale of the current
// k-block and rounded to bf16 (nearest even).
template <int EW, int J>
__device__ __forceinline__ i32x4 column_fragment_scaled(const i32x2 (&rows)[8], float scale) {
  bf16x8 out;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    float v;
    if constexpr (EW == kEI8) v = __builtin_bit_cast(float, i8_to_f32_bits<(J & 3)>(rows[e][J >> 2]));
    else v = __builtin_amdgcn_cvt_f32_fp8(rows[e][J >> 2], J & 3);
    out[e] = (__bf16)(v * scale);
  }
  return __builtin_bit_cast(i32x4, out);
}
// 16-bit weights: half-word J of each of 8 loaded 16-byte rows, two rows per byte permute.
template <int J>
__device__ __forceinline__ i32x4 column_fragment_16bit(const i32x4 (&rows)[8]) {
  i32x4 out;
#pragma unroll
  for (int h = 0; h < 4; ++h)
    out[h] = (int)__builtin_amdgcn_perm((unsigned)rows[2 * h + 1][J >> 1], (unsigned)rows[2 * h][J >> 1],
                                        (J & 1) ? 0x07060302u : 0x05040100u);
  return out;
}
// 16x16x32 MFMA on 8 contraction values per lane of either 16-bit type.
template <int EA>
__device__ __forceinline__ f32x4_t mma_16x16x32(i32x4 w, i32x4 a, f32x4_t acc) {
  if constexpr (EA == kEF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, w), __builtin_bit_cast(f16x8, a), acc, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, w), __builtin_bit_cast(bf16x8, a), acc, 0, 0, 0);
}

// EW = element kind of the weights; the lhs is bf16 for int8 weights, else of the weights' type.
// SUB (int8 weights): the scale has several blocks along k; every step fetches the 8 scales of its
// lane's columns for its k-block alongside the weights (the same unconditional pipeline; they come
// from L2, a scale row serves all the weight rows of its block) and the weights are scaled while
// they are widened, instead of one multiply per output in the epilogue.
// CPL = columns per lane; a workgroup covers BN = 16 CPL columns. 16 (int8 only) makes the loads 16
// bytes per lane and the rows a wave reads 256 bytes long, the shape 16-bit weights have at CPL 8.
// SK: the contraction of a (group, column tile) is split over p.split_k workgroups (the finer work items even out
// what each CU streams when a launch has only two or three of the unsplit ones per CU). Each writes its f32
// partial sums to p.partials and announces itself on the tile's counter; the last one to arrive adds the partials
// in the order of the split index (so the result does not depend on who that is), scales and stores. These
// workgroups wait for their group's size before they load any weights: a workgroup's slice is a few steps long,
// and loading ahead of the size would read most of an empty group's weights.
template <int EW, int kDecDepth, int kMinWgs, bool SUB = false, int CPL = 8, bool SK = false>
__global__ __launch_bounds__(kDecThreads, kMinWgs) void decode_kernel(const DecodeParams p) {
  static_assert(!SUB || EW == kEI8 || EW == kEF8 || EW == kEI4, "sub-channel scales belong to int8, int4 or fp8 weights");
  static_assert(CPL == 8 || (CPL == 16 && EW == kEI8 && !SUB), "16 columns per lane: int8 weights with per-column scales");
  constexpr int EA = (EW == kEI8 || EW == kEF8 || EW == kEI4) ? kEBF16 : EW;
  constexpr int KPR = EW == kEI4 ? 2 : 1;  // contraction rows per stored weight row
  constexpr int RPS = 8 / KPR;             // stored rows a lane loads per step
  constexpr int WESZ = WeightRow<EW, CPL>::ESZ;
  constexpr int BN = 16 * CPL;
  typedef typename WeightRow<EW, CPL>::T WRow;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  __shared__ int s_red[kDecWaves];
  __shared__ int s_last;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int splits = SK ? p.split_k : 1;
  const int tile = SK ? (int)blockIdx.x / splits : (int)blockIdx.x;
  const int split = SK ? (int)blockIdx.x - tile * splits : 0;
  const int g = tile / p.n_tiles, nt = tile - g * p.n_tiles;
  const int col0 = nt * BN;
  const bool last_group = g == p.num_groups - 1;

  // Sizes of the groups before this one (for its first row) and its own size are requested first
  // and used last: the first weight steps go out right behind them, before anything is known
  // about the group, so that one memory round trip covers both. A workgroup whose group turns out
  // empty returns with those few loads in flight (32 KB of the group's 1.5 MB, never more).
  // With a group offset the group is entry offset + g of the sizes (entries outside the array count
  // as empty) and the rows of the entries before `offset` are skipped; that costs one more dependent
  // load ahead of the sizes, which the weight loads below overlap as well.
  const int gg = g + (p.group_offset != nullptr ? __builtin_amdgcn_readfirstlane(p.group_offset[0]) : 0);
  const int first_size = p.group_sizes[min(tid, p.num_global - 1)];  // unconditional: no wait until it is used
  const int own_size = gg >= 0 && gg < p.num_global ? max(p.group_sizes[min(max(gg, 0), p.num_global - 1)], 0) : 0;
  const int preceding = min(max(gg, 0), p.num_global);  // entries whose rows come before this group's

  const bool first_of_shard = g == 0 && p.group_offset != nullptr;
  const bool zeroes_rows = split == 0 && (last_group || first_of_shard);  // rows of no group are this workgroup's
  if constexpr (SK) {
    if (__builtin_amdgcn_readfirstlane(own_size) == 0 && !zeroes_rows) return;
  }

  const int kw = p.k / (kDecWaves * splits);  // contraction slice of this wave
  const int k_begin = (split * kDecWaves + wave) * kw;
  const int steps = kw / kDecKS;       // multiple of kDecDepth (checked on the host)
  const unsigned char* wbase = p.rhs + ((int64_t)g * (p.k / KPR) + k_begin / KPR) * p.n * WESZ;
  // B loads: lane (i = lane % 16, q = lane / 16) -> rows 8q + e (e = 0..7), columns col0 + CPL i .. + CPL - 1,
  // clamped at the last CPL columns (n is a multiple of CPL; clamped lanes feed columns that are never stored).
  const int li = lane & 15, lq = lane >> 4;
  int colb = col0 + li * CPL;
  colb = colb < p.n - CPL ? colb : p.n - CPL;
  uint32_t boff[RPS];
#pragma unroll
  for (int e = 0; e < RPS; ++e) boff[e] = (uint32_t)((RPS * lq + e) * p.n + colb) * WESZ;

  WRow breg[kDecDepth][RPS];
  i32x4 areg[kDecDepth];
  i32x4 sreg[SUB ? kDecDepth : 1][2];  // SUB: f32 scales of columns 8i..8i+7 for the step's k-block
  const __amdgpu_buffer_rsrc_t sbuf = buffer_of(SUB ? p.scale + (int64_t)g * p.scale_blocks * p.n : nullptr,
                                                SUB ? (uint32_t)p.scale_blocks * (uint32_t)p.n * 4u : 0u);
  const uint32_t soff = (uint32_t)colb * 4u;
  // Nothing looks at a loaded value before its step comes up, so the only waits are the per-step
  // vmcnt of the oldest group.
  const __amdgpu_buffer_rsrc_t wbuf = buffer_of(wbase, (uint32_t)(kw / KPR) * (uint32_t)p.n * WESZ);
  const uint32_t step_bytes = (uint32_t)(kDecKS / KPR * p.n) * WESZ;
  auto issue_b = [&](int slot, int step) {
    const uint32_t so = (uint32_t)__builtin_amdgcn_readfirstlane((int)(step * step_bytes));
#pragma unroll
    for (int e = 0; e < RPS; ++e) breg[slot][e] = load_weight_row<EW, CPL>(wbuf, boff[e], so);
    if constexpr (SUB) {
      // (Past the wave's slice the block index runs past the buffer and the loads return zero.)
      const uint32_t kb = (uint32_t)(k_begin + step * kDecKS) >> p.log2_block_rows;
      const uint32_t ro = (uint32_t)__builtin_amdgcn_readfirstlane((int)(kb * (uint32_t)p.n * 4u));
      sreg[slot][0] = buffer_load_16(sbuf, soff, ro);
      sreg[slot][1] = buffer_load_16(sbuf, soff + 16u, ro);
    }
  };
#pragma unroll
  for (int d = 0; d < kDecDepth; ++d) {
    issue_b(d, d);
    __builtin_amdgcn_sched_barrier(0);
  }

  // Per-column scales of this thread's CPL epilogue columns, fetched now so that the epilogue does
  // not end on a dependent memory round trip.
  f32x4_t col_scales[CPL / 4];
#pragma unroll
  for (int t = 0; t < CPL / 4; ++t) col_scales[t] = (f32x4_t){1.f, 1.f, 1.f, 1.f};
  {
    const int col = col0 + (tid & 15) * CPL;
    if (!SUB && p.scale != nullptr && col + CPL <= p.n) {
      const float* sc = p.scale + (int64_t)g * p.n + col;
#pragma unroll
      for (int t = 0; t < CPL / 4; ++t) col_scales[t] = *reinterpret_cast<const f32x4_t*>(sc + 4 * t);
    }
  }

  // Row range of this group.
  const int size = __builtin_amdgcn_readfirstlane(own_size);
  if (size == 0 && !last_group && !first_of_shard) return;
  int before = tid < preceding ? max(first_size, 0) : 0;
  for (int j = tid + kDecThreads; j < preceding; j += kDecThreads) before += max(p.group_sizes[j], 0);  // G > 256 only
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) before += __shfl_xor(before, off);
  if (lane == 0) s_red[wave] = before;
  __syncthreads();
  int start = 0;
#pragma unroll
  for (int w = 0; w < kDecWaves; ++w) start += s_red[w];
  start = __builtin_amdgcn_readfirstlane(start);
  const int end = min(start + size, p.m);
  const int esz = p.out_dtype == TKX_F32 ? 4 : 2;

  if (zeroes_rows) {
    // Rows past the last group, and with a group offset the rows before the first, belong to no
    // group of this call: zero this workgroup's columns of them.
    const int ncol = min(BN, p.n - col0);
    const int pieces = ncol * esz / 16;  // 16-byte pieces per row
    unsigned char* c = reinterpret_cast<unsigned char*>(p.out);
    const i32x4 z = {0, 0, 0, 0};
    auto zero_rows = [&](int r0, int r1) {
      for (int idx = tid; idx < (r1 - r0) * pieces; idx += kDecThreads) {
        const int r = r0 + idx / pieces, ch = idx % pieces;
        *reinterpret_cast<i32x4*>(c + ((int64_t)r * p.n + col0) * esz + ch * 16) = z;
      }
    };
    if (last_group) zero_rows(end, p.m);
    if (first_of_shard) zero_rows(0, min(start, p.m));
  }
  if (end <= start) return;  // (every split of a tile takes this exit or none does)

  // lhs rows of this group as one buffer: rows at or past the group's end read as zero.
  const __amdgpu_buffer_rsrc_t abuf = buffer_of(p.lhs + (int64_t)start * p.k * 2, (uint32_t)(end - start) * (uint32_t)p.k * 2u);

  for (int rb = start; rb < end; rb += kDecRows) {
    // A fragments: lane (i, q) holds lhs[rb + i][k + 8q .. 8q+7].
    const uint32_t aoff = (uint32_t)((rb + li - start) * p.k + k_begin + 8 * lq) * 2u;
    auto issue_a = [&](int slot, int step) { areg[slot] = buffer_load_16(abuf, aoff, (uint32_t)(step * (kDecKS * 2))); };

    f32x4_t acc[CPL];
#pragma unroll
    for (int j = 0; j < CPL; ++j) acc[j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

#pragma unroll
    for (int d = 0; d < kDecDepth; ++d) {
      issue_a(d, d);
      __builtin_amdgcn_sched_barrier(0);
    }

    // One block = kDecDepth steps, each consuming its slot and refilling it kDecDepth steps ahead.
    // The first block is peeled off the loop: it consumes loads in the order the prologue issued
    // them (all weight steps, then all lhs steps), while its refills establish the steady-state
    // order (weights, lhs, weights, lhs, ...) that the loop then sees on entry and on its back edge,
    // so every wait inside the loop is a partial vmcnt that leaves the younger steps in flight.
    auto block = [&](int s0) {
#pragma unroll
      for (int d = 0; d < kDecDepth; ++d) {
        const int s = s0 + d;
        const i32x4 afrag = areg[d];
        // MFMA j contracts this step's 32 rows for the columns {CPL i + j}; operands are swapped, so a
        // lane ends up with one lhs row and the weight-column indices 4q..4q+3.
        float col_scale[8];  // SUB: scales of the lane's 8 columns for this step's k-block
        if constexpr (SUB) {
          const f32x4_t s_lo = __builtin_bit_cast(f32x4_t, sreg[d][0]), s_hi = __builtin_bit_cast(f32x4_t, sreg[d][1]);
          col_scale[0] = s_lo[0]; col_scale[1] = s_lo[1]; col_scale[2] = s_lo[2]; col_scale[3] = s_lo[3];
          col_scale[4] = s_hi[0]; col_scale[5] = s_hi[1]; col_scale[6] = s_hi[2]; col_scale[7] = s_hi[3];
        }
        auto column = [&](auto j_tag) {
          constexpr int J = decltype(j_tag)::value;
          if constexpr (SUB && EW == kEI4) return column_fragment_i4_scaled<J>(breg[d], col_scale[J]);
          else if constexpr (SUB) return column_fragment_scaled<EW, J>(breg[d], col_scale[J]);
          else if constexpr (EW == kEI4) return column_fragment_i4<J>(breg[d]);
          else if constexpr (EW == kEI8) return column_fragment_i8<J>(breg[d]);
          else if constexpr (EW == kEF8) return column_fragment_f8<J>(breg[d]);
          else return column_fragment_16bit<J>(breg[d]);
        };
        // Four columns at a time: widen, then their MFMAs.
        auto quad = [&](auto q_tag, auto before_mfma) {
          constexpr int Q = decltype(q_tag)::value;
          i32x4 frag[4];
          frag[0] = column(std::integral_constant<int, 4 * Q + 0>{});
          frag[1] = column(std::integral_constant<int, 4 * Q + 1>{});
          frag[2] = column(std::integral_constant<int, 4 * Q + 2>{});
          frag[3] = column(std::integral_constant<int, 4 * Q + 3>{});
          before_mfma();
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[4 * Q + j] = mma_16x16x32<EA>(frag[j], afrag, acc[4 * Q + j]);
        };
        auto nothing = [] {};
        // Refill unconditionally: past the wave's slice the weight buffer reads as zero without
        // touching memory, and a uniform loop body keeps the waits partial. The refill goes out once
        // the last of the slot's registers have been widened; the scheduling fences keep the compiler
        // from sinking the loads to the end of the block, which would collapse the pipeline to a
        // single step in flight.
        auto refill = [&] {
          __builtin_amdgcn_sched_barrier(0);
          issue_b(d, s + kDecDepth);
          __builtin_amdgcn_sched_barrier(0);
        };
        quad(std::integral_constant<int, 0>{}, nothing);
        if constexpr (CPL == 16) {
          quad(std::integral_constant<int, 1>{}, nothing);
          quad(std::integral_constant<int, 2>{}, nothing);
        }
        quad(std::integral_constant<int, CPL / 4 - 1>{}, refill);
        // The lhs refill goes into the registers the MFMAs above read, so it follows them.
        __builtin_amdgcn_sched_barrier(0);
        issue_a(d, s + kDecDepth);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    block(0);
#pragma unroll 1
    for (int s0 = kDecDepth; s0 < steps; s0 += kDecDepth) block(s0);

    // Cross-wave reduction in a fixed order. acc[j][r] of lane (i, q) is row i, column CPL (4 q + r) + j.
    float* part = reinterpret_cast<float*>(smem) + wave * (kDecRows * BN);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float* dst = part + li * BN + CPL * (4 * lq + r);
#pragma unroll
      for (int t = 0; t < CPL / 4; ++t)
        *reinterpret_cast<f32x4_t*>(dst + 4 * t) = (f32x4_t){acc[4 * t][r], acc[4 * t + 1][r], acc[4 * t + 2][r], acc[4 * t + 3][r]};
    }
    __syncthreads();
    {
      const int r = tid >> 4, c0 = (tid & 15) * CPL;  // 16 rows x 16 runs of CPL columns = 256 threads
      const int row = rb + r, col = col0 + c0;
      if (row < end && col + CPL <= p.n) {
        const int64_t idx = (int64_t)row * p.n + col;
#pragma unroll
        for (int t = 0; t < CPL / 4; ++t) {
          f32x4_t v = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int w = 0; w < kDecWaves; ++w)
            v += *reinterpret_cast<const f32x4_t*>(reinterpret_cast<const float*>(smem) + w * (kDecRows * BN) + r * BN + c0 + 4 * t);
          if constexpr (SK) {
            // Stores of device scope: they go through to memory instead of staying in this XCD's L2, so that no
            // write-back of the whole L2 is needed before the arrival below.
            float* dst = p.partials + ((int64_t)split * p.m * p.n + idx + 4 * t);
#pragma unroll
            for (int i = 0; i < 4; ++i) __hip_atomic_store(dst + i, v[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            continue;
          }
          v *= col_scales[t];
          store4(p.out, idx + 4 * t,
                 (f32x4){apply_activation(v[0], p.activation), apply_activation(v[1], p.activation),
                         apply_activation(v[2], p.activation), apply_activation(v[3], p.activation)},
                 p.out_dtype);
        }
      }
    }
    __syncthreads();  // partials are consumed before the next pass overwrites them
    if (rb + kDecRows < end) {
      // Groups with more than 16 rows stream their panel again for the next 16.
#pragma unroll
      for (int d = 0; d < kDecDepth; ++d) {
        issue_b(d, d);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  if constexpr (SK) {
    // Arrival: every thread waits for its partial sums to be written (a fence of workgroup scope is that wait and
    // nothing else; the stores themselves were of device scope) before thread 0 counts this workgroup in.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    if (tid == 0) {
      int32_t* counter = p.counters + tile;
      const int arrived = atomicAdd(counter, 1);
      s_last = arrived == splits - 1;
      if (arrived == splits - 1) atomicExch(counter, 0);  // nobody else touches it any more in this launch
    }
    __syncthreads();
    if (!s_last) return;
    // The partial sums are read with loads of device scope, which do not take a line this XCD's L2 may hold.
    const int c0 = (tid & 15) * CPL, col = col0 + c0;
    if (col + CPL > p.n) return;
    for (int row = start + (tid >> 4); row < end; row += kDecRows) {
      const int64_t idx = (int64_t)row * p.n + col;
#pragma unroll
      for (int t = 0; t < CPL / 4; ++t) {
        f32x4_t v = {0.f, 0.f, 0.f, 0.f};
        for (int sp = 0; sp < splits; ++sp) {
          const float* src = p.partials + ((int64_t)sp * p.m * p.n + idx + 4 * t);
#pragma unroll
          for (int i = 0; i < 4; ++i) v[i] += __hip_atomic_load(src + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        v *= col_scales[t];
        store4(p.out, idx + 4 * t,
               (f32x4){apply_activation(v[0], p.activation), apply_activation(v[1], p.activation),
                       apply_activation(v[2], p.activation), apply_activation(v[3], p.activation)},
               p.out_dtype);
      }
    }
  }
}

}  // namespace

constexpr int64_t kDecCounterWords = 64 * 1024;  // arrival counters of the split form: a fixed share of its workspace

// Whether the decode kernel can run this problem (else the caller uses the tiled kernel). `depth` steps of loads in
// flight per wave, `split_k` workgroups per (group, column tile).
bool decode_supported(int32_t lhs_dtype, int32_t rhs_dtype, int64_t m, int64_t k, int64_t n, int64_t G,
                      int64_t scale_blocks, int32_t block_n, int32_t depth, int32_t split_k) {
  // The lhs rows of a group are addressed through one buffer with 32-bit byte offsets (a group may hold all m rows).
  if (m * k * 2 >= (1LL << 32)) return false;
  if (split_k < 1 || split_k > 16 || depth < 1) return false;
  if (block_n != kDecBN) {
    // The wide kernel: int8 weights with per-column scales, 16 columns per lane, no split.
    if (block_n != 2 * kDecBN || rhs_dtype != TKX_I8 || scale_blocks != 1 || n % 16 != 0 || split_k != 1) return false;
  }
  if (split_k > 1 && (depth > 4 || G * ((n + block_n - 1) / block_n) > kDecCounterWords)) return false;
  if (scale_blocks != 1) {
    // Sub-channel scales: int8 weights, blocks of a power-of-two number of rows that whole steps fit.
    if ((rhs_dtype != TKX_I8 && rhs_dtype != TKX_F8E4M3FN && rhs_dtype != TKX_I4X2) || scale_blocks < 1 || k % scale_blocks != 0) return false;
    const int64_t rows = k / scale_blocks;
    if (rows % kDecKS != 0 || (rows & (rows - 1)) != 0 || scale_blocks * n * 4 >= (1LL << 31)) return false;
  }
  const bool types = (lhs_dtype == TKX_BF16 && (rhs_dtype == TKX_I8 || rhs_dtype == TKX_F8E4M3FN || rhs_dtype == TKX_BF16 ||
                                                rhs_dtype == TKX_I4X2)) ||
                     (lhs_dtype == TKX_F16 && rhs_dtype == TKX_F16);
  if (!types) return false;
  if (rhs_dtype == TKX_I4X2 && (block_n != kDecBN || (split_k > 1 && depth > 4))) return false;
  const int64_t wesz = (rhs_dtype == TKX_BF16 || rhs_dtype == TKX_F16) ? 2 : 1;
  if ((k / kDecWaves) * n * wesz >= (1LL << 31)) return false;
  // Every wave's slice is a whole number of pipeline rounds. (Unsplit: 1024, whatever the depth, as it always was.)
  const int64_t round = split_k == 1 ? kDecWaves * kDecKS * 8 : (int64_t)kDecWaves * split_k * kDecKS * (depth <= 2 ? 2 : 4);
  return k % round == 0 && n % 8 == 0 && n >= 8;
}

// Words of workspace the split form needs: the tiles' arrival counters, then the partial sums. The counters take
// the same number of words whatever the shapes, so that calls of different shapes can share one workspace without
// one call's partial sums landing where another expects zeroed counters.
int64_t decode_split_counter_words() { return kDecCounterWords; }
int64_t decode_split_workspace_words(int64_t m, int64_t n, int32_t split_k) {
  if (split_k <= 1) return 0;
  return kDecCounterWords + (int64_t)split_k * m * n;
}

namespace {
template <int EW, int D, int W, bool SUB = false>
const void* decode_fn(bool split) {
  return split ? reinterpret_cast<const void*>(&decode_kernel<EW, D, W, SUB, 8, true>)
               : reinterpret_cast<const void*>(&decode_kernel<EW, D, W, SUB, 8, false>);
}
}  // namespace

int32_t launch_decode(const void* lhs, const void* rhs, const float* scale, const int32_t* group_sizes, void* out,
                      int64_t m, int64_t k, int64_t n, int64_t G, int32_t rhs_dtype, int32_t out_dtype,
                      int32_t activation, int32_t depth, int64_t scale_blocks, int32_t block_n,
                      const int32_t* group_offset, int64_t num_global, int32_t split_k, int32_t* split_workspace,
                      hipStream_t stream) {
  DecodeParams p;
  p.group_offset = group_offset;
  p.num_global = (int32_t)num_global;
  p.scale_blocks = (int32_t)scale_blocks;
  p.log2_block_rows = 0;
  for (int64_t rows = k / scale_blocks; rows > 1; rows >>= 1) ++p.log2_block_rows;
  const bool sub = scale_blocks > 1 && scale != nullptr;
  const bool sk = split_k > 1;
  p.lhs = static_cast<const unsigned char*>(lhs);
  p.rhs = static_cast<const unsigned char*>(rhs);
  p.scale = scale;
  p.group_sizes = group_sizes;
  p.out = out;
  p.m = (int32_t)m;
  p.k = (int32_t)k;
  p.n = (int32_t)n;
  p.num_groups = (int32_t)G;
  p.n_tiles = (int32_t)((n + block_n - 1) / block_n);
  p.out_dtype = out_dtype;
  p.activation = activation;
  p.split_k = sk ? split_k : 1;
  p.counters = sk ? split_workspace : nullptr;
  p.partials = sk ? reinterpret_cast<float*>(split_workspace + kDecCounterWords) : nullptr;
  if (sk && split_workspace == nullptr) return set_error(TKX_ERR_INVALID, "a split contraction needs its workspace");
  // Dynamic LDS holds only the four partial tiles of the cross-wave reduction (4 x 16 x 128 f32 = 32 KB;
  // 64 KB for the wide kernel).
  const size_t smem = (size_t)kDecWaves * kDecRows * block_n * 4;
  const int64_t grid = G * p.n_tiles * p.split_k;
  if (grid > 0x7fffffffLL) return set_error(TKX_ERR_UNSUPPORTED, "too many workgroups");
  // `depth` = steps of loads in flight per wave; deeper pipelines need more registers and allow
  // fewer waves per CU. A step of 16-bit weights takes twice the registers of an int8 one.
  const void* fn;
  if (rhs_dtype == TKX_I4X2 && sub) {
    fn = depth <= 2 ? decode_fn<kEI4, 2, 4, true>(sk) : decode_fn<kEI4, 4, 3, true>(sk);
  } else if (rhs_dtype == TKX_I4X2) {
    // Half the registers of int8 per step in flight: the same occupancy one depth further.
    fn = depth <= 2   ? decode_fn<kEI4, 2, 4>(sk)
         : depth <= 4 ? decode_fn<kEI4, 4, 4>(sk)
                      : reinterpret_cast<const void*>(&decode_kernel<kEI4, 8, 3>);
  } else if (sub && rhs_dtype == TKX_F8E4M3FN) {
    fn = depth <= 2 ? decode_fn<kEF8, 2, 3, true>(sk) : decode_fn<kEF8, 4, 2, true>(sk);
  } else if (rhs_dtype == TKX_F8E4M3FN) {
    fn = depth <= 2 ? decode_fn<kEF8, 2, 4>(sk) : decode_fn<kEF8, 4, 3>(sk);
  } else if (sub) {
    fn = depth <= 2 ? decode_fn<kEI8, 2, 3, true>(sk) : decode_fn<kEI8, 4, 2, true>(sk);  // (8 deep would spill)
  } else if (rhs_dtype == TKX_I8 && block_n == 2 * kDecBN) {
    fn = depth <= 2 ? reinterpret_cast<const void*>(&decode_kernel<kEI8, 2, 2, false, 16>)
                    : reinterpret_cast<const void*>(&decode_kernel<kEI8, 4, 1, false, 16>);  // (2 workgroups per CU would spill)
  } else if (rhs_dtype == TKX_I8) {
    fn = depth <= 2   ? decode_fn<kEI8, 2, 4>(sk)
         : depth <= 4 ? decode_fn<kEI8, 4, 3>(sk)
                      : reinterpret_cast<const void*>(&decode_kernel<kEI8, 8, 2>);
  } else if (rhs_dtype == TKX_BF16) {
    fn = depth <= 2 ? decode_fn<kEBF16, 2, 3>(sk) : decode_fn<kEBF16, 4, 2>(sk);
  } else {
    fn = depth <= 2 ? decode_fn<kEF16, 2, 3>(sk) : decode_fn<kEF16, 4, 2>(sk);
  }
  if (smem + 64 > 64 * 1024) {
    // Past the default limit of dynamic LDS: raised once per (device, kernel).
    static std::mutex mu;
    static std::vector<std::pair<int, const void*>> raised;
    int dev = 0;
    TKX_HIP_CHECK(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(mu);
    bool found = false;
    for (auto& r : raised) found = found || (r.first == dev && r.second == fn);
    if (!found) {
      TKX_HIP_CHECK(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
      raised.emplace_back(dev, fn);
    }
  }
  DecodeParams params = p;
  void* args[] = {&params};
  TKX_HIP_CHECK(hipLaunchKernel(fn, dim3((unsigned)grid), dim3(kDecThreads), args, smem, stream));
  return TKX_OK;
}

}  // namespace tkx
