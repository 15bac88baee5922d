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

#include <cstdio>
#include <cstdlib>
#include <mutex>

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
  // Persistent form: whether the workgroups of empty groups help (the host clears it when the grid is not resident
  // as a whole), and how many steps less than a home workgroup a helper gets.
  int32_t helpers, margin;
  int32_t lds_bytes;  // dynamic LDS of the launch
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

// (kEI4, packed int4 weights: a stored row holds two contraction rows)

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
    // Arrival: every thread waits until its own partial-sum stores have completed (`s_waitcnt vmcnt(0)`: the stores
    // were of device scope, so completion means they are visible to every XCD) before the barrier behind which
    // thread 0 counts this workgroup in. The fence only keeps the compiler from moving the stores past this point;
    // at workgroup scope it emits no wait of its own. This ordering leans on the hardware's behaviour (a completed
    // device-scope store is visible to a later device-scope load), not on a release/acquire pair of the HIP memory
    // model: an agent-scope release would write the whole L2 back, once per workgroup.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
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

// ---- the persistent form: workgroups of empty groups help --------------------------------------------------
// The launch above gives every (group, column tile) a workgroup, and the workgroups of empty groups return: what a CU
// then streams depends on how many non-empty tiles it was dealt (two or three of 262 KB on the Qwen3-like decode
// shape), and the launch takes as long as the fullest CU. Here the grid is the same and all of it is resident at
// once, but the workgroup of an empty group stays and takes a share of the others' weight bytes:
//   * the "home" workgroup of a non-empty tile contracts the first h of its tile's k / 32 steps (a step = 32
//     contraction rows = 4 KB of int8 weights). It starts them at once, before it knows anything about the groups,
//     exactly as the kernel above does; its waves take the steps in turn (step s belongs to wave s % 4), so that
//     the first loads do not depend on h;
//   * the remaining r = k / 32 - h steps of all non-empty tiles, listed tile by tile, are cut into equal contiguous
//     ranges, one per WAVE of a "helper" (the workgroup of an empty group's tile). A helper wave contracts its
//     pieces one after the other with its loads in flight across the piece boundaries, writes each piece's f32
//     partial tile to the workspace (stores of device scope) and, when all are written, adds each piece's steps to
//     the counter of the tile's home workgroup. No barrier, no LDS: the waves of a helper do not meet;
//   * h is chosen so that a helper wave has `margin` steps less to do than a home wave: when the home workgroup has
//     reduced its own part, its counter normally reads r already. It waits for that (a bounded spin), adds the
//     pieces in a fixed order (so the bits do not depend on timing), scales, stores and clears the counter.
// Every wave derives all of this from the group sizes itself (4 groups per lane, two wave scans). A launch in which
// a group has more than 16 rows, or no group is empty, runs as the kernel above does (every home workgroup contracts
// its whole tile, pass by pass), and so does one whose grid the device cannot hold at once (decided on the host): a
// home workgroup must never wait for a helper that has no CU to run on. Should a helper not arrive within the spin
// bound all the same, the home workgroup contracts the tail itself; the counter protocol below returns every counter
// to zero in either case.
constexpr int kPersistGroupsPerLane = 4;
constexpr int kPersistMaxGroups = 64 * kPersistGroupsPerLane;
constexpr int kPersistMaxWgs = 1024;
constexpr int kPersistMaxPieces = 4;                   // partial tiles a home workgroup may have to add
constexpr int kPersistSlotFloats = kDecRows * kDecBN;  // one partial tile
constexpr int kPersistGaveUp = 1 << 24;                // added to a counter by a home workgroup that stopped waiting
constexpr int kPersistSpinLimit = 1 << 18;
constexpr int kPersistCounterStride = 64;              // words between two counters: one 256-byte piece of memory each, so
                                                       // that the polling of many home workgroups spreads over the channels

__device__ __forceinline__ int wave_inclusive_scan(int v, int lane) {
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int t = __shfl_up(v, off);
    if (lane >= off) v += t;
  }
  return v;
}

template <int EW, int kDecDepth, int kMinWgs>
__global__ __launch_bounds__(kDecThreads, kMinWgs) void decode_persistent_kernel(const DecodeParams p) {
  constexpr int EA = (EW == kEI8 || EW == kEF8 || EW == kEI4) ? kEBF16 : EW;
  constexpr int KPR = EW == kEI4 ? 2 : 1;
  constexpr int RPS = 8 / KPR;
  constexpr int CPL = 8, BN = kDecBN;
  constexpr int WESZ = WeightRow<EW, CPL>::ESZ;
  typedef typename WeightRow<EW, CPL>::T WRow;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  __shared__ int s_start[kPersistMaxGroups], s_rows[kPersistMaxGroups], s_rank[kPersistMaxGroups];
  __shared__ int s_flag, s_seen[kDecWaves];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int li = lane & 15, lq = lane >> 4;
  const int b = (int)blockIdx.x, n_tiles = p.n_tiles, KS = p.k / kDecKS;
  const int g = b / n_tiles, nt = b - g * n_tiles;

  // t = 0: the group sizes (the whole table) ...
  const int goff = p.group_offset != nullptr ? __builtin_amdgcn_readfirstlane(p.group_offset[0]) : 0;
  int sz[kPersistGroupsPerLane];
#pragma unroll
  for (int j = 0; j < kPersistGroupsPerLane; ++j) {
    const int gj = lane * kPersistGroupsPerLane + j, gg = gj + goff;
    const bool ok = gj < p.num_groups && gg >= 0 && gg < p.num_global;
    const int v = p.group_sizes[min(max(gg, 0), p.num_global - 1)];
    sz[j] = ok ? max(v, 0) : 0;
  }

  // A segment of a wave's work: `count` steps s0, s0 + stride, ... of one tile, contracted with 16 lhs rows. The
  // tile's weights are one buffer that ends behind the segment's last step (steps past it read zero without touching
  // memory: the buffer's range check counts the scalar offset in), the lhs rows another. Lane (i, q) holds columns
  // 8 i .. 8 i + 7 of the weight rows 8 q .. 8 q + 7 of a step: one lane offset, the row inside the step goes into
  // the scalar offset.
  struct Seg {
    __amdgpu_buffer_rsrc_t wbuf, abuf;
    uint32_t voff;
    int s0, stride, count;
  };
  const uint32_t row_bytes = (uint32_t)p.n * WESZ, step_bytes = (uint32_t)(kDecKS / KPR) * row_bytes;
  const uint32_t aoff = (uint32_t)(li * p.k + 8 * lq) * 2u;
  auto set_weights = [&](Seg& sg, int tg, int tnt, int s0, int stride, int count) {
    sg.s0 = s0;
    sg.stride = stride;
    sg.count = count;
    const int bound = count > 0 ? s0 + stride * (count - 1) + 1 : 0;
    sg.wbuf = buffer_of(p.rhs + (int64_t)tg * (p.k / KPR) * row_bytes, (uint32_t)bound * step_bytes);
    int colb = tnt * BN + li * CPL;
    colb = colb < p.n - CPL ? colb : p.n - CPL;
    sg.voff = (uint32_t)(RPS * lq) * row_bytes + (uint32_t)colb * WESZ;
  };
  auto set_rows = [&](Seg& sg, int rb, int nrows) {  // (rows past the last one read zero)
    sg.abuf = buffer_of(p.lhs + (int64_t)rb * p.k * 2, (uint32_t)max(nrows, 0) * (uint32_t)p.k * 2u);
  };
  WRow breg[kDecDepth][RPS];
  i32x4 areg[kDecDepth];
  auto issue_b = [&](int slot, const Seg& sg, int ord) {
    const uint32_t so = (uint32_t)__builtin_amdgcn_readfirstlane((sg.s0 + sg.stride * ord) * (int)step_bytes);
#pragma unroll
    for (int e = 0; e < RPS; ++e) breg[slot][e] = load_weight_row<EW, CPL>(sg.wbuf, sg.voff, so + (uint32_t)e * row_bytes);
  };
  auto issue_a = [&](int slot, const Seg& sg, int ord) {
    areg[slot] = buffer_load_16(sg.abuf, aoff, (uint32_t)((sg.s0 + sg.stride * ord) * (kDecKS * 2)));
  };

  // ... and the home tile's first steps, before anything is known about the groups.
  Seg home;
  set_weights(home, g, nt, wave, kDecWaves, (KS - wave + kDecWaves - 1) / kDecWaves);
#pragma unroll
  for (int d = 0; d < kDecDepth; ++d) {
    issue_b(d, home, d);
    __builtin_amdgcn_sched_barrier(0);
  }

  // The group table: lane l holds groups 4 l .. 4 l + 3.
  int lead = 0;  // rows of the entries before this shard's first group
  if (p.group_offset != nullptr) {
    const int pre = min(max(goff, 0), p.num_global);
    for (int j = lane; j < pre; j += 64) lead += max(p.group_sizes[j], 0);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) lead += __shfl_xor(lead, off);
    lead = min(__builtin_amdgcn_readfirstlane(lead), p.m);
  }
  int ne_incl[kPersistGroupsPerLane];  // non-empty groups up to and including this one
  int nonempty_groups, total_end;
  bool any_tall;
  {
    const int mine = sz[0] + sz[1] + sz[2] + sz[3];
    int run = wave_inclusive_scan(mine, lane) - mine + lead;
    int st[kPersistGroupsPerLane], rows[kPersistGroupsPerLane];
    int nmine = 0, tall = 0;
#pragma unroll
    for (int j = 0; j < kPersistGroupsPerLane; ++j) {
      st[j] = min(run, p.m);
      run = (int)min((int64_t)run + sz[j], (int64_t)p.m);  // (sizes are unchecked device data: no overflow)
      rows[j] = run - st[j];
      nmine += rows[j] > 0;
      tall |= rows[j] > kDecRows;
    }
    const int nincl = wave_inclusive_scan(nmine, lane);
    int nrun = nincl - nmine;
#pragma unroll
    for (int j = 0; j < kPersistGroupsPerLane; ++j) {
      const int gj = lane * kPersistGroupsPerLane + j;
      if (wave == 0) {
        s_start[gj] = st[j];
        s_rows[gj] = rows[j];
        s_rank[gj] = nrun;  // non-empty groups before this one
      }
      nrun += rows[j] > 0;
      ne_incl[j] = nrun;
    }
    nonempty_groups = __builtin_amdgcn_readlane(nincl, 63);
    total_end = __builtin_amdgcn_readlane(run, 63);  // end of the last group, clipped to m
    any_tall = __ballot(tall != 0) != 0;
  }
  __syncthreads();
  const int start = __builtin_amdgcn_readfirstlane(s_start[g]), own_rows = __builtin_amdgcn_readfirstlane(s_rows[g]);
  const int rank = __builtin_amdgcn_readfirstlane(s_rank[g]);

  // Shares. T tiles have a home workgroup, the waves of E workgroups help. A home wave contracts h / 4 steps, a helper
  // wave at most Rw, `margin` fewer.
  const int T = nonempty_groups * n_tiles, E = (p.num_groups - nonempty_groups) * n_tiles;
  const bool helping = p.helpers != 0 && !any_tall && E > 0 && T > 0;
  int h = KS, r = 0, Rw = 1;
  if (helping) {
    h = min(KS, (T * KS + E * kDecWaves * p.margin + T + E - 1) / (T + E));
    r = KS - h;
    // (A tail is cut into at most kPersistMaxPieces - 1 whole ranges plus one: with more helpers than that the
    // surplus ones get nothing.)
    Rw = max(max((T * r + kDecWaves * E - 1) / (kDecWaves * E), (r + kPersistMaxPieces - 2) / (kPersistMaxPieces - 1)), 1);
  }

  // Rows of no group (past the last group, and with a group offset before the first) are zero: the workgroups of the
  // last group and of the shard's first group clear their columns of them.
  {
    const bool last_group = g == p.num_groups - 1, first_of_shard = g == 0 && p.group_offset != nullptr;
    if ((last_group && total_end < p.m) || (first_of_shard && lead > 0)) {
      const int esz = p.out_dtype == TKX_F32 ? 4 : 2;
      const int ncol = min(BN, p.n - nt * BN);
      const int pieces = ncol * esz / 16;  // 16-byte pieces per row
      unsigned char* c = reinterpret_cast<unsigned char*>(p.out);
      const i32x4 z = {0, 0, 0, 0};
      auto zero_rows = [&](int r0, int r1) {
        for (int idx = tid; idx < (r1 - r0) * pieces; idx += kDecThreads) {
          const int rr = r0 + idx / pieces, ch = idx % pieces;
          *reinterpret_cast<i32x4*>(c + ((int64_t)rr * p.n + nt * BN) * esz + ch * 16) = z;
        }
      };
      if (last_group) zero_rows(total_end, p.m);
      if (first_of_shard) zero_rows(0, lead);
    }
  }

  // Streams segments seg(0), seg(1), ... of this wave one after the other with kDecDepth steps of loads in flight
  // throughout: the last steps of a segment refill their slots from the next one. flush(i, acc) is called with the
  // sums of segment i (acc[j][r] of lane (i, q) is lhs row i, tile column 8 (4 q + r) + j) and says whether another
  // segment follows. `b_out`: the first segment's first weight loads have been issued.
  auto stream = [&](Seg cur, bool b_out, auto more_after, auto seg, auto flush, auto before_block) {
    bool a_out = false;
    for (int i = 0;; ++i) {
      if (!b_out) {
#pragma unroll
        for (int d = 0; d < kDecDepth; ++d) {
          issue_b(d, cur, d);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      if (!a_out) {
#pragma unroll
        for (int d = 0; d < kDecDepth; ++d) {
          issue_a(d, cur, d);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      const bool has_next = more_after(i);
      Seg nxt = cur;
      if (has_next) nxt = seg(i + 1);
      f32x4_t acc[CPL];
#pragma unroll
      for (int j = 0; j < CPL; ++j) acc[j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
      // One block = kDecDepth steps, each consumed from its slot, which is then refilled with the step kDecDepth
      // further on: of this segment, or (in its last block) of the next one. The share is rounded up to whole blocks;
      // the surplus steps multiply a cleared lhs fragment (and read no memory).
      const int nblk = (cur.count + kDecDepth - 1) / kDecDepth;
      auto block = [&](int blk) {
        const bool to_next = has_next && blk + 1 == nblk;
        const Seg& rs = to_next ? nxt : cur;
        const int rord = to_next ? 0 : (blk + 1) * kDecDepth;
#pragma unroll
        for (int d = 0; d < kDecDepth; ++d) {
          const i32x4 zero = {0, 0, 0, 0};
          const i32x4 afrag = blk * kDecDepth + d < cur.count ? areg[d] : zero;
          auto column = [&](auto j_tag) {
            constexpr int J = decltype(j_tag)::value;
            if constexpr (EW == kEI4) return column_fragment_i4<J>(breg[d]);
            else if constexpr (EW == kEI8) return column_fragment_i8<J>(breg[d]);
            else if constexpr (EW == kEF8) return column_fragment_f8<J>(breg[d]);
            else return column_fragment_16bit<J>(breg[d]);
          };
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
          auto refill = [&] {
            __builtin_amdgcn_sched_barrier(0);
            issue_b(d, rs, rord + d);
            __builtin_amdgcn_sched_barrier(0);
          };
          quad(std::integral_constant<int, 0>{}, nothing);
          quad(std::integral_constant<int, 1>{}, refill);
          // The lhs refill goes into the registers the MFMAs above read, so it follows them.
          __builtin_amdgcn_sched_barrier(0);
          issue_a(d, rs, rord + d);
          __builtin_amdgcn_sched_barrier(0);
        }
      };
      // (The first block is peeled: it takes its loads in the order the code before it issued them, the loop's
      // blocks in the order a block's refills establish, so the loop's waits stay partial.)
      if (nblk > 0) {
        block(0);
#pragma unroll 1
        for (int blk = 1; blk < nblk; ++blk) {
          before_block(blk, nblk);
          block(blk);
        }
      }
      if (!flush(i, acc)) return;
      if (has_next) {
        cur = nxt;
        b_out = a_out = nblk > 0;  // (the last block's refills were the next segment's first loads)
      } else {
        cur = seg(i + 1);  // (a segment that flush() decided on)
        b_out = a_out = false;
      }
    }
  };
  const int row = tid >> 4, c0 = (tid & 15) * CPL;  // the thread's place in a 16 x 128 tile: 16 rows x 16 runs of CPL columns

  if (own_rows == 0) {
    // ---- helper: this wave's range of the tails [y0, y1), piece by piece ----
    if (!helping || r == 0) return;
    const int jw = ((g - rank) * n_tiles + nt) * kDecWaves + wave;  // this wave's place among the helper waves
    const int64_t y_begin = (int64_t)jw * Rw, y_end = (int64_t)T * r;
    if (y_begin >= y_end) return;
    const int y0 = (int)y_begin, y1 = (int)min(y_begin + Rw, y_end);
    // The i-th non-empty group: the number of groups with at most i non-empty ones up to and including them.
    auto nth_nonempty = [&](int i) {
      int cnt = 0;
#pragma unroll
      for (int jj = 0; jj < kPersistGroupsPerLane; ++jj) cnt += __builtin_popcountll(__ballot(ne_incl[jj] <= i));
      return __builtin_amdgcn_readfirstlane(cnt);
    };
    // Piece number i of the range: tails are r steps long, so the first piece may start inside one.
    const int unit0 = y0 / r;
    struct Piece { int unit, tg, tnt, off, len; };
    auto piece = [&](int i) {
      Piece pc;
      pc.unit = unit0 + i;
      const int lo = max(pc.unit * r, y0), hi = min(pc.unit * r + r, y1);
      pc.off = lo - pc.unit * r;
      pc.len = hi - lo;
      const int q = pc.unit / n_tiles;
      pc.tnt = pc.unit - q * n_tiles;
      pc.tg = nth_nonempty(q);
      return pc;
    };
    const int npieces = (y1 - 1) / r - unit0 + 1;
    auto seg_of = [&](int i) {
      const Piece pc = piece(i);
      Seg sg;
      set_weights(sg, pc.tg, pc.tnt, h + pc.off, 1, pc.len);
      set_rows(sg, __builtin_amdgcn_readfirstlane(s_start[pc.tg]), __builtin_amdgcn_readfirstlane(s_rows[pc.tg]));
      return sg;
    };
    // A finished piece's partial tile (the rows that exist) waits in this wave's own part of LDS; what does not fit
    // there goes to the workspace at once. (Stores in the middle of the stream would stand in the same in-order queue
    // as the loads behind them, and stores of device scope are slow to complete.)
    const int lds_per_wave = p.lds_bytes / kDecWaves;
    unsigned char* stage = smem + wave * lds_per_wave;
    int staged_bytes = 0;
    uint32_t staged = 0;  // bit i: piece i waits in LDS
    auto slot_of = [&](const Piece& pc) {
      const int home_wg = pc.tg * n_tiles + pc.tnt;
      const int slot = jw - (int)((int64_t)pc.unit * r / Rw);
      return p.partials + (int64_t)(home_wg * kPersistMaxPieces + slot) * kPersistSlotFloats;
    };
    stream(seg_of(0), false, [&](int i) { return i + 1 < npieces; }, seg_of, [&](int i, const f32x4_t (&acc)[CPL]) {
      const Piece pc = piece(i);
      const int nrows = __builtin_amdgcn_readfirstlane(s_rows[pc.tg]);
      const int bytes = nrows * BN * 4;
      if (i < 32 && staged_bytes + bytes <= lds_per_wave) {
        if (li < nrows) {
          float* dst = reinterpret_cast<float*>(stage + staged_bytes) + li * BN + CPL * 4 * lq;
#pragma unroll
          for (int rr = 0; rr < 4; ++rr)
#pragma unroll
            for (int t = 0; t < CPL / 4; ++t)
              *reinterpret_cast<f32x4_t*>(dst + CPL * rr + 4 * t) = (f32x4_t){acc[4 * t][rr], acc[4 * t + 1][rr], acc[4 * t + 2][rr], acc[4 * t + 3][rr]};
        }
        staged |= 1u << i;
        staged_bytes += bytes;
      } else if (li < nrows) {
        float* dst = slot_of(pc) + li * BN + CPL * 4 * lq;
#pragma unroll
        for (int rr = 0; rr < 4; ++rr)
#pragma unroll
          for (int jj = 0; jj < CPL; ++jj)
            __hip_atomic_store(dst + CPL * rr + jj, acc[jj][rr], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      return i + 1 < npieces;
    }, [](int, int) {});
    // The staged tiles go to their slots: stores of device scope (they go through to memory, not into this XCD's L2).
    {
      int off = 0;
      for (int i = 0; i < npieces && i < 32; ++i) {
        if (((staged >> i) & 1u) == 0) continue;
        const Piece pc = piece(i);
        const int bytes = __builtin_amdgcn_readfirstlane(s_rows[pc.tg]) * BN * 4;
        float* dst = slot_of(pc);
        for (int o = lane * 16; o < bytes; o += 64 * 16) {
          const f32x4_t val = *reinterpret_cast<const f32x4_t*>(stage + off + o);
#pragma unroll
          for (int e = 0; e < 4; ++e) __hip_atomic_store(dst + o / 4 + e, val[e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        off += bytes;
      }
    }
    // Every lane waits until its stores have completed, then the wave counts each piece's steps in at its home
    // workgroup (lane i takes piece i, so that the counters' round trips overlap).
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    for (int i0 = 0; i0 < npieces; i0 += 64) {
      int32_t* counter = nullptr;
      int len = 0;
      for (int i = i0; i < npieces && i < i0 + 64; ++i) {
        const Piece pc = piece(i);  // (by the whole wave: it takes a ballot)
        if (lane == i - i0) {
          counter = p.counters + (pc.tg * n_tiles + pc.tnt) * kPersistCounterStride;
          len = pc.len;
        }
      }
      if (counter != nullptr) {
        const int before = atomicAdd(counter, len);
        // (The home workgroup gave up waiting and everybody has arrived now: the last one clears the counter.)
        if (before + len == kPersistGaveUp + r) atomicExch(counter, 0);
      }
    }
    return;
  }

  // ---- home ----
  const int end = start + own_rows;
  const int passes = (own_rows + kDecRows - 1) / kDecRows;  // (more than one: a group of more than 16 rows streams its tile again)
  f32x4_t col_scales[CPL / 4];
#pragma unroll
  for (int t = 0; t < CPL / 4; ++t) col_scales[t] = (f32x4_t){1.f, 1.f, 1.f, 1.f};
  const int col = nt * BN + c0;
  if (p.scale != nullptr && col + CPL <= p.n) {
    const float* sc = p.scale + (int64_t)g * p.n + col;
#pragma unroll
    for (int t = 0; t < CPL / 4; ++t) col_scales[t] = *reinterpret_cast<const f32x4_t*>(sc + 4 * t);
  }
  bool tail_here = false;  // no helper in sight: this workgroup contracts steps [h, k / 32) as a segment of its own
  f32x4_t head[CPL / 4];
  auto seg_of = [&](int i) {
    Seg sg;
    const int lo = tail_here ? h : 0, hi = tail_here ? KS : h;
    set_weights(sg, g, nt, lo + wave, kDecWaves, max(hi - lo - wave + kDecWaves - 1, 0) / kDecWaves);
    const int rb = start + (tail_here ? 0 : i) * kDecRows;
    set_rows(sg, rb, end - rb);
    return sg;
  };
  // The tail of this tile is the helpers': when the counter of this workgroup reads r, all of it is in the workspace.
  // Every wave takes a first look two blocks before the end of its own steps, so that the answer is there when the
  // steps are done (helpers have less to do and are normally finished by then).
  int32_t* const counter = p.counters + b * kPersistCounterStride;
  int early_look = -1;
  stream(seg_of(0), true, [&](int i) { return i + 1 < passes; }, seg_of, [&](int i, const f32x4_t (&acc)[CPL]) {
    // The four waves' partial tiles meet in LDS and every thread adds up its CPL values of the tile.
    float* part = reinterpret_cast<float*>(smem) + wave * kPersistSlotFloats;
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
      float* dst = part + li * BN + CPL * (4 * lq + rr);
#pragma unroll
      for (int t = 0; t < CPL / 4; ++t)
        *reinterpret_cast<f32x4_t*>(dst + 4 * t) = (f32x4_t){acc[4 * t][rr], acc[4 * t + 1][rr], acc[4 * t + 2][rr], acc[4 * t + 3][rr]};
    }
    const bool waits = r > 0 && !tail_here;
    if (waits && lane == 0) s_seen[wave] = early_look == r;
    __syncthreads();
    const int rb = start + (tail_here ? 0 : i) * kDecRows;
    const bool mine = rb + row < end && col + CPL <= p.n;
    // The pieces of this tile's tail, in the order of the helper waves that wrote them: loads of device scope (they
    // do not take a line this XCD's L2 may hold).
    const int unit = rank * n_tiles + nt;
    const int j0 = (int)((int64_t)unit * r / Rw), j1 = (int)(((int64_t)unit * r + r - 1) / Rw);
    f32x4_t tail_sum[CPL / 4];
#pragma unroll
    for (int t = 0; t < CPL / 4; ++t) tail_sum[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    auto add_pieces = [&] {
      if (mine) {
        for (int slot = 0; slot <= j1 - j0; ++slot) {
          const float* src = p.partials + ((int64_t)(b * kPersistMaxPieces + slot) * kPersistSlotFloats + row * BN + c0);
#pragma unroll
          for (int t = 0; t < CPL / 4; ++t)
#pragma unroll
            for (int ii = 0; ii < 4; ++ii) tail_sum[t][ii] += __hip_atomic_load(src + 4 * t + ii, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    };
    const bool seen_early = waits && (s_seen[0] | s_seen[1] | s_seen[2] | s_seen[3]) != 0;
    if (seen_early) {
      add_pieces();  // (requested before the sums below are read from LDS)
      if (tid == 0) atomicExch(counter, 0);  // nobody else touches it any more in this launch
    }
    f32x4_t v[CPL / 4];
#pragma unroll
    for (int t = 0; t < CPL / 4; ++t) {
      v[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < kDecWaves; ++w)
        v[t] += *reinterpret_cast<const f32x4_t*>(reinterpret_cast<const float*>(smem) + w * kPersistSlotFloats + row * BN + c0 + 4 * t);
    }
    __syncthreads();  // the partial tiles are consumed before the next pass overwrites them
    if (tail_here) {
#pragma unroll
      for (int t = 0; t < CPL / 4; ++t) v[t] += head[t];
    } else if (waits && !seen_early) {
      // Wait until all r steps are counted in.
      if (tid == 0) {
        int seen = __hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (int spin = 0; seen != r && spin < kPersistSpinLimit; ++spin) {
          __builtin_amdgcn_s_sleep(16);
          seen = __hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        if (seen != r) seen = atomicAdd(counter, kPersistGaveUp);  // gave up; (all may have arrived in the meantime)
        if (seen == r) atomicExch(counter, 0);
        s_flag = seen == r;
      }
      __syncthreads();
      if (s_flag == 0) {
        // No helper in sight: contract the tail here, as one more segment.
#pragma unroll
        for (int t = 0; t < CPL / 4; ++t) head[t] = v[t];
        tail_here = true;
        return true;
      }
      add_pieces();
    }
#pragma unroll
    for (int t = 0; t < CPL / 4; ++t) v[t] += tail_sum[t];
    if (mine) {
      const int64_t idx = (int64_t)(rb + row) * p.n + col;
#pragma unroll
      for (int t = 0; t < CPL / 4; ++t) {
        const f32x4_t o = v[t] * col_scales[t];
        store4(p.out, idx + 4 * t,
               (f32x4){apply_activation(o[0], p.activation), apply_activation(o[1], p.activation),
                       apply_activation(o[2], p.activation), apply_activation(o[3], p.activation)},
               p.out_dtype);
      }
    }
    return !tail_here && i + 1 < passes;
  }, [&](int blk, int nblk) {
    if (r > 0 && !tail_here && blk + 2 == nblk) early_look = __hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  });
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

namespace {
__global__ void clear_words_kernel(int32_t* words, int64_t count) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) words[i] = 0;
}
}  // namespace
// Clears the counter block of a split / persistent workspace with a fill kernel (a memset node recorded into a captured
// graph is what callers under capture should not have to rely on).
int32_t launch_clear_decode_counters(int32_t* workspace, hipStream_t stream) {
  clear_words_kernel<<<dim3((unsigned)(kDecCounterWords / 256)), dim3(256), 0, stream>>>(workspace, kDecCounterWords);
  TKX_HIP_CHECK(hipGetLastError());
  return TKX_OK;
}
int64_t decode_split_workspace_words(int64_t m, int64_t n, int32_t split_k) {
  if (split_k <= 1) return 0;
  return kDecCounterWords + (int64_t)split_k * m * n;
}

// Whether the persistent form (the workgroups of empty groups help) can run this problem: one-byte weights (int8, fp8,
// packed int4) under a bf16 lhs with one scale per (group, column), 128-column tiles, at most 256 groups and 1024
// tiles, any k that is a multiple of 32.
bool decode_persistent_supported(int32_t lhs_dtype, int32_t rhs_dtype, int64_t m, int64_t k, int64_t n, int64_t G,
                                 int64_t scale_blocks, int32_t block_n, int32_t depth) {
  if (block_n != kDecBN || scale_blocks != 1 || depth < 1 || depth > 4) return false;
  if (G < 1 || G > kPersistMaxGroups || G * ((n + kDecBN - 1) / kDecBN) > kPersistMaxWgs) return false;
  if (lhs_dtype != TKX_BF16 || (rhs_dtype != TKX_I8 && rhs_dtype != TKX_F8E4M3FN && rhs_dtype != TKX_I4X2)) return false;
  if (k % (rhs_dtype == TKX_I4X2 ? 2 * kDecKS : kDecKS) != 0 || n % 8 != 0 || n < 8) return false;
  // A tile is addressed through one buffer with 32-bit offsets (a few steps past its end included), the lhs rows
  // of a pass likewise.
  return (k + 1024) * n < (1LL << 31) && (int64_t)m * k * 2 < (1LL << 32);
}

// Words of workspace of the persistent form: the arrival counters (the same block as the split form's, zero on
// entry and on exit), then kPersistMaxPieces partial tiles per workgroup.
int64_t decode_persistent_workspace_words() {
  return 64 * 1024 + (int64_t)kPersistMaxWgs * kPersistMaxPieces * kPersistSlotFloats;
}

namespace {
// Raises a kernel's limit of dynamic LDS past the default 64 KB, once per (device, kernel, size). Fixed table: no
// allocation after the library is loaded.
int32_t raise_dynamic_lds(const void* fn, size_t bytes) {
  if (bytes + 4096 <= 64 * 1024) return TKX_OK;
  struct Entry { int dev; const void* fn; size_t bytes; };
  constexpr int kSlots = 512;
  static std::mutex mu;
  static Entry raised[kSlots];
  static int used = 0;
  int dev = 0;
  TKX_HIP_CHECK(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(mu);
  for (int i = 0; i < used; ++i)
    if (raised[i].dev == dev && raised[i].fn == fn && raised[i].bytes >= bytes) return TKX_OK;
  TKX_HIP_CHECK(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
  if (used < kSlots) raised[used++] = {dev, fn, bytes};  // (a full table only means the attribute is set again)
  return TKX_OK;
}

// Steps by which a helper wave's share is smaller than a home wave's, so that its partial tiles are in memory before
// the home workgroup looks for them (a wave of a workgroup that shares a CU with two others takes about 2 us for a
// step of 4 KB), 4 steps (the best of 0..8 measured on the 2048-deep decode shape), at most a quarter of a wave's share of a tile.
int32_t persistent_margin_steps(int64_t k) {
  const int64_t steps = k / kDecKS / kDecWaves;
  int64_t margin = 4;
  if (margin > steps / 4) margin = steps / 4;
  return (int32_t)margin;
}

// Workgroups of a kernel that fit a CU at once with `lds` bytes of dynamic LDS each, as the runtime's occupancy
// calculator sees it; remembered per (device, kernel, lds) in a fixed table.
int32_t resident_workgroups_per_cu(const void* fn, size_t lds, int* out) {
  struct Entry { int dev; const void* fn; size_t lds; int resident; };
  constexpr int kSlots = 256;
  static std::mutex mu;
  static Entry known[kSlots];
  static int used = 0;
  int dev = 0;
  TKX_HIP_CHECK(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(mu);
  for (int i = 0; i < used; ++i)
    if (known[i].dev == dev && known[i].fn == fn && known[i].lds == lds) {
      *out = known[i].resident;
      return TKX_OK;
    }
  int resident = 0;
  TKX_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&resident, fn, kDecThreads, lds));
  if (used < kSlots) known[used++] = {dev, fn, lds, resident};
  *out = resident;
  return TKX_OK;
}

// The persistent kernel for (one-byte weights, depth) that keeps its registers with `wgs_per_cu` workgroups resident per
// CU, or null: 3 per CU at depth 2 (packed int4: 4), 2 at depth 4. (The 16-bit instances spill and are not built.)
template <int EW>
const void* decode_persistent_fn(int depth, int wgs_per_cu) {
  if (depth <= 2) {
    if constexpr (EW == kEI4) {
      if (wgs_per_cu == 4) return reinterpret_cast<const void*>(&decode_persistent_kernel<EW, 2, 4>);
    }
    if (wgs_per_cu <= 3) return reinterpret_cast<const void*>(&decode_persistent_kernel<EW, 2, 3>);
    return nullptr;
  }
  if (wgs_per_cu <= 2) return reinterpret_cast<const void*>(&decode_persistent_kernel<EW, 4, 2>);
  return nullptr;
}
const void* decode_persistent_entry(int32_t rhs_dtype, int depth, int wgs_per_cu) {
  return rhs_dtype == TKX_I4X2       ? decode_persistent_fn<kEI4>(depth, wgs_per_cu)
         : rhs_dtype == TKX_F8E4M3FN ? decode_persistent_fn<kEF8>(depth, wgs_per_cu)
         : rhs_dtype == TKX_I8       ? decode_persistent_fn<kEI8>(depth, wgs_per_cu)
                                     : nullptr;
}

template <int EW, int D, int W, bool SUB = false>
const void* decode_fn(bool split) {
  return split ? reinterpret_cast<const void*>(&decode_kernel<EW, D, W, SUB, 8, true>)
               : reinterpret_cast<const void*>(&decode_kernel<EW, D, W, SUB, 8, false>);
}
}  // namespace

int32_t launch_decode(const void* lhs, const void* rhs, const float* scale, const int32_t* group_sizes, void* out,
                      int64_t m, int64_t k, int64_t n, int64_t G, int32_t rhs_dtype, int32_t out_dtype,
                      int32_t activation, int32_t depth, int64_t scale_blocks, int32_t block_n,
                      const int32_t* group_offset, int64_t num_global, int32_t split_k, int32_t persistent,
                      int32_t* split_workspace, hipStream_t stream) {
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
  p.helpers = 0;
  p.margin = 0;
  p.lds_bytes = 0;
  p.counters = sk ? split_workspace : nullptr;
  p.partials = sk ? reinterpret_cast<float*>(split_workspace + kDecCounterWords) : nullptr;
  if (sk && split_workspace == nullptr) return set_error(TKX_ERR_INVALID, "a split contraction needs its workspace");
  if (persistent > 0) {
    // The workgroups of empty groups help: that needs the whole grid resident at once (a home workgroup waits for
    // its helpers), so every workgroup asks for an equal share of a CU's LDS, which also keeps the hardware from
    // placing more of them on one CU than on another. A grid the device cannot hold runs as the plain kernel.
    if (split_workspace == nullptr) return set_error(TKX_ERR_INVALID, "the persistent form needs its workspace");
    int cus = 0;
    int32_t st = device_compute_units(&cus);
    if (st != TKX_OK) return st;
    const int64_t wgs = G * p.n_tiles;
    const int per_cu = (int)((wgs + cus - 1) / cus);
    const void* fn = per_cu <= 4 ? decode_persistent_entry(rhs_dtype, depth, per_cu) : nullptr;
    // LDS per workgroup: enough less than a 1 / per_cu share of the CU's 160 KB to survive the allocation granule
    // (the kernel's static arrays take 4 KB more), enough more than a 1 / (per_cu + 1) share to keep one more
    // workgroup off the CU. What the runtime's occupancy calculator then says decides.
    size_t lds = (size_t)kDecWaves * kPersistSlotFloats * 4;
    if (fn != nullptr) {
      const size_t share = (size_t)160 * 1024 / (size_t)per_cu, next_share = (size_t)160 * 1024 / (size_t)(per_cu + 1);
      size_t want = (share - 8192) / 1024 * 1024;
      if (want < next_share) want = (share - 5120) / 1024 * 1024;
      if (lds < want) lds = want;
      st = raise_dynamic_lds(fn, lds);
      if (st != TKX_OK) return st;
      int resident = 0;
      st = resident_workgroups_per_cu(fn, lds, &resident);
      if (st != TKX_OK) return st;
      if (resident < per_cu) fn = nullptr;
    }
    if (fn != nullptr) {
      p.split_k = 1;
      p.counters = split_workspace;
      p.partials = reinterpret_cast<float*>(split_workspace + kDecCounterWords);
      p.helpers = 1;
      p.margin = persistent_margin_steps(k);
      p.lds_bytes = (int32_t)lds;
      DecodeParams params = p;
      void* args[] = {&params};
      TKX_HIP_CHECK(hipLaunchKernel(fn, dim3((unsigned)wgs), dim3(kDecThreads), args, lds, stream));
      return TKX_OK;
    }
  }
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
                      : reinterpret_cast<const void*>(&decode_kernel<kEI4, 8, 2>);  // (3 workgroups per CU would spill)
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
    int32_t rst = raise_dynamic_lds(fn, smem);
    if (rst != TKX_OK) return rst;
  }
  DecodeParams params = p;
  void* args[] = {&params};
  TKX_HIP_CHECK(hipLaunchKernel(fn, dim3((unsigned)grid), dim3(kDecThreads), args, smem, stream));
  return TKX_OK;
}

}  // namespace tkx
