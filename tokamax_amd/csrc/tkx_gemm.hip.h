// Grouped (ragged) GEMM for gfx950: one templated kernel behind every dtype / mode.
//
//   C[rows, cols] = sum over the contraction of A(row, kc) * B(kc, col)
//
//   mode kFwd  : A = lhs  [m,k]  contraction-contiguous   B = rhs[g] [k,n]  column-contiguous
//   mode kFwdGlu: as kFwd with B = rhs[g] [k, 2 n] = [gate | up] and C[m,n] = act(A.gate) * (A.up)
//   mode kDlhs : A = dout [m,n]  contraction-contiguous   B = rhs[g] [k,n]  contraction-contiguous
//                (C[m,k] = dout . rhs[g]^T: rhs is read in place, never transposed in memory)
//   mode kDrhs : A = lhs  [m,k]  row(k-index)-contiguous  B = dout [m,n]    column-contiguous
//                (C[g][k,n] = lhs[rows_g]^T . dout[rows_g]; contraction = the group's row range)
//
// A workgroup owns one BM x BN tile of C. k-steps of BK contraction elements are staged through a
// ring of NS LDS stages with direct-to-LDS loads (global_load_lds_dwordx4), all stages in flight: a
// stage is refilled right after the barrier that releases it, between the MFMAs of the step's last
// k-atom, and fragments are double-buffered in registers. Operands that are contraction-contiguous
// are read from LDS with ds_read_b128; operands that are contiguous along the other axis are read
// with the gfx950 transposing LDS loads (ds_read_b64_tr_b16 / _tr_b8), so no operand is ever
// transposed in memory. The 32x32 MFMA is issued with its operands swapped (B-fragment first) so
// that each lane ends up holding runs of 4 consecutive C columns of one C row; the epilogue applies
// scales, bias and activation in registers and writes whole row segments through LDS.
#pragma once

#include <type_traits>

#include "tkx_common.h"

namespace tkx {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
typedef __attribute__((address_space(3))) i32x2 lds_i32x2;

// gfx950 transposing LDS loads (see load_frag for the lane <-> element mapping).
__device__ __forceinline__ i32x2 lds_read_tr16(const unsigned char* p) {
  return __builtin_bit_cast(i32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p)));
}
__device__ __forceinline__ i32x2 lds_read_tr8(const unsigned char* p) {
  return __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_i32x2*)(p));
}

// (kEI4: weights only, two 4-bit values to a byte along the contraction; a tile of them is a tile of bytes half as deep)
enum ElemKind { kEF32 = TKX_F32, kEBF16 = TKX_BF16, kEF16 = TKX_F16, kEF8 = TKX_F8E4M3FN, kEI8 = TKX_I8, kEI4 = TKX_I4X2 };
enum OperandLayout { kKC = 0 /* contraction-contiguous */, kMC = 1 /* contiguous along rows/cols */ };

__host__ __device__ constexpr int elem_bytes(int e) { return e == kEF32 ? 4 : (e == kEBF16 || e == kEF16) ? 2 : 1; }

// MFMA flavour chosen by the A element kind: contraction elements per 32x32 atom and fragment bytes.
template <int EA> struct Mma;
template <> struct Mma<kEBF16> { static constexpr int KA = 16; typedef i32x4 Frag; };
template <> struct Mma<kEF16> { static constexpr int KA = 16; typedef i32x4 Frag; };
template <> struct Mma<kEF32> { static constexpr int KA = 8; typedef i32x4 Frag; };
template <> struct Mma<kEF8> { static constexpr int KA = 64; typedef i32x8 Frag; };
// int8 x int8 -> int32: the accumulator registers hold int32 bits (kept in the f32x16 type the kernel uses).
template <> struct Mma<kEI8> { static constexpr int KA = 32; typedef i32x4 Frag; };

template <int EA>
__device__ __forceinline__ f32x16 mma_atom(const typename Mma<EA>::Frag& first, const typename Mma<EA>::Frag& second,
                                           f32x16 acc) {
  if constexpr (EA == kEBF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, first),
                                                   __builtin_bit_cast(bf16x8, second), acc, 0, 0, 0);
  } else if constexpr (EA == kEF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, first),
                                                  __builtin_bit_cast(f16x8, second), acc, 0, 0, 0);
  } else if constexpr (EA == kEI8) {
    typedef int i32x16_t __attribute__((ext_vector_type(16)));
    return __builtin_bit_cast(f32x16, __builtin_amdgcn_mfma_i32_32x32x32_i8(first, second, __builtin_bit_cast(i32x16_t, acc), 0, 0, 0));
  } else if constexpr (EA == kEF32) {
    f32x4 a = __builtin_bit_cast(f32x4, first), b = __builtin_bit_cast(f32x4, second);
#pragma unroll
    for (int t = 0; t < 4; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t], b[t], acc, 0, 0, 0);
    return acc;
  } else {
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(first, second, acc, 0, 0, 0, 0, 0, 0);
  }
}

// ---- LDS tile addressing ------------------------------------------------------------------------
// Contraction-contiguous tile: [rows][ROW_BYTES], 16-byte chunks XOR-swizzled by the row so that the
// 16 lanes of one ds_read_b128 phase (16 consecutive rows, one chunk each: 256 bytes, every bank
// once) touch distinct banks. A row covers CPR of the 16 chunk slots of a 256-byte bank line, so
// the swizzle has to tell apart the 16 / CPR rows that start on the same slot: with 4 chunks per
// row those are rows r, r + 4, r + 8, r + 12 (row bits 2 and 3), with 8 chunks per row r, r + 2, ...
template <int ROW_BYTES>
__device__ __forceinline__ int kc_swizzle(int row) {
  constexpr int CPR = ROW_BYTES / 16;
  if constexpr (CPR == 4) return (row >> 2) & 3;
  else return ((row & 7) ^ ((row >> 3) & 1)) & (CPR - 1);
}
template <int ROW_BYTES>
__device__ __forceinline__ int kc_offset(int row, int chunk) {
  return row * ROW_BYTES + ((chunk ^ kc_swizzle<ROW_BYTES>(row)) << 4);
}

// Row/column-contiguous tile: [BK rows of k][ROW_BYTES], 32-byte granules XOR-swizzled by k.
// E selects the pattern that suits the read instruction used for that element size.
template <int ROW_BYTES, int E>
__device__ __forceinline__ int mc_swizzle(int krow) {
  constexpr int NG = ROW_BYTES / 32;
  int f;
  if constexpr (E == kEF32) f = ((krow >> 2) & 1) << 2;
  else if constexpr (E == kEBF16 || E == kEF16) f = ((krow & 3) << 1) ^ ((krow >> 1) & 1);
  else f = krow & 7;
  return f & (NG - 1);
}
template <int ROW_BYTES, int E>
__device__ __forceinline__ int mc_offset(int krow, int byte_in_row) {
  const int g = (byte_in_row >> 5) ^ mc_swizzle<ROW_BYTES, E>(krow);
  return krow * ROW_BYTES + (g << 5) + (byte_in_row & 31);
}

__device__ __forceinline__ i32x4 lds_read_b128(const unsigned char* base, int off) {
  return *reinterpret_cast<const i32x4*>(base + off);
}

// int8 x8 (two dwords) -> bf16 x8 (exact: |v| <= 128 fits the 8-bit significand of bf16). Each byte is
// sign-extended and converted to f32 (one SDWA instruction); the upper halves of two f32 are the
// two bf16 and are packed with one byte permute.
__device__ __forceinline__ i32x4 i8x8_to_bf16x8(i32x2 v) {
  i32x4 out;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int w = v[h];
    const float f0 = (float)(signed char)(w & 0xff);
    const float f1 = (float)(signed char)((w >> 8) & 0xff);
    const float f2 = (float)(signed char)((w >> 16) & 0xff);
    const float f3 = (float)(signed char)((w >> 24) & 0xff);
    const unsigned u0 = __builtin_bit_cast(unsigned, f0), u1 = __builtin_bit_cast(unsigned, f1);
    const unsigned u2 = __builtin_bit_cast(unsigned, f2), u3 = __builtin_bit_cast(unsigned, f3);
    // v_perm_b32 picks bytes from {first operand: bytes 7..4, second operand: bytes 3..0}.
    out[2 * h] = (int)__builtin_amdgcn_perm(u1, u0, 0x07060302u);
    out[2 * h + 1] = (int)__builtin_amdgcn_perm(u3, u2, 0x07060302u);
  }
  return out;
}

// Four packed bytes (eight signed 4-bit values: byte u holds contraction entries 2 u in bits 0-3 and 2 u + 1 in bits
// 4-7) -> bf16 x8 in contraction order, each value TIMES 16: a nibble moved to the top of its byte is the int8 value
// 16 v, which converts like the int8 weights do (one SDWA instruction per value, one byte permute per pair, three
// instructions to line the nibbles up for all eight). |16 v| <= 128 is exact in bf16; the kernel takes the factor
// out of its sums again (kPackedInt4Unscale, exact).
constexpr float kPackedInt4Unscale = 0.0625f;
__device__ __forceinline__ i32x4 i4x8_to_bf16x8_times16(int w) {
  const int lo = (w << 4) & (int)0xF0F0F0F0u, hi = w & (int)0xF0F0F0F0u;
  i32x4 out;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const float f0 = (float)(signed char)((lo >> (8 * u)) & 0xff);
    const float f1 = (float)(signed char)((hi >> (8 * u)) & 0xff);
    out[u] = (int)__builtin_amdgcn_perm(__builtin_bit_cast(unsigned, f1), __builtin_bit_cast(unsigned, f0), 0x07060302u);
  }
  return out;
}

// Fragment of one 32-wide atom at row/column base `rc0` + `rc_step`, contraction atom `kk`.
//   ES = storage element kind in LDS, EC = compute (MFMA) kind.
// `rc_step` (a multiple of 16) is the part of the base that is a compile-time constant at the call (the wave's
// row block i sits i * WM * 32 rows below its first). A contraction-contiguous tile's swizzle looks at row bits
// 0..3 only, so those rows add a constant number of bytes to the address: kept apart from the lane's part, the
// constant goes into the read instruction's offset field and the blocks of a wave share their address registers.
// `PAIRED` (contraction-contiguous 16-bit tiles): atoms 2 d and 2 d + 1 share their 32 contraction entries the way a
// lane's eight packed int4 bytes hold them: lanes 0-31 own entries 0-15 (first half in the even atom, second in the
// odd one) and lanes 32-63 entries 16-31, instead of 8 entries per half-wave and atom in ascending order.
template <int LAYOUT, int ES, int EC, int ROW_BYTES, bool PAIRED = false>
__device__ __forceinline__ typename Mma<EC>::Frag load_frag(const unsigned char* tile, int rc0, int kk, int lane, int rc_step = 0) {
  typedef typename Mma<EC>::Frag Frag;
  constexpr int KA = Mma<EC>::KA;
  if constexpr (LAYOUT == kKC) {
    static_assert(ES == EC, "contraction-contiguous operands are stored in the compute type");
    const int row = rc0 + (lane & 31), q = lane >> 5;
    tile += rc_step * ROW_BYTES;
    if constexpr (EC == kEF8) {
      const int c0 = kk * 4 + q * 2;
      i32x4 lo = lds_read_b128(tile, kc_offset<ROW_BYTES>(row, c0));
      i32x4 hi = lds_read_b128(tile, kc_offset<ROW_BYTES>(row, c0 + 1));
      Frag f;
      f[0] = lo[0]; f[1] = lo[1]; f[2] = lo[2]; f[3] = lo[3];
      f[4] = hi[0]; f[5] = hi[1]; f[6] = hi[2]; f[7] = hi[3];
      return f;
    } else {
      return lds_read_b128(tile, kc_offset<ROW_BYTES>(row, PAIRED ? (kk >> 1) * 4 + 2 * q + (kk & 1) : kk * 2 + q));
    }
  } else {
    rc0 += rc_step;
    const int kb = kk * KA;
    if constexpr (ES == kEF32) {
      const int col = rc0 + (lane & 31), q = lane >> 5;
      Frag f;
#pragma unroll
      for (int t = 0; t < 4; ++t)
        f[t] = *reinterpret_cast<const int*>(tile + mc_offset<ROW_BYTES, ES>(kb + 4 * q + t, col * 4));
      return f;
    } else if constexpr (ES == kEBF16 || ES == kEF16) {
      // ds_read_b64_tr_b16: in each block of 16 lanes, lane s supplies the address of 4 consecutive
      // columns of k-row (s / 4); lane i receives column i of those 4 k-rows.
      const int blk = lane >> 4, s = lane & 15;
      const int krow = kb + 8 * (blk >> 1) + (s >> 2);
      const int col = rc0 + 16 * (blk & 1) + 4 * (s & 3);
      const i32x2 l2 = lds_read_tr16(tile + mc_offset<ROW_BYTES, ES>(krow, col * 2));
      const i32x2 h2 = lds_read_tr16(tile + mc_offset<ROW_BYTES, ES>(krow + 4, col * 2));
      Frag f;
      f[0] = l2[0]; f[1] = l2[1]; f[2] = h2[0]; f[3] = h2[1];
      return f;
    } else {
      // ds_read_b64_tr_b8: in each block of 16 lanes, lane s supplies the address of 8 consecutive
      // columns of k-row (s / 2); lane i receives column i of those 8 k-rows.
      const int blk = lane >> 4, s = lane & 15;
      const int col = rc0 + 16 * (blk & 1) + 8 * (s & 1);
      if constexpr (EC == kEF8) {
        Frag f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int krow = kb + 32 * (blk >> 1) + 8 * j + (s >> 1);
          const i32x2 v = lds_read_tr8(tile + mc_offset<ROW_BYTES, ES>(krow, col));
          f[2 * j] = v[0];
          f[2 * j + 1] = v[1];
        }
        return f;
      } else if constexpr (EC == kEI8) {
        // 16 contraction values per lane: k rows 16 (l / 32) .. + 15 of the atom.
        const int krow = kb + 16 * (blk >> 1) + (s >> 1);
        const i32x2 lo = lds_read_tr8(tile + mc_offset<ROW_BYTES, ES>(krow, col));
        const i32x2 hi = lds_read_tr8(tile + mc_offset<ROW_BYTES, ES>(krow + 8, col));
        Frag f;
        f[0] = lo[0]; f[1] = lo[1]; f[2] = hi[0]; f[3] = hi[1];
        return f;
      } else {
        static_assert(EC == kEBF16 && ES == kEI8, "1-byte storage feeds fp8, int8 or bf16(int8) MFMAs only");
        const int krow = kb + 8 * (blk >> 1) + (s >> 1);
        const i32x2 v = lds_read_tr8(tile + mc_offset<ROW_BYTES, ES>(krow, col));
        return i8x8_to_bf16x8(v);
      }
    }
  }
}

// 32 packed int4 values of one column (16 bytes, byte r = contraction entries 2 r and 2 r + 1, low nibble first) as the
// 32 fp8 bytes 0000uuuu, u = nibble ^ 8, in contraction order: the e4m3 denormal (w + 8) / 512 for the weight w.
__device__ __forceinline__ i32x8 i4x32_to_biased_f8x32(i32x4 w) {
  i32x8 out;
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const unsigned x = (unsigned)w[d] ^ 0x88888888u;
    const unsigned lo = x & 0x0F0F0F0Fu, hi = (x >> 4) & 0x0F0F0F0Fu;
    out[2 * d] = (int)__builtin_amdgcn_perm(hi, lo, 0x05010400u);
    out[2 * d + 1] = (int)__builtin_amdgcn_perm(hi, lo, 0x07030602u);
  }
  return out;
}

// 16 packed int4 values of one column (8 bytes, byte r = contraction entries 2 r and 2 r + 1, low nibble first) as the
// 16 int8 values 16 w in contraction order: each nibble at the top of a byte of its own.
__device__ __forceinline__ i32x4 i4x16_to_i8x16_times16(i32x2 w) {
  i32x4 out;
#pragma unroll
  for (int d = 0; d < 2; ++d) {
    const unsigned lo = ((unsigned)w[d] << 4) & 0xF0F0F0F0u, hi = (unsigned)w[d] & 0xF0F0F0F0u;
    out[2 * d] = (int)__builtin_amdgcn_perm(hi, lo, 0x05010400u);
    out[2 * d + 1] = (int)__builtin_amdgcn_perm(hi, lo, 0x07030602u);
  }
  return out;
}

// Eight packed int4 values (see i4x8_to_bf16x8_times16) times one scale, rounded to bf16; `scale16` is the column's
// scale for the current k-block divided by 16.
__device__ __forceinline__ i32x4 i4x8_to_bf16x8_scaled(int w, float scale16) {
  const int lo = (w << 4) & (int)0xF0F0F0F0u, hi = w & (int)0xF0F0F0F0u;
  bf16x8 out;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    out[2 * u] = (__bf16)((float)(signed char)((lo >> (8 * u)) & 0xff) * scale16);
    out[2 * u + 1] = (__bf16)((float)(signed char)((hi >> (8 * u)) & 0xff) * scale16);
  }
  return __builtin_bit_cast(i32x4, out);
}

// The same 8 int8 values times one scale (the column's scale for the current k-block), rounded to bf16.
__device__ __forceinline__ i32x4 i8x8_to_bf16x8_scaled(i32x2 v, float scale) {
  bf16x8 out;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int w = v[h];
    out[4 * h + 0] = (__bf16)((float)(signed char)(w & 0xff) * scale);
    out[4 * h + 1] = (__bf16)((float)(signed char)((w >> 8) & 0xff) * scale);
    out[4 * h + 2] = (__bf16)((float)(signed char)((w >> 16) & 0xff) * scale);
    out[4 * h + 3] = (__bf16)((float)(signed char)((w >> 24) & 0xff) * scale);
  }
  return __builtin_bit_cast(i32x4, out);
}

// 8 fp8 (e4m3fn) values times one scale, rounded to bf16.
__device__ __forceinline__ i32x4 f8x8_to_bf16x8_scaled(i32x2 v, float scale) {
  bf16x8 out;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int w = v[h];
    out[4 * h + 0] = (__bf16)(__builtin_amdgcn_cvt_f32_fp8(w, 0) * scale);
    out[4 * h + 1] = (__bf16)(__builtin_amdgcn_cvt_f32_fp8(w, 1) * scale);
    out[4 * h + 2] = (__bf16)(__builtin_amdgcn_cvt_f32_fp8(w, 2) * scale);
    out[4 * h + 3] = (__bf16)(__builtin_amdgcn_cvt_f32_fp8(w, 3) * scale);
  }
  return __builtin_bit_cast(i32x4, out);
}

// ---- global -> LDS, fast path: direct-to-LDS loads -------------------------------------------
// global_load_lds_dwordx4 moves 16 bytes per lane straight into LDS; one wave instruction fills
// 1024 contiguous LDS bytes (lane l lands at base + 16*l). The LDS swizzle is therefore applied
// on the global side: each lane fetches the chunk that belongs at its fixed LDS position.
// Out-of-range rows/columns are clamped to valid memory (their products are never stored).
// Only whole k-steps go this way; a partial last step is zero-filled through TileStage below.
// The loads are issued from inline assembly on purpose: the compiler guards every LDS read that
// follows a direct-to-LDS load it can see with a full vmcnt(0) wait (it cannot tell which LDS bytes
// the load writes), which would serialise each k-step's loads with its MFMAs. Ordering is enforced
// explicitly instead, by barrier_after_direct_loads(). M0 carries the LDS destination.
__device__ __forceinline__ unsigned lds_address(const unsigned char* p) {
  return __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)p);
}
__device__ __forceinline__ const unsigned char* uniform_pointer(const unsigned char* p) {
  const uint64_t v = (uint64_t)(uintptr_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return (const unsigned char*)(uintptr_t)(((uint64_t)hi << 32) | lo);
}
// LDS byte address of a pointer into the workgroup's shared memory (wave-uniform).
__device__ __forceinline__ unsigned lds_address32(const void* p) {
  return __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)p);  // low half of a generic LDS pointer = LDS offset
}
// 16 bytes per lane: LDS[lds + 16*lane] <- *(sbase + voff)
__device__ __forceinline__ void direct_load_16(const unsigned char* sbase, uint32_t voff, unsigned lds) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds), "v"(voff), "s"(sbase)
               : "memory", "m0");
}
// Workgroup barrier that also orders direct-to-LDS loads: a wave's loads count on vmcnt, and other
// waves read the bytes they deposit, so every wave must drain vmcnt BEFORE it arrives at the
// barrier (the compiler only guards a wave's own later LDS reads).
// N = number of this wave's most recent direct loads that may stay in flight (they belong to
// later stages); loads complete in issue order.
template <int N>
__device__ __forceinline__ void barrier_after_direct_loads() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  // s_waitcnt immediate: vmcnt = bits [3:0] and [15:14], expcnt = [6:4] (7: no wait), lgkmcnt = [11:8] (0: all).
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4));
  __syncthreads();
}

template <int LAYOUT, int ES, int RC /* rows or cols of C covered */, int BK, int NWAVES>
struct DirectLoader {
  static constexpr int ESZ = elem_bytes(ES);
  static constexpr int ROW_BYTES = (LAYOUT == kKC) ? BK * ESZ : RC * ESZ;
  static constexpr int ROWS = (LAYOUT == kKC) ? RC : BK;
  static constexpr int BYTES = ROWS * ROW_BYTES;
  static constexpr int INSTRS = BYTES / 1024;
  static constexpr int PER = (INSTRS + NWAVES - 1) / NWAVES;
  static_assert(BYTES % 1024 == 0, "tile must be a whole number of wave-wide 16-byte loads");

  // Rows between two consecutive instructions of one wave. In the row/column-contiguous layout the
  // rows are contraction indices (never clamped) and the swizzle repeats every 8 rows, so when this
  // is a multiple of 8 the per-lane offsets of a wave's instructions differ by a wave-uniform
  // stride: one per-lane offset is kept and the stride goes into the scalar base pointer.
  static constexpr int ROWS_PER_INSTR_STEP = NWAVES * 1024 / ROW_BYTES;
  static constexpr bool STRIDED = LAYOUT == kMC && (NWAVES * 1024) % ROW_BYTES == 0 && ROWS_PER_INSTR_STEP % 8 == 0;
  static constexpr int NOFF = STRIDED ? 1 : PER;

  uint32_t voff[NOFF];  // per-lane byte offset from the wave-uniform base pointer of a k-step
  int64_t stride;       // STRIDED: bytes between consecutive instructions of one wave

  // Base pointer of the k-step that starts at contraction index kc0 (uniform across the workgroup).
  static __device__ __forceinline__ int64_t step_base(int rc0, int64_t ld, int kc0) {
    if constexpr (LAYOUT == kKC) return ((int64_t)rc0 * ld + kc0) * ESZ;
    else return (int64_t)kc0 * ld * ESZ;
  }
  static __device__ __forceinline__ int64_t step_bytes(int64_t ld) {
    if constexpr (LAYOUT == kKC) return (int64_t)BK * ESZ;
    else return (int64_t)BK * ld * ESZ;
  }

  // `rc_lo`, `rc_hi`: the rows (contraction-contiguous layout) whose data the caller uses. Rows
  // outside are redirected to the nearest one inside: that keeps every address valid, and the
  // lanes of a load that fall outside all fetch one row's cache lines instead of one each.
  // `glu_tn` > 0 (row/column-contiguous layout only): the tile's columns are [gate | up] pairs. The
  // tile is cut into blocks of 32 columns, `glu_tn` blocks per wave column; the first half of a wave
  // column's blocks comes from the gate columns [rc0, rc0 + RC/2) and the second half from the up
  // columns `glu_up` further on, so that accumulator block j and block j + glu_tn/2 of a lane hold
  // gate and up of the same output column.
  __device__ __forceinline__ void init(int rc0, int rc_ext, int64_t ld, int wave, int lane, int rc_lo, int rc_hi,
                                       int glu_tn = 0, int glu_up = 0) {
    stride = (int64_t)ROWS_PER_INSTR_STEP * ld * ESZ;
#pragma unroll
    for (int i = 0; i < NOFF; ++i) {
      const int j = i * NWAVES + wave;
      const int off = j * 1024 + lane * 16;
      const int row = off / ROW_BYTES, pc = (off % ROW_BYTES) >> 4;
      if constexpr (LAYOUT == kKC) {
        const int lc = pc ^ kc_swizzle<ROW_BYTES>(row);
        int grow = rc0 + row;
        grow = grow < rc_hi ? grow : rc_hi - 1;
        grow = (grow > rc_lo ? grow : rc_lo) - rc0;
        voff[i] = (uint32_t)(grow * (int)ld * ESZ + lc * 16);
      } else {
        const int lc = ((((pc >> 1) ^ mc_swizzle<ROW_BYTES, ES>(row))) << 1) | (pc & 1);
        int colb = rc0 * ESZ + lc * 16;
        if (glu_tn > 0) {
          const int c = lc * (16 / ESZ), blk = c >> 5, half = glu_tn >> 1;
          const int w = blk / glu_tn, j = blk % glu_tn;
          colb = ((j < half ? rc0 : rc0 + glu_up) + (w * half + j % half) * 32 + (c & 31)) * ESZ;
        }
        const int lim = rc_ext * ESZ - 16;
        colb = colb < lim ? colb : lim;
        voff[i] = (uint32_t)(row * (int)ld * ESZ + colb);
      }
    }
  }

  // Instruction i (0 <= i < PER) of this wave's share: `base` = wave-uniform pointer of the k-step,
  // `tile_lds` = LDS byte address of the destination tile (wave-uniform).
  __device__ __forceinline__ void issue_one(int i, const unsigned char* base, unsigned tile_lds, int wave) const {
    const int j = i * NWAVES + wave;
    if (INSTRS % NWAVES != 0 && j >= INSTRS) return;
    if constexpr (STRIDED) direct_load_16(base + i * stride, voff[0], tile_lds + j * 1024);
    else direct_load_16(base, voff[i], tile_lds + j * 1024);
  }
  __device__ __forceinline__ void issue(const unsigned char* base, unsigned tile_lds, int wave) const {
#pragma unroll
    for (int i = 0; i < PER; ++i) issue_one(i, base, tile_lds, wave);
  }
};

// ---- global -> register -> LDS, masked path (a partial last k-step) ---------------------------
// One operand tile moved in 16-byte chunks; chunk q of the tile belongs to thread (q % THREADS).
// Contraction indices at or past `k_hi` are zero-filled.
template <int LAYOUT, int ES, int RC, int BK, int THREADS>
struct TileStage {
  static constexpr int ESZ = elem_bytes(ES);
  static constexpr int ROW_BYTES = (LAYOUT == kKC) ? BK * ESZ : RC * ESZ;
  static constexpr int ROWS = (LAYOUT == kKC) ? RC : BK;
  static constexpr int CPR = ROW_BYTES / 16;
  static constexpr int CHUNKS = ROWS * CPR;
  static constexpr int PER = (CHUNKS + THREADS - 1) / THREADS;
  static constexpr int BYTES = ROWS * ROW_BYTES;
  static_assert(ROW_BYTES % 32 == 0 && (CPR & (CPR - 1)) == 0, "tile rows must be a power-of-two number of chunks");

  // base: operand pointer already offset to the group; ld in elements; rc0 = first row/col of the
  // tile; rc_ext = extent of that axis; kc0 = first contraction index of this k-step.
  static __device__ __forceinline__ void copy(const unsigned char* base, int64_t ld, int rc0, int rc_ext, int kc0,
                                              int k_hi, unsigned char* tile, int tid) {
    const i32x4 z = {0, 0, 0, 0};
#pragma unroll 2
    for (int i = 0; i < PER; ++i) {
      const int q = tid + i * THREADS;
      if (CHUNKS % THREADS != 0 && q >= CHUNKS) break;
      const int r = q / CPR, c = q % CPR;
      i32x4 v = z;
      int off;
      if constexpr (LAYOUT == kKC) {
        int row = rc0 + r;
        row = row < rc_ext ? row : rc_ext - 1;
        const int kcol = kc0 + c * (16 / ESZ);
        if (kcol < k_hi) v = *reinterpret_cast<const i32x4*>(base + ((int64_t)row * ld + kcol) * ESZ);
        off = kc_offset<ROW_BYTES>(r, c);
      } else {
        const int krow = kc0 + r;
        int colb = rc0 * ESZ + c * 16;
        const int lim = rc_ext * ESZ - 16;
        colb = colb < lim ? colb : lim;
        if (krow < k_hi) v = *reinterpret_cast<const i32x4*>(base + (int64_t)krow * ld * ESZ + colb);
        off = mc_offset<ROW_BYTES, ES>(r, c * 16);
      }
      *reinterpret_cast<i32x4*>(tile + off) = v;
    }
  }
};

__device__ __forceinline__ float apply_activation(float x, int act) {
  switch (act) {
    case TKX_ACT_RELU: return x > 0.f ? x : 0.f;
    case TKX_ACT_TANH: return tanhf(x);
    case TKX_ACT_SILU: return x / (1.f + __expf(-x));
    case TKX_ACT_SIGMOID: return 1.f / (1.f + __expf(-x));
    case TKX_ACT_GELU_TANH: {
      const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
      return 0.5f * x * (1.f + tanhf(u));
    }
    default: return x;
  }
}

__device__ __forceinline__ void store4(void* C, int64_t idx, f32x4 v, int out_dtype) {
  if (out_dtype == TKX_F32) {
    *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(C) + idx) = v;
  } else if (out_dtype == TKX_BF16) {
    bf16x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = (__bf16)v[e];
    *reinterpret_cast<bf16x4*>(reinterpret_cast<__bf16*>(C) + idx) = o;
  } else {
    f16x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = (_Float16)v[e];
    *reinterpret_cast<f16x4*>(reinterpret_cast<_Float16*>(C) + idx) = o;
  }
}

// 4 consecutive outputs at a byte address, in a compile-time output type. (The pointer is rebuilt
// from integers upstream, so the global address space is named here: a generic pointer would turn
// every store into a flat one.)
template <int OUT>
__device__ __forceinline__ void store4_as(unsigned char* ptr, f32x4 v) {
  if constexpr (OUT == TKX_F32) {
    *(__attribute__((address_space(1))) f32x4*)ptr = v;
  } else if constexpr (OUT == TKX_BF16) {
    bf16x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = (__bf16)v[e];
    *(__attribute__((address_space(1))) bf16x4*)ptr = o;
  } else {
    f16x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = (_Float16)v[e];
    *(__attribute__((address_space(1))) f16x4*)ptr = o;
  }
}

// ---- the kernel ---------------------------------------------------------------------------------
// Calls f(integral_constant<int, sel>) for a run-time sel in [I, N].
template <int I, int N, class Fn>
__device__ __forceinline__ void dispatch_upto(int sel, Fn&& f) {
  if constexpr (I < N) {
    if (sel == I) f(std::integral_constant<int, I>{});
    else dispatch_upto<I + 1, N>(sel, f);
  } else {
    f(std::integral_constant<int, N>{});
  }
}

// How many of the most recently issued direct loads a wave may leave in flight at the barrier of compute step
// `kt` of the split pipeline (GemmKernel with HB > 0). Loads go out in a fixed order: step t issues, if t is odd,
// the PA loads of A double-step (t - 1) / 2 + NS and then the PB loads of B step t + HB (negative t: the
// prologue, which follows the same order from t = -max(HB, 2 NS) on). The barrier of step kt needs B step kt + 1
// and A double-step (kt + 1) / 2 complete; loads complete in issue order, so everything issued after the later of
// the two may stay in flight. kt = -1 is the barrier before the first step.
constexpr int split_loads_in_flight(int kt, int NS, int HB, int PA, int PB) {
  const int look = HB > 2 * NS ? HB : 2 * NS;
  int after_a = -1, after_b = -1, count = 0;
  for (int t = kt - 1; t >= -look; --t) {  // backwards: within a step the B loads were issued last
    const int s = t + HB;
    if (s >= 0) {
      if (s == kt + 1) after_b = count;
      count += PB;
    }
    if (t & 1) {
      const int j = (t - 1) / 2 + NS;
      if (j >= 0) {
        if (j == (kt + 1) / 2) after_a = count;
        count += PA;
      }
    }
  }
  return after_a < after_b ? after_a : after_b;
}

// HB > 0 ("split pipeline", forward with a contraction-contiguous A): BK is the depth of an A stage and half of it
// the depth of a compute step and of a B stage; NS A stages and HB B stages. A row of an A stage is then a whole
// 128-byte line for 16-bit elements at BK = 64, where a stage as deep as a compute step holds half a line per row
// and every line of A is requested from L2 twice, once by each of two consecutive steps.
template <int MODE, int EA, int EB, int BM, int BN, int BK, int WM, int WN, int NS, int HB = 0>
struct GemmKernel {
  static constexpr bool SPLIT = HB > 0;
  static constexpr int BKC = SPLIT ? BK / 2 : BK;  // contraction elements per compute step
  static constexpr int THREADS = WM * WN * 64;
  static constexpr int LA = (MODE == kDrhs) ? kMC : kKC;
  static constexpr int LB = (MODE == kDlhs) ? kKC : kMC;
  static constexpr bool GLU = MODE == kFwdGlu;
  static constexpr bool SUBK = MODE == kFwdSubK;
  // fp8 x fp8 with scales per k-block on both sides (xs[row, k_sub] ws[g, k_sub, n],
  // pallas_mosaic_gpu_kernel_sm100_i8_quant.py:51-102): the MFMAs of a k-step (= one k-block or a part of one)
  // accumulate into partial accumulators, which are folded into the result with the block's scales.
  // int8 x int8 runs the same way on the int8 MFMAs (int32 partial sums, exact), also with one block.
  static constexpr bool SUBP = SUBK && (EA == kEF8 || EA == kEI8);
  static_assert(!SUBK || ((EB == kEI8 || EB == kEF8 || EB == kEI4) &&
                          (EA == kEBF16 || (SUBP && EB == EA) || (EA == kEF8 && EB == kEI4 && BK == 128) ||
                           (EA == kEI8 && EB == kEI4)) && BN == 256),
                "per-k-block scales: bf16 lhs with int8, packed int4 or fp8 weights, fp8 x fp8, int8 x int8 or fp8 x packed int4"
                " (whose row sums come per 128-deep k-step); one 1 KB scale row per k-step");
  static constexpr int BNO = GLU ? BN / 2 : BN;  // output columns of a tile
  static constexpr int EC = EA;  // MFMA type follows A; B may be stored narrower (int8 weights)
  // Packed int4 weights: a B stage is a byte tile of half the depth; a lane's transposing read of 8 bytes of its
  // column gives it 16 consecutive contraction entries, the B fragments of two atoms, and the lhs fragments are read
  // in the matching order (load_frag's PAIRED), so nothing is permuted.
  static constexpr bool I4 = EB == kEI4;
  // bf16 activations: the nibbles are converted to bf16 (times 16) on their way into the MFMAs.
  static constexpr bool I4P = I4 && EA == kEBF16;
  // fp8 activations (pallas_mosaic_gpu_kernel_sm100_fp8_quant.py:258-300): a nibble w becomes the fp8 byte
  // 0000uuuu with u = w + 8 = nibble ^ 8, which e4m3 reads as the denormal u / 512, exactly; the fp8 MFMAs then
  // give sum(x u) / 512 and the epilogue takes 8 sum(x) off again: sum(x w) = 512 acc - 8 rowsum(x). The row sums
  // of x lie behind its m_ext row scales.
  static constexpr bool I4F = I4 && EA == kEF8;
  // int8 activations (pallas_mosaic_gpu_kernel_sm100_i8_quant.py:114-190, int8 x int4 on the native int8 matrix
  // instructions): a nibble moved to the top of its byte is the int8 value 16 w; the int32 sums are exact and the
  // factor 16 is taken out where they become floats.
  static constexpr bool I4I = I4 && EA == kEI8;
  static constexpr int EBS = I4 ? (int)kEI8 : EB;  // element kind of a B stage in LDS
  static constexpr int KA = Mma<EC>::KA;
  static constexpr int WTM = BM / WM, WTN = BN / WN;
  static constexpr int TM = WTM / 32, TN = WTN / 32;
  // Kernels that can quantise their result to fp8 with one scale per (row, 128 columns): the plain forward of bf16 and
  // fp8 operands, with whole quantisation tiles inside a workgroup's tile and inside or across whole wave columns.
  static constexpr bool QOUT = MODE == kFwd && (EA == kEBF16 || EA == kEF8) && EB == EA && BN % 128 == 0 &&
                               (128 % WTN == 0 || WTN % 128 == 0);
  static_assert(MODE != kFwdGlu || TN % 2 == 0, "gate-up tiles pair the two halves of a wave's column blocks");
  static constexpr int TNO = MODE == kFwdGlu ? TN / 2 : TN, WTNO = MODE == kFwdGlu ? WTN / 2 : WTN;
  static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0 && BK % KA == 0, "tile does not split into 32x32 atoms");
  static constexpr int KSTEPS = BKC / KA;
  // Lean fragments: the 32-byte fragments of the fp8 MFMA, double-buffered for a 4 x 2 wave tile, take 96 registers
  // next to 128 accumulators. The lhs fragments are then kept once: row block i's is re-read for the next atom right
  // after the atom's last MFMA on it (TM * TN - TN MFMAs of 64 cycles before its next use); the two rhs fragments stay
  // double-buffered.
  static constexpr bool LEAN = EA == kEF8 && (EB == kEF8 || EB == kEI4) && !SUBK && !SPLIT && TM * TN >= 8;
  // fp8 activations over packed int4 weights on a lean tile with two or more column blocks per wave: the MFMAs of an
  // atom run column block by column block, so that the bytes read ahead (`rawf`) are the only second copy of the
  // rhs fragments: fragment 0 of the next atom is converted once the MFMAs on the current one are issued, fragment
  // c >= 1 at the start of its own atom, while the MFMAs on fragment 0 run. 16 registers fewer than two sets of
  // converted fragments, which is what lets the 256 x 256 x 128 tile live in 256.
  static constexpr bool JOUT = LEAN && I4F && TN >= 2;
  static_assert(KSTEPS % 2 == 0, "the fragment double buffer assumes an even number of k-atoms per step");
  static_assert(!SPLIT || (MODE == kFwd && EA == EB && BK % 2 == 0), "split pipeline: plain forward, operands of one type");
  static_assert(!I4 || (((I4P && (MODE == kFwd || MODE == kFwdGlu || MODE == kFwdSubK)) || (I4F && (MODE == kFwd || MODE == kFwdGlu || MODE == kFwdSubK)) ||
                        (I4I && (MODE == kFwd || MODE == kFwdGlu || MODE == kFwdSubK))) && !SPLIT),
                "packed int4 weights: forward with bf16, fp8 or int8 activations");
  static constexpr int BKB = I4 ? BKC / 2 : BKC;  // rows of a B stage
  typedef TileStage<LA, EA, BM, BK, THREADS> StageA;
  typedef TileStage<LB, EBS, BN, BKB, THREADS> StageB;
  // Every wave takes an equal share of a k-step's direct-to-LDS loads.
  static constexpr int NLOAD = WM * WN;
  typedef DirectLoader<LA, EA, BM, BK, NLOAD> DirA;
  typedef DirectLoader<LB, EBS, BN, BKB, NLOAD> DirB;
  static constexpr int SCALE_BYTES = (SUBK && !SUBP) ? BN * 4 : 0;  // kFwdSubK: the k-step's scale row behind its two tiles
  static constexpr int STAGE_BYTES = StageA::BYTES + StageB::BYTES + SCALE_BYTES;
  // fp8 x fp8: the scales of a k-step (BN weight-column scales, then BM lhs-row scales) are still needed when its
  // stage is already being refilled, so they live in a ring of NS + 1 slots behind the stages.
  // (fp8 x packed int4: behind them the BM row sums of the k-step's activations)
  static constexpr int RING_SLOT = SUBP ? (BN + BM + (I4F ? BM : 0)) * 4 : 0;
  static constexpr int SMEM_BYTES = SPLIT ? NS * StageA::BYTES + HB * StageB::BYTES : NS * STAGE_BYTES + (NS + 1) * RING_SLOT;
  // Workgroups the register budget is set for: two 4-wave workgroups share a CU when their LDS fits twice (256
  // registers per lane each); every other shape has the CU, and a SIMD's 512 registers per lane, to itself or to the
  // two waves of one 8-wave workgroup.
  // (An 8-wave workgroup on one row of waves with 64 accumulators per lane, the 128 x 256 tile, fits twice as well
  // when its LDS does: 128 registers each.)
  static constexpr int kWorkgroupsPerCu =
      (THREADS <= 256 || (WM == 1 && TM * TN * 16 <= 64)) && 2 * SMEM_BYTES <= 160 * 1024 ? 2 : 1;
  // What the launch bound asks for: waves per SIMD with that many workgroups on the CU.
  static constexpr int kWavesPerSimd = (THREADS / 64 + 3) / 4 * kWorkgroupsPerCu;
  static_assert(NS >= 2 && SMEM_BYTES <= 160 * 1024, "stages must fit the 160 KB LDS");

  // QO: the instantiation that stores fp8 with one scale per (row, 128 columns) (QOUT kernels only). It is a kernel of
  // its own so that the plain one carries none of its code or registers.
  // Kernels that can split the tiles of a launch's last round along the contraction (GemmParams::split_k).
  static constexpr bool SPLITK = (MODE == kFwd || MODE == kDlhs) && BM >= 128;
  // SK: the instantiation that does (a kernel of its own, like the quantising one).
  template <bool QO = false, bool SK = false>
  static __device__ __forceinline__ void run(const GemmParams& p, unsigned char* smem) {
    static_assert(!QO || QOUT, "this kernel has no quantising epilogue");
    static_assert(!SK || (SPLITK && !QO), "this kernel has no split of the last round");
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // in a scalar register: all that derives from it is uniform
    const int wm = wave / WN, wn = wave % WN;
    // The wave's TM row blocks (32 rows each) are interleaved with those of the other waves along
    // m: block i of wave row wm is block i * WM + wm of the tile. A task that owns only part of the
    // tile's rows (a group boundary) then leaves every wave row about the same number of blocks
    // with rows to compute, instead of all of them to one wave row.
    auto row_block = [&](int i) { return i * WM + wm; };
    const int32_t* ws = p.ws;
    const int b = blockIdx.x;

    int group, row0, act_start, act_end, col0, kc_begin, kc_end;
    int part = 0, parts = 1, split_unit = 0;  // (fwd/dlhs) this workgroup contracts part `part` of `parts` of its tile
    if constexpr (MODE != kDrhs) {
      // (Group sizes are device data nobody has checked: when they add up to more than m_ext rows the schedule
      // holds more tasks than its arrays have slots for. Every task with a row below m_ext has a slot, so the rest
      // are dropped here, and the tasks kept store no row at or past m_ext.)
      const int num_tasks = min(ws[0], p.tid_size);
      // Split of the last round: the launch's tiles beyond the last multiple of `split_cus` (a round of workgroups
      // that would leave most CUs idle) are cut along the contraction into `parts` parts. Part 0 is the tile's own
      // workgroup, the others are workgroups behind the zeroing ones.
      const int total = num_tasks * p.n_tiles;
      int first_split = total;  // list index of the first tile that is split
      if (SK && p.split_k > 1) {
        const int full = total / p.split_cus * p.split_cus, rem = total - full;
        const int s = rem > 0 ? min(p.split_k, p.split_cus / rem) : 1;
        if (s > 1) {
          first_split = full;
          parts = s;
        }
      }
      int L = -1;
      if (b >= p.real_slots + p.zero_wgs) {
        if (parts < 2) return;
        const int x = b - p.real_slots - p.zero_wgs, t = x / (parts - 1);
        if (t >= total - first_split) return;
        L = first_split + t;
        part = 1 + x - t * (parts - 1);
      } else if (b >= p.real_slots) {
        // Tail duty: rows [total_rows, m_ext), and with a group offset the rows before the first
        // group, belong to no group of this call and are defined to be zero.
        const int total_rows = min(ws[1], p.m_ext), lead_rows = min(ws[2], p.m_ext);
        const int64_t esz = QO ? 1 : p.out_dtype == TKX_F32 ? 4 : 2;
        const int64_t lo = (int64_t)total_rows * p.ldc * esz, hi = (int64_t)p.m_ext * p.ldc * esz;
        if constexpr (QO) {
          // Quantised output: rows of no group are zeros with scale 1, what quantising a row of zeros gives.
          const int64_t per_row = p.ldc / 128, id = (int64_t)(b - p.real_slots) * THREADS + tid, step = p.zero_wgs * (int64_t)THREADS;
          for (int64_t o = total_rows * per_row + id; o < (int64_t)p.m_ext * per_row; o += step) p.c_scale[o] = 1.f;
          for (int64_t o = id; o < (int64_t)lead_rows * per_row; o += step) p.c_scale[o] = 1.f;
        }
        unsigned char* c = reinterpret_cast<unsigned char*>(p.C);
        const int64_t nzb = p.zero_wgs;
        const i32x4 z = {0, 0, 0, 0};
        const int64_t first = ((int64_t)(b - p.real_slots) * THREADS + tid) * 16;
        for (int64_t o = lo + first; o < hi; o += nzb * THREADS * 16) *reinterpret_cast<i32x4*>(c + o) = z;
        const int64_t lead_bytes = (int64_t)lead_rows * p.ldc * esz;
        for (int64_t o = first; o < lead_bytes; o += nzb * THREADS * 16) *reinterpret_cast<i32x4*>(c + o) = z;
        return;
      }
      // XCD-aware order: consecutive workgroup ids land on different XCDs (id % 8). The tile list is
      // dealt out in chunks of kXcdChunk consecutive tiles, chunk c to XCD c % 8, so that the
      // workgroups an XCD runs at a time are consecutive in the list and the 8 XCDs work on
      // neighbouring chunks. The list goes span by span (a span = up to `grid_tile_width`
      // consecutive m-tasks of one group, laid out by the scheduler); inside a span its m-tasks take
      // an n-panel of the group's weights back to back, then the next n-panel: the tiles of a chunk
      // share panels in their XCD's L2, and neighbouring chunks share the span's lhs panels in the
      // memory-side cache.
      if (L < 0) {
        const int idx = b >> 3, xcd = b & 7;
        L = ((idx / kXcdChunk) * 8 + xcd) * kXcdChunk + idx % kXcdChunk;
        if (L >= total) return;
        if (L < first_split) parts = 1;
      }
      split_unit = (L - first_split) * parts + part;
      const int t0 = L / p.n_tiles;  // some task of the span that holds L (every task owns n_tiles list entries)
      const int first = ws[p.ws_span_first + t0], width = ws[p.ws_span_width + t0];
      const int rem = L - first * p.n_tiles;
      const int nt = rem / width;
      const int mt = first + (rem - nt * width);
      if (mt >= p.tid_size) return;  // (a span that runs past the last slot: rows past m_ext only)
      group = ws[p.ws_gid + mt];
      row0 = ws[p.ws_bstart + mt];
      act_end = min(ws[p.ws_aend + mt], p.m_ext);
      act_start = min(ws[p.ws_astart + mt], act_end);
      if (act_start >= act_end) return;  // (every row of the task lies at or past m_ext)
      col0 = nt * BNO;
      kc_begin = 0;
      kc_end = p.k_ext;
      if (parts > 1) {
        // This part's share of the contraction, in whole A stages (the last part takes what is left over).
        const int steps = (p.k_ext + BK - 1) / BK;
        kc_begin = min((int)((int64_t)steps * part / parts) * BK, p.k_ext);
        if (part + 1 < parts) kc_end = min((int)((int64_t)steps * (part + 1) / parts) * BK, p.k_ext);
      }
    } else {
      const int per_group = p.m_tiles * p.n_tiles;
      group = b / per_group;
      const int r = b - group * per_group;
      const int mt = r / p.n_tiles, nt = r - mt * p.n_tiles;
      row0 = mt * BM;
      col0 = nt * BN;
      act_start = row0;
      act_end = min(row0 + BM, p.m_ext);
      kc_begin = min(ws[p.ws_offsets + group], p.k_ext);
      kc_end = min(ws[p.ws_offsets + group + 1], p.k_ext);
    }

    const unsigned char* Ab = reinterpret_cast<const unsigned char*>(p.A);
    const unsigned char* Bb = reinterpret_cast<const unsigned char*>(p.B);
    if constexpr (MODE != kDrhs) Bb += (int64_t)group * p.b_group_stride * elem_bytes(EB);

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    f32x16 pacc[SUBP ? TM : 1][SUBP ? TN : 1];  // (fp8 x fp8 with k-block scales) the current k-step's products
    typedef typename Mma<EC>::Frag Frag;
    // Row blocks (32 rows) of this wave that hold at least one row the task stores. A task at a
    // group boundary can have only a few such rows; the blocks without any skip their LDS reads and
    // MFMAs (the wave still takes part in the loads and barriers). `full` selects at compile time
    // the path without the per-block tests, which whole tiles take.
    uint32_t rmask = 0;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int r0 = row0 + row_block(i) * 32;
      if (r0 < act_end && r0 + 32 > act_start) rmask |= 1u << i;
    }
    rmask = __builtin_amdgcn_readfirstlane(rmask);
    // The blocks with rows are the first `nv` of the wave (a task's rows start in the tile's first 8 rows and the
    // blocks of a wave ascend through the tile), so the k loop is compiled once per count: straight-line code for
    // whole and partial tiles alike, no test around an MFMA. (Any other pattern computes every block.)
    const int nv_count = __builtin_popcount(rmask);
    const int nv_sel = rmask == (1u << nv_count) - 1u ? nv_count : TM;
    // B fragment j of k-atom kk of a stage. kFwdSubK: the int8 values of the lane's column (lane % 32 of the
    // block) are multiplied by that column's scale for the stage's k-block, which lies behind the tiles.
    // (fp8 activations over packed int4 weights) the 16 bytes of the lane's column that hold the 32 contraction
    // entries of its half of k-atom kk: packed rows 32 kk + 16 (lane / 32) .. + 15.
    [[maybe_unused]] auto load_b_raw = [&](const unsigned char* stage, int j, int kk) -> i32x4 {
      const int blk = lane >> 4, s_ = lane & 15;
      const int col = wn * WTN + j * 32 + 16 * (blk & 1) + 8 * (s_ & 1);
      const int krow = kk * (KA / 2) + 16 * (blk >> 1) + (s_ >> 1);
      const i32x2 lo = lds_read_tr8(stage + StageA::BYTES + mc_offset<StageB::ROW_BYTES, EBS>(krow, col));
      const i32x2 hi = lds_read_tr8(stage + StageA::BYTES + mc_offset<StageB::ROW_BYTES, EBS>(krow + 8, col));
      return i32x4{lo[0], lo[1], hi[0], hi[1]};
    };
    // (int8 activations over packed int4 weights) the 8 bytes that hold the 16 contraction entries of the lane's half
    // of k-atom kk: packed rows 16 kk + 8 (lane / 32) .. + 7.
    [[maybe_unused]] auto load_b_raw8 = [&](const unsigned char* stage, int j, int kk) -> i32x2 {
      const int blk = lane >> 4, s_ = lane & 15;
      const int col = wn * WTN + j * 32 + 16 * (blk & 1) + 8 * (s_ & 1);
      const int krow = kk * (KA / 2) + 8 * (blk >> 1) + (s_ >> 1);
      return lds_read_tr8(stage + StageA::BYTES + mc_offset<StageB::ROW_BYTES, EBS>(krow, col));
    };
    auto load_b_frag = [&](const unsigned char* stage, int j, int kk) -> Frag {
      if constexpr (SUBK && !SUBP) {
        const int blk = lane >> 4, s_ = lane & 15;
        const int col = wn * WTN + j * 32 + 16 * (blk & 1) + 8 * (s_ & 1);
        const int krow = kk * KA + 8 * (blk >> 1) + (s_ >> 1);
        const i32x2 v = lds_read_tr8(stage + StageA::BYTES + mc_offset<StageB::ROW_BYTES, EB>(krow, col));
        const float scale = *reinterpret_cast<const float*>(stage + StageA::BYTES + StageB::BYTES +
                                                            4 * (wn * WTN + j * 32 + (lane & 31)));
        if constexpr (EB == kEI8) return i8x8_to_bf16x8_scaled(v, scale);
        else return f8x8_to_bf16x8_scaled(v, scale);
      } else if constexpr (I4F) {
        return i4x32_to_biased_f8x32(load_b_raw(stage, j, kk));
      } else if constexpr (I4I) {
        return i4x16_to_i8x16_times16(load_b_raw8(stage, j, kk));
      } else {
        return load_frag<LB, EBS, EC, StageB::ROW_BYTES>(stage + StageA::BYTES, wn * WTN + j * 32, kk, lane);
      }
    };
    const int span = kc_end - kc_begin;
    const int nfull = span > 0 ? span / BKC : 0;  // whole k-steps: direct-to-LDS, software pipelined
    // (split pipeline: whole A stages, i.e. an even number of compute steps)
    const int nmain = SPLIT ? (span > 0 ? span / BK * 2 : 0) : nfull;
    const bool tail = span > nmain * BKC;         // the rest of the contraction: zero-filled steps through registers

    if constexpr (SPLIT) {
      // The pipelined loop takes whole A stages (pairs of compute steps); what is left of the contraction, less than
      // one A stage, goes through the masked path below.
      const int nfull = nmain;
      DirA da;
      DirB db;
      const int a_hi = max(min(act_end, p.m_ext), 1), a_lo = min(max(act_start, 0), a_hi - 1);
      da.init(row0, p.m_ext, p.lda, wave, lane, a_lo, a_hi);
      db.init(col0, p.nb_ext, p.ldb, wave, lane, 0, p.nb_ext);
      const unsigned char* const gA0 = Ab + DirA::step_base(row0, p.lda, kc_begin);
      const unsigned char* const gB0 = Bb + DirB::step_base(col0, p.ldb, kc_begin);
      const int64_t stepA = DirA::step_bytes(p.lda), stepB = DirB::step_bytes(p.ldb);
      const unsigned smem_lds = lds_address32(smem);
      constexpr int A_BYTES = StageA::BYTES, B_BYTES = StageB::BYTES, B_REGION = NS * A_BYTES;
      constexpr int PA = DirA::PER, PB = DirB::PER;
      static_assert(DirA::INSTRS % NLOAD == 0 && DirB::INSTRS % NLOAD == 0, "split pipeline: the loads split evenly over the waves");
      constexpr int LOOK = HB > 2 * NS ? HB : 2 * NS;  // steps between the issue of a load and the last step that may need it
      constexpr int kFirst = split_loads_in_flight(-1, NS, HB, PA, PB);
      constexpr int kEven = split_loads_in_flight(4 * LOOK, NS, HB, PA, PB), kOdd = split_loads_in_flight(4 * LOOK + 1, NS, HB, PA, PB);
      static_assert(kFirst >= 0 && kEven >= 0 && kOdd >= 0 && kFirst < 64, "split pipeline: load order does not cover a needed step");
      const int ndouble = nfull / 2;
      auto issue_a = [&](int q, int dstep, int stage) {
        da.issue_one(q, uniform_pointer(gA0 + dstep * stepA), smem_lds + stage * A_BYTES, wave);
      };
      auto issue_b = [&](int q, int step, int stage) {
        db.issue_one(q, uniform_pointer(gB0 + step * stepB), smem_lds + B_REGION + stage * B_BYTES, wave);
      };
      // Prologue, in the order of the steady state (steps -LOOK .. -1).
#pragma unroll
      for (int t = -LOOK; t < 0; ++t) {
        if (t & 1) {
          const int j = (t - 1) / 2 + NS;
          if (j >= 0 && j < ndouble) {
#pragma unroll
            for (int q = 0; q < PA; ++q) issue_a(q, j, j);
          }
        }
        const int s_ = t + HB;
        if (s_ >= 0 && s_ < nfull) {
#pragma unroll
          for (int q = 0; q < PB; ++q) issue_b(q, s_, s_);
        }
      }
      if (nfull >= LOOK) barrier_after_direct_loads<kFirst>();
      else barrier_after_direct_loads<0>();

      auto k_loop = [&](auto nv_tag) {
        constexpr int NV = decltype(nv_tag)::value;  // row blocks of this wave that hold rows of the task
        Frag fa[2][TM], fb[2][TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[0][i] = fa[1][i] = Frag{};
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[0][j] = fb[1][j] = Frag{};
        // Read number r of an atom, in the order its MFMAs (row block major) first use the fragments.
        auto read_frag = [&](Frag* a, Frag* b, int r, const unsigned char* atile, int akk, const unsigned char* btile, int bkk) {
          if (r >= TM + TN) return;
          const int f = r == 0 ? 0 : r <= TN ? TM + r - 1 : r - TN;
          if (f < TM) {
            if (f < NV) a[f] = load_frag<LA, EA, EC, StageA::ROW_BYTES>(atile, wm * 32, akk, lane, f * WM * 32);
          } else {
            if (NV > 0) b[f - TM] = load_frag<LB, EB, EC, StageB::ROW_BYTES>(btile, wn * WTN + (f - TM) * 32, bkk, lane);
          }
        };
        constexpr int NM = TM * TN;
        constexpr int RPM = (TM + TN + NM - 1) / NM;
        // One atom: its MFMAs with, threaded between them, the reads of the next atom's fragments and (`NL` > 0) load
        // slots 0 .. NL - 1 of `issue`.
        auto atom = [&](auto nl_tag, const Frag* a, const Frag* b, Frag* na, Frag* nb, const unsigned char* atile, int akk,
                        const unsigned char* btile, int bkk, auto issue) {
          constexpr int NL = decltype(nl_tag)::value;
          constexpr int LPM = (NL + NM - 1) / NM;
#pragma unroll
          for (int t = 0; t < NM; ++t) {
            const int i = t / TN, j = t % TN;
            if (i < NV) acc[i][j] = mma_atom<EC>(b[j], a[i], acc[i][j]);
#pragma unroll
            for (int r = 0; r < RPM; ++r) read_frag(na, nb, t * RPM + r, atile, akk, btile, bkk);
#pragma unroll
            for (int q = 0; q < LPM; ++q)
              if (t * LPM + q < NL) issue(t * LPM + q);
            __builtin_amdgcn_sched_barrier(0);
          }
        };
        auto no_loads = [](int) {};
#pragma unroll
        for (int f = 0; f < TM + TN; ++f) read_frag(fa[0], fb[0], f, smem, 0, smem + B_REGION, 0);
        int a_idx = 0, b_idx = 0;  // stages of the current step
        // One compute step. ODD: second half of its A stage, which it releases. STEADY: every load this step and the
        // LOOK steps before it could issue exists, so the loads in flight are known at compile time; the other steps
        // (the last few of a tile) issue what is left in one piece and wait for everything.
        auto k_step = [&](auto odd_tag, auto steady_tag, int kt) {
          constexpr bool ODD = decltype(odd_tag)::value, STEADY = decltype(steady_tag)::value;
          const unsigned char* const a_cur = smem + a_idx * A_BYTES;
          const unsigned char* const b_cur = smem + B_REGION + b_idx * B_BYTES;
          constexpr int akk0 = ODD ? KSTEPS : 0;
          const int a_freed = a_idx, b_freed = b_idx;
          if (ODD) a_idx = a_idx + 1 == NS ? 0 : a_idx + 1;
          b_idx = b_idx + 1 == HB ? 0 : b_idx + 1;
          const unsigned char* const a_nxt = smem + a_idx * A_BYTES;
          const unsigned char* const b_nxt = smem + B_REGION + b_idx * B_BYTES;
          constexpr int nkk0 = ODD ? 0 : KSTEPS;
          // (Pointers of the refills are computed here, far ahead of the MFMAs they are issued between.)
          const unsigned char* const src_b = uniform_pointer(gB0 + (int64_t)(kt + HB) * stepB);
          const unsigned char* const src_a = uniform_pointer(gA0 + (int64_t)((kt - 1) / 2 + NS) * stepA);
          const unsigned dst_b = smem_lds + B_REGION + b_freed * B_BYTES, dst_a = smem_lds + a_freed * A_BYTES;
#pragma unroll
          for (int kk = 0; kk + 1 < KSTEPS; ++kk)
            atom(std::integral_constant<int, 0>{}, fa[kk & 1], fb[kk & 1], fa[(kk + 1) & 1], fb[(kk + 1) & 1], a_cur,
                 akk0 + kk + 1, b_cur, kk + 1, no_loads);
          // All LDS reads of this step are issued. After the barrier the next step's operands are complete and this
          // step's B stage (and, after an odd step, its A stage) is free.
          if constexpr (STEADY) {
            barrier_after_direct_loads<(ODD ? kOdd : kEven)>();
            auto issue = [&](int q) {
              if (ODD && q < PA) da.issue_one(q, src_a, dst_a, wave);
              else db.issue_one(q - (ODD ? PA : 0), src_b, dst_b, wave);
            };
            atom(std::integral_constant<int, (ODD ? PA : 0) + PB>{}, fa[(KSTEPS - 1) & 1], fb[(KSTEPS - 1) & 1], fa[0], fb[0],
                 a_nxt, nkk0, b_nxt, 0, issue);
          } else {
            barrier_after_direct_loads<0>();
            if (ODD && (kt - 1) / 2 + NS < ndouble) {
#pragma unroll
              for (int q = 0; q < PA; ++q) da.issue_one(q, src_a, dst_a, wave);
            }
            if (kt + HB < nfull) {
#pragma unroll
              for (int q = 0; q < PB; ++q) db.issue_one(q, src_b, dst_b, wave);
            }
            // (After the last step the reads below fetch fragments nobody uses, from LDS that is there.)
            atom(std::integral_constant<int, 0>{}, fa[(KSTEPS - 1) & 1], fb[(KSTEPS - 1) & 1], fa[0], fb[0], a_nxt, nkk0,
                 b_nxt, 0, no_loads);
          }
        };
        int kt = 0;
        for (; kt + 2 + LOOK <= nfull; kt += 2) {
          k_step(std::false_type{}, std::true_type{}, kt);
          k_step(std::true_type{}, std::true_type{}, kt + 1);
        }
        for (; kt < nfull; kt += 2) {
          k_step(std::false_type{}, std::false_type{}, kt);
          k_step(std::true_type{}, std::false_type{}, kt + 1);
        }
      };
      if (nfull > 0) dispatch_upto<0, TM>(nv_sel, k_loop);
    } else if (nfull > 0) {
      DirA da;
      DirB db;
      const int a_hi = max(min(act_end, p.m_ext), 1), a_lo = min(max(act_start, 0), a_hi - 1);
      da.init(row0, p.m_ext, p.lda, wave, lane, a_lo, a_hi);
      db.init(col0, p.nb_ext, p.ldb, wave, lane, 0, p.nb_ext, GLU ? TN : 0, GLU ? p.n_ext : 0);
      const unsigned char* const gA0 = Ab + DirA::step_base(row0, p.lda, kc_begin);
      const unsigned char* const gB0 = Bb + DirB::step_base(col0, p.ldb, I4 ? kc_begin / 2 : kc_begin);
      const int64_t stepA = DirA::step_bytes(p.lda), stepB = DirB::step_bytes(p.ldb);
      const unsigned smem_lds = lds_address32(smem);
      // A load wave may leave the loads of the NS-2 k-steps after the needed one in flight; that
      // count is only known at compile time when the tile splits evenly over the load waves.
      constexpr bool kExact = DirA::INSTRS % NLOAD == 0 && DirB::INSTRS % NLOAD == 0;
      // One k-step of loads is a list of NLD per-wave instructions; slot q of the list can be issued
      // on its own, so that the list can be threaded between MFMAs. kFwdSubK adds one: the 1 KB scale
      // row of the step's k-block, of which every wave fetches its 1/NLOAD with that many of its lanes
      // (so that all waves count the same number of loads).
      constexpr int NLD = DirA::PER + DirB::PER + (SUBP ? (I4F ? 3 : 2) : SUBK ? 1 : 0);
      constexpr int kInFlight = kExact ? (NS - 2) * NLD : 0;
      static_assert(kInFlight < 64 && (NS - 1) * NLD < 64, "too many direct loads in flight for vmcnt");
      struct StepPtrs { const unsigned char *a, *b, *s, *x, *xsum; unsigned lds, ring; };
      // (kFwdSubK) scales of this tile's columns: row `block` of the group's [scale_blocks, n] table; lanes past
      // the last column re-read the last four (their products are never stored).
      const unsigned char* const gS0 =
          SUBK ? reinterpret_cast<const unsigned char*>(p.b_scale + (int64_t)group * p.scale_blocks * p.nb_ext) : nullptr;
      constexpr int SCALE_LANES = 64 / NLOAD;  // lanes of a wave that fetch 16 bytes of the scale row each
      const uint32_t scale_voff = SUBK ? (uint32_t)min(col0 + 4 * (wave * SCALE_LANES + lane), p.nb_ext - 4) * 4u : 0u;
      // (fp8 x fp8) lhs scales [scale_blocks, m]: the BM rows of the tile, 4 per lane; chunks past the last row
      // re-read the last four (m and row0 are multiples of 4, so a chunk is all inside or all outside).
      constexpr int XS_LANES = BM / 4 / NLOAD;
      static_assert(!SUBP || BM / 4 % NLOAD == 0, "the lhs scales of a tile split evenly over the load waves");
      const uint32_t xs_voff = SUBP ? (uint32_t)min(row0 + 4 * (wave * XS_LANES + lane), p.m_ext - 4) * 4u : 0u;
      auto step_ptrs = [&](int step, int stage) {
        StepPtrs sp;
        sp.a = uniform_pointer(gA0 + step * stepA);
        sp.b = uniform_pointer(gB0 + step * stepB);
        sp.s = nullptr;
        if constexpr (SUBK)
          sp.s = uniform_pointer(gS0 + (int64_t)((kc_begin + step * BK) >> p.log2_block_rows) * p.nb_ext * 4);
        if constexpr (SUBP) {
          const int64_t block = (kc_begin + step * BK) >> p.log2_block_rows;
          sp.x = uniform_pointer(reinterpret_cast<const unsigned char*>(p.a_scale) + block * p.m_ext * 4);
          // (fp8 x packed int4) behind the scale_blocks rows of lhs scales: one row of row sums per 128-deep k-step
          if constexpr (I4F)
            sp.xsum = uniform_pointer(reinterpret_cast<const unsigned char*>(p.a_scale) +
                                      (int64_t)(p.scale_blocks + (kc_begin + step * BK) / BK) * p.m_ext * 4);
          sp.ring = smem_lds + NS * STAGE_BYTES + (step % (NS + 1)) * RING_SLOT;
        }
        sp.lds = smem_lds + stage * STAGE_BYTES;
        return sp;
      };
      auto issue_slot = [&](int q, const StepPtrs& sp) {
        if (q < DirA::PER) da.issue_one(q, sp.a, sp.lds, wave);
        else if (q < DirA::PER + DirB::PER) db.issue_one(q - DirA::PER, sp.b, sp.lds + StageA::BYTES, wave);
        else if (SUBK && q == DirA::PER + DirB::PER) {
          const unsigned dst = SUBP ? sp.ring : sp.lds + StageA::BYTES + StageB::BYTES;
          if (lane < SCALE_LANES) direct_load_16(sp.s, scale_voff, dst + wave * (SCALE_LANES * 16));
        } else if (SUBP && q == DirA::PER + DirB::PER + 1) {
          if (lane < XS_LANES) direct_load_16(sp.x, xs_voff, sp.ring + BN * 4 + wave * (XS_LANES * 16));
        } else if (SUBP && I4F && q == DirA::PER + DirB::PER + 2) {
          if (lane < XS_LANES) direct_load_16(sp.xsum, xs_voff, sp.ring + (BN + BM) * 4 + wave * (XS_LANES * 16));
        }
      };
      // Every wave drains the loads the next k-step needs before it arrives at a barrier.
      auto step_barrier = [&](bool partial) {
        if (partial) barrier_after_direct_loads<kInFlight>();
        else barrier_after_direct_loads<0>();
      };

      // Prologue: every stage gets a k-step; wait for the first.
#pragma unroll
      for (int s_ = 0; s_ < NS; ++s_) {
        if (s_ < nfull) {
          const StepPtrs sp = step_ptrs(s_, s_);
#pragma unroll
          for (int q = 0; q < NLD; ++q) issue_slot(q, sp);
        }
      }
      if (kExact && nfull >= NS) barrier_after_direct_loads<(NS - 1) * NLD>();
      else barrier_after_direct_loads<0>();

      // The k loop. Each 32-wide (KA-deep) atom is a run of TM*TN MFMAs; the LDS reads of the next
      // atom's fragments and, in the last atom of a k-step, the global loads that refill the stage
      // just released are threaded between those MFMAs one by one, so that the matrix pipe is
      // never left waiting behind a block of memory instructions.
      auto k_loop = [&](auto nv_tag) {
        constexpr int NV = decltype(nv_tag)::value;  // row blocks of this wave that hold rows of the task
        Frag fa[LEAN ? 1 : 2][TM], fb[2][TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[0][i] = fa[LEAN ? 0 : 1][i] = Frag{};
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[0][j] = fb[1][j] = Frag{};
        // Read number r of an atom, in the order the atom's MFMAs (row block major) first use the
        // fragments: A0, B0, B1, ..., then A1, A2, ... Every fragment is then requested at least
        // TM*TN - 2 MFMAs before its first use. A fragment f < TM is the A fragment of row block f,
        // else the B fragment f - TM.
        // Packed int4 weights: the 8 bytes a lane reads for an even atom hold the B fragments of that atom and of the
        // next; they are kept as read (`raw`) and converted half by half. The list of an even atom is then A0, the
        // byte reads, A1, ..., and last the conversions of the first halves; that of an odd atom A0, the conversions
        // of the second halves, A1, ...
        [[maybe_unused]] i32x2 raw[I4P ? TN : 1];
        [[maybe_unused]] i32x4 rawf[I4F ? TN : 1];  // (fp8 activations) a fragment's bytes as read
        [[maybe_unused]] i32x2 rawi[I4I ? TN : 1];  // (int8 activations) likewise
        // (kFwdSubK: times the scale of the lane's column for the stage's k-block, like load_b_frag)
        [[maybe_unused]] auto convert_i4 = [&](int w, const unsigned char* stage, int j) -> i32x4 {
          if constexpr (SUBK) {
            const float scale = *reinterpret_cast<const float*>(stage + StageA::BYTES + StageB::BYTES +
                                                                4 * (wn * WTN + j * 32 + (lane & 31)));
            return i4x8_to_bf16x8_scaled(w, scale * kPackedInt4Unscale);
          } else {
            return i4x8_to_bf16x8_times16(w);
          }
        };
        constexpr int NRD = I4 ? TM + 2 * TN : TM + TN;  // (fp8 activations: A0, the byte reads, A1, ..., the conversions)  // entries of an atom's list
        auto read_frag = [&](Frag* a, Frag* b, int r, const unsigned char* stage, int kk) {
          if (r >= NRD) return;
          const int f = r == 0 ? 0 : r <= TN ? TM + r - 1 : r < TM + TN ? r - TN : r;
          if (f < TM) {
            if (f < NV) a[f] = load_frag<LA, EA, EC, StageA::ROW_BYTES, I4P>(stage, wm * 32, kk, lane, f * WM * 32);
          } else if (f < TM + TN) {
            if constexpr (I4F) {
              if (NV > 0) rawf[f - TM] = load_b_raw(stage, f - TM, kk);
            } else if constexpr (I4I) {
              if (NV > 0) rawi[f - TM] = load_b_raw8(stage, f - TM, kk);
            } else if constexpr (I4P) {
              const int j = f - TM;
              if (NV > 0) {
                if (kk & 1) {
                  b[j] = convert_i4(raw[j][1], stage, j);
                } else {
                  const int blk = lane >> 4, s_ = lane & 15;
                  const int col = wn * WTN + j * 32 + 16 * (blk & 1) + 8 * (s_ & 1);
                  const int krow = (kk >> 1) * 16 + 8 * (blk >> 1) + (s_ >> 1);
                  raw[j] = lds_read_tr8(stage + StageA::BYTES + mc_offset<StageB::ROW_BYTES, EBS>(krow, col));
                }
              }
            } else {
              if (NV > 0) b[f - TM] = load_b_frag(stage, f - TM, kk);
            }
          } else if constexpr (I4F) {
            if (NV > 0) b[f - TM - TN] = i4x32_to_biased_f8x32(rawf[f - TM - TN]);
          } else if constexpr (I4I) {
            if (NV > 0) b[f - TM - TN] = i4x16_to_i8x16_times16(rawi[f - TM - TN]);
          } else if constexpr (I4P) {
            if (NV > 0 && !(kk & 1)) b[f - TM - TN] = convert_i4(raw[f - TM - TN][0], stage, f - TM - TN);
          }
        };
        constexpr int NM = TM * TN;                      // MFMAs per atom
        constexpr int RPM = (NRD + NM - 1) / NM;         // list entries threaded after each MFMA
        constexpr int LPM = (NLD + NM - 1) / NM;         // load slots threaded after each MFMA
        // (`reads` and `loads` are compile-time tags: a run-time test after every MFMA would put two
        // branches into each MFMA slot.)
        auto atom = [&](auto reads_tag, auto loads_tag, const Frag* a, const Frag* b, Frag* na, Frag* nb,
                        const unsigned char* rd_stage, int rd_kk, const StepPtrs& sp, auto first_tag) {
          constexpr bool reads = decltype(reads_tag)::value, loads = decltype(loads_tag)::value;
          constexpr bool first_of_step = decltype(first_tag)::value;  // (SUBP) the partial accumulators start at zero
          if constexpr (JOUT) {
#pragma unroll
            for (int t = 0; t < NM; ++t) {
              const int j = t / TM, i = t % TM;
              if (i < NV) acc[i][j] = mma_atom<EC>(fb[0][j], fa[0][i], acc[i][j]);
              if (t < TN - 1 && NV > 0) fb[0][t + 1] = i4x32_to_biased_f8x32(rawf[t + 1]);
              if (reads) {
                // (the buffer of fragment 0's bytes is free since the previous atom, that of fragment t since the line above)
                if (t < TN && NV > 0) rawf[t] = load_b_raw(rd_stage, t, rd_kk);
                if (t == TM && NV > 0) fb[0][0] = i4x32_to_biased_f8x32(rawf[0]);
                if (j == TN - 1 && i < NV)
                  fa[0][i] = load_frag<LA, EA, EC, StageA::ROW_BYTES>(rd_stage, wm * 32, rd_kk, lane, i * WM * 32);
              }
              if (loads) {
#pragma unroll
                for (int q = 0; q < LPM; ++q) issue_slot(t * LPM + q, sp);
              }
              __builtin_amdgcn_sched_barrier(0);
            }
            return;
          }
#pragma unroll
          for (int t = 0; t < NM; ++t) {
            const int i = t / TN, j = t % TN;
            if constexpr (SUBP) {
              if (i < NV) {
                f32x16 c = pacc[i][j];
                if constexpr (first_of_step) {
#pragma unroll
                  for (int e = 0; e < 16; ++e) c[e] = 0.f;
                }
                pacc[i][j] = mma_atom<EC>(b[j], a[i], c);
              }
            } else {
              if (i < NV) acc[i][j] = mma_atom<EC>(b[j], a[i], acc[i][j]);
            }
            if (reads) {
              if constexpr (LEAN) {
                // rhs fragment t after MFMA t; the lhs fragment of a row block after the block's last MFMA
                if (t < TN) read_frag(na, nb, t + 1, rd_stage, rd_kk);
                if (j == TN - 1) read_frag(na, nb, i == 0 ? 0 : TN + i, rd_stage, rd_kk);
                if constexpr (I4F) {
                  // the bytes of rhs fragment c become fp8 two MFMAs or more after their read was issued
                  constexpr int LAG = TN == 1 ? 2 : TN;
                  if (t >= LAG && t < LAG + TN) read_frag(na, nb, TM + TN + t - LAG, rd_stage, rd_kk);
                }
              } else {
#pragma unroll
                for (int r = 0; r < RPM; ++r) read_frag(na, nb, t * RPM + r, rd_stage, rd_kk);
              }
            }
            if (loads) {
#pragma unroll
              for (int q = 0; q < LPM; ++q) issue_slot(t * LPM + q, sp);
            }
            __builtin_amdgcn_sched_barrier(0);
          }
        };

        if constexpr (JOUT) {
#pragma unroll
          for (int i = 0; i < TM; ++i)
            if (i < NV) fa[0][i] = load_frag<LA, EA, EC, StageA::ROW_BYTES>(smem, wm * 32, 0, lane, i * WM * 32);
#pragma unroll
          for (int j = 0; j < TN; ++j)
            if (NV > 0) rawf[j] = load_b_raw(smem, j, 0);
          if (NV > 0) fb[0][0] = i4x32_to_biased_f8x32(rawf[0]);
        } else {
#pragma unroll
          for (int f = 0; f < NRD; ++f) read_frag(fa[0], fb[0], f, smem, 0);
        }
        int cur_stage = 0;
        const StepPtrs none = {};
        // One k-step. `refill_tag`: the stage it releases is refilled with k-step kt + NS;
        // `more_tag`: another k-step follows, so the next stage's first fragments are read.
        auto k_step = [&](auto refill_tag, auto more_tag, int kt) {
          const unsigned char* cur = smem + cur_stage * STAGE_BYTES;
          const int freed = cur_stage;
          cur_stage = cur_stage + 1 == NS ? 0 : cur_stage + 1;
          const unsigned char* nxt = smem + cur_stage * STAGE_BYTES;
          // (Pointers of the refill are computed here, far ahead of the MFMAs they are issued between.)
          const StepPtrs sp = decltype(refill_tag)::value ? step_ptrs(kt + NS, freed) : none;
          static_assert(!(SUBP && EC == kEF8) || KSTEPS == 2, "the partial accumulators restart with the first of two atoms");
          // int8: the int32 sums stay exact over a whole k-block, so they are folded in at the end of the block
          // only (a fold costs as much vector work as three k-steps of int8 MFMAs); fp8: after every k-step.
          [[maybe_unused]] bool block_end = true;
          if constexpr (SUBP && EC == kEI8) {
            const int mask = (1 << p.log2_block_rows) - 1;
            const int k0 = kc_begin + kt * BK;
            block_end = ((k0 + BK) & mask) == 0 || kt + 1 == nfull;
            if ((k0 & mask) == 0) {
#pragma unroll
              for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                  for (int e = 0; e < 16; ++e) pacc[i][j][e] = 0.f;
            }
#pragma unroll
            for (int kk = 0; kk + 1 < KSTEPS; ++kk)
              atom(std::true_type{}, std::false_type{}, fa[kk & 1], fb[kk & 1], fa[(kk + 1) & 1], fb[(kk + 1) & 1], cur,
                   kk + 1, none, std::false_type{});
          } else if constexpr (SUBP) {
            atom(std::true_type{}, std::false_type{}, fa[0], fb[0], fa[1], fb[1], cur, 1, none, std::true_type{});
          } else {
#pragma unroll
            for (int kk = 0; kk + 1 < KSTEPS; ++kk)
              atom(std::true_type{}, std::false_type{}, fa[LEAN ? 0 : kk & 1], fb[kk & 1], fa[LEAN ? 0 : (kk + 1) & 1],
                   fb[(kk + 1) & 1], cur, kk + 1, none, std::false_type{});
          }
          // All LDS reads of `cur` are issued. After the barrier the next stage is complete and `cur`
          // is free: the last atom's MFMAs cover the first fragment reads of the next stage and the
          // issue of the loads that refill `cur` with k-step kt + NS.
          step_barrier(decltype(refill_tag)::value || kt + NS - 1 < nfull);
          atom(more_tag, refill_tag, fa[LEAN ? 0 : (KSTEPS - 1) & 1], fb[(KSTEPS - 1) & 1], fa[0], fb[0], nxt, 0, sp, std::false_type{});
          if constexpr (SUBP) if (block_end) {
            // Fold the products into the result with the scales of their k-block: lane l holds row l % 32
            // and, for t = 0..3, columns 8 t + 4 (l / 32) + {0..3} of every 32 x 32 block.
            const unsigned char* slot = smem + NS * STAGE_BYTES + (kt % (NS + 1)) * RING_SLOT;
            float xs[TM];
            // (fp8 x packed int4: the weights went in as (w + 8) / 512, so a product sum is 512 part - 8 rowsum(x); with
            // xs' = 512 xs and xoff = -8 rowsum xs a fold is two fused multiply-adds per element: ws (xs' part + xoff))
            [[maybe_unused]] float xoff[TM];
#pragma unroll
            for (int i = 0; i < TM; ++i) {
              xs[i] = *reinterpret_cast<const float*>(slot + BN * 4 + 4 * (row_block(i) * 32 + (lane & 31)));
              if constexpr (I4I) xs[i] *= kPackedInt4Unscale;  // (the weights went into the MFMAs times 16)
              if constexpr (I4F) {
                xoff[i] = -8.f * xs[i] * *reinterpret_cast<const float*>(slot + (BN + BM) * 4 + 4 * (row_block(i) * 32 + (lane & 31)));
                xs[i] *= 512.f;
              }
            }
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
              for (int t = 0; t < 4; ++t) {
                const f32x4 wsc = *reinterpret_cast<const f32x4*>(slot + 4 * (wn * WTN + j * 32 + 8 * t + 4 * (lane >> 5)));
#pragma unroll
                for (int i = 0; i < TM; ++i)
                  if (i < NV) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                      float part = pacc[i][j][4 * t + e];
                      if constexpr (EC == kEI8) part = (float)__builtin_bit_cast(int, part);  // int32 partial sums
                      if constexpr (I4F) acc[i][j][4 * t + e] = fmaf(wsc[e], fmaf(xs[i], part, xoff[i]), acc[i][j][4 * t + e]);
                      else acc[i][j][4 * t + e] += part * (xs[i] * wsc[e]);
                    }
                  }
              }
          }
        };
        // Steady state first (every step refills), then the last NS steps in loops of their own, so
        // that the hot loop is one straight-line body.
        int kt = 0;
        for (; kt + NS < nfull; ++kt) k_step(std::true_type{}, std::true_type{}, kt);
        for (; kt + 1 < nfull; ++kt) k_step(std::false_type{}, std::true_type{}, kt);
        for (; kt < nfull; ++kt) k_step(std::false_type{}, std::false_type{}, kt);
      };
      dispatch_upto<0, TM>(nv_sel, k_loop);
      if constexpr (I4P && !SUBK) {
        // (the weights went into the MFMAs times 16)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) acc[i][j] *= kPackedInt4Unscale;
      }
    }
    // (gate-up, per-k-block-scale and packed-int4 problems are taken only with whole k-steps)
    if constexpr (!GLU && !SUBK && !I4) if (tail) {
      typedef TileStage<LA, EA, BM, BKC, THREADS> TailA;  // (an A tile as deep as a compute step)
      for (int kc0 = kc_begin + nmain * BKC; kc0 < kc_end; kc0 += BKC) {
        if (kc0 > kc_begin) __syncthreads();  // the tile's last reads of the LDS written below are done
        TailA::copy(Ab, p.lda, row0, p.m_ext, kc0, kc_end, smem, tid);
        StageB::copy(Bb, p.ldb, col0, p.nb_ext, kc0, kc_end, smem + TailA::BYTES, tid);
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < KSTEPS; ++kk) {
          Frag fa[TM], fb[TN];
#pragma unroll
          for (int i = 0; i < TM; ++i) fa[i] = Frag{};
#pragma unroll
          for (int j = 0; j < TN; ++j) fb[j] = Frag{};
#pragma unroll
          for (int i = 0; i < TM; ++i)
            if ((rmask >> i) & 1u) fa[i] = load_frag<LA, EA, EC, TailA::ROW_BYTES>(smem, row_block(i) * 32, kk, lane);
          if (rmask != 0) {
#pragma unroll
            for (int j = 0; j < TN; ++j)
              fb[j] = load_frag<LB, EB, EC, StageB::ROW_BYTES>(smem + TailA::BYTES, wn * WTN + j * 32, kk, lane);
          }
#pragma unroll
          for (int i = 0; i < TM; ++i)
            if ((rmask >> i) & 1u) {
#pragma unroll
              for (int j = 0; j < TN; ++j) acc[i][j] = mma_atom<EC>(fb[j], fa[i], acc[i][j]);
            }
        }
      }
    }

    if constexpr (SK) if (parts > 1) {
      // A tile in parts: every part writes its f32 sums to its slot of the workspace (stores of device scope: they go
      // through to memory instead of staying in this XCD's L2), waits for them to complete and counts itself in at
      // the tile's counter. Whoever arrives last adds all parts in the order of their index (its own from memory as
      // well, so that the bits do not depend on who that is) and goes on to the epilogue; the others are done.
      // Lane-major layout: quarter q of accumulator block (i, j) of thread t is 16 bytes at ((i TN + j) 4 + q) THREADS + t.
      constexpr int TILE_FLOATS = BM * BN;
      const uint32_t lane_off = (uint32_t)tid * 16u;
      auto slot = [&](int unit) {
        const unsigned char* ptr = uniform_pointer(reinterpret_cast<const unsigned char*>(p.split_partials + (int64_t)unit * TILE_FLOATS));
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char*>(ptr), 0, TILE_FLOATS * 4, 0x00020000);
      };
      constexpr int kDeviceScope = 16;  // cache-policy operand of buffer accesses: sc1
      {
        const __amdgpu_buffer_rsrc_t mine = slot(split_unit);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const f32x4 v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
              __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(i32x4, v), mine, (int)lane_off,
                                                     ((i * TN + j) * 4 + q) * THREADS * 16, kDeviceScope);
            }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();  // (also: every wave is done reading the last stage, whose first word carries the verdict below)
      int* verdict = reinterpret_cast<int*>(smem);
      if (tid == 0) {
        int32_t* counter = const_cast<int32_t*>(ws) + p.ws_split_counters + (split_unit - part) / parts;
        const int arrived = atomicAdd(counter, 1);
        *verdict = arrived == parts - 1;
        if (arrived == parts - 1) atomicExch(counter, 0);
      }
      __syncthreads();
      const bool last = *verdict != 0;
      __syncthreads();
      if (!last) return;
#pragma unroll 1
      for (int pp = 0; pp < parts; ++pp) {
        const __amdgpu_buffer_rsrc_t theirs = slot(split_unit - part + pp);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          // (One row block's loads in flight at a time: all of a part's at once need as many registers again as the
          // accumulators they are added to.)
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const f32x4 v = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(
                                                            theirs, (int)lane_off, ((i * TN + j) * 4 + q) * THREADS * 16, kDeviceScope));
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                if constexpr (EC == kEI8 && !SUBP) {
                  // (int8 x int8: the registers hold the bits of exact int32 sums)
                  // (scalar copies first: a bit cast applied to a vector's element read element 0)
                  const float have = acc[i][j][4 * q + e], add = v[e];
                  const int sum = __builtin_bit_cast(int, have) + __builtin_bit_cast(int, add);
                  acc[i][j][4 * q + e] = pp == 0 ? add : __builtin_bit_cast(float, sum);
                } else {
                  acc[i][j][4 * q + e] = pp == 0 ? v[e] : acc[i][j][4 * q + e] + v[e];
                }
              }
            }
        }
      }
    }

    // Epilogue. After the swapped MFMA, lane l of atom (i, j) holds C row (l % 32) and, for
    // t = 0..3, columns 8t + 4*(l / 32) + {0,1,2,3} of that atom. Scales and the activation are
    // applied to the accumulators in registers first (each in one pass, with the run-time choices
    // made outside the unrolled loops); the stores then only convert and write. A store's address
    // is the tile's (uniform) base plus one lane offset per row block plus a constant.
    {
      unsigned char* Cg = reinterpret_cast<unsigned char*>(p.C);
      if constexpr (MODE == kDrhs) Cg += (int64_t)group * p.c_group_stride * (p.out_dtype == TKX_F32 ? 4 : 2);
      if constexpr (EC == kEI8 && !SUBP) {
        // int8 x int8 with one scale per row and per column: the accumulators hold the exact int32 sums.
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
              const float bits = acc[i][j][e];  // (a scalar copy first: a bit cast straight from a vector element misreads)
              acc[i][j][e] = (float)__builtin_bit_cast(int, bits) * (I4I ? kPackedInt4Unscale : 1.f);
            }
      }
      const bool inside = col0 + BNO <= p.n_ext;
      // Column of B (of its scales and bias) behind accumulator block j, element group t of this lane.
      auto b_col = [&](int j, int t) {
        const int c = GLU ? (j < TNO ? 0 : p.n_ext) + col0 + wn * WTNO + (j % TNO) * 32 : col0 + wn * WTN + j * 32;
        return min(c + 4 * (lane >> 5) + 8 * t, p.nb_ext - 4);
      };
      if (!SUBP && p.a_scale != nullptr) {  // (SUBP: folded in per k-block)
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          const int row = min(row0 + row_block(i) * 32 + (lane & 31), p.m_ext - 1);
          const float rs = p.a_scale[row];
          if constexpr (I4F) {
            const float off = 8.f * p.a_scale[p.m_ext + row];
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
              for (int e = 0; e < 16; ++e) acc[i][j][e] = 512.f * acc[i][j][e] - off;
          }
#pragma unroll
          for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] *= rs;
        }
      }
      if (!SUBK && p.b_scale != nullptr) {  // (kFwdSubK: applied to the weights on their way into the MFMAs)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const f32x4 cs = *reinterpret_cast<const f32x4*>(p.b_scale + (int64_t)group * p.nb_ext + b_col(j, t));
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
              for (int e = 0; e < 4; ++e) acc[i][j][4 * t + e] *= cs[e];
          }
        }
      }
      if (p.b_bias != nullptr) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const f32x4 cb = *reinterpret_cast<const f32x4*>(p.b_bias + (int64_t)group * p.nb_ext + b_col(j, t));
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
              for (int e = 0; e < 4; ++e) acc[i][j][4 * t + e] += cb[e];
          }
        }
      }
      if constexpr (GLU) {
        // The clamped gate-up forms clip the gate from above and the up part from both sides first;
        // "swigluoai" multiplies by up + 1.
        if (p.activation == TKX_ACT_SWIGLU_OAI || p.activation == TKX_ACT_SILU_CLAMP) {
          const float limit = p.activation == TKX_ACT_SWIGLU_OAI ? 7.f : 10.f;
          const float shift = p.activation == TKX_ACT_SWIGLU_OAI ? 1.f : 0.f;
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TNO; ++j)
#pragma unroll
              for (int e = 0; e < 16; ++e) {
                acc[i][j][e] = fminf(acc[i][j][e], limit);
                acc[i][j + TNO][e] = fminf(fmaxf(acc[i][j + TNO][e], -limit), limit) + shift;
              }
        }
      }
      if (p.activation != TKX_ACT_NONE) {
        // tanh(x) = 1 - 2 / (exp(2x) + 1): a handful of instructions per element with the hardware
        // exponential and reciprocal.
        auto fast_tanh = [](float x) { return 1.f - 2.f * __builtin_amdgcn_rcpf(__expf(2.f * x) + 1.f); };
        // Block by block, with the choice of the function inside: one choice around all blocks made every
        // accumulator meet again after six branches, and the register allocator spilled one of them on the way.
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TNO; ++j) {  // (gate-up: the gate blocks only)
            f32x16 c = acc[i][j];
            auto apply = [&](auto fn) {
#pragma unroll
              for (int e = 0; e < 16; ++e) c[e] = fn(c[e]);
            };
            if (p.activation == TKX_ACT_RELU) apply([](float x) { return x > 0.f ? x : 0.f; });
            else if (p.activation == TKX_ACT_TANH) apply(fast_tanh);
            else if (p.activation == TKX_ACT_SILU || p.activation == TKX_ACT_SILU_CLAMP)
              apply([](float x) { return x * __builtin_amdgcn_rcpf(1.f + __expf(-x)); });
            else if (p.activation == TKX_ACT_SWIGLU_OAI)
              apply([](float x) { return x * __builtin_amdgcn_rcpf(1.f + __expf(-1.702f * x)); });
            else if (p.activation == TKX_ACT_SIGMOID) apply([](float x) { return __builtin_amdgcn_rcpf(1.f + __expf(-x)); });
            else if (p.activation == TKX_ACT_GELU_TANH)
              apply([&](float x) { return 0.5f * x * (1.f + fast_tanh(0.7978845608028654f * (x + 0.044715f * x * x * x))); });
            acc[i][j] = c;
          }
      }
      if constexpr (GLU) {
        // act(gate) * up: block j and block j + TNO of a lane are gate and up of the same output columns.
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TNO; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] *= acc[i][j + TNO][e];
      }
      // The stores go through LDS (free once the k loop is done): as the MFMA leaves them, a
      // lane's values are 4 columns of one row, so a store straight from registers writes 16-byte
      // pieces of 32 different rows and the memory pipeline takes it apart line by line. Each wave
      // lays its part of the tile out row-major in its own slice of LDS and reads it back 16 bytes
      // per lane, so that a store instruction writes whole 128-byte (or longer) row segments.
      __syncthreads();  // every wave is done reading the last stage
      // fp8 output: one scale per (row, 128 columns) = absmax / 448 (1 for a run of zeros), values multiplied by the
      // reciprocal of the scale and converted with saturation: the arithmetic of the reference's fused quantisation
      // (pallas_mosaic_gpu_kernel_sm100_fp8_quant.py:802-822). (The standalone pass, launch_quantize, divides, as a
      // quantiser that never sees the accumulator would: the two can differ by one fp8 step where a quotient lies on
      // a rounding boundary.) A row's 128 columns lie in 128 / WTN wave columns: each wave reduces its part of every
      // row (a lane's 16 TN values, then the lane 32 further on, which holds the row's other columns) and the waves
      // exchange them through LDS.
      float row_scale[TM][WTN > 128 ? WTN / 128 : 1];
      if constexpr (QO) {
        {
          constexpr int QW = WTN >= 128 ? 1 : 128 / WTN;   // wave columns per quantisation tile
          constexpr int QT = WTN > 128 ? WTN / 128 : 1;    // quantisation tiles per wave column
          constexpr int JT = TN / QT;                      // accumulator blocks per quantisation tile
          float* xchg = reinterpret_cast<float*>(smem);    // [waves][TM * 32 rows][QT]
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int q = 0; q < QT; ++q) {
              float mx = 0.f;
#pragma unroll
              for (int j = q * JT; j < (q + 1) * JT; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) mx = fmaxf(mx, fabsf(acc[i][j][e]));
              mx = fmaxf(mx, __shfl_xor(mx, 32));
              if (lane < 32) xchg[(wave * TM * 32 + i * 32 + lane) * QT + q] = mx;
            }
          __syncthreads();
          const int wn0 = wn / QW * QW;  // first wave column of this wave's quantisation tile
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int q = 0; q < QT; ++q) {
              float mx = 0.f;
#pragma unroll
              for (int w = 0; w < QW; ++w) mx = fmaxf(mx, xchg[((wm * WN + wn0 + w) * TM * 32 + i * 32 + (lane & 31)) * QT + q]);
              const float scale = mx == 0.f ? 1.f : mx / 448.f;
              row_scale[i][q] = 1.f / scale;  // (the values are multiplied by the reciprocal, as the reference's epilogue does)
              const int row = row0 + row_block(i) * 32 + (lane & 31);
              const int qcol = (col0 + wn * WTN) / 128 + q;
              if (lane < 32 && wn == wn0 && row >= act_start && row < act_end && qcol * 128 < p.n_ext)
                p.c_scale[(int64_t)row * (p.ldc / 128) + qcol] = scale;
            }
          __syncthreads();  // the exchange area is part of the staging slices below
        }
      }
      auto emit = [&](auto out_tag) {
        constexpr int OUT = decltype(out_tag)::value;
        constexpr int ESZ = OUT == TKX_F32 ? 4 : OUT == TKX_F8E4M3FN ? 1 : 2;
        constexpr int ROW_BYTES = WTNO * ESZ;
        constexpr int PITCH = ROW_BYTES + 16;                     // keeps 16-byte alignment, staggers banks
        constexpr int WAVE_LDS = (SMEM_BYTES / (WM * WN)) / 16 * 16;
        constexpr int AP = (WAVE_LDS / PITCH) / 32 < TM ? (WAVE_LDS / PITCH) / 32 : TM;  // atoms (32 rows) per pass
        static_assert(AP >= 1, "a wave's LDS slice must hold 32 output rows");
        constexpr int CPR = ROW_BYTES / 16;                       // 16-byte chunks per row
        constexpr int RPI = 64 / CPR;                             // rows per store instruction
        static_assert(64 % CPR == 0 && CPR <= 64, "a store instruction must cover whole rows");
        static_assert(32 % RPI == 0, "a store instruction must stay inside one 32-row block");
        unsigned char* const slice = smem + wave * WAVE_LDS;
        unsigned char* const tile = const_cast<unsigned char*>(uniform_pointer(Cg + ((int64_t)row0 * p.ldc + col0) * ESZ));
        const int rd_row = lane / CPR, rd_chunk = lane % CPR;
        const int gcol = col0 + wn * WTNO + rd_chunk * (16 / ESZ);
        const bool col_ok = inside || gcol + 16 / ESZ <= p.n_ext;
        const uint32_t voff = (uint32_t)(((wm * 32 + rd_row) * (int)p.ldc + wn * WTNO + rd_chunk * (16 / ESZ)) * ESZ);
#pragma unroll
        for (int i0 = 0; i0 < TM; i0 += AP) {
#pragma unroll
          for (int ii = 0; ii < AP; ++ii) {
            if (i0 + ii >= TM) break;
            const int i = i0 + ii;
#pragma unroll
            for (int j = 0; j < TNO; ++j) {
#pragma unroll
              for (int t = 0; t < 4; ++t) {
                f32x4 v;
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = acc[i][j][4 * t + e];
                unsigned char* dst = slice + (ii * 32 + (lane & 31)) * PITCH + (j * 32 + 8 * t + 4 * (lane >> 5)) * ESZ;
                if constexpr (OUT == TKX_F8E4M3FN) {
                  constexpr int JT = TN / (WTN > 128 ? WTN / 128 : 1);
                  const float inv = row_scale[i][j / JT];
                  float q4[4];
#pragma unroll
                  for (int e = 0; e < 4; ++e) q4[e] = fminf(fmaxf(v[e] * inv, -448.f), 448.f);
                  int w = 0;
                  w = __builtin_amdgcn_cvt_pk_fp8_f32(q4[0], q4[1], w, false);
                  w = __builtin_amdgcn_cvt_pk_fp8_f32(q4[2], q4[3], w, true);
                  *reinterpret_cast<int*>(dst) = w;
                } else if constexpr (OUT == TKX_F32) {
                  *reinterpret_cast<f32x4*>(dst) = v;
                } else if constexpr (OUT == TKX_BF16) {
                  bf16x4 o;
#pragma unroll
                  for (int e = 0; e < 4; ++e) o[e] = (__bf16)v[e];
                  *reinterpret_cast<bf16x4*>(dst) = o;
                } else {
                  f16x4 o;
#pragma unroll
                  for (int e = 0; e < 4; ++e) o[e] = (_Float16)v[e];
                  *reinterpret_cast<f16x4*>(dst) = o;
                }
              }
            }
          }
          constexpr int ROWS = AP * 32;
#pragma unroll
          for (int s_ = 0; s_ < ROWS / RPI; ++s_) {
            const int srow = s_ * RPI;                                // first slice row of this instruction
            const int i = i0 + srow / 32;                             // the wave's row block it belongs to
            if (i >= TM) continue;
            const int trow = i * WM * 32 + srow % 32;                 // tile row, less the lane part in voff
            const int row = row0 + trow + wm * 32 + rd_row;
            const i32x4 val = *reinterpret_cast<const i32x4*>(slice + (s_ * RPI + rd_row) * PITCH + rd_chunk * 16);
            // (Non-temporal: the output is not read again by this kernel and should not displace
            // the operand panels the other workgroups of the XCD share in L2.)
            if (row >= act_start && row < act_end && col_ok)
              __builtin_nontemporal_store(val, (__attribute__((address_space(1))) i32x4*)(tile + (size_t)trow * p.ldc * ESZ + voff));
          }
        }
      };
      if constexpr (QO) emit(std::integral_constant<int, TKX_F8E4M3FN>{});
      else if (p.out_dtype == TKX_BF16) emit(std::integral_constant<int, TKX_BF16>{});
      else if (p.out_dtype == TKX_F32) emit(std::integral_constant<int, TKX_F32>{});
      else emit(std::integral_constant<int, TKX_F16>{});
    }
  }
};

// (4-wave workgroups whose LDS lets two of them share a CU: at most 256 registers per lane, so that two do fit.)
template <class K>
__global__ __launch_bounds__(K::THREADS, K::kWavesPerSimd) void gemm_entry(const GemmParams p) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char tkx_smem[];
  K::run(p, tkx_smem);
}
template <class K>
__global__ __launch_bounds__(K::THREADS, K::kWavesPerSimd) void gemm_entry_fp8_out(const GemmParams p) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char tkx_smem[];
  K::template run<true>(p, tkx_smem);
}
template <class K>
__global__ __launch_bounds__(K::THREADS, K::kWavesPerSimd) void gemm_entry_split(const GemmParams p) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char tkx_smem[];
  K::template run<false, true>(p, tkx_smem);
}
// The entry that splits the last round of a kernel that has one, else null.
template <class K>
const void* split_entry() {
  if constexpr (K::SPLITK) return reinterpret_cast<const void*>(&gemm_entry_split<K>);
  else return nullptr;
}
// The quantising entry of a kernel that has one, else null.
template <class K>
const void* fp8_out_entry() {
  if constexpr (K::QOUT) return reinterpret_cast<const void*>(&gemm_entry_fp8_out<K>);
  else return nullptr;
}

#define TKX_VARIANT_SPLIT(MODE, EA, EB, BM, BN, BK, WM, WN, NS, HB)                                           \
  {                                                                                                            \
    MODE, EA, EB, BM, BN, BK, WM, WN, NS, ::tkx::GemmKernel<MODE, EA, EB, BM, BN, BK, WM, WN, NS, HB>::SMEM_BYTES, \
        reinterpret_cast<const void*>(&::tkx::gemm_entry<::tkx::GemmKernel<MODE, EA, EB, BM, BN, BK, WM, WN, NS, HB>>), HB, \
        ::tkx::fp8_out_entry<::tkx::GemmKernel<MODE, EA, EB, BM, BN, BK, WM, WN, NS, HB>>(),                      \
        ::tkx::split_entry<::tkx::GemmKernel<MODE, EA, EB, BM, BN, BK, WM, WN, NS, HB>>()                         \
  }

#define TKX_VARIANT(MODE, EA, EB, BM, BN, BK, WM, WN, NS)                                            \
  {                                                                                                  \
    MODE, EA, EB, BM, BN, BK, WM, WN, NS, ::tkx::GemmKernel<MODE, EA, EB, BM, BN, BK, WM, WN, NS>::SMEM_BYTES, \
        reinterpret_cast<const void*>(&::tkx::gemm_entry<::tkx::GemmKernel<MODE, EA, EB, BM, BN, BK, WM, WN, NS>>), 0, \
        ::tkx::fp8_out_entry<::tkx::GemmKernel<MODE, EA, EB, BM, BN, BK, WM, WN, NS>>(),                       \
        ::tkx::split_entry<::tkx::GemmKernel<MODE, EA, EB, BM, BN, BK, WM, WN, NS>>()                          \
  }

}  // namespace tkx
