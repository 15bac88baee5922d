// Grouped (ragged) GEMM for gfx950: one templated kernel behind every dtype / mode.
//
//   C[rows, cols] = sum over the contraction of A(row, kc) * B(kc, col)
//
//   mode kFwd  : A = lhs  [m,k]  contraction-contiguous   B = rhs[g] [k,n]  column-contiguous
//   mode kDlhs : A = dout [m,n]  contraction-contiguous   B = rhs[g] [k,n]  contraction-contiguous
//                (C[m,k] = dout . rhs[g]^T: rhs is read in place, never transposed in memory)
//   mode kDrhs : A = lhs  [m,k]  row(k-index)-contiguous  B = dout [m,n]    column-contiguous
//                (C[g][k,n] = lhs[rows_g]^T . dout[rows_g]; contraction = the group's row range)
//
// A workgroup owns one BM x BN tile of C. k-steps of BK contraction elements are staged through
// two LDS buffers (global -> registers -> LDS, the next step's global loads in flight during the
// MFMAs of the current one). Operands that are contraction-contiguous are read from LDS with
// ds_read_b128; operands that are contiguous along the other axis are read with the gfx950
// transposing LDS loads (ds_read_b64_tr_b16 / _tr_b8), so no operand is ever transposed in memory.
// The 32x32 MFMA is issued with its operands swapped (B-fragment first) so that each lane ends up
// holding runs of 4 consecutive C columns of one C row: the epilogue stores 8/16-byte vectors.
#pragma once

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

enum ElemKind { kEF32 = TKX_F32, kEBF16 = TKX_BF16, kEF16 = TKX_F16, kEF8 = TKX_F8E4M3FN, kEI8 = TKX_I8 };
enum OperandLayout { kKC = 0 /* contraction-contiguous */, kMC = 1 /* contiguous along rows/cols */ };

__host__ __device__ constexpr int elem_bytes(int e) { return e == kEF32 ? 4 : (e == kEBF16 || e == kEF16) ? 2 : 1; }

// MFMA flavour chosen by the A element kind: contraction elements per 32x32 atom and fragment bytes.
template <int EA> struct Mma;
template <> struct Mma<kEBF16> { static constexpr int KA = 16; typedef i32x4 Frag; };
template <> struct Mma<kEF16> { static constexpr int KA = 16; typedef i32x4 Frag; };
template <> struct Mma<kEF32> { static constexpr int KA = 8; typedef i32x4 Frag; };
template <> struct Mma<kEF8> { static constexpr int KA = 64; typedef i32x8 Frag; };

template <int EA>
__device__ __forceinline__ f32x16 mma_atom(const typename Mma<EA>::Frag& first, const typename Mma<EA>::Frag& second,
                                           f32x16 acc) {
  if constexpr (EA == kEBF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, first),
                                                   __builtin_bit_cast(bf16x8, second), acc, 0, 0, 0);
  } else if constexpr (EA == kEF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, first),
                                                  __builtin_bit_cast(f16x8, second), acc, 0, 0, 0);
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
// 16/32 lanes of one ds_read_b128 phase touch distinct banks.
template <int ROW_BYTES>
__device__ __forceinline__ int kc_offset(int row, int chunk) {
  constexpr int CPR = ROW_BYTES / 16;
  const int s = ((row & 7) ^ ((row >> 3) & 1)) & (CPR - 1);
  return row * ROW_BYTES + ((chunk ^ s) << 4);
}

// Row/column-contiguous tile: [BK rows of k][ROW_BYTES], 32-byte granules XOR-swizzled by k.
// E selects the pattern that suits the read instruction used for that element size.
template <int ROW_BYTES, int E>
__device__ __forceinline__ int mc_offset(int krow, int byte_in_row) {
  constexpr int NG = ROW_BYTES / 32;
  int f;
  if constexpr (E == kEF32) f = ((krow >> 2) & 1) << 2;
  else if constexpr (E == kEBF16 || E == kEF16) f = ((krow & 3) << 1) ^ ((krow >> 1) & 1);
  else f = krow & 7;
  const int g = (byte_in_row >> 5) ^ (f & (NG - 1));
  return krow * ROW_BYTES + (g << 5) + (byte_in_row & 31);
}

__device__ __forceinline__ i32x4 lds_read_b128(const unsigned char* base, int off) {
  return *reinterpret_cast<const i32x4*>(base + off);
}

// int8 x8 (two dwords) -> bf16 x8 (exact: |v| <= 128 fits the 8-bit significand of bf16).
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
    out[2 * h] = (int)((u0 >> 16) | (u1 & 0xffff0000u));
    out[2 * h + 1] = (int)((u2 >> 16) | (u3 & 0xffff0000u));
  }
  return out;
}

// Fragment of one 32-wide atom at row/column base `rc0`, contraction atom `kk`.
//   ES = storage element kind in LDS, EC = compute (MFMA) kind.
template <int LAYOUT, int ES, int EC, int ROW_BYTES>
__device__ __forceinline__ typename Mma<EC>::Frag load_frag(const unsigned char* tile, int rc0, int kk, int lane) {
  typedef typename Mma<EC>::Frag Frag;
  constexpr int KA = Mma<EC>::KA;
  if constexpr (LAYOUT == kKC) {
    static_assert(ES == EC, "contraction-contiguous operands are stored in the compute type");
    const int row = rc0 + (lane & 31), q = lane >> 5;
    if constexpr (EC == kEF8) {
      const int c0 = kk * 4 + q * 2;
      i32x4 lo = lds_read_b128(tile, kc_offset<ROW_BYTES>(row, c0));
      i32x4 hi = lds_read_b128(tile, kc_offset<ROW_BYTES>(row, c0 + 1));
      Frag f;
      f[0] = lo[0]; f[1] = lo[1]; f[2] = lo[2]; f[3] = lo[3];
      f[4] = hi[0]; f[5] = hi[1]; f[6] = hi[2]; f[7] = hi[3];
      return f;
    } else {
      return lds_read_b128(tile, kc_offset<ROW_BYTES>(row, kk * 2 + q));
    }
  } else {
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
      } else {
        static_assert(EC == kEBF16 && ES == kEI8, "1-byte storage feeds fp8 or bf16(int8) MFMAs only");
        const int krow = kb + 8 * (blk >> 1) + (s >> 1);
        const i32x2 v = lds_read_tr8(tile + mc_offset<ROW_BYTES, ES>(krow, col));
        return i8x8_to_bf16x8(v);
      }
    }
  }
}

// ---- global -> register -> LDS staging ------------------------------------------------------
// One operand tile of a k-step, moved in 16-byte chunks; chunk q of the tile belongs to thread
// (q % THREADS). Out-of-range rows/columns are clamped to valid memory (their products are never
// stored); contraction indices at or past `k_hi` are zero-filled, which only the last k-step of
// a tile can need (a workgroup-uniform test keeps the other steps free of per-lane masking).
template <int LAYOUT, int ES, int RC /* rows or cols of C covered */, int BK, int THREADS>
struct TileStage {
  static constexpr int ESZ = elem_bytes(ES);
  static constexpr int ROW_BYTES = (LAYOUT == kKC) ? BK * ESZ : RC * ESZ;
  static constexpr int ROWS = (LAYOUT == kKC) ? RC : BK;
  static constexpr int CPR = ROW_BYTES / 16;
  static constexpr int CHUNKS = ROWS * CPR;
  static constexpr int PER = (CHUNKS + THREADS - 1) / THREADS;
  static constexpr int BYTES = ROWS * ROW_BYTES;
  static_assert(ROW_BYTES % 32 == 0 && (CPR & (CPR - 1)) == 0, "tile rows must be a power-of-two number of chunks");

  i32x4 regs[PER];

  // base: operand pointer already offset to the group; ld in elements; rc0 = first row/col of the
  // tile; rc_ext = extent of that axis; kc0 = first contraction index of this k-step;
  // k_hi = end of the valid contraction range.
  __device__ __forceinline__ void load(const unsigned char* base, int64_t ld, int rc0, int rc_ext, int kc0, int k_hi,
                                       int tid) {
    const bool full = kc0 + BK <= k_hi;  // uniform across the workgroup
    const i32x4 z = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int q = tid + i * THREADS;
      if (CHUNKS % THREADS != 0 && q >= CHUNKS) break;
      const int r = q / CPR, c = q % CPR;
      if constexpr (LAYOUT == kKC) {
        int row = rc0 + r;
        row = row < rc_ext ? row : rc_ext - 1;
        const int kcol = kc0 + c * (16 / ESZ);
        const unsigned char* p = base + ((int64_t)row * ld + kcol) * ESZ;
        if (full) {
          regs[i] = *reinterpret_cast<const i32x4*>(p);
        } else {
          regs[i] = z;
          if (kcol < k_hi) regs[i] = *reinterpret_cast<const i32x4*>(p);
        }
      } else {
        const int krow = kc0 + r;
        int colb = rc0 * ESZ + c * 16;
        const int lim = rc_ext * ESZ - 16;
        colb = colb < lim ? colb : lim;
        const unsigned char* p = base + (int64_t)krow * ld * ESZ + colb;
        if (full) {
          regs[i] = *reinterpret_cast<const i32x4*>(p);
        } else {
          regs[i] = z;
          if (krow < k_hi) regs[i] = *reinterpret_cast<const i32x4*>(p);
        }
      }
    }
  }

  __device__ __forceinline__ void store(unsigned char* tile, int tid) const {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int q = tid + i * THREADS;
      if (CHUNKS % THREADS != 0 && q >= CHUNKS) break;
      const int r = q / CPR, c = q % CPR;
      int off;
      if constexpr (LAYOUT == kKC) off = kc_offset<ROW_BYTES>(r, c);
      else off = mc_offset<ROW_BYTES, ES>(r, c * 16);
      *reinterpret_cast<i32x4*>(tile + off) = regs[i];
    }
  }
};

__device__ __forceinline__ float apply_activation(float x, int act) {
  switch (act) {
    case TKX_ACT_RELU: return x > 0.f ? x : 0.f;
    case TKX_ACT_TANH: return tanhf(x);
    case TKX_ACT_SILU: return x / (1.f + __expf(-x));
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

// ---- the kernel ---------------------------------------------------------------------------------
template <int MODE, int EA, int EB, int BM, int BN, int BK, int WM, int WN>
struct GemmKernel {
  static constexpr int THREADS = WM * WN * 64;
  static constexpr int LA = (MODE == kDrhs) ? kMC : kKC;
  static constexpr int LB = (MODE == kDlhs) ? kKC : kMC;
  static constexpr int EC = EA;  // MFMA type follows A; B may be stored narrower (int8 weights)
  static constexpr int KA = Mma<EC>::KA;
  static constexpr int WTM = BM / WM, WTN = BN / WN;
  static constexpr int TM = WTM / 32, TN = WTN / 32;
  static_assert(BM % (WM * 32) == 0 && BN % (WN * 32) == 0 && BK % KA == 0, "tile does not split into 32x32 atoms");
  typedef TileStage<LA, EA, BM, BK, THREADS> StageA;
  typedef TileStage<LB, EB, BN, BK, THREADS> StageB;
  static constexpr int STAGE_BYTES = StageA::BYTES + StageB::BYTES;
  static constexpr int SMEM_BYTES = 2 * STAGE_BYTES;

  static __device__ __forceinline__ void run(const GemmParams& p, unsigned char* smem) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int32_t* ws = p.ws;
    const int b = blockIdx.x;

    int group, row0, act_start, act_end, col0, kc_begin, kc_end;
    if constexpr (MODE != kDrhs) {
      const int num_tasks = ws[0];
      if (b >= p.real_slots) {
        // Tail duty: rows [total_rows, m_ext) belong to no group and are defined to be zero.
        const int total_rows = min(ws[1], p.m_ext);
        const int64_t esz = p.out_dtype == TKX_F32 ? 4 : 2;
        const int64_t lo = (int64_t)total_rows * p.ldc * esz, hi = (int64_t)p.m_ext * p.ldc * esz;
        unsigned char* c = reinterpret_cast<unsigned char*>(p.C);
        const int64_t nzb = gridDim.x - p.real_slots;
        const i32x4 z = {0, 0, 0, 0};
        for (int64_t o = lo + ((int64_t)(b - p.real_slots) * THREADS + tid) * 16; o < hi; o += nzb * THREADS * 16)
          *reinterpret_cast<i32x4*>(c + o) = z;
        return;
      }
      // XCD-aware order: consecutive workgroup ids land on different XCDs (id % 8), so give XCD x
      // the x-th contiguous eighth of the tile list; within it, `grid_tile_width` m-tasks share an
      // n-panel of B back to back, then move to the next n-panel.
      const int total = num_tasks * p.n_tiles;
      const int per_xcd = (total + 7) >> 3;
      const int idx = b >> 3, xcd = b & 7;
      if (idx >= per_xcd) return;
      const int L = xcd * per_xcd + idx;
      if (L >= total) return;
      const int W = p.grid_tile_width;
      const int span = W * p.n_tiles;
      const int sg = L / span, rem = L - sg * span;
      const int wcur = min(W, num_tasks - sg * W);
      const int nt = rem / wcur;
      const int mt = sg * W + (rem - nt * wcur);
      group = ws[p.ws_gid + mt];
      row0 = ws[p.ws_bstart + mt];
      act_start = ws[p.ws_astart + mt];
      act_end = ws[p.ws_aend + mt];
      col0 = nt * BN;
      kc_begin = 0;
      kc_end = p.k_ext;
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

    const int nk = (kc_end - kc_begin + BK - 1) / BK;
    StageA sa;
    StageB sb;
    if (nk > 0) {
      sa.load(Ab, p.lda, row0, p.m_ext, kc_begin, kc_end, tid);
      sb.load(Bb, p.ldb, col0, p.n_ext, kc_begin, kc_end, tid);
      sa.store(smem, tid);
      sb.store(smem + StageA::BYTES, tid);
    }
    __syncthreads();

    for (int kt = 0; kt < nk; ++kt) {
      const unsigned char* tA = smem + (kt & 1) * STAGE_BYTES;
      const unsigned char* tB = tA + StageA::BYTES;
      const bool more = kt + 1 < nk;
      if (more) {
        const int kc0 = kc_begin + (kt + 1) * BK;
        sa.load(Ab, p.lda, row0, p.m_ext, kc0, kc_end, tid);
        sb.load(Bb, p.ldb, col0, p.n_ext, kc0, kc_end, tid);
      }
#pragma unroll
      for (int kk = 0; kk < BK / KA; ++kk) {
        typename Mma<EC>::Frag fa[TM], fb[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i)
          fa[i] = load_frag<LA, EA, EC, StageA::ROW_BYTES>(tA, wm * WTM + i * 32, kk, lane);
#pragma unroll
        for (int j = 0; j < TN; ++j)
          fb[j] = load_frag<LB, EB, EC, StageB::ROW_BYTES>(tB, wn * WTN + j * 32, kk, lane);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) acc[i][j] = mma_atom<EC>(fb[j], fa[i], acc[i][j]);
      }
      if (more) {
        unsigned char* nA = smem + ((kt + 1) & 1) * STAGE_BYTES;
        sa.store(nA, tid);
        sb.store(nA + StageA::BYTES, tid);
      }
      __syncthreads();
    }

    // Epilogue. After the swapped MFMA, lane l of atom (i, j) holds C row (l % 32) and, for
    // t = 0..3, columns 8t + 4*(l / 32) + {0,1,2,3} of that atom.
    unsigned char* Cb = reinterpret_cast<unsigned char*>(p.C);
    if constexpr (MODE == kDrhs)
      Cb += (int64_t)group * p.c_group_stride * (p.out_dtype == TKX_F32 ? 4 : 2);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int row = row0 + wm * WTM + i * 32 + (lane & 31);
      const bool row_ok = row >= act_start && row < act_end;
      float rs = 1.f;
      if (p.a_scale != nullptr && row_ok) rs = p.a_scale[row];
#pragma unroll
      for (int j = 0; j < TN; ++j) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const int col = col0 + wn * WTN + j * 32 + 8 * t + 4 * (lane >> 5);
          if (!row_ok || col + 4 > p.n_ext) continue;
          f32x4 v;
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = acc[i][j][4 * t + e];
          if (p.a_scale != nullptr) {
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] *= rs;
          }
          if (p.b_scale != nullptr) {
            const f32x4 cs = *reinterpret_cast<const f32x4*>(p.b_scale + (int64_t)group * p.n_ext + col);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] *= cs[e];
          }
          if (p.activation != TKX_ACT_NONE) {
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = apply_activation(v[e], p.activation);
          }
          store4(Cb, (int64_t)row * p.ldc + col, v, p.out_dtype);
        }
      }
    }
  }
};

template <class K>
__global__ __launch_bounds__(K::THREADS) void gemm_entry(const GemmParams p) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char tkx_smem[];
  K::run(p, tkx_smem);
}

#define TKX_VARIANT(MODE, EA, EB, BM, BN, BK, WM, WN)                                           \
  {                                                                                             \
    MODE, EA, EB, BM, BN, BK, WM, WN, ::tkx::GemmKernel<MODE, EA, EB, BM, BN, BK, WM, WN>::SMEM_BYTES, \
        reinterpret_cast<const void*>(&::tkx::gemm_entry<::tkx::GemmKernel<MODE, EA, EB, BM, BN, BK, WM, WN>>) \
  }

}  // namespace tkx
