// bf16 activations x int8 weights forward variants (weights converted to bf16 on the way from LDS
// to the MFMA; per-(group, column) scales in the epilogue, or per-(group, k-block, column) scales
// multiplied in during that conversion: kFwdSubK, 256-column tiles).
// Variants with waves (1, 8) or (1, 4): one row of waves, every weight fragment converted once per workgroup
// (1.04-1.2 x over two rows; the 128 x 256 x 64 one with two stages shares a CU with a second workgroup).
#include "tkx_gemm.hip.h"

namespace tkx {
#define FWD(BM, BN, BK, WM, WN, NS) TKX_VARIANT(kFwd, kEBF16, kEI8, BM, BN, BK, WM, WN, NS)
// Gate-up fusion over int8 weights [gate | up] with one scale per (group, column).
#define GLU(BM, BN, BK, WM, WN, NS) TKX_VARIANT(kFwdGlu, kEBF16, kEI8, BM, BN, BK, WM, WN, NS)
#define SUBK(BM, BN, BK, WM, WN, NS) TKX_VARIANT(kFwdSubK, kEBF16, kEI8, BM, BN, BK, WM, WN, NS)
// The same with fp8 (e4m3fn) weights: bf16 activations x fp8 weights exist in this form only (one scale block
// covers the case of one scale per (group, column)).
#define SUBK_F8(BM, BN, BK, WM, WN, NS) TKX_VARIANT(kFwdSubK, kEBF16, kEF8, BM, BN, BK, WM, WN, NS)

static const Variant kVariants[] = {
    FWD(256, 256, 32, 2, 4, 4),
    FWD(256, 256, 64, 2, 4, 2),
    FWD(256, 256, 64, 2, 4, 3),
    FWD(256, 256, 64, 1, 8, 3),
    FWD(128, 256, 64, 2, 4, 3),
    FWD(128, 256, 64, 1, 8, 3),
    FWD(128, 256, 64, 1, 8, 2),
    FWD(128, 128, 64, 2, 2, 4),
    FWD(128, 128, 64, 1, 4, 4),
    FWD(64, 128, 64, 2, 2, 4),
    FWD(64, 128, 64, 1, 4, 4),
    FWD(32, 128, 64, 1, 4, 4),
    FWD(32, 256, 64, 1, 4, 4),
    FWD(32, 128, 128, 1, 4, 4),
    FWD(32, 128, 128, 1, 4, 2),
    GLU(256, 256, 64, 2, 4, 3),
    GLU(128, 256, 64, 2, 4, 3),
    GLU(128, 256, 64, 1, 4, 2),
    GLU(32, 256, 64, 1, 4, 4),
    SUBK(256, 256, 64, 2, 4, 3),
    SUBK(256, 256, 64, 1, 8, 3),
    SUBK(256, 256, 32, 2, 4, 4),
    SUBK(128, 256, 64, 2, 4, 3),
    SUBK(128, 256, 64, 1, 8, 3),
    SUBK(128, 256, 64, 1, 8, 2),
    SUBK(32, 256, 64, 1, 4, 4),
    // int8 activations x int8 weights on the int8 MFMAs: int32 sums of a k-step, folded into the f32 result with
    // the scales of its k-block (one block = one scale per row and per (group, column)).
    // (one scale per row and per (group, column): plain forward variants, the scales in the epilogue)
    TKX_VARIANT(kFwd, kEI8, kEI8, 256, 256, 128, 2, 4, 2),
    TKX_VARIANT(kFwd, kEI8, kEI8, 128, 256, 128, 2, 4, 3),
    TKX_VARIANT(kFwd, kEI8, kEI8, 64, 128, 128, 2, 2, 4),
    TKX_VARIANT(kFwd, kEI8, kEI8, 32, 128, 128, 1, 4, 4),
    TKX_VARIANT(kFwdSubK, kEI8, kEI8, 128, 256, 128, 2, 4, 3),
    TKX_VARIANT(kFwdSubK, kEI8, kEI8, 128, 256, 64, 2, 4, 3),
    TKX_VARIANT(kFwdSubK, kEI8, kEI8, 64, 256, 64, 2, 2, 4),
    TKX_VARIANT(kFwdSubK, kEI8, kEI8, 32, 256, 64, 1, 4, 3),
    SUBK_F8(256, 256, 64, 2, 4, 3),
    SUBK_F8(256, 256, 64, 1, 8, 3),
    SUBK_F8(256, 256, 32, 2, 4, 4),
    SUBK_F8(128, 256, 64, 2, 4, 3),
    SUBK_F8(128, 256, 64, 1, 8, 3),
    SUBK_F8(128, 256, 64, 1, 8, 2),
    SUBK_F8(32, 256, 64, 1, 4, 4),
};

const Variant* variants_i8w(int* count) {
  *count = (int)(sizeof(kVariants) / sizeof(kVariants[0]));
  return kVariants;
}
}  // namespace tkx
