// bf16 (and, last in the list, fp8 and int8) activations x packed int4 weights (TKX_I4X2: two values to a byte along the contraction) forward variants.
// A weight stage is a byte tile half as deep as the k-step; the nibbles are taken apart and converted to bf16 on the
// way from LDS to the MFMA; per-(group, column) scales in the epilogue, or per-(group, k-block, column) scales
// multiplied in during that conversion (kFwdSubK, 256-column tiles). Whole k-steps only (k % block_k == 0).
// Variants with waves (1, 8) or (1, 4): one row of waves, every weight fragment converted once per workgroup; the
// 128 x 256 x 64 ones keep 72-75 KB of LDS and 128 registers, so two of their workgroups share a CU.
#include "tkx_gemm.hip.h"

namespace tkx {
#define FWD(BM, BN, BK, WM, WN, NS) TKX_VARIANT(kFwd, kEBF16, kEI4, BM, BN, BK, WM, WN, NS)
// Gate-up fusion over weights [gate | up] with one scale per (group, column).
#define GLU(BM, BN, BK, WM, WN, NS) TKX_VARIANT(kFwdGlu, kEBF16, kEI4, BM, BN, BK, WM, WN, NS)
#define SUBK(BM, BN, BK, WM, WN, NS) TKX_VARIANT(kFwdSubK, kEBF16, kEI4, BM, BN, BK, WM, WN, NS)
// fp8 activations: the nibbles go to the fp8 MFMAs as the e4m3 denormals (w + 8) / 512 and the epilogue takes the bias
// off with the activations' row sums (lhs_scale holds [row scales | row sums]). The 256 x 256 x 128 tile runs an atom's
// MFMAs column block by column block and keeps one set of converted rhs fragments (GemmKernel::JOUT).
#define F8FWD(BM, BN, BK, WM, WN, NS) TKX_VARIANT(kFwd, kEF8, kEI4, BM, BN, BK, WM, WN, NS)
#define F8GLU(BM, BN, BK, WM, WN, NS) TKX_VARIANT(kFwdGlu, kEF8, kEI4, BM, BN, BK, WM, WN, NS)
// Scales per k-block on both sides (and row sums per 128-deep k-step): every k-step's products are folded in with them.
#define F8SUBK(BM, BN, BK, WM, WN, NS) TKX_VARIANT(kFwdSubK, kEF8, kEI4, BM, BN, BK, WM, WN, NS)
// int8 activations: a nibble at the top of its byte is the int8 value 16 w; exact int32 sums on the int8 MFMAs, the
// factor 16 taken out where they become floats. One scale per row and per (group, column), or scales per k-block on
// both sides (the sums of a k-block are folded in at its end).
#define I8FWD(BM, BN, BK, WM, WN, NS) TKX_VARIANT(kFwd, kEI8, kEI4, BM, BN, BK, WM, WN, NS)
#define I8SUBK(BM, BN, BK, WM, WN, NS) TKX_VARIANT(kFwdSubK, kEI8, kEI4, BM, BN, BK, WM, WN, NS)
#define I8GLU(BM, BN, BK, WM, WN, NS) TKX_VARIANT(kFwdGlu, kEI8, kEI4, BM, BN, BK, WM, WN, NS)

static const Variant kVariants[] = {
    FWD(256, 256, 64, 2, 4, 2),
    FWD(256, 256, 64, 2, 4, 3),
    FWD(256, 256, 64, 2, 4, 4),
    FWD(256, 256, 64, 1, 8, 3),
    FWD(128, 256, 64, 2, 4, 3),
    FWD(128, 256, 64, 1, 8, 3),
    FWD(128, 128, 64, 2, 2, 4),
    FWD(128, 128, 64, 1, 4, 4),
    FWD(64, 128, 64, 2, 2, 4),
    FWD(64, 128, 64, 1, 4, 4),
    FWD(32, 128, 64, 1, 4, 4),
    GLU(256, 256, 64, 2, 4, 3),
    GLU(128, 256, 64, 2, 4, 3),
    GLU(128, 256, 64, 1, 4, 3),
    GLU(32, 256, 64, 1, 4, 4),
    SUBK(256, 256, 64, 2, 4, 3),
    SUBK(256, 256, 64, 1, 8, 3),
    SUBK(128, 256, 64, 2, 4, 3),
    SUBK(128, 256, 64, 1, 8, 3),
    SUBK(32, 256, 64, 1, 4, 4),
    F8FWD(256, 256, 128, 2, 4, 3),
    F8GLU(256, 256, 128, 2, 4, 3),
    F8GLU(128, 256, 128, 2, 4, 3),
    F8GLU(128, 256, 128, 1, 4, 2),
    F8GLU(64, 256, 128, 2, 4, 3),
    F8GLU(32, 256, 128, 1, 4, 4),
    F8SUBK(128, 256, 128, 2, 4, 3),
    F8SUBK(128, 256, 128, 1, 8, 3),
    F8SUBK(64, 256, 128, 2, 2, 3),
    F8SUBK(32, 256, 128, 1, 4, 3),
    I8FWD(256, 256, 128, 2, 4, 3),
    I8FWD(128, 256, 128, 2, 4, 3),
    I8FWD(128, 256, 128, 1, 8, 3),
    I8FWD(128, 256, 128, 1, 8, 2),
    I8FWD(128, 256, 128, 1, 4, 2),
    I8FWD(64, 128, 128, 2, 2, 4),
    I8FWD(32, 128, 128, 1, 4, 4),
    I8GLU(256, 256, 128, 2, 4, 3),
    I8GLU(128, 256, 128, 2, 4, 3),
    I8GLU(128, 256, 128, 1, 4, 2),
    I8GLU(64, 256, 128, 2, 4, 3),
    I8GLU(32, 256, 128, 1, 4, 4),
    I8SUBK(128, 256, 128, 2, 4, 3),
    I8SUBK(128, 256, 128, 1, 8, 3),
    I8SUBK(128, 256, 64, 2, 4, 4),
    I8SUBK(64, 256, 128, 2, 2, 3),
    I8SUBK(32, 256, 128, 1, 4, 3),
    F8FWD(128, 256, 128, 2, 4, 3),
    F8FWD(128, 256, 128, 1, 8, 3),
    F8FWD(128, 256, 128, 1, 8, 4),
    F8FWD(128, 256, 128, 1, 4, 2),
    F8FWD(128, 128, 128, 2, 2, 4),
    F8FWD(64, 128, 128, 2, 2, 4),
    F8FWD(32, 128, 128, 1, 4, 4),
};

const Variant* variants_i4w(int* count) {
  *count = (int)(sizeof(kVariants) / sizeof(kVariants[0]));
  return kVariants;
}
}  // namespace tkx
