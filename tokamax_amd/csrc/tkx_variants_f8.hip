// OCP fp8 (e4m3fn) x fp8 forward variants; per-row / per-(group, column) scales in the epilogue, or
// (kFwdSubK) scales per k-block on both operands folded in after every k-step.
#include "tkx_gemm.hip.h"

namespace tkx {
#define FWD(BM, BN, BK, WM, WN, NS) TKX_VARIANT(kFwd, kEF8, kEF8, BM, BN, BK, WM, WN, NS)

static const Variant kVariants[] = {
    FWD(256, 256, 128, 2, 4, 2),  // (lhs fragments kept once, GemmKernel::LEAN: 32-byte fragments next to 128 accumulators)
    FWD(128, 256, 128, 2, 4, 3),
    FWD(128, 128, 128, 2, 2, 4),
    FWD(64, 128, 128, 2, 2, 4),
    FWD(32, 128, 128, 1, 4, 4),
    TKX_VARIANT(kFwdSubK, kEF8, kEF8, 128, 256, 128, 2, 4, 3),
    TKX_VARIANT(kFwdSubK, kEF8, kEF8, 64, 256, 128, 2, 2, 3),
    TKX_VARIANT(kFwdSubK, kEF8, kEF8, 32, 256, 128, 1, 4, 3),
};

const Variant* variants_f8(int* count) {
  *count = (int)(sizeof(kVariants) / sizeof(kVariants[0]));
  return kVariants;
}
}  // namespace tkx
