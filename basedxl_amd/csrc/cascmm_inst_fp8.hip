// Instantiations: fp8 (OCP e4m3) terms with a power-of-two tensor scale, fp32 operands in memory.
#include "cascmm_variants.h"

namespace cascmm {

#define F32 CASCMM_DT_F32
#define F8 CASCMM_FMT_FP8

static const VariantDesc kTable[] = {
    // the fp8-rate MFMA (32x32x64), operands split into the workspace first; right operand raw / prepared
    CASCMM_F8K64_VARIANT("t256x160x64_f8k64_fp8x3_tri", false, 2),
    CASCMM_F8K64_VARIANT("t256x160x64_f8k64_fp8x3_tri_bpre", true, 2),
    CASCMM_F8K64_VARIANT("t128x160x64_f8k64_fp8x3_tri", false, 1),
    CASCMM_F8K64_VARIANT("t128x160x64_f8k64_fp8x3_tri_bpre", true, 1),
    CASCMM_F8K64_VARIANT("k64x160x64_f8k64wk4_fp8x3_tri", false, 0),
    CASCMM_F8K64_VARIANT("k64x160x64_f8k64wk4_fp8x3_tri_bpre", true, 0),
    // three terms (12 significand bits), six products.  name, BM, BN, BK, WM, WN, WK, DEPTH
    CASCMM_TILE_VARIANT("t128x128x32_w4x2x1_d2_fp8x3_tri", 128, 128, 32, 4, 2, 1, 2, F32, F8, 3, false, true),
    CASCMM_TILE_VARIANT("t64x64x64_w2x2x1_d2_fp8x3_tri", 64, 64, 64, 2, 2, 1, 2, F32, F8, 3, false, true),
    CASCMM_TILE_VARIANT("t128x128x32_w2x2x1_d2_fp8x3_tri", 128, 128, 32, 2, 2, 1, 2, F32, F8, 3, false, true),
    CASCMM_TILE_VARIANT("t64x128x64_w2x2x2_d2_fp8x3_tri", 64, 128, 64, 2, 2, 2, 2, F32, F8, 3, false, true),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d1_fp8x3_tri_generic", 64, 64, 32, 2, 2, 1, 1, F32, F8, 3, false, false),
    CASCMM_TILE_VARIANT("t128x128x32_w4x2x1_d2_fp8x2_tri", 128, 128, 32, 4, 2, 1, 2, F32, F8, 2, false, true),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d1_fp8x2_tri_generic", 64, 64, 32, 2, 2, 1, 1, F32, F8, 2, false, false),
    CASCMM_TILE_VARIANT("t128x128x32_w4x2x1_d2_fp8x1", 128, 128, 32, 4, 2, 1, 2, F32, F8, 1, false, true),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d1_fp8x1_generic", 64, 64, 32, 2, 2, 1, 1, F32, F8, 1, false, false),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d1_fp8x3_full_generic", 64, 64, 32, 2, 2, 1, 1, F32, F8, 3, true, false),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d1_fp8x2_full_generic", 64, 64, 32, 2, 2, 1, 1, F32, F8, 2, true, false),
};

const VariantDesc* variants_fp8(int* n) {
  *n = (int)(sizeof(kTable) / sizeof(kTable[0]));
  return kTable;
}

}  // namespace cascmm
