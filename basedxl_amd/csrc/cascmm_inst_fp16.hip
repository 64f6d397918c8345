// Instantiations: fp16 terms (term i scaled by 2^(11 i)), fp32 operands in memory.
#include "cascmm_variants.h"

namespace cascmm {

#define F32 CASCMM_DT_F32
#define FP CASCMM_FMT_FP16

static const VariantDesc kTable[] = {
    CASCMM_TILE_VARIANT("t128x128x32_w4x2x1_d2_fp16x3_tri", 128, 128, 32, 4, 2, 1, 2, F32, FP, 3, false, true),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d3_fp16x3_tri", 64, 64, 32, 2, 2, 1, 3, F32, FP, 3, false, true),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d1_fp16x3_tri_generic", 64, 64, 32, 2, 2, 1, 1, F32, FP, 3, false, false),
    CASCMM_TILE_VARIANT("t128x128x32_w4x2x1_d2_fp16x2_tri", 128, 128, 32, 4, 2, 1, 2, F32, FP, 2, false, true),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d1_fp16x2_tri_generic", 64, 64, 32, 2, 2, 1, 1, F32, FP, 2, false, false),
    CASCMM_TILE_VARIANT("t128x128x32_w4x1x1_d3_fp16x1", 128, 128, 32, 4, 1, 1, 3, F32, FP, 1, false, true),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d1_fp16x1_generic", 64, 64, 32, 2, 2, 1, 1, F32, FP, 1, false, false),
    CASCMM_TILE_VARIANT("t128x128x32_w4x2x1_d2_fp16x2_full", 128, 128, 32, 4, 2, 1, 2, F32, FP, 2, true, true),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d1_fp16x2_full_generic", 64, 64, 32, 2, 2, 1, 1, F32, FP, 2, true, false),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d1_fp16x3_full_generic", 64, 64, 32, 2, 2, 1, 1, F32, FP, 3, true, false),
    // both operands split into pre-scaled operand slots first (cascmm_f16k_kernel.h)
    CASCMM_F16K_VARIANT("t256x160x32_f16k_fp16x3_tri", false),
    CASCMM_F16K_VARIANT("k64x160x32_f16wk4_fp16x3_tri", true),
};

const VariantDesc* variants_fp16(int* n) {
  *n = (int)(sizeof(kTable) / sizeof(kTable[0]));
  return kTable;
}

}  // namespace cascmm
