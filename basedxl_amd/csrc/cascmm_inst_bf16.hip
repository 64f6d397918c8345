// Instantiations: bf16 terms, fp32 operands in memory.
#include "cascmm_variants.h"

namespace cascmm {

#define F32 CASCMM_DT_F32
#define BF CASCMM_FMT_BF16

static const VariantDesc kTable[] = {
    // headline: two terms, three products.  name, BM, BN, BK, WM, WN, WK, DEPTH (4 producer waves)
    CASCMM_TILE_VARIANT("t64x160x64_w2x1x2_d2_bf16x2_tri", 64, 160, 64, 2, 1, 2, 2, F32, BF, 2, false, true),
    CASCMM_TILE_VARIANT("t256x128x32_w4x1x1_d2_bf16x2_tri", 256, 128, 32, 4, 1, 1, 2, F32, BF, 2, false, true),
    CASCMM_TILE_VARIANT("t128x128x32_w4x1x1_d3_bf16x2_tri", 128, 128, 32, 4, 1, 1, 3, F32, BF, 2, false, true),
    CASCMM_TILE_VARIANT("t128x128x64_w2x1x2_d2_bf16x2_tri", 128, 128, 64, 2, 1, 2, 2, F32, BF, 2, false, true),
    CASCMM_TILE_VARIANT("t64x128x64_w2x1x2_d3_bf16x2_tri", 64, 128, 64, 2, 1, 2, 3, F32, BF, 2, false, true),
    CASCMM_TILE_VARIANT("t64x64x64_w2x2x1_d3_bf16x2_tri", 64, 64, 64, 2, 2, 1, 3, F32, BF, 2, false, true),
    CASCMM_TILE_VARIANT_P("t64x160x64_w2x1x2_d2_p8_bf16x2_tri", 64, 160, 64, 2, 1, 2, 2, 8, F32, BF, 2, false, true),
    CASCMM_TILE_VARIANT_P("t128x128x64_w4x1x1_d2_p8_bf16x2_tri", 128, 128, 64, 4, 1, 1, 2, 8, F32, BF, 2, false, true),
    // (its permuted B columns are staged in 8 x 2 blocks: every producer thread gets the same units; 3 % faster here)
    CASCMM_TILE_VARIANT_PAIRS("t256x160x32_w4x1x1_d2_bf16x2_tri", 256, 160, 32, 4, 1, 1, 2, 4, F32, BF, 2, false, true),
    // four waves of 512 registers, 256 x 320 tile (needs the workspace for the left operand's slots)
    CASCMM_W512_VARIANT("t256x320x32_w512_bf16x2_tri", 0),
    // K split over the eight waves of a workgroup: one launch, no workspace
    CASCMM_WAVEK_VARIANT("t32x32x32_wavek_bf16x2_tri", 1),
    CASCMM_WAVEK_VARIANT("t32x64x32_wavek_bf16x2_tri", 2),
    CASCMM_SKINNY_VARIANT("skinny64x128x64_bf16x2_tri", 64, 4, 64, 2, 4, BF, 2, false),
    CASCMM_SKINNY_VARIANT("skinny32x128x64_bf16x2_tri", 32, 4, 64, 2, 4, BF, 2, false),
    CASCMM_BD_VARIANT("bd128x128x64_d3_p4_bf16x2_tri", 128, 4, 64, 3, 4, BF, 2, false),
    CASCMM_BD_VARIANT("bd96x128x64_d3_p4_bf16x2_tri", 96, 4, 64, 3, 4, BF, 2, false),
    CASCMM_BD_VARIANT("bd64x128x64_d3_p4_bf16x2_tri", 64, 4, 64, 3, 4, BF, 2, false),
    CASCMM_BD_VARIANT("bd192x128x64_d2_p4_bf16x2_tri", 192, 4, 64, 2, 4, BF, 2, false),
    CASCMM_BD_VARIANT("bd128x128x32_d3_p4_bf16x2_tri", 128, 4, 32, 3, 4, BF, 2, false),
    CASCMM_BD_VARIANT("bd128x128x64_d3_p2_bf16x2_tri", 128, 4, 64, 3, 2, BF, 2, false),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d1_bf16x2_tri_generic", 64, 64, 32, 2, 2, 1, 1, F32, BF, 2, false, false),
    // other term counts / product sets
    CASCMM_TILE_VARIANT("t128x128x32_w4x1x1_d3_bf16x1", 128, 128, 32, 4, 1, 1, 3, F32, BF, 1, false, true),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d1_bf16x1_generic", 64, 64, 32, 2, 2, 1, 1, F32, BF, 1, false, false),
    CASCMM_TILE_VARIANT("t128x128x32_w4x1x1_d3_bf16x2_full", 128, 128, 32, 4, 1, 1, 3, F32, BF, 2, true, true),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d1_bf16x2_full_generic", 64, 64, 32, 2, 2, 1, 1, F32, BF, 2, true, false),
    CASCMM_TILE_VARIANT("t128x128x32_w4x2x1_d2_bf16x3_tri", 128, 128, 32, 4, 2, 1, 2, F32, BF, 3, false, true),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d3_bf16x3_tri", 64, 64, 32, 2, 2, 1, 3, F32, BF, 3, false, true),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d1_bf16x3_tri_generic", 64, 64, 32, 2, 2, 1, 1, F32, BF, 3, false, false),
    CASCMM_TILE_VARIANT("t128x128x32_w4x2x1_d2_bf16x3_full", 128, 128, 32, 4, 2, 1, 2, F32, BF, 3, true, true),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d1_bf16x3_full_generic", 64, 64, 32, 2, 2, 1, 1, F32, BF, 3, true, false),
};

const VariantDesc* variants_bf16(int* n) {
  *n = (int)(sizeof(kTable) / sizeof(kTable[0]));
  return kTable;
}

}  // namespace cascmm
