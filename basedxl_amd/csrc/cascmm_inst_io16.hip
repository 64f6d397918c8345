// Instantiations: fp16 / bf16 operands in memory (the dtype the reference runs its UNet in).
// A 16-bit operand is exactly one fp16 (bf16) term, so fp16x1 (bf16x1) reproduces it without
// loss and the products are accumulated in fp32; the longer cascades are there for mixed
// use (bf16 terms of fp16 data and the reverse).  Bounds-checked element-wise loader only.
#include "cascmm_variants.h"

namespace cascmm {

#define H CASCMM_DT_F16
#define B CASCMM_DT_BF16
#define BF CASCMM_FMT_BF16
#define FP CASCMM_FMT_FP16

static const VariantDesc kTable[] = {
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d1_fp16x1_generic_ioh", 64, 64, 32, 2, 2, 1, 1, H, FP, 1, false, false),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d1_bf16x1_generic_ioh", 64, 64, 32, 2, 2, 1, 1, H, BF, 1, false, false),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d1_bf16x2_tri_generic_ioh", 64, 64, 32, 2, 2, 1, 1, H, BF, 2, false, false),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d1_fp16x2_tri_generic_ioh", 64, 64, 32, 2, 2, 1, 1, H, FP, 2, false, false),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d1_fp16x1_generic_iob", 64, 64, 32, 2, 2, 1, 1, B, FP, 1, false, false),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d1_bf16x1_generic_iob", 64, 64, 32, 2, 2, 1, 1, B, BF, 1, false, false),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d1_bf16x2_tri_generic_iob", 64, 64, 32, 2, 2, 1, 1, B, BF, 2, false, false),
    CASCMM_TILE_VARIANT("t64x64x32_w2x2x1_d1_fp16x2_tri_generic_iob", 64, 64, 32, 2, 2, 1, 1, B, FP, 2, false, false),
};

const VariantDesc* variants_io16(int* n) {
  *n = (int)(sizeof(kTable) / sizeof(kTable[0]));
  return kTable;
}

}  // namespace cascmm
