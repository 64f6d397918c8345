// Instantiations: right operand prepared (split once, stored as operand slots), fp32 left operand.
#include "cascmm_variants.h"

namespace cascmm {

#define BF CASCMM_FMT_BF16
#define FP CASCMM_FMT_FP16
#define F8 CASCMM_FMT_FP8

static const VariantDesc kTable[] = {
    // name, BM, BN, BK, WM, WN, WK, DEPTH, producer waves
    CASCMM_TILE_VARIANT_BPRE("t64x160x64_w2x1x2_d2_bf16x2_tri_bpre", 64, 160, 64, 2, 1, 2, 2, 4, BF, 2, false),
    CASCMM_TILE_VARIANT_BPRE("t64x160x64_w2x1x2_d3_bf16x2_tri_bpre", 64, 160, 64, 2, 1, 2, 3, 4, BF, 2, false),
    CASCMM_TILE_VARIANT_BPRE("t128x128x64_w2x2x1_d2_bf16x2_tri_bpre", 128, 128, 64, 2, 2, 1, 2, 4, BF, 2, false),
    CASCMM_TILE_VARIANT_BPRE("t128x160x32_w2x1x2_d3_bf16x2_tri_bpre", 128, 160, 32, 2, 1, 2, 3, 4, BF, 2, false),
    CASCMM_TILE_VARIANT_BPRE("t256x128x32_w4x1x1_d2_bf16x2_tri_bpre", 256, 128, 32, 4, 1, 1, 2, 4, BF, 2, false),
    CASCMM_TILE_VARIANT_BPRE("t64x64x64_w2x2x1_d3_bf16x2_tri_bpre", 64, 64, 64, 2, 2, 1, 3, 4, BF, 2, false),
    CASCMM_TILE_VARIANT_BPRE("t64x256x32_w1x4x1_d3_bf16x2_tri_bpre", 64, 256, 32, 1, 4, 1, 3, 4, BF, 2, false),
    CASCMM_TILE_VARIANT_BPRE("t256x160x32_w4x1x1_d2_bf16x2_tri_bpre", 256, 160, 32, 4, 1, 1, 2, 4, BF, 2, false),
    // the large-tile kernel fed with prepared slots of B (A still raw fp32, split at fragment-read time)
    CASCMM_W512_VARIANT("t256x320x32_w512_bf16x2_tri_bpre", 1),
    CASCMM_TILE_VARIANT_BPRE("t128x128x32_w4x2x1_d2_bf16x3_tri_bpre", 128, 128, 32, 4, 2, 1, 2, 4, BF, 3, false),
    CASCMM_TILE_VARIANT_BPRE("t128x128x32_w4x2x1_d2_fp16x3_tri_bpre", 128, 128, 32, 4, 2, 1, 2, 4, FP, 3, false),
    CASCMM_TILE_VARIANT_BPRE("t128x128x32_w4x2x1_d2_fp8x3_tri_bpre", 128, 128, 32, 4, 2, 1, 2, 4, F8, 3, false),
    // 16-bit tensors (what the reference runs its UNet in): a plain fp16 / bf16 GEMM with fp32 accumulation
    CASCMM_TILE_VARIANT_BPRE16("t256x128x64_w4x1x1_d2_fp16x1_bpre_ioh", 256, 128, 64, 4, 1, 1, 2, 4, CASCMM_DT_F16, FP),
    CASCMM_TILE_VARIANT_BPRE16("t128x128x64_w2x2x1_d3_fp16x1_bpre_ioh", 128, 128, 64, 2, 2, 1, 3, 4, CASCMM_DT_F16, FP),
    CASCMM_TILE_VARIANT_BPRE16("t64x160x64_w2x1x2_d3_fp16x1_bpre_ioh", 64, 160, 64, 2, 1, 2, 3, 4, CASCMM_DT_F16, FP),
    CASCMM_TILE_VARIANT_BPRE16("t64x64x64_w2x2x1_d3_fp16x1_bpre_ioh", 64, 64, 64, 2, 2, 1, 3, 4, CASCMM_DT_F16, FP),
    CASCMM_TILE_VARIANT_BPRE16("t256x128x64_w4x1x1_d2_bf16x1_bpre_iob", 256, 128, 64, 4, 1, 1, 2, 4, CASCMM_DT_BF16, BF),
    CASCMM_TILE_VARIANT_BPRE16("t128x128x64_w2x2x1_d3_bf16x1_bpre_iob", 128, 128, 64, 2, 2, 1, 3, 4, CASCMM_DT_BF16, BF),
    CASCMM_TILE_VARIANT_BPRE16("t64x160x64_w2x1x2_d3_bf16x1_bpre_iob", 64, 160, 64, 2, 1, 2, 3, 4, CASCMM_DT_BF16, BF),
    CASCMM_TILE_VARIANT_BPRE16("t64x64x64_w2x2x1_d3_bf16x1_bpre_iob", 64, 64, 64, 2, 2, 1, 3, 4, CASCMM_DT_BF16, BF),
};

const VariantDesc* variants_bpre(int* n) {
  *n = (int)(sizeof(kTable) / sizeof(kTable[0]));
  return kTable;
}

}  // namespace cascmm
