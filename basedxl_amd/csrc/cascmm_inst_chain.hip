// Instantiations and launchers of the chained feed-forward path: the GEMM whose operands are both
// operand slots, and the pass that writes a left operand as slots (the gated store of the first GEMM
// writes the same layout directly; this pass is its stand-alone counterpart).
#include "cascmm_variants.h"
#include "cascmm_slotk_kernel.h"
#include "cascmm_slotn_kernel.h"

namespace cascmm {

// Thread (row, k group) reads its 8 values of A (two 16-byte pieces: positions 0..3 of the slot are
// k = 16 t + 4 g + 0..3, positions 4..7 the same + 8, for k group 2 t + g), splits them and writes the
// two terms' slots.  Four consecutive threads cover 32 consecutive k of one row (128 bytes read);
// a wave writes 256-byte runs of 16 consecutive rows.
__global__ __launch_bounds__(256) void prepare_left_kernel(const float* A, int M, int K, int64_t lda, u32x4* out) {
  const int kgroups = K >> 3;
  const int row_blocks = (M + 63) / 64;   // a one-dimensional grid: row blocks fastest (the other grid dimensions end at 65535)
  const int kg = (int)(blockIdx.x / row_blocks) * 4 + (threadIdx.x & 3);
  const int m = (int)(blockIdx.x % row_blocks) * 64 + (threadIdx.x >> 2);
  if (m >= M || kg >= kgroups) return;
  const float* src = A + (int64_t)m * lda + 16 * (kg >> 1) + 4 * (kg & 1);
  const f32x4 x0 = *(const f32x4*)src, x1 = *(const f32x4*)(src + 8);
  float r[8] = {x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
  u32x4 t[2];
  split8<CASCMM_FMT_BF16, 2>(r, t);
  out[(int64_t)kg * M + m] = t[0];
  out[((int64_t)kgroups + kg) * M + m] = t[1];
}

int launch_prepare_left(const float* A, int M, int K, int64_t lda, void* out, hipStream_t stream) {
  const int64_t blocks = (int64_t)((M + 63) / 64) * (((K >> 3) + 3) / 4);   // < 2^18: the caller keeps 4 M K below 2 GiB
  if (blocks <= 0 || blocks > 0x7FFFFFFF) return CASCMM_ERR_TOO_LARGE;
  return launch_kernel(prepare_left_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, A, M, K, lda, (u32x4*)out) == hipSuccess
             ? CASCMM_OK
             : CASCMM_ERR_LAUNCH;
}

const void* slotk_kernel_handle(int araw) { return araw ? (const void*)cascmm_slotk_kernel<1> : (const void*)cascmm_slotk_kernel<0>; }

template <int ARAW>
static int launch_slotk_t(const SlotKParams& q, hipStream_t stream) {
  typedef SlotK T;
  auto kfn = cascmm_slotk_kernel<ARAW>;
  static LdsFlags lds_set;
  if (!ensure_lds((const void*)kfn, T::LDS_BYTES, lds_set)) return CASCMM_ERR_LAUNCH;
  SlotKParams p = q;
  p.tiles_m = (q.M + T::BM - 1) / T::BM;
  p.tiles_n = (q.N + T::BN - 1) / T::BN;
  p.group_m = SlotK::GROUP_M;
  const int64_t grid = (int64_t)p.tiles_m * p.tiles_n;
  if (grid <= 0 || grid > 0x7FFFFFFF) return CASCMM_ERR_TOO_LARGE;
  return launch_kernel(kfn, dim3((unsigned)grid), dim3(T::NT), (size_t)T::LDS_BYTES, stream, p) == hipSuccess ? CASCMM_OK
                                                                                                              : CASCMM_ERR_LAUNCH;
}

int launch_slotk(const SlotKParams& q, int araw, hipStream_t stream) {
  return araw ? launch_slotk_t<1>(q, stream) : launch_slotk_t<0>(q, stream);
}

// the variant-table face of the kernel: raw fp32 left operand, prepared right operand
static int launch_slotk_variant(const GroupParams& p, hipStream_t stream) {
  if (p.kernel_out) { *p.kernel_out = (const void*)cascmm_slotk_kernel<1>; return CASCMM_OK; }
  if (p.count != 1 || p.glu || p.k_splits > 1) return CASCMM_ERR_BAD_VARIANT;
  if (p.K % (2 * SlotK::BK) != 0 || p.K < 2 * SlotK::BK) return CASCMM_ERR_BAD_VARIANT;   // raw A comes in pairs of stages
  if ((int64_t)p.M * p.lda * 4 > 0x7FFFFFFF || (int64_t)p.K * p.N * 4 > 0x7FFFFFFF || p.ldc * (int64_t)(SlotK::BM * 4) > 0x7FFFFFFF)
    return CASCMM_ERR_TOO_LARGE;
  SlotKParams q;
  memset(&q, 0, sizeof(q));
  q.a = p.A[0]; q.b_slots = p.B[0]; q.C = (float*)p.C[0]; q.bias = (const float*)p.bias[0];
  q.M = p.M; q.N = p.N; q.K = p.K; q.lda = p.lda; q.ldc = p.ldc;
  return launch_slotk_t<1>(q, stream);
}

// the 64 x 80 tile of the same design, for problems that make too few 64 x 160 tiles to occupy the chip
static int launch_slotn_variant(const GroupParams& p, hipStream_t stream) {
  typedef SlotN T;
  auto kfn = cascmm_slotn_kernel<0>;
  if (p.kernel_out) { *p.kernel_out = (const void*)kfn; return CASCMM_OK; }
  if (p.count != 1 || p.glu || p.k_splits > 1) return CASCMM_ERR_BAD_VARIANT;
  if (p.K % T::BK != 0 || p.K < T::BK) return CASCMM_ERR_BAD_VARIANT;
  if ((int64_t)p.M * p.lda * 4 > 0x7FFFFFFF || (int64_t)p.K * p.N * 4 > 0x7FFFFFFF || p.ldc * (int64_t)(T::BM * 4) > 0x7FFFFFFF)
    return CASCMM_ERR_TOO_LARGE;
  static LdsFlags lds_set;
  if (!ensure_lds((const void*)kfn, T::LDS_BYTES, lds_set)) return CASCMM_ERR_LAUNCH;
  SlotKParams q;
  memset(&q, 0, sizeof(q));
  q.a = p.A[0]; q.b_slots = p.B[0]; q.C = (float*)p.C[0]; q.bias = (const float*)p.bias[0];
  q.M = p.M; q.N = p.N; q.K = p.K; q.lda = p.lda; q.ldc = p.ldc;
  q.tiles_m = (p.M + T::BM - 1) / T::BM;
  q.tiles_n = (p.N + T::BN - 1) / T::BN;
  q.group_m = T::GROUP_M;
  const int64_t grid = (int64_t)q.tiles_m * q.tiles_n;
  if (grid <= 0 || grid > 0x7FFFFFFF) return CASCMM_ERR_TOO_LARGE;
  return launch_kernel(kfn, dim3((unsigned)grid), dim3(T::NT), (size_t)T::LDS_BYTES, stream, q) == hipSuccess ? CASCMM_OK
                                                                                                              : CASCMM_ERR_LAUNCH;
}

// both operands raw fp32
static int launch_rawk_variant(const GroupParams& p, hipStream_t stream) {
  typedef SlotK T;
  if (p.kernel_out) { *p.kernel_out = (const void*)cascmm_rawk_kernel; return CASCMM_OK; }
  if (p.count != 1 || p.glu || p.k_splits > 1) return CASCMM_ERR_BAD_VARIANT;
  if (p.K % (2 * T::BK) != 0 || p.K < 2 * T::BK || p.N % 4 != 0) return CASCMM_ERR_BAD_VARIANT;   // raw A comes in pairs of stages
  if ((int64_t)p.M * p.lda * 4 > 0x7FFFFFFF || (int64_t)p.K * p.ldb * 4 > 0x7FFFFFFF || p.ldc * (int64_t)(T::BM * 4) > 0x7FFFFFFF)
    return CASCMM_ERR_TOO_LARGE;
  auto kfn = cascmm_rawk_kernel;
  static LdsFlags lds_set;
  if (!ensure_lds((const void*)kfn, T::LDS_BYTES, lds_set)) return CASCMM_ERR_LAUNCH;
  SlotKParams q;
  memset(&q, 0, sizeof(q));
  q.a = p.A[0]; q.b_slots = p.B[0]; q.C = (float*)p.C[0]; q.bias = (const float*)p.bias[0];
  q.M = p.M; q.N = p.N; q.K = p.K; q.lda = p.lda; q.ldb = p.ldb; q.ldc = p.ldc;
  q.tiles_m = (p.M + T::BM - 1) / T::BM;
  q.tiles_n = (p.N + T::BN - 1) / T::BN;
  q.group_m = SlotK::GROUP_M;
  const int64_t grid = (int64_t)q.tiles_m * q.tiles_n;
  if (grid <= 0 || grid > 0x7FFFFFFF) return CASCMM_ERR_TOO_LARGE;
  const int c_vec = p.ldc % 4 == 0 && (uintptr_t)p.C[0] % 16 == 0;
  return launch_kernel(kfn, dim3((unsigned)grid), dim3(T::NT), (size_t)T::LDS_BYTES, stream, q, c_vec) == hipSuccess ? CASCMM_OK
                                                                                                                     : CASCMM_ERR_LAUNCH;
}

static const VariantDesc kChainTable[] = {
    {"k64x160x16_wk4_bf16x2_tri", KIND_SLOTK, CASCMM_DT_F32, CASCMM_FMT_BF16, 2, false, SlotK::BM, SlotK::BN, SlotK::BK, SlotK::NT,
     SlotK::LDS_BYTES, true, false, &launch_rawk_variant, false, false},
    {"k64x160x16_wk4_bf16x2_tri_bpre", KIND_SLOTK, CASCMM_DT_F32, CASCMM_FMT_BF16, 2, false, SlotK::BM, SlotK::BN, SlotK::BK, SlotK::NT,
     SlotK::LDS_BYTES, true, false, &launch_slotk_variant, true, false},
    {"k64x80x32_wk4_bf16x2_tri_bpre", KIND_SLOTK, CASCMM_DT_F32, CASCMM_FMT_BF16, 2, false, SlotN::BM, SlotN::BN, SlotN::BK, SlotN::NT,
     SlotN::LDS_BYTES, true, false, &launch_slotn_variant, true, false},
};

const VariantDesc* variants_chain(int* n) {
  *n = (int)(sizeof(kChainTable) / sizeof(kChainTable[0]));
  return kChainTable;
}

}  // namespace cascmm
