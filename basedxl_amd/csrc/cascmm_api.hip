// extern "C" entry points: argument checks, kernel selection, small utility kernels.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <dlfcn.h>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "cascmm_variants.h"

namespace cascmm {

// ---------------------------------------------------------------------------------------
// variant table (immutable after first use)
// ---------------------------------------------------------------------------------------
static const std::vector<VariantDesc>& table() {
  static const std::vector<VariantDesc> t = [] {
    std::vector<VariantDesc> v;
    int n = 0;
    const VariantDesc* p = variants_bf16(&n);
    v.insert(v.end(), p, p + n);
    p = variants_fp16(&n);
    v.insert(v.end(), p, p + n);
    p = variants_fp8(&n);
    v.insert(v.end(), p, p + n);
    p = variants_io16(&n);
    v.insert(v.end(), p, p + n);
    p = variants_bpre(&n);
    v.insert(v.end(), p, p + n);
    p = variants_chain(&n);
    v.insert(v.end(), p, p + n);
    return v;
  }();
  return t;
}

struct TunedCost;
// per variant, resolved once when the table is built: its measured cost constants (or none) and what
// kind of kernel its name says it is
struct VariantInfo { const TunedCost* tuned; bool p8; bool bdirect; };
static const std::vector<VariantInfo>& variant_info();

static bool aligned_to(const void* p, size_t a) { return ((uintptr_t)p % a) == 0; }
static size_t dtype_size(int dt) { return dt == CASCMM_DT_F32 ? 4 : 2; }

struct Problem {
  int64_t M, N, K, lda, ldb, ldc;
  int dtype, fmt, terms, products;
  bool bpre = false;  // B is a prepared (already split) weight buffer
  bool glu = false;   // gated epilogue: B prepared by cascmm_prepare_weight_glu, C has N / 2 columns
  bool glu_slots = false;   // ... written as the left operand slots of the next GEMM (large-tile kernel only)
};

// Three fp8 terms with K a multiple of 64 are prepared for the fp8-rate kernel: [term][K/16][N] slots
// of 16 k each (the gated layout keeps the older form, whose kernels have the gated store)
static bool prepared_as_k16_slots(int64_t K, int fmt, int terms, bool glu) {
  return fmt == CASCMM_FMT_FP8 && terms == 3 && K > 0 && K % F8K64::BK == 0 && !glu;
}

// bytes of a prepared weight: planes x ceil(K/8) x N operand slots of 16 bytes
static int64_t prepared_bytes(int64_t K, int64_t N, int fmt, int terms, bool glu = false) {
  if (prepared_as_k16_slots(K, fmt, terms, glu)) return f8k64_slot_bytes(N, K);
  const int planes = fmt == CASCMM_FMT_FP8 ? (terms + 1) / 2 : terms;
  int64_t slots = 0, bytes = 0;   // (saturates instead of overflowing: callers compare the result with limits)
  if (__builtin_mul_overflow((int64_t)planes * ((K + 7) / 8), N, &slots) || __builtin_mul_overflow(slots, (int64_t)16, &bytes))
    return INT64_MAX;
  return bytes;
}

static int check_problem(const Problem& q) {
  if (q.dtype != CASCMM_DT_F32 && q.dtype != CASCMM_DT_F16 && q.dtype != CASCMM_DT_BF16) return CASCMM_ERR_BAD_DTYPE;
  if (q.fmt != CASCMM_FMT_BF16 && q.fmt != CASCMM_FMT_FP16 && q.fmt != CASCMM_FMT_FP8) return CASCMM_ERR_BAD_FORMAT;
  if (q.terms < 1 || q.terms > 3) return CASCMM_ERR_BAD_FORMAT;
  if (q.products != CASCMM_PROD_TRI && q.products != CASCMM_PROD_FULL) return CASCMM_ERR_BAD_FORMAT;
  if (q.M < 0 || q.N < 0 || q.K < 0) return CASCMM_ERR_BAD_SHAPE;
  if (q.M > INT32_MAX || q.N > INT32_MAX || q.K > INT32_MAX) return CASCMM_ERR_TOO_LARGE;
  if (q.lda < q.K || q.ldb < q.N || q.ldc < (q.glu ? q.N / 2 : q.N)) return CASCMM_ERR_BAD_SHAPE;
  return CASCMM_OK;
}

// what the fast (buffer-load, 16-byte accesses, no K tail) kernels need apart from K % BK == 0
static bool fast_ok(const Problem& q, const void* A, const void* B) {
  if (q.dtype != CASCMM_DT_F32) {
    // 16-bit operands: only with a prepared right operand, as one term of their own format
    return q.bpre && q.terms == 1 &&
           ((q.dtype == CASCMM_DT_F16 && q.fmt == CASCMM_FMT_FP16) || (q.dtype == CASCMM_DT_BF16 && q.fmt == CASCMM_FMT_BF16)) &&
           q.lda % 8 == 0 && (A == nullptr || aligned_to(A, 16)) && q.lda * 2 * 512 < INT32_MAX;
  }
  return q.dtype == CASCMM_DT_F32 && q.lda % 4 == 0 && (A == nullptr || aligned_to(A, 16)) &&
         q.ldb % 4 == 0 && q.N % 4 == 0 && (B == nullptr || aligned_to(B, 16)) &&
         q.lda * 4 * 512 < INT32_MAX && q.ldb * 4 * 136 < INT32_MAX &&  // 32-bit byte offsets inside a tile
         (q.bpre || q.K * q.ldb * 4 < INT32_MAX);  // ... and down a column block of B (buffer offsets are 32-bit)
}

static bool variant_matches(const VariantDesc& v, const Problem& q, bool fast) {
  const int full = (q.products == CASCMM_PROD_FULL && q.terms > 1) ? 1 : 0;
  if (v.iodt != q.dtype || v.fmt != q.fmt || v.terms != q.terms || v.full != full || v.bpre != q.bpre) return false;
  if (v.fast && (!fast || q.K % v.BK != 0)) return false;
  if (v.kind == KIND_SPLITK && (q.M > 5 * v.BM || q.K < 4 * v.BK)) return false;  // skinny: few row tiles, deep K
  if (v.kind == KIND_F8K64 && (q.products != CASCMM_PROD_TRI || q.K % v.BK != 0 || q.K == 0 || q.glu ||
                               f8k64_slot_bytes(q.M, q.K) > INT32_MAX || f8k64_slot_bytes(q.N, q.K) > INT32_MAX))
    return false;
  if (v.kind == KIND_F16K && (q.products != CASCMM_PROD_TRI || q.K % v.BK != 0 || q.K == 0 || q.glu || q.bpre ||
                              (v.BM == F16K::BM && q.K > F16K::MAX_K) || q.K * q.ldb * 4 > INT32_MAX ||
                              f16k_slot_bytes(q.M, q.K) > INT32_MAX || f16k_slot_bytes(q.N, q.K) > INT32_MAX))
    return false;
  if (v.bpre && v.kind != KIND_F8K64 && prepared_as_k16_slots(q.K, q.fmt, q.terms, q.glu)) return false;   // other layout
  if (v.kind == KIND_W512 && (q.M % v.BM != 0 || q.N % v.BN != 0 || q.M * q.lda * 4 > INT32_MAX ||
                              (!q.bpre && q.K * q.ldb * 4 > INT32_MAX) || q.ldc * (int64_t)(v.BM * 4) > INT32_MAX))
    return false;
  if (v.kind == KIND_WAVEK && (q.N % v.BN != 0 || q.M * q.lda * 4 > INT32_MAX || q.K == 0)) return false;
  if (v.kind == KIND_SLOTK && (q.K % 32 != 0 || q.K < 32 || q.glu || q.M * q.lda * 4 > INT32_MAX || q.ldc * (int64_t)(v.BM * 4) > INT32_MAX))
    return false;
  if (q.glu && !v.glu) return false;
  if (q.glu_slots && v.kind != KIND_W512) return false;
  return true;
}

// Cost model.  The two-term bf16 and three-term fp8 kernels, which carry the SDXL workload, are costed from
// constants measured on MI355X (sweep over the UNet's Linear shapes, HIP-graph replay): a launch
// takes  rounds x (K/64 x step64 + fixed)  microseconds, where a partly filled last round counts
// as  tail + (1 - tail) x fill  of a full one, with one `tail` for a launch that has no full
// round (its tiles run faster: less contention for the caches) and one for later rounds.  Other kernels use the analytic form the constants were first fitted with: a
// 64-deep K step of a full round costs about (BM*BN + 64*(BM+BN)) / 20000 microseconds (MFMA
// work grows with BM*BN; loading, splitting and staging grow with BM+BN and weigh about as much
// at these tile sizes).
struct TunedCost { const char* name; double step64_us, fixed_us, tail_first, tail_later; };
static const TunedCost kTuned[] = {
    {"t64x160x64_w2x1x2_d2_bf16x2_tri", 1.228, 4.34, 1.00, 0.80},
    {"t256x128x32_w4x1x1_d2_bf16x2_tri", 2.294, 7.99, 0.80, 0.80},
    {"t128x128x32_w4x1x1_d3_bf16x2_tri", 1.464, 5.83, 0.90, 0.80},
    {"t128x128x64_w2x1x2_d2_bf16x2_tri", 1.189, 8.10, 0.90, 0.80},
    {"t64x128x64_w2x1x2_d3_bf16x2_tri", 0.922, 4.17, 1.00, 0.90},
    {"t64x64x64_w2x2x1_d3_bf16x2_tri", 0.671, 2.34, 1.00, 1.00},
    {"t64x160x64_w2x1x2_d2_p8_bf16x2_tri", 1.064, 4.69, 0.90, 0.80},
    {"t128x128x64_w4x1x1_d2_p8_bf16x2_tri", 1.224, 6.84, 0.80, 0.70},
    {"t256x160x32_w4x1x1_d2_bf16x2_tri", 3.250, 5.00, 0.70, 0.50},
    {"t256x320x32_w512_bf16x2_tri", 5.65, 16.0, 1.00, 1.00},
    // three fp16 / bf16 terms
    {"t128x128x32_w4x2x1_d2_fp16x3_tri", 3.107, 7.22, 0.90, 0.80},
    {"t64x64x32_w2x2x1_d3_fp16x3_tri", 1.088, 2.27, 1.00, 1.00},
    {"t128x128x32_w4x2x1_d2_bf16x3_tri", 2.596, 7.02, 0.80, 0.70},
    {"t64x64x32_w2x2x1_d3_bf16x3_tri", 0.910, 2.20, 1.00, 1.00},
    // three fp8 terms (static tensor scales)
    {"t128x128x32_w4x2x1_d2_fp8x3_tri", 2.547, 6.33, 1.00, 0.90},
    {"t64x64x64_w2x2x1_d2_fp8x3_tri", 1.016, 2.50, 1.00, 1.00},
    {"t128x128x32_w2x2x1_d2_fp8x3_tri", 2.211, 6.93, 0.90, 0.80},
    {"t64x128x64_w2x2x2_d2_fp8x3_tri", 1.409, 4.91, 1.00, 0.90},
    // right operand prepared (sweep over M in 1024..8192 of the UNet's (K, N) pairs)
    {"t64x160x64_w2x1x2_d2_bf16x2_tri_bpre", 0.925, 5.57, 0.80, 0.60},
    {"t64x160x64_w2x1x2_d3_bf16x2_tri_bpre", 0.891, 6.26, 0.90, 0.80},
    {"t128x128x64_w2x2x1_d2_bf16x2_tri_bpre", 1.193, 6.27, 0.90, 0.80},
    {"t128x160x32_w2x1x2_d3_bf16x2_tri_bpre", 1.501, 9.45, 0.70, 0.50},
    {"t256x128x32_w4x1x1_d2_bf16x2_tri_bpre", 2.192, 9.64, 0.70, 0.70},
    {"t64x64x64_w2x2x1_d3_bf16x2_tri_bpre", 0.515, 2.08, 1.00, 1.00},
    {"t64x256x32_w1x4x1_d3_bf16x2_tri_bpre", 1.250, 5.89, 0.80, 0.50},
    {"t256x160x32_w4x1x1_d2_bf16x2_tri_bpre", 2.837, 12.00, 0.60, 0.50},
    {"t256x320x32_w512_bf16x2_tri_bpre", 5.50, 16.0, 1.00, 1.00},
    // K split over the waves: a round of 256 tiles costs 0.011 us per k + 8 us, and rounds do not overlap
    // (2048 x {1280, 5120} x 1280: 21.7 / 64.3 us; 1024 x 1280 x 1280: 17.4 us -- 7 % less than with raw A fetched
    // in half lines, A/B on one box)
    {"k64x160x16_wk4_bf16x2_tri_bpre", 0.71, 8.0, 0.65, 0.95},
    {"k64x80x32_wk4_bf16x2_tri_bpre", 0.445, 5.4, 0.69, 0.95},
    // ... both operands raw (2048 x {1280, 5120} x 1280: 24.0 / 77.2 us; 8192 x 2560 x 640, two rounds: 79.3 us)
    {"k64x160x16_wk4_bf16x2_tri", 0.887, 6.3, 0.65, 0.95},
};

constexpr int kMaxTileSplits = 4;
// the fp8-rate kernel with K over the waves: us per 64-k stage of a wave, and per round of tiles
constexpr double kF8WKStageUs = 2.25, kF8WKFixedUs = 6.0;   // (fit: 2048 x {1280, 5120} x 1280, 4096 x {640, 2560} x 640)

static const std::vector<VariantInfo>& variant_info() {
  static const std::vector<VariantInfo> info = [] {
    std::vector<VariantInfo> v;
    for (const VariantDesc& d : table()) {
      VariantInfo i{nullptr, strstr(d.name, "_p8_") != nullptr, d.name[0] == 'b' && d.name[1] == 'd'};
      for (const TunedCost& t : kTuned)
        if (strcmp(t.name, d.name) == 0) i.tuned = &t;
      v.push_back(i);
    }
    return v;
  }();
  return info;
}

// The kernel that splits K over the waves of a workgroup (KIND_WAVEK) moves (32 + BN) x K x 4 bytes
// into every workgroup and is bound by that: a CU pulled in 85 bytes per ns with the 32-wide and
// 60 with the 64-wide tile, all CUs together 17 KB per ns (154 x 2048 x {640, 1280, 2560}); a launch
// costs 2.5 us, prologue and the meeting of the partial tiles 0.6 us per round of workgroups.
static bool wavek_eligible(const Problem& q) {
  return q.dtype == CASCMM_DT_F32 && q.fmt == CASCMM_FMT_BF16 && q.terms == 2 && q.products == CASCMM_PROD_TRI && !q.bpre &&
         !q.glu && q.K > 0 && q.K % 32 == 0 && q.N % 32 == 0 && q.M * q.lda * 4 <= INT32_MAX;
}
static double wavek_estimate_us(const Problem& q, int count, int bn) {
  if (q.N % bn != 0) return 1e9;
  const double items = (double)count * (double)((q.M + 31) / 32) * (double)(q.N / bn);
  const double active = items < kNumCUs ? items : kNumCUs;
  const double per_cu = bn == 32 ? 85.0e3 : 60.0e3;                       // bytes per us
  const double rate = per_cu < 17.0e6 / active ? per_cu : 17.0e6 / active;
  const double rounds = (double)(int64_t)((items + kNumCUs - 1) / kNumCUs);
  return 2.5 + rounds * (0.6 + (double)(32 + bn) * (double)q.K * 4.0 / rate);
}
static double wavek_estimate_us(const Problem& q, int count) {
  const double a = wavek_estimate_us(q, count, 32), b = wavek_estimate_us(q, count, 64);
  return a < b ? a : b;
}
// The skinny split-K path for comparison (its 32-row variant, the one preferred among them): two
// launches, a workgroup's (32 + 128) x K / splits x 4 bytes at 70 bytes per ns, the partial results
// written and read back at about 4 TB/s (fitted on the same shapes).
static double skinny_estimate_us(const Problem& q) {
  const int sp = skinny_splits(q.M, q.N, q.K, 32, 128, 64);
  return 8.5 + 160.0 * (double)(q.K / sp) * 4.0 / 70.0e3 + 2.0 * sp * (double)q.M * (double)q.N * 4.0 / 4.0e6;
}

// ws_bytes: workspace the caller brought; *splits_out: K split the cost was computed for (the
// LDS-tiled two-term bf16 kernels may split K over up to kMaxTileSplits work items per tile when a
// single problem has too few tiles to occupy the chip and the workspace holds the partials)
static double variant_cost(int vi, const Problem& q, int count, size_t ws_bytes = 0,
                           int* splits_out = nullptr) {
  const VariantDesc& v = table()[vi];
  const VariantInfo& info = variant_info()[vi];
  if (splits_out) *splits_out = 1;
  const double tiles = (double)count * (double)((q.M + v.BM - 1) / v.BM) * (double)((q.N + v.BN - 1) / v.BN);
  const double full = (double)(int64_t)(tiles / kNumCUs);
  const double rem = tiles - full * kNumCUs;
  if (v.kind == KIND_SPLITK) {
    // Problems with too few tiles to occupy the chip: splitting K wins whenever the plain tile
    // kernels would leave more than half of the CUs idle; among the split-K variants the
    // smaller row tile was faster wherever both were measured.
    if ((double)((q.M + 63) / 64) * (double)((q.N + 127) / 128) >= kNumCUs / 2) return 1e9;
    // ... unless the one-launch kernel that splits K over its waves is expected to be faster
    if (wavek_eligible(q) && wavek_estimate_us(q, count) < skinny_estimate_us(q)) return 1e9;
    return 1e-6 * (double)(((q.M + v.BM - 1) / v.BM) * v.BM) + 1e-8 * v.BM;
  }
  if (v.kind == KIND_WAVEK) return wavek_estimate_us(q, count, v.BN);
  if (v.kind == KIND_F8K64) {
    // stages of 64 k at ~2.1 us per resident round, the K split the launcher will use, and the passes
    // around the GEMM: the split of A (and of B unless prepared), the reduction of a K split
    const int sp = f8k64_splits(q.M, q.N, q.K, v.BM);
    const double items = tiles * sp;
    const double rounds_ = items <= kNumCUs ? 1.0 : (double)(int64_t)(items / kNumCUs) + ((int64_t)items % kNumCUs ? 0.8 : 0.0);
    // (the 64-row tile splits K over the four waves of its workgroup: a quarter of the stages per wave, in pairs,
    // and rounds of one tile per CU that do not overlap)
    const double gemm_us = v.BM == F8WK::BM ? rounds_ * ((double)((q.K / 64 + 7) / 8 * 2) * kF8WKStageUs + kF8WKFixedUs)
                                            : rounds_ * ((double)(q.K / 64 / sp) * f8k64_stage_us(v.BM) + (v.BM == 256 ? 6.0 : 4.0));
    double us = gemm_us + 6.0 + (double)q.M * q.K * 7.0 / 4.0e6;
    if (!q.bpre) us += 3.0 + (double)q.K * q.N * 7.0 / 4.0e6;
    if (sp > 1) us += 3.0 + (double)(sp + 1) * q.M * q.N * 4.0 / 4.0e6;
    return us;
  }
  if (v.kind == KIND_F16K) {
    // Stages of 32 k (the K-over-waves kernel: a wave's own stages, in pairs) at the measured 3.0 / 2.45 us with 10 / 8 us
    // per round beside them (fit: 2048 x {1280, 5120} x 1280, 2048 x 1280 x {3840, 10240}, 8192 x 640 x 5120), and the
    // two passes around the GEMM: both operands read twice and written once as slots, 14 bytes per element at 5.7 TB/s.
    const double rounds_ = tiles <= kNumCUs ? 1.0 : (double)(int64_t)(tiles / kNumCUs) + ((int64_t)tiles % kNumCUs ? 0.8 : 0.0);
    const double gemm_us = v.BM == F16WK::BM ? rounds_ * ((double)((q.K / 32 + 7) / 8 * 2) * 3.0 + 10.0)
                                             : rounds_ * ((double)(q.K / 32) * 2.45 + 8.0);
    return gemm_us + 4.0 + ((double)q.M * q.K + (double)q.K * q.N) * 14.0 / 5.7e6;
  }
  if (info.tuned) {
    const TunedCost& t = *info.tuned;
    const double tail = full == 0 ? t.tail_first : t.tail_later;
    const double rounds = full + (rem > 0 ? tail + (1.0 - tail) * rem / kNumCUs : 0.0);
    // tiles that hang over the edge of C take the bounds-checked epilogue and load clamped
    // columns: measured about a quarter slower (32768 x 640 x 320 on the 128-wide tile)
    const double edge = (q.N % v.BN != 0 || q.M % v.BM != 0) ? 1.25 : 1.0;
    // (the kernels that split K over their waves run whole trips of four stages per wave: K in steps of 256)
    const double k_run = v.kind == KIND_SLOTK ? (double)((q.K + 255) / 256 * 256) : (double)q.K;
    double best = edge * rounds * (k_run / 64.0 * t.step64_us + t.fixed_us);
    if (v.kind == KIND_TILE && count == 1 && q.dtype == CASCMM_DT_F32 && q.N % 4 == 0 && full == 0 && !q.glu) {
      const int64_t ksteps = (q.K + v.BK - 1) / v.BK;
      for (int sp = 2; sp <= kMaxTileSplits; ++sp) {
        if (ksteps % sp != 0 || ksteps / sp < 4 || tiles * sp > kNumCUs) continue;
        if (ws_bytes < (size_t)sp * q.M * q.N * sizeof(float)) continue;
        const double r = t.tail_first + (1.0 - t.tail_first) * tiles * sp / kNumCUs;
        // the second pass: a launch plus writing and reading the partial results at about 4 TB/s
        const double reduce_us = 2.0 + (double)(sp + 1) * q.M * q.N * 4.0 / 4.0e6;
        const double c = edge * r * ((double)q.K / sp / 64.0 * t.step64_us + t.fixed_us) + reduce_us;
        if (c < best) {
          best = c;
          if (splits_out) *splits_out = sp;
        }
      }
    }
    return best;
  }
  const double rounds = full + (rem > 0 ? 0.55 + 0.45 * rem / kNumCUs : 0.0);
  double step = ((double)v.BM * v.BN + 64.0 * (v.BM + v.BN)) / 20000.0;
  if (info.p8) step *= 0.94;
  const double ksteps = (double)((q.K + 63) / 64);
  // the plain B-direct kernels were slower than the LDS-tiled ones on every shape measured:
  // they stay selectable by index only
  if (info.bdirect) return 1e6 + rounds * step * ksteps;
  double best = rounds * (step * ksteps + 5.0) + (v.fast ? 0.0 : 1e3);
  // the same K split as above for the kernels without measured constants (three-term and fp8
  // cascades on the shapes that leave CUs idle)
  if (v.fast && count == 1 && q.dtype == CASCMM_DT_F32 && q.N % 4 == 0 && full == 0 && !q.glu && !q.bpre) {
    const int64_t bk_steps = (q.K + v.BK - 1) / v.BK;
    for (int sp = 2; sp <= kMaxTileSplits; ++sp) {
      if (bk_steps % sp != 0 || bk_steps / sp < 4 || tiles * sp > kNumCUs) continue;
      if (ws_bytes < (size_t)sp * q.M * q.N * sizeof(float)) continue;
      const double r = 0.55 + 0.45 * tiles * sp / kNumCUs;
      const double reduce_us = 2.0 + (double)(sp + 1) * q.M * q.N * 4.0 / 4.0e6;
      const double c = r * (step * ksteps / sp + 5.0) + reduce_us;
      if (c < best) {
        best = c;
        if (splits_out) *splits_out = sp;
      }
    }
  }
  return best;
}

// ws_bytes: workspace the caller brought (split-K variants that need more are skipped)
// The selection walks the whole table and costs every candidate; a model calls the same few dozen
// problems over and over (eagerly, ~750 Linear calls per UNet step), so the answers are remembered.
struct SelectKey {
  int64_t M, N, K;
  size_t ws_bytes;
  // flags: fast | bpre << 1 | glu << 2, and what variant_matches reads of the leading dimensions (the
  // 32-bit addressing limits of some kernels): M lda, K ldb and 1024 ldc beyond 2^31 bytes << 3, 4, 5
  int dtype, fmt, terms, products, count, flags;
  bool operator==(const SelectKey& o) const {
    return M == o.M && N == o.N && K == o.K && ws_bytes == o.ws_bytes && dtype == o.dtype && fmt == o.fmt &&
           terms == o.terms && products == o.products && count == o.count && flags == o.flags;
  }
};
struct SelectKeyHash {
  size_t operator()(const SelectKey& k) const {
    uint64_t h = 1469598103934665603ull;
    auto mix = [&](uint64_t v) { h = (h ^ v) * 1099511628211ull; };
    mix((uint64_t)k.M); mix((uint64_t)k.N); mix((uint64_t)k.K); mix((uint64_t)k.ws_bytes);
    mix(((uint64_t)k.dtype << 40) ^ ((uint64_t)k.fmt << 32) ^ ((uint64_t)k.terms << 24) ^ ((uint64_t)k.products << 16) ^
        ((uint64_t)k.count << 8) ^ (uint64_t)k.flags);
    return (size_t)h;
  }
};
struct SelectHit { int variant, splits; };

static int select_variant_uncached(const Problem& q, bool fast, int count, size_t ws_bytes, int* splits_out);

// a x b x c > 2^31 - 1, for any non-negative 64-bit factors (the product itself may not fit 64 bits)
static bool beyond_i32(int64_t a, int64_t b, int64_t c) {
  int64_t ab = 0, abc = 0;
  return __builtin_mul_overflow(a, b, &ab) || __builtin_mul_overflow(ab, c, &abc) || abc > INT32_MAX;
}

static int select_variant(const Problem& q, bool fast, int count, size_t ws_bytes = (size_t)-1,
                          int* splits_out = nullptr) {
  static std::mutex mu;
  static std::unordered_map<SelectKey, SelectHit, SelectKeyHash> memo;
  const SelectKey key{q.M, q.N, q.K, ws_bytes, q.dtype, q.fmt, q.terms, q.products, count,
                      (fast ? 1 : 0) | (q.bpre ? 2 : 0) | (q.glu ? 4 : 0) | (q.glu_slots ? 64 : 0) | (beyond_i32(q.M, q.lda, 4) ? 8 : 0) |
                          (beyond_i32(q.K, q.ldb, 4) ? 16 : 0) | (beyond_i32(q.ldc, 1024, 1) ? 32 : 0)};
  {
    std::lock_guard<std::mutex> lock(mu);
    auto it = memo.find(key);
    if (it != memo.end()) {
      if (splits_out) *splits_out = it->second.splits;
      return it->second.variant;
    }
  }
  int splits = 1;
  const int v = select_variant_uncached(q, fast, count, ws_bytes, &splits);
  {
    std::lock_guard<std::mutex> lock(mu);
    if (memo.size() >= 4096) memo.clear();
    memo[key] = SelectHit{v, splits};
  }
  if (splits_out) *splits_out = splits;
  return v;
}

static int select_variant_uncached(const Problem& q, bool fast, int count, size_t ws_bytes, int* splits_out) {
  const auto& t = table();
  int best = -1;
  double best_cost = 0;
  if (splits_out) *splits_out = 1;
  for (int i = 0; i < (int)t.size(); ++i) {
    if (!variant_matches(t[i], q, fast)) continue;
    if (count > 1 && !t[i].grouped) continue;
    if (t[i].kind == KIND_SPLITK &&
        skinny_workspace_bytes(q.M, q.N, q.K, t[i].BM, t[i].BN, t[i].BK) > ws_bytes)
      continue;
    if (t[i].kind == KIND_F8K64 && f8k64_workspace_bytes(q.M, q.N, q.K, q.bpre, t[i].BM) > ws_bytes) continue;
    if (t[i].kind == KIND_F16K && f16k_workspace_bytes(q.M, q.N, q.K) > ws_bytes) continue;
    int sp = 1;
    const double c = variant_cost(i, q, count, ws_bytes, &sp);
    if (best < 0 || c < best_cost) {
      best = i;
      best_cost = c;
      if (splits_out) *splits_out = sp;
    }
  }
  return best < 0 ? (int)CASCMM_ERR_BAD_FORMAT : best;
}

// ---------------------------------------------------------------------------------------
// utility kernels
// ---------------------------------------------------------------------------------------
template <int IODT>
__global__ void fill_bias_kernel(void* C, const void* bias, int M, int N, int64_t ldc) {
  typedef typename IoType<IODT>::T T;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)M * N) return;
  const int r = (int)(i / N), c = (int)(i % N);
  IoType<IODT>::store((T*)C + (int64_t)r * ldc + c, bias ? IoType<IODT>::load((const T*)bias + c) : 0.f);
}

// fp8 tensor scale, three stream-ordered steps on the caller's int32: zero it, fold in the bit
// pattern of max|x| (non-negative floats order like their bit patterns), turn it into the
// exponent e with max|x| * 2^e in (224, 448]
__global__ void amax_begin_kernel(int32_t* exp_out) { *exp_out = 0; }

template <int IODT>
__global__ __launch_bounds__(256) void amax_kernel(const void* x, int64_t rows, int64_t cols, int64_t ld, int32_t* exp_out) {
  const unsigned best = amax_scan<IODT>(x, rows, cols, ld);
  if ((threadIdx.x & 63) == 0 && best != 0) atomicMax((unsigned*)exp_out, best);
}

__global__ void amax_end_kernel(int32_t* exp_out) { *exp_out = exp_of_amax((unsigned)*exp_out); }

// The same search in ONE launch.  scratch = {running max, arrival count}, both zero on entry: every
// workgroup folds its maximum in, fences, and takes a ticket; the one that draws the last ticket sees
// every other workgroup's contribution, writes {e_x, *second} and leaves the scratch zeroed for the
// next call.  No workgroup waits for another.
template <int IODT>
__global__ __launch_bounds__(1024) void amax_single_launch_kernel(const void* x, int64_t rows, int64_t cols, int64_t ld,
                                                                  const int32_t* second, int32_t* exps_out, unsigned* scratch) {
  __shared__ unsigned wave_best[16];
  const unsigned best = amax_scan<IODT>(x, rows, cols, ld);
  if ((threadIdx.x & 63) == 0) wave_best[threadIdx.x >> 6] = best;
  __syncthreads();
  if (threadIdx.x != 0) return;
  unsigned b = 0;
  for (unsigned w = 0; w < (blockDim.x >> 6); ++w) b = wave_best[w] > b ? wave_best[w] : b;
  // atomics of all workgroups on one word run one after another: skip the one that cannot raise
  // the maximum (the running value only grows within a call, so a stale read errs on the safe side)
  if (b > __hip_atomic_load(&scratch[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) atomicMax(&scratch[0], b);
  __threadfence();
  const unsigned ticket = atomicAdd(&scratch[1], 1u);
  if (ticket != gridDim.x - 1) return;
  __threadfence();
  const unsigned bits = atomicExch(&scratch[0], 0u);
  atomicExch(&scratch[1], 0u);
  exps_out[0] = exp_of_amax(bits);
  if (second) exps_out[1] = *second;
}

template <int IODT, int FMT, int TERMS>
__global__ void split_terms_kernel(const void* x, float* out, int64_t n, int tensor_exp) {
  typedef typename IoType<IODT>::T T;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float r[8];
  r[0] = IoType<IODT>::load((const T*)x + i) * __builtin_ldexpf(1.0f, tensor_exp);
#pragma unroll
  for (int e = 1; e < 8; ++e) r[e] = 0.f;
  u32x4 t[Lowp<FMT>::planes(TERMS)];
  split8<FMT, TERMS>(r, t);
#pragma unroll
  for (int k = 0; k < TERMS; ++k) {
    out[(int64_t)k * n + i] = Lowp<FMT>::element0(t[Lowp<FMT>::plane(k)], k);
  }
}

template <int IODT, int FMT>
static int launch_split(const void* x, float* out, int64_t n, int terms, int tensor_exp, hipStream_t s) {
  const unsigned grid = (unsigned)((n + 255) / 256);
  hipError_t err = hipSuccess;
  switch (terms) {
    case 1: CASCMM_LAUNCH(err, (split_terms_kernel<IODT, FMT, 1>), dim3(grid), dim3(256), 0, s, x, out, n, tensor_exp); break;
    case 2: CASCMM_LAUNCH(err, (split_terms_kernel<IODT, FMT, 2>), dim3(grid), dim3(256), 0, s, x, out, n, tensor_exp); break;
    case 3: CASCMM_LAUNCH(err, (split_terms_kernel<IODT, FMT, 3>), dim3(grid), dim3(256), 0, s, x, out, n, tensor_exp); break;
    default: return CASCMM_ERR_BAD_FORMAT;
  }
  return err == hipSuccess ? CASCMM_OK : CASCMM_ERR_LAUNCH;
}

// Splits a weight once: thread (kg, n) reads the 8 values B[8 kg .. 8 kg + 7][n] (zero beyond K),
// splits them like the GEMM kernels do and writes one 16-byte operand slot per plane to
// out[(plane * K/8 + kg) * N + n].
template <int IODT, int FMT, int TERMS>
__global__ __launch_bounds__(256) void prepare_weight_kernel(const void* B, int K, int N, int64_t ldb,
                                                            const int32_t* tensor_exp, u32x4* out, int flags) {
  typedef typename IoType<IODT>::T T;
  const int glu = flags & 1, chained = flags & 2;
  const int kgs = (K + 7) / 8;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)kgs * N) return;
  const int kg = (int)(i / N), n = (int)(i - (int64_t)kg * N);
  // gated layout: prepared columns alternate 32 value columns (first half of B) and their 32
  // gate columns (second half)
  const int src = glu ? (n >> 6) * 32 + (n & 31) + ((n >> 5) & 1) * (N >> 1) : n;
  float r[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    // chained: the k order of the left operand's slots as the gated store writes them (see
    // cascmm_prepare_left): positions 0..3 are k = 16 t + 4 g + 0..3 and 4..7 the same + 8, kg = 2 t + g
    const int k = chained ? 16 * (kg >> 1) + 8 * (e >> 2) + 4 * (kg & 1) + (e & 3) : kg * 8 + e;
    r[e] = k < K ? IoType<IODT>::load((const T*)B + (int64_t)k * ldb + src) : 0.f;
  }
  constexpr int PL = Lowp<FMT>::planes(TERMS);
  u32x4 t[PL];
  float scale = 1.f;
  if constexpr (Lowp<FMT>::kTensorScaled) {
    if (tensor_exp) scale = __builtin_ldexpf(1.f, *tensor_exp);
  }
  split8<FMT, TERMS>(r, t, scale);
#pragma unroll
  for (int pl = 0; pl < PL; ++pl) out[((int64_t)pl * kgs + kg) * N + n] = t[pl];
}

template <int IODT, int FMT>
static int launch_prepare(const void* B, int K, int N, int64_t ldb, int terms, const int32_t* e, u32x4* out, hipStream_t s,
                          int glu) {
  const int64_t total = (int64_t)((K + 7) / 8) * N;
  const unsigned grid = (unsigned)((total + 255) / 256);
  hipError_t err = hipSuccess;
  switch (terms) {
    case 1: CASCMM_LAUNCH(err, (prepare_weight_kernel<IODT, FMT, 1>), dim3(grid), dim3(256), 0, s, B, K, N, ldb, e, out, glu); break;
    case 2: CASCMM_LAUNCH(err, (prepare_weight_kernel<IODT, FMT, 2>), dim3(grid), dim3(256), 0, s, B, K, N, ldb, e, out, glu); break;
    case 3: CASCMM_LAUNCH(err, (prepare_weight_kernel<IODT, FMT, 3>), dim3(grid), dim3(256), 0, s, B, K, N, ldb, e, out, glu); break;
    default: return CASCMM_ERR_BAD_FORMAT;
  }
  return err == hipSuccess ? CASCMM_OK : CASCMM_ERR_LAUNCH;
}

template <int IODT>
static int launch_prepare_fmt(const void* B, int K, int N, int64_t ldb, int fmt, int terms, const int32_t* e, u32x4* out,
                              hipStream_t s, int glu) {
  if (fmt == CASCMM_FMT_BF16) return launch_prepare<IODT, CASCMM_FMT_BF16>(B, K, N, ldb, terms, e, out, s, glu);
  if (fmt == CASCMM_FMT_FP16) return launch_prepare<IODT, CASCMM_FMT_FP16>(B, K, N, ldb, terms, e, out, s, glu);
  if (fmt == CASCMM_FMT_FP8) return launch_prepare<IODT, CASCMM_FMT_FP8>(B, K, N, ldb, terms, e, out, s, glu);
  return CASCMM_ERR_BAD_FORMAT;
}

// 16-bit tensors multiplied as one term of their own format can use the prepared-operand kernels
// when the caller brought room for the re-laid B
// (a grouped launch needs `count` such buffers, one behind the other)
static bool onthefly_prepare_ok(const Problem& q, int count, const void* const* A, const void* const* B,
                                const void* workspace, size_t workspace_bytes) {
  if (q.bpre || q.dtype == CASCMM_DT_F32 || q.terms != 1 || q.K % 64 != 0) return false;
  if (!((q.dtype == CASCMM_DT_F16 && q.fmt == CASCMM_FMT_FP16) || (q.dtype == CASCMM_DT_BF16 && q.fmt == CASCMM_FMT_BF16)))
    return false;
  if (q.lda % 8 != 0) return false;
  for (int i = 0; i < count; ++i)
    if (!A[i] || !B[i] || !aligned_to(A[i], 16) || !aligned_to(B[i], 2)) return false;
  const int64_t need = prepared_bytes(q.K, q.N, q.fmt, 1);
  return workspace && aligned_to(workspace, 16) && need <= INT32_MAX && workspace_bytes >= (size_t)need * count;
}

// One launch for `count` problems of one shape (count == 1: a plain GEMM).
// exps_dyn (fp8-rate kernel only, count == 1): the launch finds the left operand's scale exponent
// itself and leaves {e_A, *b_exp_src} there; CASCMM_ERR_BAD_VARIANT when another kernel is selected.
static int gemm_impl(int count, const void* const* A, const void* const* B, void* const* C, const void* const* bias,
                     const Problem& q, const int32_t* tensor_exps, void* workspace, size_t workspace_bytes,
                     hipStream_t stream, int variant, int32_t* exps_dyn = nullptr, const int32_t* b_exp_src = nullptr) {
  int st = check_problem(q);
  if (st != CASCMM_OK) return st;
  if (count < 1 || count > kMaxGroup) return CASCMM_ERR_BAD_SHAPE;
  if (q.M == 0 || q.N == 0) return CASCMM_OK;
  const size_t es = dtype_size(q.dtype);
  for (int i = 0; i < count; ++i) {
    if (!C[i]) return CASCMM_ERR_NULL_POINTER;
    if (!aligned_to(C[i], es) || (bias && !aligned_to(bias[i], es))) return CASCMM_ERR_ALIGNMENT;
  }
  if (q.glu && (q.N % 64 != 0 || q.K == 0)) return CASCMM_ERR_BAD_SHAPE;
  if (q.K == 0) {
    const int64_t total = q.M * q.N;
    const unsigned grid = (unsigned)((total + 255) / 256);
    hipError_t err = hipSuccess;
    for (int i = 0; i < count; ++i) {
      const void* b = bias ? bias[i] : nullptr;
      if (q.dtype == CASCMM_DT_F32)
        CASCMM_LAUNCH(err, (fill_bias_kernel<CASCMM_DT_F32>), dim3(grid), dim3(256), 0, stream, C[i], b, (int)q.M, (int)q.N, q.ldc);
      else if (q.dtype == CASCMM_DT_F16)
        CASCMM_LAUNCH(err, (fill_bias_kernel<CASCMM_DT_F16>), dim3(grid), dim3(256), 0, stream, C[i], b, (int)q.M, (int)q.N, q.ldc);
      else
        CASCMM_LAUNCH(err, (fill_bias_kernel<CASCMM_DT_BF16>), dim3(grid), dim3(256), 0, stream, C[i], b, (int)q.M, (int)q.N, q.ldc);
    }
    return err == hipSuccess ? CASCMM_OK : CASCMM_ERR_LAUNCH;
  }
  if (onthefly_prepare_ok(q, count, A, B, workspace, workspace_bytes)) {
    // fp16 x fp16 (bf16 x bf16) tensors as one term: re-lay B as operand slots in the workspace
    // (one pass over B), then the copy-only kernels
    const size_t each = (size_t)prepared_bytes(q.K, q.N, q.fmt, 1);
    const void* bp[kMaxGroup];
    for (int i = 0; i < count; ++i) {
      void* dst = (char*)workspace + (size_t)i * each;
      bp[i] = dst;
      int same = -1;   // the same weight twice in one group is prepared once
      for (int j = 0; j < i && same < 0; ++j)
        if (B[j] == B[i]) same = j;
      if (same >= 0) {
        bp[i] = bp[same];
        continue;
      }
      st = cascmm_prepare_weight(B[i], q.K, q.N, q.ldb, q.dtype, q.fmt, 1, nullptr, dst, each, (void*)stream);
      if (st != CASCMM_OK) return st;
    }
    Problem qp = q;
    qp.bpre = true;
    qp.ldb = q.N;
    const int r = gemm_impl(count, A, bp, C, bias, qp, tensor_exps, nullptr, 0, stream, variant < 0 ? -1 : variant);
    if (r != CASCMM_ERR_BAD_FORMAT && r != CASCMM_ERR_BAD_VARIANT) return r;
  }
  bool fast = true;
  for (int i = 0; i < count; ++i) {
    if (!A[i] || !B[i]) return CASCMM_ERR_NULL_POINTER;
    if (!aligned_to(A[i], es) || !aligned_to(B[i], q.bpre ? 16 : es)) return CASCMM_ERR_ALIGNMENT;
    fast = fast && fast_ok(q, A[i], q.bpre ? nullptr : B[i]);
  }
  if (q.bpre) {
    // prepared weights only have the fast kernels: fp32 A with 16-byte aligned rows, K a multiple
    // of the kernel's K step (checked per variant), and a buffer the 32-bit offsets can span
    if (!fast) return CASCMM_ERR_ALIGNMENT;
    if (prepared_bytes(q.K, q.N, q.fmt, q.terms, q.glu) > INT32_MAX) return CASCMM_ERR_TOO_LARGE;
  }

  const auto& t = table();
  int splits = 1;
  if (variant < 0) {
    variant = select_variant(q, fast, count, workspace ? workspace_bytes : 0, &splits);
    if (variant < 0 && count > 1) {
      // no kernel takes these problems in one launch (the fp8-rate kernel runs one at a time): one
      // launch each, in order on the stream, sharing the workspace
      for (int i = 0; i < count; ++i) {
        const void* bi = bias ? bias[i] : nullptr;
        const int st1 = gemm_impl(1, A + i, B + i, C + i, bias ? &bi : nullptr, q, tensor_exps ? tensor_exps + 2 * i : nullptr,
                                  workspace, workspace_bytes, stream, -1);
        if (st1 != CASCMM_OK) return st1;
      }
      return CASCMM_OK;
    }
    if (variant < 0) return variant;
  } else {
    splits = (variant >> 16) > 0 ? (variant >> 16) : 1;   // forced: kernel index | K splits << 16
    variant &= 0xFFFF;
    if (splits > kMaxTileSplits) return CASCMM_ERR_BAD_VARIANT;
    if (variant >= (int)t.size()) return CASCMM_ERR_BAD_VARIANT;
    if (!variant_matches(t[variant], q, fast)) return CASCMM_ERR_BAD_VARIANT;
  }
  const VariantDesc& v = t[variant];
  if (exps_dyn && (v.kind != KIND_F8K64 || count != 1)) return CASCMM_ERR_BAD_VARIANT;
  if (count > 1 && !v.grouped) {
    // a forced kernel that runs one problem per launch: one launch each, in order on the stream
    if (v.kind == KIND_SPLITK) return CASCMM_ERR_BAD_VARIANT;
    for (int i = 0; i < count; ++i) {
      const void* bi = bias ? bias[i] : nullptr;
      const int st1 = gemm_impl(1, A + i, B + i, C + i, bias ? &bi : nullptr, q, tensor_exps ? tensor_exps + 2 * i : nullptr,
                                workspace, workspace_bytes, stream, variant | (splits > 1 ? splits << 16 : 0));
      if (st1 != CASCMM_OK) return st1;
    }
    return CASCMM_OK;
  }
  GroupParams p;
  memset(&p, 0, sizeof(p));
  p.M = (int)q.M; p.N = (int)q.N; p.K = (int)q.K;
  p.lda = q.lda; p.ldb = q.ldb; p.ldc = q.ldc;
  const int64_t tm = (q.M + v.BM - 1) / v.BM, tn = (q.N + v.BN - 1) / v.BN;
  if (tm * tn * count > INT32_MAX) return CASCMM_ERR_TOO_LARGE;
  p.tiles_m = (int)tm; p.tiles_n = (int)tn;
  p.count = count;
  p.workspace = workspace;
  p.workspace_bytes = workspace_bytes;
  p.k_splits = v.kind == KIND_TILE ? splits : 1;
  p.tensor_exps = q.fmt == CASCMM_FMT_FP8 ? tensor_exps : nullptr;
  p.glu = q.glu_slots ? 2 : (q.glu ? 1 : 0);
  p.exps_dyn = exps_dyn;
  p.b_exp_src = b_exp_src;
  for (int i = 0; i < count; ++i) {
    p.A[i] = A[i]; p.B[i] = B[i]; p.C[i] = C[i]; p.bias[i] = bias ? bias[i] : nullptr;
  }
  return v.launch(p, stream);
}

}  // namespace cascmm

using namespace cascmm;

// Built-in scratch of cascmm_gemm_noalloc: the K-split partial results that cascmm_gemm keeps in the
// caller's workspace.  One copy per GPU the library runs on, held until the process ends.  In host
// code the array's name is only a handle for hipGetSymbolAddress; the device address it returns
// (per device) is what kernels and copies are given.
static __device__ __align__(256) unsigned char scratch[CASCMM_NOALLOC_SCRATCH_BYTES];

static int noalloc_scratch(void** out) {
  static std::mutex mu;
  static void* ptr_of_device[kMaxDevices] = {nullptr};
  const int d = device_index();
  if (d < 0) return CASCMM_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(mu);
  if (!ptr_of_device[d]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return CASCMM_ERR_LAUNCH;
    ptr_of_device[d] = p;
  }
  *out = ptr_of_device[d];
  return CASCMM_OK;
}

extern "C" {

int cascmm_init(void) {
  void* p = nullptr;
  return noalloc_scratch(&p);
}

int cascmm_gemm_noalloc(const void* A, const void* B, void* C, const void* bias, int64_t M, int64_t N, int64_t K,
                        int64_t lda, int64_t ldb, int64_t ldc, int dtype, int fmt, int terms, int products,
                        const int32_t* tensor_exps, void* stream) {
  const Problem q{M, N, K, lda, ldb, ldc, dtype, fmt, terms, products};
  const int st = check_problem(q);
  if (st != CASCMM_OK) return st;
  if (M == 0 || N == 0 || K == 0) return cascmm_gemm(A, B, C, bias, M, N, K, lda, ldb, ldc, dtype, fmt, terms, products,
                                                     tensor_exps, nullptr, 0, stream);
  // the scratch that the kernel cascmm_gemm would pick with an unlimited workspace needs for this problem
  size_t need = 0;
  const void* const a1[1] = {A};
  const void* const b1[1] = {B};
  if (onthefly_prepare_ok(q, 1, a1, b1, (void*)16, (size_t)-1)) {
    need = (size_t)prepared_bytes(K, N, fmt, 1);            // 16-bit tensors: B re-laid as operand slots
  } else if (A && B) {
    int splits = 1;
    int v = select_variant(q, fast_ok(q, A, B), 1, (size_t)-1, &splits);
    if (v < 0) return v;
    if ((table()[v].kind == KIND_F8K64 && f8k64_workspace_bytes(M, N, K, false, table()[v].BM) > (size_t)CASCMM_NOALLOC_SCRATCH_BYTES) ||
        (table()[v].kind == KIND_F16K && f16k_workspace_bytes(M, N, K) > (size_t)CASCMM_NOALLOC_SCRATCH_BYTES)) {
      // the fp8-rate kernel is a choice, not a need: without room for its operand slots the choice is
      // made among the kernels that split inside the GEMM
      v = select_variant(q, fast_ok(q, A, B), 1, (size_t)CASCMM_NOALLOC_SCRATCH_BYTES, &splits);
      if (v < 0) return v;
    }
    const VariantDesc& d = table()[v];
    if (d.kind == KIND_SPLITK) need = skinny_workspace_bytes(M, N, K, d.BM, d.BN, d.BK);
    else if (d.kind == KIND_F8K64) need = f8k64_workspace_bytes(M, N, K, false, d.BM);
    else if (d.kind == KIND_F16K) need = f16k_workspace_bytes(M, N, K);
    else if (splits > 1) need = (size_t)splits * (size_t)M * (size_t)N * sizeof(float);
  }
  if (need > (size_t)CASCMM_NOALLOC_SCRATCH_BYTES) return CASCMM_ERR_SCRATCH_LIMIT;
  void* ws = nullptr;
  if (need > 0) {
    const int ss = noalloc_scratch(&ws);
    if (ss != CASCMM_OK) return ss;
  }
  // (nothing in the scratch has to start at zero: a launch reads back only the partial results it wrote)
  return gemm_impl(1, &A, &B, &C, bias ? &bias : nullptr, q, tensor_exps, ws, need, (hipStream_t)stream, -1);
}

int cascmm_gemm_variant(const void* A, const void* B, void* C, const void* bias, int64_t M, int64_t N, int64_t K,
                        int64_t lda, int64_t ldb, int64_t ldc, int dtype, int fmt, int terms, int products,
                        const int32_t* tensor_exps, void* workspace, size_t workspace_bytes, void* stream,
                        int variant) {
  const Problem q{M, N, K, lda, ldb, ldc, dtype, fmt, terms, products};
  return gemm_impl(1, &A, &B, &C, bias ? &bias : nullptr, q, tensor_exps, workspace, workspace_bytes, (hipStream_t)stream,
                   variant);
}

int cascmm_gemm_grouped(int count, const void* const* A, const void* const* B, void* const* C, const void* const* bias,
                        int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int dtype, int fmt,
                        int terms, int products, const int32_t* tensor_exps, void* workspace, size_t workspace_bytes,
                        void* stream, int variant) {
  if (!A || !B || !C) return CASCMM_ERR_NULL_POINTER;
  const Problem q{M, N, K, lda, ldb, ldc, dtype, fmt, terms, products};
  return gemm_impl(count, A, B, C, bias, q, tensor_exps, workspace, workspace_bytes, (hipStream_t)stream, variant);
}

int cascmm_select_variant_glu(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int dtype, int fmt,
                              int terms, int products) {
  Problem q{M, N, K, lda, ldb, ldc, dtype, fmt, terms, products};
  q.glu = true;
  const int st = check_problem(q);
  if (st != CASCMM_OK) return st;
  if (N % 64 != 0 || K == 0) return CASCMM_ERR_BAD_SHAPE;
  const bool fast = fast_ok(q, nullptr, nullptr);
  const int v = select_variant(q, fast, 1);
  if (v < 0) return v;
  // worth it?  The alternative is the best plain kernel for the product plus the caller's gate, which
  // reads M x N values and writes half as many (measured at about 3.5 TB/s, two launches); the kernel
  // with the gated store may be a poor fit for the shape (too few tiles for the chip).
  Problem plain = q;
  plain.glu = false;
  plain.ldc = N;
  const int vp = select_variant(plain, fast, 1);
  if (vp >= 0) {
    const double gate_us = 2.0 + (double)M * (double)N * 6.0 / 3.5e6;
    if (variant_cost(v, q, 1) > variant_cost(vp, plain, 1) + gate_us) return CASCMM_ERR_BAD_FORMAT;
  }
  return v;
}

int cascmm_gemm_glu(const void* A, const void* B, void* C, const void* bias, int64_t M, int64_t N, int64_t K, int64_t lda,
                    int64_t ldb, int64_t ldc, int dtype, int fmt, int terms, int products, void* stream, int variant) {
  Problem q{M, N, K, lda, ldb, ldc, dtype, fmt, terms, products};
  q.glu = true;
  return gemm_impl(1, &A, &B, &C, bias ? &bias : nullptr, q, nullptr, nullptr, 0, (hipStream_t)stream, variant);
}

int cascmm_gemm(const void* A, const void* B, void* C, const void* bias, int64_t M, int64_t N, int64_t K, int64_t lda,
                int64_t ldb, int64_t ldc, int dtype, int fmt, int terms, int products, const int32_t* tensor_exps,
                void* workspace, size_t workspace_bytes, void* stream) {
  return cascmm_gemm_variant(A, B, C, bias, M, N, K, lda, ldb, ldc, dtype, fmt, terms, products, tensor_exps,
                             workspace, workspace_bytes, stream, -1);
}

size_t cascmm_prepared_bytes(int64_t K, int64_t N, int fmt, int terms) {
  if (K < 0 || N < 0 || terms < 1 || terms > 3) return 0;
  if (fmt != CASCMM_FMT_BF16 && fmt != CASCMM_FMT_FP16 && fmt != CASCMM_FMT_FP8) return 0;
  // (three fp8 terms have two layouts, for the plain and the gated preparation: room for either)
  return (size_t)std::max(prepared_bytes(K, N, fmt, terms, false), prepared_bytes(K, N, fmt, terms, true));
}

static int prepare_weight_impl(const void* B, int64_t K, int64_t N, int64_t ldb, int dtype, int fmt, int terms,
                               const int32_t* tensor_exp, void* out, size_t out_bytes, void* stream, int glu) {
  if (K < 0 || N < 0 || ldb < N || (glu && N % 64 != 0)) return CASCMM_ERR_BAD_SHAPE;
  if (K > INT32_MAX || N > INT32_MAX) return CASCMM_ERR_TOO_LARGE;
  if (terms < 1 || terms > 3) return CASCMM_ERR_BAD_FORMAT;
  if (fmt != CASCMM_FMT_BF16 && fmt != CASCMM_FMT_FP16 && fmt != CASCMM_FMT_FP8) return CASCMM_ERR_BAD_FORMAT;
  if (K == 0 || N == 0) return CASCMM_OK;
  if (!B || !out) return CASCMM_ERR_NULL_POINTER;
  if (!aligned_to(out, 16)) return CASCMM_ERR_ALIGNMENT;
  if (out_bytes < (size_t)prepared_bytes(K, N, fmt, terms, glu != 0)) return CASCMM_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  if (prepared_as_k16_slots(K, fmt, terms, glu != 0)) {
    // the layout of the fp8-rate kernel: [term][K/16][N] slots of 16 k
    if (dtype != CASCMM_DT_F32) return CASCMM_ERR_BAD_DTYPE;
    const int64_t units = (K >> 4) * N;
    return launch_kernel(f8k64_split_cols_kernel<0>, dim3((unsigned)((units + 255) / 256)), dim3(256), 0, s, (const float*)B, (int)K,
                         (int)N, ldb, tensor_exp, (u32x4*)out) == hipSuccess ? CASCMM_OK : CASCMM_ERR_LAUNCH;
  }
  if (dtype == CASCMM_DT_F32) return launch_prepare_fmt<CASCMM_DT_F32>(B, (int)K, (int)N, ldb, fmt, terms, tensor_exp, (u32x4*)out, s, glu);
  if (dtype == CASCMM_DT_F16) return launch_prepare_fmt<CASCMM_DT_F16>(B, (int)K, (int)N, ldb, fmt, terms, tensor_exp, (u32x4*)out, s, glu);
  if (dtype == CASCMM_DT_BF16) return launch_prepare_fmt<CASCMM_DT_BF16>(B, (int)K, (int)N, ldb, fmt, terms, tensor_exp, (u32x4*)out, s, glu);
  return CASCMM_ERR_BAD_DTYPE;
}

int cascmm_prepare_weight(const void* B, int64_t K, int64_t N, int64_t ldb, int dtype, int fmt, int terms,
                          const int32_t* tensor_exp, void* out, size_t out_bytes, void* stream) {
  return prepare_weight_impl(B, K, N, ldb, dtype, fmt, terms, tensor_exp, out, out_bytes, stream, 0);
}

int cascmm_prepare_weight_glu(const void* B, int64_t K, int64_t N, int64_t ldb, int dtype, int fmt, int terms,
                              const int32_t* tensor_exp, void* out, size_t out_bytes, void* stream) {
  return prepare_weight_impl(B, K, N, ldb, dtype, fmt, terms, tensor_exp, out, out_bytes, stream, 1);
}

int cascmm_gemm_prepared_glu(int count, const void* const* A, const void* const* Bprep, void* const* C,
                             const void* const* bias, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldc,
                             int dtype, int fmt, int terms, int products, const int32_t* tensor_exps, void* stream,
                             int variant) {
  if (!A || !Bprep || !C) return CASCMM_ERR_NULL_POINTER;
  Problem q{M, N, K, lda, N, ldc, dtype, fmt, terms, products};
  q.bpre = true;
  q.glu = true;
  return gemm_impl(count, A, Bprep, C, bias, q, tensor_exps, nullptr, 0, (hipStream_t)stream, variant);
}

int cascmm_gemm_prepared(int count, const void* const* A, const void* const* Bprep, void* const* C,
                         const void* const* bias, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldc, int dtype,
                         int fmt, int terms, int products, const int32_t* tensor_exps, void* workspace,
                         size_t workspace_bytes, void* stream, int variant) {
  if (!A || !Bprep || !C) return CASCMM_ERR_NULL_POINTER;
  Problem q{M, N, K, lda, N, ldc, dtype, fmt, terms, products};
  q.bpre = true;
  return gemm_impl(count, A, Bprep, C, bias, q, tensor_exps, workspace, workspace_bytes, (hipStream_t)stream, variant);
}

int cascmm_select_variant_prepared(int count, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldc, int dtype, int fmt,
                                   int terms, int products) {
  if (count < 1 || count > kMaxGroup) return CASCMM_ERR_BAD_SHAPE;
  Problem q{M, N, K, lda, N, ldc, dtype, fmt, terms, products};
  q.bpre = true;
  const int st = check_problem(q);
  if (st != CASCMM_OK) return st;
  return select_variant(q, fast_ok(q, nullptr, nullptr), count);
}

size_t cascmm_workspace_bytes(int64_t M, int64_t N, int64_t K, int dtype, int fmt, int terms, int products) {
  // upper bound over the skinny variants that could be selected for this problem (the
  // selection also depends on pointer alignment, which is not known here)
  const Problem q{M, N, K, K, N, N, dtype, fmt, terms, products};
  if (check_problem(q) != CASCMM_OK) return 0;
  size_t need = 0;
  for (const auto& v : table()) {
    if (v.kind != KIND_SPLITK || !variant_matches(v, q, fast_ok(q, nullptr, nullptr))) continue;
    const size_t n = skinny_workspace_bytes(M, N, K, v.BM, v.BN, v.BK);
    need = n > need ? n : need;
  }
  // three fp8 terms on the fp8-rate kernel: the operand slots of A and B
  for (const auto& v : table()) {
    if (v.kind != KIND_F8K64 || v.bpre || !variant_matches(v, q, fast_ok(q, nullptr, nullptr))) continue;
    const size_t n = f8k64_workspace_bytes(M, N, K, false, v.BM);
    need = n > need ? n : need;
  }
  // three fp16 terms on operand slots: the slots of A and B
  for (const auto& v : table()) {
    if (v.kind != KIND_F16K || !variant_matches(v, q, fast_ok(q, nullptr, nullptr))) continue;
    const size_t n = f16k_workspace_bytes(M, N, K);
    need = n > need ? n : need;
  }
  // 16-bit tensors as one term of their own format: room for B re-laid as operand slots
  if (((dtype == CASCMM_DT_F16 && fmt == CASCMM_FMT_FP16) || (dtype == CASCMM_DT_BF16 && fmt == CASCMM_FMT_BF16)) &&
      terms == 1 && K % 64 == 0) {
    const int64_t n = prepared_bytes(K, N, fmt, 1);
    if (n <= INT32_MAX && (size_t)n > need) need = (size_t)n;
  }
  // K split of the LDS-tiled kernels: up to kMaxTileSplits partial results when some kernel
  // would run the problem with at most half the CUs busy
  if (dtype == CASCMM_DT_F32 && N % 4 == 0) {
    for (int vi = 0; vi < (int)table().size(); ++vi) {
      const VariantDesc& v = table()[vi];
      if (v.kind != KIND_TILE || !variant_matches(v, q, fast_ok(q, nullptr, nullptr))) continue;
      int sp = 1;
      variant_cost(vi, q, 1, (size_t)-1, &sp);
      const size_t n = sp > 1 ? (size_t)kMaxTileSplits * M * N * sizeof(float) : 0;
      need = n > need ? n : need;
    }
  }
  return need;
}

int cascmm_select_variant(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int dtype, int fmt,
                          int terms, int products) {
  const Problem q{M, N, K, lda, ldb, ldc, dtype, fmt, terms, products};
  const int st = check_problem(q);
  if (st != CASCMM_OK) return st;
  return select_variant(q, fast_ok(q, nullptr, nullptr), 1);
}

int cascmm_select_variant_grouped(int count, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                                  int dtype, int fmt, int terms, int products) {
  if (count < 1 || count > kMaxGroup) return CASCMM_ERR_BAD_SHAPE;
  const Problem q{M, N, K, lda, ldb, ldc, dtype, fmt, terms, products};
  const int st = check_problem(q);
  if (st != CASCMM_OK) return st;
  return select_variant(q, fast_ok(q, nullptr, nullptr), count);
}

int cascmm_variant_count(void) { return (int)table().size(); }

const char* cascmm_variant_name(int variant) {
  if (variant < 0 || variant >= (int)table().size()) return nullptr;
  return table()[variant].name;
}

const char* cascmm_variant_kernel(int variant) {
  if (variant < 0 || variant >= (int)table().size()) return nullptr;
  const void* handle = nullptr;
  GroupParams p;
  memset(&p, 0, sizeof(p));
  p.kernel_out = &handle;
  if (table()[variant].launch(p, nullptr) != CASCMM_OK || !handle) return nullptr;
  // the handle of a kernel is an exported object of this library that carries the kernel's name
  Dl_info info;
  if (!dladdr(handle, &info) || !info.dli_sname || info.dli_saddr != handle) return nullptr;
  return info.dli_sname;
}

int cascmm_tensor_exp(const void* x, int64_t rows, int64_t cols, int64_t ld, int dtype, int32_t* exp_out,
                      void* stream) {
  if (dtype != CASCMM_DT_F32 && dtype != CASCMM_DT_F16 && dtype != CASCMM_DT_BF16) return CASCMM_ERR_BAD_DTYPE;
  if (rows < 0 || cols < 0 || ld < cols) return CASCMM_ERR_BAD_SHAPE;
  if (!exp_out || (rows * cols > 0 && !x)) return CASCMM_ERR_NULL_POINTER;
  if (rows > INT32_MAX || cols > INT32_MAX) return CASCMM_ERR_TOO_LARGE;
  hipStream_t s = (hipStream_t)stream;
  // *exp_out holds the bit pattern of the running max|x| until the last kernel replaces it
  hipError_t err = hipSuccess;
  CASCMM_LAUNCH(err, amax_begin_kernel, dim3(1), dim3(1), 0, s, exp_out);
  const int64_t total = rows * cols;
  if (total > 0) {
    const unsigned grid = (unsigned)std::min<int64_t>((total + 4095) / 4096, 1024);
    if (dtype == CASCMM_DT_F32)
      CASCMM_LAUNCH(err, (amax_kernel<CASCMM_DT_F32>), dim3(grid), dim3(256), 0, s, x, rows, cols, ld, exp_out);
    else if (dtype == CASCMM_DT_F16)
      CASCMM_LAUNCH(err, (amax_kernel<CASCMM_DT_F16>), dim3(grid), dim3(256), 0, s, x, rows, cols, ld, exp_out);
    else
      CASCMM_LAUNCH(err, (amax_kernel<CASCMM_DT_BF16>), dim3(grid), dim3(256), 0, s, x, rows, cols, ld, exp_out);
  }
  CASCMM_LAUNCH(err, amax_end_kernel, dim3(1), dim3(1), 0, s, exp_out);
  return err == hipSuccess ? CASCMM_OK : CASCMM_ERR_LAUNCH;
}

int cascmm_tensor_exps(const void* x, int64_t rows, int64_t cols, int64_t ld, int dtype, const int32_t* second_exp,
                       int32_t* exps_out, int32_t* scratch, void* stream) {
  if (dtype != CASCMM_DT_F32 && dtype != CASCMM_DT_F16 && dtype != CASCMM_DT_BF16) return CASCMM_ERR_BAD_DTYPE;
  if (rows < 0 || cols < 0 || ld < cols) return CASCMM_ERR_BAD_SHAPE;
  if (!exps_out || !scratch || (rows * cols > 0 && !x)) return CASCMM_ERR_NULL_POINTER;
  if (rows > INT32_MAX || cols > INT32_MAX) return CASCMM_ERR_TOO_LARGE;
  hipStream_t s = (hipStream_t)stream;
  const int64_t total = rows * cols;
  // (an empty tensor: one workgroup that scans nothing and writes e = 0)
  hipError_t err = hipSuccess;
  // few, large workgroups: every workgroup ends in a ticket atomic on one word, and those serialise
  const unsigned grid = (unsigned)std::max<int64_t>(1, std::min<int64_t>((total + 16383) / 16384, device_cus() / 2));
  if (dtype == CASCMM_DT_F32)
    CASCMM_LAUNCH(err, (amax_single_launch_kernel<CASCMM_DT_F32>), dim3(grid), dim3(1024), 0, s, x, rows, cols, ld, second_exp,
                       exps_out, (unsigned*)scratch);
  else if (dtype == CASCMM_DT_F16)
    CASCMM_LAUNCH(err, (amax_single_launch_kernel<CASCMM_DT_F16>), dim3(grid), dim3(1024), 0, s, x, rows, cols, ld, second_exp,
                       exps_out, (unsigned*)scratch);
  else
    CASCMM_LAUNCH(err, (amax_single_launch_kernel<CASCMM_DT_BF16>), dim3(grid), dim3(1024), 0, s, x, rows, cols, ld, second_exp,
                       exps_out, (unsigned*)scratch);
  return err == hipSuccess ? CASCMM_OK : CASCMM_ERR_LAUNCH;
}

int cascmm_gemm_fp8_autoscale(const void* A, const void* B, int b_prepared, void* C, const void* bias, int64_t M, int64_t N,
                              int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int terms, int products, const int32_t* b_exp,
                              int32_t* exps_out, int32_t* scratch, void* workspace, size_t workspace_bytes, void* stream) {
  if (!exps_out || !scratch) return CASCMM_ERR_NULL_POINTER;
  Problem q{M, N, K, lda, b_prepared ? N : ldb, ldc, CASCMM_DT_F32, CASCMM_FMT_FP8, terms, products};
  q.bpre = b_prepared != 0;
  const int st = check_problem(q);
  if (st != CASCMM_OK) return st;
  const void* bias1 = bias;
  if (M > 0 && N > 0 && K > 0 && A && B) {
    // the fp8-rate kernel splits A in a pass of its own anyway: the search rides on it
    const bool fast = fast_ok(q, A, q.bpre ? nullptr : B);
    if (!q.bpre || fast) {
      const int v = select_variant(q, fast, 1, workspace ? workspace_bytes : 0);
      if (v >= 0 && table()[v].kind == KIND_F8K64)
        return gemm_impl(1, &A, &B, &C, bias ? &bias1 : nullptr, q, nullptr, workspace, workspace_bytes, (hipStream_t)stream, v,
                         exps_out, b_exp);
    }
  }
  // any other kernel: the one-launch search, then the GEMM with its result
  const int se = cascmm_tensor_exps(A, M, K, lda, CASCMM_DT_F32, b_exp, exps_out, scratch, stream);
  if (se != CASCMM_OK) return se;
  if (!b_exp) {
    // (exps_out[1] must be defined: a NULL b_exp means e_B = 0)
    hipError_t err = hipSuccess;
    CASCMM_LAUNCH(err, amax_begin_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, exps_out + 1);
    if (err != hipSuccess) return CASCMM_ERR_LAUNCH;
  }
  return gemm_impl(1, &A, &B, &C, bias ? &bias1 : nullptr, q, exps_out, workspace, workspace_bytes, (hipStream_t)stream, -1);
}

int cascmm_split_terms(const void* x, float* out, int64_t n, int dtype, int fmt, int terms, int tensor_exp,
                       void* stream) {
  if (n < 0) return CASCMM_ERR_BAD_SHAPE;
  if (n == 0) return CASCMM_OK;
  if (!x || !out) return CASCMM_ERR_NULL_POINTER;
  if (dtype != CASCMM_DT_F32) return CASCMM_ERR_BAD_DTYPE;
  hipStream_t s = (hipStream_t)stream;
  if (fmt == CASCMM_FMT_BF16) return launch_split<CASCMM_DT_F32, CASCMM_FMT_BF16>(x, out, n, terms, tensor_exp, s);
  if (fmt == CASCMM_FMT_FP16) return launch_split<CASCMM_DT_F32, CASCMM_FMT_FP16>(x, out, n, terms, tensor_exp, s);
  if (fmt == CASCMM_FMT_FP8) return launch_split<CASCMM_DT_F32, CASCMM_FMT_FP8>(x, out, n, terms, tensor_exp, s);
  return CASCMM_ERR_BAD_FORMAT;
}

const char* cascmm_strerror(int status) {
  switch (status) {
    case CASCMM_OK: return "ok";
    case CASCMM_ERR_NULL_POINTER: return "null pointer argument";
    case CASCMM_ERR_BAD_SHAPE: return "bad shape or leading dimension";
    case CASCMM_ERR_BAD_DTYPE: return "unsupported element type";
    case CASCMM_ERR_BAD_FORMAT: return "unsupported format / terms / products combination";
    case CASCMM_ERR_WORKSPACE: return "workspace missing or too small";
    case CASCMM_ERR_ALIGNMENT: return "pointer not aligned to its element size";
    case CASCMM_ERR_LAUNCH: return "HIP launch failed";
    case CASCMM_ERR_BAD_VARIANT: return "kernel variant unknown or unable to run this problem";
    case CASCMM_ERR_TOO_LARGE: return "dimension too large";
    case CASCMM_ERR_SCRATCH_LIMIT: return "problem needs more scratch than the library's built-in buffer holds (use cascmm_gemm with a workspace)";
    default: return "unknown status";
  }
}

int cascmm_selftest(void) {
  int bad = 0;
  const auto& t = table();
  for (const TunedCost& c : kTuned) {
    int hits = 0;
    for (const VariantDesc& d : t) hits += strcmp(c.name, d.name) == 0 ? 1 : 0;
    bad += hits == 1 ? 0 : 1;
  }
  for (size_t i = 0; i < t.size(); ++i)
    for (size_t j = i + 1; j < t.size(); ++j) bad += strcmp(t[i].name, t[j].name) == 0 ? 1 : 0;
  return bad;
}

// ---- chained feed-forward: both operands as slots -------------------------------------------------
size_t cascmm_left_slots_bytes(int64_t M, int64_t K) {
  if (M <= 0 || K <= 0 || K % 16 != 0) return 0;
  int64_t mk = 0, bytes = 0;
  if (__builtin_mul_overflow(M, K, &mk) || __builtin_mul_overflow(mk, (int64_t)4, &bytes)) return 0;
  return (size_t)bytes;
}

int cascmm_prepare_left(const void* A, int64_t M, int64_t K, int64_t lda, void* out, size_t out_bytes, void* stream) {
  if (M < 0 || K < 0 || lda < K || K % 16 != 0) return CASCMM_ERR_BAD_SHAPE;
  if (M > INT32_MAX || K > INT32_MAX) return CASCMM_ERR_TOO_LARGE;
  if (M == 0 || K == 0) return CASCMM_OK;
  if (!A || !out) return CASCMM_ERR_NULL_POINTER;
  if (!aligned_to(A, 16) || !aligned_to(out, 16) || lda % 4 != 0) return CASCMM_ERR_ALIGNMENT;
  const size_t need = cascmm_left_slots_bytes(M, K);
  if (need == 0 || need > (size_t)INT32_MAX) return CASCMM_ERR_TOO_LARGE;
  if (out_bytes < need) return CASCMM_ERR_WORKSPACE;
  return launch_prepare_left((const float*)A, (int)M, (int)K, lda, out, (hipStream_t)stream);
}

int cascmm_prepare_weight_chained(const void* B, int64_t K, int64_t N, int64_t ldb, void* out, size_t out_bytes, void* stream) {
  if (K < 0 || N < 0 || ldb < N || K % 16 != 0) return CASCMM_ERR_BAD_SHAPE;
  if (K > INT32_MAX || N > INT32_MAX) return CASCMM_ERR_TOO_LARGE;
  if (K == 0 || N == 0) return CASCMM_OK;
  if (!B || !out) return CASCMM_ERR_NULL_POINTER;
  if (!aligned_to(out, 16)) return CASCMM_ERR_ALIGNMENT;
  if (out_bytes < (size_t)prepared_bytes(K, N, CASCMM_FMT_BF16, 2)) return CASCMM_ERR_WORKSPACE;
  return launch_prepare<CASCMM_DT_F32, CASCMM_FMT_BF16>(B, (int)K, (int)N, ldb, 2, nullptr, (u32x4*)out, (hipStream_t)stream, 2);
}

int cascmm_gemm_glu_chained(const void* A, const void* B, int b_prepared, void* out_slots, size_t out_bytes, const void* bias,
                            int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, void* stream) {
  if (N % 64 != 0) return CASCMM_ERR_BAD_SHAPE;
  Problem q{M, N, K, lda, b_prepared ? N : ldb, N / 2, CASCMM_DT_F32, CASCMM_FMT_BF16, 2, CASCMM_PROD_TRI};
  q.bpre = b_prepared != 0;
  q.glu = true;
  q.glu_slots = true;
  const int st = check_problem(q);
  if (st != CASCMM_OK) return st;
  if (M == 0 || N == 0) return CASCMM_OK;
  if (!out_slots) return CASCMM_ERR_NULL_POINTER;
  if (!aligned_to(out_slots, 16)) return CASCMM_ERR_ALIGNMENT;
  const size_t need = cascmm_left_slots_bytes(M, N / 2);
  if (need == 0 || need > (size_t)INT32_MAX) return CASCMM_ERR_TOO_LARGE;
  if (out_bytes < need) return CASCMM_ERR_WORKSPACE;
  return gemm_impl(1, &A, &B, &out_slots, bias ? &bias : nullptr, q, nullptr, nullptr, 0, (hipStream_t)stream, -1);
}

int cascmm_chained_supported(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K < 16 || K % 16 != 0) return 0;
  if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return 0;
  if (beyond_i32(M, K, 4) || beyond_i32(N, K, 4)) return 0;   // both slot buffers below 2 GiB
  return 1;
}

int cascmm_gemm_chained(const void* Aslots, const void* Bslots, void* C, const void* bias, int64_t M, int64_t N, int64_t K,
                        int64_t ldc, void* stream) {
  if (M < 0 || N < 0 || K < 0 || ldc < N) return CASCMM_ERR_BAD_SHAPE;
  if (M == 0 || N == 0) return CASCMM_OK;
  if (!cascmm_chained_supported(M, N, K)) return CASCMM_ERR_BAD_FORMAT;
  if (!Aslots || !Bslots || !C) return CASCMM_ERR_NULL_POINTER;
  if (!aligned_to(Aslots, 16) || !aligned_to(Bslots, 16) || !aligned_to(C, 4) || !aligned_to(bias, 4)) return CASCMM_ERR_ALIGNMENT;
  if (beyond_i32(ldc, SlotK::BM, 4)) return CASCMM_ERR_TOO_LARGE;
  SlotKParams q;
  memset(&q, 0, sizeof(q));
  q.a = Aslots; q.b_slots = Bslots; q.C = (float*)C; q.bias = (const float*)bias;
  q.M = (int)M; q.N = (int)N; q.K = (int)K; q.ldc = ldc;
  return launch_slotk(q, 0, (hipStream_t)stream);
}

int cascmm_version(void) { return CASCMM_VERSION; }

}  // extern "C"
