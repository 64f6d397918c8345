// LDS-tiled MFMA kernel of the cascade GEMM (gfx950).
//
// One workgroup computes a BM x BN tile of C.  Per K step of BK:
//   global (row-major)  --VGPR: split into TERMS low-precision terms-->  LDS  -->  MFMA
// Both operands are staged in LDS already split, in "slot" form: one 16-byte slot holds 8
// consecutive-k values of one row (A) or one column (B) of one term, i.e. exactly what one
// lane feeds to v_mfma_f32_32x32x16 (lane l: row/col l%32, k-group l/32).  A plane is all
// slots of one k-group, BM (or BN) slots long; 16 consecutive lanes of a fragment read
// therefore fetch 256 contiguous bytes and planes start at multiples of 256 bytes, which is
// what the 64-bank LDS needs for full-rate ds_read_b128.  A-side stores come from lanes
// that walk k fastest (coalesced global loads), so rows are XOR-swizzled per k-group to keep
// eight consecutive lanes on eight different 16-byte bank groups.
//
// B columns come in groups of 128.  A producer lane loads a 8(k) x 4(n) block with eight
// 16-byte loads and owns four slots; slot i*32 + j of the group holds column 4*j + i, so the
// four slot writes of 64 lanes are contiguous (no bank conflicts) and, in the epilogue, lane
// j of the four 32-column MFMA blocks of a group holds columns 4*j .. 4*j+3 of a row: one
// 16-byte store.  Wide loads also keep the number of loads in flight under the 6-bit vmcnt
// limit, without which the prefetch ring cannot be waited on selectively.  Columns left over
// after the last whole group (a multiple of 32) are loaded one per lane, unpermuted.
//
// The 32x32x16 MFMA is used rather than 16x16x32: it sustains a higher rate on this part and,
// more important here, leaves room for about six other VALU instructions per MFMA (the
// 16x16x32 form leaves two), which is what hides the three VALU operations per element that
// the operand split costs.
//
// Global loads are raw buffer loads: the per-lane offset is fixed for the whole K loop and the
// K position is a scalar offset, so the loop spends no VALU work on addresses.  Rows and
// columns past the matrix edge are clamped to the last valid one (their results are never
// stored).  Each thread keeps DEPTH K-steps of operands in flight in registers (a ring
// indexed by compile-time constants), the LDS stage is double buffered, and there is one
// barrier per K step.
//
// The kernel is persistent and grouped: a launch covers `count` GEMMs of one shape, the grid
// is at most one workgroup per CU, and a workgroup walks its work items (tiles) in turn.  The
// producers' prefetch ring runs across item boundaries, so the load latency of a tile's first
// operands is hidden behind the previous tile's last steps and result stores.
//
// The workgroup is specialised.  WM x WN x WK "consumer" waves only read fragments from LDS
// and issue MFMAs; NP "producer" waves only load, split and write LDS.  With one wave of each
// kind per SIMD, the producer's VALU work issues in the gaps the consumer's MFMAs leave on
// the VALU port, and neither kind ever waits for the other except at the one barrier per K
// step.  Producers hold no accumulators, so their registers go to a deep prefetch ring.
// With WK = 2 the two consumer groups take alternate 16-wide k slices of every stage and
// their accumulators are added through LDS at the end.
//
// All partial products of one (m-tile, n-tile) reuse the same fragments in registers; the
// cross-term sum happens in the accumulator registers (one accumulator per scale class).
#pragma once
#include "cascmm_common.h"

namespace cascmm {

template <int BM_, int BN_, int BK_, int WM_, int WN_, int WK_ = 1, int DEPTH_ = 2, int NP_ = 4, bool QUADS_ = true,
          bool PAIRS_ = false>
struct Tile {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_, WK = WK_, DEPTH = DEPTH_, NP = NP_;
  static constexpr int NCW = WM * WN * WK;   // consumer waves
  static constexpr int NTP = NP * kWave;     // producer threads
  static constexpr int NT = (NCW + NP) * kWave;
  static constexpr int KG = BK / 8;          // k-groups (planes) per stage
  static constexpr int WTM = BM / WM, WTN = BN / WN;
  static constexpr int MT = WTM / 32, NTL = WTN / 32;
  static constexpr int KSUB = BK / 16;       // MFMA k slices per stage
  // B columns: the first BNQ (whole groups of 128) are loaded four at a time (16-byte loads)
  // and stored permuted in LDS; the remaining BNS columns are loaded one at a time.
  // (QUADS_ = false: every column one at a time, which gives units small enough to spread
  // evenly over eight producer waves.)
  static constexpr int BNQ = QUADS_ ? (BN / 128) * 128 : 0, BNS = BN - BNQ;
  // PAIRS_: the permuted columns are staged two at a time (8-byte loads, 8 k x 2 n per unit)
  // instead of four: twice as many, half as large units, so that every producer thread gets
  // the same mix of units and needs a smaller register ring
  static constexpr int QN = PAIRS_ ? 2 : 4;
  // a consumer wave must own whole runs of permuted blocks: all four of a group, or two
  static_assert(BNQ == 0 || WTN % 128 == 0 || WTN == 64 || (WN == 1), "wave tile vs permuted B columns");
  static_assert(BNQ == 0 || WN == 1 || BNS == 0, "mixed B column layouts need one consumer wave column");
  static_assert(BK == 32 || BK == 64 || BK == 128, "BK");
  static_assert(BM % (32 * WM) == 0 && BN % (32 * WN) == 0, "wave tile must be a multiple of 32");
  static_assert(KSUB % WK == 0, "k slices must divide evenly among the wave groups");
  static_assert(WK == 1 || WK == 2, "WK");
  static_assert(DEPTH >= 1 && DEPTH <= 4, "DEPTH");
};

template <class TL, int TERMS>
struct LdsLayout {
  // in slots (16 bytes)
  static constexpr int kAPlane = TL::BM;
  static constexpr int kBPlane = TL::BN;
  static constexpr int kATerm = TL::KG * kAPlane;
  static constexpr int kBTerm = TL::KG * kBPlane;
  static constexpr int kStage = TERMS * (kATerm + kBTerm);
  static constexpr int kReduce = (TL::WK > 1) ? TL::BM * TL::BN / 4 : 0;  // fp32 tile, in slots
  static constexpr int kSlots = (2 * kStage > kReduce) ? 2 * kStage : kReduce;
  static constexpr int kBytes = kSlots * 16;
  // XOR applied to the row index of an A slot in k-group kg: lanes walk k-groups fastest, so
  // 8 consecutive lanes cover 8/KG' rows x KG' k-groups (KG' = min(KG, 8)); the XOR spreads
  // them over 8 different 16-byte bank groups.
  static __device__ __forceinline__ int swz(int kg) { return (kg * (TL::KG >= 8 ? 1 : 8 / TL::KG)) & 7; }
};

// XCD-aware tile order.  Workgroup ids are dealt round-robin to the 8 XCDs, each with its own
// L2: give every XCD one contiguous range of tile ids.  Inside the range, tile ids walk
// kGroupM rows of tiles down before moving one tile to the right, so the workgroups that are
// resident together on one XCD cover a roughly square block and share both A and B tiles in
// that L2.
constexpr int kGroupM = 4;
__device__ __forceinline__ void tile_coords(int bid, int tiles_m, int tiles_n, int& tm, int& tn, int group_m = kGroupM) {
  const int total = tiles_m * tiles_n;
  const int per = total >> 3;
  int id = bid;
  if (bid < (per << 3)) id = (bid & 7) * per + (bid >> 3);
  const int group = group_m * tiles_n;
  const int g = id / group;
  const int first = g * group_m;
  const int rows = (tiles_m - first) < group_m ? (tiles_m - first) : group_m;
  const int in = id - g * group;
  tm = first + in % rows;
  tn = in / rows;
}

// Raw buffer loads through the LLVM intrinsics: address = base + voffset + soffset, voffset a
// per-lane VGPR, soffset a wave-uniform SGPR.
typedef int i32x4 __attribute__((ext_vector_type(4)));
__device__ float llvm_raw_buffer_load_f32(i32x4 rsrc, int voffset, int soffset, int aux) __asm("llvm.amdgcn.raw.buffer.load.f32");
__device__ f32x4 llvm_raw_buffer_load_v4f32(i32x4 rsrc, int voffset, int soffset, int aux) __asm("llvm.amdgcn.raw.buffer.load.v4f32");
typedef float f32x2_ld __attribute__((ext_vector_type(2)));
__device__ f32x2_ld llvm_raw_buffer_load_v2f32(i32x4 rsrc, int voffset, int soffset, int aux) __asm("llvm.amdgcn.raw.buffer.load.v2f32");
__device__ void llvm_raw_buffer_store_f32(float v, i32x4 rsrc, int voffset, int soffset, int aux) __asm("llvm.amdgcn.raw.buffer.store.f32");
__device__ void llvm_raw_buffer_store_v4f32(f32x4 v, i32x4 rsrc, int voffset, int soffset, int aux) __asm("llvm.amdgcn.raw.buffer.store.v4f32");
typedef float f32x2 __attribute__((ext_vector_type(2)));
__device__ void llvm_raw_buffer_store_v2f32(f32x2 v, i32x4 rsrc, int voffset, int soffset, int aux) __asm("llvm.amdgcn.raw.buffer.store.v2f32");
__device__ void llvm_raw_buffer_store_i16(short v, i32x4 rsrc, int voffset, int soffset, int aux) __asm("llvm.amdgcn.raw.buffer.store.i16");

// Cache policy of the result stores: sc1 (agent scope) for the kernels with small tiles, the default for the
// large ones.  A/B on one box, whole kernels: 2048x1280x1280 27.1 -> 26.4 us, 4096x640x640 18.2 -> 17.6 us,
// 8192x640x640 31.7 -> 30.5 us, 2048x5120x1280 83.3 -> 82.7 us with sc1; the 256x320 and the fp8-rate tiles,
// whose workgroups store 160-320 KB each at the same moment, measured 0.0-0.4 % slower with it and keep the
// default.  (A bare store loop of the large tile's pattern is faster with sc1, 16.5 -> 13.9 us for 84 MB, and
// slower with nt, 18.2 us.)
constexpr int kResultStoreAux = 16;
constexpr int kLargeTileStoreAux = 0;

// gfx9-family raw buffer descriptor: 48-bit base, stride 0, byte count, 32-bit data format
__device__ __forceinline__ i32x4 make_rsrc(const void* base, int64_t bytes) {
  const uint64_t b = (uint64_t)base;
  i32x4 r;
  r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)b);
  r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)((b >> 32) & 0xFFFFu));
  r[2] = __builtin_amdgcn_readfirstlane(bytes > 0x7FFFFFFF ? 0x7FFFFFFF : (int)bytes);
  r[3] = 0x00020000;
  return r;
}

// BPRE: the right operand comes already split ("prepared", see prepare_weight_kernel in
// cascmm_api.hip): B[i] points to 16-byte operand slots [plane][K/8][N], the producers copy
// slots to LDS without touching the VALU.  Fast path only, every column staged singly.
template <class TL, int IODT, int FMT, int TERMS, bool FULL, bool BPRE = false>
struct TileGemm {
  typedef Lowp<FMT> LP;
  typedef typename LP::Vec Vec;
  static constexpr int PL = LP::planes(TERMS);   // LDS planes per operand
  typedef LdsLayout<TL, PL> LL;
  typedef ProductSet<TERMS, FULL> PS;
  typedef AccClasses<FMT, TERMS, FULL> AC;
  typedef typename IoType<IODT>::T IoT;
  static constexpr int ES = sizeof(IoT);
  static constexpr int NCLS = AC::kCount;
  static constexpr int A_UNITS = TL::KG * TL::BM;
  static constexpr int Q_UNITS = TL::KG * (TL::BNQ / TL::QN);   // 8(k) x 4(n) (or 8 x 2) blocks of B
  static constexpr int B_UNITS = TL::KG * TL::BNS;         // 8(k) x 1(n) columns of B
  static constexpr int D = TL::DEPTH;
  static_assert(!BPRE || TL::BNQ == 0, "prepared B is staged column by column");
  // 16-bit operands on the fast path: A is fp16 (bf16) data multiplied as one fp16 (bf16) term, so
  // 8 consecutive elements of a row ARE the operand slot: the producers copy 16 bytes, no split
  static constexpr bool RAW16 = IODT != CASCMM_DT_F32;
  static constexpr int BREGS = BPRE ? 4 * PL : 8;            // registers of one B unit in the ring
  // the gated epilogue needs prepared B (columns in any order at no cost) and a consumer wave that
  // owns whole value / gate pairs of 32-column blocks
  static constexpr bool kGluCapable = BPRE && TL::BNQ == 0 && TL::NTL % 2 == 0;
  static __device__ __forceinline__ float gated(float v, float g) { return gated_value(v, g); }
  static constexpr int QN = TL::QN;
  static constexpr int QW = TL::BNQ > 0 ? TL::BNQ / QN : 1;   // blocks per row of the permuted part
  static constexpr int SW = TL::BNS > 0 ? TL::BNS : 1;       // columns of the unpermuted part
  static constexpr int QUADS = TL::BNQ > 0 ? TL::BNQ / 4 : 1;   // groups of four permuted columns

  // ---- producer waves: global -> split -> LDS, one stage per barrier interval -----------------
  // Barrier protocol over the global step sequence g of a workgroup (every wave executes the
  // same number of barriers):
  //   producer:  store(0) B0 store(1) B1 store(2) B2 ...
  //   consumer:           B0 compute(0) B1 compute(1) B2 ...
  // store(g) writes LDS buffer g&1 between B(g-1) and B(g); the last reader of that buffer,
  // compute(g-2), finished before B(g-1), and its first reader, compute(g), starts after B(g).
  // At the end of an item with WK == 2 both sides add three barriers around the reduction of
  // the two K halves, which reuses the stage buffers.
  //
  // ROLE says which staging units a producer wave handles: every kind (kAll), or, when the
  // workgroup has eight producer waves, the 8x4 blocks of B for the first four (kQuads) and A
  // plus the single B columns for the last four (kRest).  Two producer waves per SIMD with
  // different roles keep the VALU busy while the other wave waits on the LDS or load queues.
  enum { kAll = 0, kQuads = 1, kRest = 2 };
  template <int ROLE>
  struct Prod {
    static constexpr bool HAS_A = ROLE != kQuads, HAS_Q = ROLE != kRest, HAS_S = ROLE != kQuads;
    static constexpr int NTR = ROLE == kAll ? TL::NTP : TL::NTP / 2;    // threads of this role
    static constexpr int T0 = ROLE == kRest ? TL::NTP / 2 : 0;          // first producer thread of it
    static constexpr int Q_IT = HAS_Q ? (Q_UNITS + NTR - 1) / NTR : 0;
    // Weighted deal of the A units: when only the first Q_UNITS threads of the role have an 8x4
    // block of B (32 elements, as much as four A units), they get four A units fewer than the
    // other threads, so that every wave stages the same number of elements per K step.
    static constexpr int NQT = (HAS_A && HAS_Q && Q_UNITS < NTR) ? Q_UNITS : 0;   // threads with a B block
    static constexpr int A_LO_NUM = A_UNITS - 4 * (NTR - NQT);
    // (not with twelve waves per workgroup: at three waves per SIMD a wave has 168 registers, and the
    // A_HI-deep ring of the weighted deal makes the producer loop spill)
    static constexpr bool WEIGHTED = NQT > 0 && A_LO_NUM >= 0 && A_LO_NUM % NTR == 0 && NQT % kWave == 0 && TL::NT <= 512;
    static constexpr int A_LO = WEIGHTED ? A_LO_NUM / NTR : 0, A_HI = A_LO + 4;
    static constexpr int A_IT = !HAS_A ? 0 : WEIGHTED ? A_HI : (A_UNITS + NTR - 1) / NTR;
    static constexpr bool A_ALL = !WEIGHTED && A_UNITS % NTR == 0;   // every thread has A_IT valid units
    // A unit number of (thread, iteration), or a number >= A_UNITS when there is none
    static __device__ __forceinline__ int a_unit(int rtid, int it) {
      if constexpr (WEIGHTED) {
        if (rtid < NQT) return it < A_LO ? it * NQT + rtid : A_UNITS;
        return NQT * A_LO + it * (NTR - NQT) + (rtid - NQT);
      } else {
        return rtid + it * NTR;
      }
    }
    static constexpr int B_IT = HAS_S ? (B_UNITS + NTR - 1) / NTR : 0;
    static_assert((A_IT * 2 + Q_IT * 8 + B_IT * (BPRE ? PL : 8)) * D <= 60, "too many loads in flight for the vmcnt counter");

    // one k row of a block of QN consecutive columns: a 16-byte or an 8-byte load
    static __device__ __forceinline__ void load_block(i32x4 rsrc, int voff, int soff, float (&dst)[QN]) {
      if constexpr (QN == 4) {
        const f32x4 v = llvm_raw_buffer_load_v4f32(rsrc, voff, soff, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) dst[i] = v[i];
      } else {
        const f32x2_ld v = llvm_raw_buffer_load_v2f32(rsrc, voff, soff, 0);
        dst[0] = v[0];
        dst[1] = v[1];
      }
    }

    struct Regs {
      float a[A_IT > 0 ? A_IT : 1][8];
      float q[Q_IT > 0 ? Q_IT : 1][8][QN];
      float b[B_IT > 0 ? B_IT : 1][BREGS];
    };

    struct Ctx {
      i32x4 ra, rb;
      int voff_a[A_IT > 0 ? A_IT : 1];   // bytes: row * lda + kg * 8
      int voff_q[Q_IT > 0 ? Q_IT : 1];   // bytes: kg * 8 * ldb + 4 * quad
      int voff_b[B_IT > 0 ? B_IT : 1];   // bytes: kg * 8 * ldb + col
      int lds_a[A_IT > 0 ? A_IT : 1];    // slot index inside a term plane set, -1 if this thread has no such unit
      int lds_q[Q_IT > 0 ? Q_IT : 1];    // slot of column 4*quad (the other three follow at +32, +64, +96)
      int lds_b[B_IT > 0 ? B_IT : 1];
      int ldb_bytes;                     // prepared B: bytes of one k-group row of slots (N * 16)
      int plane_bytes;                   // prepared B: bytes of one plane (K/8 * N * 16)
      float scale_a, scale_b;            // tensor scales 2^e_A, 2^e_B (fp8), else 1
    };

    // LDS slot of every unit this thread stages (fixed for the whole kernel)
    static __device__ __forceinline__ void init_lds(Ctx& c, int rtid) {
#pragma unroll
      for (int it = 0; it < A_IT; ++it) {
        const int u = a_unit(rtid, it);
        const int kg = u % TL::KG, r = u / TL::KG;
        c.lds_a[it] = u < A_UNITS ? kg * LL::kAPlane + (r ^ LL::swz(kg)) : -1;
      }
#pragma unroll
      for (int it = 0; it < Q_IT; ++it) {
        const int u = rtid + it * NTR;
        // column 4 * quad + QN * sub is the block's first; consecutive threads take consecutive
        // quads (consecutive LDS slots), the second halves of the quads follow the first halves
        const int blk = u % QW, kg = u / QW;
        const int quad = blk % QUADS, sub = blk / QUADS;
        c.lds_q[it] = u < Q_UNITS ? kg * LL::kBPlane + (quad >> 5) * 128 + (quad & 31) + QN * sub * 32 : -1;
      }
#pragma unroll
      for (int it = 0; it < B_IT; ++it) {
        const int u = rtid + it * NTR;
        const int n = TL::BNQ + u % SW, kg = u / SW;
        c.lds_b[it] = u < B_UNITS ? kg * LL::kBPlane + n : -1;
      }
    }

    // point the loads at tile (m0, n0) of problem `prob`: buffer descriptors at the tile origin
    // and per-lane offsets with rows / columns clamped to the last valid one
    static __device__ __forceinline__ void set_tile(Ctx& c, const GroupParams& p, int prob, int m0, int n0, int rtid) {
      const IoT* A = (const IoT*)p.A[prob] + (int64_t)m0 * p.lda;
      const IoT* B = (const IoT*)p.B[prob] + n0;
      // bytes from the tile origin to the end of the matrix; rows and columns are also clamped
      // below, so no access relies on the hardware range check
      c.ra = make_rsrc(A, ((int64_t)(p.M - 1 - m0) * p.lda + p.K) * ES);
      c.rb = make_rsrc(B, ((int64_t)(p.K - 1) * p.ldb + (p.N - n0)) * ES);
      c.ldb_bytes = (int)(p.ldb * ES);
      c.plane_bytes = 0;
      if constexpr (BPRE) {
        // the descriptor covers the whole prepared buffer; the tile's column goes into the
        // per-lane offsets (the host checked that the buffer is smaller than 2 GiB)
        const int kgs = (p.K + 7) / 8;
        c.ldb_bytes = p.N * 16;
        c.plane_bytes = kgs * c.ldb_bytes;
        c.rb = make_rsrc(p.B[prob], (int64_t)PL * c.plane_bytes);
      }
      c.scale_a = c.scale_b = 1.f;
      if constexpr (LP::kTensorScaled) {
        if (p.tensor_exps) {
          c.scale_a = __builtin_ldexpf(1.f, p.tensor_exps[2 * prob]);
          c.scale_b = __builtin_ldexpf(1.f, p.tensor_exps[2 * prob + 1]);
        }
      }
      const int last_row = p.M - 1 - m0, last_col = p.N - 1 - n0;
#pragma unroll
      for (int it = 0; it < A_IT; ++it) {
        int u = a_unit(rtid, it);
        u = u < A_UNITS ? u : A_UNITS - 1;
        const int kg = u % TL::KG, r = u / TL::KG;
        const int rc = r < last_row ? r : last_row;
        c.voff_a[it] = (int)((rc * p.lda + kg * 8) * ES);
      }
#pragma unroll
      for (int it = 0; it < Q_IT; ++it) {
        int u = rtid + it * NTR;
        u = u < Q_UNITS ? u : Q_UNITS - 1;
        const int blk = u % QW, kg = u / QW;
        const int quad = blk % QUADS, sub = blk / QUADS;
        const int last_quad = last_col >> 2;  // fast path: N % 4 == 0, a quad is wholly in or out
        const int qc = quad < last_quad ? quad : last_quad;
        c.voff_q[it] = (int)((kg * 8 * p.ldb + 4 * qc + QN * sub) * ES);
      }
#pragma unroll
      for (int it = 0; it < B_IT; ++it) {
        int u = rtid + it * NTR;
        u = u < B_UNITS ? u : B_UNITS - 1;
        const int n = TL::BNQ + u % SW, kg = u / SW;
        const int nc = n < last_col ? n : last_col;
        c.voff_b[it] = BPRE ? kg * c.ldb_bytes + (n0 + nc) * 16 : (int)((kg * 8 * p.ldb + nc) * ES);
      }
    }

    // global -> registers (fast path: fp32, K % BK == 0, 16-byte aligned rows)
    static __device__ __forceinline__ void load_fast(const Ctx& c, int k0, Regs& r) {
      const int soff_a = k0 * ES;
#pragma unroll
      for (int it = 0; it < A_IT; ++it) {
        if (WEIGHTED && c.lds_a[it] < 0) continue;   // (uniform over a wave)
        const f32x4 v0 = llvm_raw_buffer_load_v4f32(c.ra, c.voff_a[it], soff_a, 0);
#pragma unroll
        for (int e = 0; e < 4; ++e) r.a[it][e] = v0[e];
        if constexpr (!RAW16) {
          const f32x4 v1 = llvm_raw_buffer_load_v4f32(c.ra, c.voff_a[it] + 16, soff_a, 0);
#pragma unroll
          for (int e = 0; e < 4; ++e) r.a[it][4 + e] = v1[e];
        }
      }
      if constexpr (BPRE) {
        load_prepared(c, k0, r);
        return;
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int soff_b = (k0 + e) * c.ldb_bytes;
#pragma unroll
        for (int it = 0; it < Q_IT; ++it) {
          load_block(c.rb, c.voff_q[it], soff_b, r.q[it][e]);
        }
#pragma unroll
        for (int it = 0; it < B_IT; ++it) r.b[it][e] = llvm_raw_buffer_load_f32(c.rb, c.voff_b[it], soff_b, 0);
      }
    }

    // prepared B: one 16-byte slot per plane and unit
    static __device__ __forceinline__ void load_prepared_unit(const Ctx& c, int k0, int it, Regs& r) {
      const int soff = (k0 >> 3) * c.ldb_bytes;
#pragma unroll
      for (int pl = 0; pl < PL; ++pl) {
        const f32x4 v = llvm_raw_buffer_load_v4f32(c.rb, c.voff_b[it] + pl * c.plane_bytes, soff, 0);
#pragma unroll
        for (int e = 0; e < 4; ++e) r.b[it][4 * pl + e] = v[e];
      }
    }
    static __device__ __forceinline__ void load_prepared(const Ctx& c, int k0, Regs& r) {
#pragma unroll
      for (int it = 0; it < B_IT; ++it) load_prepared_unit(c, k0, it, r);
    }

    // global -> registers (generic: any dtype, any K, element-wise, bounds-checked)
    static __device__ __forceinline__ void load_generic(const GroupParams& p, int prob, int m0, int n0, int k0, int rtid, Regs& r) {
      const IoT* A = (const IoT*)p.A[prob];
      const IoT* B = (const IoT*)p.B[prob];
#pragma unroll
      for (int it = 0; it < A_IT; ++it) {
        int u = a_unit(rtid, it);
        u = u < A_UNITS ? u : A_UNITS - 1;
        const int kg = u % TL::KG;
        int row = m0 + u / TL::KG;
        row = row < p.M ? row : p.M - 1;
        const int k = k0 + kg * 8;
        const IoT* src = A + (int64_t)row * p.lda + k;
#pragma unroll
        for (int e = 0; e < 8; ++e) r.a[it][e] = (k + e < p.K) ? IoType<IODT>::load(src + e) : 0.f;
      }
#pragma unroll
      for (int it = 0; it < Q_IT; ++it) {
        int u = rtid + it * NTR;
        u = u < Q_UNITS ? u : Q_UNITS - 1;
        const int blk = u % QW, kg = u / QW;
        const int k = k0 + kg * 8;
        const int quad = blk % QUADS, sub = blk / QUADS;
#pragma unroll
        for (int i = 0; i < QN; ++i) {
          int col = n0 + 4 * quad + QN * sub + i;
          col = col < p.N ? col : p.N - 1;
          const IoT* src = B + (int64_t)k * p.ldb + col;
#pragma unroll
          for (int e = 0; e < 8; ++e) r.q[it][e][i] = (k + e < p.K) ? IoType<IODT>::load(src + (int64_t)e * p.ldb) : 0.f;
        }
      }
#pragma unroll
      for (int it = 0; it < B_IT; ++it) {
        int u = rtid + it * NTR;
        u = u < B_UNITS ? u : B_UNITS - 1;
        const int kg = u / SW;
        int col = n0 + TL::BNQ + u % SW;
        col = col < p.N ? col : p.N - 1;
        const int k = k0 + kg * 8;
        const IoT* src = B + (int64_t)k * p.ldb + col;
#pragma unroll
        for (int e = 0; e < 8; ++e) r.b[it][e] = (k + e < p.K) ? IoType<IODT>::load(src + (int64_t)e * p.ldb) : 0.f;
      }
    }

    // registers -> split -> LDS, and refill of the ring slot.
    // Unit by unit: split one unit, write its slots, and right away issue the loads that refill
    // that unit's registers for K step k_next (ISSUE).  Spreading the loads between the VALU
    // batches keeps the texture-address unit busy while the splits run; issued in one burst
    // they would stall the wave on the full address FIFO with no VALU work to overlap.
    template <bool ISSUE, bool RAW = false>
    static __device__ __forceinline__ void restage(const Ctx& c, u32x4* stage, Regs& r, int k_next) {
      u32x4* sb = stage + PL * LL::kATerm;
      const int soff_a = k_next * ES;
#pragma unroll
      for (int it = 0; it < A_IT; ++it) {
        if (A_ALL || c.lds_a[it] >= 0) {
          if constexpr (RAW) {
            const f32x4 v = {r.a[it][0], r.a[it][1], r.a[it][2], r.a[it][3]};
            stage[c.lds_a[it]] = __builtin_bit_cast(u32x4, v);
          } else {
            u32x4 t[PL];
            split8<FMT, TERMS>(r.a[it], t, c.scale_a);
#pragma unroll
            for (int i = 0; i < PL; ++i) stage[i * LL::kATerm + c.lds_a[it]] = t[i];
          }
        }
        if (ISSUE && (!WEIGHTED || c.lds_a[it] >= 0)) {
          const f32x4 v0 = llvm_raw_buffer_load_v4f32(c.ra, c.voff_a[it], soff_a, 0);
#pragma unroll
          for (int e = 0; e < 4; ++e) r.a[it][e] = v0[e];
          if constexpr (!RAW) {
            const f32x4 v1 = llvm_raw_buffer_load_v4f32(c.ra, c.voff_a[it] + 16, soff_a, 0);
#pragma unroll
            for (int e = 0; e < 4; ++e) r.a[it][4 + e] = v1[e];
          }
        }
      }
#pragma unroll
      for (int it = 0; it < Q_IT; ++it) {
        if (Q_UNITS % NTR == 0 || c.lds_q[it] >= 0) {
#pragma unroll
          for (int i = 0; i < QN; ++i) {
            float x[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) x[e] = r.q[it][e][i];
            u32x4 t[PL];
            split8<FMT, TERMS>(x, t, c.scale_b);
#pragma unroll
            for (int tt = 0; tt < PL; ++tt) sb[tt * LL::kBTerm + c.lds_q[it] + i * 32] = t[tt];
          }
        }
        if (ISSUE) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            load_block(c.rb, c.voff_q[it], (k_next + e) * c.ldb_bytes, r.q[it][e]);
          }
        }
      }
#pragma unroll
      for (int it = 0; it < B_IT; ++it) {
        if constexpr (BPRE) {
          if (B_UNITS % NTR == 0 || c.lds_b[it] >= 0) {
#pragma unroll
            for (int i = 0; i < PL; ++i) {
              const f32x4 v = {r.b[it][4 * i], r.b[it][4 * i + 1], r.b[it][4 * i + 2], r.b[it][4 * i + 3]};
              sb[i * LL::kBTerm + c.lds_b[it]] = __builtin_bit_cast(u32x4, v);
            }
          }
          if (ISSUE) load_prepared_unit(c, k_next, it, r);
        } else {
          if (B_UNITS % NTR == 0 || c.lds_b[it] >= 0) {
            u32x4 t[PL];
            split8<FMT, TERMS>(r.b[it], t, c.scale_b);
#pragma unroll
            for (int i = 0; i < PL; ++i) sb[i * LL::kBTerm + c.lds_b[it]] = t[i];
          }
          if (ISSUE) {
#pragma unroll
            for (int e = 0; e < 8; ++e)
              r.b[it][e] = llvm_raw_buffer_load_f32(c.rb, c.voff_b[it], (k_next + e) * c.ldb_bytes, 0);
          }
        }
      }
    }

    // The producer walks the global step sequence gs = 0 .. items * ktiles - 1 of this
    // workgroup (item j = work item blockIdx.x + j * gridDim.x, step gs % ktiles of it).  The
    // prefetch ring runs across item boundaries, so the first operands of the next tile are
    // already in registers while the consumers finish the current one and store its result.
    template <bool FAST>
    static __device__ __forceinline__ void loop(const GroupParams& p, u32x4* lds, int ktiles, int nitems) {
      static_assert(FAST || !BPRE, "prepared B has no bounds-checked loader");
      constexpr bool RAW = FAST && RAW16;
      static_assert(!RAW || (BPRE && TERMS == 1 &&
                             ((IODT == CASCMM_DT_F16 && FMT == CASCMM_FMT_FP16) || (IODT == CASCMM_DT_BF16 && FMT == CASCMM_FMT_BF16))),
                    "16-bit operands on the fast path: one term of their own format, prepared B");
      const int rtid = threadIdx.x - TL::NCW * kWave - T0;
      const int tiles = p.tiles_m * p.tiles_n;
      const int gsteps = nitems * ktiles;
      Ctx ctx;
      init_lds(ctx, rtid);
      Regs ring[D];
      // Loads for the next global step: target() is called once per global step, in order
      // (0, 1, 2 ... gsteps - 1), and keeps its position in counters, so the K loop holds no
      // integer division; the item is decoded (and the descriptors retargeted) on its first step.
      int next_item = 0, next_kt = 0, prob = 0, m0 = 0, n0 = 0, kbase = 0;
      auto target = [&](int /* g */) {
        if (next_kt == 0) {
          int item = blockIdx.x + next_item * gridDim.x;
          const int split = item / (p.count * tiles);   // K split: items are (split, problem, tile)
          item -= split * (p.count * tiles);
          kbase = split * ktiles * TL::BK;
          prob = item / tiles;
          int tm, tn;
          tile_coords(item - prob * tiles, p.tiles_m, p.tiles_n, tm, tn);
          m0 = tm * TL::BM;
          n0 = tn * TL::BN;
          set_tile(ctx, p, prob, m0, n0, rtid);
        }
        const int k0 = kbase + next_kt * TL::BK;
        if (++next_kt == ktiles) {
          next_kt = 0;
          ++next_item;
        }
        return k0;
      };
      auto issue = [&](int g, Regs& r) {
        const int k0 = target(g);
        if (FAST) load_fast(ctx, k0, r);
        else load_generic(p, prob, m0, n0, k0, rtid, r);
      };
      // after the last step of an item the consumers reduce their K halves through LDS (WK == 2):
      // three barriers during which nothing may be staged (called once per staged step, in order)
      int staged_kt = 0;
      auto item_end = [&](int /* g */) {
        if (TL::WK > 1) {
          if (++staged_kt == ktiles) {
            staged_kt = 0;
            __syncthreads();
            __syncthreads();
            __syncthreads();
          }
        }
      };
#pragma unroll
      for (int d = 0; d < D; ++d)
        if (d < gsteps) issue(d, ring[d]);
      int g = 0;
      for (; g + 2 * D <= gsteps; g += D) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
          if (FAST) {
            const int k_next = target(g + d + D);
            restage<true, RAW>(ctx, lds + ((g + d) & 1) * LL::kStage, ring[d], k_next);
          } else {
            restage<false, RAW>(ctx, lds + ((g + d) & 1) * LL::kStage, ring[d], 0);
            issue(g + d + D, ring[d]);
          }
          __syncthreads();
          item_end(g + d);
        }
      }
#pragma unroll
      for (int dd = 0; dd < 2 * D; ++dd) {
        const int d = dd % D;
        if (g + dd < gsteps) {
          if (FAST && g + dd + D < gsteps) {
            const int k_next = target(g + dd + D);
            restage<true, RAW>(ctx, lds + ((g + dd) & 1) * LL::kStage, ring[d], k_next);
          } else {
            restage<false, RAW>(ctx, lds + ((g + dd) & 1) * LL::kStage, ring[d], 0);
            if (g + dd + D < gsteps) issue(g + dd + D, ring[d]);
          }
          __syncthreads();
          item_end(g + dd);
        }
      }
    }
  };

  // ---- LDS -> MFMA ----------------------------------------------------------------------
  static __device__ __forceinline__ void compute(const u32x4* stage, int wm0, int wn0, int wk,
                                                 f32x16 (&acc)[NCLS][TL::MT][TL::NTL]) {
    const int lane = threadIdx.x & 63, l31 = lane & 31, g = lane >> 5;
    const u32x4* sa = stage;
    const u32x4* sb = stage + PL * LL::kATerm;
#pragma unroll
    for (int kk = 0; kk < TL::KSUB / TL::WK; ++kk) {
      const int ks = kk * TL::WK + wk;
      const int kg = ks * 2 + g;
      u32x4 a[PL][TL::MT], b[PL][TL::NTL];
#pragma unroll
      for (int i = 0; i < PL; ++i) {
#pragma unroll
        for (int mi = 0; mi < TL::MT; ++mi)
          a[i][mi] = sa[i * LL::kATerm + kg * LL::kAPlane + wm0 + mi * 32 + (l31 ^ LL::swz(kg))];
#pragma unroll
        for (int ni = 0; ni < TL::NTL; ++ni)
          b[i][ni] = sb[i * LL::kBTerm + kg * LL::kBPlane + wn0 + ni * 32 + l31];
      }
      // smallest products first; consecutive MFMAs go to different accumulators
#pragma unroll
      for (int s = 2 * TERMS - 2; s >= 0; --s)
#pragma unroll
        for (int i = 0; i < TERMS; ++i) {
          const int j = s - i;
          if (j < 0 || j >= TERMS || !PS::keep(i, j)) continue;
          const int cls = AC::index(s);
#pragma unroll
          for (int mi = 0; mi < TL::MT; ++mi)
#pragma unroll
            for (int ni = 0; ni < TL::NTL; ++ni)
              acc[cls][mi][ni] = LP::mfma(LP::operand(a[LP::plane(i)][mi], i), LP::operand(b[LP::plane(j)][ni], j),
                                          acc[cls][mi][ni]);
        }
    }
  }

  // ---- consumer waves: LDS -> MFMA, then the epilogue, item after item --------------------------
  static __device__ __forceinline__ void consumer(const GroupParams& p, u32x4* lds, int ktiles, int nitems, int wave) {
    const int wk = wave / (TL::WM * TL::WN);
    const int wmn = wave - wk * (TL::WM * TL::WN);
    const int wm0 = (wmn / TL::WN) * TL::WTM, wn0 = (wmn % TL::WN) * TL::WTN;
    const int tiles = p.tiles_m * p.tiles_n;
    constexpr int kChunkSteps = (AC::kChunkK / TL::BK) > 0 ? (AC::kChunkK / TL::BK) : 1;
    int g = 0;
    for (int j = 0; j < nitems; ++j) {
      int item = blockIdx.x + j * gridDim.x;
      const int split = item / (p.count * tiles);
      item -= split * (p.count * tiles);
      const int prob = item / tiles;
      int tm, tn;
      tile_coords(item - prob * tiles, p.tiles_m, p.tiles_n, tm, tn);
      const int m0 = tm * TL::BM, n0 = tn * TL::BN;

      f32x16 acc[NCLS][TL::MT][TL::NTL];
#pragma unroll
      for (int c = 0; c < NCLS; ++c)
#pragma unroll
        for (int mi = 0; mi < TL::MT; ++mi)
#pragma unroll
          for (int ni = 0; ni < TL::NTL; ++ni)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[c][mi][ni][e] = 0.f;

      // Blocked accumulation for the cascades whose error sits at the fp32 rounding floor: the
      // big class-0 sum is collected in chunks of kChunkK and the chunks are added into a master
      // accumulator, so the chunk sums round at a fraction of the final magnitude and the master
      // rounds K / kChunkK times instead of K / 16 times.
      f32x16 master[AC::kChunked ? TL::MT : 1][AC::kChunked ? TL::NTL : 1];
      if constexpr (AC::kChunked) {
#pragma unroll
        for (int mi = 0; mi < TL::MT; ++mi)
#pragma unroll
          for (int ni = 0; ni < TL::NTL; ++ni)
#pragma unroll
            for (int e = 0; e < 16; ++e) master[mi][ni][e] = 0.f;
      }

      for (int kt = 0; kt < ktiles; ++kt, ++g) {
        __syncthreads();
        compute(lds + (g & 1) * LL::kStage, wm0, wn0, wk, acc);
        if constexpr (AC::kChunked) if ((kt % kChunkSteps) == kChunkSteps - 1) {
#pragma unroll
          for (int mi = 0; mi < TL::MT; ++mi)
#pragma unroll
            for (int ni = 0; ni < TL::NTL; ++ni) {
              master[mi][ni] += acc[0][mi][ni];
#pragma unroll
              for (int e = 0; e < 16; ++e) acc[0][mi][ni][e] = 0.f;
            }
        }
      }
      if constexpr (AC::kChunked) {
#pragma unroll
        for (int mi = 0; mi < TL::MT; ++mi)
#pragma unroll
          for (int ni = 0; ni < TL::NTL; ++ni) acc[0][mi][ni] += master[mi][ni];
      }
      finish(p, lds, prob, split, m0, n0, wk, wmn, wm0, wn0, acc);
    }
  }

  // ---- end of an item: fold, reduce the K halves, store -----------------------------------------
  static __device__ __forceinline__ void finish(const GroupParams& p, u32x4* lds, int prob, int split, int m0, int n0, int wk, int wmn,
                                                int wm0, int wn0, f32x16 (&acc)[NCLS][TL::MT][TL::NTL]) {
    // fold the scale classes (smallest first), then the cross-wave-group reduction (WK == 2):
    // group 1 parks its tile in LDS, group 0 adds it
    f32x16 res[TL::MT][TL::NTL];
    float out_scale = 1.f;   // undoes the tensor scales of both operands (fp8)
    if constexpr (LP::kTensorScaled) {
      if (p.tensor_exps) out_scale = __builtin_ldexpf(1.f, -(p.tensor_exps[2 * prob] + p.tensor_exps[2 * prob + 1]));
    }
#pragma unroll
    for (int mi = 0; mi < TL::MT; ++mi)
#pragma unroll
      for (int ni = 0; ni < TL::NTL; ++ni) {
        f32x16 v = acc[NCLS - 1][mi][ni];
#pragma unroll
        for (int c = NCLS - 2; c >= 0; --c) v = v * AC::kFoldScale + acc[c][mi][ni];
        if constexpr (LP::kTensorScaled) v = v * out_scale;
        res[mi][ni] = v;
      }
    const int lane = threadIdx.x & 63, l31 = lane & 31, g = lane >> 5;
    if (TL::WK > 1) {
      // the reduction buffer overlays the stage buffers: barrier 1 = every consumer is done
      // reading them, barrier 2 = the parked tiles are visible, barrier 3 = they have been read
      // (the producers, which execute the same three barriers, may stage again)
      f32x4* red = (f32x4*)lds + wmn * (TL::MT * TL::NTL * 4 * 64) + lane;
      __syncthreads();
      if (wk == 1) {
#pragma unroll
        for (int mi = 0; mi < TL::MT; ++mi)
#pragma unroll
          for (int ni = 0; ni < TL::NTL; ++ni)
#pragma unroll
            for (int q = 0; q < 4; ++q)
              red[((mi * TL::NTL + ni) * 4 + q) * 64] =
                  (f32x4){res[mi][ni][4 * q], res[mi][ni][4 * q + 1], res[mi][ni][4 * q + 2], res[mi][ni][4 * q + 3]};
      }
      __syncthreads();
      if (wk == 0) {
#pragma unroll
        for (int mi = 0; mi < TL::MT; ++mi)
#pragma unroll
          for (int ni = 0; ni < TL::NTL; ++ni)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const f32x4 o = red[((mi * TL::NTL + ni) * 4 + q) * 64];
#pragma unroll
              for (int e = 0; e < 4; ++e) res[mi][ni][4 * q + e] += o[e];
            }
      }
      __syncthreads();
      if (wk == 1) return;
    }

    // epilogue: of every 32x32 tile a lane holds column lane%32 and rows 8*q + 4*(lane/32) + e
    IoT* C = (IoT*)p.C[prob];
    const IoT* bias = (const IoT*)p.bias[prob];
    int64_t ldc = p.ldc;
    if (p.k_splits > 1) {
      // K split (fp32 only): this item's partial result goes to the workspace, [split][M][N];
      // splitk_reduce_kernel adds the splits in order and applies the bias
      C = (IoT*)p.workspace + ((int64_t)(prob * p.k_splits + split) * p.M) * p.N;
      bias = nullptr;
      ldc = p.N;
    }
    const bool interior = (m0 + TL::BM <= p.M) && (n0 + TL::BN <= p.N) && ldc * (int64_t)(TL::BM * ES) < 0x7FFFFFFF;
    // Column blocks of this wave that hold permuted columns come in runs of RUN blocks of one
    // 128-column group: block b of the tile (b = wn0/32 + ni), lane l31 <-> column
    // 128*(b/4) + 4*l31 + b%4.
    constexpr int NQ = (TL::BNQ == 0) ? 0 : (TL::WN == 1 ? TL::BNQ / 32 : TL::NTL);
    constexpr int RUN = (NQ % 4 == 0) ? 4 : 2;
    const int b0 = wn0 >> 5;
    if constexpr (kGluCapable) if (p.glu) {
      // gated epilogue: blocks 2j (value) and 2j + 1 (gate) of this wave, same lane and register,
      // make block j of the output, whose row has N/2 columns
      const int half = p.N >> 1;
      const int oc0 = (n0 + wn0) >> 1;   // first output column of this wave
      if (interior) {
        const i32x4 rc = make_rsrc(C + (int64_t)(m0 + wm0) * ldc, 0x7FFFFFFF);
        const int ldc_bytes = (int)ldc * ES;
#pragma unroll
        for (int nj = 0; nj < TL::NTL / 2; ++nj) {
          const int col = oc0 + nj * 32 + l31;
          const int voff = g * 4 * ldc_bytes + col * ES;
          const float bv = bias ? IoType<IODT>::load(bias + col) : 0.f, bg = bias ? IoType<IODT>::load(bias + half + col) : 0.f;
#pragma unroll
          for (int mi = 0; mi < TL::MT; ++mi)
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                const float y = gated(res[mi][2 * nj][4 * q + e] + bv, res[mi][2 * nj + 1][4 * q + e] + bg);
                const int soff = (mi * 32 + q * 8 + e) * ldc_bytes;
                if constexpr (IODT == CASCMM_DT_F32) llvm_raw_buffer_store_f32(y, rc, voff, soff, kResultStoreAux);
                else llvm_raw_buffer_store_i16(__builtin_bit_cast(short, (IoT)y), rc, voff, soff, kResultStoreAux);
              }
        }
        return;
      }
#pragma unroll
      for (int nj = 0; nj < TL::NTL / 2; ++nj) {
        const int col = oc0 + nj * 32 + l31;
        if (col >= half) continue;
        const float bv = bias ? IoType<IODT>::load(bias + col) : 0.f, bg = bias ? IoType<IODT>::load(bias + half + col) : 0.f;
#pragma unroll
        for (int mi = 0; mi < TL::MT; ++mi) {
          const int row0 = m0 + wm0 + mi * 32 + g * 4;
          IoT* dst = C + (int64_t)row0 * ldc + col;
#pragma unroll
          for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (row0 + q * 8 + e < p.M)
                IoType<IODT>::store(dst + (int64_t)(q * 8 + e) * ldc,
                                    gated(res[mi][2 * nj][4 * q + e] + bv, res[mi][2 * nj + 1][4 * q + e] + bg));
        }
      }
      return;
    }
    if (IODT == CASCMM_DT_F32 && interior && (ldc & 3) == 0 && (((uintptr_t)C) & 15) == 0 &&
        (bias == nullptr || (((uintptr_t)bias) & 15) == 0)) {
      // whole tile inside C: buffer stores, the row as a scalar offset, nothing to mask
      const i32x4 rc = make_rsrc(C + (int64_t)(m0 + wm0) * ldc + n0, 0x7FFFFFFF);
      const int ldc_bytes = (int)ldc * ES;
#pragma unroll
      for (int r0 = 0; r0 < NQ; r0 += RUN) {
        const int b = b0 + r0;
        const int col = (b >> 2) * 128 + 4 * l31 + (b & 3);
        const int voff = g * 4 * ldc_bytes + col * ES;
        float bv[RUN];
#pragma unroll
        for (int i = 0; i < RUN; ++i) bv[i] = bias ? IoType<IODT>::load(bias + n0 + col + i) : 0.f;
#pragma unroll
        for (int mi = 0; mi < TL::MT; ++mi)
#pragma unroll
          for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int soff = (mi * 32 + q * 8 + e) * ldc_bytes;
              if constexpr (RUN == 4) {
                const f32x4 v = {res[mi][r0][4 * q + e] + bv[0], res[mi][r0 + 1][4 * q + e] + bv[1],
                                 res[mi][r0 + 2][4 * q + e] + bv[2], res[mi][r0 + 3][4 * q + e] + bv[3]};
                llvm_raw_buffer_store_v4f32(v, rc, voff, soff, kResultStoreAux);
              } else {
                const f32x2 v = {res[mi][r0][4 * q + e] + bv[0], res[mi][r0 + 1][4 * q + e] + bv[1]};
                llvm_raw_buffer_store_v2f32(v, rc, voff, soff, kResultStoreAux);
              }
            }
      }
      // unpermuted blocks: a store instruction writes two full 128-byte row segments
#pragma unroll
      for (int ni = NQ; ni < TL::NTL; ++ni) {
        const int col = wn0 + ni * 32 + l31;
        const int voff = g * 4 * ldc_bytes + col * ES;
        const float bv = bias ? IoType<IODT>::load(bias + n0 + col) : 0.f;
#pragma unroll
        for (int mi = 0; mi < TL::MT; ++mi)
#pragma unroll
          for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int e = 0; e < 4; ++e)
              llvm_raw_buffer_store_f32(res[mi][ni][4 * q + e] + bv, rc, voff, (mi * 32 + q * 8 + e) * ldc_bytes, kResultStoreAux);
      }
      return;
    }
    if constexpr (IODT != CASCMM_DT_F32 && NQ == 0) if (interior) {
      // 16-bit output, whole tile inside C: 2-byte buffer stores, the row as a scalar offset
      const i32x4 rc = make_rsrc(C + (int64_t)(m0 + wm0) * ldc + n0, 0x7FFFFFFF);
      const int ldc_bytes = (int)ldc * ES;
#pragma unroll
      for (int ni = 0; ni < TL::NTL; ++ni) {
        const int col = wn0 + ni * 32 + l31;
        const int voff = g * 4 * ldc_bytes + col * ES;
        const float bv = bias ? IoType<IODT>::load(bias + n0 + col) : 0.f;
#pragma unroll
        for (int mi = 0; mi < TL::MT; ++mi)
#pragma unroll
          for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const IoT h = (IoT)(res[mi][ni][4 * q + e] + bv);
              llvm_raw_buffer_store_i16(__builtin_bit_cast(short, h), rc, voff, (mi * 32 + q * 8 + e) * ldc_bytes, kResultStoreAux);
            }
      }
      return;
    }
#pragma unroll
    for (int ni = 0; ni < TL::NTL; ++ni) {
      const int b = b0 + ni;
      const int col = n0 + (ni < NQ ? (b >> 2) * 128 + 4 * l31 + (b & 3) : wn0 + ni * 32 + l31);
      if (col >= p.N) continue;
      const float bv = bias ? IoType<IODT>::load(bias + col) : 0.f;
#pragma unroll
      for (int mi = 0; mi < TL::MT; ++mi) {
        const int row0 = m0 + wm0 + mi * 32 + g * 4;
        IoT* dst = C + (int64_t)row0 * ldc + col;
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (row0 + q * 8 + e < p.M) IoType<IODT>::store(dst + (int64_t)(q * 8 + e) * ldc, res[mi][ni][4 * q + e] + bv);
          }
      }
    }
  }

  template <bool FAST>
  static __device__ __forceinline__ void run(const GroupParams& p, u32x4* lds) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int splits = p.k_splits > 1 ? p.k_splits : 1;
    const int ktiles = (p.K + TL::BK - 1) / TL::BK / splits;   // K steps of one item (the host picks a divisor)
    const int total = splits * p.count * p.tiles_m * p.tiles_n;
    const int nitems = (total - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;  // grid <= total
    if (wave < TL::NCW) {
      consumer(p, lds, ktiles, nitems, wave);
    } else if constexpr (TL::NP < 8 || TL::BNQ == 0) {
      Prod<kAll>::template loop<FAST>(p, lds, ktiles, nitems);
    } else {
      if (wave < TL::NCW + TL::NP / 2) Prod<kQuads>::template loop<FAST>(p, lds, ktiles, nitems);
      else Prod<kRest>::template loop<FAST>(p, lds, ktiles, nitems);
    }
  }
};

template <class TL, int IODT, int FMT, int TERMS, bool FULL, bool FAST, bool BPRE = false>
__global__ __launch_bounds__(TL::NT) void cascmm_tile_kernel(const GroupParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char cascmm_smem[];
  TileGemm<TL, IODT, FMT, TERMS, FULL, BPRE>::template run<FAST>(p, (u32x4*)cascmm_smem);
}

}  // namespace cascmm
