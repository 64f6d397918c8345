// Two-term bf16 cascade on a prepared right operand with K split over the waves of a workgroup
// (gfx950): the kernel of the mid-size Linear layers and of the second GEMM of a feed-forward block.
//
// The right operand comes as MFMA operand slots (cascmm_prepare_weight: 16 bytes = 8 k of one column
// of one term, [term][K/8][N]): a lane's operand is one 16-byte load and 32 consecutive lanes read 512
// contiguous bytes, so B needs no transposition through LDS.  One workgroup computes a 64 x 160 tile of
// C; its four waves split K: wave w takes the 16-k stages w, w + 4, w + 8, ... (raw left operand: the pairs
// of stages w, w + 4, ...) and owns the whole tile (ten 32 x 32 accumulator blocks) over them.  Nothing is shared between waves until the end, so every
// wave streams its own operands, B straight into registers four stages deep, and the main loop has no
// barrier.  A 2048 x 1280 result is 256 tiles, one per CU, whatever K is: no partial results through
// memory, no second kernel.  At the end the four partial tiles meet in LDS: every wave owns two or three
// of the ten blocks, receives the other waves' partial sums of them and adds the four in wave order
// (deterministic), then stores its blocks with the bias.
//
// The left operand comes in one of two forms:
//   ARAW = 0: operand slots as well, [term][K/8][M] (written by the gated store of the preceding GEMM
//     or by cascmm_prepare_left): loaded like B, straight into registers; no LDS access and no VALU
//     work in the loop.  The order of k inside a 16-k stage is whatever the two slot buffers agree on.
//   ARAW = 1: raw fp32 rows.  A pair of stages, 64 rows x 128 bytes (whole lines: with 64 bytes per row the
//     L1 fetched every line of A twice), goes to a private LDS ring of the wave without passing registers
//     (eight `buffer_load ... lds` of 1 KB, four per stage: eight consecutive lanes fetch the eight 16-byte
//     chunks of a row, rotated by row / 2 so that fragment reads spread over all banks), six stages ahead;
//     the fragments of the next stage are read and split in registers between the MFMAs of the current one.
//
// What bounds it: a workgroup pulls (64 + 160) x 4 bytes per k through its CU's vector memory path,
// which for 256 CUs is 84 % of what the eight L2s can deliver while the MFMAs of that k take as long; with
// both operands raw (cascmm_rawk_kernel below) the two splits fill the issue slots beside the MFMAs first.
#pragma once
#include <type_traits>

#include "cascmm_wavek_kernel.h"

namespace cascmm {

// Host-checked: K % 16 == 0, K >= 16 (raw A: K % 32 == 0), the slot buffers 16-byte aligned and below 2 GiB,
// raw A 16-byte aligned with lda % 4 == 0 and M * lda * 4 below 2 GiB, C rows addressable with 32-bit
// byte offsets inside a tile.
template <int ARAW>
__global__ __launch_bounds__(SlotK::NT) __attribute__((amdgpu_waves_per_eu(1, 1))) void cascmm_slotk_kernel(const SlotKParams p) {
  typedef SlotK T;
  extern __shared__ __attribute__((aligned(1024))) unsigned char slotk_smem[];
  const int tid = threadIdx.x, lane = tid & 63, l31 = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Tile order: every XCD (its own L2; workgroup ids are dealt to the XCDs round-robin) gets one
  // contiguous range of tile ids, and ids walk GROUP_M tile rows down before moving one tile to the right:
  // a tile's B slots are 2.5 times its A slots, so the block of tiles that share an L2 is taller than wide.
  int tm, tn;
  tile_coords((int)blockIdx.x, p.tiles_m, p.tiles_n, tm, tn, p.group_m);
  const int m0 = tm * T::BM, n0 = tn * T::BN;
  const int kgroups = p.K >> 3;
  const int ksteps = p.K >> 4;
  // Which 16-k stages of the problem a wave owns.  A as slots: every fourth one, own stage i = stage
  // wave + 4 i.  A raw: every fourth PAIR of stages, own stage i = stage 8 (i / 2) + 2 wave + i % 2, so that
  // what the wave fetches of a row for a pair is one whole 128-byte line (with every fourth stage it was half
  // a line, and the L1 fetched the whole line for either half: 1.8 requests per line of A, counted).
  // n_own: the number of own stages, 0 for the last waves of a very short K (they add zeros).
  const int n_own = ARAW ? 2 * (ksteps >> 3) + (((ksteps & 7) - 2 * wave) < 0 ? 0 : ((ksteps & 7) - 2 * wave) > 2 ? 2 : ((ksteps & 7) - 2 * wave))
                         : (ksteps - wave + T::NW - 1) / T::NW;
  auto stage_of = [&](int i) { return ARAW ? 8 * (i >> 1) + 2 * wave + (i & 1) : wave + T::NW * i; };
  // The loop below runs in trips of D stages and has no branch inside a trip (a branch costs the compiler
  // its count of the loads in flight, and it then waits for all of them).  A wave whose number of stages is
  // not a multiple of D runs up to D - 1 stages past its last one: their slot loads point beyond the end of
  // the buffers and return zeros, whose products add nothing (raw A: finite values of the problem's first
  // stage, times the zero slots of B).

  // ---- right operand: lane (l31, g) reads k group 2 step + g, column block ni 512 bytes further ----
  const i32x4 rb = make_rsrc(p.b_slots, (int64_t)2 * kgroups * p.N * 16);
  const int vb = (g * p.N + n0 + l31) * 16;
  const int b_term = kgroups * p.N * 16;   // from term 0 to term 1
  const int b_step = 2 * p.N * 16;         // from one 16-k stage to the next
  u32x4 Br[T::D][T::NTL][2];               // [ring buffer][column block][term]
  const int b_end = 2 * b_term;            // the buffer's size: every offset from there on is outside
  auto issue_b = [&](int i, int buf, int ni) {
    const int base = i < n_own ? stage_of(i) * b_step : b_end;
#pragma unroll
    for (int t = 0; t < 2; ++t)
      Br[buf][ni][t] = __builtin_bit_cast(u32x4, llvm_raw_buffer_load_v4f32(rb, vb + ni * 512, base + t * b_term, 0));
  };

  // ---- left operand as slots ------------------------------------------------------------------------
  const i32x4 ra = make_rsrc(p.a, ARAW ? (int64_t)16 : (int64_t)2 * kgroups * p.M * 16);
  const int va = (g * p.M + m0 + l31) * 16;
  const int a_term = kgroups * p.M * 16, a_step = 2 * p.M * 16;
  u32x4 Ar[ARAW ? 2 : T::D][T::MT][2];     // slots: [ring buffer][row block][term]; raw: [stage parity] after the split
  auto issue_a1 = [&](int i, int buf, int mi, int t) {
    const int base = i < n_own ? stage_of(i) * a_step : 2 * a_term;
    Ar[buf][mi][t] = __builtin_bit_cast(u32x4, llvm_raw_buffer_load_v4f32(ra, va + mi * 512, base + t * a_term, 0));
  };

  // ---- left operand raw -----------------------------------------------------------------------------
  // rows past M read as zero: the buffer ends with row M - 1
  const int64_t a_bytes = ((int64_t)(p.M - 1) * p.lda + p.K) * 4;
  const __amdgpu_buffer_rsrc_t rar =
      __builtin_amdgcn_make_buffer_rsrc((void*)p.a, 0, ARAW ? (int)(a_bytes > 0x7FFFFFFF ? 0x7FFFFFFF : a_bytes) : 0, 0x00020000);
  unsigned char* ring = slotk_smem + wave * T::RING;
  // A pair of stages in LDS: 64 rows x 128 bytes (eight 16-byte chunks of 4 k).  Load j of a pair (0 .. 7)
  // brings rows 8 j + lane / 8; position pos of a row holds chunk (pos - row / 2) mod 8, which spreads the
  // fragment reads of 16 consecutive rows over all banks.  (row / 2) mod 8 = (4 j + lane / 16) mod 8: two
  // offsets per lane, by the parity of j.  K % 32 == 0 (host-checked for raw A), so a wave's pairs are whole.
  int dma_voff[2];
#pragma unroll
  for (int jp = 0; jp < 2; ++jp)
    dma_voff[jp] = (int)(((int64_t)(m0 + (lane >> 3)) * p.lda + (((lane & 7) - (4 * jp + (lane >> 4))) & 7) * 4) * 4);
  const int dma_rows8 = (int)p.lda * 32;   // bytes from one load's rows to the next one's
  // the part ni (0 .. 3) of own stage i's share of its pair's loads: load 4 sp + ni of pair i / 2, sp = i % 2
  // (passed separately: a constant where i is not); past the wave's last pair: the problem's first pair
  // (finite values for the zero slots of B to multiply, whatever lies beyond K)
  // The four loads of a stage go to consecutive kilobytes of LDS: one M0 and one scalar offset for the four, the
  // kilobytes as the instruction's immediate offset, which the lane offset takes back out of the memory address
  // (lda >= 32, so it stays non-negative; the sum the range check sees is the same).
  int dma_v[4];
#pragma unroll
  for (int ni = 0; ni < 4; ++ni) dma_v[ni] = dma_voff[ni & 1] + ni * (dma_rows8 - 1024);
  auto dma_a = [&](int i, int ni, int sp) {
    const int q = i >> 1;
    const int koff = (2 * q < n_own ? stage_of(2 * q) * (T::BK * 4) : 0) + 4 * sp * dma_rows8;
    wavek_load_lds_kb(rar, ring + (q & (T::RA / 2 - 1)) * (2 * T::A_STAGE) + sp * 4096, dma_v[ni], koff, ni);
  };
  // fragment of lane (l31, g), row block mi, stage parity s: row 32 mi + l31, chunks 4 s + 2 g and 4 s + 2 g + 1
  // at their rotated places
  int a_frag[2][2];
#pragma unroll
  for (int sp = 0; sp < 2; ++sp)
#pragma unroll
    for (int x = 0; x < 2; ++x) a_frag[sp][x] = l31 * 128 + ((4 * sp + 2 * g + x + (l31 >> 1)) & 7) * 16;
  f32x4 X[T::MT][2];   // raw fragments of the next stage on their way to the split
  auto read_a = [&](int i, int mi, int sp) {   // sp = i % 2
    const unsigned char* st = ring + ((i >> 1) & (T::RA / 2 - 1)) * (2 * T::A_STAGE) + mi * 4096;
    X[mi][0] = *(const f32x4*)(st + a_frag[sp][0]);
    X[mi][1] = *(const f32x4*)(st + a_frag[sp][1]);
  };
  auto split_a = [&](int buf, int mi) {
    float r[8] = {X[mi][0][0], X[mi][0][1], X[mi][0][2], X[mi][0][3], X[mi][1][0], X[mi][1][1], X[mi][1][2], X[mi][1][3]};
    u32x4 t[2];
    split8<CASCMM_FMT_BF16, 2>(r, t);
    Ar[buf][mi][0] = t[0];
    Ar[buf][mi][1] = t[1];
  };

  // ---- prologue ---------------------------------------------------------------------------------------
  // B: stages 0 .. D - 2 whole, of stage D - 1 the column blocks 0 .. 3 (its last column block is loaded
  // during stage 0, like that of every later stage: see the loop).  A as slots: stages 0 .. D - 2.
  // A raw: stages 0 .. AHEAD - 1 (three pairs) FIRST, then stage 0 of B, then the rest: the wait below names
  // exactly the rest, so everything the first AHEAD - 1 stages read from LDS has landed when the loop starts
  // (later stages: see the wait at the top of a stage).
  constexpr int AHEAD = T::RA - 2;   // raw A: stage i + AHEAD's share of its pair is requested during stage i
  static_assert(AHEAD % 2 == 0, "a stage and the one AHEAD of it sit at the same place of their pairs");
  f32x16 acc[T::MT][T::NTL];
  if (ARAW) {
#pragma unroll
    for (int d = 0; d < AHEAD; ++d)
#pragma unroll
      for (int j = 0; j < 4; ++j) dma_a(d, j, d & 1);
#pragma unroll
    for (int ni = 0; ni < T::NTL; ++ni) issue_b(0, 0, ni);
    __builtin_amdgcn_sched_barrier(0);   // (the wait below counts on everything above being older than everything below)
  }
#pragma unroll
  for (int d = ARAW ? 1 : 0; d < T::D; ++d) {
#pragma unroll
    for (int ni = 0; ni < T::NTL; ++ni)
      if (d < T::D - 1 || ni < T::NTL - 1) issue_b(d, d, ni);
    if (!ARAW && d < T::D - 1) {
#pragma unroll
      for (int x = 0; x < 4; ++x) issue_a1(d, d, x >> 1, x & 1);
    }
  }
#pragma unroll
  for (int mi = 0; mi < T::MT; ++mi)
#pragma unroll
    for (int ni = 0; ni < T::NTL; ++ni)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[mi][ni][e] = 0.f;
  if (ARAW) {
    constexpr int LATER = (T::D - 2) * 2 * T::NTL + 2 * (T::NTL - 1);   // 28: B of stages 1 .. D - 1
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0x0F70 | (LATER & 0xF) | ((LATER >> 4) << 14));
#pragma unroll
    for (int mi = 0; mi < T::MT; ++mi) read_a(0, mi, 0);
#pragma unroll
    for (int mi = 0; mi < T::MT; ++mi) split_a(0, mi);
  }

  auto mfma = [&](u32x4 a, u32x4 b, f32x16 c) -> f32x16 {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  };
  // Stage i multiplies B from ring buffer i % D.  Its six MFMAs of column block ni are interleaved with
  // loads into registers that are free by then: the two slots of column block ni - 1 of stage i + D
  // (same buffer; ni = 0: the last column block of the previous buffer's next stage) and, A as slots,
  // one of the four row slots of the previous buffer's next stage, i + D - 1.  A raw: one of the four
  // loads of stage i + AHEAD's pair into the ring (its place was last read during stage i - 2 or earlier),
  // and the fragments of stage i + 1.  An odd stage reads the first fragments of a new pair, whose last loads
  // were requested during stage i + 2 - AHEAD; a stage issues 14 loads and nothing moves across a stage's end,
  // so once at most 14 (AHEAD - 3) loads are outstanding at the top of an odd stage the pair has landed, for
  // the even stage after it as well (the wait is explicit: the compiler does not connect a load into LDS
  // with the read of that LDS address).
  for (int i0 = 0; i0 < n_own; i0 += T::D) {
#pragma unroll
    for (int u = 0; u < T::D; ++u) {
      const int i = i0 + u;
      if (ARAW && (u & 1)) {
        constexpr int YOUNGER = 14 * (AHEAD - 3);   // 42
        static_assert(YOUNGER <= 63, "the wait counter has six bits");
        __builtin_amdgcn_s_waitcnt(0x0F70 | (YOUNGER & 0xF) | ((YOUNGER >> 4) << 14));
      }
      constexpr int P = T::D - 1;               // (u + P) % D: the previous stage's buffer
      const int ab = ARAW ? (u & 1) : u;        // where this stage's A operands are
#pragma unroll
      for (int ni = 0; ni < T::NTL; ++ni) {
        // products lo.hi, hi.lo, hi.hi: smallest first, consecutive MFMAs on different accumulators
#pragma unroll
        for (int mi = 0; mi < T::MT; ++mi) acc[mi][ni] = mfma(Ar[ab][mi][1], Br[u][ni][0], acc[mi][ni]);
#pragma unroll
        for (int mi = 0; mi < T::MT; ++mi) acc[mi][ni] = mfma(Ar[ab][mi][0], Br[u][ni][1], acc[mi][ni]);
#pragma unroll
        for (int mi = 0; mi < T::MT; ++mi) acc[mi][ni] = mfma(Ar[ab][mi][0], Br[u][ni][0], acc[mi][ni]);
        if (ni == 0) issue_b(i + P, (u + P) % T::D, T::NTL - 1);
        else issue_b(i + T::D, u, ni - 1);
        if (ni < 4) {
          if (ARAW) dma_a(i + AHEAD, ni, u & 1);
          else issue_a1(i + P, (u + P) % T::D, ni >> 1, ni & 1);
        }
        if (ARAW) {
          if (ni < T::MT) read_a(i + 1, ni, (u + 1) & 1);
          if (ni >= 1 && ni <= T::MT) split_a(ab ^ 1, ni - 1);
        }
        // two MFMAs, one load, three times (the last block has two loads)
#pragma unroll
        for (int x = 0; x < (ni < 4 ? 3 : 2); ++x) {
          __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
          __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        }
        if (ni == 4) __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // ---- the four partial tiles meet in LDS ---------------------------------------------------------
  // block b = mi * 5 + ni is owned by wave b % 4; a non-owner w puts its partial block at
  // [b][(w - owner - 1) mod 4], 16 bytes per lane and register quad
  if (ARAW) {
    // the area overlaps the rings: every load into them has landed and every wave has read its last fragments
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
  }
  auto reduce_and_store = [&](auto owner_tag) {
    constexpr int W = decltype(owner_tag)::value;
#pragma unroll
    for (int b = 0; b < T::BLOCKS; ++b) {
      if (b % T::NW == W) continue;
      const int slot = ((W - b % T::NW - 1) & 3);
      unsigned char* dst = slotk_smem + (b * 3 + slot) * T::BLOCK_BYTES + lane * 16;
      const f32x16& v = acc[b / T::NTL][b % T::NTL];
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) *(f32x4*)(dst + r4 * 1024) = (f32x4){v[4 * r4], v[4 * r4 + 1], v[4 * r4 + 2], v[4 * r4 + 3]};
    }
    __syncthreads();
    const int ldc_bytes = (int)p.ldc * 4;
    // rows past M fall beyond the end of the buffer and are dropped
    const int64_t c_bytes = ((int64_t)(p.M - 1 - m0) * p.ldc + (p.N - n0)) * 4;
    const i32x4 rc = make_rsrc(p.C + (int64_t)m0 * p.ldc + n0, c_bytes);
#pragma unroll
    for (int b = W; b < T::BLOCKS; b += T::NW) {
      const int mi = b / T::NTL, ni = b % T::NTL;
      if (n0 + ni * 32 >= p.N) continue;
      f32x16 sum;
      // partial sums in wave order 0, 1, 2, 3: the own one at its place
#pragma unroll
      for (int w = 0; w < T::NW; ++w) {
        f32x16 part;
        if (w == W) {
          part = acc[mi][ni];
        } else {
          const unsigned char* src = slotk_smem + (b * 3 + ((w - W - 1) & 3)) * T::BLOCK_BYTES + lane * 16;
#pragma unroll
          for (int r4 = 0; r4 < 4; ++r4) {
            const f32x4 x = *(const f32x4*)(src + r4 * 1024);
            part[4 * r4] = x[0]; part[4 * r4 + 1] = x[1]; part[4 * r4 + 2] = x[2]; part[4 * r4 + 3] = x[3];
          }
        }
        if (w == 0) sum = part;
        else
#pragma unroll
          for (int e = 0; e < 16; ++e) sum[e] += part[e];
      }
      // columns past N (a ragged last tile; their slots were some other column's) are sent beyond the end too
      const bool inside = n0 + ni * 32 + l31 < p.N;
      const float bv = (p.bias && inside) ? p.bias[n0 + ni * 32 + l31] : 0.f;
      const int voff = inside ? (g * 4 * ldc_bytes) + (ni * 32 + l31) * 4 : (int)(c_bytes > 0x7FFFFFFF ? 0x7FFFFFFF : c_bytes);
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          llvm_raw_buffer_store_f32(sum[4 * q + e] + bv, rc, voff, (mi * 32 + q * 8 + e) * ldc_bytes, kResultStoreAux);
    }
  };
  if (wave == 0) reduce_and_store(std::integral_constant<int, 0>{});
  else if (wave == 1) reduce_and_store(std::integral_constant<int, 1>{});
  else if (wave == 2) reduce_and_store(std::integral_constant<int, 2>{});
  else reduce_and_store(std::integral_constant<int, 3>{});
}


// ---------------------------------------------------------------------------------------------------
// The same design with BOTH operands raw fp32 (the operator's plain call: nothing prepared).
//
// A as in the kernel above (ARAW = 1).  B [K][N] row-major needs no LDS either: the 32 columns of an
// MFMA block may be any 32 columns of the tile as long as the store knows which, so a lane takes FOUR
// ADJACENT columns as its column of blocks 0 .. 3 (block j of lane l31 is column 4 l31 + j of the tile's
// first 128) and column 128 + l31 as its column of block 4.  Its eight k of a stage are then eight 16-byte
// loads (32 lanes: 512 contiguous bytes of one row of B) plus eight 4-byte loads, straight into registers,
// four stages deep like the slots above; component j of the eight loads is the lane's operand of block
// j, split in registers right before its MFMAs (one block ahead).  The store writes the four adjacent
// columns of a row as 16 bytes.
// At the end every wave owns one register quad (eight rows) of all ten blocks instead of whole blocks:
// the same LDS traffic, and the 16-byte stores stay possible.
// ---------------------------------------------------------------------------------------------------
struct RawK {
  static constexpr int D = 4, AHEAD = 6;   // B ring in registers; raw A requested this many stages ahead (even: whole pairs)
};

// Host-checked: fp32 operands, K % 32 == 0, N % 4 == 0, lda % 4 == 0, ldb % 4 == 0, A and B 16-byte
// aligned, M * lda * 4 and K * ldb * 4 below 2 GiB, C rows addressable with 32-bit byte offsets inside a
// tile.  c_vec: ldc % 4 == 0 and C 16-byte aligned (16-byte stores).
__global__ __launch_bounds__(SlotK::NT) __attribute__((amdgpu_waves_per_eu(1, 1))) void cascmm_rawk_kernel(const SlotKParams p, int c_vec) {
  typedef SlotK T;
  constexpr int D = RawK::D, AHEAD = RawK::AHEAD;
  extern __shared__ __attribute__((aligned(1024))) unsigned char slotk_smem[];
  const int tid = threadIdx.x, lane = tid & 63, l31 = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int tm, tn;
  tile_coords((int)blockIdx.x, p.tiles_m, p.tiles_n, tm, tn, p.group_m);
  const int m0 = tm * T::BM, n0 = tn * T::BN;
  const int ksteps = p.K >> 4;
  // a wave owns every fourth PAIR of 16-k stages (see the kernel above): own stage i = stage 8 (i / 2) + 2 wave + i % 2
  const int own_tail = (ksteps & 7) - 2 * wave;
  const int n_own = 2 * (ksteps >> 3) + (own_tail < 0 ? 0 : own_tail > 2 ? 2 : own_tail);   // 0 for the last waves of a very short K: they add zeros
  auto stage_of = [&](int i) { return 8 * (i >> 1) + 2 * wave + (i & 1); };
  const int ldb_bytes = (int)p.ldb * 4;

  // ---- B: rows 8 g .. 8 g + 7 of a stage; beyond the last stage the loads point past the end of the
  // buffer and return zeros (see the kernel above) ----
  const int64_t b_bytes64 = ((int64_t)(p.K - 1) * p.ldb + p.N) * 4;
  const int b_bytes = (int)(b_bytes64 > 0x7FFFFFFF ? 0x7FFFFFFF : b_bytes64);
  const i32x4 rb = make_rsrc(p.b_slots, b_bytes);
  const int vbq = 8 * g * ldb_bytes + (n0 + 4 * l31) * 4;
  const int vbs = 8 * g * ldb_bytes + (n0 + 128 + l31) * 4;
  f32x4 Bq[D][8];   // [ring buffer][k]: columns 4 l31 .. 4 l31 + 3
  float Bs[D][8];   // column 128 + l31
  auto b_base = [&](int i) { return i < n_own ? stage_of(i) * (T::BK * ldb_bytes) : b_bytes; };
  // (the stage's place goes into the lane offset, one addition per stage, and the row's into the scalar offset, eight
  // values that never change: a scalar offset of stage + row would be one more instruction in front of every load, and
  // this loop is bound by the number of instructions a wave can issue)
  auto issue_bq = [&](int i, int buf, int e) { Bq[buf][e] = llvm_raw_buffer_load_v4f32(rb, vbq + b_base(i), e * ldb_bytes, 0); };
  auto issue_bs = [&](int i, int buf, int e) { Bs[buf][e] = llvm_raw_buffer_load_f32(rb, vbs + b_base(i), e * ldb_bytes, 0); };
  u32x4 H[2], L[2];   // the split operand of the current / next block
  auto split_b = [&](int buf, int ni, int dst) {
    float r[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = ni < 4 ? Bq[buf][e][ni] : Bs[buf][e];
    u32x4 t[2];
    split8<CASCMM_FMT_BF16, 2>(r, t);
    H[dst] = t[0];
    L[dst] = t[1];
  };

  // ---- A: as in cascmm_slotk_kernel<1> ----
  const int64_t a_bytes = ((int64_t)(p.M - 1) * p.lda + p.K) * 4;
  const __amdgpu_buffer_rsrc_t rar =
      __builtin_amdgcn_make_buffer_rsrc((void*)p.a, 0, (int)(a_bytes > 0x7FFFFFFF ? 0x7FFFFFFF : a_bytes), 0x00020000);
  unsigned char* ring = slotk_smem + wave * T::RING;
  int dma_voff[2];
#pragma unroll
  for (int jp = 0; jp < 2; ++jp)
    dma_voff[jp] = (int)(((int64_t)(m0 + (lane >> 3)) * p.lda + (((lane & 7) - (4 * jp + (lane >> 4))) & 7) * 4) * 4);
  const int dma_rows8 = (int)p.lda * 32;
  int dma_v[4];   // (as in the kernel above: one M0 and one scalar offset for the four loads of a stage)
#pragma unroll
  for (int ni = 0; ni < 4; ++ni) dma_v[ni] = dma_voff[ni & 1] + ni * (dma_rows8 - 1024);
  auto dma_a = [&](int i, int ni, int sp) {   // sp = i % 2
    const int q = i >> 1;
    const int koff = (2 * q < n_own ? stage_of(2 * q) * (T::BK * 4) : 0) + 4 * sp * dma_rows8;
    wavek_load_lds_kb(rar, ring + (q & (T::RA / 2 - 1)) * (2 * T::A_STAGE) + sp * 4096, dma_v[ni], koff, ni);
  };
  int a_frag[2][2];
#pragma unroll
  for (int sp = 0; sp < 2; ++sp)
#pragma unroll
    for (int x = 0; x < 2; ++x) a_frag[sp][x] = l31 * 128 + ((4 * sp + 2 * g + x + (l31 >> 1)) & 7) * 16;
  f32x4 X[T::MT][2];
  u32x4 Ar[2][T::MT][2];   // [stage parity][row block][term]
  auto read_a = [&](int i, int mi, int sp) {   // sp = i % 2
    const unsigned char* st = ring + ((i >> 1) & (T::RA / 2 - 1)) * (2 * T::A_STAGE) + mi * 4096;
    X[mi][0] = *(const f32x4*)(st + a_frag[sp][0]);
    X[mi][1] = *(const f32x4*)(st + a_frag[sp][1]);
  };
  auto split_a = [&](int buf, int mi) {
    float r[8] = {X[mi][0][0], X[mi][0][1], X[mi][0][2], X[mi][0][3], X[mi][1][0], X[mi][1][1], X[mi][1][2], X[mi][1][3]};
    u32x4 t[2];
    split8<CASCMM_FMT_BF16, 2>(r, t);
    Ar[buf][mi][0] = t[0];
    Ar[buf][mi][1] = t[1];
  };

  // ---- prologue: raw A of stages 0 .. AHEAD - 1 (three pairs) and stage 0 of B first (40 loads), then the
  // rest of B (40 loads: the wait below names exactly those) ----
  f32x16 acc[T::MT][T::NTL];
#pragma unroll
  for (int d = 0; d < AHEAD; ++d)
#pragma unroll
    for (int j = 0; j < 4; ++j) dma_a(d, j, d & 1);
#pragma unroll
  for (int e = 0; e < 8; ++e) issue_bq(0, 0, e);
#pragma unroll
  for (int e = 0; e < 8; ++e) issue_bs(0, 0, e);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int d = 1; d < D; ++d)
#pragma unroll
    for (int e = 0; e < 8; ++e) issue_bq(d, d, e);
#pragma unroll
  for (int d = 1; d < D - 1; ++d)
#pragma unroll
    for (int e = 0; e < 8; ++e) issue_bs(d, d, e);
#pragma unroll
  for (int mi = 0; mi < T::MT; ++mi)
#pragma unroll
    for (int ni = 0; ni < T::NTL; ++ni)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[mi][ni][e] = 0.f;
  {
    constexpr int LATER = 8 * (D - 1) + 8 * (D - 2);   // 40
    static_assert(LATER <= 63, "the wait counter has six bits");
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0x0F70 | (LATER & 0xF) | ((LATER >> 4) << 14));
#pragma unroll
    for (int mi = 0; mi < T::MT; ++mi) read_a(0, mi, 0);
#pragma unroll
    for (int mi = 0; mi < T::MT; ++mi) split_a(0, mi);
    split_b(0, 0, 0);
  }

  auto mfma = [&](u32x4 a, u32x4 b, f32x16 c) -> f32x16 {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  };
  // Stage i, ring buffer u = i % D.  During column block ni: the MFMAs of the block; the split of the next
  // block (ni = 4: block 0 of the next stage); loads into registers that are free by then -- ni = 0 .. 2:
  // the single column of the PREVIOUS buffer's next stage (its last reader was the split during the
  // previous stage's block 3), ni = 3, 4: the four adjacent columns of this buffer's next stage (last read
  // by the split during block 2); ni = 0 .. 3: one load of raw A into the LDS ring; ni = 0, 1: the A
  // fragments of the next stage, split during ni = 1, 2.  An odd stage reads the first fragments of a new
  // pair, whose last loads were requested during stage i + 2 - AHEAD; a stage issues 20 loads and nothing
  // moves across a stage's end, so once at most 20 (AHEAD - 3) = 60 loads are outstanding at the top of an
  // odd stage the pair has landed, for the even stage after it as well.
  for (int i0 = 0; i0 < n_own; i0 += D) {
#pragma unroll
    for (int u = 0; u < D; ++u) {
      const int i = i0 + u;
      if (u & 1) {
        constexpr int YOUNGER = 20 * (AHEAD - 3);
        static_assert(YOUNGER <= 63, "the wait counter has six bits");
        __builtin_amdgcn_s_waitcnt(0x0F70 | (YOUNGER & 0xF) | ((YOUNGER >> 4) << 14));
      }
      constexpr int P = D - 1;
      const int ab = u & 1;
#pragma unroll
      for (int ni = 0; ni < T::NTL; ++ni) {
        const int cur = (u * T::NTL + ni) & 1;
#pragma unroll
        for (int mi = 0; mi < T::MT; ++mi) acc[mi][ni] = mfma(Ar[ab][mi][1], H[cur], acc[mi][ni]);
#pragma unroll
        for (int mi = 0; mi < T::MT; ++mi) acc[mi][ni] = mfma(Ar[ab][mi][0], L[cur], acc[mi][ni]);
#pragma unroll
        for (int mi = 0; mi < T::MT; ++mi) acc[mi][ni] = mfma(Ar[ab][mi][0], H[cur], acc[mi][ni]);
        if (ni < T::NTL - 1) split_b(u, ni + 1, cur ^ 1);
        else split_b((u + 1) % D, 0, cur ^ 1);
        if (ni < 3) {
#pragma unroll
          for (int e = 3 * ni; e < (ni == 2 ? 8 : 3 * ni + 3); ++e) issue_bs(i + P, (u + P) % D, e);
        } else {
#pragma unroll
          for (int e = 4 * (ni - 3); e < 4 * (ni - 3) + 4; ++e) issue_bq(i + D, u, e);
        }
        if (ni < 4) dma_a(i + AHEAD, ni, u & 1);
        if (ni < T::MT) read_a(i + 1, ni, (u + 1) & 1);
        if (ni >= 1 && ni <= T::MT) split_a(ab ^ 1, ni - 1);
        // loads of this block: 4, 4, 3, 5, 4 -- one behind each of the first MFMAs
        constexpr int kLoads[5] = {4, 4, 3, 5, 4};
#pragma unroll
        for (int x = 0; x < 6; ++x) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if (x < kLoads[ni]) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // ---- the four partial tiles meet in LDS: wave W owns register quad W (rows 8 W + 4 g + e) of all ten
  // blocks; a non-owner w puts its quad q of block b at [q][(w - q - 1) mod 4][b], 16 bytes per lane ----
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();
  auto reduce_and_store = [&](auto owner_tag) {
    constexpr int W = decltype(owner_tag)::value;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (q == W) continue;
      const int slot = (W - q - 1) & 3;
#pragma unroll
      for (int b = 0; b < T::BLOCKS; ++b) {
        const f32x16& v = acc[b / T::NTL][b % T::NTL];
        *(f32x4*)(slotk_smem + ((q * 3 + slot) * T::BLOCKS + b) * 1024 + lane * 16) = (f32x4){v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]};
      }
    }
    __syncthreads();
    f32x4 sum[T::MT][T::NTL];
#pragma unroll
    for (int b = 0; b < T::BLOCKS; ++b) {
      const f32x16& v = acc[b / T::NTL][b % T::NTL];
      f32x4 s4;
      // partial sums in wave order 0, 1, 2, 3: the own one at its place
#pragma unroll
      for (int w = 0; w < T::NW; ++w) {
        const f32x4 part = w == W ? (f32x4){v[4 * W], v[4 * W + 1], v[4 * W + 2], v[4 * W + 3]}
                                  : *(const f32x4*)(slotk_smem + ((W * 3 + ((w - W - 1) & 3)) * T::BLOCKS + b) * 1024 + lane * 16);
        if (w == 0) s4 = part;
        else s4 += part;
      }
      sum[b / T::NTL][b % T::NTL] = s4;
    }
    const int ldc_bytes = (int)p.ldc * 4;
    const int64_t c_bytes64 = ((int64_t)(p.M - 1 - m0) * p.ldc + (p.N - n0)) * 4;   // rows past M fall beyond the end: dropped
    const int c_bytes = (int)(c_bytes64 > 0x7FFFFFFF ? 0x7FFFFFFF : c_bytes64);
    const i32x4 rc = make_rsrc(p.C + (int64_t)m0 * p.ldc + n0, c_bytes);
    // columns past N (a ragged last tile) are sent beyond the end as well
    const int colq = 4 * l31, cols = 128 + l31;
    const bool inq = n0 + colq < p.N, ins = n0 + cols < p.N;   // (N % 4 == 0: four adjacent columns are inside together)
    f32x4 bq = {0.f, 0.f, 0.f, 0.f};
    float bs = 0.f;
    if (p.bias && inq) {
#pragma unroll
      for (int j = 0; j < 4; ++j) bq[j] = p.bias[n0 + colq + j];
    }
    if (p.bias && ins) bs = p.bias[n0 + cols];
    const int voq = inq ? (g * 4 * ldc_bytes) + colq * 4 : c_bytes;
    const int vos = ins ? (g * 4 * ldc_bytes) + cols * 4 : c_bytes;
#pragma unroll
    for (int mi = 0; mi < T::MT; ++mi)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int soff = (mi * 32 + W * 8 + e) * ldc_bytes;
        const f32x4 v4 = {sum[mi][0][e] + bq[0], sum[mi][1][e] + bq[1], sum[mi][2][e] + bq[2], sum[mi][3][e] + bq[3]};
        if (c_vec) {
          llvm_raw_buffer_store_v4f32(v4, rc, voq, soff, kResultStoreAux);
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) llvm_raw_buffer_store_f32(v4[j], rc, inq ? voq + 4 * j : c_bytes, soff, kResultStoreAux);
        }
        llvm_raw_buffer_store_f32(sum[mi][4][e] + bs, rc, vos, soff, kResultStoreAux);
      }
  };
  if (wave == 0) reduce_and_store(std::integral_constant<int, 0>{});
  else if (wave == 1) reduce_and_store(std::integral_constant<int, 1>{});
  else if (wave == 2) reduce_and_store(std::integral_constant<int, 2>{});
  else reduce_and_store(std::integral_constant<int, 3>{});
}

}  // namespace cascmm
