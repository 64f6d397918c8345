// Large-tile kernel of the two-term bf16 cascade (gfx950): four waves with 512 registers each.
//
// One workgroup = four waves (one per SIMD, 2 x 2) computes a 256 x 320 tile of C; a wave owns
// 128 x 160 of it, twenty 32 x 32 accumulator blocks: sixteen in the 256 accumulation registers
// and four in ordinary vector registers.  Against a 64 x 160 wave tile this cuts the LDS bytes read per
// MFMA by a third and the bytes staged per MFMA by 30 %, and those bytes, not issue slots, are what
// the chip's power management charges for: with every CU busy the clock settles where the power
// fits, so fewer bytes moved per MFMA is a higher clock.
//
// There are no producer waves (a kernel has one register allocation, so a wave with 512 registers
// fills its SIMD).  Both operands reach LDS as raw fp32 without passing registers (wave-wide
// `buffer_load ... lds`, 1 KB each), and every wave splits the values of its own fragments in
// registers right after reading them:
//   * A: 256 rows x 16 k per stage; four consecutive lanes fetch the four 16-byte chunks of one row's
//     64 bytes (whole cache lines), rotated by row / 4 inside the row so that the fragment reads (lane
//     l: row l%32, chunks 2 (l/32) and 2 (l/32) + 1) spread over all banks;
//   * B: 16 k rows x 320 columns per stage, 256 consecutive floats per load; lane l of a fragment reads
//     column l%32 at k = 8 (l/32) .. +7 with eight ds_read_b32 (rows of the odd k-group are rotated by
//     32 columns, which keeps the two half waves on different banks).
// Two waves share every row block and every column block, so each value is split twice per
// workgroup; the split's VALU work issues in the gaps between the wave's own MFMAs, as do the LDS
// reads and the loads of later stages, and it costs no measurable time there.
//
// Stages are 16 k deep (60 MFMAs per wave), four of them in LDS (144 KB).  At the barrier that opens
// stage s, stage s + 1 has landed as well, so the first fragments of the next stage are read before
// its barrier and no LDS latency is exposed after it; the loads of stage s + 3 are issued during
// stage s.  Loads are issued unconditionally (past the last stage the last one is fetched again into
// a dead buffer): a wave that is alone on its SIMD pays tens of cycles for every branch.
//
// The order of everything between two MFMAs is pinned with scheduling fences; the four blocks held
// in vector registers use the MFMA through inline assembly, because the compiler gives every MFMA it
// selects an accumulator in the accumulation registers (of which there are sixteen blocks' worth).
#pragma once
#include "cascmm_tile_kernel.h"

namespace cascmm {

struct W512 {
  static constexpr int BM = 256, BN = 320, BK = 16, NS = 4, NT = 256;
  static constexpr int WTM = 128, WTN = 160, MT = 4, NTL = 5;
  static constexpr int A_STAGE = BM * BK * 4;       // raw fp32: 64 bytes per row
  static constexpr int B_STAGE = BK * BN * 4;       // raw fp32
  static constexpr int STAGE = A_STAGE + B_STAGE;   // 36 KB
  static constexpr int LDS_BYTES = NS * STAGE;      // 144 KB
  static constexpr int LOADS = 9;                   // direct loads per wave and stage: 4 of A, 5 of B
};

typedef __attribute__((address_space(3))) void* w512_lds_ptr;

// MFMA with the accumulator in ordinary vector registers
__device__ __forceinline__ void w512_mfma_v(u32x4 a, u32x4 b, f32x16& c) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
}
__device__ __forceinline__ f32x16 w512_mfma_a(u32x4 a, u32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// Host-checked: M % 256 == 0, N % 320 == 0, K % 32 == 0, lda % 4 == 0, ldb % 4 == 0, A and B 16-byte
// aligned, M * lda * 4 and K * ldb * 4 below 2 GiB, C rows addressable with 32-bit byte offsets
// inside a tile.
// GLU = 1: the gated store (C has N / 2 columns, see GroupParams); a raw operand's gate columns are
// fetched from N / 2 further right, so that both kinds of operand fill the same accumulator blocks.
// (An instantiation of its own: the plain kernel stays as it is, without the scratch bytes this epilogue's
// register allocation asks for.)
// GLU = 2: the gated store writes its result as the LEFT OPERAND SLOTS of the next GEMM (two bf16 terms,
// [term][(N / 2) / 8][M] x 16 bytes at C) instead of fp32.  The MFMAs then take their operands the other
// way round, which leaves every accumulator block transposed in the registers: a lane holds one row of C
// and four consecutive columns per register quad, i.e. half a slot per quad -- the slot of k group
// 2 t + g holds columns 16 t + 4 g + 0..3 and 16 t + 8 + 4 g + 0..3 -- and 32 consecutive lanes write 32
// consecutive slots, 512 contiguous bytes.  (cascmm_prepare_weight_chained gives the next GEMM's weight
// the same order of k.)
// BPRE = 1: the right operand comes already split (cascmm_prepare_weight: 16-byte slots of 8 k of one
// column of one term, [term][K/8][N], below 2 GiB).  A stage then holds the same 20 KB of B as slots
// [term][k group][320], copied by the same twenty 1 KB loads; a lane reads its two operands with two
// 16-byte reads instead of eight 4-byte ones, and the split of B, 55 % of the kernel's VALU work,
// is gone.  Same terms, same order of products: the results equal the raw kernel's bit for bit.
// (a template, so that only the translation unit that lists the variant compiles it)
template <int BPRE, int GLU = 0>
__global__ __launch_bounds__(W512::NT) __attribute__((amdgpu_waves_per_eu(1, 1))) void cascmm_w512_kernel(const GroupParams p) {
  typedef W512 T;
  extern __shared__ __attribute__((aligned(1024))) unsigned char w512_smem[];
  unsigned char* smem = w512_smem;
  const int tid = threadIdx.x, lane = tid & 63, l31 = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave >> 1) * T::WTM, wn0 = (wave & 1) * T::WTN;
  int tm, tn;
  tile_coords(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
  const int m0 = tm * T::BM, n0 = tn * T::BN;
  const int ksteps = p.K / T::BK;
  const int ldb_bytes = (int)p.ldb * 4;

  const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc((void*)p.A[0], 0, 0x7FFFFFFF, 0x00020000);
  // (one record fewer than A's: with equal words the compiler keeps one copy of them and rebuilds this descriptor from it
  // in front of every B load)
  const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc((void*)p.B[0], 0, 0x7FFFFFFE, 0x00020000);
  // per wave and stage: 4 loads of A (16 rows x 64 bytes each; LDS position 4 row + pos holds chunk
  // (pos - row / 4) mod 4 of the row) and 5 loads of B (256 consecutive floats of the stage's [16][320]
  // area)
  int a_voff[4], b_voff[5];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int inst = wave * 4 + j;
    const int row = inst * 16 + (lane >> 2);
    const int chunk = ((lane & 3) - (row >> 2)) & 3;
    a_voff[j] = (int)(((int64_t)(m0 + row) * p.lda + chunk * 4) * 4);
  }
#pragma unroll
  for (int j = 0; j < 5; ++j) {
    const int inst = wave * 5 + j;
    if (BPRE) {
      // run inst = (term * 2 + k group) * 5 + run of 64 columns; lane = column inside the run
      const int tk = inst / 5, run = inst % 5;
      b_voff[j] = (((tk >> 1) * (p.K >> 3) + (tk & 1)) * p.N + n0 + run * 64 + lane) * 16;
    } else {
      const int f = inst * 256 + lane * 4;
      const int k = f / T::BN, pos = f % T::BN;
      int n = pos - 32 * ((k >> 3) & 1);
      n = n < 0 ? n + T::BN : n;
      int col = n0 + n;
      // gated store: the tile's ten column blocks are value 0, gate 0, value 1, ... of output columns
      // n0 / 2 + 32 j + l; the raw operand keeps its gate columns N / 2 further right
      if (GLU) col = ((n >> 5) & 1) * (p.N >> 1) + (n0 >> 1) + 32 * (n >> 6) + (n & 31);
      b_voff[j] = k * ldb_bytes + col * 4;
    }
  }
  const int b_step = BPRE ? 2 * p.N * 16 : T::BK * ldb_bytes;   // bytes of B per stage
  // The loads of a wave land in consecutive kilobytes of LDS: the LDS address is M0 plus the instruction's immediate
  // offset, so a wave's A loads of a stage share one M0 and differ in the immediate; the immediate moves the memory
  // address too, which the lane offsets make up for (they stay non-negative: load j starts at least j KB into its
  // operand).  The fifth B load is 4 KB further, beyond the immediate's range, and takes an M0 of its own.
#pragma unroll
  for (int j = 1; j < 4; ++j) {
    a_voff[j] -= j * 1024;
    b_voff[j] -= j * 1024;
  }
  auto issue1 = [&](int step_, int j) {
    const int step = step_ < ksteps - 1 ? step_ : ksteps - 1;
    const int st = step_ % T::NS;
    const w512_lds_ptr al = (w512_lds_ptr)(smem + st * T::STAGE + wave * 4096);
    const w512_lds_ptr bl = (w512_lds_ptr)(smem + st * T::STAGE + T::A_STAGE + wave * 5120);
    const int as = step * T::BK * 4, bs = step * b_step;
    switch (j) {
      case 0: __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, al, 16, a_voff[0], as, 0, 0); break;
      case 1: __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, al, 16, a_voff[1], as, 1024, 0); break;
      case 2: __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, al, 16, a_voff[2], as, 2048, 0); break;
      case 3: __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, al, 16, a_voff[3], as, 3072, 0); break;
      case 4: __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, bl, 16, b_voff[0], bs, 0, 0); break;
      case 5: __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, bl, 16, b_voff[1], bs, 1024, 0); break;
      case 6: __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, bl, 16, b_voff[2], bs, 2048, 0); break;
      case 7: __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, bl, 16, b_voff[3], bs, 3072, 0); break;
      default: __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (w512_lds_ptr)(smem + st * T::STAGE + T::A_STAGE + wave * 5120 + 4096), 16, b_voff[4], bs, 0, 0); break;
    }
  };

  // fragment addresses (bytes inside a stage)
  const int a_row = wm0 + l31;                          // + mi * 32 rows = mi * 2048 bytes (same rotation: 32 / 4 = 8)
  const int a_frag0 = a_row * 64 + ((2 * g + (a_row >> 2)) & 3) * 16;
  const int a_frag1 = a_row * 64 + ((2 * g + 1 + (a_row >> 2)) & 3) * 16;
  int b_frag[T::NTL];
#pragma unroll
  for (int ni = 0; ni < T::NTL; ++ni) {
    int pos = wn0 + ni * 32 + l31 + 32 * g;
    pos = pos >= T::BN ? pos - T::BN : pos;
    b_frag[ni] = T::A_STAGE + (8 * g * T::BN + pos) * 4;   // + e * BN * 4
    // prepared: slot (term 0, k group g, column) -- term 1 is 2 * BN slots further
    if (BPRE) b_frag[ni] = T::A_STAGE + (g * T::BN + wn0 + ni * 32 + l31) * 16;
  }

  f32x16 acc[T::MT][T::NTL];

  // ---- software pipeline ---------------------------------------------------------------------
  // Blocks are numbered t = stage * 5 + ni.  While the 12 MFMAs of block t issue, the raw B values of
  // block t + 2 are read from LDS and those of block t + 1 (read one block earlier) are split; the A
  // values of row block ni of the next stage are read and split during block ni (0 .. 3), two loads of
  // a later stage are issued per block.
#define W512_FENCE() __builtin_amdgcn_sched_barrier(0)
  u32x4 Af[2][2][T::MT];   // [buffer][hi / lo][mi]
  float R[2][8];           // raw B values of two blocks in flight
  float RA[8];             // raw A values of one row block of the next stage
  u32x4 H[2], L[2];        // split B of the current / next block
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  typedef float f32x2v __attribute__((ext_vector_type(2)));

  auto read_raw = [&](float (&dst)[8], const unsigned char* stp, int ni, int e0, int e1) {
#pragma unroll
    for (int e = e0; e < e1; ++e) dst[e] = *(const float*)(stp + b_frag[ni] + e * T::BN * 4);
  };
  // prepared B: the two terms of a block (the second term is needed four MFMAs later than the first)
  auto read_slot_hi = [&](int buf, const unsigned char* stp, int ni) { H[buf] = *(const u32x4*)(stp + b_frag[ni]); };
  auto read_slot_lo = [&](int buf, const unsigned char* stp, int ni) { L[buf] = *(const u32x4*)(stp + b_frag[ni] + 2 * T::BN * 16); };
  // the split of one pair of consecutive k in two halves of three VALU instructions each
  auto split_1 = [&](float (&x)[8], u32x4& hi, int e) {
    const f32x2v v = {x[2 * e], x[2 * e + 1]};
    const unsigned hp = __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2));
    hi[e] = hp;
    x[2 * e] = x[2 * e] - __builtin_bit_cast(float, hp << 16);
  };
  auto split_2 = [&](float (&x)[8], const u32x4& hi, u32x4& lo, int e) {
    const f32x2v r = {x[2 * e], x[2 * e + 1] - __builtin_bit_cast(float, hi[e] & 0xFFFF0000u)};
    lo[e] = __builtin_bit_cast(unsigned, __builtin_convertvector(r, bf16x2));
  };

#pragma unroll
  for (int s = 0; s < T::NS - 1; ++s)
#pragma unroll
    for (int j = 0; j < T::LOADS; ++j) issue1(s, j);
  // the accumulators are cleared while the first loads are in flight: not before them, which would hold
  // the loads back, and not after the barrier, where the first MFMA would wait for it
  W512_FENCE();
#pragma unroll
  for (int mi = 0; mi < T::MT; ++mi)
#pragma unroll
    for (int ni = 0; ni < T::NTL; ++ni)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[mi][ni][e] = 0.f;
  // (an empty statement that "uses" every block makes the zeros real here; left alone the compiler creates them
  // right before the first MFMAs)
#pragma unroll
  for (int mi = 0; mi < T::MT; ++mi)
#pragma unroll
    for (int ni = 0; ni < T::NTL; ++ni) {
      if (ni < 4) asm volatile("" : "+a"(acc[mi][ni]));
      else asm volatile("" : "+v"(acc[mi][ni]));
    }
  W512_FENCE();
  __builtin_amdgcn_s_waitcnt(0x0F70 | (18 & 0xF) | ((18 >> 4) << 14));   // vmcnt(18): stage 0 has landed
  __builtin_amdgcn_s_barrier();
  {
#pragma unroll
    for (int mi = 0; mi < T::MT; ++mi) {
      const f32x4 x0 = *(const f32x4*)(smem + a_frag0 + mi * 2048), x1 = *(const f32x4*)(smem + a_frag1 + mi * 2048);
      float x[8] = {x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        split_1(x, Af[0][0][mi], e);
        split_2(x, Af[0][0][mi], Af[0][1][mi], e);
      }
    }
    if (BPRE) {
      read_slot_hi(0, smem, 0);
      read_slot_lo(0, smem, 0);
    } else {
      read_raw(R[0], smem, 0, 0, 8);
      read_raw(R[1], smem, 1, 0, 8);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        split_1(R[0], H[0], e);
        split_2(R[0], H[0], L[0], e);
      }
    }
  }

  for (int s = 0; s < ksteps; s += 2) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      // top of stage s + j: the own loads of stage s + j + 1 have landed, then everybody's
      __builtin_amdgcn_s_waitcnt(0x0F70 | T::LOADS);                     // vmcnt(9)
      __builtin_amdgcn_s_barrier();
      const unsigned char* st0 = smem + ((s + j) % T::NS) * T::STAGE;       // this stage
      const unsigned char* st1 = smem + ((s + j + 1) % T::NS) * T::STAGE;   // the next one
#pragma unroll
      for (int ni = 0; ni < T::NTL; ++ni) {
        const int t = j * T::NTL + ni;        // block number inside the trip: its parity is static
        const int cur = t & 1, nxt = cur ^ 1;
        const int n2 = (ni + 2) % T::NTL;
        const unsigned char* st2 = (ni + 2 < T::NTL) ? st0 : st1;
        const int n1 = (ni + 1) % T::NTL;                                  // prepared B: the next block's slots are read whole
        const unsigned char* stn = (ni + 1 < T::NTL) ? st0 : st1;
        u32x4(&Ah)[T::MT] = Af[j][0];
        u32x4(&Al)[T::MT] = Af[j][1];
        // products lo.hi, hi.lo, hi.hi of the four row blocks: smallest first, consecutive MFMAs on
        // different accumulators
        auto mm = [&](int idx) {
          const int prod = idx >> 2, mi = idx & 3;
          const u32x4 a = prod == 0 ? Al[mi] : Ah[mi];
          const u32x4 b = prod == 1 ? L[cur] : H[cur];
          if (GLU == 2) {   // operands swapped: the block comes out transposed
            if (ni < 4) acc[mi][ni] = w512_mfma_a(b, a, acc[mi][ni]);
            else w512_mfma_v(b, a, acc[mi][ni]);
          } else {
            if (ni < 4) acc[mi][ni] = w512_mfma_a(a, b, acc[mi][ni]);
            else w512_mfma_v(a, b, acc[mi][ni]);
          }
        };
        auto dl = [&](int k) {   // two load slots per block: 10 per stage, 9 used
          const int slot = ni * 2 + k;
          if (slot < T::LOADS) issue1(s + j + T::NS - 1, slot);
        };
        // What goes between MFMA g and MFMA g + 1 of the block.  A wave alone on its SIMD issues one instruction
        // every four cycles or so, whatever its kind, and an MFMA holds the matrix pipe for 32: more than six
        // instructions in a gap leave the pipe waiting.  The sixteen half-splits of the block (three VALU
        // instructions each: B's in gaps 0 .. 7, A's in gaps 4 .. 11) and the LDS reads and loads are spread so
        // that no gap holds more than six (2202 shader-clock cycles per stage against 2228 with the LDS reads in
        // gaps 0 .. 2 and all the splits in gaps 3 .. 10; 1920 are the MFMAs).
        // LDS answers in order: one wait at the top of a block covers everything the block before it read (the
        // compiler would put a wait of its own, an instruction each, in front of the first use of every read),
        // a second one in gap 4 the block's A fragments (younger than them: the raw B reads of gaps 1 and 2)
        auto gap = [&](int gi) {
          if (gi == 0) { __builtin_amdgcn_s_waitcnt(0xC07F); W512_FENCE(); }                          // lgkmcnt(0)
          if (gi == 4 && ni < 4) { __builtin_amdgcn_s_waitcnt(BPRE ? 0xC07F : 0xC47F); W512_FENCE(); }   // lgkmcnt(0) / lgkmcnt(4)
          if (gi == 0 && ni < 4) {   // row block ni of the next stage
            const f32x4 x0 = *(const f32x4*)(st1 + a_frag0 + ni * 2048), x1 = *(const f32x4*)(st1 + a_frag1 + ni * 2048);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              RA[e] = x0[e];
              RA[4 + e] = x1[e];
            }
          }
          if (!BPRE && gi == 1) read_raw(R[cur], st2, n2, 0, 4);
          if (!BPRE && gi == 2) read_raw(R[cur], st2, n2, 4, 8);
          if (!BPRE && gi < 8) {
            if (gi & 1) split_2(R[nxt], H[nxt], L[nxt], gi >> 1);
            else split_1(R[nxt], H[nxt], gi >> 1);
          }
          if (ni < 4 && gi >= 4) {
            const int h = gi - 4;
            if (h & 1) split_2(RA, Af[j ^ 1][0][ni], Af[j ^ 1][1][ni], h >> 1);
            else split_1(RA, Af[j ^ 1][0][ni], h >> 1);
          }
          if (BPRE && gi == 4) read_slot_hi(nxt, stn, n1);     // seven MFMAs before the next block's first
          if (BPRE && gi == 8) read_slot_lo(nxt, stn, n1);
          // the stage's nine loads: two per block, apart from each other and in gaps that hold one half-split
          // (several loads in neighbouring gaps of one block cost 30 cycles each: counted)
          if (gi == 9) dl(0);
          if (gi == 10) dl(1);
        };
#pragma unroll
        for (int gi = 0; gi < 12; ++gi) {
          mm(gi); W512_FENCE();
          gap(gi); W512_FENCE();
        }
      }
    }
  }
#undef W512_FENCE
  __builtin_amdgcn_s_waitcnt(0x0F70);   // the redundant loads of the last stages land before LDS is given up
  // the MFMAs written as assembly are invisible to the compiler's hazard handling: their passes
  // must have drained before the accumulators are read
  asm volatile("s_nop 7\n s_nop 7\n s_nop 7" ::: "memory");

  // ---- epilogue: of every block a lane holds column l31, rows 8 q + 4 g + e -----------------------
  // (the lane number is taken afresh: a register kept alive through the main loop for it would be spilled)
  const int elane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
  const int el31 = elane & 31, eg = elane >> 5;
  const float* bias = (const float*)p.bias[0];
  const int ldc_bytes = (int)p.ldc * 4;
  if constexpr (GLU == 2) {
    // Gated store as operand slots.  Blocks are transposed: of block (mi, ni) a lane holds row 32 mi + l31
    // and columns 8 q + 4 g + e in register 4 q + e.  Pairs of blocks as below (value j, gate j); the gate
    // of pair 2 crosses from the right wave to the left one through LDS, same lanes and registers.
    const int half = p.N >> 1, c0 = n0 >> 1;
    const int kgroups = half >> 3;                                  // k groups of the next GEMM
    float* xbuf = (float*)smem + (wave >> 1) * (T::MT * 16 * 64);
    __builtin_amdgcn_s_barrier();
    auto bias_at = [&](int col) { return bias ? bias[col] : 0.f; };
    if (wave & 1) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float bg = bias_at(half + c0 + 64 + 8 * (r >> 2) + 4 * eg + (r & 3));
#pragma unroll
        for (int mi = 0; mi < T::MT; ++mi) xbuf[(mi * 16 + r) * 64 + elane] = gelu_value(acc[mi][0][r] + bg);
      }
    }
    __syncthreads();
    // 4 M K2 bytes of slots, below 2 GiB (host-checked)
    const i32x4 rc = make_rsrc(p.C[0], (int64_t)2 * kgroups * p.M * 16);
    const int voff = (eg * p.M + m0 + wm0 + el31) * 16;             // + mi * 512
    const int term1 = kgroups * p.M * 16;
    auto out_pair = [&](int pair, int vb, int gb, bool gate_in_lds) {
      const int col0 = c0 + 32 * pair;                              // first output column of the pair
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {                              // k groups 4 (col0 / 32) + 2 s2 + g
        float bv[8], bgt[8];
#pragma unroll
        for (int x = 0; x < 8; ++x) {
          const int col = col0 + 16 * s2 + 8 * (x >> 2) + 4 * eg + (x & 3);
          bv[x] = bias_at(col);
          bgt[x] = gate_in_lds ? 0.f : bias_at(half + col);
        }
        const int soff = ((col0 >> 3) + 2 * s2) * p.M * 16;
#pragma unroll
        for (int mi = 0; mi < T::MT; ++mi) {
          float r8[8];
#pragma unroll
          for (int x = 0; x < 8; ++x) {
            const int r = 8 * s2 + x;                               // register 4 q + e with q = 2 s2 + x / 4
            const float gl = gate_in_lds ? xbuf[(mi * 16 + r) * 64 + elane] : gelu_value(acc[mi][gb][r] + bgt[x]);
            r8[x] = (acc[mi][vb][r] + bv[x]) * gl;
            // the slots are the split of this product ROUNDED to fp32, as a separate pass over the fp32
            // result would split it: keep the compiler from folding the multiplication into the split's
            // subtraction (a fused multiply-subtract would take the residual of the unrounded product)
            asm volatile("" : "+v"(r8[x]));
          }
          u32x4 t[2];
          split8<CASCMM_FMT_BF16, 2>(r8, t);
          llvm_raw_buffer_store_v4f32(__builtin_bit_cast(f32x4, t[0]), rc, voff + mi * 512, soff, kLargeTileStoreAux);
          llvm_raw_buffer_store_v4f32(__builtin_bit_cast(f32x4, t[1]), rc, voff + mi * 512, soff + term1, kLargeTileStoreAux);
        }
      }
    };
    if ((wave & 1) == 0) {
      out_pair(0, 0, 1, false);
      out_pair(1, 2, 3, false);
      out_pair(2, 4, 0, true);
    } else {
      out_pair(3, 1, 2, false);
      out_pair(4, 3, 4, false);
    }
    return;
  }
  if constexpr (GLU == 1) {
    // Gated store: C[m][n0 / 2 + 32 j + l] = (value j + bias) x gelu(gate j + bias), j = 0 .. 4.  The
    // left wave of a row pair holds value 0, gate 0, value 1, gate 1, value 2, the right one gate 2,
    // value 3, gate 3, value 4, gate 4: pair 2 is the only one that spans two waves; the right wave
    // evaluates its gate (which evens out the two waves' arithmetic) and hands gelu(gate), same lanes and
    // registers, over through the LDS the main loop has given up.
    const int half = p.N >> 1, c0 = n0 >> 1;
    float* xbuf = (float*)smem + (wave >> 1) * (T::MT * 16 * 64);   // 16 KB per row pair of waves
    __builtin_amdgcn_s_barrier();                                    // every wave has read its last fragments
    if (wave & 1) {
      const float bg = bias ? bias[half + c0 + 64 + el31] : 0.f;
#pragma unroll
      for (int mi = 0; mi < T::MT; ++mi)
#pragma unroll
        for (int r = 0; r < 16; ++r) xbuf[(mi * 16 + r) * 64 + elane] = gelu_value(acc[mi][0][r] + bg);
    }
    __syncthreads();
    float* C = (float*)p.C[0] + (int64_t)(m0 + wm0) * p.ldc + c0;
    const i32x4 rc = make_rsrc(C, 0x7FFFFFFF);
    auto out_pair = [&](int pair, int vb, int gb, bool gate_in_lds) {
      const float bv = bias ? bias[c0 + 32 * pair + el31] : 0.f;
      const float bg = (bias && !gate_in_lds) ? bias[half + c0 + 32 * pair + el31] : 0.f;
      const int voff = eg * 4 * ldc_bytes + (pair * 32 + el31) * 4;
#pragma unroll
      for (int mi = 0; mi < T::MT; ++mi)
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int r = 4 * q + e;
            const float gl = gate_in_lds ? xbuf[(mi * 16 + r) * 64 + elane] : gelu_value(acc[mi][gb][r] + bg);
            llvm_raw_buffer_store_f32((acc[mi][vb][r] + bv) * gl, rc, voff, (mi * 32 + q * 8 + e) * ldc_bytes, kLargeTileStoreAux);
          }
    };
    if ((wave & 1) == 0) {
      out_pair(0, 0, 1, false);
      out_pair(1, 2, 3, false);
      out_pair(2, 4, 0, true);
    } else {
      out_pair(3, 1, 2, false);
      out_pair(4, 3, 4, false);
    }
    return;
  }
  float* C = (float*)p.C[0] + (int64_t)(m0 + wm0) * p.ldc + n0 + wn0;
  const i32x4 rc = make_rsrc(C, 0x7FFFFFFF);
#pragma unroll
  for (int ni = 0; ni < T::NTL; ++ni) {
    const float bv = bias ? bias[n0 + wn0 + ni * 32 + el31] : 0.f;
    const int voff = eg * 4 * ldc_bytes + (ni * 32 + el31) * 4;
#pragma unroll
    for (int mi = 0; mi < T::MT; ++mi)
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          llvm_raw_buffer_store_f32(acc[mi][ni][4 * q + e] + bv, rc, voff, (mi * 32 + q * 8 + e) * ldc_bytes, kLargeTileStoreAux);
  }
}

}  // namespace cascmm
