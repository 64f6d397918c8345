// Two-term bf16 cascade on a prepared right operand, 64 x 80 tile, K split over the waves of a workgroup
// (gfx950): cascmm_slotk_kernel<1> for problems that make only about 128 of its 64 x 160 tiles (the 1024-row
// Linear layers of one GPU's half-latent share).  A CU pulls its operands at a rate of its own, whatever the other
// CUs do, so a launch takes as long as the largest per-CU share of bytes: 256 tiles of 64 x 80 move 576 bytes
// per k and CU (64 fp32 of A, 80 x 2 slots of B) where 128 tiles of 64 x 160 move 896.
//
// An 80-wide tile is five 16-wide blocks, so the MFMA is v_mfma_f32_16x16x32_bf16: a lane supplies row (column)
// lane % 16 and the eight k of k group lane / 16 -- one operand slot of the prepared weight ([term][K/8][N], a
// 16-byte load, 16 lanes reading 256 contiguous bytes) -- and a stage is 32 k, one MFMA deep.  Wave w owns
// stages w, w + 4, ... and the whole tile (4 x 5 blocks, 80 accumulator registers) over them; nothing is
// shared between waves until the four partial tiles meet in LDS at the end.
//   B: straight into registers, two stages ahead (the ring of two stage buffers is refilled block by block).
//   A: raw fp32 rows.  A stage of a row is one 128-byte line; `buffer_load ... lds` brings 64 rows x 128 bytes to
//      a private ring of the wave (eight loads of 1 KB: eight consecutive lanes fetch the eight 16-byte chunks
//      of a row, rotated by a function of half the row number so that the sixteen lanes an LDS read serves
//      together spread over all banks), three stages ahead; the fragments of the next stage are read and split in
//      registers between the MFMAs of the current one.
#pragma once
#include <type_traits>

#include "cascmm_wavek_kernel.h"

namespace cascmm {

struct SlotN {
  static constexpr int BM = 64, BN = 80, BK = 32, NW = 4, NT = 256, GROUP_M = 4;
  static constexpr int MB = 4, NB = 5, BLOCKS = MB * NB;           // 16 x 16 accumulator blocks of a wave
  static constexpr int D = 2;                                      // B: stages in flight (register ring)
  static constexpr int RA = 4, AHEAD = 3, A_STAGE = BM * BK * 4;   // raw A: ring of four stages of 8 KB per wave
  static constexpr int RING = RA * A_STAGE;                        // 32 KB
  static constexpr int BLOCK_BYTES = 64 * 16;                      // one wave's 16 x 16 partial block
  static constexpr int RED_BYTES = NW * BLOCKS * BLOCK_BYTES;      // 80 KB: every wave's partial tile
  static constexpr int LDS_BYTES = NW * RING > RED_BYTES ? NW * RING : RED_BYTES;   // 128 KB
};

// Host-checked: K % 32 == 0, K >= 32, the slot buffer 16-byte aligned and below 2 GiB, A 16-byte aligned with
// lda % 4 == 0 and M * lda * 4 below 2 GiB, C rows addressable with 32-bit byte offsets inside a tile.
// (SlotKParams: a = fp32 [M][lda], b_slots = [2][K/8][N] x 16 bytes.)
template <int UNUSED>
__global__ __launch_bounds__(SlotN::NT) __attribute__((amdgpu_waves_per_eu(1, 1))) void cascmm_slotn_kernel(const SlotKParams p) {
  typedef SlotN T;
  extern __shared__ __attribute__((aligned(1024))) unsigned char slotn_smem[];
  const int tid = threadIdx.x, lane = tid & 63, l15 = lane & 15, kg = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int tm, tn;
  tile_coords((int)blockIdx.x, p.tiles_m, p.tiles_n, tm, tn, p.group_m);
  const int m0 = tm * T::BM, n0 = tn * T::BN;
  const int kgroups = p.K >> 3;
  const int ksteps = p.K >> 5;
  const int n_own = (ksteps - wave + T::NW - 1) / T::NW;   // 0 for the last waves of a very short K: they add zeros
  // The loop runs in trips of two stages without a branch inside; a wave with an odd number of stages runs one
  // stage past its last: its B loads point beyond the end of the buffer and return zeros, its A loads fetch the
  // problem's first stage (finite values for the zeros to multiply).

  // ---- B: lane (l15, kg) reads k group 4 stage + kg of column n0 + 16 nb + l15 ----
  const int b_term = kgroups * p.N * 16, b_end = 2 * b_term;
  const i32x4 rb = make_rsrc(p.b_slots, (int64_t)b_end);
  const int vb = (kg * p.N + n0 + l15) * 16;
  const int b_step = 4 * p.N * 16;
  u32x4 Br[T::D][T::NB][2];
  auto issue_b = [&](int i, int buf, int nb) {
    const int base = i < n_own ? (wave + T::NW * i) * b_step : b_end;
#pragma unroll
    for (int t = 0; t < 2; ++t)
      Br[buf][nb][t] = __builtin_bit_cast(u32x4, llvm_raw_buffer_load_v4f32(rb, vb + nb * 256, base + t * b_term, 0));
  };

  // ---- A: rows past M read as zero (the buffer ends with row M - 1) ----
  const int64_t a_bytes = ((int64_t)(p.M - 1) * p.lda + p.K) * 4;
  const __amdgpu_buffer_rsrc_t rar =
      __builtin_amdgcn_make_buffer_rsrc((void*)p.a, 0, (int)(a_bytes > 0x7FFFFFFF ? 0x7FFFFFFF : a_bytes), 0x00020000);
  unsigned char* ring = slotn_smem + wave * T::RING;
  // Load j of a stage (0 .. 7) brings rows 8 j + lane / 8 to LDS bytes j * 1024 + 16 lane, i.e. lane % 8 is the
  // position inside the row's 128 bytes; position pos of row r holds chunk (pos - rot(h)) mod 8 with h = (r / 2) mod 8
  // = 4 (j mod 2) + lane / 16.  A 16-byte LDS read is served sixteen lanes at a time, and conflict-free when their
  // sixteen 16-byte units (8 (r mod 2) + position) differ.  The sixteen are not consecutive lanes: lanes 0-3, 12-15,
  // 20-23 and 24-27 go together, then 4-7, 8-11, 16-19 and 28-31 (likewise in the upper half of the wave) -- here rows
  // 0-3 and 12-15 of k group 0 with rows 4-11 of k group 1, whose chunks are two further on.  rot = (1, 3, 0, 2, 4, 6,
  // 5, 7) gives the row pairs 0, 1, 6, 7 the odd rotations and the pairs 2 .. 5 the even ones, so that either sixteen
  // cover every unit once (a rotation by h itself reads every fragment in eight passes instead of four: counted).
  auto rot = [](int h) { return (0x75642031u >> (4 * h)) & 7u; };
  int dma_voff[2];
#pragma unroll
  for (int jp = 0; jp < 2; ++jp)
    dma_voff[jp] = (int)(((int64_t)(m0 + (lane >> 3)) * p.lda + (((lane & 7) - (int)rot(4 * jp + (lane >> 4))) & 7) * 4) * 4);
  const int dma_rows8 = (int)p.lda * 32;
  auto dma_a = [&](int i, int j) {
    const int koff = i < n_own ? (wave + T::NW * i) * (T::BK * 4) : 0;
    wavek_load_lds(rar, ring + (i & (T::RA - 1)) * T::A_STAGE + j * 1024, dma_voff[j & 1], koff + j * dma_rows8);
  };
  // fragment of lane (l15, kg), row block mb: row 16 mb + l15, chunks 2 kg and 2 kg + 1 at their rotated places
  int a_frag[2];
#pragma unroll
  for (int x = 0; x < 2; ++x) a_frag[x] = l15 * 128 + ((2 * kg + x + (int)rot(l15 >> 1)) & 7) * 16;
  f32x4 X[T::MB][2];
  u32x4 Ar[2][T::MB][2];   // [stage parity][row block][term]
  auto read_a = [&](int i, int mb) {
    const unsigned char* st = ring + (i & (T::RA - 1)) * T::A_STAGE + mb * 2048;
    X[mb][0] = *(const f32x4*)(st + a_frag[0]);
    X[mb][1] = *(const f32x4*)(st + a_frag[1]);
  };
  auto split_a = [&](int buf, int mb) {
    float r[8] = {X[mb][0][0], X[mb][0][1], X[mb][0][2], X[mb][0][3], X[mb][1][0], X[mb][1][1], X[mb][1][2], X[mb][1][3]};
    u32x4 t[2];
    split8<CASCMM_FMT_BF16, 2>(r, t);
    Ar[buf][mb][0] = t[0];
    Ar[buf][mb][1] = t[1];
  };

  // ---- prologue: A of stages 0 .. AHEAD - 1 first, then B of stages 0 and 1; the wait names exactly the loads
  // issued after stage 0 of A, so what the first fragment reads need has landed ----
#pragma unroll
  for (int d = 0; d < T::AHEAD; ++d)
#pragma unroll
    for (int j = 0; j < 8; ++j) dma_a(d, j);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int d = 0; d < T::D; ++d)
#pragma unroll
    for (int nb = 0; nb < T::NB; ++nb) issue_b(d, d, nb);
  f32x4 acc[T::MB][T::NB];
#pragma unroll
  for (int mb = 0; mb < T::MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < T::NB; ++nb) {
      acc[mb][nb] = (f32x4){0.f, 0.f, 0.f, 0.f};
      // (the zeros are made here, a prologue away from the first MFMA: the MFMAs below are assembly, and the compiler
      // would not keep the distance a register write needs from an MFMA it does not recognise)
      asm volatile("" : "+a"(acc[mb][nb]));
    }
  {
    constexpr int LATER = 8 * (T::AHEAD - 1) + 2 * T::NB * T::D;   // 36
    static_assert(LATER <= 63, "the wait counter has six bits");
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0x0F70 | (LATER & 0xF) | ((LATER >> 4) << 14));
#pragma unroll
    for (int mb = 0; mb < T::MB; ++mb) read_a(0, mb);
#pragma unroll
    for (int mb = 0; mb < T::MB; ++mb) split_a(0, mb);
  }

  // The MFMA as assembly, its accumulator tied to its result in the accumulation registers: left to itself the
  // compiler gives result and addend different registers and moves the eighty accumulators back into place once per
  // trip (120 moves per 120 MFMAs, in a loop that is bound by the number of instructions the wave can issue: an MFMA
  // of this shape holds the matrix pipe for 16 cycles, four instructions' worth).  The compiler's hazard handling does
  // not see such an MFMA: consecutive ones write different accumulators, and the accumulators are read only after the
  // loop and a pause (below).
  auto mfma = [&](const u32x4& a, const u32x4& b, f32x4& c) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  };
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  typedef float f32x2v __attribute__((ext_vector_type(2)));
  // The split of pair e (elements 2 e, 2 e + 1 of a lane's eight) of row block mb in three steps of two VALU
  // instructions, one step behind each MFMA: {hi pair, hi of the even element as fp32}, {its residual, hi of the odd
  // element}, {its residual, lo pair}.
  unsigned hp = 0;
  float hf = 0.f;
  auto split_step = [&](int buf, int mb, int e, int t) {
    const int q = e >> 1, c0 = (2 * e) & 3, c1 = c0 + 1;
    if (t == 0) {
      const f32x2v v = {X[mb][q][c0], X[mb][q][c1]};
      hp = __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2));
      Ar[buf][mb][0][e] = hp;
      hf = __builtin_bit_cast(float, hp << 16);
    } else if (t == 1) {
      X[mb][q][c0] = X[mb][q][c0] - hf;
      hf = __builtin_bit_cast(float, hp & 0xFFFF0000u);
    } else {
      const f32x2v r = {X[mb][q][c0], X[mb][q][c1] - hf};
      Ar[buf][mb][1][e] = __builtin_bit_cast(unsigned, __builtin_convertvector(r, bf16x2));
    }
  };
  auto issue_b1 = [&](int i, int buf, int nb, int t) {
    const int base = i < n_own ? (wave + T::NW * i) * b_step : b_end;
    Br[buf][nb][t] = __builtin_bit_cast(u32x4, llvm_raw_buffer_load_v4f32(rb, vb + nb * 256, base + t * b_term, 0));
  };
#define SLOTN_FENCE() __builtin_amdgcn_sched_barrier(0)
  // Stage i, buffers u = i % 2.  At its top: the eight loads of A's stage i + AHEAD into the ring (that place was
  // last read during stage i - 2), then the wait for A's stage i + 1 -- requested at the top of stage i + 1 - AHEAD,
  // followed since by the ten B loads of that stage, one whole stage and the eight loads just issued: at most
  // 10 + 18 (AHEAD - 2) + 8 loads may still be outstanding -- and the fragment reads of stage i + 1.  Then the
  // twelve MFMAs of each column block (lo.hi, hi.lo, hi.hi over the four row blocks: consecutive MFMAs on different
  // accumulators).  Behind MFMA g of block nb: a step of the split of row block nb of stage i + 1 (nb < 4; the LDS
  // answers in order, so one wait in front of the block's first step covers its two reads), and behind the first two
  // MFMAs one of the two slot loads that refill block nb - 1 for stage i + 2 (its last MFMA has been issued);
  // block 4's follow the stage's last MFMA.
  for (int i0 = 0; i0 < n_own; i0 += 2) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int i = i0 + u;
#pragma unroll
      for (int j = 0; j < 8; ++j) dma_a(i + T::AHEAD, j);
      {
        constexpr int YOUNGER = 2 * T::NB + 18 * (T::AHEAD - 2) + 8;   // 36
        static_assert(YOUNGER <= 63, "the wait counter has six bits");
        SLOTN_FENCE();
        __builtin_amdgcn_s_waitcnt(0x0F70 | (YOUNGER & 0xF) | ((YOUNGER >> 4) << 14));
      }
#pragma unroll
      for (int mb = 0; mb < T::MB; ++mb) read_a(i + 1, mb);
      SLOTN_FENCE();
#pragma unroll
      for (int nb = 0; nb < T::NB; ++nb) {
#pragma unroll
        for (int g = 0; g < 12; ++g) {
          const int prod = g >> 2, mb = g & 3;
          mfma(prod == 0 ? Ar[u][mb][1] : Ar[u][mb][0], prod == 1 ? Br[u][nb][1] : Br[u][nb][0], acc[mb][nb]);
          SLOTN_FENCE();
          if (g == 0) {   // lgkmcnt(6 - 2 nb): the reads of the later row blocks may still be on their way
            if (nb == 0) __builtin_amdgcn_s_waitcnt(0xC67F);
            if (nb == 1) __builtin_amdgcn_s_waitcnt(0xC47F);
            if (nb == 2) __builtin_amdgcn_s_waitcnt(0xC27F);
            if (nb == 3) __builtin_amdgcn_s_waitcnt(0xC07F);
            SLOTN_FENCE();
          }
          if (nb < T::MB) split_step(u ^ 1, nb, g / 3, g % 3);
          if (nb >= 1 && g < 2) issue_b1(i + T::D, u, nb - 1, g);
          SLOTN_FENCE();
        }
      }
      issue_b1(i + T::D, u, T::NB - 1, 0);
      issue_b1(i + T::D, u, T::NB - 1, 1);
      SLOTN_FENCE();
    }
  }
#undef SLOTN_FENCE
  // the passes of the last MFMAs have to drain before the accumulators are read (the compiler does not know)
  asm volatile("s_nop 7\n s_nop 7" ::: "memory");

  // ---- the four partial tiles meet in LDS: every wave puts its twenty blocks at [wave][block] (16 bytes per
  // lane), wave w then adds the four partial sums of blocks w, w + 4, ... in wave order and stores them ----
  __builtin_amdgcn_s_waitcnt(0x0F70);   // every load into the rings has landed; the area overlaps them
  __syncthreads();
#pragma unroll
  for (int b = 0; b < T::BLOCKS; ++b)
    *(f32x4*)(slotn_smem + (wave * T::BLOCKS + b) * T::BLOCK_BYTES + lane * 16) = acc[b / T::NB][b % T::NB];
  __syncthreads();
  const int ldc_bytes = (int)p.ldc * 4;
  // rows past M fall beyond the end of the buffer and are dropped
  const int64_t c_bytes64 = ((int64_t)(p.M - 1 - m0) * p.ldc + (p.N - n0)) * 4;
  const int c_bytes = (int)(c_bytes64 > 0x7FFFFFFF ? 0x7FFFFFFF : c_bytes64);
  const i32x4 rc = make_rsrc(p.C + (int64_t)m0 * p.ldc + n0, c_bytes);
#pragma unroll
  for (int x = 0; x < T::BLOCKS / T::NW; ++x) {
    const int b = wave + T::NW * x;          // (wave-uniform)
    const int mb = b / T::NB, nb = b % T::NB;
    f32x4 sum = *(const f32x4*)(slotn_smem + b * T::BLOCK_BYTES + lane * 16);
#pragma unroll
    for (int w = 1; w < T::NW; ++w) sum += *(const f32x4*)(slotn_smem + (w * T::BLOCKS + b) * T::BLOCK_BYTES + lane * 16);
    // a lane holds column l15 of the block, rows 4 kg + e; columns past N (a ragged last tile; their slots were
    // some other column's) are sent beyond the end of the buffer
    const int col = nb * 16 + l15;
    const bool inside = n0 + col < p.N;
    const float bv = (p.bias && inside) ? p.bias[n0 + col] : 0.f;
    const int voff = inside ? kg * 4 * ldc_bytes + col * 4 : c_bytes;
#pragma unroll
    for (int e = 0; e < 4; ++e) llvm_raw_buffer_store_f32(sum[e] + bv, rc, voff, (mb * 16 + e) * ldc_bytes, kResultStoreAux);
  }
}

}  // namespace cascmm
