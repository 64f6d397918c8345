// Three-term fp16 cascade on operand slots (gfx950): the fp16 counterparts of cascmm_f8k64_kernel<2> (256 x 160
// tile staged through LDS, for problems of many tiles) and cascmm_f8wk_kernel (64 x 160 tile with K split over
// the waves of a workgroup, for problems of about one tile per CU), with the passes that write the slots.
//
// Terms.  With the tensor scaled by a power of two 2^e so that max|x| 2^e lies in (7, 14], y = x 2^e:
//   u0 = fp16(y), r1 = y - u0;  u1 = fp16(r1 2^11), r2 = r1 - u1 2^-11;  u2 = fp16(r2 2^22)
// (the cascade's three terms with its 11-bit term shift; every residual is exact in fp32).  What is stored is
//   S0 = u0 2^11,  S1 = u1,  S2 = u2 2^-11
// (S0 exact: |u0| <= 14; S2 may lose low bits of elements below 2^-3 of the maximum to fp16's subnormal range:
// an error of 2^-36 of the maximum at most, far below the product terms the cascade drops).  Every kept product
// S_i S_j, i + j <= 2, then carries the same factor 2^22 on the true product of the scaled operands, so all six go
// into one sum and no accumulator per scale class is needed; the store multiplies by 2^-(22 + e_A + e_B).
//
// Accumulation.  A result at the fp32 rounding floor is spoilt by every addition into a long running sum, whatever
// the size of what is added.  The MFMAs of a 32 x 32 block (twelve per 32-k stage: six products x two 16-k halves)
// are chained in a temporary block over four stages, starting from zero; the temporary is then added to the
// block's running sum by VALU additions placed behind the MFMAs of the next block: one rounding of the running
// sum per 128 k instead of 48.
//
// Slots: 16 bytes = 8 consecutive k of one row (column) of one stored term, [term][K/8][rows]; a stage is four
// slot columns, 32 k.  A lane's fragment of a stage is slot columns 2 h and 2 h + 1 (h = lane / 32), eight
// registers as in the fp8 kernels; the MFMA of half s takes registers 4 s .. 4 s + 3 of both operands, i.e. slot
// column 2 h + s: the order of k inside a stage is the same permutation for both operands.
#pragma once
#include <type_traits>

#include "cascmm_f8wk_kernel.h"

namespace cascmm {

constexpr int kF16KResultExp = 22;   // the factor 2^22 that every stored product carries

struct F16K {
  static constexpr int MT = 2, NTL = 5;                    // 32 x 32 blocks of a wave: MT x NTL
  static constexpr int WTM = 32 * MT, BM = 4 * WTM, BN = 160, BK = 32, NT = 256, TERMS = 3;
  static constexpr int KU = 4;                             // 8-k slot columns per stage
  static constexpr int A_STAGE = TERMS * KU * BM * 16;     // 48 KB
  static constexpr int B_STAGE = TERMS * KU * BN * 16;     // 30 KB
  static constexpr int STAGE = A_STAGE + B_STAGE;          // 78 KB
  static constexpr int LDS_BYTES = 2 * STAGE;              // 156 KB
  static constexpr int A_LOADS = TERMS * KU * BM / 64 / 4; // 12 per wave
  static constexpr int B_LOADS_MAX = 8;                    // 30 instructions over 4 waves: 8, 8, 7, 7
  static constexpr int LOADS = A_LOADS + B_LOADS_MAX;      // 20
  // The running sum of a block takes one addition per 128 k and the temporaries are not chained over more: beyond
  // this depth the kernel is not offered (its error has been checked against the oracle's up to here; the
  // K-over-waves kernel, whose waves each see a quarter of K, takes deeper problems).
  static constexpr int MAX_K = 1536;
};

struct F16WK {
  static constexpr int BM = 64, BN = 160, BK = 32, NW = 4, NT = 256, TERMS = 3, GROUP_M = 8;
  static constexpr int MT = 2, NTL = 5, BLOCKS = MT * NTL;
  static constexpr int BLOCK_BYTES = 16 * 64 * 4;              // one wave's 32 x 32 block of running sums
  static constexpr int WAVE_BYTES = BLOCKS * BLOCK_BYTES;      // 40 KB
  static constexpr int LDS_BYTES = NW * WAVE_BYTES;            // 160 KB: the four waves' running sums
};

inline __host__ __device__ int64_t f16k_slot_bytes(int64_t rows, int64_t K) {
  int64_t slots = 0, bytes = 0;
  if (__builtin_mul_overflow((int64_t)F16K::TERMS * (K / 8), rows, &slots) || __builtin_mul_overflow(slots, (int64_t)16, &bytes))
    return INT64_MAX;
  return bytes;
}

// the exponent e with max|x| 2^e in (7, 14]
// (kept within +-60 so that the scales and their product stay normal fp32 numbers: a tensor whose largest element
// is below 2^-57 is split less finely, and one whose largest element is above 2^64 overflows fp16 in its first
// term, as the cascade without a tensor scale does above 65504)
__device__ __forceinline__ int f16k_exp_of_amax(unsigned bits) {
  if (bits == 0) return 0;
  const int e = exp_of_amax(bits) - 5;
  return e < -60 ? -60 : e > 60 ? 60 : e;
}

// eight consecutive k of a row or column -> the three stored terms
__device__ __forceinline__ void f16k_split8(const float (&x)[8], float scale, u32x4 (&t)[3]) {
  f16x8 s0, s1, s2;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float y = x[e] * scale;
    const _Float16 u0 = (_Float16)y;
    const float r1 = y - (float)u0;
    const _Float16 u1 = (_Float16)(r1 * 2048.f);
    const float r2 = __builtin_fmaf(-(float)u1, 1.f / 2048.f, r1);
    const _Float16 u2 = (_Float16)(r2 * 4194304.f);
    s0[e] = (_Float16)((float)u0 * 2048.f);
    s1[e] = u1;
    s2[e] = (_Float16)((float)u2 * (1.f / 2048.f));
  }
  t[0] = __builtin_bit_cast(u32x4, s0);
  t[1] = __builtin_bit_cast(u32x4, s1);
  t[2] = __builtin_bit_cast(u32x4, s2);
}

// max|x| over the finite elements of a workgroup's share of A [M, K] (workgroups 0 .. n_a - 1) or of B [K, N] (the
// others), as a bit pattern -> amax_a[0 .. n_a) and amax_b[0 .. gridDim.x - n_a): one launch for both operands
template <int UNUSED>
__global__ __launch_bounds__(1024) void f16k_amax_kernel(const float* __restrict__ A, int64_t M, int64_t K, int64_t lda, int n_a,
                                                        const float* __restrict__ B, int64_t N, int64_t ldb,
                                                        unsigned* __restrict__ amax_a, unsigned* __restrict__ amax_b) {
  __shared__ unsigned wave_best[16];
  const bool left = (int)blockIdx.x < n_a;
  const unsigned best = left ? amax_scan<CASCMM_DT_F32, true>(A, M, K, lda, blockIdx.x, n_a)
                             : amax_scan<CASCMM_DT_F32, true>(B, K, N, ldb, blockIdx.x - n_a, gridDim.x - n_a);
  if ((threadIdx.x & 63) == 0) wave_best[threadIdx.x >> 6] = best;
  __syncthreads();
  if (threadIdx.x != 0) return;
  unsigned b = 0;
  for (unsigned w = 0; w < (blockDim.x >> 6); ++w) b = wave_best[w] > b ? wave_best[w] : b;
  if (left) amax_a[blockIdx.x] = b;
  else amax_b[blockIdx.x - n_a] = b;
}

// every workgroup of a split kernel reduces the per-workgroup maxima itself (1 KB from L2, behind its loads);
// the first one leaves the exponent in *exp_out for the GEMM
__device__ __forceinline__ int f16k_find_exp(const unsigned* __restrict__ amax, int n_amax, int32_t* __restrict__ exp_out, int* shared_e, bool first) {
  if (threadIdx.x < 64) {
    unsigned best = 0;
    for (int i = threadIdx.x; i < n_amax; i += 64) best = amax[i] > best ? amax[i] : best;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const unsigned other = (unsigned)__shfl_xor((int)best, off, 64);
      best = other > best ? other : best;
    }
    if (threadIdx.x == 0) {
      *shared_e = f16k_exp_of_amax(best);
      if (first) *exp_out = *shared_e;
    }
  }
  __syncthreads();
  return *shared_e;
}

// Split of the LEFT operand: A [M, K] fp32 row-major -> slots[term][K/8][M].  A workgroup converts 64 rows x 32 k
// (a thread: 8 consecutive k of a row) and transposes through LDS so that the slots leave as 1 KB runs along M.
__device__ __forceinline__ void f16k_split_rows(int block, const float* __restrict__ A, int M, int K, int64_t lda, u32x4* __restrict__ out,
                                                float scale, u32x4 (*slots)[4][64]) {
  const int kus = K >> 3;
  const int ku_tiles = (kus + 3) >> 2;
  const int m0 = (block / ku_tiles) * 64, ku0 = (block % ku_tiles) * 4;
  {
    const int row = threadIdx.x >> 2, ku = threadIdx.x & 3;
    if (m0 + row < M && ku0 + ku < kus) {
      const float* src = A + (int64_t)(m0 + row) * lda + (ku0 + ku) * 8;
      const f32x4 v0 = *(const f32x4*)src, v1 = *(const f32x4*)(src + 4);
      const float r[8] = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
      u32x4 t[3];
      f16k_split8(r, scale, t);
#pragma unroll
      for (int i = 0; i < 3; ++i) slots[i][ku][row] = t[i];
    }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    const int v = threadIdx.x + 256 * i;
    const int row = v & 63, ku = (v >> 6) & 3, term = v >> 8;
    if (m0 + row < M && ku0 + ku < kus) out[((int64_t)term * kus + ku0 + ku) * M + m0 + row] = slots[term][ku][row];
  }
}

// Split of the RIGHT operand: B [K, N] fp32 row-major -> slots[term][K/8][N]; thread (ku, n) walks 8 rows of
// column n (consecutive threads: consecutive columns, coalesced both ways).
__device__ __forceinline__ void f16k_split_cols(int block, const float* __restrict__ B, int K, int N, int64_t ldb, u32x4* __restrict__ out,
                                                float scale) {
  const int kus = K >> 3;
  const int64_t i = (int64_t)block * 256 + threadIdx.x;
  if (i >= (int64_t)kus * N) return;
  const int ku = (int)(i / N), n = (int)(i - (int64_t)ku * N);
  const float* src = B + (int64_t)ku * 8 * ldb + n;
  float r[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) r[e] = src[(int64_t)e * ldb];
  u32x4 t[3];
  f16k_split8(r, scale, t);
#pragma unroll
  for (int j = 0; j < 3; ++j) out[((int64_t)j * kus + ku) * N + n] = t[j];
}

// Both splits in one launch: workgroups 0 .. a_blocks - 1 split A, the others B.  Every workgroup first reduces its
// operand's per-workgroup maxima; exps_out[0] = e_A, exps_out[1] = e_B are left by the first workgroup of either part.
template <int UNUSED>
__global__ __launch_bounds__(256) void f16k_split_kernel(const float* __restrict__ A, int M, int K, int64_t lda, u32x4* __restrict__ a_out,
                                                        const unsigned* __restrict__ amax_a, int n_a, int a_blocks,
                                                        const float* __restrict__ B, int N, int64_t ldb, u32x4* __restrict__ b_out,
                                                        const unsigned* __restrict__ amax_b, int n_b, int32_t* __restrict__ exps_out) {
  __shared__ u32x4 slots[3][4][64];
  __shared__ int e_found;
  const bool left = (int)blockIdx.x < a_blocks;
  const int block = left ? (int)blockIdx.x : (int)blockIdx.x - a_blocks;
  const float scale = __builtin_ldexpf(1.f, f16k_find_exp(left ? amax_a : amax_b, left ? n_a : n_b, exps_out + (left ? 0 : 1), &e_found, block == 0));
  if (left) f16k_split_rows(block, A, M, K, lda, a_out, scale, slots);
  else f16k_split_cols(block, B, K, N, ldb, b_out, scale);
}

__device__ __forceinline__ f16x8 f16k_half(const i32x8& v, int s) {
  return __builtin_bit_cast(f16x8, (u32x4){(unsigned)v[4 * s], (unsigned)v[4 * s + 1], (unsigned)v[4 * s + 2], (unsigned)v[4 * s + 3]});
}

// ---------------------------------------------------------------------------------------------------
// 256 x 160 tile staged through LDS: the data path of cascmm_f8k64_kernel<2> (wave-wide `buffer_load ... lds`
// of slots, double-buffered stages of 78 KB, one barrier per stage in front of its last column block, A
// fragments of a whole stage and B fragments of one column block double buffered in registers), with 120
// MFMAs of 32 cycles per stage where the fp8 kernel has 60 of 64.
// Host-checked: K % 32 == 0, 32 <= K <= MAX_K, the slot buffers below 2 GiB, C rows addressable with 32-bit byte
// offsets inside a tile; p.k_splits is not used.
// ---------------------------------------------------------------------------------------------------
template <int UNUSED>
__global__ __launch_bounds__(F16K::NT) __attribute__((amdgpu_waves_per_eu(1, 1))) void cascmm_f16k_kernel(const F8K64Params p) {
  typedef F16K T;
  extern __shared__ __attribute__((aligned(1024))) unsigned char f16k_smem[];
  unsigned char* smem = f16k_smem;
  const int tid = threadIdx.x, lane = tid & 63, l31 = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = wave * T::WTM;
  int tm, tn;
  tile_coords((int)blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
  const int m0 = tm * T::BM, n0 = tn * T::BN;
  const int ksteps = p.K / T::BK;
  const int kus = p.K >> 3;

  const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc((void*)p.a_slots, 0, 0x7FFFFFFF, 0x00020000);
  const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc((void*)p.b_slots, 0, 0x7FFFFFFF, 0x00020000);
  // A: a stage holds, per (term, ku), BM slots = four runs of 64 rows, run r at byte r * 1024; this wave loads
  // runs wave, wave + 4, ...; lane = row inside the run (clamped to the last valid row)
  const int a_plane = kus * p.M * 16;          // bytes between terms
  const int a_ku = p.M * 16;                   // bytes between slot columns
  constexpr int CH = T::BM / 64;
  static_assert(CH == 4, "run wave + 4 j is chunk `wave` of (term, ku) j: one row offset for every load");
  int a_row = m0 + wave * 64 + lane;
  a_row = a_row < p.M ? a_row : p.M - 1;
  const int a_voff = a_row * 16;
  int a_soff[T::A_LOADS];
#pragma unroll
  for (int j = 0; j < T::A_LOADS; ++j) a_soff[j] = (j / T::KU) * a_plane + (j % T::KU) * a_ku;   // j = term * KU + ku
  // B: the stage's 1920 slots as 30 runs of 64; this wave takes runs wave, wave + 4, ...
  int b_voff[T::B_LOADS_MAX], b_lds[T::B_LOADS_MAX];
#pragma unroll
  for (int j = 0; j < T::B_LOADS_MAX; ++j) {
    int run = wave + 4 * j;
    run = run < 30 ? run : 29;                 // (waves 2 and 3 repeat their last run: same bytes to the same place)
    const int s = run * 64 + lane;
    const int term = s / (T::KU * T::BN), ku = (s / T::BN) % T::KU;
    int col = n0 + s % T::BN;
    col = col < p.N ? col : p.N - 1;
    b_lds[j] = T::A_STAGE + run * 1024;
    b_voff[j] = ((term * kus + ku) * p.N + col) * 16;
  }
  const int b_step = T::KU * p.N * 16;         // bytes per stage
  auto issue_a = [&](int step_, int j) {
    const int step = step_ < ksteps - 1 ? step_ : ksteps - 1;
    f8k64_load_lds(ra, smem + (step_ & 1) * T::STAGE + (wave + 4 * j) * 1024, a_voff, a_soff[j] + step * T::KU * a_ku);
  };
  auto issue_b = [&](int step_, int j) {
    const int step = step_ < ksteps - 1 ? step_ : ksteps - 1;
    f8k64_load_lds(rb, smem + (step_ & 1) * T::STAGE + b_lds[j], b_voff[j], step * b_step);
  };

  // fragment addresses inside a stage: lane (row l31, half h) reads slots (term, ku = 2 h) and (term, 2 h + 1)
  const int a_frag = (2 * h * T::BM + wm0 + l31) * 16;                  // + term * KU * BM * 16 + mi * 512, second slot + BM * 16
  const int b_frag = T::A_STAGE + (2 * h * T::BN + l31) * 16;           // + term * KU * BN * 16 + ni * 512, second slot + BN * 16

  // acc: the running sums, added to by VALU instructions only; X: the sums of up to four stages, the MFMAs' accumulators
  f32x16 acc[T::MT][T::NTL];
  f32x16 X[T::MT][T::NTL];
#pragma unroll
  for (int mi = 0; mi < T::MT; ++mi)
#pragma unroll
    for (int ni = 0; ni < T::NTL; ++ni)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[mi][ni][e] = X[mi][ni][e] = 0.f;

#define F16K_FENCE() __builtin_amdgcn_sched_barrier(0)
  auto issue = [&](int step_, int k) {     // load k (0 .. LOADS - 1) of a stage: those of A, then 8 of B
    if (k < T::A_LOADS) issue_a(step_, k);
    else issue_b(step_, k - T::A_LOADS);
  };
  auto frag = [&](const unsigned char* base, int second) {
    const u32x4 lo = *(const u32x4*)base, hi = *(const u32x4*)(base + second);
    return (i32x8){(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
  };

#pragma unroll
  for (int k = 0; k < T::LOADS; ++k) issue(0, k);

  // Fragments: A of the whole stage (the wave's own rows) and B of one column block, each held ONCE: the products
  // of a block run in an order in which every term of either operand is done with at least two products (eight
  // MFMAs) before the next block, or the next stage, needs it again, and its registers are refilled in that time.
  i32x8 a[T::TERMS][T::MT];
  i32x8 b[T::TERMS];
  auto read_a = [&](const unsigned char* st, int t) {
#pragma unroll
    for (int mi = 0; mi < T::MT; ++mi) a[t][mi] = frag(st + a_frag + t * T::KU * T::BM * 16 + mi * 512, T::BM * 16);
  };
  auto read_b = [&](const unsigned char* st, int ni, int t) {
    b[t] = frag(st + b_frag + t * T::KU * T::BN * 16 + ni * 512, T::BN * 16);
  };
  __builtin_amdgcn_s_waitcnt(0x0F70);       // vmcnt(0): stage 0 has landed
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int t = 0; t < T::TERMS; ++t) {
    read_a(smem, t);
    read_b(smem, 0, t);
  }
  // the first six loads of stage 1 before stage 0 begins (the others follow inside stage 0)
#pragma unroll
  for (int k = 0; k < 6; ++k) issue(1, k);

  const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  // Every column block is folded into the running sums after the stages s with s % 4 == 3 (every 128 k: the same
  // k for every block, so a column's result does not depend on where in the matrix it stands), by VALU additions
  // behind the MFMAs of the block that follows it; its next MFMA then starts from zero.  The loop is unrolled by
  // four stages so that all of this is static.
  // The barrier that opens stage s + 1 sits in front of the LAST column block of stage s: by then the wave has read
  // everything it needs of stage s from LDS, so the first fragments of stage s + 1 are read behind that block's MFMAs.
  auto stage = [&](int s, auto PH) {
    constexpr int ph = decltype(PH)::value;        // s % 4
    const unsigned char* st = smem + (s & 1) * T::STAGE;
    const unsigned char* st_next = smem + ((s + 1) & 1) * T::STAGE;
#pragma unroll
    for (int ni = 0; ni < T::NTL; ++ni) {
      // the block before this one (of the stage before: its last) and whether it is folded now
      const int pni = ni == 0 ? T::NTL - 1 : ni - 1;
      const bool fold_prev = ni == 0 ? ph == 0 : ph == 3;
      const bool from_zero = ph == 0;                   // folded after the stage before
      const bool last = ni == T::NTL - 1;
      if (last) {
        // everything this wave needs of stage s is in registers: open stage s + 1 (own loads of it have landed,
        // own reads of stage s have returned; the loads that follow the barrier overwrite that buffer)
        __builtin_amdgcn_s_waitcnt(0x0070);     // vmcnt(0), lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
      }
      // where the next block's fragments come from
      const unsigned char* nb = last ? st_next : st;
      const int nni = last ? 0 : ni + 1;
      int n_issued = 0;
      auto gap = [&]() {     // behind every second MFMA; products end behind gaps 1, 3, 5, 7, 9, 11
        F16K_FENCE();
        // B of the next block: term 2 is done with after product 1, term 1 after product 5, term 0 after product 6
        if (n_issued == 2) read_b(nb, nni, 2);
        if (n_issued == 10) read_b(nb, nni, 1);
        if (n_issued == 11) read_b(nb, nni, 0);
        if (!last) {
          // loads 6 .. 19 of stage s + 1 (its buffer was given up at the barrier inside stage s - 1): gaps 3 .. 9 of
          // blocks 0 and 1, which leaves them two and a half blocks to land
          if (ni < 2 && n_issued >= 3 && n_issued <= 9) issue(s + 1, 6 + 7 * ni + n_issued - 3);
        } else {
          // A of the next stage: term 0 is done with after product 3, term 1 after product 5, term 2 after product 6;
          // and loads 0 .. 5 of stage s + 2
          if (n_issued == 6) read_a(st_next, 0);
          if (n_issued == 10) read_a(st_next, 1);
          if (n_issued == 11) read_a(st_next, 2);
          if (n_issued >= 3 && n_issued <= 5) issue(s + 2, n_issued - 3);
          if (n_issued >= 7 && n_issued <= 9) issue(s + 2, n_issued - 4);
        }
        // three of the 32 additions of a fold (the last MFMA of that block is at least four MFMAs old from gap 1 on)
        if (fold_prev && n_issued >= 1) {
#pragma unroll
          for (int u = 0; u < 3; ++u) {
            const int x = (n_issued - 1) * 3 + u;
            if (x < 32) acc[x >> 4][pni][x & 15] += X[x >> 4][pni][x & 15];
          }
        }
        F16K_FENCE();
        ++n_issued;
      };
#define F16K_PRODUCT(I, J, FIRST)                                                                                           \
  _Pragma("unroll") for (int s2 = 0; s2 < 2; ++s2) {                                                                        \
    _Pragma("unroll") for (int mi = 0; mi < T::MT; ++mi)                                                                    \
      X[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f16k_half(a[I][mi], s2), f16k_half(b[J], s2),                      \
                                                         (FIRST) && s2 == 0 && from_zero ? zero : X[mi][ni], 0, 0, 0);      \
    gap();                                                                                                                  \
  }
      F16K_PRODUCT(0, 2, true)
      F16K_PRODUCT(0, 1, false)
      F16K_PRODUCT(0, 0, false)
      F16K_PRODUCT(1, 0, false)
      F16K_PRODUCT(1, 1, false)
      F16K_PRODUCT(2, 0, false)
#undef F16K_PRODUCT
    }
  };
  int s = 0;
  for (; s + 4 <= ksteps; s += 4) {
    stage(s, std::integral_constant<int, 0>{});
    stage(s + 1, std::integral_constant<int, 1>{});
    stage(s + 2, std::integral_constant<int, 2>{});
    stage(s + 3, std::integral_constant<int, 3>{});
  }
  if (s < ksteps) stage(s, std::integral_constant<int, 0>{});
  if (s + 1 < ksteps) stage(s + 1, std::integral_constant<int, 1>{});
  if (s + 2 < ksteps) stage(s + 2, std::integral_constant<int, 2>{});
#undef F16K_FENCE
  __builtin_amdgcn_s_waitcnt(0x0F70);       // the redundant loads of the last stage land before LDS is given up
  // what the temporaries still hold: after a last stage with s % 4 == 3 only the last block's sums (the others were
  // folded behind the blocks that followed them), otherwise the sums of every block since the last fold
  const bool folded = ((ksteps - 1) & 3) == 3;
#pragma unroll
  for (int ni = 0; ni < T::NTL; ++ni) {
    if (ni < T::NTL - 1 && folded) continue;
#pragma unroll
    for (int mi = 0; mi < T::MT; ++mi) acc[mi][ni] += X[mi][ni];
  }

  // ---- epilogue: undo the scales, add the bias; a lane holds column l31, rows 8 q + 4 h + e ----
  const float out_scale = __builtin_ldexpf(1.f, -(p.tensor_exps[0] + p.tensor_exps[1]) - kF16KResultExp);
  const int row_base = m0 + wm0 + 4 * h;
  if (m0 + T::BM <= p.M && n0 + T::BN <= p.N && p.ldc * (int64_t)(T::BM * 4) < 0x7FFFFFFF) {
    // whole tile inside C: buffer stores, the row as a scalar offset, nothing to mask
    const i32x4 rc = make_rsrc(p.C + (int64_t)(m0 + wm0) * p.ldc + n0, 0x7FFFFFFF);
    const int ldc_bytes = (int)p.ldc * 4;
#pragma unroll
    for (int ni = 0; ni < T::NTL; ++ni) {
      const float bv = p.bias ? p.bias[n0 + ni * 32 + l31] : 0.f;
      const int voff = h * 4 * ldc_bytes + (ni * 32 + l31) * 4;
#pragma unroll
      for (int mi = 0; mi < T::MT; ++mi)
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int e = 0; e < 4; ++e)
            llvm_raw_buffer_store_f32(acc[mi][ni][4 * q + e] * out_scale + bv, rc, voff, (mi * 32 + q * 8 + e) * ldc_bytes, kLargeTileStoreAux);
    }
    return;
  }
#pragma unroll
  for (int ni = 0; ni < T::NTL; ++ni) {
    const int col = n0 + ni * 32 + l31;
    if (col >= p.N) continue;
    const float bv = p.bias ? p.bias[col] : 0.f;
#pragma unroll
    for (int mi = 0; mi < T::MT; ++mi)
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int row = row_base + mi * 32 + q * 8 + e;
          if (row < p.M) p.C[(int64_t)row * p.ldc + col] = acc[mi][ni][4 * q + e] * out_scale + bv;
        }
  }
}

// ---------------------------------------------------------------------------------------------------
// 64 x 160 tile with K split over the four waves of a workgroup: the data path of cascmm_f8wk_kernel (both
// operands as slots straight into registers, a stage ahead; no LDS and no barrier in the loop; the four partial
// tiles meet in LDS at the end and are added in wave order).  Wave w owns the 32-k stages w, w + 4, ...: a
// quarter of the additions into a running sum, so K is not limited.
// Host-checked: K % 32 == 0, K >= 32, the slot buffers 16-byte aligned and below 2 GiB, C rows addressable with
// 32-bit byte offsets inside a tile.
// ---------------------------------------------------------------------------------------------------
template <int UNUSED>
__global__ __launch_bounds__(F16WK::NT) __attribute__((amdgpu_waves_per_eu(1, 1))) void cascmm_f16wk_kernel(const F8K64Params p) {
  typedef F16WK T;
  extern __shared__ __attribute__((aligned(1024))) unsigned char f16wk_smem[];
  const int tid = threadIdx.x, lane = tid & 63, l31 = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  int tm, tn;
  tile_coords((int)blockIdx.x, p.tiles_m, p.tiles_n, tm, tn, T::GROUP_M);
  const int m0 = tm * T::BM, n0 = tn * T::BN;
  const int kus = p.K >> 3;          // 8-k slot columns
  const int ksteps = p.K >> 5;       // 32-k stages
  const int n_own = (ksteps - wave + T::NW - 1) / T::NW;   // 0 for the last waves of a very short K: they add zeros

  // a stage past the wave's last one is loaded from beyond the end of the buffers, which returns zeros (the loop
  // has no branch inside a trip of two stages)
  const int a_ku = p.M * 16, a_plane = kus * a_ku, a_end = T::TERMS * a_plane;
  const int b_ku = p.N * 16, b_plane = kus * b_ku, b_end = T::TERMS * b_plane;
  const i32x4 ra = make_rsrc(p.a_slots, (int64_t)a_end);
  const i32x4 rb = make_rsrc(p.b_slots, (int64_t)b_end);
  const int va = (2 * h * p.M + m0 + l31) * 16;
  const int vb = (2 * h * p.N + n0 + l31) * 16;
  auto load2 = [&](const i32x4& r, int voff, int soff, int second) {
    const f32x4 lo = llvm_raw_buffer_load_v4f32(r, voff, soff, 0), hi = llvm_raw_buffer_load_v4f32(r, voff, soff + second, 0);
    const u32x4 l = __builtin_bit_cast(u32x4, lo), u = __builtin_bit_cast(u32x4, hi);
    return (i32x8){(int)l[0], (int)l[1], (int)l[2], (int)l[3], (int)u[0], (int)u[1], (int)u[2], (int)u[3]};
  };
  i32x8 a[2][T::TERMS][T::MT];      // [stage parity][term][row block]
  i32x8 b[T::TERMS][T::NTL - 1];    // column blocks 0 .. 3: refilled for the next stage right after their MFMAs
  i32x8 b4[2][T::TERMS];            // column block 4, by stage parity
  auto a_base = [&](int i) { return i < n_own ? (wave + T::NW * i) * 4 * a_ku : a_end; };
  auto b_base = [&](int i) { return i < n_own ? (wave + T::NW * i) * 4 * b_ku : b_end; };
  auto issue_a = [&](int i, int buf, int t, int mi) { a[buf][t][mi] = load2(ra, va + mi * 512, a_base(i) + t * a_plane, a_ku); };
  auto issue_b = [&](int i, int t, int ni) { b[t][ni] = load2(rb, vb + ni * 512, b_base(i) + t * b_plane, b_ku); };
  auto issue_b4 = [&](int i, int buf, int t) { b4[buf][t] = load2(rb, vb + 4 * 512, b_base(i) + t * b_plane, b_ku); };

#pragma unroll
  for (int t = 0; t < T::TERMS; ++t) {
#pragma unroll
    for (int mi = 0; mi < T::MT; ++mi) issue_a(0, 0, t, mi);
#pragma unroll
    for (int ni = 0; ni < T::NTL - 1; ++ni) issue_b(0, t, ni);
    issue_b4(0, 0, t);
  }
  // X: the MFMAs' accumulators, the sums of up to two own stages.  The running sums of the wave live in LDS (its own
  // 40 KB: block b at b * 4096, 16 bytes per lane and register quad), where the four waves' tiles meet at the end.
  f32x16 X[T::MT][T::NTL];
  unsigned char* own = f16wk_smem + wave * T::WAVE_BYTES + lane * 16;
#pragma unroll
  for (int mi = 0; mi < T::MT; ++mi)
#pragma unroll
    for (int ni = 0; ni < T::NTL; ++ni) {
#pragma unroll
      for (int e = 0; e < 16; ++e) X[mi][ni][e] = 0.f;
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) *(f32x4*)(own + (mi * T::NTL + ni) * T::BLOCK_BYTES + r4 * 1024) = (f32x4){0.f, 0.f, 0.f, 0.f};
    }
  const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  auto fold = [&](int ni) {     // running sums of column block ni += X
#pragma unroll
    for (int mi = 0; mi < T::MT; ++mi)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        f32x4* at = (f32x4*)(own + (mi * T::NTL + ni) * T::BLOCK_BYTES + r4 * 1024);
        const f32x4 v = *at;
        *at = (f32x4){v[0] + X[mi][ni][4 * r4], v[1] + X[mi][ni][4 * r4 + 1], v[2] + X[mi][ni][4 * r4 + 2], v[3] + X[mi][ni][4 * r4 + 3]};
      }
  };

  // The wave's stages run in trips of four, then in trips of two while stages are left (so a wave runs at most one
  // stage of zeros past its last one); stage u of a trip uses register set u % 2 of the left operand.
  // Every column block is folded into the running sums after the last stage of a trip (every 128 k of the wave's
  // own: the same k for every block, and the same whatever zeros are appended to K), behind the MFMAs of the block
  // that follows it, and its next MFMA starts from zero.  A block is twelve pairs of MFMAs; behind pair x, between
  // scheduling fences: one operand of stage i + 1 (two 16-byte loads: the three terms of column block ni - 1, or of
  // block 4 into the other set when ni = 0, behind pairs 0, 2, 4; ni < 3: two of the six (term, row block) operands
  // of A behind pairs 6, 8) and a share of the fold -- chunk c of its eight (four accumulator registers of a block)
  // is read from LDS behind pair c and added and written back behind pair c + 2.
  f32x4 fold_in[3];
  auto trip = [&](int i0, auto fold_tag) {
    constexpr int FOLD = decltype(fold_tag)::value;
    static_assert(FOLD == 2 || FOLD == 4, "whole pairs of stages: the register sets alternate");
#pragma unroll
    for (int uu = 0; uu < FOLD; ++uu) {
      const int i = i0 + uu;
      const int u = uu & 1;
#pragma unroll
      for (int ni = 0; ni < T::NTL; ++ni) {
        const bool from_zero = uu == 0;                             // folded after the stage before
        const bool fold_prev = ni == 0 ? uu == 0 : uu == FOLD - 1;  // the block before this one is folded now
        const int pni = ni == 0 ? T::NTL - 1 : ni - 1;
        auto bop = [&](int t) { return ni < T::NTL - 1 ? b[t][ni < T::NTL - 1 ? ni : 0] : b4[u][t]; };
        int x = 0;
        auto gap = [&]() {
          __builtin_amdgcn_sched_barrier(0);
          if (x == 0 || x == 2 || x == 4) {
            if (ni == 0) issue_b4(i + 1, u ^ 1, x >> 1);
            else issue_b(i + 1, x >> 1, ni - 1);
          }
          if (ni < 3 && (x == 6 || x == 8)) {
            const int o = 2 * ni + (x == 8 ? 1 : 0);
            issue_a(i + 1, u ^ 1, o >> 1, o & 1);
          }
          if (fold_prev) {
            if (x >= 2 && x <= 9) {
              const int c = x - 2, mi = c >> 2, r4 = c & 3;
              const f32x4 v = fold_in[c % 3];
              *(f32x4*)(own + (mi * T::NTL + pni) * T::BLOCK_BYTES + r4 * 1024) =
                  (f32x4){v[0] + X[mi][pni][4 * r4], v[1] + X[mi][pni][4 * r4 + 1], v[2] + X[mi][pni][4 * r4 + 2], v[3] + X[mi][pni][4 * r4 + 3]};
            }
            if (x <= 7) fold_in[x % 3] = *(const f32x4*)(own + ((x >> 2) * T::NTL + pni) * T::BLOCK_BYTES + (x & 3) * 1024);
          }
          __builtin_amdgcn_sched_barrier(0);
          ++x;
        };
#define F16WK_PRODUCT(I, J, FIRST)                                                                                        \
  _Pragma("unroll") for (int s2 = 0; s2 < 2; ++s2) {                                                                      \
    _Pragma("unroll") for (int mi = 0; mi < T::MT; ++mi)                                                                  \
      X[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f16k_half(a[u][I][mi], s2), f16k_half(bop(J), s2),              \
                                                         (FIRST) && s2 == 0 && from_zero ? zero : X[mi][ni], 0, 0, 0);   \
    gap();                                                                                                                \
  }
        F16WK_PRODUCT(0, 2, true)
        F16WK_PRODUCT(1, 1, false)
        F16WK_PRODUCT(2, 0, false)
        F16WK_PRODUCT(0, 1, false)
        F16WK_PRODUCT(1, 0, false)
        F16WK_PRODUCT(0, 0, false)
#undef F16WK_PRODUCT
      }
    }
  };
  const int n4 = n_own & ~3;
  for (int i0 = 0; i0 < n4; i0 += 4) trip(i0, std::integral_constant<int, 4>{});
  for (int i0 = n4; i0 < n_own; i0 += 2) trip(i0, std::integral_constant<int, 2>{});
  // What the temporaries still hold.  The loop runs whole trips, so the last stage was the last of a trip: blocks
  // 0 .. 3 were folded behind the blocks that followed them, block 4 waits for its fold.
  fold(4);

  // ---- the four partial tiles meet: block b = mi * 5 + ni is owned by wave b % 4, which adds the four waves'
  // running sums of it in wave order ----
  const float out_scale = __builtin_ldexpf(1.f, -(p.tensor_exps[0] + p.tensor_exps[1]) - kF16KResultExp);
  __syncthreads();
  auto reduce_and_store = [&](auto owner_tag) {
    constexpr int W = decltype(owner_tag)::value;
    const int ldc_bytes = (int)p.ldc * 4;
    // rows past M fall beyond the end of the buffer and are dropped
    const int64_t c_bytes = ((int64_t)(p.M - 1 - m0) * p.ldc + (p.N - n0)) * 4;
    const i32x4 rc = make_rsrc(p.C + (int64_t)m0 * p.ldc + n0, c_bytes);
#pragma unroll
    for (int bk = W; bk < T::BLOCKS; bk += T::NW) {
      const int mi = bk / T::NTL, ni = bk % T::NTL;
      if (n0 + ni * 32 >= p.N) continue;
      f32x16 sum;
#pragma unroll
      for (int w = 0; w < T::NW; ++w) {
        const unsigned char* src = f16wk_smem + w * T::WAVE_BYTES + bk * T::BLOCK_BYTES + lane * 16;
#pragma unroll
        for (int r4 = 0; r4 < 4; ++r4) {
          const f32x4 x = *(const f32x4*)(src + r4 * 1024);
#pragma unroll
          for (int e = 0; e < 4; ++e) sum[4 * r4 + e] = w == 0 ? x[e] : sum[4 * r4 + e] + x[e];
        }
      }
      // columns past N (a ragged last tile; their slots were some other column's) are sent beyond the end too
      const bool inside = n0 + ni * 32 + l31 < p.N;
      const float bv = (p.bias && inside) ? p.bias[n0 + ni * 32 + l31] : 0.f;
      const int voff = inside ? (h * 4 * ldc_bytes) + (ni * 32 + l31) * 4 : (int)(c_bytes > 0x7FFFFFFF ? 0x7FFFFFFF : c_bytes);
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          llvm_raw_buffer_store_f32(sum[4 * q + e] * out_scale + bv, rc, voff, (mi * 32 + q * 8 + e) * ldc_bytes, kResultStoreAux);
    }
  };
  if (wave == 0) reduce_and_store(std::integral_constant<int, 0>{});
  else if (wave == 1) reduce_and_store(std::integral_constant<int, 1>{});
  else if (wave == 2) reduce_and_store(std::integral_constant<int, 2>{});
  else reduce_and_store(std::integral_constant<int, 3>{});
}

}  // namespace cascmm
