// Three-term fp8 (e4m3) cascade on the fp8-rate MFMA of gfx950, v_mfma_scale_f32_32x32x64_f8f6f4.
//
// That instruction multiplies 32 x 64 by 64 x 32 fp8 values in 16 passes (64 cycles, measured): twice
// the rate of the bf16 and legacy fp8 forms, so the six products of a three-term cascade cost what
// the three products of the two-term bf16 cascade cost.  A lane supplies 32 consecutive k of its row
// (column) in eight registers, lanes 0..31 the first half of the 64, lanes 32..63 the second, and one
// E8M0 scale byte that the hardware applies to those 32 values.  The scales carry the term scaling:
// term i of either operand is stored as lowp(r_i * 2^(e + 4 i)) and multiplied with scale 2^(-4 i),
// so all six products of a block land in ONE accumulator with their weights 2^(-4 (i + j)) applied
// before the addition (measured: a lane's scale applies to exactly its own 32 values; products are
// added in fp32 with an alignment window of about 15 bits inside groups of neighbouring k and about
// 18 bits across them, as in the legacy instruction).
//
// Both operands are split before the GEMM, by small kernels, into operand slots: 16 bytes = 16
// consecutive k of one row (column) of one term, [term][K/16][rows].  Activations are split in every
// call (their tensor scale is found first, by a pass of its own); a weight can be split once
// (cascmm_prepare_weight writes this layout for three fp8 terms when K is a multiple of 64).  The
// GEMM then moves nothing through registers but fragments: wave-wide `buffer_load ... lds` copies
// slots to LDS (64 consecutive rows per instruction; rows past the edge are clamped to the last one),
// a lane reads two slots per term and block, no VALU work is left in the loop.
//
// Workgroup: four waves (one per SIMD) stacked along M, tile 256 x 160, wave tile 64 x 160 (ten
// accumulator blocks).  A stage is one MFMA deep (64 k): 78 KB of slots, double buffered; one barrier
// per stage, 60 MFMAs = 3840 cycles per wave between barriers, the loads of the next stage issued in
// the gaps (unconditionally: past the last stage the last one is fetched again).  The barrier sits in
// front of a stage's last column block, whose fragments are already in registers, so the first
// fragments of the next stage are read behind that block's MFMAs.
// A second instantiation has half the rows (tile 128 x 160, wave tile 32 x 160, 30 MFMAs per stage):
// twice the tiles for problems that would otherwise leave CUs idle or need their K split over
// workgroups (and its partial results written out and added by a second kernel).  Its stages are too
// short to spread the loads: all loads of stage s + 2 are issued right behind the barrier that frees
// their buffer, a whole stage before they are needed.
#pragma once
#include <type_traits>

#include "cascmm_tile_kernel.h"

namespace cascmm {

template <int MT_>
struct F8K64T {
  static constexpr int MT = MT_, NTL = 5;                  // 32 x 32 accumulator blocks of a wave: MT x NTL
  static constexpr int WTM = 32 * MT, BM = 4 * WTM, BN = 160, BK = 64, NT = 256, TERMS = 3;
  static constexpr int KU = BK / 16;                       // 16-k slot columns per stage
  static constexpr int A_STAGE = TERMS * KU * BM * 16;     // 48 KB (24 KB)
  static constexpr int B_STAGE = TERMS * KU * BN * 16;     // 30 KB
  static constexpr int STAGE = A_STAGE + B_STAGE;          // 78 KB (54 KB)
  static constexpr int LDS_BYTES = 2 * STAGE;              // 156 KB (108 KB)
  static constexpr int A_LOADS = TERMS * KU * BM / 64 / 4; // per wave: the stage's runs of 64 rows, dealt round robin
  static constexpr int B_SLOTS = TERMS * KU * BN;          // 1920 = 30 x 64
  static constexpr int B_LOADS_MAX = 8;                    // 30 instructions over 4 waves: 8, 8, 7, 7
  static constexpr int LOADS = A_LOADS + B_LOADS_MAX;      // 20 (14)
  static constexpr int GB = 6 * MT;                        // MFMAs (and the gaps behind them) per column block
};
typedef F8K64T<2> F8K64;   // the 256 x 160 tile; what is common to both (BN, BK, slot layout) is read from it

typedef int i32x8 __attribute__((ext_vector_type(8)));

// bytes of the slots of an operand with `rows` rows (columns) and K (multiple of 16) deep
// (saturates instead of overflowing: callers compare the result with limits)
inline __host__ __device__ int64_t f8k64_slot_bytes(int64_t rows, int64_t K) {
  int64_t slots = 0, bytes = 0;
  if (__builtin_mul_overflow((int64_t)F8K64::TERMS * (K / 16), rows, &slots) || __builtin_mul_overflow(slots, (int64_t)16, &bytes))
    return INT64_MAX;
  return bytes;
}

// max|a| of this workgroup's share of A [M, K] (bit pattern) -> amax_out[blockIdx.x]; no atomics, no
// meeting point: the kernel that splits A reduces the gridDim.x values.
template <int UNUSED>
__global__ __launch_bounds__(1024) void f8k64_amax_kernel(const float* __restrict__ A, int64_t M, int64_t K, int64_t lda,
                                                         unsigned* __restrict__ amax_out) {
  __shared__ unsigned wave_best[16];
  const unsigned best = amax_scan<CASCMM_DT_F32>(A, M, K, lda);
  if ((threadIdx.x & 63) == 0) wave_best[threadIdx.x >> 6] = best;
  __syncthreads();
  if (threadIdx.x != 0) return;
  unsigned b = 0;
  for (unsigned w = 0; w < (blockDim.x >> 6); ++w) b = wave_best[w] > b ? wave_best[w] : b;
  amax_out[blockIdx.x] = b;
}

// Split of the LEFT operand: A [M, K] fp32 row-major -> slots[term][K/16][M].  A workgroup converts
// 64 rows x 64 k (a thread: 16 consecutive k of a row) and transposes through LDS so that the slots
// leave as 1 KB runs along M.
// The scale exponent is *tensor_exp (NULL: 0), or, when `amax` is given, found here: amax[0 .. n_amax)
// are the per-workgroup maxima |a| (bit patterns) of a preceding f8k64_amax_kernel; every workgroup
// reduces them itself (1 KB from L2, behind its loads of A), and the first one leaves {e_A, *b_exp}
// in exps_out for the GEMM.
template <int UNUSED>
__global__ __launch_bounds__(256) void f8k64_split_rows_kernel(const float* __restrict__ A, int M, int K, int64_t lda,
                                                              const int32_t* __restrict__ tensor_exp, u32x4* __restrict__ out,
                                                              const unsigned* __restrict__ amax, int n_amax,
                                                              const int32_t* __restrict__ b_exp, int32_t* __restrict__ exps_out) {
  __shared__ u32x4 slots[3][4][64];
  __shared__ int e_found;
  const int kus = K >> 4;
  const int ku_tiles = (kus + 3) >> 2;
  const int m0 = (blockIdx.x / ku_tiles) * 64, ku0 = (blockIdx.x % ku_tiles) * 4;
  int e = tensor_exp ? *tensor_exp : 0;
  if (amax) {   // (uniform over the grid)
    if (threadIdx.x < 64) {
      unsigned best = 0;
      for (int i = threadIdx.x; i < n_amax; i += 64) best = amax[i] > best ? amax[i] : best;
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        const unsigned other = (unsigned)__shfl_xor((int)best, off, 64);
        best = other > best ? other : best;
      }
      if (threadIdx.x == 0) e_found = exp_of_amax(best);
    }
    __syncthreads();
    e = e_found;
    if (blockIdx.x == 0 && threadIdx.x == 0) {
      exps_out[0] = e;
      exps_out[1] = b_exp ? *b_exp : 0;
    }
  }
  const float scale = __builtin_ldexpf(1.f, e);
  {
    const int row = threadIdx.x >> 2, ku = threadIdx.x & 3;
    if (m0 + row < M && ku0 + ku < kus) {
      const float* src = A + (int64_t)(m0 + row) * lda + (ku0 + ku) * 16;
      u32x4 t[3];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const f32x4 v0 = *(const f32x4*)(src + 8 * h), v1 = *(const f32x4*)(src + 8 * h + 4);
        float r[8] = {v0[0] * scale, v0[1] * scale, v0[2] * scale, v0[3] * scale, v1[0] * scale, v1[1] * scale, v1[2] * scale, v1[3] * scale};
        const u32x2 t0 = Lowp<CASCMM_FMT_FP8>::peel<false>(r);
        const u32x2 t1 = Lowp<CASCMM_FMT_FP8>::peel<false>(r);
        const u32x2 t2 = Lowp<CASCMM_FMT_FP8>::peel<true>(r);
        t[0][2 * h] = t0[0]; t[0][2 * h + 1] = t0[1];
        t[1][2 * h] = t1[0]; t[1][2 * h + 1] = t1[1];
        t[2][2 * h] = t2[0]; t[2][2 * h + 1] = t2[1];
      }
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

// Split of the RIGHT operand: B [K, N] fp32 row-major -> slots[term][K/16][N]; thread (ku, n) walks
// 16 rows of column n (consecutive threads: consecutive columns, coalesced both ways).
template <int UNUSED>
__global__ __launch_bounds__(256) void f8k64_split_cols_kernel(const float* __restrict__ B, int K, int N, int64_t ldb,
                                                              const int32_t* __restrict__ tensor_exp, u32x4* __restrict__ out) {
  const int kus = K >> 4;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (int64_t)kus * N) return;
  const int ku = (int)(i / N), n = (int)(i - (int64_t)ku * N);
  const float scale = tensor_exp ? __builtin_ldexpf(1.f, *tensor_exp) : 1.f;
  const float* src = B + (int64_t)ku * 16 * ldb + n;
  u32x4 t[3];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    float r[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = src[(int64_t)(8 * h + e) * ldb] * scale;
    const u32x2 t0 = Lowp<CASCMM_FMT_FP8>::peel<false>(r);
    const u32x2 t1 = Lowp<CASCMM_FMT_FP8>::peel<false>(r);
    const u32x2 t2 = Lowp<CASCMM_FMT_FP8>::peel<true>(r);
    t[0][2 * h] = t0[0]; t[0][2 * h + 1] = t0[1];
    t[1][2 * h] = t1[0]; t[1][2 * h + 1] = t1[1];
    t[2][2 * h] = t2[0]; t[2][2 * h + 1] = t2[1];
  }
#pragma unroll
  for (int j = 0; j < 3; ++j) out[((int64_t)j * kus + ku) * N + n] = t[j];
}

struct F8K64Params {
  const u32x4* a_slots;   // [3][K/16][M]
  const u32x4* b_slots;   // [3][K/16][N]
  float* C;
  const float* bias;
  const int32_t* tensor_exps;   // {e_A, e_B} or NULL
  int M, N, K;
  int64_t ldc;
  int tiles_m, tiles_n;
  int k_splits;           // > 1: workgroup (split, tile) multiplies K range split and writes partials[split][M][N]
  float* partials;
};

typedef __attribute__((address_space(3))) void* f8k64_lds_ptr;

// 64 lanes x 16 bytes from a buffer straight into LDS at dst + 16 lane.  (A function of its own: in a
// call whose arguments depend on a template parameter the host pass of the compiler rejects the
// builtin without a message and then leaves out the kernel's launch stub.)
__device__ __forceinline__ void f8k64_load_lds(__amdgpu_buffer_rsrc_t rsrc, unsigned char* dst, int voffset, int soffset) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (f8k64_lds_ptr)dst, 16, voffset, soffset, 0, 0);
}

// Host-checked: K % 64 == 0, the slot buffers below 2 GiB, C rows addressable with 32-bit byte offsets
// inside a tile.  MT = 2: 256 x 160 tile, MT = 1: 128 x 160.
template <int MT>
__global__ __launch_bounds__(F8K64T<MT>::NT) __attribute__((amdgpu_waves_per_eu(1, 1))) void cascmm_f8k64_kernel(const F8K64Params p) {
  typedef F8K64T<MT> T;
  extern __shared__ __attribute__((aligned(1024))) unsigned char f8k64_smem[];
  unsigned char* smem = f8k64_smem;
  const int tid = threadIdx.x, lane = tid & 63, l31 = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = wave * T::WTM;
  const int tiles = p.tiles_m * p.tiles_n;
  const int split = p.k_splits > 1 ? (int)blockIdx.x / tiles : 0;
  int tm, tn;
  tile_coords((int)blockIdx.x - split * tiles, p.tiles_m, p.tiles_n, tm, tn);
  const int m0 = tm * T::BM, n0 = tn * T::BN;
  const int ksteps = p.K / T::BK / (p.k_splits > 1 ? p.k_splits : 1);   // stages of this workgroup (the host picks a divisor)
  const int step0 = split * ksteps;
  const int kus = p.K >> 4;

  const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc((void*)p.a_slots, 0, 0x7FFFFFFF, 0x00020000);
  const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc((void*)p.b_slots, 0, 0x7FFFFFFF, 0x00020000);
  // A: a stage holds, per (term, ku), BM slots = BM / 64 runs of 64 rows, run r at byte r * 1024; this
  // wave loads runs wave, wave + 4, ...; lane = row inside the run (clamped to the last valid row)
  const int a_plane = kus * p.M * 16;          // bytes between terms
  const int a_ku = p.M * 16;                   // bytes between 16-k slot columns
  constexpr int CH = T::BM / 64;               // runs per (term, ku)
  int a_voff[T::A_LOADS], a_soff[T::A_LOADS];
#pragma unroll
  for (int j = 0; j < T::A_LOADS; ++j) {
    const int run = wave + 4 * j;
    const int tk = run / CH, chunk = run % CH;           // tk = term * KU + ku
    int row = m0 + chunk * 64 + lane;
    row = row < p.M ? row : p.M - 1;
    a_voff[j] = row * 16;
    a_soff[j] = (tk / T::KU) * a_plane + (tk % T::KU) * a_ku;
  }
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
    const int step = step0 + (step_ < ksteps - 1 ? step_ : ksteps - 1);
    f8k64_load_lds(ra, smem + (step_ & 1) * T::STAGE + (wave + 4 * j) * 1024, a_voff[j], a_soff[j] + step * T::KU * a_ku);
  };
  auto issue_b = [&](int step_, int j) {
    const int step = step0 + (step_ < ksteps - 1 ? step_ : ksteps - 1);
    f8k64_load_lds(rb, smem + (step_ & 1) * T::STAGE + b_lds[j], b_voff[j], step * b_step);
  };

  // fragment addresses inside a stage: lane (row l31, k half h) reads slots (term, ku = 2 h) and (term, 2 h + 1)
  const int a_frag = (2 * h * T::BM + wm0 + l31) * 16;                  // + term * KU * BM * 16 + mi * 512, second slot + BM * 16
  const int b_frag = T::A_STAGE + (2 * h * T::BN + l31) * 16;           // + term * KU * BN * 16 + ni * 512, second slot + BN * 16
  const int scales = 0x00777B7F;                                        // E8M0 bytes 2^0, 2^-4, 2^-8: op_sel picks the term's

  f32x16 acc[T::MT][T::NTL];
#pragma unroll
  for (int mi = 0; mi < T::MT; ++mi)
#pragma unroll
    for (int ni = 0; ni < T::NTL; ++ni)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[mi][ni][e] = 0.f;

#define F8K64_FENCE() __builtin_amdgcn_sched_barrier(0)
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

  // Fragments: A of the whole stage (the wave's own rows), B of one column block, both double
  // buffered in registers.  The barrier that opens stage s + 1 sits in front of the LAST column block
  // of stage s: by then the wave has read everything it needs of stage s from LDS (the last block's
  // fragments are prefetched during the block before), so the first fragments of stage s + 1 are read
  // behind that block's MFMAs and no LDS latency is exposed after a barrier.
  i32x8 a[2][T::TERMS][T::MT];
  i32x8 b[2][T::TERMS];
  auto read_a = [&](int buf, const unsigned char* st, int t) {
#pragma unroll
    for (int mi = 0; mi < T::MT; ++mi) a[buf][t][mi] = frag(st + a_frag + t * T::KU * T::BM * 16 + mi * 512, T::BM * 16);
  };
  auto read_b = [&](int buf, const unsigned char* st, int ni, int t) {
    b[buf][t] = frag(st + b_frag + t * T::KU * T::BN * 16 + ni * 512, T::BN * 16);
  };
  __builtin_amdgcn_s_waitcnt(0x0F70);       // vmcnt(0): stage 0 has landed
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int t = 0; t < T::TERMS; ++t) {
    read_a(0, smem, t);
    read_b(0, smem, 0, t);
  }
  // Loads of stage s + 1 that are issued before stage s begins (the others follow inside stage s):
  // MT = 2: the first six; MT = 1: all of them
  constexpr int EARLY = MT == 2 ? 6 : T::LOADS;
#pragma unroll
  for (int k = 0; k < EARLY; ++k) issue(1, k);

  // ksteps is even or odd: the stage loop is unrolled by two so that the register buffers are static
  auto stage = [&](int s, auto BUF) {
    constexpr int ab = decltype(BUF)::value;       // A buffer of this stage; B block ni uses buffer (ab * 5 + ni) & 1
    const unsigned char* st = smem + (s & 1) * T::STAGE;
    const unsigned char* st_next = smem + ((s + 1) & 1) * T::STAGE;
#pragma unroll
    for (int ni = 0; ni < T::NTL; ++ni) {
      const int cur = (ab * T::NTL + ni) & 1, nxt = cur ^ 1;
      if (ni == T::NTL - 1) {
        // everything this wave needs of stage s is in registers: open stage s + 1
        // own loads of stage s + 1 have landed (issued a stage ago), and own reads of stage s have returned
        // (the last of them were issued three MFMAs ago: the loads that follow the barrier overwrite that buffer)
        __builtin_amdgcn_s_waitcnt(0x0070);     // vmcnt(0), lgkmcnt(0)
        __builtin_amdgcn_s_barrier();           // everybody's; and nobody reads stage s any more
      }
      int n_issued = 0;
      auto gap = [&]() {
        F8K64_FENCE();
        if (ni < T::NTL - 1) {
          if (n_issued < 3) read_b(nxt, st, ni + 1, n_issued);   // the fragments of the next column block
          if (MT == 2) {
            // loads 6 .. 19 of stage s + 1 (its buffer was given up at the barrier inside stage s - 1): gaps
            // 3 .. 11 of block 0 and 3 .. 7 of block 1, which leaves them two and a half blocks to land
            const int k = ni == 0 ? n_issued + 3 : ni == 1 ? n_issued + 12 : -1;
            if (n_issued >= 3 && k >= 6 && k < T::LOADS) issue(s + 1, k);
          }
        } else if (MT == 2) {
          // behind the last block: the first fragments of stage s + 1, then loads 0 .. 5 of stage s + 2
          if (n_issued < 3) read_b(nxt, st_next, 0, n_issued);
          else if (n_issued < 6) read_a(ab ^ 1, st_next, n_issued - 3);
          else issue(s + 2, n_issued - 6);
        } else {
          // six gaps: a fragment read and up to three loads of stage s + 2 in each (all fourteen)
          if (n_issued < 3) read_b(nxt, st_next, 0, n_issued);
          else read_a(ab ^ 1, st_next, n_issued - 3);
#pragma unroll
          for (int u = 0; u < 3; ++u)
            if (n_issued * 3 + u < T::LOADS) issue(s + 2, n_issued * 3 + u);
        }
        F8K64_FENCE();
        ++n_issued;
      };
      // (the term numbers are the instruction's op_sel fields: literals)
#define F8K64_PRODUCT(I, J)                                                                                                              \
  _Pragma("unroll") for (int mi = 0; mi < T::MT; ++mi) {                                                                                 \
    acc[mi][ni] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[ab][I][mi], b[cur][J], acc[mi][ni], 0, 0, I, scales, J, scales);     \
    gap();                                                                                                                               \
  }
      F8K64_PRODUCT(0, 2)
      F8K64_PRODUCT(1, 1)
      F8K64_PRODUCT(2, 0)
      F8K64_PRODUCT(0, 1)
      F8K64_PRODUCT(1, 0)
      F8K64_PRODUCT(0, 0)
#undef F8K64_PRODUCT
    }
  };
  int s = 0;
  for (; s + 2 <= ksteps; s += 2) {
    stage(s, std::integral_constant<int, 0>{});
    stage(s + 1, std::integral_constant<int, 1>{});
  }
  if (s < ksteps) stage(s, std::integral_constant<int, 0>{});
#undef F8K64_FENCE
  __builtin_amdgcn_s_waitcnt(0x0F70);       // the redundant loads of the last stage land before LDS is given up

  // ---- epilogue: undo the tensor scales, add the bias; a lane holds column l31, rows 8 q + 4 h + e ----
  float out_scale = 1.f;
  if (p.tensor_exps) out_scale = __builtin_ldexpf(1.f, -(p.tensor_exps[0] + p.tensor_exps[1]));
  const int row_base = m0 + wm0 + 4 * h;
  float* C = p.C;
  int64_t ldc = p.ldc;
  const float* bias = p.bias;
  if (p.k_splits > 1) {   // partial result (scaled, no bias): the reduction kernel adds the splits in order
    C = p.partials + (int64_t)split * p.M * p.N;
    ldc = p.N;
    bias = nullptr;
  }
  if (m0 + T::BM <= p.M && n0 + T::BN <= p.N && ldc * (int64_t)(T::BM * 4) < 0x7FFFFFFF) {
    // whole tile inside C: buffer stores, the row as a scalar offset, nothing to mask
    const i32x4 rc = make_rsrc(C + (int64_t)(m0 + wm0) * ldc + n0, 0x7FFFFFFF);
    const int ldc_bytes = (int)ldc * 4;
#pragma unroll
    for (int ni = 0; ni < T::NTL; ++ni) {
      const float bv = bias ? bias[n0 + ni * 32 + l31] : 0.f;
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
    const float bv = bias ? bias[col] : 0.f;
#pragma unroll
    for (int mi = 0; mi < T::MT; ++mi)
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int row = row_base + mi * 32 + q * 8 + e;
          if (row < p.M) C[(int64_t)row * ldc + col] = acc[mi][ni][4 * q + e] * out_scale + bv;
        }
  }
}

}  // namespace cascmm
