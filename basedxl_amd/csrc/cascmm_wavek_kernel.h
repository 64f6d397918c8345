// Skinny problems (few rows, e.g. the 77 or 154 text tokens of a cross-attention K/V projection) in
// ONE launch and without a workspace: K is split over the eight waves of a workgroup instead of
// over workgroups, so the partial sums meet in LDS and never travel through memory.
//
// One workgroup computes a 32 x (32 NB) tile of C over the whole K.  Wave w takes the 32-wide K
// steps w, w + 8, w + 16, ...; it streams its own operands and shares nothing with the other waves
// until the end, so the main loop has no barrier:
//   * A (32 rows x 32 k fp32 per step, 4 KB) goes to the wave's private LDS ring without passing
//     registers (four `buffer_load ... lds` of 1 KB; eight consecutive lanes fetch the eight
//     16-byte chunks of one row's 128 bytes, a whole cache line, rotated by row / 2 inside the row
//     so that the fragment reads spread over all banks);
//   * B needs no transposition: lane (c, g) of an MFMA wants B[k0 + 8 g + e][column c], e = 0..7,
//     which is one coalesced 4-byte (NB = 2: 8-byte, the wave's two column blocks are the even
//     and the odd columns) load per e straight into registers.
// Three steps beyond the current one are in flight (60 loads, the limit of the wave's load
// counter), 24 KB per wave.  The values are split in registers right before their MFMAs, like in
// the large-tile kernel.  At the end the eight partial tiles are added in wave order through LDS
// (deterministic) and written with the bias.
//
// The shape is bound by what one CU can pull in, (32 + 32 NB) x K x 4 bytes, at the 64 bytes per
// clock of its vector memory path, not by HBM (the weights are 10 MB) and not by the MFMAs.
#pragma once
#include "cascmm_tile_kernel.h"

namespace cascmm {

template <int NB>
struct WaveK {
  static constexpr int BM = 32, BN = 32 * NB, BK = 32, NW = 8, NT = 512, NS = 4;
  static constexpr int A_STAGE = BM * BK * 4;           // 4 KB
  static constexpr int RING = NS * A_STAGE;             // 16 KB per wave
  static constexpr int LDS_BYTES = NW * RING;           // 128 KB
  static constexpr int LOADS = 4 + 16;                  // per wave and step
};

typedef __attribute__((address_space(3))) void* wavek_lds_ptr;

// 64 lanes x 16 bytes from a buffer straight into LDS at dst + 16 lane.  (Not called from the kernel
// template directly: in a call whose arguments depend on a template parameter the host pass of the
// compiler rejects the builtin without a message and then leaves out the kernel's launch stub.)
__device__ __forceinline__ void wavek_load_lds(__amdgpu_buffer_rsrc_t rsrc, unsigned char* dst, int voffset, int soffset) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (wavek_lds_ptr)dst, 16, voffset, soffset, 0, 0);
}
// The same with the instruction's immediate offset, kb KB (0 .. 3): it is added to the LDS address AND to the memory
// address, so loads into consecutive kilobytes of LDS can share one M0 (one scalar instruction less per load) if the
// lane offset makes up for it on the memory side.
__device__ __forceinline__ void wavek_load_lds_kb(__amdgpu_buffer_rsrc_t rsrc, unsigned char* dst, int voffset, int soffset, int kb) {
  switch (kb) {
    case 0: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (wavek_lds_ptr)dst, 16, voffset, soffset, 0, 0); break;
    case 1: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (wavek_lds_ptr)dst, 16, voffset, soffset, 1024, 0); break;
    case 2: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (wavek_lds_ptr)dst, 16, voffset, soffset, 2048, 0); break;
    default: __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (wavek_lds_ptr)dst, 16, voffset, soffset, 3072, 0); break;
  }
}

// Host-checked: fp32 operands, two bf16 terms, products hi.hi + hi.lo + lo.hi; K % 32 == 0,
// N % (32 NB) == 0, lda % 4 == 0 and A 16-byte aligned, NB == 2: ldb % 2 == 0 and B 8-byte aligned;
// M * lda * 4 and K * ldb * 4 below 2 GiB.
template <int NB>
__global__ __launch_bounds__(WaveK<NB>::NT) void cascmm_wavek_kernel(const GroupParams p) {
  typedef WaveK<NB> T;
  extern __shared__ __attribute__((aligned(1024))) unsigned char wavek_smem[];
  const int tid = threadIdx.x, lane = tid & 63, l31 = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  unsigned char* ring = wavek_smem + wave * T::RING;

  // work item: consecutive items run down the row tiles of one column band, and an XCD (which
  // gets every eighth workgroup) takes a contiguous range of items, so a band of B is pulled
  // into one L2 only
  const int tiles = p.tiles_m * p.tiles_n;
  const int total = tiles * p.count;
  const int per = total >> 3;
  int id = blockIdx.x;
  if (id < (per << 3)) id = (id & 7) * per + (id >> 3);
  const int prob = id / tiles;
  const int t = id - prob * tiles;
  const int tn = t / p.tiles_m, tm = t - tn * p.tiles_m;
  const int m0 = tm * T::BM, n0 = tn * T::BN;
  const int steps = p.K / T::BK;                              // all of them
  const int my_steps = (steps - wave + T::NW - 1) / T::NW;    // those of this wave: wave, wave + 8, ...
  const int trips = (steps + T::NW - 1) / T::NW;              // of wave 0, the longest
  const int ldb_bytes = (int)p.ldb * 4;

  // rows past M read as zero: the buffer ends with row M - 1
  const __amdgpu_buffer_rsrc_t ra =
      __builtin_amdgcn_make_buffer_rsrc((void*)p.A[prob], 0, (int)((int64_t)p.M * p.lda * 4), 0x00020000);
  const i32x4 rb = make_rsrc(p.B[prob], (int)((int64_t)p.K * p.ldb * 4));
  int a_voff[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = j * 8 + (lane >> 3);
    const int chunk = ((lane & 7) - (row >> 1)) & 7;
    a_voff[j] = (int)(((int64_t)(m0 + row) * p.lda + chunk * 4) * 4);
  }
  const int b_voff = 8 * g * ldb_bytes + (n0 + NB * l31) * 4;
  // fragment addresses inside a stage: row l31, chunks 4 j2 + 2 g and + 1 at their rotated places
  int a_frag[2][2];
#pragma unroll
  for (int j2 = 0; j2 < 2; ++j2)
#pragma unroll
    for (int h = 0; h < 2; ++h) a_frag[j2][h] = l31 * 128 + (((4 * j2 + 2 * g + h) + (l31 >> 1)) & 7) * 16;

  typedef float bvec __attribute__((ext_vector_type(NB)));
  bvec Bv[T::NS][2][8];   // raw B of the steps in flight: [stage][k half][e]

  // the loads of this wave's i-th step (clamped: past its last step a wave fetches that step again
  // into a stage nobody reads any more)
  auto issue = [&](int i, int st) {
    const int ii = i < my_steps ? i : my_steps - 1;
    const int step = wave + ii * T::NW;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      wavek_load_lds(ra, ring + st * T::A_STAGE + j * 1024, a_voff[j], step * T::BK * 4);
#pragma unroll
    for (int j2 = 0; j2 < 2; ++j2)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int soff = (step * T::BK + 16 * j2 + e) * ldb_bytes;
        if constexpr (NB == 1) Bv[st][j2][e] = (bvec){llvm_raw_buffer_load_f32(rb, b_voff, soff, 0)};
        else Bv[st][j2][e] = __builtin_bit_cast(bvec, llvm_raw_buffer_load_v2f32(rb, b_voff, soff, 0));
      }
  };

  f32x16 acc[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[nb][e] = 0.f;

  if (my_steps > 0) {
#pragma unroll
    for (int s = 0; s < T::NS - 1; ++s) issue(s, s);
  }
  // `trips` is the same for every wave of the workgroup; a wave with fewer steps idles through
  // its last trip (the trip count is wave-uniform, so the tests below are scalar branches)
  for (int i0 = 0; i0 < trips; i0 += T::NS) {
#pragma unroll
    for (int u = 0; u < T::NS; ++u) {
      const int i = i0 + u;
      if (i < my_steps) {
        issue(i + T::NS - 1, (u + T::NS - 1) % T::NS);
        __builtin_amdgcn_s_waitcnt(0x0F70 | ((3 * T::LOADS) & 0xF) | (((3 * T::LOADS) >> 4) << 14));   // vmcnt(60)
        const unsigned char* stp = ring + u * T::A_STAGE;
#pragma unroll
        for (int j2 = 0; j2 < 2; ++j2) {
          const f32x4 x0 = *(const f32x4*)(stp + a_frag[j2][0]), x1 = *(const f32x4*)(stp + a_frag[j2][1]);
          float xa[8] = {x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
          u32x4 ta[2];
          split8<CASCMM_FMT_BF16, 2>(xa, ta);
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) {
            float xb[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) xb[e] = Bv[u][j2][e][nb];
            u32x4 tb[2];
            split8<CASCMM_FMT_BF16, 2>(xb, tb);
            typedef Lowp<CASCMM_FMT_BF16> L;
            // smallest products first
            acc[nb] = L::mfma(L::operand(ta[1], 1), L::operand(tb[0], 0), acc[nb]);
            acc[nb] = L::mfma(L::operand(ta[0], 0), L::operand(tb[1], 1), acc[nb]);
            acc[nb] = L::mfma(L::operand(ta[0], 0), L::operand(tb[0], 0), acc[nb]);
          }
        }
      }
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);   // the redundant loads land before the ring is reused
  __syncthreads();

  // ---- the eight partial tiles meet in LDS: [wave][nb][reg][lane] fp32 -------------------------
  float* part = (float*)wavek_smem;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int e = 0; e < 16; ++e) part[((wave * NB + nb) * 16 + e) * 64 + lane] = acc[nb][e];
  __syncthreads();
  // thread -> (nb, reg, lane) positions tid, tid + 512, ...; of a block a lane holds column l31,
  // rows 8 (reg / 4) + 4 g + reg % 4
  float* C = (float*)p.C[prob];
  const float* bias = (const float*)p.bias[prob];
#pragma unroll
  for (int q = 0; q < NB * 16 * 64 / T::NT; ++q) {
    const int pos = q * T::NT + tid;
    const int nb = pos / (16 * 64), e = (pos / 64) % 16, ln = pos % 64;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < T::NW; ++w) sum += part[((w * NB + nb) * 16 + e) * 64 + ln];
    const int row = m0 + 8 * (e >> 2) + 4 * (ln >> 5) + (e & 3);
    const int col = n0 + NB * (ln & 31) + nb;
    if (row < p.M) C[(int64_t)row * p.ldc + col] = sum + (bias ? bias[col] : 0.f);
  }
}

}  // namespace cascmm
