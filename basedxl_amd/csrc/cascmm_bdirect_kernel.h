// "B-direct" MFMA kernel of the cascade GEMM (gfx950): the right operand never touches LDS.
//
// B is [K, N] row-major, so the 32 lanes that hold the 32 columns of one MFMA operand block
// read 128 contiguous bytes of a B row: a consumer wave can load its B fragments straight into
// the v_mfma_f32_32x32x16 operand layout (lane l: column l%32, k rows 8*(l/32) .. +7) with eight
// fully coalesced dword loads per 16-deep k slice, split them into terms in registers, and
// feed the MFMAs.  Consumer waves are laid out 1 x WN, each owning 32 columns of the tile and
// all of its rows, so no B element is loaded or split twice inside a workgroup.  The split's
// VALU instructions issue in the gaps between the wave's own MFMAs.
//
// Only A goes through LDS: producer waves load it with 16-byte buffer loads, split it and
// write the 16-byte operand slots (layout and swizzle as in the LDS-tiled kernel), one stage
// per barrier interval, double buffered.  Compared with staging both operands this halves
// the LDS write volume and the producers' VALU work, which measurement showed to be what
// bounds the LDS-tiled kernel on the SDXL shapes.
#pragma once
#include "cascmm_tile_kernel.h"

namespace cascmm {

template <int BM_, int WN_, int BK_, int DEPTH_, int NP_>
struct TileBD {
  static constexpr int BM = BM_, WN = WN_, BN = 32 * WN_, BK = BK_, DEPTH = DEPTH_, NP = NP_;
  static constexpr int WM = 1, WK = 1;
  static constexpr int NCW = WN;
  static constexpr int NTP = NP * kWave;
  static constexpr int NT = (NCW + NP) * kWave;
  static constexpr int KG = BK / 8;
  static constexpr int MT = BM / 32;
  static constexpr int KSUB = BK / 16;
  static_assert(BM % 32 == 0, "BM");
  static_assert(BK == 32 || BK == 64, "BK");
  static_assert(KSUB * 8 <= 32, "the B loads of two K steps in flight must fit the vmcnt counter");
};

template <class TL, int TERMS>
struct LdsLayoutA {
  static constexpr int kAPlane = TL::BM;
  static constexpr int kATerm = TL::KG * kAPlane;
  static constexpr int kStage = TERMS * kATerm;
  static constexpr int kBytes = 2 * kStage * 16;
  static __device__ __forceinline__ int swz(int kg) { return (kg * (TL::KG >= 8 ? 1 : 8 / TL::KG)) & 7; }
};

// SPLITK: the grid is tiles x k_splits; workgroup (tile, split) multiplies the K range
// [split * k_per_split, (split + 1) * k_per_split) and leaves an fp32 partial tile in the
// workspace; splitk_reduce_kernel adds the partials in split order and writes C.  (Letting the
// last workgroup of a tile do the sum inside this kernel was measured 3x slower: the
// device-scope release / acquire it needs writes back and invalidates the whole L2 of the
// XCD for every workgroup.)  This is the path for skinny problems (M of a few row blocks, e.g. the 2 x 77 text
// tokens of the cross-attention K/V projections): they have too few tiles to occupy the
// chip and are bound by the latency of streaming the weight matrix, so K is split until
// about half the CUs have a workgroup, each reading its slab of the weights once.
template <class TL, int FMT, int TERMS, bool FULL, bool SPLITK = false>
struct BDirectGemm {
  typedef Lowp<FMT> LP;
  typedef typename LP::Vec Vec;
  typedef LdsLayoutA<TL, TERMS> LL;
  typedef ProductSet<TERMS, FULL> PS;
  typedef AccClasses<FMT, TERMS, FULL> AC;
  static constexpr int ES = 4;
  static constexpr int NCLS = AC::kCount;
  static constexpr int A_UNITS = TL::KG * TL::BM;
  static constexpr int A_IT = (A_UNITS + TL::NTP - 1) / TL::NTP;
  static constexpr int D = TL::DEPTH;
  static_assert(A_UNITS % TL::NTP == 0, "A units must divide evenly among the producer threads");
  static_assert(A_IT * 2 * D <= 60, "too many A loads in flight");

  // ---- producers: A only ---------------------------------------------------------------------
  static __device__ __forceinline__ void producer(const GemmParams& p, u32x4* lds, int m0, int ktiles, int kbase) {
    const int ptid = threadIdx.x - TL::NCW * kWave;
    const float* A = (const float*)p.A + (int64_t)m0 * p.lda + kbase;
    const i32x4 ra = make_rsrc(A, ((int64_t)(p.M - 1 - m0) * p.lda + p.K - kbase) * ES);
    const int last_row = p.M - 1 - m0;
    int voff[A_IT], slot[A_IT];
#pragma unroll
    for (int it = 0; it < A_IT; ++it) {
      const int u = ptid + it * TL::NTP;
      const int kg = u % TL::KG, r = u / TL::KG;
      const int rc = r < last_row ? r : last_row;
      voff[it] = (int)((rc * p.lda + kg * 8) * ES);
      slot[it] = kg * LL::kAPlane + (r ^ LL::swz(kg));
    }
    float ring[D][A_IT][8];
    auto issue = [&](int s, float (&r)[A_IT][8]) {
#pragma unroll
      for (int it = 0; it < A_IT; ++it) {
        const f32x4 v0 = llvm_raw_buffer_load_v4f32(ra, voff[it], s * TL::BK * ES, 0);
        const f32x4 v1 = llvm_raw_buffer_load_v4f32(ra, voff[it] + 16, s * TL::BK * ES, 0);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          r[it][e] = v0[e];
          r[it][4 + e] = v1[e];
        }
      }
    };
    // split one ring slot into LDS stage s&1 and, unit by unit, refill it for step s_next
    auto restage = [&](int s, float (&r)[A_IT][8], bool refill, int s_next) {
      u32x4* stage = lds + (s & 1) * LL::kStage;
#pragma unroll
      for (int it = 0; it < A_IT; ++it) {
        u32x4 t[TERMS];
        split8<FMT, TERMS>(r[it], t);
#pragma unroll
        for (int i = 0; i < TERMS; ++i) stage[i * LL::kATerm + slot[it]] = t[i];
        if (refill) {
          const f32x4 v0 = llvm_raw_buffer_load_v4f32(ra, voff[it], s_next * TL::BK * ES, 0);
          const f32x4 v1 = llvm_raw_buffer_load_v4f32(ra, voff[it] + 16, s_next * TL::BK * ES, 0);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            r[it][e] = v0[e];
            r[it][4 + e] = v1[e];
          }
        }
      }
    };
#pragma unroll
    for (int d = 0; d < D; ++d)
      if (d < ktiles) issue(d, ring[d]);
    int s = 0;
    for (; s + 2 * D <= ktiles; s += D) {
#pragma unroll
      for (int d = 0; d < D; ++d) {
        restage(s + d, ring[d], true, s + d + D);
        __syncthreads();
      }
    }
#pragma unroll
    for (int dd = 0; dd < 2 * D; ++dd) {
      const int d = dd % D;
      if (s + dd < ktiles) {
        restage(s + dd, ring[d], s + dd + D < ktiles, s + dd + D);
        __syncthreads();
      }
    }
    __syncthreads();
  }

  // ---- consumers: B straight from global memory, A fragments from LDS ----------------------------
  static __device__ __forceinline__ void consumer(const GemmParams& p, u32x4* lds, int m0, int n0, int ktiles, int wave,
                                                  int kbase, int split) {
    const int lane = threadIdx.x & 63, l31 = lane & 31, g = lane >> 5;
    const int wn0 = wave * 32;
    // this lane's column, clamped (results of clamped columns are never stored)
    const int col = (n0 + wn0 + l31 < p.N) ? (n0 + wn0 + l31) : (p.N - 1);
    const float* B = (const float*)p.B + (int64_t)kbase * p.ldb;
    const i32x4 rb = make_rsrc(B, ((int64_t)(p.K - 1 - kbase) * p.ldb + p.N) * ES);
    const int ldb_bytes = (int)(p.ldb * ES);
    const int voff_b = (g * 8) * ldb_bytes + col * ES;

    f32x16 acc[NCLS][TL::MT];
#pragma unroll
    for (int c = 0; c < NCLS; ++c)
#pragma unroll
      for (int mi = 0; mi < TL::MT; ++mi)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[c][mi][e] = 0.f;
    f32x16 master[AC::kChunked ? TL::MT : 1];
    if constexpr (AC::kChunked) {
#pragma unroll
      for (int mi = 0; mi < TL::MT; ++mi)
#pragma unroll
        for (int e = 0; e < 16; ++e) master[mi][e] = 0.f;
    }
    constexpr int kChunkSteps = (AC::kChunkK / TL::BK) > 0 ? (AC::kChunkK / TL::BK) : 1;

    // raw B of a K step: KSUB slices x 8 k rows (this lane's k-group) of this lane's column; two
    // steps are kept in flight (the loads of step kt + 2 are issued as soon as step kt is split)
    float raw[2][TL::KSUB][8];
    auto load_b = [&](int kt, float (&r)[TL::KSUB][8]) {
#pragma unroll
      for (int sub = 0; sub < TL::KSUB; ++sub)
#pragma unroll
        for (int e = 0; e < 8; ++e)
          r[sub][e] = llvm_raw_buffer_load_f32(rb, voff_b, (kt * TL::BK + sub * 16 + e) * ldb_bytes, 0);
    };
    if (ktiles > 0) load_b(0, raw[0]);
    if (ktiles > 1) load_b(1, raw[1]);

    __syncthreads();
    for (int kt2 = 0; kt2 < ktiles; kt2 += 2)
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int kt = kt2 + half;
      if (kt >= ktiles) break;
      const u32x4* sa = lds + (kt & 1) * LL::kStage;
      // split this step's B (frees its raw registers), then refill them for the step after next
      u32x4 bt[TL::KSUB][TERMS];
#pragma unroll
      for (int sub = 0; sub < TL::KSUB; ++sub) split8<FMT, TERMS>(raw[half][sub], bt[sub]);
      if (kt + 2 < ktiles) load_b(kt + 2, raw[half]);
#pragma unroll
      for (int sub = 0; sub < TL::KSUB; ++sub) {
        const int kg = sub * 2 + g;
        Vec a[TERMS][TL::MT];
#pragma unroll
        for (int i = 0; i < TERMS; ++i)
#pragma unroll
          for (int mi = 0; mi < TL::MT; ++mi)
            a[i][mi] = __builtin_bit_cast(Vec, sa[i * LL::kATerm + kg * LL::kAPlane + mi * 32 + (l31 ^ LL::swz(kg))]);
#pragma unroll
        for (int s = 2 * TERMS - 2; s >= 0; --s)
#pragma unroll
          for (int i = 0; i < TERMS; ++i) {
            const int j = s - i;
            if (j < 0 || j >= TERMS || !PS::keep(i, j)) continue;
            const int cls = AC::index(s);
#pragma unroll
            for (int mi = 0; mi < TL::MT; ++mi)
              acc[cls][mi] = LP::mfma(a[i][mi], __builtin_bit_cast(Vec, bt[sub][j]), acc[cls][mi]);
          }
      }
      if constexpr (AC::kChunked) if ((kt % kChunkSteps) == kChunkSteps - 1) {
#pragma unroll
        for (int mi = 0; mi < TL::MT; ++mi) {
          master[mi] += acc[0][mi];
#pragma unroll
          for (int e = 0; e < 16; ++e) acc[0][mi][e] = 0.f;
        }
      }
      __syncthreads();
    }
    if constexpr (AC::kChunked) {
#pragma unroll
      for (int mi = 0; mi < TL::MT; ++mi) acc[0][mi] += master[mi];
    }

    // epilogue: lane holds column l31 and rows 8*q + 4*g + e of every 32-row block
    const int ccol = n0 + wn0 + l31;
    if (SPLITK && p.k_splits > 1) {
      // fp32 partial tile of this K range, no bias: workspace [split][M][N], leading dimension N
      if (ccol >= p.N) return;
      float* dst0 = p.partials + ((int64_t)split * p.M) * p.N + ccol;
#pragma unroll
      for (int mi = 0; mi < TL::MT; ++mi) {
        f32x16 v = acc[NCLS - 1][mi];
#pragma unroll
        for (int c = NCLS - 2; c >= 0; --c) v = v * AC::kFoldScale + acc[c][mi];
        const int row0 = m0 + mi * 32 + g * 4;
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (row0 + q * 8 + e < p.M) dst0[(int64_t)(row0 + q * 8 + e) * p.N] = v[4 * q + e];
      }
      return;
    }
    float* C = (float*)p.C;
    const float* bias = (const float*)p.bias;
    const bool interior = (m0 + TL::BM <= p.M) && (n0 + wn0 + 32 <= p.N) && p.ldc * (int64_t)(TL::BM * ES) < 0x7FFFFFFF;
    if (interior) {
      const i32x4 rc = make_rsrc(C + (int64_t)m0 * p.ldc, 0x7FFFFFFF);
      const int ldc_bytes = (int)p.ldc * ES;
      const int voff = g * 4 * ldc_bytes + ccol * ES;
      const float bv = bias ? bias[ccol] : 0.f;
#pragma unroll
      for (int mi = 0; mi < TL::MT; ++mi) {
        f32x16 v = acc[NCLS - 1][mi];
#pragma unroll
        for (int c = NCLS - 2; c >= 0; --c) v = v * AC::kFoldScale + acc[c][mi];
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int e = 0; e < 4; ++e)
            llvm_raw_buffer_store_f32(v[4 * q + e] + bv, rc, voff, (mi * 32 + q * 8 + e) * ldc_bytes, kResultStoreAux);
      }
      return;
    }
    if (ccol >= p.N) return;
    const float bv = bias ? bias[ccol] : 0.f;
#pragma unroll
    for (int mi = 0; mi < TL::MT; ++mi) {
      f32x16 v = acc[NCLS - 1][mi];
#pragma unroll
      for (int c = NCLS - 2; c >= 0; --c) v = v * AC::kFoldScale + acc[c][mi];
      const int row0 = m0 + mi * 32 + g * 4;
      float* dst = C + (int64_t)row0 * p.ldc + ccol;
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (row0 + q * 8 + e < p.M) dst[(int64_t)(q * 8 + e) * p.ldc] = v[4 * q + e] + bv;
    }
  }

  static __device__ __forceinline__ void run(const GemmParams& p, u32x4* lds) {
    int tm, tn, split = 0, kbase = 0;
    int ktiles = p.K / TL::BK;  // the host only selects this kernel when K % BK == 0
    if (SPLITK) {
      // the splits of one tile are neighbours in the grid: they run at the same time
      const int tile = blockIdx.x / p.k_splits;
      split = blockIdx.x - tile * p.k_splits;
      tm = tile / p.tiles_n;
      tn = tile - tm * p.tiles_n;
      kbase = split * p.k_per_split;
      ktiles = p.k_per_split / TL::BK;
    } else {
      tile_coords(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
    }
    const int m0 = tm * TL::BM, n0 = tn * TL::BN;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (wave >= TL::NCW) producer(p, lds, m0, ktiles, kbase);
    else consumer(p, lds, m0, n0, ktiles, wave, kbase, split);
  }
};

template <class TL, int FMT, int TERMS, bool FULL, bool SPLITK>
__global__ __launch_bounds__(TL::NT) void cascmm_bdirect_kernel(const GemmParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char cascmm_smem[];
  BDirectGemm<TL, FMT, TERMS, FULL, SPLITK>::run(p, (u32x4*)cascmm_smem);
}

// Second pass of the split-K path: C[m][n] = bias[n] + sum over splits, in split order (so the
// result does not depend on scheduling), of partials[split][m][n].  Four consecutive columns
// per thread (N % 4 == 0 on this path), the loads of eight splits in flight.
static __global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ partials, int k_splits, int M,
                                                                   int N, const float* __restrict__ bias,
                                                                   float* __restrict__ C, int64_t ldc, int vec_out) {
  const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  const int64_t total = (int64_t)M * N;
  if (i >= total) return;
  const int m = (int)(i / N), n = (int)(i - (int64_t)m * N);
  const f32x4* src = (const f32x4*)(partials + i);
  const int64_t stride = total / 4;
  f32x4 s = src[0];
  int k = 1;
  // two to four splits (what the LDS-tiled kernels use): every load in flight before the first addition;
  // the general loop below waits for each load of its tail in turn.  Same order of additions.
  if (k_splits == 4) {
    const f32x4 v1 = __builtin_nontemporal_load(src + stride), v2 = __builtin_nontemporal_load(src + 2 * stride),
                v3 = __builtin_nontemporal_load(src + 3 * stride);
    s += v1;
    s += v2;
    s += v3;
    k = 4;
  } else if (k_splits == 3) {
    const f32x4 v1 = __builtin_nontemporal_load(src + stride), v2 = __builtin_nontemporal_load(src + 2 * stride);
    s += v1;
    s += v2;
    k = 3;
  }
  for (; k + 8 <= k_splits; k += 8) {
    f32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(src + (int64_t)(k + u) * stride);
#pragma unroll
    for (int u = 0; u < 8; ++u) s += v[u];
  }
  for (; k < k_splits; ++k) s += __builtin_nontemporal_load(src + (int64_t)k * stride);
  if (vec_out) {  // C rows and bias 16-byte aligned
    if (bias) s += *(const f32x4*)(bias + n);
    *(f32x4*)(C + (int64_t)m * ldc + n) = s;
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) C[(int64_t)m * ldc + n + e] = s[e] + (bias ? bias[n + e] : 0.f);
  }
}

}  // namespace cascmm
