// Shared device/host helpers of the cascaded low-precision matmul kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <tuple>
#include <utility>

#include "../../include/cascmm.h"

namespace cascmm {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

// Kernel launch whose status is the return value of the launch call itself: polling the runtime's
// "last error" afterwards would also return (and clear) an error some unrelated earlier call of the
// process left behind.
template <typename... KArgs, typename... Args>
inline hipError_t launch_kernel(void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t lds_bytes, hipStream_t stream,
                                Args&&... args) {
  static_assert(sizeof...(KArgs) == sizeof...(Args), "argument count does not match the kernel's signature");
  std::tuple<KArgs...> vals{static_cast<KArgs>(args)...};
  return std::apply(
      [&](auto&... v) {
        void* ptrs[] = {(void*)&v...};
        return hipLaunchKernel((const void*)kernel, grid, block, ptrs, lds_bytes, stream);
      },
      vals);
}
// keeps the first failure of a sequence of launches in ERR
#define CASCMM_LAUNCH(ERR, ...)                                \
  do {                                                         \
    const hipError_t cascmm_e_ = launch_kernel(__VA_ARGS__);   \
    if ((ERR) == hipSuccess) (ERR) = cascmm_e_;                \
  } while (0)

// ---------------------------------------------------------------------------------------
// memory element types (what A, B, C, bias are stored as)
// ---------------------------------------------------------------------------------------
template <int DT> struct IoType;
template <> struct IoType<CASCMM_DT_F32> {
  typedef float T;
  static __device__ __forceinline__ float load(const float* p) { return *p; }
  static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
};
template <> struct IoType<CASCMM_DT_F16> {
  typedef _Float16 T;
  static __device__ __forceinline__ float load(const _Float16* p) { return (float)*p; }
  static __device__ __forceinline__ void store(_Float16* p, float v) { *p = (_Float16)v; }
};
template <> struct IoType<CASCMM_DT_BF16> {
  typedef __bf16 T;
  static __device__ __forceinline__ float load(const __bf16* p) { return (float)*p; }
  static __device__ __forceinline__ void store(__bf16* p, float v) { *p = (__bf16)v; }
};

// ---------------------------------------------------------------------------------------
// low-precision term formats: rounding, term scaling, packing of 8 values into one 16-byte
// LDS slot (bf16 / fp16) and the MFMA that consumes two such slots.
//   r_0 = x;  t_i = lowp(r_i * 2^(shift*i));  r_{i+1} = r_i - t_i * 2^(-shift*i)
// Both the scaling and the residual are exact in fp32 (power-of-two scale, and the
// residual of a round-to-nearest needs fewer significand bits than fp32 has).
// ---------------------------------------------------------------------------------------
template <int FMT> struct Lowp;

template <> struct Lowp<CASCMM_FMT_BF16> {
  static constexpr int kShift = 0;
  static constexpr bool kTensorScaled = false;
  typedef bf16x8 Vec;
  // LDS planes (16-byte slots per 8 k of one row) that hold `terms` terms, the plane of term i
  // and the MFMA operand of term i inside a slot read from that plane
  static constexpr __host__ __device__ int planes(int terms) { return terms; }
  static constexpr __host__ __device__ int plane(int i) { return i; }
  static __device__ __forceinline__ Vec operand(u32x4 slot, int) { return __builtin_bit_cast(Vec, slot); }
  static __device__ __forceinline__ float element0(u32x4 slot, int) { return (float)__builtin_bit_cast(Vec, slot)[0]; }
  static __device__ __forceinline__ f32x16 mfma(Vec a, Vec b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  // round 8 residuals to the format, update the residuals, return the packed slot.
  // Pairwise: one packed convert gives two terms; their fp32 values are the two halves of
  // the packed word moved to the top 16 bits (1 shift, 1 and), then two subtractions.
  template <int TERM, bool LAST>
  static __device__ __forceinline__ u32x4 peel(float (&r)[8]) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    u32x4 out;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const f32x2 x = {r[2 * e], r[2 * e + 1]};
      const unsigned hp = __builtin_bit_cast(unsigned, __builtin_convertvector(x, bf16x2));
      out[e] = hp;
      if (!LAST) {
        r[2 * e] = r[2 * e] - __builtin_bit_cast(float, hp << 16);
        r[2 * e + 1] = r[2 * e + 1] - __builtin_bit_cast(float, hp & 0xFFFF0000u);
      }
    }
    return out;
  }
};

template <> struct Lowp<CASCMM_FMT_FP16> {
  static constexpr int kShift = 11;
  static constexpr bool kTensorScaled = false;
  typedef f16x8 Vec;
  static constexpr __host__ __device__ int planes(int terms) { return terms; }
  static constexpr __host__ __device__ int plane(int i) { return i; }
  static __device__ __forceinline__ Vec operand(u32x4 slot, int) { return __builtin_bit_cast(Vec, slot); }
  static __device__ __forceinline__ float element0(u32x4 slot, int) { return (float)__builtin_bit_cast(Vec, slot)[0]; }
  static __device__ __forceinline__ f32x16 mfma(Vec a, Vec b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  template <int TERM, bool LAST>
  static __device__ __forceinline__ u32x4 peel(float (&r)[8]) {
    constexpr float s = (float)(1u << (kShift * TERM > 30 ? 30 : kShift * TERM));
    constexpr float inv = 1.0f / s;
    Vec v;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      _Float16 t = (_Float16)(r[e] * s);
      v[e] = t;
      if (!LAST) r[e] = __builtin_fmaf(-(float)t, inv, r[e]);
    }
    return __builtin_bit_cast(u32x4, v);
  }
};

// fp8 (OCP e4m3, finite range +-448): 8 values of a term are 8 bytes, so one 16-byte slot
// holds two terms of the same 8 k (terms 0 | 1 in plane 0, term 2 in the low half of plane 1)
// and v_mfma_f32_32x32x16_fp8_fp8 takes a 64-bit half slot as its operand.  The term shift
// is 4 bits; the tensor scale 2^e (max|x| * 2^e in (224, 448]) is applied before the split and
// undone once on the result.
template <> struct Lowp<CASCMM_FMT_FP8> {
  static constexpr int kShift = 4;
  static constexpr bool kTensorScaled = true;
  typedef long Vec;
  static constexpr __host__ __device__ int planes(int terms) { return (terms + 1) / 2; }
  static constexpr __host__ __device__ int plane(int i) { return i / 2; }
  static __device__ __forceinline__ Vec operand(u32x4 slot, int i) {
    const unsigned lo = (i & 1) ? slot[2] : slot[0], hi = (i & 1) ? slot[3] : slot[1];
    return (long)(((unsigned long)hi << 32) | lo);
  }
  static __device__ __forceinline__ float element0(u32x4 slot, int i) {
    return __builtin_amdgcn_cvt_pk_f32_fp8((int)((i & 1) ? slot[2] : slot[0]), false)[0];
  }
  static __device__ __forceinline__ f32x16 mfma(Vec a, Vec b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(a, b, c, 0, 0, 0);
  }
  // round the 8 residuals (already scaled for this term) to fp8: two packed words; unless LAST,
  // the residuals become (r - t) * 16, the input of the next term (both steps exact)
  template <bool LAST>
  static __device__ __forceinline__ u32x2 peel(float (&r)[8]) {
    u32x2 out;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      int w = 0;
      w = __builtin_amdgcn_cvt_pk_fp8_f32(r[4 * h], r[4 * h + 1], w, false);
      w = __builtin_amdgcn_cvt_pk_fp8_f32(r[4 * h + 2], r[4 * h + 3], w, true);
      out[h] = (unsigned)w;
      if (!LAST) {
        const auto lo = __builtin_amdgcn_cvt_pk_f32_fp8(w, false);
        const auto hi = __builtin_amdgcn_cvt_pk_f32_fp8(w, true);
        r[4 * h] = (r[4 * h] - lo[0]) * 16.f;
        r[4 * h + 1] = (r[4 * h + 1] - lo[1]) * 16.f;
        r[4 * h + 2] = (r[4 * h + 2] - hi[0]) * 16.f;
        r[4 * h + 3] = (r[4 * h + 3] - hi[1]) * 16.f;
      }
    }
    return out;
  }
};

// split 8 consecutive k of one row / column into the LDS slots of every plane; in_scale is the
// tensor scale (formats with kTensorScaled only)
template <int FMT, int TERMS>
__device__ __forceinline__ void split8(float (&r)[8], u32x4 (&out)[Lowp<FMT>::planes(TERMS)], float in_scale = 1.f) {
  if constexpr (FMT == CASCMM_FMT_FP8) {
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] *= in_scale;
    const u32x2 t0 = Lowp<FMT>::template peel<TERMS == 1>(r);
    u32x2 t1 = {0u, 0u}, t2 = {0u, 0u};
    if constexpr (TERMS > 1) t1 = Lowp<FMT>::template peel<TERMS == 2>(r);
    if constexpr (TERMS > 2) t2 = Lowp<FMT>::template peel<true>(r);
    out[0] = (u32x4){t0[0], t0[1], t1[0], t1[1]};
    if constexpr (TERMS > 2) out[1] = (u32x4){t2[0], t2[1], 0u, 0u};
  } else {
    out[0] = Lowp<FMT>::template peel<0, TERMS == 1>(r);
    if constexpr (TERMS > 1) out[1] = Lowp<FMT>::template peel<1, TERMS == 2>(r);
    if constexpr (TERMS > 2) out[2] = Lowp<FMT>::template peel<2, TERMS == 3>(r);
  }
}

// scale class of product (i, j) is i + j; products kept: i + j <= TERMS-1 (tri) or all (full)
template <int TERMS, bool FULL> struct ProductSet {
  static constexpr int kClasses = FULL ? (2 * TERMS - 1) : TERMS;
  static constexpr __host__ __device__ bool keep(int i, int j) { return FULL || (i + j <= TERMS - 1); }
  static constexpr int count() {
    int n = 0;
    for (int i = 0; i < TERMS; ++i)
      for (int j = 0; j < TERMS; ++j) n += keep(i, j) ? 1 : 0;
    return n;
  }
};

// Accumulators.  Products of scale class s = i + j carry the factor 2^(-shift*s), so formats
// with a term shift need one accumulator per class.  bf16 terms are unscaled: one accumulator
// serves two terms (the dropped lo.lo product dominates the error there), but with three
// terms the result is at the fp32 rounding floor, and adding the small classes into the big
// hi.hi sum would round it once per MFMA; the classes are kept apart and added once at the end.
template <int FMT, int TERMS, bool FULL> struct AccClasses {
  static constexpr bool kScaled = Lowp<FMT>::kShift != 0;
  static constexpr int kCount = kScaled ? ProductSet<TERMS, FULL>::kClasses : (TERMS >= 3 ? 3 : 1);
  static constexpr float kFoldScale = kScaled ? 1.0f / (float)(1 << Lowp<FMT>::kShift) : 1.0f;
  static constexpr __host__ __device__ int index(int s) { return kCount == 1 ? 0 : (s < kCount ? s : kCount - 1); }
  // cascades that reach the fp32 rounding floor accumulate class 0 in blocks of kChunkK
  // (not fp8: its 12 bits of three terms stay far above that floor)
  static constexpr bool kChunked = FMT == CASCMM_FMT_FP8 ? false : (kScaled ? (TERMS >= 2) : (TERMS >= 3));
  static constexpr int kChunkK = 256;
};

// ---------------------------------------------------------------------------------------
// fp8 tensor scale: max|x| as a bit pattern (non-negative floats order like their bit patterns)
// ---------------------------------------------------------------------------------------
// bit pattern of max|x| over the elements this thread visits, reduced over its wave
// (FINITE_ONLY: infinities and NaNs are passed over, so that the scale serves the finite elements)
template <int IODT, bool FINITE_ONLY = false>
__device__ __forceinline__ unsigned amax_scan(const void* x, int64_t rows, int64_t cols, int64_t ld, unsigned block, unsigned blocks) {
  typedef typename IoType<IODT>::T T;
  const T* src = (const T*)x;
  unsigned best = 0;
  auto fold = [&](float v) {
    unsigned bits = __builtin_bit_cast(unsigned, v) & 0x7FFFFFFFu;
    if (FINITE_ONLY && bits >= 0x7F800000u) bits = 0;
    best = bits > best ? bits : best;
  };
  if (ld == cols) {
    // contiguous: one flat range, 16-byte loads where the element type and alignment allow
    const int64_t total = rows * cols;
    if (IODT == CASCMM_DT_F32 && ((uintptr_t)x % 16) == 0) {
      const int64_t quads = total / 4;
      const int64_t step = (int64_t)blocks * blockDim.x;
      int64_t i = (int64_t)block * blockDim.x + threadIdx.x;
      // four independent loads in flight per thread
      for (; i + 3 * step < quads; i += 4 * step) {
        f32x4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = ((const f32x4*)x)[i + u * step];
#pragma unroll
        for (int u = 0; u < 4; ++u) { fold(v[u][0]); fold(v[u][1]); fold(v[u][2]); fold(v[u][3]); }
      }
      for (; i < quads; i += step) {
        const f32x4 v = ((const f32x4*)x)[i];
        fold(v[0]); fold(v[1]); fold(v[2]); fold(v[3]);
      }
      if (block == 0 && threadIdx.x < total - quads * 4) fold(IoType<IODT>::load(src + quads * 4 + threadIdx.x));
    } else {
      for (int64_t i = (int64_t)block * blockDim.x + threadIdx.x; i < total; i += (int64_t)blocks * blockDim.x)
        fold(IoType<IODT>::load(src + i));
    }
  } else {
    for (int64_t r = block; r < rows; r += blocks)
      for (int64_t c = threadIdx.x; c < cols; c += blockDim.x) fold(IoType<IODT>::load(src + r * ld + c));
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const unsigned other = (unsigned)__shfl_xor((int)best, off, 64);
    best = other > best ? other : best;
  }
  return best;
}

template <int IODT, bool FINITE_ONLY = false>
__device__ __forceinline__ unsigned amax_scan(const void* x, int64_t rows, int64_t cols, int64_t ld) {
  return amax_scan<IODT, FINITE_ONLY>(x, rows, cols, ld, blockIdx.x, gridDim.x);
}

// the exponent e with max|x| * 2^e in (224, 448], from the bit pattern of max|x|
__device__ __forceinline__ int exp_of_amax(unsigned bits) {
  int e = 0;
  if (bits != 0 && bits < 0x7F800000u) {   // finite and non-zero
    int ex;
    const float m = frexpf(__builtin_bit_cast(float, bits), &ex);   // m in [0.5, 1)
    e = m <= 0.875f ? 9 - ex : 8 - ex;                              // 448 = 0.875 * 2^9
  }
  return e;
}

struct GemmParams {
  const void* A;
  const void* B;
  void* C;
  const void* bias;
  int M, N, K;
  int64_t lda, ldb, ldc;
  int tiles_m, tiles_n;
  int k_splits;          // split-K path only
  int k_per_split;       // split-K path only (multiple of the kernel's BK)
  float* partials;       // split-K workspace: [k_splits][M][N] fp32
  const int32_t* tensor_exps;
};

// A group of GEMMs of one shape launched as one kernel (count == 1 for a plain GEMM).  Work
// item i = problem i / tiles, tile i % tiles; workgroup w runs items w, w + grid, w + 2 grid ...
constexpr int kMaxGroup = 8;
// gelu(g) = 0.5 g (1 + erf(g / sqrt 2)) = 0.5 g erfc(-g / sqrt 2), and value x gelu(gate).
// With x = |g| / sqrt 2 <= 4:  t = erfc(x) = 2^P(x), P a degree-11 fit of log2 erfc on [0, 4]
// (|P - log2 erfc| < 4e-8, so t is good to a few 1e-6 RELATIVE down to erfc(4) = 1.5e-8), and
// 1 + erf(g / sqrt 2) = t for g < 0, 2 - t otherwise: no cancellation in the negative tail, no
// branch, one v_exp_f32.  Evaluated in fp32 the gate is within 4e-7 (one ulp at its largest)
// of the exact gelu, like the textbook formula on a correctly rounded erff.
__device__ __forceinline__ float gelu_value(float g) {
  const float ax = __builtin_fabsf(g) * 0.70710678118654752f;
  const float x = __builtin_fminf(ax, 4.0f);
  float p = 1.133601089e-07f;
  p = __builtin_fmaf(p, x, -2.984485036e-06f);
  p = __builtin_fmaf(p, x, 3.493388431e-05f);
  p = __builtin_fmaf(p, x, -2.373710740e-04f);
  p = __builtin_fmaf(p, x, 1.004358870e-03f);
  p = __builtin_fmaf(p, x, -2.405994106e-03f);
  p = __builtin_fmaf(p, x, 7.954029570e-05f);
  p = __builtin_fmaf(p, x, 2.782256342e-02f);
  p = __builtin_fmaf(p, x, -1.483802944e-01f);
  p = __builtin_fmaf(p, x, -9.184222221e-01f);
  p = __builtin_fmaf(p, x, -1.627909303e+00f);
  p = __builtin_fmaf(p, x, 3.292588246e-08f);
  const float t = ax > 4.0f ? 0.f : __builtin_amdgcn_exp2f(p);   // beyond: erfc < 1.6e-8, taken as 0
  return 0.5f * g * (g < 0.f ? t : 2.f - t);
}
__device__ __forceinline__ float gated_value(float v, float g) { return v * gelu_value(g); }

struct GroupParams {
  int M, N, K;
  int64_t lda, ldb, ldc;
  int tiles_m, tiles_n;
  int count;
  const void* A[kMaxGroup];
  const void* B[kMaxGroup];
  void* C[kMaxGroup];
  const void* bias[kMaxGroup];
  void* workspace;          // split-K partials: fp32 [k_splits][M][N]
  size_t workspace_bytes;
  int k_splits;             // LDS-tiled kernels: work item = (split, problem, tile); 0 or 1 = no split
  const int32_t* tensor_exps;  // fp8: {e_A, e_B} of problem i at [2i], [2i + 1]; NULL = all zero
  // Gated epilogue: C has N/2 columns, C[m][32 j + l] = (v + bias[32 j + l]) * gelu(g + bias[N/2 + 32 j + l])
  // with v and g the entries of A x B in row m whose columns of B are, for a prepared operand (which
  // alternates 32 "value" and 32 "gate" columns), 64 j + l and 64 j + 32 + l, and for a raw operand
  // (value columns in the first half, gate columns in the second) 32 j + l and N/2 + 32 j + l.
  // glu == 2 (large-tile kernel only): the gated result leaves as the left operand slots of the next GEMM,
  // two bf16 terms, [term][(N / 2) / 8][M] x 16 bytes at C (see cascmm_prepare_left for the order of k)
  int glu;
  // fp8-rate kernel only: the left operand's scale exponent is found inside the launch (two kernels:
  // per-workgroup maxima, then the operand split reduces them) and written, with *b_exp_src, to
  // exps_dyn[0..1], which the GEMM then reads instead of tensor_exps
  int32_t* exps_dyn;
  const int32_t* b_exp_src;
  // host side only: when set, the variant's launch function stores the handle of its GEMM kernel here
  // and returns without checking or launching anything (the library names its kernels this way)
  const void** kernel_out;
};

}  // namespace cascmm
