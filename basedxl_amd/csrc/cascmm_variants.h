// Host-side table of compiled kernel variants and the launcher template that fills it.
#pragma once
#include <atomic>
#include <cstring>
#include <mutex>

#include "cascmm_bdirect_kernel.h"
#include "cascmm_w512_kernel.h"
#include "cascmm_f8k64_kernel.h"
#include "cascmm_f16k_kernel.h"
#include "cascmm_wavek_kernel.h"

namespace cascmm {

// KIND_W512: the large-tile kernel (whole 256 x 320 tiles only, one problem per launch)
// KIND_F8K64: three fp8 terms on the fp8-rate MFMA; splits its operands into the workspace first
// KIND_F16K: three fp16 terms on operand slots; finds both scales and splits its operands into the workspace first
// KIND_WAVEK: skinny problems in one launch, K split over the waves of a workgroup (no workspace)
// KIND_SLOTK: prepared right operand, K split over the waves of a workgroup (64 x 160 tiles, one problem per launch)
enum VariantKind { KIND_TILE = 0, KIND_SPLITK = 1, KIND_W512 = 2, KIND_F8K64 = 3, KIND_WAVEK = 4, KIND_SLOTK = 5, KIND_F16K = 6 };
constexpr int kNumCUs = 256;  // MI355X: what the cost model's constants were measured on
constexpr int kMaxDevices = 64;

// compute units of the current device (asked once per device; kNumCUs when no device answers, as in
// a build container, where only the host-side selection logic runs)
inline int device_index() {
  int d = 0;
  if (hipGetDevice(&d) != hipSuccess || d < 0 || d >= kMaxDevices) {
    (void)hipGetLastError();   // a failure of this query is handled here and not left behind
    return -1;
  }
  return d;
}
inline int device_cus() {
  static std::atomic<int> cus[kMaxDevices];   // (zero-initialised; every thread that finds 0 stores the same answer)
  const int d = device_index();
  if (d < 0) return kNumCUs;
  int n = cus[d].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, d) != hipSuccess || n <= 0) n = kNumCUs;
    cus[d].store(n, std::memory_order_relaxed);
  }
  return n;
}

// More than 64 KB of dynamic LDS must be asked for once per kernel and device.  `done` is the kernel's
// own per-device record (zero-initialised atomics: host threads may launch at once; the attribute call
// is idempotent, so two threads that both find the flag clear both make it and both succeed).
typedef std::atomic<bool> LdsFlags[kMaxDevices];
inline bool ensure_lds(const void* kfn, int lds_bytes, LdsFlags& done) {
  const int d = device_index();
  if (d < 0) return false;
  if (done[d].load(std::memory_order_acquire)) return true;
  if (hipFuncSetAttribute(kfn, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) != hipSuccess) return false;
  done[d].store(true, std::memory_order_release);
  return true;
}

struct VariantDesc {
  const char* name;
  int kind;
  int iodt, fmt, terms, full;
  int BM, BN, BK, threads;
  int lds_bytes;
  bool fast;  // needs fp32 operands, K % BK == 0, 16-byte aligned A rows
  bool grouped;  // one launch may run several same-shape problems and several tiles per workgroup
  int (*launch)(const GroupParams&, hipStream_t);
  bool bpre = false;  // takes the right operand already split (cascmm_prepare_weight)
  bool glu = false;   // has the gated epilogue
};

template <class TL, int IODT, int FMT, int TERMS, bool FULL, bool FAST, bool BPRE = false>
int launch_tile(const GroupParams& p, hipStream_t stream) {
  auto kfn = cascmm_tile_kernel<TL, IODT, FMT, TERMS, FULL, FAST, BPRE>;
  if (p.kernel_out) { *p.kernel_out = (const void*)kfn; return CASCMM_OK; }
  constexpr int lds = LdsLayout<TL, Lowp<FMT>::planes(TERMS)>::kBytes;
  static_assert(lds <= 160 * 1024, "tile does not fit the 160 KB LDS");
  if (lds > 64 * 1024) {
    static LdsFlags lds_set;
    if (!ensure_lds((const void*)kfn, lds, lds_set)) return CASCMM_ERR_LAUNCH;
  }
  // persistent grid: at most as many workgroups as can be resident at once on this device
  static std::atomic<int> occupancy[kMaxDevices];
  const int dev = device_index();
  if (dev < 0) return CASCMM_ERR_LAUNCH;
  int per_cu = occupancy[dev].load(std::memory_order_relaxed);
  if (per_cu == 0) {
    int n = 0;
    per_cu = (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, (const void*)kfn, TL::NT, lds) == hipSuccess && n > 0) ? n : 1;
    occupancy[dev].store(per_cu, std::memory_order_relaxed);
  }
  const int splits = p.k_splits > 1 ? p.k_splits : 1;
  if (splits > 1) {
    // K split: fp32 only, one problem, partial results [split][M][N] in the workspace
    if (p.glu) return CASCMM_ERR_BAD_VARIANT;
    if (IODT != CASCMM_DT_F32 || p.count != 1 || p.N % 4 != 0 || ((p.K + TL::BK - 1) / TL::BK) % splits != 0)
      return CASCMM_ERR_BAD_VARIANT;
    if (!p.workspace || p.workspace_bytes < (size_t)splits * p.M * p.N * sizeof(float)) return CASCMM_ERR_WORKSPACE;
    if ((uintptr_t)p.workspace % 16 != 0) return CASCMM_ERR_ALIGNMENT;
  }
  const int64_t total = (int64_t)splits * p.count * p.tiles_m * p.tiles_n;
  const int64_t resident = (int64_t)device_cus() * per_cu;
  const unsigned grid = (unsigned)(total < resident ? total : resident);
  if (launch_kernel(kfn, dim3(grid), dim3(TL::NT), lds, stream, p) != hipSuccess) return CASCMM_ERR_LAUNCH;
  if (splits > 1) {
    const int64_t elems = (int64_t)p.M * p.N;
    const int vec_out = p.ldc % 4 == 0 && (uintptr_t)p.C[0] % 16 == 0 && (uintptr_t)p.bias[0] % 16 == 0;
    if (launch_kernel(splitk_reduce_kernel, dim3((unsigned)((elems / 4 + 255) / 256)), dim3(256), 0, stream,
                      (const float*)p.workspace, splits, p.M, p.N, (const float*)p.bias[0], (float*)p.C[0], p.ldc,
                      vec_out) != hipSuccess)
      return CASCMM_ERR_LAUNCH;
  }
  return CASCMM_OK;
}

#define CASCMM_TILE_VARIANT(NAME, BM, BN, BK, WM, WN, WK, DEPTH, IODT, FMT, TERMS, FULL, FAST)         \
  {NAME, KIND_TILE, IODT, FMT, TERMS, FULL, BM, BN, BK, Tile<BM, BN, BK, WM, WN, WK, DEPTH>::NT,       \
   LdsLayout<Tile<BM, BN, BK, WM, WN, WK, DEPTH>, Lowp<FMT>::planes(TERMS)>::kBytes, FAST, true,       \
   &launch_tile<Tile<BM, BN, BK, WM, WN, WK, DEPTH>, IODT, FMT, TERMS, FULL, FAST>}

// same with the number of producer waves given explicitly
#define CASCMM_TILE_VARIANT_P(NAME, BM, BN, BK, WM, WN, WK, DEPTH, NP, IODT, FMT, TERMS, FULL, FAST)    \
  {NAME, KIND_TILE, IODT, FMT, TERMS, FULL, BM, BN, BK, Tile<BM, BN, BK, WM, WN, WK, DEPTH, NP>::NT,   \
   LdsLayout<Tile<BM, BN, BK, WM, WN, WK, DEPTH, NP>, Lowp<FMT>::planes(TERMS)>::kBytes, FAST, true,   \
   &launch_tile<Tile<BM, BN, BK, WM, WN, WK, DEPTH, NP>, IODT, FMT, TERMS, FULL, FAST>}

// permuted B columns staged in 8 x 2 blocks (Tile's PAIRS flag)
#define CASCMM_TILE_VARIANT_PAIRS(NAME, BM, BN, BK, WM, WN, WK, DEPTH, NP, IODT, FMT, TERMS, FULL, FAST)             \
  {NAME, KIND_TILE, IODT, FMT, TERMS, FULL, BM, BN, BK, Tile<BM, BN, BK, WM, WN, WK, DEPTH, NP, true, true>::NT,    \
   LdsLayout<Tile<BM, BN, BK, WM, WN, WK, DEPTH, NP, true, true>, Lowp<FMT>::planes(TERMS)>::kBytes, FAST, true,    \
   &launch_tile<Tile<BM, BN, BK, WM, WN, WK, DEPTH, NP, true, true>, IODT, FMT, TERMS, FULL, FAST>}

// K splits of the skinny path: enough workgroups to occupy every CU, each with at least one
// K step of `bk`; the same function sizes the workspace
inline int skinny_splits(int64_t M, int64_t N, int64_t K, int bm, int bn, int bk) {
  const int64_t tiles = ((M + bm - 1) / bm) * ((N + bn - 1) / bn);
  int best = 1;
  for (int s = 1; s <= 64; ++s) {
    if (K % ((int64_t)s * bk) != 0) continue;
    best = s;
    if (tiles * s >= kNumCUs / 2) break;  // measured optimum on 154 x 2048 x 1280
  }
  return best;
}

// Split-K workspace: one fp32 [M][N] partial result per split
inline size_t skinny_workspace_bytes(int64_t M, int64_t N, int64_t K, int bm, int bn, int bk) {
  const int splits = skinny_splits(M, N, K, bm, bn, bk);
  return splits <= 1 ? 0 : (size_t)splits * (size_t)M * (size_t)N * sizeof(float);
}

template <class TL, int FMT, int TERMS, bool FULL, bool SPLITK>
int launch_bdirect(const GroupParams& gp, hipStream_t stream) {
  if (gp.kernel_out) { *gp.kernel_out = (const void*)cascmm_bdirect_kernel<TL, FMT, TERMS, FULL, SPLITK>; return CASCMM_OK; }
  if (gp.count != 1) return CASCMM_ERR_BAD_VARIANT;
  GemmParams p;
  memset(&p, 0, sizeof(p));
  p.A = gp.A[0]; p.B = gp.B[0]; p.C = gp.C[0]; p.bias = gp.bias[0];
  p.M = gp.M; p.N = gp.N; p.K = gp.K; p.lda = gp.lda; p.ldb = gp.ldb; p.ldc = gp.ldc;
  p.tiles_m = gp.tiles_m; p.tiles_n = gp.tiles_n;
  p.k_splits = 1;
  p.k_per_split = gp.K;
  if (SPLITK) {
    p.k_splits = skinny_splits(gp.M, gp.N, gp.K, TL::BM, TL::BN, TL::BK);
    p.k_per_split = gp.K / p.k_splits;
    if (p.k_splits > 1) {
      const size_t need = skinny_workspace_bytes(gp.M, gp.N, gp.K, TL::BM, TL::BN, TL::BK);
      if (!gp.workspace || gp.workspace_bytes < need) return CASCMM_ERR_WORKSPACE;
      if ((uintptr_t)gp.workspace % 16 != 0) return CASCMM_ERR_ALIGNMENT;
      p.partials = (float*)gp.workspace;
    }
  }
  auto kfn = cascmm_bdirect_kernel<TL, FMT, TERMS, FULL, SPLITK>;
  constexpr int lds = LdsLayoutA<TL, TERMS>::kBytes;
  static_assert(lds <= 160 * 1024, "tile does not fit the 160 KB LDS");
  if (lds > 64 * 1024) {
    static LdsFlags lds_set;
    if (!ensure_lds((const void*)kfn, lds, lds_set)) return CASCMM_ERR_LAUNCH;
  }
  const unsigned grid = (unsigned)p.tiles_m * (unsigned)p.tiles_n * (unsigned)p.k_splits;
  if (launch_kernel(kfn, dim3(grid), dim3(TL::NT), lds, stream, p) != hipSuccess) return CASCMM_ERR_LAUNCH;
  if (SPLITK && p.k_splits > 1) {
    const int64_t total = (int64_t)gp.M * gp.N;
    const int vec_out = gp.ldc % 4 == 0 && (uintptr_t)p.C % 16 == 0 && (uintptr_t)p.bias % 16 == 0;
    if (launch_kernel(splitk_reduce_kernel, dim3((unsigned)((total / 4 + 255) / 256)), dim3(256), 0, stream, p.partials,
                      p.k_splits, gp.M, gp.N, (const float*)p.bias, (float*)p.C, gp.ldc, vec_out) != hipSuccess)
      return CASCMM_ERR_LAUNCH;
  }
  return CASCMM_OK;
}

// the large-tile kernel (BPRE = 1: right operand prepared)
template <int BPRE, int GLU>
int launch_w512_kernel(const GroupParams& p, hipStream_t stream) {
  typedef W512 T;
  auto kfn = cascmm_w512_kernel<BPRE, GLU>;
  static LdsFlags lds_set;
  if (!ensure_lds((const void*)kfn, T::LDS_BYTES, lds_set)) return CASCMM_ERR_LAUNCH;
  const unsigned grid = (unsigned)(p.tiles_m * p.tiles_n);
  if (launch_kernel(kfn, dim3(grid), dim3(T::NT), (size_t)T::LDS_BYTES, stream, p) != hipSuccess) return CASCMM_ERR_LAUNCH;
  return CASCMM_OK;
}

template <int BPRE>
int launch_w512(const GroupParams& p, hipStream_t stream) {
  typedef W512 T;
  if (p.kernel_out) { *p.kernel_out = (const void*)cascmm_w512_kernel<BPRE, 0>; return CASCMM_OK; }
  if (p.count != 1 || p.k_splits > 1) return CASCMM_ERR_BAD_VARIANT;
  if (p.M % T::BM != 0 || p.N % T::BN != 0 || p.K % 32 != 0 || p.K < 32) return CASCMM_ERR_BAD_VARIANT;
  if ((int64_t)p.M * p.lda * 4 > 0x7FFFFFFF || (int64_t)p.K * p.ldb * 4 > 0x7FFFFFFF || p.ldc * (int64_t)(T::BM * 4) > 0x7FFFFFFF)
    return CASCMM_ERR_TOO_LARGE;
  // (the gated stores are instantiations of their own; glu == 2: the result leaves as operand slots)
  if (p.glu == 2) return launch_w512_kernel<BPRE, 2>(p, stream);
  return p.glu ? launch_w512_kernel<BPRE, 1>(p, stream) : launch_w512_kernel<BPRE, 0>(p, stream);
}

// skinny problems, K split over the waves of a workgroup
template <int NB>
int launch_wavek(const GroupParams& p, hipStream_t stream) {
  typedef WaveK<NB> T;
  if (p.kernel_out) { *p.kernel_out = (const void*)cascmm_wavek_kernel<NB>; return CASCMM_OK; }
  if (p.glu || p.k_splits > 1 || p.count < 1) return CASCMM_ERR_BAD_VARIANT;
  if (p.N % T::BN != 0 || p.K % T::BK != 0) return CASCMM_ERR_BAD_VARIANT;
  if ((int64_t)p.M * p.lda * 4 > 0x7FFFFFFF || (int64_t)p.K * p.ldb * 4 > 0x7FFFFFFF) return CASCMM_ERR_TOO_LARGE;
  auto kfn = cascmm_wavek_kernel<NB>;
  static LdsFlags lds_set;
  if (!ensure_lds((const void*)kfn, T::LDS_BYTES, lds_set)) return CASCMM_ERR_LAUNCH;
  GroupParams q = p;
  q.tiles_m = (p.M + T::BM - 1) / T::BM;
  q.tiles_n = p.N / T::BN;
  const int64_t grid = (int64_t)q.count * q.tiles_m * q.tiles_n;
  if (grid <= 0 || grid > 0x7FFFFFFF) return CASCMM_ERR_TOO_LARGE;
  if (launch_kernel(kfn, dim3((unsigned)grid), dim3(T::NT), (size_t)T::LDS_BYTES, stream, q) != hipSuccess) return CASCMM_ERR_LAUNCH;
  return CASCMM_OK;
}

// K split of the fp8-rate kernel (row tile bm = 256 or 128) for problems with fewer tiles than CUs:
// the split count that minimises stages-per-workgroup x the stage time + the round trip of the
// partial results at ~4 TB/s
inline double f8k64_stage_us(int bm) { return bm == 256 ? 2.1 : 1.15; }
// the tile of a variant: MT = 2, 1: the LDS-tiled kernel's 256 / 128 rows; MT = 0: the 64 x 160 tile whose K is split over
// the waves of a workgroup (cascmm_f8wk_kernel.h: one launch, never a K split over workgroups)
template <int MT> struct F8Tile { typedef F8K64T<MT> T; };
template <> struct F8Tile<0> { typedef F8WK T; };
inline int f8k64_splits(int64_t M, int64_t N, int64_t K, int bm) {
  if (bm == F8WK::BM) return 1;
  const int64_t tiles = ((M + bm - 1) / bm) * ((N + F8K64::BN - 1) / F8K64::BN);
  const int64_t steps = K / F8K64::BK;
  int best = 1;
  double best_us = (double)steps * f8k64_stage_us(bm);
  for (int sp = 2; sp <= 16; ++sp) {
    if (steps % sp != 0 || tiles * sp > kNumCUs) continue;
    const double us = (double)(steps / sp) * f8k64_stage_us(bm) + 3.0 + (double)(sp + 1) * (double)M * (double)N * 4.0 / 4.0e6;
    if (us < best_us) {
      best_us = us;
      best = sp;
    }
  }
  return best;
}

// Workspace of the fp8-rate kernel: the slots of A, those of B unless B comes prepared, the partial
// results of a K split (each rounded up to 256 bytes so that the next buffer stays aligned), and the
// per-workgroup maxima of a scale search done inside the launch
constexpr int kF8K64AmaxGroups = 256;
inline size_t f8k64_up(int64_t b) { return (size_t)((b + 255) / 256 * 256); }
inline size_t f8k64_workspace_bytes(int64_t M, int64_t N, int64_t K, bool bpre, int bm) {
  const int sp = f8k64_splits(M, N, K, bm);
  return f8k64_up(f8k64_slot_bytes(M, K)) + (bpre ? 0 : f8k64_up(f8k64_slot_bytes(N, K))) +
         (sp > 1 ? f8k64_up((int64_t)sp * M * N * 4) : 0) + kF8K64AmaxGroups * sizeof(unsigned);
}

// the fp8-rate kernel: split A (and B) into operand slots, then the GEMM on the slots
template <bool BPRE, int MT>
int launch_f8k64(const GroupParams& p, hipStream_t stream) {
  typedef typename F8Tile<MT>::T T;
  void (*kfn)(const F8K64Params) = MT == 0 ? cascmm_f8wk_kernel<0> : cascmm_f8k64_kernel<(MT == 0 ? 1 : MT)>;
  if (p.kernel_out) { *p.kernel_out = (const void*)kfn; return CASCMM_OK; }
  if (p.count != 1 || p.glu || p.k_splits > 1 || p.K % T::BK != 0 || p.K == 0) return CASCMM_ERR_BAD_VARIANT;
  const size_t need = f8k64_workspace_bytes(p.M, p.N, p.K, BPRE, T::BM);
  if (!p.workspace || p.workspace_bytes < need) return CASCMM_ERR_WORKSPACE;
  if ((uintptr_t)p.workspace % 16 != 0) return CASCMM_ERR_ALIGNMENT;
  if (f8k64_slot_bytes(p.M, p.K) > 0x7FFFFFFF || f8k64_slot_bytes(p.N, p.K) > 0x7FFFFFFF) return CASCMM_ERR_TOO_LARGE;
  static LdsFlags lds_set;
  if (!ensure_lds((const void*)kfn, T::LDS_BYTES, lds_set)) return CASCMM_ERR_LAUNCH;
  u32x4* a_slots = (u32x4*)p.workspace;
  const u32x4* b_slots = (const u32x4*)p.B[0];
  char* ws_next = (char*)p.workspace + f8k64_up(f8k64_slot_bytes(p.M, p.K));
  const int kus = p.K >> 4;
  const unsigned a_grid = (unsigned)(((p.M + 63) / 64) * ((kus + 3) / 4));
  const int32_t* exps = p.tensor_exps;
  const int32_t* b_exp = p.tensor_exps ? p.tensor_exps + 1 : (const int32_t*)nullptr;
  const unsigned* amax = nullptr;
  int n_amax = 0;
  if (p.exps_dyn) {
    // the scale of A is not known yet: per-workgroup maxima now, reduced by the split of A, which
    // leaves {e_A, e_B} in exps_dyn for the GEMM (no atomics, no pass of its own for the reduction)
    unsigned* am = (unsigned*)((char*)p.workspace + need - kF8K64AmaxGroups * sizeof(unsigned));
    const int64_t total = (int64_t)p.M * p.K;
    n_amax = (int)std::max<int64_t>(1, std::min<int64_t>((total + 8191) / 8192, kF8K64AmaxGroups));
    if (launch_kernel(f8k64_amax_kernel<0>, dim3((unsigned)n_amax), dim3(1024), 0, stream, (const float*)p.A[0], (int64_t)p.M,
                      (int64_t)p.K, p.lda, am) != hipSuccess)
      return CASCMM_ERR_LAUNCH;
    amax = am;
    exps = p.exps_dyn;
    b_exp = p.b_exp_src;
  }
  if (launch_kernel(f8k64_split_rows_kernel<0>, dim3(a_grid), dim3(256), 0, stream, (const float*)p.A[0], p.M, p.K, p.lda,
                    p.exps_dyn ? (const int32_t*)nullptr : p.tensor_exps, a_slots, amax, n_amax, b_exp, p.exps_dyn) != hipSuccess)
    return CASCMM_ERR_LAUNCH;
  if (!BPRE) {
    u32x4* bs = (u32x4*)ws_next;
    ws_next += f8k64_up(f8k64_slot_bytes(p.N, p.K));
    const int64_t units = (int64_t)kus * p.N;
    if (launch_kernel(f8k64_split_cols_kernel<0>, dim3((unsigned)((units + 255) / 256)), dim3(256), 0, stream, (const float*)p.B[0],
                      p.K, p.N, p.ldb, b_exp, bs) != hipSuccess)
      return CASCMM_ERR_LAUNCH;
    b_slots = bs;
  }
  F8K64Params q;
  q.a_slots = a_slots; q.b_slots = b_slots; q.C = (float*)p.C[0]; q.bias = (const float*)p.bias[0];
  q.tensor_exps = exps;
  q.M = p.M; q.N = p.N; q.K = p.K; q.ldc = p.ldc;
  q.tiles_m = (p.M + T::BM - 1) / T::BM; q.tiles_n = (p.N + T::BN - 1) / T::BN;
  q.k_splits = f8k64_splits(p.M, p.N, p.K, T::BM);
  q.partials = (float*)ws_next;
  const unsigned grid = (unsigned)(q.tiles_m * q.tiles_n * q.k_splits);
  if (launch_kernel(kfn, dim3(grid), dim3(T::NT), (size_t)T::LDS_BYTES, stream, q) != hipSuccess) return CASCMM_ERR_LAUNCH;
  if (q.k_splits > 1) {
    const int64_t elems = (int64_t)p.M * p.N;
    const int vec_out = p.ldc % 4 == 0 && p.N % 4 == 0 && (uintptr_t)p.C[0] % 16 == 0 && (uintptr_t)p.bias[0] % 16 == 0;
    if (launch_kernel(splitk_reduce_kernel, dim3((unsigned)((elems / 4 + 255) / 256)), dim3(256), 0, stream,
                      (const float*)q.partials, q.k_splits, p.M, p.N, (const float*)p.bias[0], (float*)p.C[0], p.ldc,
                      vec_out) != hipSuccess)
      return CASCMM_ERR_LAUNCH;
  }
  return CASCMM_OK;
}

// Workspace of the three-term fp16 kernels on operand slots: the slots of A and of B (each rounded up to 256 bytes),
// the per-workgroup maxima of the two scale searches, the two exponents
inline size_t f16k_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  return f8k64_up(f16k_slot_bytes(M, K)) + f8k64_up(f16k_slot_bytes(N, K)) + 2 * kF8K64AmaxGroups * sizeof(unsigned) + 256;
}

// the three-term fp16 kernels on operand slots: find both scales, split A and B into slots, then the GEMM on the slots
// (WK: the 64 x 160 tile with K over the waves of a workgroup; otherwise the 256 x 160 tile staged through LDS)
template <bool WK>
int launch_f16k(const GroupParams& p, hipStream_t stream) {
  typedef typename std::conditional<WK, F16WK, F16K>::type T;
  void (*kfn)(const F8K64Params) = WK ? cascmm_f16wk_kernel<0> : cascmm_f16k_kernel<0>;
  if (p.kernel_out) { *p.kernel_out = (const void*)kfn; return CASCMM_OK; }
  if (p.count != 1 || p.glu || p.k_splits > 1 || p.K % T::BK != 0 || p.K == 0 || (!WK && p.K > F16K::MAX_K)) return CASCMM_ERR_BAD_VARIANT;
  const size_t need = f16k_workspace_bytes(p.M, p.N, p.K);
  if (!p.workspace || p.workspace_bytes < need) return CASCMM_ERR_WORKSPACE;
  if ((uintptr_t)p.workspace % 16 != 0) return CASCMM_ERR_ALIGNMENT;
  if (f16k_slot_bytes(p.M, p.K) > 0x7FFFFFFF || f16k_slot_bytes(p.N, p.K) > 0x7FFFFFFF) return CASCMM_ERR_TOO_LARGE;
  static LdsFlags lds_set;
  if (!ensure_lds((const void*)kfn, T::LDS_BYTES, lds_set)) return CASCMM_ERR_LAUNCH;
  char* ws = (char*)p.workspace;
  u32x4* a_slots = (u32x4*)ws;
  ws += f8k64_up(f16k_slot_bytes(p.M, p.K));
  u32x4* b_slots = (u32x4*)ws;
  ws += f8k64_up(f16k_slot_bytes(p.N, p.K));
  unsigned* amax_a = (unsigned*)ws;
  unsigned* amax_b = amax_a + kF8K64AmaxGroups;
  int32_t* exps = (int32_t*)(amax_b + kF8K64AmaxGroups);
  const int n_a = (int)std::max<int64_t>(1, std::min<int64_t>(((int64_t)p.M * p.K + 8191) / 8192, kF8K64AmaxGroups));
  const int n_b = (int)std::max<int64_t>(1, std::min<int64_t>(((int64_t)p.K * p.N + 8191) / 8192, kF8K64AmaxGroups));
  if (launch_kernel(f16k_amax_kernel<0>, dim3((unsigned)(n_a + n_b)), dim3(1024), 0, stream, (const float*)p.A[0], (int64_t)p.M,
                    (int64_t)p.K, p.lda, n_a, (const float*)p.B[0], (int64_t)p.N, p.ldb, amax_a, amax_b) != hipSuccess)
    return CASCMM_ERR_LAUNCH;
  const int kus = p.K >> 3;
  const int a_blocks = ((p.M + 63) / 64) * ((kus + 3) / 4);
  const int64_t b_blocks = ((int64_t)kus * p.N + 255) / 256;
  if (launch_kernel(f16k_split_kernel<0>, dim3((unsigned)(a_blocks + b_blocks)), dim3(256), 0, stream, (const float*)p.A[0], p.M, p.K,
                    p.lda, a_slots, (const unsigned*)amax_a, n_a, a_blocks, (const float*)p.B[0], p.N, p.ldb, b_slots,
                    (const unsigned*)amax_b, n_b, exps) != hipSuccess)
    return CASCMM_ERR_LAUNCH;
  F8K64Params q;
  q.a_slots = a_slots; q.b_slots = b_slots; q.C = (float*)p.C[0]; q.bias = (const float*)p.bias[0];
  q.tensor_exps = exps;
  q.M = p.M; q.N = p.N; q.K = p.K; q.ldc = p.ldc;
  q.tiles_m = (p.M + T::BM - 1) / T::BM; q.tiles_n = (p.N + T::BN - 1) / T::BN;
  q.k_splits = 1;
  q.partials = nullptr;
  const unsigned grid = (unsigned)(q.tiles_m * q.tiles_n);
  if (launch_kernel(kfn, dim3(grid), dim3(T::NT), (size_t)T::LDS_BYTES, stream, q) != hipSuccess) return CASCMM_ERR_LAUNCH;
  return CASCMM_OK;
}

#define CASCMM_F16K_VARIANT(NAME, WK)                                                                                      \
  {NAME, KIND_F16K, CASCMM_DT_F32, CASCMM_FMT_FP16, 3, false, std::conditional<WK, F16WK, F16K>::type::BM,              \
   std::conditional<WK, F16WK, F16K>::type::BN, std::conditional<WK, F16WK, F16K>::type::BK,                           \
   std::conditional<WK, F16WK, F16K>::type::NT, std::conditional<WK, F16WK, F16K>::type::LDS_BYTES, true, false,       \
   &launch_f16k<WK>, false}

#define CASCMM_F8K64_VARIANT(NAME, BPRE, MT)                                                                                  \
  {NAME, KIND_F8K64, CASCMM_DT_F32, CASCMM_FMT_FP8, 3, false, F8Tile<MT>::T::BM, F8Tile<MT>::T::BN, F8Tile<MT>::T::BK, \
   F8Tile<MT>::T::NT, F8Tile<MT>::T::LDS_BYTES, true, false, &launch_f8k64<BPRE, MT>, BPRE}

#define CASCMM_WAVEK_VARIANT(NAME, NB)                                                                                \
  {NAME, KIND_WAVEK, CASCMM_DT_F32, CASCMM_FMT_BF16, 2, false, WaveK<NB>::BM, WaveK<NB>::BN, WaveK<NB>::BK, WaveK<NB>::NT, \
   WaveK<NB>::LDS_BYTES, true, true, &launch_wavek<NB>}

#define CASCMM_W512_VARIANT(NAME, BPRE)                                                                             \
  {NAME, KIND_W512, CASCMM_DT_F32, CASCMM_FMT_BF16, 2, false, W512::BM, W512::BN, 32, W512::NT, W512::LDS_BYTES, true, \
   false, &launch_w512<BPRE>, BPRE != 0, true}

// eight producer waves, every B column loaded singly (all producer threads share A and B evenly)
#define CASCMM_TILE_VARIANT_PS(NAME, BM, BN, BK, WM, WN, WK, DEPTH, NP, IODT, FMT, TERMS, FULL, FAST)          \
  {NAME, KIND_TILE, IODT, FMT, TERMS, FULL, BM, BN, BK, Tile<BM, BN, BK, WM, WN, WK, DEPTH, NP, false>::NT,  \
   LdsLayout<Tile<BM, BN, BK, WM, WN, WK, DEPTH, NP, false>, Lowp<FMT>::planes(TERMS)>::kBytes, FAST, true,  \
   &launch_tile<Tile<BM, BN, BK, WM, WN, WK, DEPTH, NP, false>, IODT, FMT, TERMS, FULL, FAST>}

// right operand already split: every B column staged singly, fp32 A, fast path only
#define CASCMM_TILE_VARIANT_BPRE(NAME, BM, BN, BK, WM, WN, WK, DEPTH, NP, FMT, TERMS, FULL)                           \
  {NAME, KIND_TILE, CASCMM_DT_F32, FMT, TERMS, FULL, BM, BN, BK, Tile<BM, BN, BK, WM, WN, WK, DEPTH, NP, false>::NT, \
   LdsLayout<Tile<BM, BN, BK, WM, WN, WK, DEPTH, NP, false>, Lowp<FMT>::planes(TERMS)>::kBytes, true, true,          \
   &launch_tile<Tile<BM, BN, BK, WM, WN, WK, DEPTH, NP, false>, CASCMM_DT_F32, FMT, TERMS, FULL, true, true>, true,    \
   ((BN) / (WN)) % 64 == 0}

// fp16 (bf16) operands in memory multiplied as one fp16 (bf16) term, right operand prepared: the
// producers only copy
#define CASCMM_TILE_VARIANT_BPRE16(NAME, BM, BN, BK, WM, WN, WK, DEPTH, NP, IODT, FMT)                       \
  {NAME, KIND_TILE, IODT, FMT, 1, false, BM, BN, BK, Tile<BM, BN, BK, WM, WN, WK, DEPTH, NP, false>::NT,     \
   LdsLayout<Tile<BM, BN, BK, WM, WN, WK, DEPTH, NP, false>, 1>::kBytes, true, true,                         \
   &launch_tile<Tile<BM, BN, BK, WM, WN, WK, DEPTH, NP, false>, IODT, FMT, 1, false, true, true>, true,      \
   ((BN) / (WN)) % 64 == 0}

// B-direct kernels: fp32 operands, fast path only
#define CASCMM_BD_VARIANT(NAME, BM, WN, BK, DEPTH, NP, FMT, TERMS, FULL)                                \
  {NAME, KIND_TILE, CASCMM_DT_F32, FMT, TERMS, FULL, BM, 32 * WN, BK, TileBD<BM, WN, BK, DEPTH, NP>::NT, \
   LdsLayoutA<TileBD<BM, WN, BK, DEPTH, NP>, TERMS>::kBytes, true, false,                               \
   &launch_bdirect<TileBD<BM, WN, BK, DEPTH, NP>, FMT, TERMS, FULL, false>}

// skinny split-K kernels (one row tile): B-direct + partials + reduction
#define CASCMM_SKINNY_VARIANT(NAME, BM, WN, BK, DEPTH, NP, FMT, TERMS, FULL)                            \
  {NAME, KIND_SPLITK, CASCMM_DT_F32, FMT, TERMS, FULL, BM, 32 * WN, BK, TileBD<BM, WN, BK, DEPTH, NP>::NT, \
   LdsLayoutA<TileBD<BM, WN, BK, DEPTH, NP>, TERMS>::kBytes, true, false,                               \
   &launch_bdirect<TileBD<BM, WN, BK, DEPTH, NP>, FMT, TERMS, FULL, true>}

// the kernels with K split over the waves of a workgroup and the chained feed-forward path
// (cascmm_slotk_kernel.h, cascmm_inst_chain.hip)
struct SlotK {
  static constexpr int BM = 64, BN = 160, BK = 16, NW = 4, NT = 256, D = 4, GROUP_M = 8;
  static constexpr int MT = 2, NTL = 5, BLOCKS = MT * NTL;
  static constexpr int BLOCK_BYTES = 16 * 64 * 4;                  // one wave's 32 x 32 partial block
  static constexpr int RED_BYTES = BLOCKS * 3 * BLOCK_BYTES;       // 120 KB: every block from its three non-owners
  static constexpr int RA = 8, A_STAGE = BM * BK * 4;              // raw A: ring of 8 stages of 4 KB per wave
  static constexpr int RING = RA * A_STAGE;
  static constexpr int LDS_BYTES = NW * RING > RED_BYTES ? NW * RING : RED_BYTES;   // 128 KB
};

struct SlotKParams {
  const void* a;         // ARAW = 0: slots [2][K/8][M] x 16 bytes; ARAW = 1: fp32 [M][lda]
  const void* b_slots;   // [2][K/8][N] x 16 bytes
  float* C;
  const float* bias;
  int M, N, K;
  int64_t lda, ldb, ldc;   // ldb: cascmm_rawk_kernel only (raw B)
  int tiles_m, tiles_n;
  int group_m;             // tile rows an XCD's range of tiles walks down before moving one tile to the right
};

int launch_slotk(const SlotKParams& q, int araw, hipStream_t stream);
int launch_prepare_left(const float* A, int M, int K, int64_t lda, void* out, hipStream_t stream);
const void* slotk_kernel_handle(int araw);

// each instantiation unit exports its slice of the table
const VariantDesc* variants_bf16(int* n);
const VariantDesc* variants_fp16(int* n);
const VariantDesc* variants_fp8(int* n);
const VariantDesc* variants_io16(int* n);
const VariantDesc* variants_bpre(int* n);
const VariantDesc* variants_chain(int* n);

}  // namespace cascmm
