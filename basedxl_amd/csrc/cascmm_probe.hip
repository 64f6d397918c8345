// Measurement hooks: what this GPU sustains on the two resources the roofline of the cascade prices
// against -- the bf16 MFMA pipes (a loop that touches registers only) and HBM (a streaming read, a
// copy).  The published peaks assume the boost clock; these kernels show what the board holds.
#include "cascmm_common.h"

namespace cascmm {

// Every wave issues `iters` rounds of four independent 32x32x16 bf16 MFMAs (operands that differ per
// lane, fixed over the loop) and leaves one value per lane so that nothing is optimised away.
__global__ __launch_bounds__(256) void probe_mfma_kernel(int iters, float* out) {
  const int lane = threadIdx.x & 63;
  u32x4 a, b;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    // bf16 pairs with varied mantissas, magnitudes near 1
    a[e] = 0x3F803F80u + 0x00010003u * (unsigned)(lane * 7 + e * 13 + 1);
    b[e] = 0x3F803F80u + 0x00030001u * (unsigned)(lane * 5 + e * 11 + 2);
  }
  typedef Lowp<CASCMM_FMT_BF16> L;
  f32x16 c0, c1, c2, c3;
#pragma unroll
  for (int e = 0; e < 16; ++e) c0[e] = c1[e] = c2[e] = c3[e] = 0.f;
  for (int i = 0; i < iters; ++i) {
    c0 = L::mfma(L::operand(a, 0), L::operand(b, 0), c0);
    c1 = L::mfma(L::operand(a, 0), L::operand(b, 0), c1);
    c2 = L::mfma(L::operand(a, 0), L::operand(b, 0), c2);
    c3 = L::mfma(L::operand(a, 0), L::operand(b, 0), c3);
  }
  out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = c0[0] + c1[5] + c2[10] + c3[15];
}

// Grid-stride pass over `n16` 16-byte pieces: read them all (COPY = 0: one partial sum per thread is
// written at the end) or copy them to dst (COPY = 1).
template <int COPY>
__global__ __launch_bounds__(256) void probe_stream_kernel(const f32x4* src, f32x4* dst, size_t n16, float* sums) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) {
    const f32x4 v = __builtin_nontemporal_load(src + i);
    if (COPY) __builtin_nontemporal_store(v, dst + i);
    else acc += v;
  }
  if (!COPY) sums[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = acc[0] + acc[1] + acc[2] + acc[3];
}

}  // namespace cascmm

using namespace cascmm;

extern "C" {

int cascmm_probe_mfma(int workgroups, int iters, float* out, size_t out_bytes, void* stream) {
  if (workgroups < 1 || workgroups > 65536 || iters < 0) return CASCMM_ERR_BAD_SHAPE;
  if (!out) return CASCMM_ERR_NULL_POINTER;
  if (out_bytes < (size_t)workgroups * 256 * sizeof(float)) return CASCMM_ERR_WORKSPACE;
  if (launch_kernel(probe_mfma_kernel, dim3((unsigned)workgroups), dim3(256), 0, (hipStream_t)stream, iters, out) != hipSuccess)
    return CASCMM_ERR_LAUNCH;
  return CASCMM_OK;
}

int cascmm_probe_stream(const void* src, void* dst, size_t bytes, int workgroups, float* sums, size_t sums_bytes,
                        void* stream) {
  if (workgroups < 1 || workgroups > 65536 || bytes % 16 != 0) return CASCMM_ERR_BAD_SHAPE;
  if (!src || (!dst && !sums)) return CASCMM_ERR_NULL_POINTER;
  if ((uintptr_t)src % 16 != 0 || (uintptr_t)dst % 16 != 0) return CASCMM_ERR_ALIGNMENT;
  if (!dst && sums_bytes < (size_t)workgroups * 256 * sizeof(float)) return CASCMM_ERR_WORKSPACE;
  hipError_t e;
  if (dst)
    e = launch_kernel(probe_stream_kernel<1>, dim3((unsigned)workgroups), dim3(256), 0, (hipStream_t)stream, (const f32x4*)src,
                      (f32x4*)dst, bytes / 16, (float*)nullptr);
  else
    e = launch_kernel(probe_stream_kernel<0>, dim3((unsigned)workgroups), dim3(256), 0, (hipStream_t)stream, (const f32x4*)src,
                      (f32x4*)nullptr, bytes / 16, sums);
  return e == hipSuccess ? CASCMM_OK : CASCMM_ERR_LAUNCH;
}

}  // extern "C"
