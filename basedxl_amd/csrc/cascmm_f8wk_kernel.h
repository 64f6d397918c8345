// Three-term fp8 cascade on the fp8-rate MFMA with K split over the waves of a workgroup (gfx950): the
// fp8 counterpart of cascmm_slotk_kernel<0> for problems with about one 64 x 160 tile per CU (the
// 1280- and 640-channel projections, the feed-forward down-projections), which on the LDS-tiled fp8-rate
// kernel leave CUs idle or need their K split over workgroups and a second kernel.
//
// Both operands come as the k16 operand slots of cascmm_f8k64_kernel.h ([term][K/16][rows] x 16 bytes,
// written by its split kernels or by cascmm_prepare_weight).  A lane's MFMA operand (32 consecutive k of
// its row or column) is two slots: two 16-byte loads, 32 lanes reading 512 contiguous bytes, straight into
// registers; no LDS and no VALU work in the loop.  One workgroup computes a 64 x 160 tile; wave w owns the
// whole tile (ten accumulator blocks) over the 64-k stages w, w + 4, ...  A stage is 42 loads and 60 MFMAs
// (3840 cycles): the slots of a column block are loaded for the next stage as soon as the block's MFMAs of
// this stage are over, those of the left operand into a second register set, so every load has one stage
// to arrive and the six-bit load counter is never the limit.  At the end the four partial tiles meet in
// LDS and are added in wave order, as in cascmm_slotk_kernel.
#pragma once
#include <type_traits>

#include "cascmm_f8k64_kernel.h"

namespace cascmm {

struct F8WK {
  static constexpr int BM = 64, BN = 160, BK = 64, NW = 4, NT = 256, TERMS = 3, GROUP_M = 8;
  static constexpr int MT = 2, NTL = 5, BLOCKS = MT * NTL;
  static constexpr int BLOCK_BYTES = 16 * 64 * 4;                  // one wave's 32 x 32 partial block
  static constexpr int LDS_BYTES = BLOCKS * 3 * BLOCK_BYTES;       // 120 KB: every block from its three non-owners
};

// Host-checked: K % 64 == 0, K >= 64, the slot buffers 16-byte aligned and below 2 GiB, C rows addressable
// with 32-bit byte offsets inside a tile.  p.k_splits is not used (one launch, no partial results).
// (A template, like the other kernels of this header family, so that every translation unit that includes the
// header may hold the definition.)
template <int UNUSED>
__global__ __launch_bounds__(F8WK::NT) __attribute__((amdgpu_waves_per_eu(1, 1))) void cascmm_f8wk_kernel(const F8K64Params p) {
  typedef F8WK T;
  extern __shared__ __attribute__((aligned(1024))) unsigned char f8wk_smem[];
  const int tid = threadIdx.x, lane = tid & 63, l31 = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // tile order as in cascmm_slotk_kernel: one contiguous range of tile ids per XCD, GROUP_M tile rows down
  // before one tile to the right
  int tm, tn;
  tile_coords((int)blockIdx.x, p.tiles_m, p.tiles_n, tm, tn, T::GROUP_M);
  const int m0 = tm * T::BM, n0 = tn * T::BN;
  const int kus = p.K >> 4;          // 16-k slot columns
  const int ksteps = p.K >> 6;       // 64-k stages
  const int n_own = (ksteps - wave + T::NW - 1) / T::NW;   // 0 for the last waves of a very short K: they add zeros

  // lane (l31, h) reads slot columns 2 h and 2 h + 1 of a stage's four; a stage past the wave's last one is
  // loaded from beyond the end of the buffers, which returns zeros (the loop has no branch inside a trip)
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
  i32x8 b4[2][T::TERMS];            // column block 4, by stage parity (its refill would otherwise have four blocks to arrive, not five)
  auto a_base = [&](int i) { return i < n_own ? (wave + T::NW * i) * 4 * a_ku : a_end; };
  auto b_base = [&](int i) { return i < n_own ? (wave + T::NW * i) * 4 * b_ku : b_end; };
  auto issue_a = [&](int i, int buf, int t, int mi) { a[buf][t][mi] = load2(ra, va + mi * 512, a_base(i) + t * a_plane, a_ku); };
  auto issue_b = [&](int i, int t, int ni) { b[t][ni] = load2(rb, vb + ni * 512, b_base(i) + t * b_plane, b_ku); };
  auto issue_b4 = [&](int i, int buf, int t) { b4[buf][t] = load2(rb, vb + 4 * 512, b_base(i) + t * b_plane, b_ku); };

  // ---- prologue: everything of stage 0 ----
#pragma unroll
  for (int t = 0; t < T::TERMS; ++t) {
#pragma unroll
    for (int mi = 0; mi < T::MT; ++mi) issue_a(0, 0, t, mi);
#pragma unroll
    for (int ni = 0; ni < T::NTL - 1; ++ni) issue_b(0, t, ni);
    issue_b4(0, 0, t);
  }
  f32x16 acc[T::MT][T::NTL];
#pragma unroll
  for (int mi = 0; mi < T::MT; ++mi)
#pragma unroll
    for (int ni = 0; ni < T::NTL; ++ni)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[mi][ni][e] = 0.f;

  const int scales = 0x00777B7F;   // E8M0 bytes 2^0, 2^-4, 2^-8: op_sel picks the term's
  // Stage i, register set u = i % 2 of the left operand.  Behind the MFMAs of column block ni: the slots of
  // block ni - 1 for stage i + 1 (ni = 0: block 4, into the other set) and, ni < 3, a third of the left operand's.
  for (int i0 = 0; i0 < n_own; i0 += 2) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int i = i0 + u;
#pragma unroll
      for (int ni = 0; ni < T::NTL; ++ni) {
        // (the term numbers are the instruction's op_sel fields: literals); smallest products first
#define F8WK_PRODUCT(I, J)                                                                                            \
  _Pragma("unroll") for (int mi = 0; mi < T::MT; ++mi) acc[mi][ni] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4( \
      a[u][I][mi], bop(J), acc[mi][ni], 0, 0, I, scales, J, scales);
        auto bop = [&](int t) { return ni < T::NTL - 1 ? b[t][ni < T::NTL - 1 ? ni : 0] : b4[u][t]; };
        F8WK_PRODUCT(0, 2)
        F8WK_PRODUCT(1, 1)
        F8WK_PRODUCT(2, 0)
        F8WK_PRODUCT(0, 1)
        F8WK_PRODUCT(1, 0)
        F8WK_PRODUCT(0, 0)
#undef F8WK_PRODUCT
#pragma unroll
        for (int t = 0; t < T::TERMS; ++t) {
          if (ni == 0) issue_b4(i + 1, u ^ 1, t);
          else issue_b(i + 1, t, ni - 1);
        }
        if (ni < 3) {
          // the six (term, row block) slot pairs of the left operand over the first three blocks
#pragma unroll
          for (int x = 2 * ni; x < 2 * ni + 2; ++x) issue_a(i + 1, u ^ 1, x >> 1, x & 1);
        }
        // loads of this block: 10, 10, 10, 6, 6 -- one behind each of the first MFMAs
        constexpr int kLoads[5] = {10, 10, 10, 6, 6};
#pragma unroll
        for (int x = 0; x < 12; ++x) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if (x < kLoads[ni]) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // ---- the four partial tiles meet in LDS: block b = mi * 5 + ni is owned by wave b % 4; a non-owner w puts
  // its partial block at [b][(w - owner - 1) mod 4], 16 bytes per lane and register quad ----
  float out_scale = 1.f;
  if (p.tensor_exps) out_scale = __builtin_ldexpf(1.f, -(p.tensor_exps[0] + p.tensor_exps[1]));
  auto reduce_and_store = [&](auto owner_tag) {
    constexpr int W = decltype(owner_tag)::value;
#pragma unroll
    for (int bk = 0; bk < T::BLOCKS; ++bk) {
      if (bk % T::NW == W) continue;
      const int slot = ((W - bk % T::NW - 1) & 3);
      unsigned char* dst = f8wk_smem + (bk * 3 + slot) * T::BLOCK_BYTES + lane * 16;
      const f32x16& v = acc[bk / T::NTL][bk % T::NTL];
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) *(f32x4*)(dst + r4 * 1024) = (f32x4){v[4 * r4], v[4 * r4 + 1], v[4 * r4 + 2], v[4 * r4 + 3]};
    }
    __syncthreads();
    const int ldc_bytes = (int)p.ldc * 4;
    // rows past M fall beyond the end of the buffer and are dropped
    const int64_t c_bytes = ((int64_t)(p.M - 1 - m0) * p.ldc + (p.N - n0)) * 4;
    const i32x4 rc = make_rsrc(p.C + (int64_t)m0 * p.ldc + n0, c_bytes);
#pragma unroll
    for (int bk = W; bk < T::BLOCKS; bk += T::NW) {
      const int mi = bk / T::NTL, ni = bk % T::NTL;
      if (n0 + ni * 32 >= p.N) continue;
      f32x16 sum;
      // partial sums in wave order 0, 1, 2, 3: the own one at its place
#pragma unroll
      for (int w = 0; w < T::NW; ++w) {
        f32x16 part;
        if (w == W) {
          part = acc[mi][ni];
        } else {
          const unsigned char* src = f8wk_smem + (bk * 3 + ((w - W - 1) & 3)) * T::BLOCK_BYTES + lane * 16;
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
