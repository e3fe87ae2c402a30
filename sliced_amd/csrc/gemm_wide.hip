// The 128 x 128 tile on EIGHT waves (2 x 4, each 64 x 32 = two 32 x 32 accumulators) instead of
// four.  Same staging, same k loop, same LDS footprint as the four-wave kernel (gemm.hip); what
// changes is who shares a SIMD: a tile grid that gives every CU one workgroup leaves the four-wave
// kernel with ONE wave per SIMD, whose LDS reads, stores and barriers then stall the matrix core
// with nobody to fill in; here two waves of the same workgroup take turns (2048^3: 110 -> 117
// TFLOP/s for A*B, 117 -> 124 for A*Bt; with two workgroups to a CU it is 6-10 % slower than the
// four-wave kernel, so it only takes grids of at most one workgroup per CU).  A third LDS stage,
// which lets the fragment reads run on across the k-tile barrier, measured the same.  A translation unit
// of its own, like the spread-tail kernel: the four-wave kernel's speed moves with the code around it.
#include "gemm_tile.hpp"

namespace slhip {

template <bool TA, bool TB, bool ONLY_FAST>
__global__ __launch_bounds__(512) void gemm_wide_kernel(GemmArgs g) {
  __shared__ __attribute__((aligned(16))) float lds_a[2][Cfg<GEMM_BK, 128>::STAGE_FLOATS];
  __shared__ __attribute__((aligned(16))) float lds_b[2][Cfg<GEMM_BK, 128>::STAGE_FLOATS];
  gemm_whole_tile<TA, TB, GEMM_BK, ONLY_FAST, 2, 1, 2, 4>(g, lds_a, lds_b);
}

// g is planned for 128 x 128 tiles (tiles_m, tiles_n, splits, k_chunk); the doubly transposed form
// is not instantiated (returns SLHIP_EINVAL: the caller does not choose this kernel for it).
int32_t gemm_wide_launch(slhip_ctx* ctx, bool ta, bool tb, bool only_fast, const GemmArgs& g) {
  if (ta && tb) return SLHIP_EINVAL;
  const dim3 grid(g.tiles_m * g.tiles_n, g.splits);
#define SL_WIDE(TA_, TB_)                                                                                   \
  do {                                                                                                      \
    if (only_fast) hipLaunchKernelGGL((gemm_wide_kernel<TA_, TB_, true>), grid, dim3(512), 0, ctx->stream, g); \
    else hipLaunchKernelGGL((gemm_wide_kernel<TA_, TB_, false>), grid, dim3(512), 0, ctx->stream, g);        \
  } while (0)
  if (!ta && !tb) SL_WIDE(false, false);
  else if (!ta && tb) SL_WIDE(false, true);
  else SL_WIDE(true, false);
#undef SL_WIDE
  return post_launch();
}

}  // namespace slhip
