// The 128 x 128 tile on EIGHT waves (2 x 4, each 64 x 32 = two 32 x 32 accumulators) instead of
// four.  Same staging, same k loop, same LDS footprint as the four-wave kernel (gemm.hip); what
// changes is who shares a SIMD.  With 124 vector registers a wave, two such workgroups fit a CU and
// put FOUR waves on every SIMD where the four-wave kernel has two: while one wave reads fragments,
// stores a stage or waits at the k-tile barrier, three others can issue to the matrix core
// (4096^3 per launch: 142.2 -> 146.3 TFLOP/s, MFMA-busy share 0.93 -> 0.96; 8192^3 144.0 -> 150.4, 0.98;
// 8192 x 2048 x 784 128.9 -> 133.1).  A grid that gives every CU ONE workgroup leaves the four-wave
// kernel with one wave per SIMD and this one with two (2048^3: 118 -> 133), and a last round that is
// at most half full runs in 0.525 of a full round's time.  It is the kernel of every whole-tile
// launch of the 128 x 128 tile (the spread tail and the bit-mask kernels have their own eight-wave
// forms); the four-wave kernel stays for the doubly transposed form and behind the tile policy.
// Where the loop starts relative to a 32-byte boundary and where in the k tile the refill sits
// measured within 0.5 % of each other on this kernel; a third LDS stage measured the same.
// A translation unit of its own, like the spread-tail kernel: the four-wave kernel's speed moves
// with the code around it.
#include "gemm_tile.hpp"

namespace slhip {

template <bool TA, bool TB, bool ONLY_FAST>
__global__ __launch_bounds__(512, 2) void gemm_wide_kernel(GemmArgs g) {  // two workgroups to a CU: at most 128 VGPRs
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

// The 64 x 64 tile on eight waves: two sets of 2 x 2 waves that split every k tile between them and add
// their accumulators through LDS at the end.  For grids that give a CU one workgroup of the small tile
// (1024^3: 256 tiles), where the four-wave form leaves each SIMD a single wave.
template <bool TA, bool TB, bool ONLY_FAST>
__global__ __launch_bounds__(512) void gemm_small8_kernel(GemmArgs g) {
  __shared__ __attribute__((aligned(16))) float lds_a[2][Cfg<GEMM_BK, 64>::STAGE_FLOATS];
  __shared__ __attribute__((aligned(16))) float lds_b[2][Cfg<GEMM_BK, 64>::STAGE_FLOATS];
  gemm_whole_tile<TA, TB, GEMM_BK, ONLY_FAST, 1, 1, 2, 2, 2>(g, lds_a, lds_b);
}

int32_t gemm_small8_launch(slhip_ctx* ctx, bool ta, bool tb, bool only_fast, const GemmArgs& g) {
  if ((ta && tb) || g.splits != 1) return SLHIP_EINVAL;
  const dim3 grid(g.tiles_m * g.tiles_n, 1);
#define SL_S8(TA_, TB_)                                                                                       \
  do {                                                                                                        \
    if (only_fast) hipLaunchKernelGGL((gemm_small8_kernel<TA_, TB_, true>), grid, dim3(512), 0, ctx->stream, g); \
    else hipLaunchKernelGGL((gemm_small8_kernel<TA_, TB_, false>), grid, dim3(512), 0, ctx->stream, g);        \
  } while (0)
  if (!ta && !tb) SL_S8(false, false);
  else if (!ta && tb) SL_S8(false, true);
  else SL_S8(true, false);
#undef SL_S8
  return post_launch();
}

// The 128 x 128 tile on SIXTEEN waves, two sets of 2 x 4 that split every k tile: one such workgroup puts four
// waves on every SIMD, as two eight-wave workgroups do.  For grids of more than half a round and at most one
// tile per CU (2048^3, 2048 x 2048 x 8192), where the eight-wave kernel leaves a SIMD two waves - or needs a
// k split into two workgroups per tile and a combine launch to get four.
template <bool TA, bool TB, bool ONLY_FAST>
__global__ __launch_bounds__(1024) void gemm_wide16_kernel(GemmArgs g) {
  __shared__ __attribute__((aligned(16))) float lds_a[2][Cfg<GEMM_BK, 128>::STAGE_FLOATS];
  __shared__ __attribute__((aligned(16))) float lds_b[2][Cfg<GEMM_BK, 128>::STAGE_FLOATS];
  gemm_whole_tile<TA, TB, GEMM_BK, ONLY_FAST, 2, 1, 2, 4, 2>(g, lds_a, lds_b);
}

int32_t gemm_wide16_launch(slhip_ctx* ctx, bool ta, bool tb, bool only_fast, const GemmArgs& g) {
  if ((ta && tb) || g.splits != 1) return SLHIP_EINVAL;
  const dim3 grid(g.tiles_m * g.tiles_n, 1);
#define SL_W16(TA_, TB_)                                                                                       \
  do {                                                                                                         \
    if (only_fast) hipLaunchKernelGGL((gemm_wide16_kernel<TA_, TB_, true>), grid, dim3(1024), 0, ctx->stream, g); \
    else hipLaunchKernelGGL((gemm_wide16_kernel<TA_, TB_, false>), grid, dim3(1024), 0, ctx->stream, g);        \
  } while (0)
  if (!ta && !tb) SL_W16(false, false);
  else if (!ta && tb) SL_W16(false, true);
  else SL_W16(true, false);
#undef SL_W16
  return post_launch();
}

}  // namespace slhip
