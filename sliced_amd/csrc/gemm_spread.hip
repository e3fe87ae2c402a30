// The spread tail of the tiled f32 GEMM: a launch whose tile count is not a multiple of the
// chip's workgroup slots would leave most CUs idle during its last round.  Here the whole rounds
// run as whole tiles, and the k tiles of the remaining tiles - taken as one long sequence - are
// dealt out evenly to one more round of workgroups in the same launch (they start as the
// whole-tile workgroups retire).  Such a workgroup writes raw partial tiles to the context
// workspace; a second kernel sums them per tile in ascending k order, so the result does not
// depend on timing, and applies beta / bias / relu.
#include "gemm_tile.hpp"

namespace slhip {

// A workgroup of the spread tail: up to two runs of k tiles, each inside one tile of C, each
// written as a raw partial tile (row-major, the tile's own size) to workspace slot 2*w + run.
template <bool TA, bool TB, int BK, bool ONLY_FAST, int WM, int WN, int WGM = 2, int WGN = 2>
__device__ __forceinline__ void gemm_spread_worker(const GemmArgs& g, const SpreadArgs& sp,
                                                   float (*lds_a)[Cfg<BK, 32 * WM * WGM>::STAGE_FLOATS],
                                                   float (*lds_b)[Cfg<BK, 32 * WN * WGN>::STAGE_FLOATS]) {
  constexpr int TM = 32 * WM * WGM, TN = 32 * WN * WGN;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = wave / WGN, wn = wave % WGN;
  const int r = lane & 31, h = lane >> 5;
  const unsigned w = blockIdx.x - sp.first;
  unsigned u = w * sp.units;
  const unsigned u_end = u + sp.units < sp.total ? u + sp.units : sp.total;
  for (int run = 0; run < 2 && u < u_end; ++run) {
    const unsigned ti = u / sp.kt_total;
    const int ka = (int)(u % sp.kt_total);
    const int kb = (u_end - u) < (sp.kt_total - (unsigned)ka) ? ka + (int)(u_end - u) : (int)sp.kt_total;
    u += (unsigned)(kb - ka);
    unsigned tm, tn;
    tile_of_block(sp.first + ti, g.tiles_m, g.tiles_n, tm, tn);
    const size_t m0 = (size_t)tm * TM, n0 = (size_t)tn * TN;

    floatx16 acc[WM][WN];
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    gemm_k_range<TA, TB, BK, ONLY_FAST, WM, WN, WGM, WGN>(g, ka, kb, 0, g.K, m0, n0, lds_a, lds_b, acc);

    float* slot = g.partial + ((size_t)2 * w + run) * (TM * TN);
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v)
          slot[(block_of<WGM>(wm, i) + 8 * (v / 4) + 4 * h + (v % 4)) * TN + block_of<WGN>(wn, j) + r] = acc[i][j][v];
  }
}

template <bool TA, bool TB, int BK, bool ONLY_FAST, int WM, int WN>
__global__ __launch_bounds__(256, 2) void gemm_spread_kernel(GemmArgs g, SpreadArgs sp) {
  __shared__ __attribute__((aligned(16))) float lds_a[2][Cfg<BK, 64 * WM>::STAGE_FLOATS];
  __shared__ __attribute__((aligned(16))) float lds_b[2][Cfg<BK, 64 * WN>::STAGE_FLOATS];
  if (blockIdx.x >= sp.first) gemm_spread_worker<TA, TB, BK, ONLY_FAST, WM, WN>(g, sp, lds_a, lds_b);
  else gemm_whole_tile<TA, TB, BK, ONLY_FAST, WM, WN>(g, lds_a, lds_b);
}

// The same on eight waves (the 128 x 128 tile as 2 x 4 waves of 64 x 32 each, as gemm_wide_kernel): two
// such workgroups put four waves on a SIMD.
template <bool TA, bool TB, int BK, bool ONLY_FAST>
__global__ __launch_bounds__(512, 2) void gemm_spread_wide_kernel(GemmArgs g, SpreadArgs sp) {
  __shared__ __attribute__((aligned(16))) float lds_a[2][Cfg<BK, 128>::STAGE_FLOATS];
  __shared__ __attribute__((aligned(16))) float lds_b[2][Cfg<BK, 128>::STAGE_FLOATS];
  if (blockIdx.x >= sp.first) gemm_spread_worker<TA, TB, BK, ONLY_FAST, 2, 1, 2, 4>(g, sp, lds_a, lds_b);
  else gemm_whole_tile<TA, TB, BK, ONLY_FAST, 2, 1, 2, 4>(g, lds_a, lds_b);
}

// The tiles of a spread tail: C tile = sum of its partial tiles in ascending k order (workgroup
// order), then beta / bias / relu as in the kernel's own epilogue.  One float4 of the tile per
// thread (sixteen workgroups per 128 x 128 tile, four per 64 x 64 tile) - a tile of a long-K product can have hundreds of
// partial tiles (64 x 64 x 1048576: one tile, 512 partials; four workgroups summing them one after
// the other took 650 us of that product's 930).  Workgroup spread_first + w holds k tiles
// [w*U, (w+1)*U) of the tail's sequence, so tile ti is covered by workgroups (ti*KT)/U ..
// ((ti+1)*KT - 1)/U.  Only the first of them can have started in the tile before (U <= KT): its
// partial of this tile is its run ti - (w*U)/KT; every later one's is its run 0.
template <int TM, int TN>
__global__ __launch_bounds__(256) void spread_fixup_kernel(GemmArgs g, SpreadArgs sp) {
  constexpr int PARTS = TM * TN / 4 / 256;  // workgroups per tile
  constexpr int SLOT = TM * TN;
  const unsigned ti = blockIdx.x / PARTS, part = blockIdx.x % PARTS;
  unsigned tm, tn;
  tile_of_block(sp.first + ti, g.tiles_m, g.tiles_n, tm, tn);
  const size_t m0 = (size_t)tm * TM, n0 = (size_t)tn * TN;
  const unsigned KT = sp.kt_total, U = sp.units;
  const unsigned w_first = (ti * KT) / U, w_last = ((ti + 1) * KT - 1) / U;
  constexpr int PER = 1;  // float4 per thread
  float4 s[PER], c[PER], mk[PER];
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const int f = threadIdx.x + 256 * (int)part;
    const int row_l = f / (TN / 4), c4 = f % (TN / 4);
    const float* p0 = g.partial + row_l * TN + 4 * c4;
    float4 sum = ld4(p0 + ((size_t)2 * w_first + (ti - (w_first * U) / KT)) * SLOT);
    auto add = [&](const float4& p) { sum.x += p.x; sum.y += p.y; sum.z += p.z; sum.w += p.w; };
    unsigned w = w_first + 1;
    for (; w + 3 <= w_last; w += 4) {  // four loads in flight, added in ascending order
      const float4 q0 = ld4(p0 + (size_t)2 * w * SLOT), q1 = ld4(p0 + (size_t)2 * (w + 1) * SLOT),
                   q2 = ld4(p0 + (size_t)2 * (w + 2) * SLOT), q3 = ld4(p0 + (size_t)2 * (w + 3) * SLOT);
      add(q0); add(q1); add(q2); add(q3);
    }
    for (; w <= w_last; ++w) add(ld4(p0 + (size_t)2 * w * SLOT));
    s[e] = sum;
    const size_t row = m0 + row_l, col = n0 + 4 * c4;
    c[e] = make_float4(0.f, 0.f, 0.f, 0.f);
    mk[e] = c[e];
    auto read4 = [&](const float* base) {  // a float4 of a row of C's shape, clipped at the row's end
      const float* cp = base + row * g.N + col;
      if (col + 3 < g.N) return ld4g(cp);
      return make_float4(col < g.N ? cp[0] : 0.f, col + 1 < g.N ? cp[1] : 0.f, col + 2 < g.N ? cp[2] : 0.f, 0.f);
    };
    if (row < g.M) {  // every read of C and of the mask source before the first store
      if (g.beta != 0.0f) c[e] = read4(g.C);
      if (g.mask) mk[e] = read4(g.mask);
    }
  }
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const int f = threadIdx.x + 256 * (int)part;
    const int row_l = f / (TN / 4), c4 = f % (TN / 4);
    const size_t row = m0 + row_l, col = n0 + 4 * c4;
    if (row >= g.M || col >= g.N) continue;
    float v[4] = {s[e].x, s[e].y, s[e].z, s[e].w};
    const float cv[4] = {c[e].x, c[e].y, c[e].z, c[e].w};
    const float mv[4] = {mk[e].x, mk[e].y, mk[e].z, mk[e].w};
    const int n_in = col + 3 < g.N ? 4 : (int)(g.N - col);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (g.mask) v[q] = (mv[q] >= 0.0f ? 1.0f : 0.0f) * v[q];
      if (g.beta != 0.0f) v[q] = g.beta * cv[q] + v[q];
      if (g.bias) v[q] = v[q] + (q < n_in ? g.bias[col + q] : 0.0f);
    }
    const size_t idx = row * g.N + col;
    if (n_in == 4) {
      if (g.pre_act) st4g(g.pre_act + idx, make_float4(v[0], v[1], v[2], v[3]));
      if (g.relu) {
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] = (v[q] >= 0.0f ? 1.0f : 0.0f) * v[q];
      }
      st4g(g.C + idx, make_float4(v[0], v[1], v[2], v[3]));
    } else {
#pragma unroll
      for (int q = 0; q < 3; ++q) {
        if (q < n_in) {
          if (g.pre_act) g.pre_act[idx + q] = v[q];
          g.C[idx + q] = g.relu ? (v[q] >= 0.0f ? 1.0f : 0.0f) * v[q] : v[q];
        }
      }
    }
  }
}

int32_t gemm_spread_launch(slhip_ctx* ctx, bool ta, bool tb, bool only_fast, bool small_tile, const GemmArgs& g,
                           const SpreadArgs& sp, size_t workers, size_t tail_tiles, bool wide) {
  const dim3 grid((unsigned)(sp.first + workers));
  if (wide && !small_tile && !(ta && tb)) {
#define SL_WIDE(TA_, TB_)                                                                                                     \
  do {                                                                                                                        \
    if (only_fast)                                                                                                            \
      hipLaunchKernelGGL((gemm_spread_wide_kernel<TA_, TB_, GEMM_BK, true>), grid, dim3(512), 0, ctx->stream, g, sp);         \
    else                                                                                                                      \
      hipLaunchKernelGGL((gemm_spread_wide_kernel<TA_, TB_, GEMM_BK, false>), grid, dim3(512), 0, ctx->stream, g, sp);        \
  } while (0)
    if (!ta && !tb) SL_WIDE(false, false);
    else if (!ta && tb) SL_WIDE(false, true);
    else SL_WIDE(true, false);
#undef SL_WIDE
    ctx->last_gemm.waves = 8;
    int32_t rcw = post_launch();
    if (rcw) return rcw;
    hipLaunchKernelGGL((spread_fixup_kernel<128, 128>), dim3((unsigned)(16 * tail_tiles)), dim3(256), 0, ctx->stream, g, sp);
    return post_launch();
  }
#define SL_GEMM3(TA_, TB_, WM_, WN_)                                                                                          \
  do {                                                                                                                        \
    if (only_fast)                                                                                                            \
      hipLaunchKernelGGL((gemm_spread_kernel<TA_, TB_, GEMM_BK, true, WM_, WN_>), grid, dim3(256), 0, ctx->stream, g, sp);    \
    else                                                                                                                      \
      hipLaunchKernelGGL((gemm_spread_kernel<TA_, TB_, GEMM_BK, false, WM_, WN_>), grid, dim3(256), 0, ctx->stream, g, sp);   \
  } while (0)
#define SL_GEMM(TA_, TB_)                      \
  do {                                         \
    if (small_tile) SL_GEMM3(TA_, TB_, 1, 1);  \
    else SL_GEMM3(TA_, TB_, 2, 2);             \
  } while (0)
  if (!ta && !tb) SL_GEMM(false, false);
  else if (!ta && tb) SL_GEMM(false, true);
  else if (ta && !tb) SL_GEMM(true, false);
  else SL_GEMM3(true, true, 2, 2);
#undef SL_GEMM
#undef SL_GEMM3
  int32_t rc = post_launch();
  if (rc) return rc;
  if (small_tile) hipLaunchKernelGGL((spread_fixup_kernel<64, 64>), dim3((unsigned)(4 * tail_tiles)), dim3(256), 0, ctx->stream, g, sp);
  else hipLaunchKernelGGL((spread_fixup_kernel<128, 128>), dim3((unsigned)(16 * tail_tiles)), dim3(256), 0, ctx->stream, g, sp);
  return post_launch();
}

}  // namespace slhip
