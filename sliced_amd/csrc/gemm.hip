// f32 GEMM for gfx950 on the fp32 matrix cores: C[m×n] = op(A)·op(B) (+ beta·C) (+ bias, relu).
//
// One kernel template serves A·B, A·Bᵀ and Aᵀ·B without ever materialising a transpose: an
// operand whose k index is contiguous in memory is staged in LDS as [x][k] and its MFMA
// fragments are read with one 128-bit LDS load per 4 k-steps; an operand whose m/n index is
// contiguous is staged as [k][x] and read with 32-bit loads.  Because a dot product does not
// care in which order k is visited, both layouts feed v_mfma_f32_32x32x2_f32 with the same
// k permutation inside every group of 8: instruction t (0..3) multiplies k = t for lanes 0..31
// and k = 4 + t for lanes 32..63.
//
// Tiling (gemm_tile.hpp): a 128x128 macro tile, BK = 32 per LDS stage, two LDS stages with register
// prefetch of the next stage (one barrier per stage), MFMA fragments read one k-group ahead; on 512
// threads = 8 waves in a 2x4 grid, each wave 64x32 = two 32x32 accumulators (gemm_wide.hip: the form
// every whole-tile launch takes, two workgroups to a CU), or on 256 threads = 4 waves in a 2x2 grid,
// each wave 64x64 (the kernel below: the doubly transposed form, the 64x64 tile, the tile policy).
// Tiles are numbered so that each XCD (its own L2) works along one tile row at a time.
//
// This file: the plain kernel (one workgroup per tile and k chunk), the wave-per-tile kernel for
// small and skinny products, the split-K combine, and the host-side plan - which kernel, how
// many k splits, or the spread tail (gemm_spread.hip) for tile grids that do not fill the chip's
// last round of workgroups.  Partial products go to the context workspace and are combined in a
// fixed order, so every plan is deterministic.
#include "gemm_tile.hpp"

namespace slhip {

template <bool TA, bool TB, int BK, bool ONLY_FAST, int WM, int WN>
__global__ __launch_bounds__(256, 2) void gemm_kernel(GemmArgs g) {
  __shared__ __attribute__((aligned(16))) float lds_a[2][Cfg<BK, 64 * WM>::STAGE_FLOATS];
  __shared__ __attribute__((aligned(16))) float lds_b[2][Cfg<BK, 64 * WN>::STAGE_FLOATS];
  gemm_whole_tile<TA, TB, BK, ONLY_FAST, WM, WN>(g, lds_a, lds_b);
}

// Small and skinny problems.  One wave owns one 32x32 tile of C and feeds the matrix core straight
// from global memory: per group of 8 k it loads 4 + 4 scalars per lane (the k permutation of the
// header comment makes them 4 MFMA operand pairs) and issues 4 MFMAs; up to 16 waves of a
// workgroup split the k range of one tile and combine their accumulators through LDS in wave
// order, so the result does not depend on timing.  Next to the tiled kernel it wastes matrix-core
// cycles on narrow tiles and reads operands uncoalesced, but its code is a few hundred bytes:
// the tiled kernel spends about 13 us per launch before its first MFMA retires (fetching
// its long unrolled code cold), which is most of the time of a [1024 x 64] x [64 x 64] product.
// NG = groups of 8 k whose loads are issued together: 8 for small problems (latency is all that
// matters: [1024x64]x[64x64] 7.2 -> 5.9 us), 1 for large skinny ones, which have waves enough to
// hide latency and measured 15-20 % slower with 2, 4 or 8 (8192x10x2048: 41 us against 48).
// FULL = the whole groups of a k range run without bounds checks and a k-contiguous operand comes
// in as one (dword-aligned) float4 per group; a last, partial group is checked.  (Checked element by
// element, 257 x 17 x 33333 took 78 us as A*Bt - 0.5 TB/s - and 1000 x 17 x 33333 250 us.)
// COLSUM (the At*B form only): the workgroups of tile row 0 also add the column sums of B over
// this launch's k range to colsum[N] - the bias gradient of a Linear layer, whose weight gradient
// xT*g reads the very same g.  `nw` = waves that share this tile's k range; a workgroup may hold
// more (the pair kernel below), the others only keep the barrier company.
template <bool TA, bool TB, int NG, bool FULL, bool COLSUM>
__device__ __forceinline__ void wave_tile(const GemmArgs& g, float* red, const unsigned tile, const unsigned ky, const int nw,
                                          float* colsum) {
  const int lane = threadIdx.x & 63, wk = threadIdx.x >> 6;
  const int r = lane & 31, h = lane >> 5;
  const size_t tm = tile / g.tiles_n, tn = tile % g.tiles_n;
  const size_t m0 = tm * 32, n0 = tn * 32;
  const size_t kbeg = (size_t)ky * g.k_chunk;
  const size_t kend = kbeg + g.k_chunk < g.K ? kbeg + g.k_chunk : g.K;
  const size_t groups = (kend - kbeg + 7) / 8, per = (groups + nw - 1) / nw;
  const size_t gbeg = (size_t)wk * per < groups ? (size_t)wk * per : groups;
  const size_t gend = gbeg + per < groups ? gbeg + per : groups;  // empty for waves past nw
  // rows / columns past the edge are clamped: they compute copies that are never stored
  const size_t row = m0 + r < g.M ? m0 + r : g.M - 1, col = n0 + r < g.N ? n0 + r : g.N - 1;
  const float* ap = TA ? g.A + row : g.A + row * g.K;
  const float* bp = TB ? g.B + col * g.K : g.B + col;
  const size_t astep = TA ? g.M : 1, bstep = TB ? 1 : g.N;

  // Accumulator register v of lane (r, h): row 8*(v/4) + 4*h + v%4, column r.  With several waves to
  // a tile, register v is finished by the wave with v % nw == wk (nw is a power of two).  What the
  // epilogue reads from memory (bias, ReLU mask, C for beta) is requested here, ahead of the k
  // loop: asked for after it, each of these loads would put one more trip to memory on the
  // critical path of a kernel that is a handful of such trips long.
  const bool raw = g.splits > 1;
  const size_t c = n0 + r;
  auto idx_of = [&](int v) { return (m0 + 8 * (v / 4) + 4 * h + (v % 4)) * g.N + c; };
  bool mine[16];
#pragma unroll
  for (int v = 0; v < 16; ++v) mine[v] = (v & (nw - 1)) == wk && m0 + 8 * (v / 4) + 4 * h + (v % 4) < g.M && c < g.N;
  float bias = 0.0f, mask_v[16], c_old[16];
  const bool with_mask = !raw && g.mask != nullptr, with_c = !raw && g.beta != 0.0f;
  if (!raw && g.bias && c < g.N) bias = g.bias[c];
  if (with_mask) {
#pragma unroll
    for (int v = 0; v < 16; ++v) mask_v[v] = mine[v] ? g.mask[idx_of(v)] : 0.0f;
  }
  if (with_c) {
#pragma unroll
    for (int v = 0; v < 16; ++v) c_old[v] = mine[v] ? g.C[idx_of(v)] : 0.0f;
  }

  floatx16 acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
  float cs = 0.0f;  // COLSUM: this lane's share of column n0 + r (its half of every group of 8 k)
  // NG groups of 8 k at a time: all 8*NG loads are issued before the first MFMA needs one
  auto run_groups = [&](size_t gi, auto ng_tag, auto checked_tag) {
    constexpr int N = decltype(ng_tag)::value;
    constexpr bool CHECKED = decltype(checked_tag)::value;
    float a[N][4], b[N][4];
#pragma unroll
    for (int u = 0; u < N; ++u) {
      const size_t k = kbeg + (gi + u) * 8 + 4 * h;
      if (FULL && !CHECKED) {
        if (!TA) {
          const float4 v = ld4g(ap + k);
          a[u][0] = v.x; a[u][1] = v.y; a[u][2] = v.z; a[u][3] = v.w;
        } else {
#pragma unroll
          for (int t = 0; t < 4; ++t) a[u][t] = ap[(k + t) * astep];
        }
        if (TB) {
          const float4 v = ld4g(bp + k);
          b[u][0] = v.x; b[u][1] = v.y; b[u][2] = v.z; b[u][3] = v.w;
        } else {
#pragma unroll
          for (int t = 0; t < 4; ++t) b[u][t] = bp[(k + t) * bstep];
        }
      } else {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const bool in = k + t < kend;
          const size_t kc = in ? k + t : kend - 1;
          const float av = ap[kc * astep], bv = bp[kc * bstep];
          a[u][t] = in ? av : 0.0f;
          b[u][t] = in ? bv : 0.0f;
        }
      }
    }
#pragma unroll
    for (int u = 0; u < N; ++u)
#pragma unroll
      for (int t = 0; t < 4; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u][t], b[u][t], acc, 0, 0, 0);
    if (COLSUM) {
#pragma unroll
      for (int u = 0; u < N; ++u)
#pragma unroll
        for (int t = 0; t < 4; ++t) cs += b[u][t];
    }
  };
  // FULL: the whole groups of the k range without a check; a range that ends in a partial group (a
  // K that is not a multiple of 8: only the last range has one) finishes with that group, checked
  const size_t whole = FULL ? (kend - kbeg) / 8 : 0;
  const size_t gfast = FULL ? (gend < whole ? gend : whole) : gbeg;
  size_t gi = gbeg;
  if (FULL) {
    using U = std::false_type;
    for (; gi + NG <= gfast; gi += NG) run_groups(gi, std::integral_constant<int, NG>(), U());
    if (NG > 4)
      for (; gi + 4 <= gfast; gi += 4) run_groups(gi, std::integral_constant<int, 4>(), U());
    for (; gi < gfast; ++gi) run_groups(gi, std::integral_constant<int, 1>(), U());
    for (; gi < gend; ++gi) run_groups(gi, std::integral_constant<int, 1>(), std::true_type());
  } else {
    using C = std::true_type;
    for (; gi + NG <= gend; gi += NG) run_groups(gi, std::integral_constant<int, NG>(), C());
    if (NG > 4)
      for (; gi + 4 <= gend; gi += 4) run_groups(gi, std::integral_constant<int, 4>(), C());
    for (; gi < gend; ++gi) run_groups(gi, std::integral_constant<int, 1>(), C());
  }

  const bool sums = COLSUM && colsum != nullptr && tm == 0;
  if (sums) cs += __shfl_xor(cs, 32);  // the two halves of every group of 8 k
  if (nw > 1) {
    if (wk < nw) {
#pragma unroll
      for (int v = 0; v < 16; ++v) red[(wk * 16 + v) * 64 + lane] = acc[v];
      if (sums && h == 0) red[nw * 16 * 64 + wk * 32 + r] = cs;
    }
    __syncthreads();
  }
  if (wk >= nw) return;
  if (sums && wk == 0 && h == 0 && n0 + r < g.N) {
    float t = cs;
    if (nw > 1) {
      t = red[nw * 16 * 64 + r];
      for (int w = 1; w < nw; ++w) t += red[nw * 16 * 64 + w * 32 + r];
    }
    colsum[n0 + r] += t;
  }
  float* dst = raw ? g.partial + (size_t)ky * g.M * g.N : g.C;
  if (c >= g.N) return;
  float val[16];
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    val[v] = acc[v];
    if (nw > 1 && mine[v]) {
      float t = red[v * 64 + lane];
      for (int w = 1; w < nw; ++w) t += red[(w * 16 + v) * 64 + lane];
      val[v] = t;
    }
  }
  if (!raw) {
    if (with_mask) {
#pragma unroll
      for (int v = 0; v < 16; ++v) val[v] = (mask_v[v] >= 0.0f ? 1.0f : 0.0f) * val[v];
    }
    if (with_c) {
#pragma unroll
      for (int v = 0; v < 16; ++v) val[v] = g.beta * c_old[v] + val[v];
    }
    if (g.bias) {
#pragma unroll
      for (int v = 0; v < 16; ++v) val[v] = val[v] + bias;
    }
    if (g.pre_act) {
#pragma unroll
      for (int v = 0; v < 16; ++v)
        if (mine[v]) g.pre_act[idx_of(v)] = val[v];
    }
    if (g.relu) {
#pragma unroll
      for (int v = 0; v < 16; ++v) val[v] = (val[v] >= 0.0f ? 1.0f : 0.0f) * val[v];
    }
  }
#pragma unroll
  for (int v = 0; v < 16; ++v)
    if (mine[v]) dst[idx_of(v)] = val[v];
}

template <bool TA, bool TB, int NG, bool FULL>
__global__ __launch_bounds__(1024) void gemm_wave_kernel(GemmArgs g) {
  extern __shared__ float red[];  // [waves][16][64]
  wave_tile<TA, TB, NG, FULL, false>(g, red, blockIdx.x, blockIdx.y, blockDim.x >> 6, nullptr);
}

// Both products of a small Linear layer's backward pass in one launch: workgroups below `tiles_x`
// compute tiles of x.grad = g*wT (optionally masked by a ReLU's pre-activation), the others tiles of
// w.grad = xT*g, and those of its first tile row the bias gradient as well.  Each product keeps the
// plan (waves per tile, order of its sums) that a launch of its own would use, so the results are
// the same bits; what is saved is two launches per layer of a step that is all launch latency.
template <bool FULLX, bool FULLW>
__global__ __launch_bounds__(512) void gemm_wave_pair_kernel(GemmArgs gx, GemmArgs gw, float* colsum, unsigned tiles_x, int nw_x,
                                                             int nw_w) {
  extern __shared__ float red[];  // [waves][16][64] + [waves][32]
  if (blockIdx.x < tiles_x) wave_tile<false, true, 8, FULLX, false>(gx, red, blockIdx.x, 0, nw_x, nullptr);
  else wave_tile<true, false, 8, FULLW, true>(gw, red, blockIdx.x - tiles_x, 0, nw_w, colsum);
}

// C = sum_z partial[z] (z ascending) + beta*C, then bias / relu.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(size_t mn, size_t N, unsigned splits,
                                                            const float* __restrict__ partial, float* C, float beta,
                                                            const float* __restrict__ bias, int relu, float* pre_act,
                                                            const float* __restrict__ mask, int vec) {
  const size_t stride = (size_t)gridDim.x * 256;
  const size_t tid = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (vec) {
    for (size_t i = tid; i < (mn >> 2); i += stride) {
      float4 s = ld4g(partial + 4 * i);
      unsigned z = 1;
      for (; z + 4 <= splits; z += 4) {  // four loads in flight, added in the same order as one by one
        float4 p[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) p[u] = ld4g(partial + (size_t)(z + u) * mn + 4 * i);
#pragma unroll
        for (int u = 0; u < 4; ++u) { s.x += p[u].x; s.y += p[u].y; s.z += p[u].z; s.w += p[u].w; }
      }
      for (; z < splits; ++z) {
        float4 p = ld4g(partial + (size_t)z * mn + 4 * i);
        s.x += p.x; s.y += p.y; s.z += p.z; s.w += p.w;
      }
      if (mask) {
        float4 m = ld4g(mask + 4 * i);
        s.x *= (m.x >= 0.f ? 1.f : 0.f); s.y *= (m.y >= 0.f ? 1.f : 0.f);
        s.z *= (m.z >= 0.f ? 1.f : 0.f); s.w *= (m.w >= 0.f ? 1.f : 0.f);
      }
      if (beta != 0.0f) {
        float4 c = ld4g(C + 4 * i);
        s.x = beta * c.x + s.x; s.y = beta * c.y + s.y; s.z = beta * c.z + s.z; s.w = beta * c.w + s.w;
      }
      if (bias) {
        if (N % 4 == 0) {
          float4 b = ld4g(bias + (4 * i) % N);
          s.x += b.x; s.y += b.y; s.z += b.z; s.w += b.w;
        } else {  // the vector runs over a row end
          const size_t c = (4 * i) % N;
          s.x += bias[c]; s.y += bias[(c + 1) % N]; s.z += bias[(c + 2) % N]; s.w += bias[(c + 3) % N];
        }
      }
      if (pre_act) st4g(pre_act + 4 * i, s);
      if (relu) {
        s.x = (s.x >= 0.f ? 1.f : 0.f) * s.x; s.y = (s.y >= 0.f ? 1.f : 0.f) * s.y;
        s.z = (s.z >= 0.f ? 1.f : 0.f) * s.z; s.w = (s.w >= 0.f ? 1.f : 0.f) * s.w;
      }
      st4g(C + 4 * i, s);
    }
  } else {
    for (size_t i = tid; i < mn; i += stride) {
      float s = partial[i];
      for (unsigned z = 1; z < splits; ++z) s += partial[(size_t)z * mn + i];
      if (mask) s *= (mask[i] >= 0.f ? 1.f : 0.f);
      if (beta != 0.0f) s = beta * C[i] + s;
      if (bias) s += bias[i % N];
      if (pre_act) pre_act[i] = s;
      if (relu) s = (s >= 0.f ? 1.f : 0.f) * s;
      C[i] = s;
    }
  }
}

// The same sums written transposed: C[n * M + r] = beta * C[n * M + r] + sum_z partial[z][r * N + n], for an
// M x N product with a narrow N (at most 32) that stands for the N x M product the caller asked for.
// Thread i takes element i of C (consecutive lanes: consecutive r of one n), so the stores are whole lines
// and a wave's loads cover one contiguous run of 64 rows of the partial.
__global__ __launch_bounds__(256) void splitk_reduce_t_kernel(size_t M, size_t N, unsigned splits, const float* __restrict__ partial,
                                                              float* C, float beta) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= M * N) return;
  const size_t n = i / M, r = i - n * M;
  const float* p = partial + r * N + n;
  const size_t step = M * N;
  float s = p[0];
  unsigned z = 1;
  for (; z + 8 <= splits; z += 8) {  // eight loads in flight, added in the same order as one by one
    float t[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) t[u] = p[(size_t)(z + u) * step];
#pragma unroll
    for (int u = 0; u < 8; ++u) s += t[u];
  }
  for (; z < splits; ++z) s += p[(size_t)z * step];
  C[i] = beta != 0.0f ? beta * C[i] + s : s;
}

static int32_t splitk_combine(slhip_ctx* ctx, const GemmArgs& g, size_t splits) {
  if (ctx->swap_c && !g.bias && !g.relu && !g.pre_act && !g.mask && g.beta == 0.0f && g.M * g.N <= 0xffffffffu * (size_t)256) {
    hipLaunchKernelGGL(splitk_reduce_t_kernel, dim3((unsigned)((g.M * g.N + 255) / 256)), dim3(256), 0, ctx->stream, g.M, g.N,
                       (unsigned)splits, (const float*)ctx->workspace, ctx->swap_c, ctx->swap_beta);
    ctx->swap_done = true;
    return post_launch();
  }
  const size_t mn = g.M * g.N;
  const int vec = mn % 4 == 0;  // the flat M x N array in whole vectors (each may run over a row end)
  size_t blocks = ((vec ? mn / 4 : mn) + 255) / 256;
  const size_t cap = (size_t)ctx->num_cu * 16;
  if (blocks > cap) blocks = cap;
  hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, mn, g.N, (unsigned)splits,
                     (const float*)ctx->workspace, g.C, g.beta, g.bias, g.relu, g.pre_act, g.mask, vec);
  return post_launch();
}

// Plan of the wave-per-tile kernel for an M x N x K product: waves per workgroup (at most 8 for
// small problems, where 16 measured 10-15 % slower, at most 16 for large skinny ones, where 8
// did), each keeping >= 4 groups of 8 k; then whole-grid splits of K until the chip has about 8
// waves per CU.  A split of a large problem keeps >= 8 groups per wave.  A split of a small one
// keeps >= 32: up to there the extra groups of an unsplit wave (about 1.2 us per 8) cost less than
// the combine kernel that a split brings (3-4 us, and one more node in a recorded step).
// Returns whether the problem counts as small (<= 2^25 flop).
static bool wave_plan(const slhip_ctx* ctx, size_t M, size_t N, size_t K, unsigned* nw_out, size_t* splits_out,
                      size_t* k_chunk_out) {
  const double flop = 2.0 * (double)M * (double)N * (double)K;
  const size_t tiles = ((M + 31) / 32) * ((N + 31) / 32), groups = (K + 7) / 8;
  const size_t mn_bytes = M * N * sizeof(float);
  unsigned nw = 1;
  const bool small = flop <= 33554432.0;
  while (nw < (small ? 8u : 16u) && groups >= (size_t)nw * 2 * 4) nw *= 2;
  size_t splits = 1;
  const size_t want = (size_t)ctx->num_cu * 8;
  if (tiles * nw < want) {
    splits = (want + tiles * nw - 1) / (tiles * nw);
    const size_t most = groups / ((size_t)nw * (small ? 32 : 8));
    if (splits > most) splits = most;
    if (splits > 64) splits = 64;
    if (splits > ctx->workspace_bytes / mn_bytes) splits = ctx->workspace_bytes / mn_bytes;
    if (splits < 1) splits = 1;
  }
  const size_t k_chunk = ((K + splits - 1) / splits + 7) / 8 * 8;
  *nw_out = nw;
  *k_chunk_out = k_chunk;
  *splits_out = (K + k_chunk - 1) / k_chunk;
  return small;
}

static int32_t gemm_run(slhip_ctx* ctx, bool ta, bool tb, size_t M, size_t N, size_t K, const float* A, const float* B,
                        float* C, float beta, const float* bias, int relu, float* pre_act, const float* mask) {
  // an operand that is a single row or column reads the same either way: the form measured faster
  // (16384 x 1 x 16384: A*B 186 us, A*Bt 328; 16384 x 16384 x 1: 226 against 244)
  if (N == 1 || K == 1) tb = false;
  if (M == 1 || K == 1) ta = false;
  // a row vector times a matrix is the matrix, transposed, times a column vector: the shape the
  // narrow-N kernels stream (1 x 16384 x 16384: 284-355 us as it stood, 186-193 that way round)
  if (M == 1 && N > 1 && K > 1 && !bias && !relu && !pre_act && !mask)
    return gemm_run(ctx, !tb, false, N, 1, K, B, A, C, beta, nullptr, 0, nullptr, nullptr);
  // A few rows times a large matrix (a small batch through a wide layer): C^T = op(B)^T * op(A)^T is the
  // shape the tall and narrow kernels stream - the large operand once, at 5-6 TB/s, where the wave-per-tile
  // kernel reads it in 128-byte pieces per row (16 x 16384 x 16384: 2.8-3.7 TB/s of B).  C^T goes to the top of
  // the workspace (the inner product sees a workspace that ends below it) and is transposed into C, which is
  // where beta (0 or 1) is applied - unless the inner product ends in a combine of k shares, which then writes
  // C itself, transposed (one launch less: 10 x 2048 x 8192 24 -> 20 us).  Up to 32 rows (the inner kernels'
  // columns).  Measured, us before -> after, A*B / A*Bt / At*B:
  // 16 x 16384 x 16384 313 / 399 / 319 -> 237 / 193 / 187; 10 x 4096 x 32768 246 / 322 / 254 -> 104 / 111 / 94;
  // 2 x 10000 x 10000 161 / 190 / 171 -> 88 / 114 / 83; 32 x 16384 x 16384 A*Bt 468 -> 275; 8 x 2048 x 8192 34 / 36 / 36 -> 24 / 28 / 23.
  // (17..32 rows against a B stored K x N only where N is a multiple of 32, which the inner kernel for that many columns needs)
  // From how many elements of B: 2^24; 2^23 for at most 16 rows against a B stored K x N (16 x 2048 x 4096 A*B 21.5 ->
  // 16.1 us, At*B 22.1 -> 15.2; A*Bt loses there, 22.3 -> 24.0, and so do 32 rows); 2^22 for fewer than 8 rows stored
  // K x M (4 x 2048 x 2048 At*B 19.9 -> 11.6); 2^25 for fewer than 8 rows stored M x K (the inner kernels for fewer
  // than 8 columns want them as K x M and turn them round only beside an operand that large).
  const int swap_from = !ta && M < 8 ? 25 : ta && !tb && M < 8 ? 22 : !tb && M <= 16 ? 23 : 24;
  if (M >= 2 && M <= 32 && (tb || M <= 16 || N % 32 == 0) && N >= 512 && K >= 256 && N * K >= (size_t(1) << swap_from) && !bias && !relu &&
      !pre_act && !mask && (beta == 0.0f || beta == 1.0f)) {
    const size_t tmp_bytes = (M * N * sizeof(float) + 255) & ~(size_t)255;
    if (tmp_bytes <= ((size_t)16 << 20) && ctx->workspace_bytes >= tmp_bytes + ((size_t)128 << 20)) {
      const size_t whole = ctx->workspace_bytes;
      float* ct = (float*)((char*)ctx->workspace + whole - tmp_bytes);
      ctx->workspace_bytes = whole - tmp_bytes;
      // (where the inner product ends in a combine of k shares, that combine writes C itself, transposed)
      ctx->swap_c = C; ctx->swap_beta = beta; ctx->swap_done = false;
      const int32_t rc = gemm_run(ctx, !tb, !ta, N, M, K, B, A, ct, 0.0f, nullptr, 0, nullptr, nullptr);
      const bool done = ctx->swap_done;
      ctx->swap_c = nullptr; ctx->swap_done = false;
      ctx->workspace_bytes = whole;
      if (rc != SLHIP_OK || done) return rc;
      const auto inner = ctx->last_gemm;
      const int32_t rt = slhip_transpose(ctx, N, M, ct, C, beta);
      ctx->last_gemm = inner;
      return rt;
    }
  }
  GemmArgs g;
  g.M = M; g.N = N; g.K = K; g.A = A; g.B = B; g.C = C; g.beta = beta;
  g.bias = bias; g.relu = relu; g.pre_act = pre_act; g.mask = mask;
  const size_t lda = ta ? M : K, ldb = tb ? K : N;
  g.a_vec = lda % 4 == 0;  // dword-aligned vector loads: the leading dimension decides, not the base
  g.b_vec = ldb % 4 == 0;
  // (the fast loop addresses a tile panel with 32-bit byte offsets: 127 rows of the leading dimension)
  g.m_fast = (aligned16(A) && aligned16(B) && lda < (size_t(1) << 22) && ldb < (size_t(1) << 22)) ? M : 0;
  g.partial = (float*)ctx->workspace;
  const size_t mn_bytes = M * N * sizeof(float);

  // HBM-bound skinny products with float4-friendly shapes: vector-ALU kernels of their own
  {
    int32_t rc = SLHIP_OK;
    int took = gemm_tall_launch(ctx, ta, tb, g, &rc);
    ctx->last_gemm.kind = 5;
    if (took == 0) {
      took = gemm_skinny_launch(ctx, ta, tb, g, &rc);
      ctx->last_gemm.kind = 6;
    }
    ctx->last_gemm.ta = ta; ctx->last_gemm.tb = tb; ctx->last_gemm.splits = took == 2 ? g.splits : 1;
    if (took == 1 || rc) return rc;
    if (took == 2) return splitk_combine(ctx, g, g.splits);
  }

  // Small and skinny (an output side <= 32, or K <= 16) products: wave-per-tile kernel.  "Small" is
  // <= 6e8 flop when the kernel can use its unchecked vector-load form (it then beats the tiled
  // kernel up to about 700^3: 512^3 takes 7.2 us against 17.4), <= 2^25 flop otherwise.
  const double flop = 2.0 * (double)M * (double)N * (double)K;
  // (the vector loads of a k-contiguous operand need dword alignment only; a K that is not a multiple
  // of 8 ends in one checked group)
  const bool wave_full = K >= 8;
  // products whose K or bases are off the 8-float grid go to the tiled kernels from a lower size on: the
  // staged tiles absorb the misalignment that the wave kernel's direct loads pay for
  const bool wave_aligned = K % 8 == 0 && (ta || g.a_vec) && (!tb || g.b_vec);
  // ... unless the output is a hundred 64 x 64 tiles or more and K at least four k tiles: the eight-wave small
  // tile then fills the chip and is ahead (per launch 1024^2 x 256 15.8 -> 10.3 us, 1024^2 x 128 10.0 -> 8.1,
  // 768^2 x 448 16.8 -> 13.0, 640^3 17.1 -> 14.6, 600^3 16.4 -> 15.5), where up to 64 tiles it is behind
  // (512^3 9.5 against 12.6, 448^3 9.3 / 12.8, 512^2 x 256 7.8 / 9.8)
  const bool many_tiles = ((M + 63) / 64) * ((N + 63) / 64) >= 100 && K >= 128 && flop > 33554432.0 && !(ta && tb);
  if (flop <= (wave_aligned && !many_tiles ? 6.0e8 : 33554432.0) || M <= 32 || N <= 32 || K <= 16) {
    const size_t wt_m = (M + 31) / 32, wt_n = (N + 31) / 32;
    if (wt_m * wt_n > 0x7fffffffu) {
      set_error("sgemm: %zu x %zu tiles exceed one launch", wt_m, wt_n);
      return SLHIP_EINVAL;
    }
    g.tiles_m = (unsigned)wt_m; g.tiles_n = (unsigned)wt_n;
    const size_t tiles = wt_m * wt_n;
    unsigned nw;
    size_t splits, k_chunk;
    const bool small = wave_plan(ctx, M, N, K, &nw, &splits, &k_chunk);
    g.splits = (unsigned)splits;
    g.k_chunk = k_chunk;
    dim3 wgrid((unsigned)tiles, (unsigned)splits);
    const size_t lds = nw > 1 ? (size_t)nw * 16 * 64 * sizeof(float) : 0;
    // whole groups of 8 k everywhere (k_chunk is a multiple of 8) and float4-loadable k-contiguous operands
    const bool full = wave_full;
#define SL_WGEMM2(TA_, TB_, NG_, FULL_) \
  hipLaunchKernelGGL((gemm_wave_kernel<TA_, TB_, NG_, FULL_>), wgrid, dim3(64 * nw), lds, ctx->stream, g)
#define SL_WGEMM(TA_, TB_)                                   \
  do {                                                       \
    if (small && full) SL_WGEMM2(TA_, TB_, 8, true);         \
    else if (small) SL_WGEMM2(TA_, TB_, 8, false);           \
    else if (full) SL_WGEMM2(TA_, TB_, 1, true);             \
    else SL_WGEMM2(TA_, TB_, 1, false);                      \
  } while (0)
    if (!ta && !tb) SL_WGEMM(false, false);
    else if (!ta && tb) SL_WGEMM(false, true);
    else if (ta && !tb) SL_WGEMM(true, false);
    else SL_WGEMM(true, true);
#undef SL_WGEMM
#undef SL_WGEMM2
    ctx->last_gemm = {1, ta, tb, full, false, (unsigned)splits, nw};
    int32_t rc = post_launch();
    if (rc || splits == 1) return rc;
    return splitk_combine(ctx, g, splits);
  }

  size_t tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  if ((M + 63) / 64 * ((N + 63) / 64) > 0x7fffffffu) {
    set_error("sgemm: %zu x %zu tiles exceed one launch", (M + 63) / 64, (N + 63) / 64);
    return SLHIP_EINVAL;
  }
  g.tiles_m = (unsigned)tiles_m; g.tiles_n = (unsigned)tiles_n;

  // Split K when the tile grid alone leaves CUs idle.  The split count minimises a cost model
  // fitted to MI355X timings of this kernel (512^3 ... 2048x2048x8192, 1..32 splits, within
  // about 10 %): two workgroups share a CU, a k tile takes 4.35 us when they do and 2.43 us when
  // a workgroup has the CU to itself (at most one workgroup per CU in flight); workgroups run in
  // rounds of `slots`; every round costs 6 us on top (first loads, epilogue); combining the
  // partial products costs 4 us plus their bytes, written and read once, at 5 TB/s.  Tile grids of
  // up to four rounds are considered too: 576 tiles (3072^3) unsplit run one full round and one
  // that is an eighth full, 75 TFLOP/s against 106 with four splits.
  constexpr int BK = GEMM_BK;
  size_t tiles = tiles_m * tiles_n;
  const size_t slots = (size_t)ctx->num_cu * 2;
  size_t splits = 1;
  const size_t kt_total = (K + BK - 1) / BK;
  double best = 1e300;  // modelled time of the plan chosen so far, in us
  if (tiles < 4 * slots && kt_total >= 4) {
    size_t max_splits = kt_total / 2;  // every split keeps at least two k tiles
    if (max_splits > 32) max_splits = 32;
    const size_t fit = ctx->workspace_bytes / mn_bytes;
    if (max_splits > fit) max_splits = fit;
    for (size_t sp = 1; sp <= max_splits; ++sp) {
      const size_t kt = (kt_total + sp - 1) / sp;
      const size_t wgs = tiles * sp;
      const size_t full_rounds = wgs / slots, rest = wgs % slots;
      double t;
      if (full_rounds == 0) {
        t = kt * (rest <= slots / 2 ? 2.43 : 4.35) + 6.0;
      } else {
        // workgroups are handed out as slots free up, so a partly filled last round costs about
        // half of what a strict round-by-round schedule would lose
        const double exact = (double)wgs / (double)slots, up = (double)(full_rounds + (rest ? 1 : 0));
        // (a last round more than half full puts two workgroups on some CUs, and those set its length:
        // the eight-wave kernel's single workgroups finish in 0.525 of that time and wait)
        t = (exact + (2 * rest > slots ? 0.75 : 0.5) * (up - exact)) * kt * 4.35 + up * 6.0;
      }
      if (sp > 1) t += 4.0 + 2.0 * (double)sp * (double)mn_bytes / 5.0e6;
      if (t < best) { best = t; splits = sp; }
    }
  }
  // The other remedy for a partly filled last round: the spread tail.  The whole rounds run as
  // whole tiles; the k tiles of the remaining tiles, taken as one sequence, are dealt out evenly to
  // one more round of workgroups in the same launch, which start as the whole-tile workgroups
  // retire; their partial tiles are summed in a fixed order by a second kernel.
  SpreadArgs sp;
  sp.first = sp.units = sp.total = 0;
  sp.kt_total = (unsigned)kt_total;
  size_t spread_workers = 0;
  if (tiles % slots != 0 && tiles < 16 * slots && kt_total >= 8 && kt_total < (1u << 20) && ctx->gemm_tail != SLHIP_TAIL_WHOLE) {
    const size_t full = tiles / slots * slots, tail = tiles - full;
    const size_t total = tail * kt_total;
    size_t units = (total + slots - 1) / slots;
    if (units < 4) units = 4;
    if (units > kt_total) units = kt_total;  // a workgroup's k tiles then touch at most two tiles of C
    const size_t workers = (total + units - 1) / units;
    const size_t runs = tail + workers;  // upper bound of partial tiles written
    if (2 * workers * SPREAD_SLOT * sizeof(float) <= ctx->workspace_bytes && total < (1u << 31)) {
      const double per_kt = (full == 0 && workers <= slots / 2) ? 2.43 : 4.35;
      const double t = (double)(full / slots) * ((double)kt_total * 4.35 + 6.0) + (double)units * per_kt + 6.0 + 4.0 +
                       2.0 * (double)runs * (double)(SPREAD_SLOT * sizeof(float)) / 5.0e6;
      // A last round that is at most half full gives every tile a CU of its own, where the eight-wave
      // kernel takes 0.525 of the time of a round of two workgroups per CU: spreading a tail of 0.4 to
      // 0.5 rounds gains less than the spread's own overhead (fix-up launch, partial tiles) while K is
      // short.  Measured at one to four whole rounds + 208..240 tiles: whole launches 3-17 % ahead up to
      // K = 1024, the spread tail 0-6 % ahead from K = 1536; tails of 64..128 tiles: the spread tail at every K.
      const bool whole_wide_wins = ctx->gemm_tail == SLHIP_TAIL_AUTO && ctx->gemm_tile == SLHIP_TILE_AUTO && !(ta && tb) &&
                                   full > 0 && 2 * tail <= slots && 5 * tail >= 2 * slots && kt_total <= 40;
      if (!whole_wide_wins && (t < best || ctx->gemm_tail == SLHIP_TAIL_SPREAD)) {
        best = t;
        splits = 1;
        sp.first = (unsigned)full;
        sp.units = (unsigned)units;
        sp.total = (unsigned)total;
        spread_workers = workers;
      }
    }
  }

  // 64 x 64 tiles, one workgroup per tile and no k split, for products of a few hundred such tiles
  // and a moderate K, where the plans above spend a third of their time combining partial
  // products: 1024^3 takes 33 us as 64 tiles x 4 k splits + combine and 28 us as 256 small tiles
  // (896^3 +12 %, 704^3 +25 %, 2048x512x1024 +18 %).  A small tile's k tile measures 0.75 us with
  // the CU to itself, 1.25 / 1.8 / 2.3 us when two / three / four workgroups share the CU (4096^3
  // would run at 116 TFLOP/s that way), plus 5 us per launch; it has to beat the modelled time of
  // the best 128 x 128 plan by 8 %, the models being good to about that.
  // The same small tiles with their k ranges spread over the chip (all of them: fewer tiles than
  // workgroup slots), for outputs of a few small tiles and a long K - a 64 x 64 x 1048576 product
  // uses a quarter of a 128 x 128 tile's matrix-core work: 320 us there, about a third of that here.
  bool small_tile = false;
  if (!(ta && tb)) {  // the doubly transposed form is not instantiated for the small tile
    const size_t tiles64 = ((M + 63) / 64) * ((N + 63) / 64);
    static const double per_kt[5] = {0.0, 0.75, 1.25, 1.8, 2.3};
    // (on eight waves, which up to two workgroups per CU take: 0.69 and 1.18; that is what the choice between
    // the tiles below counts with, while the choice between whole small tiles and their spread form keeps the
    // four-wave figures it was measured with)
    static const double per_kt8[3] = {0.0, 0.69, 1.18};
    const size_t slots64 = (size_t)ctx->num_cu * 4;
    const bool automatic = ctx->gemm_tile == SLHIP_TILE_AUTO && ctx->gemm_tail == SLHIP_TAIL_AUTO && best < 1e299;
    // plan 1: one workgroup per small tile
    double t_whole = 1e300;
    if (tiles64 <= slots64) t_whole = (double)kt_total * per_kt[(tiles64 + ctx->num_cu - 1) / ctx->num_cu] + 5.0;
    // plan 2: the k tiles of all small tiles dealt out evenly
    double t_spread = 1e300;
    size_t units64 = 0, workers64 = 0;
    if (tiles64 < slots64 && kt_total >= 16 && kt_total < (1u << 20) && tiles64 * kt_total < (1u << 31)) {
      const size_t total = tiles64 * kt_total;
      units64 = (total + slots64 - 1) / slots64;
      if (units64 < 8) units64 = 8;
      if (units64 > kt_total) units64 = kt_total;
      workers64 = (total + units64 - 1) / units64;
      if (2 * workers64 * 64 * 64 * sizeof(float) <= ctx->workspace_bytes)
        t_spread = (double)units64 * per_kt[(workers64 + ctx->num_cu - 1) / ctx->num_cu] + 5.0 + 4.0 +
                   2.0 * (double)(tiles64 + workers64) * (64.0 * 64.0 * sizeof(float)) / 5.0e6;
    }
    bool spread64 = false;
    if (ctx->gemm_tile == SLHIP_TILE_64X64) {
      small_tile = true;
      spread64 = ctx->gemm_tail == SLHIP_TAIL_SPREAD && t_spread < 1e299;
    } else if (automatic) {
      double t_whole8 = t_whole;
      if (tiles64 <= 2 * (size_t)ctx->num_cu) t_whole8 = (double)kt_total * per_kt8[(tiles64 + ctx->num_cu - 1) / ctx->num_cu] + 5.0;
      const double t64 = t_whole8 < t_spread ? t_whole8 : t_spread;
      small_tile = t64 < 0.92 * best;
      spread64 = small_tile && t_spread < t_whole;
    }
    // More small tiles than the chip holds at once, short K: the large tile's workgroups spend more time
    // on their first loads and their 64 KiB of results than on their few k tiles, and a last round of them
    // that is partly empty cannot be spread (too few k tiles to deal out).  The small tile is level or
    // ahead up to K = 128 whatever the grid (4096^2 x 64: 34 -> 31 us, 3000 x 5000 x 100: 49 -> 45, 10000 x 1000 x
    // 100: 40 -> 33; 8192^2 x 128 and 2048 x 8192 x 128 level), and up to K = 384 where its rounds are the fuller
    // ones (10000 x 1000 x 256: 73 -> 51, x 384: 96 -> 71; 33333 x 257 x 257: 84 -> 63); from K = 200 on a grid that
    // fills its rounds either way the large tile is 2-7 % ahead and stays.
    // Fewer than four k tiles (no large-tile plan is modelled that short) and small tiles that fit the chip
    // at once: 2610 x 160 x 70 13 -> 8 us, 1080 x 578 x 69 13 -> 8, 586 x 1419 x 33 12 -> 7, 1104 x 1156 x 75 14 -> 10.
    if (ctx->gemm_tile == SLHIP_TILE_AUTO && ctx->gemm_tail == SLHIP_TAIL_AUTO && !small_tile && kt_total < 4 && tiles64 <= slots64)
      small_tile = true;
    // And where the large tiles are a single round that is at most 85 % full (some CUs hold two workgroups,
    // the others one, which finishes early and waits): up to K = 512 the small tiles are 10-28 % ahead of
    // whatever the large-tile plans make of it (2304^2 x 512: 72 -> 57 us, 2000 x 3000 x 200: 38 -> 30, 1800 x 2600 x
    // 256: 40 -> 32, 2500^2 x 512: 71 -> 63; 2816^2, a round 95 % full, level); at K = 1024 they are level to 14 %
    // ahead, at 2048 level, and the large-tile plans stay.
    if (ctx->gemm_tile == SLHIP_TILE_AUTO && ctx->gemm_tail == SLHIP_TAIL_AUTO && !small_tile && tiles64 > slots64) {
      const size_t slots128 = (size_t)ctx->num_cu * 2;
      const double fill128 = (double)tiles / (double)((tiles + slots128 - 1) / slots128 * slots128);
      const double fill64 = (double)tiles64 / (double)((tiles64 + slots64 - 1) / slots64 * slots64);
      if (splits == 1 && spread_workers == 0 && (K <= 128 || (K <= 384 && fill64 > 1.1 * fill128))) small_tile = true;
      if (K <= 640 && tiles < slots128 && tiles * 100 <= slots128 * 85) small_tile = true;
      // ragged grids: where the small tiles waste at least 4 % less of their area on the edges of C they are
      // 12-19 % ahead up to K of about 1500 (3209 x 1809 x 1354: 161 -> 136 us, 6313 x 931 x 1164: 141 -> 120,
      // 791 x 6880 x 1230: 145 -> 130); the large-tile plans for such grids pay a spread tail and its fix-up too
      const double used128 = (double)M * (double)N / ((double)tiles * 128.0 * 128.0);
      const double used64 = (double)M * (double)N / ((double)tiles64 * 64.0 * 64.0);
      if (K <= 1536 && used64 >= 1.04 * used128) small_tile = true;
    }
    if (small_tile) {
      tiles_m = (M + 63) / 64; tiles_n = (N + 63) / 64;
      tiles = tiles64;
      g.tiles_m = (unsigned)tiles_m; g.tiles_n = (unsigned)tiles_n;
      splits = 1;
      spread_workers = 0;
      if (spread64) {
        sp.first = 0;
        sp.units = (unsigned)units64;
        sp.total = (unsigned)(tiles64 * kt_total);
        spread_workers = workers64;
      }
    }
  }
  const size_t tile_m = small_tile ? 64 : BM, tile_n = small_tile ? 64 : BN;
  // More than half a round of large tiles and at most one per CU, whole or split in two: one workgroup of
  // sixteen waves per tile, unsplit (gemm_wide.hip; 2048^3 129.2 -> 125.9 us per launch, 2048 x 2048 x 4096
  // 252.5 -> 245.0, 2048 x 2048 x 8192 484.2 with two k splits and their combine -> 478.6 without)
  const bool wide16 = ctx->gemm_tile == SLHIP_TILE_AUTO && ctx->gemm_tail == SLHIP_TAIL_AUTO && !small_tile && !(ta && tb) &&
                      spread_workers == 0 && splits <= 2 && tiles <= (size_t)ctx->num_cu && 2 * tiles > (size_t)ctx->num_cu;
  if (wide16) splits = 1;

  size_t k_chunk = (K + splits - 1) / splits;
  k_chunk = (k_chunk + BK - 1) / BK * BK;
  if (k_chunk == 0) k_chunk = BK;
  splits = (K + k_chunk - 1) / k_chunk;
  if (splits < 1) splits = 1;
  g.splits = (unsigned)splits;
  g.k_chunk = k_chunk;

  // every k tile of every workgroup complete, inside and 16-byte aligned: the kernel without the
  // clamped loops (k_chunk is a multiple of BK, so only the end of K can leave a partial tile)
  const bool only_fast = g.a_vec && g.b_vec && g.m_fast && M % tile_m == 0 && N % tile_n == 0 && K % BK == 0;
  ctx->last_gemm = {spread_workers ? 4 : 2, ta, tb, only_fast, small_tile, (unsigned)splits, 4};
  if (spread_workers) {
    // On eight waves like the whole-tile launches (two workgroups put four waves on a SIMD: 3584^3 138 -> 143
    // TFLOP/s, 4608^3 141 -> 146, 7168^3 144 -> 148), except where a short tail of an eighth to a quarter of a
    // round follows whole rounds of a short K, which measured 3-5 % behind the four-wave form
    // (10000 x 1000 x 1024: 178 against 170 us; 5000 x 2000 x 2048: 333 against 318)
    const size_t tail = tiles - sp.first;
    const bool four = ctx->gemm_tile == SLHIP_TILE_128X128 ||
                      (ctx->gemm_tile == SLHIP_TILE_AUTO && sp.first > 0 && tail * 8 > slots && tail * 4 <= slots &&
                       kt_total >= 12 && kt_total < 96);
    return gemm_spread_launch(ctx, ta, tb, only_fast, small_tile, g, sp, spread_workers, tail, !four);
  }

  if (wide16) {
    ctx->last_gemm.kind = 3;
    ctx->last_gemm.waves = 16;
    return gemm_wide16_launch(ctx, ta, tb, only_fast, g);
  }
  // The 128 x 128 tile on eight waves (gemm_wide.hip)
  const bool wide_fits = !small_tile && !(ta && tb);
  if (wide_fits && (ctx->gemm_tile == SLHIP_TILE_128X128_WIDE ||
                    (ctx->gemm_tile == SLHIP_TILE_AUTO && ctx->gemm_tail == SLHIP_TAIL_AUTO))) {
    ctx->last_gemm.kind = 3;
    ctx->last_gemm.waves = 8;
    int32_t rc = gemm_wide_launch(ctx, ta, tb, only_fast, g);
    if (rc || splits == 1) return rc;
    return splitk_combine(ctx, g, splits);
  }

  // The 64 x 64 tile with at most two workgroups per CU: on eight waves, two sets of four that split every k
  // tile (gemm_wide.hip), which doubles the waves on a SIMD: with one workgroup per CU 1024^3 24.2 -> 22.4 us per
  // launch, 896^3 21.7 -> 20.3, 1000^3 25.0 -> 23.6, 2048 x 512 x 1024 24.1 -> 22.5; with two 1536 x 1024 x 1024
  // 38.4 -> 36.0, 1400 x 1200 x 1000 39.4 -> 37.4, 1408^2 x 768 30.5 -> 29.2; level at K of 256-300
  if (small_tile && !(ta && tb) && splits == 1 && tiles <= 2 * (size_t)ctx->num_cu && ctx->gemm_tile == SLHIP_TILE_AUTO) {
    ctx->last_gemm.waves = 8;
    return gemm_small8_launch(ctx, ta, tb, only_fast, g);
  }

  dim3 grid((unsigned)tiles, (unsigned)splits);
#define SL_GEMM3(TA_, TB_, WM_, WN_)                                                                                  \
  do {                                                                                                                \
    if (only_fast) hipLaunchKernelGGL((gemm_kernel<TA_, TB_, GEMM_BK, true, WM_, WN_>), grid, dim3(256), 0, ctx->stream, g); \
    else hipLaunchKernelGGL((gemm_kernel<TA_, TB_, GEMM_BK, false, WM_, WN_>), grid, dim3(256), 0, ctx->stream, g);  \
  } while (0)
#define SL_GEMM(TA_, TB_)                       \
  do {                                          \
    if (small_tile) SL_GEMM3(TA_, TB_, 1, 1);   \
    else SL_GEMM3(TA_, TB_, 2, 2);              \
  } while (0)
  if (!ta && !tb) SL_GEMM(false, false);
  else if (!ta && tb) SL_GEMM(false, true);
  else if (ta && !tb) SL_GEMM(true, false);
  else SL_GEMM3(true, true, 2, 2);
#undef SL_GEMM3
#undef SL_GEMM
  int32_t rc = post_launch();
  if (rc || splits == 1) return rc;

  return splitk_combine(ctx, g, splits);
}

static bool overlaps(const float* a, size_t na, const float* b, size_t nb) {
  return a < b + nb && b < a + na;
}

}  // namespace slhip

using namespace slhip;

SLHIP_API int32_t slhip_sgemm(slhip_ctx* ctx, int32_t trans_a, int32_t trans_b, size_t m, size_t n, size_t k,
                              const float* a, const float* b, float* c, float beta) {
  size_t mk, kn, mn;
  SLHIP_REQUIRE(ctx && a && b && c, "null argument");
  SLHIP_REQUIRE(checked_len(m, k, &mk) && checked_len(k, n, &kn) && checked_len(m, n, &mn), "bad dims");
  if (overlaps(c, mn, a, mk) || overlaps(c, mn, b, kn)) {
    set_error("slhip_sgemm: C overlaps an input");
    return SLHIP_EALIAS;
  }
  return gemm_run(ctx, trans_a != 0, trans_b != 0, m, n, k, a, b, c, beta, nullptr, 0, nullptr, nullptr);
}

SLHIP_API int32_t slhip_sgemm_relu_mask(slhip_ctx* ctx, int32_t trans_a, int32_t trans_b, size_t m, size_t n, size_t k,
                                        const float* a, const float* b, const float* pre, float* c, float beta) {
  size_t mk, kn, mn;
  SLHIP_REQUIRE(ctx && a && b && c && pre, "null argument");
  SLHIP_REQUIRE(checked_len(m, k, &mk) && checked_len(k, n, &kn) && checked_len(m, n, &mn), "bad dims");
  if (overlaps(c, mn, a, mk) || overlaps(c, mn, b, kn) || overlaps(c, mn, pre, mn)) {
    set_error("slhip_sgemm_relu_mask: C overlaps an input");
    return SLHIP_EALIAS;
  }
  return gemm_run(ctx, trans_a != 0, trans_b != 0, m, n, k, a, b, c, beta, nullptr, 0, nullptr, pre);
}

SLHIP_API int32_t slhip_gemm_tail_policy(slhip_ctx* ctx, int32_t policy) {
  SLHIP_REQUIRE(ctx, "null argument");
  SLHIP_REQUIRE(policy == SLHIP_TAIL_AUTO || policy == SLHIP_TAIL_WHOLE || policy == SLHIP_TAIL_SPREAD, "unknown policy");
  ctx->gemm_tail = policy;
  return SLHIP_OK;
}

SLHIP_API int32_t slhip_gemm_tile_policy(slhip_ctx* ctx, int32_t policy) {
  SLHIP_REQUIRE(ctx, "null argument");
  SLHIP_REQUIRE(policy == SLHIP_TILE_AUTO || policy == SLHIP_TILE_128X128 || policy == SLHIP_TILE_64X64 ||
                    policy == SLHIP_TILE_128X128_WIDE,
                "unknown policy");
  ctx->gemm_tile = policy;
  return SLHIP_OK;
}

SLHIP_API int32_t slhip_gemm_plan_describe(slhip_ctx* ctx, char* buf, size_t len) {
  SLHIP_REQUIRE(ctx && buf && len > 0, "null argument");
  const slhip_ctx::GemmPlan& p = ctx->last_gemm;
  const char* tf[2] = {"false", "true"};
  switch (p.kind) {
    case 1:
      snprintf(buf, len, "gemm_wave_kernel<%s,%s,...,%s>: one wave per 32x32 tile, %u waves per workgroup, %u k splits, v_mfma_f32_32x32x2_f32",
               tf[p.ta], tf[p.tb], tf[p.only_fast], p.waves, p.splits);
      break;
    case 2:
    case 4:
      if (p.kind == 4 && p.waves == 8) {
        snprintf(buf, len, "gemm_spread_wide_kernel<%s,%s,%d,%s>: 128x128 tiles on 8 waves, BK=%d, %u k splits, v_mfma_f32_32x32x2_f32",
                 tf[p.ta], tf[p.tb], GEMM_BK, tf[p.only_fast], GEMM_BK, p.splits);
        break;
      }
      if (p.kind == 2 && p.small_tile && p.waves == 8) {
        snprintf(buf, len, "gemm_small8_kernel<%s,%s,%s>: 64x64 tiles on 8 waves (two sets of four, each half of every k tile), BK=%d, 1 k splits, v_mfma_f32_32x32x2_f32",
                 tf[p.ta], tf[p.tb], tf[p.only_fast], GEMM_BK);
        break;
      }
      snprintf(buf, len, "%s<%s,%s,%d,%s,%s>: %s tiles on 4 waves, BK=%d, %u k splits, v_mfma_f32_32x32x2_f32",
               p.kind == 4 ? "gemm_spread_kernel" : "gemm_kernel", tf[p.ta], tf[p.tb], GEMM_BK, tf[p.only_fast],
               p.small_tile ? "1,1" : "2,2", p.small_tile ? "64x64" : "128x128", GEMM_BK, p.splits);
      break;
    case 3:
      if (p.waves == 16)
        snprintf(buf, len, "gemm_wide16_kernel<%s,%s,%s>: 128x128 tiles on 16 waves (two sets of eight, each half of every k tile), BK=%d, 1 k splits, v_mfma_f32_32x32x2_f32",
                 tf[p.ta], tf[p.tb], tf[p.only_fast], GEMM_BK);
      else
        snprintf(buf, len, "gemm_wide_kernel<%s,%s,%s>: 128x128 tiles on 8 waves, BK=%d, %u k splits, v_mfma_f32_32x32x2_f32", tf[p.ta],
                 tf[p.tb], tf[p.only_fast], GEMM_BK, p.splits);
      break;
    case 5:
      snprintf(buf, len, "tall-A kernel (at most 32 columns), form %s,%s", tf[p.ta], tf[p.tb]);
      break;
    case 6:
      snprintf(buf, len, "skinny kernel (short K or narrow N), form %s,%s, %u k splits", tf[p.ta], tf[p.tb], p.splits);
      break;
    default:
      snprintf(buf, len, "no product has run on this context");
  }
  return SLHIP_OK;
}

SLHIP_API int32_t slhip_gemm(slhip_ctx* ctx, size_t m, size_t k, size_t n, const float* lhs, const float* rhs,
                             float* out) {
  return slhip_sgemm(ctx, 0, 0, m, n, k, lhs, rhs, out, 0.0f);
}

SLHIP_API int32_t slhip_gemm_grad(slhip_ctx* ctx, size_t m, size_t k, size_t n, const float* lhs, const float* rhs,
                                  float* lhs_grad, float* rhs_grad, const float* out_grad, float beta) {
  SLHIP_REQUIRE(ctx && lhs && rhs && out_grad, "null argument");
  // lhs_grad[m×k] = gemmT(m,k,n, out_grad, rhs): out_grad[m×n] · rhsᵀ, rhs stored k×n
  if (lhs_grad) {
    int32_t rc = slhip_sgemm(ctx, 0, 1, m, k, n, out_grad, rhs, lhs_grad, beta);
    if (rc) return rc;
  }
  // rhs_grad[k×n] = Tgemm(k,n,m, lhs, out_grad): lhsᵀ · out_grad, lhs stored m×k
  if (rhs_grad) {
    int32_t rc = slhip_sgemm(ctx, 1, 0, k, n, m, lhs, out_grad, rhs_grad, beta);
    if (rc) return rc;
  }
  return SLHIP_OK;
}

namespace slhip {

// Both gradient products (and the bias gradient) of a small layer as one launch of the pair
// kernel.  Returns false, with nothing launched, unless both products are small problems of the
// wave-per-tile kernel that need no k split and no skinny kernel would take either.
static bool linear_grad_pair(slhip_ctx* ctx, size_t m, size_t k, size_t n, const float* x, const float* w, float* x_grad,
                             const float* relu_pre, float* w_grad, float* bias_grad, const float* g, float beta, int32_t* rc) {
  if (!w_grad) return false;
  const size_t lim = size_t(1) << 18;  // below every skinny kernel's threshold
  if (m * k >= lim || k * n >= lim || m * n >= lim || 2.0 * (double)m * (double)k * (double)n > 33554432.0) return false;
  if (m == 0 || k == 0 || n == 0) return false;
  GemmArgs gx, gw;
  unsigned nwx = 1, nww = 1;
  size_t splits = 1, k_chunk = 0, tiles_x = 0;
  // x.grad[m x k] = g[m x n] * wT (w stored k x n)
  if (x_grad) {
    gx.M = m; gx.N = k; gx.K = n; gx.A = g; gx.B = w; gx.C = x_grad; gx.beta = beta;
    gx.bias = nullptr; gx.relu = 0; gx.pre_act = nullptr; gx.mask = relu_pre;
    gx.a_vec = n % 4 == 0; gx.b_vec = n % 4 == 0;
    gx.m_fast = 0; gx.partial = nullptr;
    wave_plan(ctx, m, k, n, &nwx, &splits, &k_chunk);
    if (splits != 1) return false;
    gx.splits = 1; gx.k_chunk = k_chunk;
    gx.tiles_m = (unsigned)((m + 31) / 32); gx.tiles_n = (unsigned)((k + 31) / 32);
    tiles_x = (size_t)gx.tiles_m * gx.tiles_n;
  } else {
    gx = GemmArgs();
  }
  // w.grad[k x n] = xT * g (x stored m x k)
  gw.M = k; gw.N = n; gw.K = m; gw.A = x; gw.B = g; gw.C = w_grad; gw.beta = beta;
  gw.bias = nullptr; gw.relu = 0; gw.pre_act = nullptr; gw.mask = nullptr;
  gw.a_vec = k % 4 == 0; gw.b_vec = n % 4 == 0;
  gw.m_fast = 0; gw.partial = nullptr;
  wave_plan(ctx, k, n, m, &nww, &splits, &k_chunk);
  if (splits != 1 || nwx > 8 || nww > 8) return false;
  gw.splits = 1; gw.k_chunk = k_chunk;
  gw.tiles_m = (unsigned)((k + 31) / 32); gw.tiles_n = (unsigned)((n + 31) / 32);
  const size_t tiles_w = (size_t)gw.tiles_m * gw.tiles_n;
  // the unchecked form of each product, as gemm_run decides it: at least one whole group of 8 k
  const bool fullx = n >= 8, fullw = m >= 8;
  const unsigned nw = nwx > nww ? nwx : nww;
  const size_t lds = nw > 1 ? ((size_t)nw * 16 * 64 + (size_t)nw * 32) * sizeof(float) : 0;
  const dim3 grid((unsigned)(tiles_x + tiles_w));
#define SL_PAIR(FX_, FW_)                                                                                                \
  hipLaunchKernelGGL((gemm_wave_pair_kernel<FX_, FW_>), grid, dim3(64 * nw), lds, ctx->stream, gx, gw, bias_grad, (unsigned)tiles_x, \
                     (int)nwx, (int)nww)
  if (fullx && fullw) SL_PAIR(true, true);
  else if (fullx) SL_PAIR(true, false);
  else if (fullw) SL_PAIR(false, true);
  else SL_PAIR(false, false);
#undef SL_PAIR
  *rc = post_launch();
  return true;
}

}  // namespace slhip

SLHIP_API int32_t slhip_linear_grad(slhip_ctx* ctx, size_t m, size_t k, size_t n, const float* x, const float* w, float* x_grad,
                                    const float* relu_pre, float* w_grad, float* bias_grad, const float* out_grad, float beta) {
  size_t mk, kn, mn;
  SLHIP_REQUIRE(ctx && x && w && out_grad, "null argument");
  SLHIP_REQUIRE(checked_len(m, k, &mk) && checked_len(k, n, &kn) && checked_len(m, n, &mn), "bad dims");
  SLHIP_REQUIRE(!relu_pre || x_grad, "a ReLU mask without x_grad");
  if ((x_grad && (overlaps(x_grad, mk, out_grad, mn) || overlaps(x_grad, mk, w, kn) || overlaps(x_grad, mk, x, mk))) ||
      (w_grad && (overlaps(w_grad, kn, out_grad, mn) || overlaps(w_grad, kn, x, mk) || overlaps(w_grad, kn, w, kn))) ||
      (bias_grad && overlaps(bias_grad, n, out_grad, mn))) {
    set_error("slhip_linear_grad: a gradient overlaps an input");
    return SLHIP_EALIAS;
  }
  int32_t rc = SLHIP_OK;
  if (linear_grad_pair(ctx, m, k, n, x, w, x_grad, relu_pre, w_grad, bias_grad, out_grad, beta, &rc)) return rc;
  // the same three results op by op, in the order the tape's own closures run them
  if (bias_grad) {
    rc = slhip_add_row_mut_grad(ctx, m, n, bias_grad, out_grad);
    if (rc) return rc;
  }
  if (x_grad) {
    rc = relu_pre ? slhip_sgemm_relu_mask(ctx, 0, 1, m, k, n, out_grad, w, relu_pre, x_grad, beta)
                  : slhip_sgemm(ctx, 0, 1, m, k, n, out_grad, w, x_grad, beta);
    if (rc) return rc;
  }
  if (w_grad) rc = slhip_sgemm(ctx, 1, 0, k, n, m, x, out_grad, w_grad, beta);
  return rc;
}

SLHIP_API int32_t slhip_linear_fwd(slhip_ctx* ctx, size_t m, size_t k, size_t n, const float* x, const float* w,
                                   const float* bias, int32_t relu, float* pre_act, float* out) {
  size_t mk, kn, mn;
  SLHIP_REQUIRE(ctx && x && w && out, "null argument");
  SLHIP_REQUIRE(checked_len(m, k, &mk) && checked_len(k, n, &kn) && checked_len(m, n, &mn), "bad dims");
  if (overlaps(out, mn, x, mk) || overlaps(out, mn, w, kn)) {
    set_error("slhip_linear_fwd: out overlaps an input");
    return SLHIP_EALIAS;
  }
  return gemm_run(ctx, false, false, m, n, k, x, w, out, 0.0f, bias, relu != 0, pre_act, nullptr);
}
