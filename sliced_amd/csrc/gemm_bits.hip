// The ReLU mask as one bit per element.  A fused Linear's backward needs the pre-activations of
// the layer below only for their sign; as floats they are written once by the forward pass and
// read once by the input-gradient GEMM, 4 B each way per element, and that read sits at the very
// end of a workgroup's life where nothing hides it (35-57 us per 64 MiB at batch 8192).  Here the
// forward kernel writes the mask (pre >= 0) packed 32 columns to a word, row-major
// [M][ceil(N / 32)], and the masked GEMM fetches the 128 words of its tile BEFORE its k loop:
// four registers a lane, no latency left at the end.
//
// Both kernels are the 128 x 128 tile kernel of gemm.hip with another epilogue; they live in a
// file of their own so that the plain kernel's code stays exactly as it is.  One workgroup per
// tile, no K split: meant for outputs of a few hundred tiles and more (the caller decides).
// A masked product with K <= 12 goes to the short-K vector kernel (gemm_skinny.hip) instead.
//
// Packing.  In accumulator block (i, j) of a wave, register v of lane (r, h) is row
// 8*(v/4) + 4*h + v%4 and column r of a 32 x 32 block: a wave-wide ballot of one register is the
// mask word of two rows (low half: h = 0, high half: h = 1).  Lane L < 32 keeps the word of row L
// of the block, so a block's words leave (and arrive) as one access of 32 lanes.
#include <type_traits>

#include "gemm_tile.hpp"

namespace slhip {

__host__ __device__ constexpr int bits_row_of(int v, int h) { return 8 * (v / 4) + 4 * h + v % 4; }

// WM x WN accumulator blocks per wave, WGM x WGN waves: 2, 2, 2, 2 is the four-wave tile; 2, 1, 2, 4 the eight-wave
// one (as gemm_wide_kernel: two such workgroups put four waves on a SIMD).
template <bool TA, bool TB, bool ONLY_FAST, int WM = 2, int WN = 2, int WGM = 2, int WGN = 2>
__global__ __launch_bounds__(64 * WGM * WGN, 2) void gemm_bits_kernel(GemmArgs g, const uint32_t* __restrict__ bits_in,
                                                           uint32_t* __restrict__ bits_out, size_t W) {
  constexpr int BK = GEMM_BK;
  static_assert(32 * WM * WGM == 128 && 32 * WN * WGN == 128, "a 128 x 128 tile");
  __shared__ __attribute__((aligned(16))) float lds_a[2][Cfg<BK, 128>::STAGE_FLOATS];
  __shared__ __attribute__((aligned(16))) float lds_b[2][Cfg<BK, 128>::STAGE_FLOATS];
  unsigned tm, tn;
  tile_of_block(blockIdx.x, g.tiles_m, g.tiles_n, tm, tn);
  const size_t m0 = (size_t)tm * 128, n0 = (size_t)tn * 128;
  const int ktiles = (int)((g.K + BK - 1) / BK);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = wave / WGN, wn = wave % WGN;
  const int r = lane & 31, h = lane >> 5;

  // the tile's mask words, in flight during the k loop
  uint32_t mw[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j) mw[i][j] = 0u;
  if (bits_in) {
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int j = 0; j < WN; ++j) {
        const size_t row = m0 + block_of<WGM>(wm, i) + r, cw = (n0 + block_of<WGN>(wn, j)) >> 5;
        if (h == 0 && row < g.M && cw < W) mw[i][j] = bits_in[row * W + cw];
      }
  }

  floatx16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
  gemm_k_range<TA, TB, BK, ONLY_FAST, WM, WN, WGM, WGN>(g, 0, ktiles, 0, g.K, m0, n0, lds_a, lds_b, acc);

  // Tiles inside the matrix with nothing to read back (every tile of a layer whose sides are multiples of
  // 128): no bounds, one scalar row pointer per accumulator register and one 32-bit lane offset for all of
  // them, the flags tested once.  The general form below spends some thirty-five instructions per element
  // on 64-bit index products, bounds and flag tests - 5 us per round of workgroups, which all reach their
  // epilogue together (8192 x 2048 x 2048, launches back to back: forward 497 -> 488 us, masked input
  // gradient 494 -> 484, the plain product 486 / 484; inside a training step, where the result's lines are
  // not in the caches yet and the stores set the pace, the same kernels gain 2 us each).
  if (m0 + 128 <= g.M && n0 + 128 <= g.N && g.beta == 0.0f && g.N < (size_t(1) << 28) && (bits_in == nullptr) != (bits_out == nullptr)) {
    const int uw = __builtin_amdgcn_readfirstlane(wave);
    const int uwm = uw / WGN, uwn = uw % WGN;
    const unsigned lane_off = (unsigned)(4 * h) * (unsigned)g.N + (unsigned)r;
    auto run = [&](auto in_tag) {
      constexpr bool IN = decltype(in_tag)::value;  // the mask comes in (input gradient); else it goes out (forward)
      float bias_of[WN];
#pragma unroll
      for (int j = 0; j < WN; ++j) bias_of[j] = 0.0f;
      if (!IN && g.bias) {
#pragma unroll
        for (int j = 0; j < WN; ++j) bias_of[j] = g.bias[n0 + block_of<WGN>(wn, j) + r];
      }
      const bool relu = g.relu != 0;
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j) {
          float* const block = g.C + (m0 + block_of<WGM>(uwm, i)) * g.N + n0 + block_of<WGN>(uwn, j);  // wave-uniform
          uint32_t word = 0u;
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            float val = acc[i][j][v];
            if (IN) {
              const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)mw[i][j], bits_row_of(v, 0));
              const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)mw[i][j], bits_row_of(v, 1));
              val = ((((h ? hi : lo) >> r) & 1u) ? 1.0f : 0.0f) * val;
            } else {
              val = val + bias_of[j];  // (0 without a bias: x + 0 = x for every x the product can hold but -0, whose sign no reader sees)
              const unsigned long long b = __ballot(val >= 0.0f);
              if (lane == bits_row_of(v, 0)) word = (uint32_t)b;
              if (lane == bits_row_of(v, 1)) word = (uint32_t)(b >> 32);
              const float rl = (val >= 0.0f ? 1.0f : 0.0f) * val;
              val = relu ? rl : val;
            }
            (block + (size_t)(8 * (v / 4) + v % 4) * g.N)[lane_off] = val;
          }
          if (!IN && h == 0) bits_out[(m0 + block_of<WGM>(wm, i) + r) * W + ((n0 + block_of<WGN>(wn, j)) >> 5)] = word;
        }
    };
    if (bits_in) run(std::true_type());
    else run(std::false_type());
    return;
  }

  // every read (mask words, C for beta) before the first store
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      const size_t col = n0 + block_of<WGN>(wn, j) + r;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        float val = acc[i][j][v];
        if (bits_in) {
          const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)mw[i][j], bits_row_of(v, 0));
          const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)mw[i][j], bits_row_of(v, 1));
          val = ((((h ? hi : lo) >> r) & 1u) ? 1.0f : 0.0f) * val;
        }
        if (g.beta != 0.0f) {
          const size_t row = m0 + block_of<WGM>(wm, i) + bits_row_of(v, h);
          if (row < g.M && col < g.N) val = g.beta * g.C[row * g.N + col] + val;
        }
        acc[i][j][v] = val;
      }
    }
  float bias_of[WN];
#pragma unroll
  for (int j = 0; j < WN; ++j) bias_of[j] = 0.0f;
  if (g.bias) {
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      const size_t col = n0 + block_of<WGN>(wn, j) + r;
      if (col < g.N) bias_of[j] = g.bias[col];
    }
  }
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      const size_t col = n0 + block_of<WGN>(wn, j) + r;
      const bool cin = col < g.N;
      const float bias = bias_of[j];
      uint32_t word = 0u;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        float val = acc[i][j][v];
        if (g.bias) val = val + bias;
        if (bits_out) {
          const unsigned long long b = __ballot(val >= 0.0f && cin);
          if (lane == bits_row_of(v, 0)) word = (uint32_t)b;
          if (lane == bits_row_of(v, 1)) word = (uint32_t)(b >> 32);
        }
        if (g.relu) val = (val >= 0.0f ? 1.0f : 0.0f) * val;
        const size_t row = m0 + block_of<WGM>(wm, i) + bits_row_of(v, h);
        if (row < g.M && cin) g.C[row * g.N + col] = val;
      }
      if (bits_out) {
        const size_t row = m0 + block_of<WGM>(wm, i) + r, cw = (n0 + block_of<WGN>(wn, j)) >> 5;
        if (h == 0 && row < g.M && cw < W) bits_out[row * W + cw] = word;
      }
    }
}

// Products the tiled kernel's loads are not written for: an output side of at most 32 or K of at most
// 16 (its clamped vector loads assume an x-contiguous operand at least one float4 wide, and the plain
// GEMM keeps such shapes away from it as well).  One lane per element of C, 64 columns of one row per
// wave, the k range walked in order: slow and safe - nothing that trains a layer this narrow keeps
// its mask as bits, but the entry points accept the shapes.
template <bool TA, bool TB>
__global__ __launch_bounds__(64) void gemm_bits_small_kernel(GemmArgs g, const uint32_t* __restrict__ bits_in,
                                                             uint32_t* __restrict__ bits_out, size_t W) {
  const size_t cblocks = (g.N + 63) / 64;
  const size_t row = blockIdx.x / cblocks, cb = blockIdx.x % cblocks;
  const int lane = threadIdx.x;
  const size_t col = cb * 64 + lane;
  const bool in = col < g.N;
  const size_t cc = in ? col : g.N - 1;
  const float* ap = TA ? g.A + row : g.A + row * g.K;
  const float* bp = TB ? g.B + cc * g.K : g.B + cc;
  const size_t astep = TA ? g.M : 1, bstep = TB ? 1 : g.N;
  float val = 0.0f;
  for (size_t k = 0; k < g.K; ++k) val = val + ap[k * astep] * bp[k * bstep];
  if (bits_in) val = (((bits_in[row * W + (cc >> 5)] >> (cc & 31)) & 1u) ? 1.0f : 0.0f) * val;
  if (g.beta != 0.0f && in) val = g.beta * g.C[row * g.N + col] + val;
  if (g.bias) val = val + g.bias[cc];
  if (bits_out) {
    const unsigned long long b = __ballot(val >= 0.0f && in);
    const size_t cw = cb * 2 + (lane >> 5);
    if ((lane & 31) == 0 && cw < W) bits_out[row * W + cw] = (uint32_t)(lane ? b >> 32 : b);
  }
  if (g.relu) val = (val >= 0.0f ? 1.0f : 0.0f) * val;
  if (in) g.C[row * g.N + col] = val;
}

// x_grad += bit * out_grad: the ReLU gradient (src/matrix.rs:190-199) from the packed mask.  One
// vector of four elements per thread over the flat matrix; a thread finds the row and column of
// its first element with one division and steps from there (any row length).
template <class IDX>
__global__ __launch_bounds__(256) void relu_grad_bits_kernel(size_t rows, size_t cols, size_t W, const uint32_t* __restrict__ bits,
                                                             float* x_grad, const float* __restrict__ out_grad) {
  const size_t n = rows * cols;
  const size_t e0 = 4 * ((size_t)blockIdx.x * 256 + threadIdx.x);
  if (e0 >= n) return;
  IDX r = (IDX)e0 / (IDX)cols;
  IDX c = (IDX)e0 - r * (IDX)cols;
  const bool whole = e0 + 3 < n;
  float g[4] = {0.f, 0.f, 0.f, 0.f}, o[4] = {0.f, 0.f, 0.f, 0.f};
  if (whole) {
    float4 t = ld4s(out_grad + e0);
    g[0] = t.x; g[1] = t.y; g[2] = t.z; g[3] = t.w;
    t = ld4g(x_grad + e0);
    o[0] = t.x; o[1] = t.y; o[2] = t.z; o[3] = t.w;
  } else {
    for (size_t q = 0; e0 + q < n; ++q) { g[q] = out_grad[e0 + q]; o[q] = x_grad[e0 + q]; }
  }
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    if (e0 + q < n) {
      const uint32_t bit = (bits[(size_t)r * W + (c >> 5)] >> (c & 31)) & 1u;
      o[q] = o[q] + (bit ? 1.0f : 0.0f) * g[q];
    }
    if (++c == (IDX)cols) { c = 0; ++r; }
  }
  if (whole) st4g(x_grad + e0, make_float4(o[0], o[1], o[2], o[3]));
  else
    for (size_t q = 0; e0 + q < n; ++q) x_grad[e0 + q] = o[q];
}

static int32_t gemm_bits_run(slhip_ctx* ctx, bool ta, bool tb, size_t M, size_t N, size_t K, const float* A, const float* B,
                             float* C, float beta, const float* bias, int relu, const uint32_t* bits_in, uint32_t* bits_out) {
  GemmArgs g;
  g.M = M; g.N = N; g.K = K; g.A = A; g.B = B; g.C = C; g.beta = beta;
  g.bias = bias; g.relu = relu; g.pre_act = nullptr; g.mask = nullptr;
  const size_t lda = ta ? M : K, ldb = tb ? K : N;
  g.a_vec = lda % 4 == 0;
  g.b_vec = ldb % 4 == 0;
  g.m_fast = (aligned16(A) && aligned16(B) && lda < (size_t(1) << 22) && ldb < (size_t(1) << 22)) ? M : 0;  // 32-bit tile offsets
  g.partial = nullptr;
  const size_t tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  if (tiles_m * tiles_n > 0x7fffffffu) {
    set_error("gemm with bit mask: %zu x %zu tiles exceed one launch", tiles_m, tiles_n);
    return SLHIP_EINVAL;
  }
  g.tiles_m = (unsigned)tiles_m; g.tiles_n = (unsigned)tiles_n;
  g.splits = 1;
  g.k_chunk = (K + GEMM_BK - 1) / GEMM_BK * GEMM_BK;
  if (bits_in && !bits_out) {  // K <= 12: HBM-bound, the vector kernel reads the same words (8192 x 2048 x 10: 32 -> 16 us)
    int32_t rc = SLHIP_OK;
    if (gemm_short_k_launch(ctx, ta, tb, g, bits_in, &rc)) return rc;
  }
  const size_t W = (N + 31) / 32;
  if (M <= 32 || N <= 32 || K <= 16) {
    const size_t blocks = M * ((N + 63) / 64);
    if (blocks > 0x7fffffffu) {
      set_error("gemm with bit mask: %zu x %zu is too large for the narrow-shape kernel", M, N);
      return SLHIP_EINVAL;
    }
#define SL_GBS(TA_, TB_) \
  hipLaunchKernelGGL((gemm_bits_small_kernel<TA_, TB_>), dim3((unsigned)blocks), dim3(64), 0, ctx->stream, g, bits_in, bits_out, W)
    if (!ta && !tb) SL_GBS(false, false);
    else if (!ta && tb) SL_GBS(false, true);
    else if (ta && !tb) SL_GBS(true, false);
    else SL_GBS(true, true);
#undef SL_GBS
    return post_launch();
  }
  const bool only_fast = g.a_vec && g.b_vec && g.m_fast && M % BM == 0 && N % BN == 0 && K % GEMM_BK == 0;
  const dim3 grid((unsigned)(tiles_m * tiles_n));
#define SL_GB(TA_, TB_)                                                                                                      \
  do {                                                                                                                       \
    if (only_fast) hipLaunchKernelGGL((gemm_bits_kernel<TA_, TB_, true>), grid, dim3(256), 0, ctx->stream, g, bits_in, bits_out, W); \
    else hipLaunchKernelGGL((gemm_bits_kernel<TA_, TB_, false>), grid, dim3(256), 0, ctx->stream, g, bits_in, bits_out, W);  \
  } while (0)
#define SL_GBW(TA_, TB_)                                                                                                     \
  do {                                                                                                                       \
    if (only_fast)                                                                                                           \
      hipLaunchKernelGGL((gemm_bits_kernel<TA_, TB_, true, 2, 1, 2, 4>), grid, dim3(512), 0, ctx->stream, g, bits_in, bits_out, W);  \
    else                                                                                                                     \
      hipLaunchKernelGGL((gemm_bits_kernel<TA_, TB_, false, 2, 1, 2, 4>), grid, dim3(512), 0, ctx->stream, g, bits_in, bits_out, W); \
  } while (0)
  const bool four = ctx->gemm_tile == SLHIP_TILE_128X128;  // the tile policy's four-wave form, for comparison
  if (!ta && !tb) { if (four) SL_GB(false, false); else SL_GBW(false, false); }
  else if (!ta && tb) { if (four) SL_GB(false, true); else SL_GBW(false, true); }
  else if (ta && !tb) { if (four) SL_GB(true, false); else SL_GBW(true, false); }
  else SL_GB(true, true);
#undef SL_GB
#undef SL_GBW
  return post_launch();
}

static bool overlaps_bytes(const void* a, size_t na, const void* b, size_t nb) {
  const char* p = (const char*)a;
  const char* q = (const char*)b;
  return p < q + nb && q < p + na;
}

}  // namespace slhip

using namespace slhip;

SLHIP_API int32_t slhip_linear_fwd_bits(slhip_ctx* ctx, size_t m, size_t k, size_t n, const float* x, const float* w,
                                        const float* bias, uint32_t* bits, float* out) {
  size_t mk, kn, mn;
  SLHIP_REQUIRE(ctx && x && w && bits && out, "null argument");
  SLHIP_REQUIRE(checked_len(m, k, &mk) && checked_len(k, n, &kn) && checked_len(m, n, &mn), "bad dims");
  const size_t words = m * ((n + 31) / 32);
  if (overlaps_bytes(out, mn * 4, x, mk * 4) || overlaps_bytes(out, mn * 4, w, kn * 4) || overlaps_bytes(bits, words * 4, out, mn * 4) ||
      overlaps_bytes(bits, words * 4, x, mk * 4) || overlaps_bytes(bits, words * 4, w, kn * 4)) {
    set_error("slhip_linear_fwd_bits: an output overlaps another operand");
    return SLHIP_EALIAS;
  }
  return gemm_bits_run(ctx, false, false, m, n, k, x, w, out, 0.0f, bias, 1, nullptr, bits);
}

SLHIP_API int32_t slhip_sgemm_relu_bits(slhip_ctx* ctx, int32_t trans_a, int32_t trans_b, size_t m, size_t n, size_t k,
                                        const float* a, const float* b, const uint32_t* bits, float* c, float beta) {
  size_t mk, kn, mn;
  SLHIP_REQUIRE(ctx && a && b && c && bits, "null argument");
  SLHIP_REQUIRE(checked_len(m, k, &mk) && checked_len(k, n, &kn) && checked_len(m, n, &mn), "bad dims");
  const size_t words = m * ((n + 31) / 32);
  if (overlaps_bytes(c, mn * 4, a, mk * 4) || overlaps_bytes(c, mn * 4, b, kn * 4) || overlaps_bytes(c, mn * 4, bits, words * 4)) {
    set_error("slhip_sgemm_relu_bits: C overlaps an input");
    return SLHIP_EALIAS;
  }
  return gemm_bits_run(ctx, trans_a != 0, trans_b != 0, m, n, k, a, b, c, beta, nullptr, 0, bits, nullptr);
}

SLHIP_API int32_t slhip_relu_grad_bits(slhip_ctx* ctx, size_t rows, size_t cols, const uint32_t* bits, float* x_grad,
                                       const float* out_grad) {
  size_t len;
  SLHIP_REQUIRE(ctx && bits && x_grad && out_grad, "null argument");
  SLHIP_REQUIRE(checked_len(rows, cols, &len), "bad dims");
  const size_t blocks = ((len + 3) / 4 + 255) / 256;
  SLHIP_REQUIRE(blocks <= 0x7fffffffu, "too many elements for one launch");
  if (len <= 0xffffffffu)
    hipLaunchKernelGGL((relu_grad_bits_kernel<uint32_t>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, rows, cols,
                       (cols + 31) / 32, bits, x_grad, out_grad);
  else
    hipLaunchKernelGGL((relu_grad_bits_kernel<size_t>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, rows, cols,
                       (cols + 31) / 32, bits, x_grad, out_grad);
  return post_launch();
}
