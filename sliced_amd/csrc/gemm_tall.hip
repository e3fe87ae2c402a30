// Products of one large operand that is read once and a B of at most 32 columns, on the matrix
// instructions: C = A * B and A * Bt for a tall A stored M x K (K a multiple of 4), and - second
// kernel, further down - At * B for an A stored K x M.
//
// Tall A: a wave owns 32 rows of A and the whole 32 x 32 block of C.  Per step it takes 64 k: its 32 x 64
// block of A comes in with eight loads per lane that each read 256 contiguous bytes of four rows,
// goes through a wave-private LDS block and comes back as the instruction's A operand; B waits in
// the workspace as Bt[32][K'] (column-major, zero beyond N and K) and its 32 x 64 block takes
// the same route through a block of LDS that the workgroup's four waves fill and read together
// (a lane that fetched its 128 bytes of Bt itself touched 64 cache lines per load instruction:
// 3.4-3.9 TB/s).  The instruction's k index is
// ours to assign, as long as both operands agree: lane (r, h) feeds k = 32 h + 4 j + t at issue
// (j, t), which makes both operands whole float4.  The next step's loads are requested before
// the current step's 32 instructions run.  Few rows: workgroups split K and the split-K combine
// finishes.
//
// Measured on 1 GiB of A (16384 x N x 16384, pack and combine launches included): 180-183 us for
// N up to 16 (5.9-6.0 TB/s of A) on the 16 x 16 x 4 instruction, 213-240 us for 17..32 columns
// (4.5-5.0 TB/s) on the 32 x 32 x 2 one, where the matrix pipes are busy 61 % of the time a CU holds
// the kernel and a CU holds it 77 % of the kernel's time (every workgroup is resident at once, and
// they do not finish together).  Loading B as it is stored instead of packing it first (four scalar
// loads per lane and step) saved the pack launch and cost more than that: 32 columns 225 -> 261 us.
#include "gemm_tile.hpp"

namespace slhip {

constexpr int TALL_KC = 64;             // k per wave and step
constexpr int TALL_PITCH = TALL_KC + 4; // floats per LDS row: rows 8 apart share banks, which a b128 read of 32 lanes needs anyway
constexpr int TALL_ROWS = 128;          // rows of A per workgroup (four waves)

// Bt[c][k] = B[k][c] (or B[c][k] for a B stored N x K), zero for c >= N and k >= K.
__global__ __launch_bounds__(256) void tall_pack_b_kernel(size_t K, size_t Kp, int N, int tb, const float* __restrict__ B,
                                                          float* __restrict__ Bt) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= 32 * Kp) return;
  const size_t c = i / Kp, k = i - c * Kp;
  float v = 0.0f;
  if (c < (size_t)N && k < K) v = tb ? B[c * K + k] : B[k * (size_t)N + c];
  Bt[i] = v;
}

typedef float floatx4 __attribute__((ext_vector_type(4)));

// N16: B has at most 16 columns.  The wave's 32 rows are then two blocks of 16 rows on the
// 16 x 16 x 4 instruction (half the matrix-pipe time per byte of A: a 32-column instruction with 16
// columns of zeros in it is the bound from 13 columns on), lane (r, q) = (lane % 16, lane / 16)
// feeds k = 16 q + 4 j + t at issue (j, t), and only 16 rows of Bt are staged.
template <bool N16>
__global__ __launch_bounds__(256) void gemm_tall_kernel(GemmArgs g, const float* __restrict__ Bt, size_t Kp) {
  // [4 waves][32][TALL_PITCH] of A, wave-private, then [2][32][TALL_PITCH] of Bt, shared by the four waves
  extern __shared__ __attribute__((aligned(16))) float tall_lds[];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int r = N16 ? lane & 15 : lane & 31, h = N16 ? lane >> 4 : lane >> 5;
  constexpr int KL = N16 ? 16 : 32;  // k per lane group and step
  constexpr int NJ = KL / 4;         // float4 per operand row, lane and step
  float* blk = tall_lds + w * 32 * TALL_PITCH;
  float* bblk = tall_lds + 4 * 32 * TALL_PITCH;
  const size_t M = g.M, K = g.K;
  const int N = (int)g.N;
  const size_t m0 = ((size_t)blockIdx.x * 4 + w) * 32;  // (a wave wholly past the edge works on copies of the last row)
  const size_t chunks = (K + TALL_KC - 1) / TALL_KC;
  const size_t per_y = (chunks + gridDim.y - 1) / gridDim.y;
  const size_t cbeg = (size_t)blockIdx.y * per_y;
  const size_t cend = cbeg + per_y < chunks ? cbeg + per_y : chunks;

  // load side: lane l takes the float4 at column 4 * (l % 16) of rows 4 p + l / 16 (p = 0..7) of
  // the wave's block of A, and of rows 8 w + 4 q + l / 16 (q = 0, 1; N16: rows 4 w + l / 16) of the
  // block of Bt
  constexpr int NB = N16 ? 1 : 2;
  const int lrow = lane >> 4, lcol = 4 * (lane & 15);
  const float* arow[8];
#pragma unroll
  for (int p = 0; p < 8; ++p) {
    const size_t row = m0 + 4 * p + lrow;
    arow[p] = g.A + (row < M ? row : M - 1) * K;  // rows past the edge: copies that are never stored
  }
  int bstage[NB];
  const float* brow[NB];
#pragma unroll
  for (int q = 0; q < NB; ++q) {
    bstage[q] = N16 ? 4 * w + lrow : 8 * w + 4 * q + lrow;
    brow[q] = Bt + (size_t)bstage[q] * Kp + lcol;
  }

  floatx16 acc;
  floatx4 acc4[2];
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
#pragma unroll
  for (int v = 0; v < 4; ++v) acc4[0][v] = acc4[1][v] = 0.0f;

  // two steps' loads are in flight at any time: set u holds the steps cbeg + u, cbeg + u + 2, ...
  float4 a[2][8], b[2][NB];
  auto request = [&](size_t ch, float4 (&as)[8], float4 (&bs)[NB]) {
    const size_t k0 = ch * TALL_KC;
    const size_t k = k0 + lcol;
    // K is a multiple of 4: a vector lies inside the row or wholly beyond it (then it is zeroed below)
    const size_t kc = k < K ? k : K - 4;
#pragma unroll
    for (int p = 0; p < 8; ++p) as[p] = ld4s(arow[p] + kc);
#pragma unroll
    for (int q = 0; q < NB; ++q) bs[q] = ld4g(brow[q] + k0);
  };
  if (cbeg < cend) request(cbeg, a[0], b[0]);
  if (cbeg + 1 < cend) request(cbeg + 1, a[1], b[1]);
  for (size_t ch0 = cbeg; ch0 < cend; ch0 += 2) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const size_t ch = ch0 + u;
      if (ch >= cend) break;  // the same for every wave of the workgroup
      const bool beyond = ch * TALL_KC + lcol >= K;
      float* bb = bblk + u * 32 * TALL_PITCH;
#pragma unroll
      for (int p = 0; p < 8; ++p) {
        const float4 v = beyond ? make_float4(0.f, 0.f, 0.f, 0.f) : a[u][p];
        st4(blk + (4 * p + lrow) * TALL_PITCH + lcol, v);
      }
#pragma unroll
      for (int q = 0; q < NB; ++q) st4(bb + bstage[q] * TALL_PITCH + lcol, b[u][q]);
      // one barrier per step: the other half of the Bt buffer is written in the next step, which a
      // wave enters only after every wave has passed this barrier and so has read that half
      __syncthreads();
      if (ch + 2 < cend) request(ch + 2, a[u], b[u]);
      if constexpr (N16) {
        float4 av[2][NJ], bv[NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
          av[0][j] = ld4(blk + r * TALL_PITCH + KL * h + 4 * j);
          av[1][j] = ld4(blk + (16 + r) * TALL_PITCH + KL * h + 4 * j);
          bv[j] = ld4(bb + r * TALL_PITCH + KL * h + 4 * j);
        }
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
          acc4[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[0][j].x, bv[j].x, acc4[0], 0, 0, 0);
          acc4[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[1][j].x, bv[j].x, acc4[1], 0, 0, 0);
          acc4[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[0][j].y, bv[j].y, acc4[0], 0, 0, 0);
          acc4[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[1][j].y, bv[j].y, acc4[1], 0, 0, 0);
          acc4[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[0][j].z, bv[j].z, acc4[0], 0, 0, 0);
          acc4[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[1][j].z, bv[j].z, acc4[1], 0, 0, 0);
          acc4[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[0][j].w, bv[j].w, acc4[0], 0, 0, 0);
          acc4[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[1][j].w, bv[j].w, acc4[1], 0, 0, 0);
        }
      } else {
        float4 av[NJ], bv[NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
          av[j] = ld4(blk + r * TALL_PITCH + KL * h + 4 * j);
          bv[j] = ld4(bb + r * TALL_PITCH + KL * h + 4 * j);
        }
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[j].x, bv[j].x, acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[j].y, bv[j].y, acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[j].z, bv[j].z, acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[j].w, bv[j].w, acc, 0, 0, 0);
        }
      }
    }
  }
  if (m0 >= M) return;

  // 32 columns: register v of lane (r, h) is row 8 * (v / 4) + 4 * h + v % 4 of the wave's block,
  // column r; 16 columns: register v of block hh is row 16 * hh + 4 * h + v, column r
  if (r >= N) return;
  constexpr int NV = N16 ? 8 : 16;
  auto row_of = [&](int v) -> size_t { return m0 + (N16 ? 16 * (v / 4) + 4 * h + (v % 4) : 8 * (v / 4) + 4 * h + (v % 4)); };
  const bool raw = gridDim.y > 1;
  float* dst = raw ? g.partial + (size_t)blockIdx.y * M * (size_t)N : g.C;
  float val[NV], old[NV], msk[NV];
  const bool with_mask = !raw && g.mask != nullptr, with_c = !raw && g.beta != 0.0f;
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const size_t row = row_of(v);
    const size_t at = row * (size_t)N + r;
    msk[v] = with_mask && row < M ? g.mask[at] : 0.0f;
    old[v] = with_c && row < M ? g.C[at] : 0.0f;
  }
  const float bias = !raw && g.bias ? g.bias[r] : 0.0f;
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    float x;
    if constexpr (N16) x = acc4[(v / 4) & 1][v % 4];
    else x = acc[v];
    if (with_mask) x = (msk[v] >= 0.0f ? 1.0f : 0.0f) * x;
    if (with_c) x = g.beta * old[v] + x;
    if (!raw && g.bias) x = x + bias;
    val[v] = x;
  }
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const size_t row = row_of(v);
    if (row >= M) continue;
    const size_t at = row * (size_t)N + r;
    float x = val[v];
    if (!raw) {
      if (g.pre_act) g.pre_act[at] = x;
      if (g.relu) x = (x >= 0.0f ? 1.0f : 0.0f) * x;
    }
    dst[at] = x;
  }
}

// C = At * B for an A stored K x M (the large operand: read once) and a B of at most 32 columns, stored
// K x N or N x K: the weight gradient of a narrow layer.  Both operands go from global memory straight into
// the 16 x 16 x 4 instruction, no LDS on the way: lane (i, kk) = (lane % 16, lane / 16) loads the
// float4 A[k0 + kk][m0 + 4 i .. + 3] - a wave's load instruction reads 256 contiguous bytes of four
// k rows - and component t of it is the A operand of the t-th of four instructions, whose block of C
// is therefore the rows m0 + 4 i + t, i = 0..15; the B operand of all four is B[k0 + kk][lane % 16].
// A workgroup owns 64 columns of A (rows of C) and one share of K; its four waves take the steps of
// four k in turn and add up through LDS, wave 0 first; shares of K combine in the split-K kernel.
// (Combining in the same launch - the workgroup that draws a row block's last ticket adds the
// shares up - was built and measured: the device-scope release it needs costs more than the second
// launch, 2048 x 10 x 8192 19 -> 29 us with one fence per workgroup over write-through stores, 81 us
// with one per wave.)
constexpr int TT_STEPS = 8;  // loads in flight per wave: 8 KiB of A

template <int NB>
__global__ __launch_bounds__(256) void gemm_tall_t_kernel(GemmArgs g, size_t k_share, int tb) {
  // NB = 1: at most 16 columns; NB = 2: 17..32, a second block of 16 columns on the same loads of A
  __shared__ __attribute__((aligned(16))) float part[3][64][16 * NB + 1];  // waves 1..3: [lane][accumulators], padded
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int i = lane & 15, kk = lane >> 4;
  const size_t M = g.M, K = g.K;
  const int N = (int)g.N;
  const size_t m0 = (size_t)blockIdx.x * 64;
  const size_t kbeg = (size_t)blockIdx.y * k_share;
  const size_t kend = kbeg + k_share < K ? kbeg + k_share : K;
  const size_t m = m0 + 4 * i;
  const bool m_ok = m < M;  // M is a multiple of 4: the vector lies inside the row or beyond it
  const float* ap = g.A + (m_ok ? m : 0);
  // B stored K x N, or (tb) N x K: element (k, c) at k * bk + c * bc
  const size_t bk = tb ? 1 : (size_t)N, bc = tb ? K : 1;
  bool c_ok[NB];
  const float* bp[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    c_ok[nb] = i + 16 * nb < N;
    bp[nb] = g.B + (c_ok[nb] ? (size_t)(i + 16 * nb) * bc : 0);
  }

  floatx4 acc[NB][4];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[nb][t][v] = 0.0f;

  // wave w takes the steps w, w + 4, ... of its share; step s covers the rows kbeg + 4 s .. + 3
  const size_t steps = (kend - kbeg + 3) / 4;
  // One set of loads at a time: with a second set requested before the first is multiplied the
  // kernel needs 112 VGPRs instead of 74, holds half the waves and measured 3-20 % slower.
  float4 a[TT_STEPS];
  float b[NB][TT_STEPS];
  for (size_t s0 = w; s0 < steps; s0 += 4 * TT_STEPS) {
#pragma unroll
    for (int u = 0; u < TT_STEPS; ++u) {
      const size_t k = kbeg + 4 * (s0 + 4 * (size_t)u) + kk;
      const bool k_ok = s0 + 4 * (size_t)u < steps && k < kend;
      const size_t kc = k_ok ? k : kbeg;
      a[u] = ld4s(ap + kc * M);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) b[nb][u] = bp[nb][kc * bk];
      if (!k_ok || !m_ok) a[u] = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        if (!k_ok || !c_ok[nb]) b[nb][u] = 0.0f;
    }
#pragma unroll
    for (int u = 0; u < TT_STEPS; ++u) {
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        acc[nb][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[u].x, b[nb][u], acc[nb][0], 0, 0, 0);
        acc[nb][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[u].y, b[nb][u], acc[nb][1], 0, 0, 0);
        acc[nb][2] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[u].z, b[nb][u], acc[nb][2], 0, 0, 0);
        acc[nb][3] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[u].w, b[nb][u], acc[nb][3], 0, 0, 0);
      }
    }
  }
  if (w) {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) part[w - 1][lane][16 * nb + 4 * t + v] = acc[nb][t][v];
  }
  __syncthreads();
  const bool raw = gridDim.y > 1;
  if (w == 0) {
#pragma unroll
    for (int o = 0; o < 3; ++o)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int v = 0; v < 4; ++v) acc[nb][t][v] += part[o][lane][16 * nb + 4 * t + v];

    // register v of block t in lane (i, kk): row m0 + 4 * (4 kk + v) + t of C, column i (+ 16 for the second block)
    float* dst = raw ? g.partial + (size_t)blockIdx.y * M * (size_t)N : g.C;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      if (!c_ok[nb]) continue;
      const int col = i + 16 * nb;
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const size_t row = m0 + 4 * (4 * kk + v) + t;
          if (row >= M) continue;
          const size_t at = row * (size_t)N + col;
          float x = acc[nb][t][v];
          if (!raw) {
            if (g.mask) x = (g.mask[at] >= 0.0f ? 1.0f : 0.0f) * x;
            if (g.beta != 0.0f) x = g.beta * g.C[at] + x;
            if (g.bias) x = x + g.bias[col];
            if (g.pre_act) g.pre_act[at] = x;
            if (g.relu) x = (x >= 0.0f ? 1.0f : 0.0f) * x;
          }
          dst[at] = x;
        }
    }
  }
}

// Returns 0 if the product is not this kernel's, 1 if it ran to completion (*rc = status), 2 if
// partials of g.splits k ranges wait in the workspace for the split-K combine.
int gemm_tall_launch(slhip_ctx* ctx, bool ta, bool tb, GemmArgs& g, int32_t* rc) {
  const size_t M = g.M, N = g.N, K = g.K;
  // At * B with 8..16 columns, A in whole 128-byte lines per row piece.  Against the narrow-N kernel:
  // 2048 x 10 x 8192 24.5 -> 19.1 us, 16384 x 10 / 16 x 16384 220 / 234 -> 172 / 177 (6.3 / 6.1 TB/s),
  // 2048 x 16 x 2048 16.6 -> 10.1, 256 x 16 x 262144 94 -> 65, 65536 x 10 x 1024 60 -> 46; with 4..7
  // columns the two are level (ahead on some shapes, behind on others) and the other one stays.
  // 17..32 columns: a second block of 16 columns on the same loads of A (4096 x 17 / 32 x 65536 502 -> 205 / 211 us,
  // 16384 x 24 x 16384 276 -> 203, 65536 x 32 x 1024 87 -> 63, all on the wave-per-tile kernel before).
  // (M a multiple of 32: with rows of A that start off the 128-byte grid the kernel measured 20-70 % slower than
  // the narrow-N kernel it replaces - 10000 x 10 x 10000 106 -> 130 us, 4100 x 8 x 32768 121 -> 211)
  if (ta && N <= 32 && N >= 8 && M % 32 == 0 && M >= 64 && K >= 64 && M * K >= (size_t(1) << 22)) {
    const size_t gx = (M + 63) / 64;
    if (gx > 0x7fffffffu) return 0;
    // two workgroups per CU; every wave of a share gets at least 8 steps of four k
    size_t splits = ((size_t)ctx->num_cu * 2 + gx - 1) / gx;
    if (splits > K / 128) splits = K / 128;
    if (splits > 64) splits = 64;
    if (splits > ctx->workspace_bytes / (M * N * sizeof(float))) splits = ctx->workspace_bytes / (M * N * sizeof(float));
    if (splits < 1) splits = 1;
    const size_t share = ((K + splits - 1) / splits + 3) / 4 * 4;
    splits = (K + share - 1) / share;
    g.splits = (unsigned)splits;
    if (N <= 16) hipLaunchKernelGGL(gemm_tall_t_kernel<1>, dim3((unsigned)gx, (unsigned)splits), dim3(256), 0, ctx->stream, g, share, tb ? 1 : 0);
    else hipLaunchKernelGGL(gemm_tall_t_kernel<2>, dim3((unsigned)gx, (unsigned)splits), dim3(256), 0, ctx->stream, g, share, tb ? 1 : 0);
    *rc = post_launch();
    return splits > 1 && *rc == SLHIP_OK ? 2 : 1;
  }
  // Against the sixteen-block kernel (which is bound by the matrix pipes from 13 columns on:
  // 16384 x 16 x 16384 takes it 377 us, this one 182): ahead at 8 columns and more wherever K is
  // long enough to amortise the pack and the combine (16384 x 8 / 10 / 12 x 16384: 253 / 223 / 242
  // -> 180 us; 8192 x 10 x 2048: 27.0 -> 24.8; 2048 x 10 x 8192: 33.4 -> 27.6), level at 2^23
  // elements of A, behind with K = 1024 (65536 x 8 / 12 x 1024: 50 / 64 us there, 71 here) and below 8
  // columns except on 1 GiB (16384 x 2 / 4 / 6 x 16384: 192 / 184 / 192 there, 183 / 182 / 180 here,
  // but 16384 x 2 x 8192 93 there and 101 here).
  if (ta || N > 32 || N < 8 || K % 4 != 0 || K < 256 || M < 512) return 0;
  if (N >= 13 ? M * K < (size_t(1) << 22) : (K < 2048 || M * K < (size_t(1) << 24))) return 0;
  const size_t Kp = (K + TALL_KC - 1) / TALL_KC * TALL_KC;
  const size_t bt_bytes = 32 * Kp * sizeof(float);
  if (bt_bytes > ((size_t)32 << 20) || ctx->workspace_bytes < 4 * bt_bytes + ((size_t)64 << 20)) return 0;
  // Bt at the top of the workspace, partials from its start
  float* bt = (float*)((char*)ctx->workspace + ctx->workspace_bytes - bt_bytes);
  const size_t ws_bytes = ctx->workspace_bytes - bt_bytes;
  const size_t gx = (M + TALL_ROWS - 1) / TALL_ROWS;
  if (gx > 0x7fffffffu) return 0;
  const size_t chunks = Kp / TALL_KC;
  size_t splits = 1;
  // one round of three workgroups per CU (two, three, four and eight rounds measured 3-15 % slower)
  const size_t want = (size_t)ctx->num_cu * 3;
  if (gx < want) {
    splits = (want + gx - 1) / gx;
    if (splits > chunks / 8) splits = chunks / 8;  // at least eight steps each
    if (splits > 64) splits = 64;
    if (splits > ws_bytes / (M * N * sizeof(float))) splits = ws_bytes / (M * N * sizeof(float));
    if (splits < 1) splits = 1;
    const size_t per = (chunks + splits - 1) / splits;
    splits = (chunks + per - 1) / per;
  }
  g.splits = (unsigned)splits;
  const size_t pack_blocks = (32 * Kp + 255) / 256;
  hipLaunchKernelGGL(tall_pack_b_kernel, dim3((unsigned)pack_blocks), dim3(256), 0, ctx->stream, K, Kp, (int)N, tb ? 1 : 0, g.B, bt);
  const size_t lds = (size_t)6 * 32 * TALL_PITCH * sizeof(float);
  if (N <= 16) hipLaunchKernelGGL(gemm_tall_kernel<true>, dim3((unsigned)gx, (unsigned)splits), dim3(256), lds, ctx->stream, g, (const float*)bt, Kp);
  else hipLaunchKernelGGL(gemm_tall_kernel<false>, dim3((unsigned)gx, (unsigned)splits), dim3(256), lds, ctx->stream, g, (const float*)bt, Kp);
  *rc = post_launch();
  return splits > 1 && *rc == SLHIP_OK ? 2 : 1;
}

}  // namespace slhip
