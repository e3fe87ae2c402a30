// Products with one very short dimension and a large streamed operand or result.  They are bound
// by HBM, not by the matrix cores, so they run on the vector ALUs with every global access a
// whole float4 per lane:
//
//   short K   (K <= 12, any form): C[M x N] is the large side (4 B written per 2K flop).  A thread
//             keeps the K x 4 block of B for its four columns in registers and walks down the rows;
//             the K values of A for a row are the same for the whole wave.  In a classifier this
//             is the input gradient of the last layer, G[batch x classes] * W^T.
//   narrow N  (N <= 16, A^T * B with A stored K x M): A is the large side and is read once, in
//             rows of M contiguous floats; a lane keeps 4 x N accumulators for its four columns of
//             A; the N values of B for a k are the same for the whole wave.  Sixteen waves of a
//             workgroup interleave over the k range and add up through LDS in a fixed order;
//             workgroups split K and leave partials in the workspace for the split-K combine.
//             In a classifier this is the weight gradient of the last layer, H^T * G.
//
//   narrow N, A row-major (N <= 16, A * B with A stored M x K): A is the large side again, but now
//             the reduction runs along its contiguous axis.  The 16-block matrix instruction
//             (v_mfma_f32_4x4x1: sixteen independent 4 x 4 x 1 products per issue) takes block b as
//             a k position: lane (b, i) loads a float4 of row i at k = 64 s + 4 b, so a load
//             instruction of a wave reads 256 contiguous bytes of each of four rows; B's column
//             groups wait in LDS in the order the B operand wants them; the sixteen blocks'
//             partial sums meet in four butterfly steps per row group.  In a classifier this is
//             the forward product of the last layer, H * W.
//
// Against the wave-per-tile MFMA kernel, which reads and writes 128-byte pieces per row
// (MI355X, classifier with batch 8192, hidden 2048, 10 classes): input gradient with the ReLU
// mask 33 -> 23 us (23 -> 14.5 without the mask), weight gradient with its combine 34.5 -> 29 us;
// 4096 x 16 x 16384 (256 MiB of A) 116 -> 61 us, 1024 x 4 x 65536 112 -> 54 us.
#include "gemm_tile.hpp"

namespace slhip {

// beyond 12 the wave-per-tile MFMA kernel is the faster one (4096 x 4096 x 16: 17.6 us against 19.3)
constexpr int SHORT_K_MAX = 12;
constexpr int SHORT_K_ROWS = 64;  // most rows of A a workgroup of the short-K kernel stages in LDS

template <int KP, bool TA, bool TB>
__global__ __launch_bounds__(256) void gemm_short_k_kernel(size_t M, size_t N, int K, const float* __restrict__ A,
                                                           const float* __restrict__ B, float* C, float beta,
                                                           const float* __restrict__ bias, int relu, float* pre_act,
                                                           const float* mask, const uint32_t* __restrict__ bits,
                                                           unsigned rows_per_block) {
  // The rows of A this workgroup uses, zero-padded to KP columns: every lane of a wave reads the
  // same row at the same time (one broadcast ds_read_b128 per four k).  Fetching them with
  // wave-uniform global loads instead costs K load instructions per row and store.
  __shared__ __attribute__((aligned(16))) float As[SHORT_K_ROWS][KP];
  const size_t m0 = (size_t)blockIdx.y * rows_per_block;
  const int rows = (int)(m0 + rows_per_block < M ? rows_per_block : M - m0);
  for (int idx = threadIdx.x; idx < rows * KP; idx += 256) {
    const int r = TA ? idx % rows : idx / KP, k = TA ? idx / rows : idx % KP;
    float v = 0.0f;
    if (k < K) v = TA ? A[(size_t)k * M + m0 + r] : A[(m0 + r) * (size_t)K + k];
    As[r][k] = v;
  }
  const size_t n = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
  const bool active = n < N;
  const size_t nc = active ? n : 0;
  float b[KP][4];
  if (TB) {
    // B is stored N x K: the K x 4 block of a thread is 4K contiguous floats (16-byte aligned: n is
    // a multiple of 4), K vector loads in flight together; float q*K + k of them is B[n + q][k].
    // K is one of the four values that share this KP: each gets its own unrolled unpacking.
    float f[KP * 4];
#pragma unroll
    for (int j = 0; j < KP; ++j) {
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (j < K) v = ld4g(B + nc * (size_t)K + 4 * j);
      f[4 * j] = v.x; f[4 * j + 1] = v.y; f[4 * j + 2] = v.z; f[4 * j + 3] = v.w;
    }
    auto unpack = [&](auto kc) {
      constexpr int KC = decltype(kc)::value;
#pragma unroll
      for (int k = 0; k < KP; ++k)
#pragma unroll
        for (int q = 0; q < 4; ++q) b[k][q] = k < KC ? f[(q * KC + k) % (KP * 4)] : 0.0f;
    };
    switch (KP - K) {
      case 0: unpack(std::integral_constant<int, KP>()); break;
      case 1: unpack(std::integral_constant<int, KP - 1>()); break;
      case 2: unpack(std::integral_constant<int, KP - 2>()); break;
      default: unpack(std::integral_constant<int, KP - 3>()); break;
    }
  } else {
#pragma unroll
    for (int k = 0; k < KP; ++k) {
      if (k < K) {
        const float4 v = ld4g(B + (size_t)k * N + nc);
        b[k][0] = v.x; b[k][1] = v.y; b[k][2] = v.z; b[k][3] = v.w;
      } else {
#pragma unroll
        for (int q = 0; q < 4; ++q) b[k][q] = 0.0f;
      }
    }
  }
  float4 bi = make_float4(0.f, 0.f, 0.f, 0.f);
  if (bias) bi = ld4g(bias + nc);
  __syncthreads();
  if (!active) return;
  constexpr int R = 4;  // rows per pass: their mask / C reads are in flight together
  for (int m = 0; m < rows; m += R) {
    float acc[R][4];
    size_t at[R], row[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int lr = m + r < rows ? m + r : rows - 1;  // a pass past the end repeats the last row and does not store it
      row[r] = m0 + lr;
      at[r] = row[r] * N + n;
#pragma unroll
      for (int q = 0; q < 4; ++q) acc[r][q] = 0.0f;
#pragma unroll
      for (int k = 0; k < KP; ++k) {
        const float a = As[lr][k];
#pragma unroll
        for (int q = 0; q < 4; ++q) acc[r][q] = __builtin_fmaf(a, b[k][q], acc[r][q]);
      }
    }
    // every read before the first store: C, pre_act and mask may be the same memory as far as the compiler knows
    if (mask) {
      float4 mk[R];
#pragma unroll
      for (int r = 0; r < R; ++r) mk[r] = ld4g(mask + at[r]);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        acc[r][0] *= (mk[r].x >= 0.f ? 1.f : 0.f); acc[r][1] *= (mk[r].y >= 0.f ? 1.f : 0.f);
        acc[r][2] *= (mk[r].z >= 0.f ? 1.f : 0.f); acc[r][3] *= (mk[r].w >= 0.f ? 1.f : 0.f);
      }
    }
    if (bits) {  // the mask packed 32 columns to a word, row-major: the thread's four columns share a word
      const size_t W = (N + 31) >> 5;
      uint32_t mk[R];
#pragma unroll
      for (int r = 0; r < R; ++r) mk[r] = bits[row[r] * W + (n >> 5)];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const uint32_t four = mk[r] >> (n & 31);
        acc[r][0] *= ((four & 1u) ? 1.f : 0.f); acc[r][1] *= ((four & 2u) ? 1.f : 0.f);
        acc[r][2] *= ((four & 4u) ? 1.f : 0.f); acc[r][3] *= ((four & 8u) ? 1.f : 0.f);
      }
    }
    if (beta != 0.0f) {
      float4 cc[R];
#pragma unroll
      for (int r = 0; r < R; ++r) cc[r] = ld4g(C + at[r]);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        acc[r][0] = beta * cc[r].x + acc[r][0]; acc[r][1] = beta * cc[r].y + acc[r][1];
        acc[r][2] = beta * cc[r].z + acc[r][2]; acc[r][3] = beta * cc[r].w + acc[r][3];
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (m + r >= rows) break;
      float4 v = make_float4(acc[r][0], acc[r][1], acc[r][2], acc[r][3]);
      if (bias) { v.x += bi.x; v.y += bi.y; v.z += bi.z; v.w += bi.w; }
      if (pre_act) st4g(pre_act + at[r], v);
      if (relu) {
        v.x = (v.x >= 0.f ? 1.f : 0.f) * v.x; v.y = (v.y >= 0.f ? 1.f : 0.f) * v.y;
        v.z = (v.z >= 0.f ? 1.f : 0.f) * v.z; v.w = (v.w >= 0.f ? 1.f : 0.f) * v.w;
      }
      st4g(C + at[r], v);
    }
  }
}

// partial[z] = A^T * B over the k range of workgroup z = blockIdx.y: A stored K x M, B stored K x N,
// N <= NP <= 16.  A lane owns four columns of A and 4 x NP sums; a wave walks down its share of the
// k range with eight float4 loads of A per batch, 1 KiB contiguous per load and wave, the next
// batch requested before the current one is multiplied and the first before anything else: the
// workgroup's slice of B (one contiguous run of k_chunk * N floats) goes into LDS as [k][NP] rows,
// zero beyond N and beyond the end of K, behind those loads.  In the loop a row of B is NP / 4
// broadcast ds_read_b128.  The eight waves of a workgroup then add their sums in wave order
// through LDS (one barrier) and wave 0 writes them as [M][NP] rows - the 4 x NP sums of a lane are
// contiguous there, NP float4 stores; narrow_n_combine_kernel adds the workgroups' partials in a
// fixed order.
constexpr int NARROW_WAVES = 8;      // waves per workgroup
constexpr int NARROW_BATCH = 8;      // rows of A per batch and wave
constexpr int NARROW_K_CHUNK = 512;  // most k per workgroup (its rows of B sit in LDS)
template <int NP>
__global__ __launch_bounds__(64 * NARROW_WAVES) void gemm_narrow_n_kernel(size_t M, int N, size_t K, const float* __restrict__ A,
                                                                          const float* __restrict__ B,
                                                                          float* __restrict__ partial, size_t k_chunk) {
  constexpr int U = NP > 12 ? NARROW_BATCH / 2 : NARROW_BATCH, Q = NP / 4;  // sixteen columns: 64 sums a lane, half the batch
  __shared__ __attribute__((aligned(16))) float4 red[NARROW_WAVES - 1][NP][64];
  __shared__ __attribute__((aligned(16))) float bsh[NARROW_K_CHUNK * NP];
  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const size_t m = ((size_t)blockIdx.x * 64 + lane) * 4;
  const bool active = m < M;
  // lanes past the last column read the last whole vector of the row again and are never stored
  const size_t mc = active ? m : M - 4;
  const size_t kbeg = (size_t)blockIdx.y * k_chunk;
  const size_t kend = kbeg + k_chunk < K ? kbeg + k_chunk : K;
  const int klen = (int)(kend - kbeg);
  const int per_wave = (int)(k_chunk / NARROW_WAVES);  // a multiple of 2 * U
  const int k_first = w * per_wave, k_last = k_first + per_wave;  // relative to kbeg; rows from klen on are zero in LDS
  float4 acc[NP];
#pragma unroll
  for (int n = 0; n < NP; ++n) acc[n] = make_float4(0.f, 0.f, 0.f, 0.f);
  auto load_batch = [&](float4 (&a)[U], int k0) {
#pragma unroll
    for (int u = 0; u < U; ++u) a[u] = ld4s(A + (kbeg + (k0 + u < klen ? k0 + u : klen - 1)) * M + mc);
  };
  auto multiply_batch = [&](const float4 (&a)[U], int k0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const float4* brow = reinterpret_cast<const float4*>(bsh + (size_t)(k0 + u) * NP);  // wave-uniform
#pragma unroll
      for (int q = 0; q < Q; ++q) {
        const float4 bq = brow[q];
        const float bv[4] = {bq.x, bq.y, bq.z, bq.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[4 * q + j].x = __builtin_fmaf(a[u].x, bv[j], acc[4 * q + j].x);
          acc[4 * q + j].y = __builtin_fmaf(a[u].y, bv[j], acc[4 * q + j].y);
          acc[4 * q + j].z = __builtin_fmaf(a[u].z, bv[j], acc[4 * q + j].z);
          acc[4 * q + j].w = __builtin_fmaf(a[u].w, bv[j], acc[4 * q + j].w);
        }
      }
    }
  };
  float4 a0[U], a1[U];
  const bool any = k_first < klen;
  if (any) load_batch(a0, k_first);
  {
    const float* bsrc = B + kbeg * (size_t)N;
    const int rows = (int)k_chunk;
    for (int idx = threadIdx.x; idx < rows * NP; idx += 64 * NARROW_WAVES) {
      const int k = idx / NP, n = idx % NP;
      bsh[idx] = (k < klen && n < N) ? bsrc[k * N + n] : 0.0f;
    }
  }
  __syncthreads();
  if (any) {
    for (int k0 = k_first; k0 < k_last; k0 += 2 * U) {
      load_batch(a1, k0 + U);
      multiply_batch(a0, k0);
      if (k0 + 2 * U < k_last) load_batch(a0, k0 + 2 * U);
      multiply_batch(a1, k0 + U);
    }
  }
  if (w > 0) {
#pragma unroll
    for (int n = 0; n < NP; ++n) red[w - 1][n][lane] = acc[n];
  }
  __syncthreads();
  if (w != 0 || !active) return;
  for (int v = 0; v < NARROW_WAVES - 1; ++v) {
#pragma unroll
    for (int n = 0; n < NP; ++n) {
      const float4 t = red[v][n][lane];
      acc[n].x += t.x; acc[n].y += t.y; acc[n].z += t.z; acc[n].w += t.w;
    }
  }
  // element e of the lane's 4 x NP run: row e / NP of its four, column e % NP (M is a multiple of 4)
  float* out = partial + ((size_t)blockIdx.y * M + m) * NP;
  auto elem = [&](int e) {
    const float4 s = acc[e % NP];
    const int q = e / NP;
    return q == 0 ? s.x : q == 1 ? s.y : q == 2 ? s.z : s.w;
  };
#pragma unroll
  for (int t = 0; t < NP; ++t) st4g(out + 4 * t, make_float4(elem(4 * t), elem(4 * t + 1), elem(4 * t + 2), elem(4 * t + 3)));
}

// C = sum_z partial[z] (z ascending; partial[z] is [M][NP]) + beta*C, then bias / pre-activation / relu.
template <int NP>
__global__ __launch_bounds__(256) void narrow_n_combine_kernel(size_t M, int N, unsigned splits, const float* __restrict__ partial,
                                                               float* C, float beta, const float* __restrict__ bias, int relu,
                                                               float* pre_act, const float* __restrict__ mask, int transposed) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= M * (size_t)N) return;
  // (transposed: C is N x M, element i of it is column i / M of row i % M of the product; no epilogue then)
  const size_t row = transposed ? i % M : i / N, n = transposed ? i / M : i % N;
  const float* p = partial + row * NP + n;
  const size_t step = M * NP;
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
  if (mask) s *= (mask[i] >= 0.f ? 1.f : 0.f);
  if (beta != 0.0f) s = beta * C[i] + s;
  if (bias) s += bias[n];
  if (pre_act) pre_act[i] = s;
  if (relu) s = (s >= 0.f ? 1.f : 0.f) * s;
  C[i] = s;
}

// C = A * B for a narrow B: A stored M x K (K a multiple of 4), B stored K x N, N <= 4 * G.
// A workgroup of eight waves stages a k chunk of B in LDS once ([column group][k / 4][column][k % 4],
// zero beyond N and K, so that the B operand of lane (b, j) for four consecutive k is one
// ds_read_b128 and a wave's reads are 1 KiB contiguous); a wave takes groups of four rows, issues
// ALL its loads of a chunk before the first multiply (32 float4 per lane for a chunk of 2048 k:
// the workgroup's whole share of A is in flight at once) and multiplies them as they arrive.
constexpr int ROWS_NARROW_KC = 2048;  // k per chunk: 16 KiB of LDS per column of B's groups
typedef float rn_f4 __attribute__((ext_vector_type(4)));

template <int G>
__global__ __launch_bounds__(512) void gemm_rows_narrow_kernel(GemmArgs g) {
  extern __shared__ __attribute__((aligned(16))) float rn_b[];  // [G][KC / 4][4][4]
  constexpr int KC = ROWS_NARROW_KC, KQ = KC / 4, STEPS = KC / 64;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int b = lane >> 2, ij = lane & 3;  // block of the matrix instruction; row (A operand) or column (B operand, result) in it
  const size_t M = g.M, K = g.K;
  const int N = (int)g.N;
  const size_t groups = (M + 3) / 4;
  const size_t chunks = (K + KC - 1) / KC;
  // few long rows: gridDim.y workgroups share the chunks of a row group and leave raw partial sums
  // (g.partial[y][M][N]) for the split-K combine, which then applies the epilogue
  const bool raw = gridDim.y > 1;
  const size_t per_y = (chunks + gridDim.y - 1) / gridDim.y;
  const size_t ch_beg = (size_t)blockIdx.y * per_y;
  const size_t ch_end = ch_beg + per_y < chunks ? ch_beg + per_y : chunks;
  for (size_t grp0 = (size_t)blockIdx.x * 8; grp0 < groups; grp0 += (size_t)gridDim.x * 8) {
    const size_t grp = grp0 + w;
    const bool have = grp < groups;
    const size_t row = have ? (grp * 4 + ij < M ? grp * 4 + ij : M - 1) : 0;
    rn_f4 acc[G];
#pragma unroll
    for (int gi = 0; gi < G; ++gi) acc[gi] = rn_f4{0.f, 0.f, 0.f, 0.f};
    for (size_t ch = ch_beg; ch < ch_end; ++ch) {
      const size_t k0 = ch * KC;
      const int klen = (int)(k0 + KC < K ? KC : K - k0);
      // B's chunk is staged on the first pass, and again whenever the chunk changes (K > KC), BEFORE
      // the loads of A are issued: a wave's loads return in order, so a load of B behind the loads of A
      // would not be usable before all of A has arrived.  A thread takes four whole rows of B
      // (k = thread + 512 r): N loads each, contiguous across the threads and all in flight together,
      // then 4 * G scattered LDS writes per row, which also lay down the zeros beyond N and K.
      if (grp0 == (size_t)blockIdx.x * 8 || ch_end - ch_beg > 1) {
        float f[KC / 512][4 * G];
#pragma unroll
        for (int r = 0; r < KC / 512; ++r) {
          const int k = threadIdx.x + 512 * r;
#pragma unroll
          for (int n = 0; n < 4 * G; ++n) f[r][n] = (k < klen && n < N) ? g.B[(k0 + k) * (size_t)N + n] : 0.0f;
        }
        __syncthreads();  // the previous chunk is done with
#pragma unroll
        for (int r = 0; r < KC / 512; ++r) {
          const int k = threadIdx.x + 512 * r;
#pragma unroll
          for (int n = 0; n < 4 * G; ++n) rn_b[(((n >> 2) * KQ + (k >> 2)) * 4 + (n & 3)) * 4 + (k & 3)] = f[r][n];
        }
        __syncthreads();
      }
      // this lane's share of the chunk in batches of LOADS float4, every batch in flight at once
      // (16 KiB per wave and batch; with all 32 in flight the accumulators and B's fragments no
      // longer fit beside them, and a spill's reload in this loop waits for every load of A that is
      // still in flight)
      constexpr int LOADS = 16;
      if (have) {
#pragma unroll 1
        for (int s0 = 0; s0 < STEPS && 64 * s0 < klen; s0 += LOADS) {
          float4 a[LOADS];
#pragma unroll
          for (int u = 0; u < LOADS; ++u) {
            const int k = 64 * (s0 + u) + 4 * b;
            a[u] = ld4s(g.A + row * K + k0 + (k < klen ? k : klen - 4));
          }
#pragma unroll
          for (int u = 0; u < LOADS; ++u) {
            const int s = s0 + u;
            float4 av = a[u];
            if (64 * s + 4 * b >= klen) av = make_float4(0.f, 0.f, 0.f, 0.f);  // past the end of K: B's zeros alone would not tame an inf
            float4 bv[G];
#pragma unroll
            for (int gi = 0; gi < G; ++gi) bv[gi] = ld4(rn_b + ((gi * KQ + 16 * s + b) * 4 + ij) * 4);
            // consecutive instructions use different accumulators
#pragma unroll
            for (int gi = 0; gi < G; ++gi) acc[gi] = __builtin_amdgcn_mfma_f32_4x4x1f32(av.x, bv[gi].x, acc[gi], 0, 0, 0);
#pragma unroll
            for (int gi = 0; gi < G; ++gi) acc[gi] = __builtin_amdgcn_mfma_f32_4x4x1f32(av.y, bv[gi].y, acc[gi], 0, 0, 0);
#pragma unroll
            for (int gi = 0; gi < G; ++gi) acc[gi] = __builtin_amdgcn_mfma_f32_4x4x1f32(av.z, bv[gi].z, acc[gi], 0, 0, 0);
#pragma unroll
            for (int gi = 0; gi < G; ++gi) acc[gi] = __builtin_amdgcn_mfma_f32_4x4x1f32(av.w, bv[gi].w, acc[gi], 0, 0, 0);
          }
        }
      }
    }
    if (!have) continue;
    // register v of lane (b, j) in group gi: the sum over block b's k positions for row v, column
    // 4 gi + j.  Four butterfly steps add the sixteen blocks, in the same order on every lane.
#pragma unroll
    for (int gi = 0; gi < G; ++gi)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        float x = acc[gi][v];
        x += __shfl_xor(x, 4, WAVE);
        x += __shfl_xor(x, 8, WAVE);
        x += __shfl_xor(x, 16, WAVE);
        x += __shfl_xor(x, 32, WAVE);
        acc[gi][v] = x;
      }
    if (b != 0) continue;
    if (raw) {
      float* part = g.partial + (size_t)blockIdx.y * M * (size_t)N;
#pragma unroll
      for (int gi = 0; gi < G; ++gi)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const size_t r = grp * 4 + v;
          const int c = 4 * gi + ij;
          if (r < M && c < N) part[r * (size_t)N + c] = acc[gi][v];
        }
      continue;
    }
    // lanes 0..3 hold everything: every read (mask, C for beta) before the first store
    float val[G][4];
#pragma unroll
    for (int gi = 0; gi < G; ++gi)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const size_t r = grp * 4 + v;
        const int c = 4 * gi + ij;
        float x = acc[gi][v];
        if (r < M && c < N) {
          const size_t at = r * (size_t)N + c;
          if (g.mask) x = (g.mask[at] >= 0.0f ? 1.0f : 0.0f) * x;
          if (g.beta != 0.0f) x = g.beta * g.C[at] + x;
          if (g.bias) x = x + g.bias[c];
        }
        val[gi][v] = x;
      }
#pragma unroll
    for (int gi = 0; gi < G; ++gi)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const size_t r = grp * 4 + v;
        const int c = 4 * gi + ij;
        if (r < M && c < N) {
          const size_t at = r * (size_t)N + c;
          float x = val[gi][v];
          if (g.pre_act) g.pre_act[at] = x;
          if (g.relu) x = (x >= 0.0f ? 1.0f : 0.0f) * x;
          g.C[at] = x;
        }
      }
  }
}

// Returns 1 if a skinny kernel took the product (then *rc is its result), 0 if the caller should go on.
// g carries the operands and the epilogue; g.splits is set for the caller's split-K combine.
// The short-K kernel if the product qualifies (returns 1, *rc = launch status), else 0.
int gemm_short_k_launch(slhip_ctx* ctx, bool ta, bool tb, const GemmArgs& g, const uint32_t* bits, int32_t* rc) {
  const size_t M = g.M, N = g.N, K = g.K;
  auto ok16 = [](const void* p) { return p == nullptr || aligned16(p); };
  if (!(K <= SHORT_K_MAX && N % 4 == 0 && N >= 64 && M * N >= (size_t(1) << 18) && aligned16(g.C) && ok16(g.mask) &&
        ok16(g.pre_act) && ok16(g.bias) && aligned16(g.B)))
    return 0;
  const size_t gx = (N / 4 + 255) / 256;
  // rows per workgroup: 64 (what its LDS holds; B's block is fetched once per workgroup) down to 16
  // while that leaves fewer than two workgroups per CU
  size_t rpb = SHORT_K_ROWS;
  while (rpb > 16 && (M + rpb - 1) / rpb * gx < (size_t)ctx->num_cu * 2) rpb /= 2;
  if ((M + rpb - 1) / rpb > 65535) return 0;
  const dim3 grid((unsigned)gx, (unsigned)((M + rpb - 1) / rpb));
#define SL_SK2(KP_, TA_, TB_)                                                                                         \
  hipLaunchKernelGGL((gemm_short_k_kernel<KP_, TA_, TB_>), grid, dim3(256), 0, ctx->stream, M, N, (int)K, g.A, g.B, g.C, \
                     g.beta, g.bias, g.relu, g.pre_act, g.mask, bits, (unsigned)rpb)
#define SL_SK(KP_)                       \
  do {                                   \
    if (!ta && !tb) SL_SK2(KP_, false, false); \
    else if (!ta && tb) SL_SK2(KP_, false, true);  \
    else if (ta && !tb) SL_SK2(KP_, true, false);  \
    else SL_SK2(KP_, true, true);        \
  } while (0)
  if (K <= 4) SL_SK(4);
  else if (K <= 8) SL_SK(8);
  else SL_SK(12);
#undef SL_SK
#undef SL_SK2
  *rc = post_launch();
  return 1;
}

int gemm_skinny_launch(slhip_ctx* ctx, bool ta, bool tb, GemmArgs& g, int32_t* rc) {
  const size_t M = g.M, N = g.N, K = g.K;
  // short K: the result is the large side
  if (gemm_short_k_launch(ctx, ta, tb, g, nullptr, rc)) return 1;
  // A narrow B stored N x K (the transposed form) is first turned into K x N at the top of the
  // workspace: it is at most 16 rows, and the kernels below want k to run down its columns
  // (2048 x 10 x 65536 A*Bt: 328 us through the tiled kernel, whose tile is mostly empty).
  constexpr size_t BT_RESERVE = (size_t)16 << 20;
  // (from 2^25 elements of A on: below, the extra launch costs what the better kernel gains -
  // 8192 x 10 x 2048 A*Bt 24 us through the wave kernel, 33 this way)
  const bool bt_fits = tb && N <= 16 && M * K >= (size_t(1) << 25) && K * N * sizeof(float) <= BT_RESERVE &&
                       ctx->workspace_bytes >= 4 * BT_RESERVE;
  const size_t ws_bytes = bt_fits ? ctx->workspace_bytes - BT_RESERVE : ctx->workspace_bytes;
  auto b_as_k_by_n = [&]() -> int32_t {
    if (!tb) return SLHIP_OK;
    float* bt = (float*)((char*)ctx->workspace + ws_bytes);
    const int32_t r = slhip_transpose(ctx, N, K, g.B, bt, 0.0f);
    if (r == SLHIP_OK) g.B = bt;
    return r;
  };
  // narrow N, A row-major: A (M x K) is the large side, the reduction runs along its rows
  if (!ta && (!tb || bt_fits) && N <= 16 && K % 4 == 0 && K >= 256 && M >= 32 && M * K >= (size_t(1) << 22)) {
    if ((*rc = b_as_k_by_n()) != SLHIP_OK) return 1;
    const int G = (int)((N + 3) / 4);
    const size_t lds = (size_t)ROWS_NARROW_KC * 4 * G * sizeof(float);
    const size_t groups8 = ((M + 3) / 4 + 7) / 8;  // workgroups' worth of row groups
    // one workgroup per CU (its chunk of B takes 32 KiB of LDS per column group), each looping
    // over its share of the rows
    const size_t blocks = groups8 < (size_t)ctx->num_cu ? groups8 : (size_t)ctx->num_cu;
    // few long rows (measured 2048 x 1 x 65536: 300 us with 64 workgroups): the chunks of K are
    // dealt out over several workgroups per row group, at least two chunks each
    size_t splits = 1;
    const size_t chunks = (K + ROWS_NARROW_KC - 1) / ROWS_NARROW_KC;
    if (blocks * 2 <= (size_t)ctx->num_cu && chunks >= 4) {
      splits = (size_t)ctx->num_cu / blocks;
      if (splits > chunks / 2) splits = chunks / 2;
      if (splits > 64) splits = 64;
      if (splits > ws_bytes / (M * N * sizeof(float))) splits = ws_bytes / (M * N * sizeof(float));
      if (splits < 1) splits = 1;
      const size_t per = (chunks + splits - 1) / splits;
      splits = (chunks + per - 1) / per;  // no empty share
    }
    g.splits = (unsigned)splits;
    const dim3 grid((unsigned)blocks, (unsigned)splits);
#define SL_RN(G_)                                                                                                        \
  do {                                                                                                                   \
    static bool sized = false;                                                                                           \
    if (!sized) {                                                                                                        \
      (void)hipFuncSetAttribute((const void*)gemm_rows_narrow_kernel<G_>, hipFuncAttributeMaxDynamicSharedMemorySize,   \
                                ROWS_NARROW_KC * 16 * G_);                                                              \
      sized = true;                                                                                                      \
    }                                                                                                                    \
    hipLaunchKernelGGL((gemm_rows_narrow_kernel<G_>), grid, dim3(512), lds, ctx->stream, g);                             \
  } while (0)
    if (G == 1) SL_RN(1);
    else if (G == 2) SL_RN(2);
    else if (G == 3) SL_RN(3);
    else SL_RN(4);
#undef SL_RN
    *rc = post_launch();
    return splits > 1 && *rc == SLHIP_OK ? 2 : 1;
  }
  // narrow N: A (K x M) is the large side
  if (ta && (!tb || bt_fits) && N <= 16 && M % 4 == 0 && M >= 256 && K >= 512 && M * K >= (size_t(1) << 22)) {
    const int NP = (int)((N + 3) / 4 * 4);
    const size_t gx = (M / 4 + 63) / 64;
    // K splits: one workgroup of eight waves per CU (its LDS holds seven waves' sums), every wave
    // whole double batches; the partials (splits x M x NP floats) stay a small fraction of A
    constexpr size_t GRAIN = (size_t)NARROW_WAVES * 2 * NARROW_BATCH;  // 128 k
    size_t splits = ((size_t)ctx->num_cu + gx - 1) / gx;
    const size_t most = K / GRAIN;  // K >= 512 here
    if (splits > most) splits = most;
    if (splits < (K + NARROW_K_CHUNK - 1) / NARROW_K_CHUNK) splits = (K + NARROW_K_CHUNK - 1) / NARROW_K_CHUNK;
    if (splits > 65535) splits = 65535;
    const size_t part_bytes = M * NP * sizeof(float);
    if (splits > ws_bytes / part_bytes) splits = ws_bytes / part_bytes;
    if (splits < 1) return 0;
    const size_t k_chunk = ((K + splits - 1) / splits + GRAIN - 1) / GRAIN * GRAIN;
    splits = (K + k_chunk - 1) / k_chunk;
    if (gx > 0x7fffffffu) return 0;
    if ((*rc = b_as_k_by_n()) != SLHIP_OK) return 1;
    const dim3 grid((unsigned)gx, (unsigned)splits);
    const size_t outs = M * N;
    const dim3 cgrid((unsigned)((outs + 255) / 256));
    // (a product issued as its transpose: the combine writes the caller's C)
    const bool swap = ctx->swap_c && !g.bias && !g.relu && !g.pre_act && !g.mask && g.beta == 0.0f;
#define SL_NN(NP_)                                                                                                           \
  do {                                                                                                                       \
    hipLaunchKernelGGL((gemm_narrow_n_kernel<NP_>), grid, dim3(64 * NARROW_WAVES), 0, ctx->stream, M, (int)N, K, g.A, g.B,   \
                       g.partial, k_chunk);                                                                                  \
    hipLaunchKernelGGL((narrow_n_combine_kernel<NP_>), cgrid, dim3(256), 0, ctx->stream, M, (int)N, (unsigned)splits,        \
                       (const float*)g.partial, swap ? ctx->swap_c : g.C, swap ? ctx->swap_beta : g.beta, g.bias, g.relu,    \
                       g.pre_act, g.mask, swap ? 1 : 0);                                                                     \
  } while (0)
    if (NP == 4) SL_NN(4);
    else if (NP == 8) SL_NN(8);
    else if (NP == 12) SL_NN(12);
    else SL_NN(16);
#undef SL_NN
    if (swap) ctx->swap_done = true;
    *rc = post_launch();
    return 1;
  }
  return 0;
}

}  // namespace slhip
