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
// Tiling: 256 threads = 4 waves in a 2x2 grid, 128x128 macro tile, each wave 64x64 = four
// 32x32 accumulators (64 VGPRs), BK = 32 per LDS stage, two LDS stages with register
// prefetch of the next stage (one barrier per stage), MFMA fragments read one k-group ahead.  Tiles are numbered so that each XCD (its
// own L2) works along one tile row at a time.  Small grids are split along K; the partial
// products go to the context workspace and are combined in a fixed order.
#include "common.hpp"

namespace slhip {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int BM = 128, BN = 128;
constexpr int XC_PITCH = 128 + 4;  // [k][x] layout, x contiguous; pitch keeps float4 alignment

template <int BK>
struct Cfg {
  static constexpr int KC_PITCH = BK + 4;  // [x][k] layout, k contiguous
  static constexpr int STAGE_FLOATS = 128 * KC_PITCH > BK * XC_PITCH ? 128 * KC_PITCH : BK * XC_PITCH;
  static constexpr int NV = BK * 128 / 4 / 256;  // float4 per thread per operand tile
};

struct GemmArgs {
  size_t M, N, K;
  const float* A;
  const float* B;
  float* C;
  float beta;
  const float* bias;  // may be null
  int relu;
  float* pre_act;     // may be null
  unsigned tiles_m, tiles_n;
  unsigned splits;    // > 1: write raw partial sums to `partial[z][M*N]`
  size_t k_chunk;     // multiple of BK
  float* partial;
  int a_vec, b_vec;   // operand base and leading dimension allow 16-byte loads
};

// Operand tile held in registers between the global load and the LDS store.
template <int BK>
struct Frag {
  float4 v[Cfg<BK>::NV];
};

// k-contiguous source: element (x, k) at src[x*ld + k]; tile 128 x BK.
template <int BK, bool FAST>
__device__ __forceinline__ void load_kc(Frag<BK>& f, const float* __restrict__ src, size_t ld, size_t X, size_t Kend,
                                        size_t x0, size_t k0) {
  constexpr int VPR = BK / 4, RPP = 256 / VPR;  // float4 per row, rows per pass
  const int kq = threadIdx.x % VPR, xr = threadIdx.x / VPR;
#pragma unroll
  for (int p = 0; p < Cfg<BK>::NV; ++p) {
    const size_t x = x0 + xr + RPP * p, k = k0 + 4 * kq;
    if (FAST) {
      f.v[p] = ld4(src + x * ld + k);
    } else {
      float t[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) t[q] = (x < X && k + q < Kend) ? src[x * ld + k + q] : 0.0f;
      f.v[p] = make_float4(t[0], t[1], t[2], t[3]);
    }
  }
}
template <int BK>
__device__ __forceinline__ void store_kc(const Frag<BK>& f, float* lds) {
  constexpr int VPR = BK / 4, RPP = 256 / VPR;
  const int kq = threadIdx.x % VPR, xr = threadIdx.x / VPR;
#pragma unroll
  for (int p = 0; p < Cfg<BK>::NV; ++p) st4(lds + (xr + RPP * p) * Cfg<BK>::KC_PITCH + 4 * kq, f.v[p]);
}

// x-contiguous source: element (x, k) at src[k*ld + x]; tile BK x 128.
template <int BK, bool FAST>
__device__ __forceinline__ void load_xc(Frag<BK>& f, const float* __restrict__ src, size_t ld, size_t X, size_t Kend,
                                        size_t x0, size_t k0) {
  const int xq = threadIdx.x & 31, kr = threadIdx.x >> 5;  // 32 float4 per k-row, 8 rows per pass
#pragma unroll
  for (int p = 0; p < Cfg<BK>::NV; ++p) {
    const size_t k = k0 + kr + 8 * p, x = x0 + 4 * xq;
    if (FAST) {
      f.v[p] = ld4(src + k * ld + x);
    } else {
      float t[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) t[q] = (k < Kend && x + q < X) ? src[k * ld + x + q] : 0.0f;
      f.v[p] = make_float4(t[0], t[1], t[2], t[3]);
    }
  }
}
template <int BK>
__device__ __forceinline__ void store_xc(const Frag<BK>& f, float* lds) {
  const int xq = threadIdx.x & 31, kr = threadIdx.x >> 5;
#pragma unroll
  for (int p = 0; p < Cfg<BK>::NV; ++p) st4(lds + (kr + 8 * p) * XC_PITCH + 4 * xq, f.v[p]);
}

// MFMA fragments of one 8-wide k group for the two 32-row blocks of this wave's 64 rows.
// KC = true: lds is [x][k]; false: [k][x].  x_base = first of the wave's 64 rows/cols.
template <bool KC, int BK>
__device__ __forceinline__ void read_frag(float (&out)[2][4], const float* lds, int x_base, int kk8, int r, int h) {
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    if (KC) {
      float4 t = ld4(lds + (x_base + 32 * i + r) * Cfg<BK>::KC_PITCH + kk8 * 8 + 4 * h);
      out[i][0] = t.x; out[i][1] = t.y; out[i][2] = t.z; out[i][3] = t.w;
    } else {
#pragma unroll
      for (int t = 0; t < 4; ++t) out[i][t] = lds[(kk8 * 8 + 4 * h + t) * XC_PITCH + x_base + 32 * i + r];
    }
  }
}

// Linear workgroup id -> tile.  Tiles are walked in groups of 8 tile rows, row index fastest.
// The hardware deals consecutive workgroup ids round-robin to the 8 XCDs, so with a group
// height of 8 every XCD (its own L2) keeps working along ONE tile row of the group: its A panel
// stays put in that L2 while the B panels stream through.  Measured on 4096^3: an explicit
// remap that instead gave each XCD a compact 8x8 block of tiles was no faster for A*B and
// At*B and 25 % slower for A*Bt.
__device__ __forceinline__ void tile_of_block(unsigned bid, unsigned tiles_m, unsigned tiles_n, unsigned& tm,
                                              unsigned& tn) {
  constexpr unsigned GROUP_M = 8;
  const unsigned in_group = GROUP_M * tiles_n;
  const unsigned group = bid / in_group;
  const unsigned first_m = group * GROUP_M;
  const unsigned gsize = tiles_m - first_m < GROUP_M ? tiles_m - first_m : GROUP_M;
  const unsigned local = bid % in_group;
  tm = first_m + local % gsize;
  tn = local / gsize;
}

// The k loop over tiles [kt_begin, kt_end) of one workgroup.  FAST = every tile in the range is
// complete and 16-byte loadable, so the global loads are unconditional float4 loads; otherwise
// every element is bounds-checked and zero-filled.  The two variants are separate loops on
// purpose: when both kinds of load sat behind a branch in ONE loop body the compiler folded them
// into the per-element form, which cost 19 % of the kernel's throughput.
template <bool TA, bool TB, int BK, bool FAST>
__device__ __forceinline__ void gemm_tiles(const GemmArgs& g, int kt_begin, int kt_end, size_t kbeg, size_t kend,
                                           size_t m0, size_t n0, float (*lds_a)[Cfg<BK>::STAGE_FLOATS],
                                           float (*lds_b)[Cfg<BK>::STAGE_FLOATS], floatx16 (&acc)[2][2]) {
  constexpr int KSTEPS = BK / 8;
  constexpr int REFILL_AT = (TA && !TB) ? KSTEPS - 1 : (KSTEPS > 1 ? 1 : 0);
  if (kt_begin >= kt_end) return;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = wave >> 1, wn = wave & 1;
  const int r = lane & 31, h = lane >> 5;
  // A is KC ([m][k], ld = K) unless transposed ([k][m], ld = M); B is XC ([k][n], ld = N)
  // unless transposed ([n][k], ld = K).
  const size_t lda = TA ? g.M : g.K, ldb = TB ? g.K : g.N;

  Frag<BK> fa, fb;
  auto load_stage = [&](int kt) {
    const size_t k0 = kbeg + (size_t)kt * BK;
    if (TA) load_xc<BK, FAST>(fa, g.A, lda, g.M, kend, m0, k0);
    else load_kc<BK, FAST>(fa, g.A, lda, g.M, kend, m0, k0);
    if (TB) load_kc<BK, FAST>(fb, g.B, ldb, g.N, kend, n0, k0);
    else load_xc<BK, FAST>(fb, g.B, ldb, g.N, kend, n0, k0);
  };
  auto store_stage = [&](int s) {
    if (TA) store_xc<BK>(fa, lds_a[s]); else store_kc<BK>(fa, lds_a[s]);
    if (TB) store_kc<BK>(fb, lds_b[s]); else store_xc<BK>(fb, lds_b[s]);
  };

  // Software pipeline over the k tiles.  While tile kt is multiplied out of LDS stage s:
  //   * the registers hold tile kt+1 (its global loads were issued one iteration ago);
  //   * before k-group REFILL_AT of tile kt those registers are stored to stage s^1 and the global
  //     loads of tile kt+2 are issued, so that both the LDS stores and the load issue hide behind
  //     the remaining MFMA groups (16 MFMAs = 1024 cycles each) instead of sitting between the
  //     MFMA block and the barrier.  Where in the block the refill goes was measured per form on
  //     4096^3 (TFLOP/s at group 1 / at the last group): A*B 128.9 / 125.0, A*Bt 135.7 / 135.6,
  //     At*B 122.7 / 125.3;
  //   * MFMA fragments are read from LDS one k-group ahead of the MFMAs that consume them.
  // The scheduling barriers keep the compiler from sinking the reads and stores back down.
  load_stage(kt_begin);
  store_stage(0);
  if (kt_begin + 1 < kt_end) load_stage(kt_begin + 1);
  __syncthreads();

  for (int kt = kt_begin; kt < kt_end; ++kt) {
    const int s = (kt - kt_begin) & 1;
    float a[2][2][4], b[2][2][4];
    read_frag<!TA, BK>(a[0], lds_a[s], wm * 64, 0, r, h);
    read_frag<TB, BK>(b[0], lds_b[s], wn * 64, 0, r, h);
#pragma unroll
    for (int kk8 = 0; kk8 < KSTEPS; ++kk8) {
      const int cur = kk8 & 1, nxt = cur ^ 1;
      if (kk8 + 1 < KSTEPS) {
        read_frag<!TA, BK>(a[nxt], lds_a[s], wm * 64, kk8 + 1, r, h);
        read_frag<TB, BK>(b[nxt], lds_b[s], wn * 64, kk8 + 1, r, h);
      }
      if (kk8 == REFILL_AT) {
        // stage s^1 was last read in the previous iteration, which ended with a barrier
        if (kt + 1 < kt_end) store_stage(s ^ 1);
        if (kt + 2 < kt_end) load_stage(kt + 2);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][i][t], b[cur][j][t], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();  // stage s^1 is complete, stage s is free; also leaves LDS free for whoever runs next
  }
}

template <bool TA, bool TB, int BK>
__global__ __launch_bounds__(256, 2) void gemm_kernel(GemmArgs g) {
  constexpr int STAGE = Cfg<BK>::STAGE_FLOATS;
  __shared__ __attribute__((aligned(16))) float lds_a[2][STAGE];
  __shared__ __attribute__((aligned(16))) float lds_b[2][STAGE];

  unsigned tm, tn;
  tile_of_block(blockIdx.x, g.tiles_m, g.tiles_n, tm, tn);
  const size_t m0 = (size_t)tm * BM, n0 = (size_t)tn * BN;
  const size_t kbeg = (size_t)blockIdx.y * g.k_chunk;
  const size_t kend = kbeg + g.k_chunk < g.K ? kbeg + g.k_chunk : g.K;
  const int ktiles = (int)((kend - kbeg + BK - 1) / BK);
  const int kfull = (int)((kend - kbeg) / BK);  // complete tiles

  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = wave >> 1, wn = wave & 1;
  const int r = lane & 31, h = lane >> 5;

  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  // interior workgroups run their complete k tiles through the vector-load loop; edge tiles,
  // unaligned operands and the k remainder go through the checked loop
  const bool fast = g.a_vec && g.b_vec && m0 + BM <= g.M && n0 + BN <= g.N;
  const int nfast = fast ? kfull : 0;
  gemm_tiles<TA, TB, BK, true>(g, 0, nfast, kbeg, kend, m0, n0, lds_a, lds_b, acc);
  gemm_tiles<TA, TB, BK, false>(g, nfast, ktiles, kbeg, kend, m0, n0, lds_a, lds_b, acc);

  // Epilogue.  Accumulator register v of lane (r, h) in block (i, j) is
  //   row = 32*i + 8*(v/4) + 4*h + v%4,  col = 32*j + r   within the wave's 64x64 tile.
  const bool raw = g.splits > 1;
  float* dst = raw ? g.partial + (size_t)blockIdx.y * g.M * g.N : g.C;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const size_t col = n0 + wn * 64 + 32 * j + r;
      if (col >= g.N) continue;
      const float bv = (!raw && g.bias) ? g.bias[col] : 0.0f;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const size_t row = m0 + wm * 64 + 32 * i + 8 * (v / 4) + 4 * h + (v % 4);
        if (row >= g.M) continue;
        const size_t idx = row * g.N + col;
        float val = acc[i][j][v];
        if (!raw) {
          if (g.beta != 0.0f) val = g.beta * g.C[idx] + val;
          if (g.bias) val = val + bv;
          if (g.pre_act) g.pre_act[idx] = val;
          if (g.relu) val = (val >= 0.0f ? 1.0f : 0.0f) * val;
        }
        dst[idx] = val;
      }
    }
}

// C = sum_z partial[z] (z ascending) + beta*C, then bias / relu.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(size_t mn, size_t N, unsigned splits,
                                                            const float* __restrict__ partial, float* C, float beta,
                                                            const float* __restrict__ bias, int relu, float* pre_act,
                                                            int vec) {
  const size_t stride = (size_t)gridDim.x * 256;
  const size_t tid = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (vec) {
    for (size_t i = tid; i < (mn >> 2); i += stride) {
      float4 s = ld4(partial + 4 * i);
      for (unsigned z = 1; z < splits; ++z) {
        float4 p = ld4(partial + (size_t)z * mn + 4 * i);
        s.x += p.x; s.y += p.y; s.z += p.z; s.w += p.w;
      }
      if (beta != 0.0f) {
        float4 c = ld4(C + 4 * i);
        s.x = beta * c.x + s.x; s.y = beta * c.y + s.y; s.z = beta * c.z + s.z; s.w = beta * c.w + s.w;
      }
      if (bias) {
        float4 b = ld4(bias + (4 * i) % N);
        s.x += b.x; s.y += b.y; s.z += b.z; s.w += b.w;
      }
      if (pre_act) st4(pre_act + 4 * i, s);
      if (relu) {
        s.x = (s.x >= 0.f ? 1.f : 0.f) * s.x; s.y = (s.y >= 0.f ? 1.f : 0.f) * s.y;
        s.z = (s.z >= 0.f ? 1.f : 0.f) * s.z; s.w = (s.w >= 0.f ? 1.f : 0.f) * s.w;
      }
      st4(C + 4 * i, s);
    }
  } else {
    for (size_t i = tid; i < mn; i += stride) {
      float s = partial[i];
      for (unsigned z = 1; z < splits; ++z) s += partial[(size_t)z * mn + i];
      if (beta != 0.0f) s = beta * C[i] + s;
      if (bias) s += bias[i % N];
      if (pre_act) pre_act[i] = s;
      if (relu) s = (s >= 0.f ? 1.f : 0.f) * s;
      C[i] = s;
    }
  }
}

constexpr int GEMM_BK = 32;  // measured against 16: 3-10 % faster on every form at 2048^3 and above

static int32_t gemm_run(slhip_ctx* ctx, bool ta, bool tb, size_t M, size_t N, size_t K, const float* A, const float* B,
                        float* C, float beta, const float* bias, int relu, float* pre_act) {
  GemmArgs g;
  g.M = M; g.N = N; g.K = K; g.A = A; g.B = B; g.C = C; g.beta = beta;
  g.bias = bias; g.relu = relu; g.pre_act = pre_act;
  const size_t tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  if (tiles_m * tiles_n > 0x7fffffffu) {
    set_error("sgemm: %zu x %zu tiles exceed one launch", tiles_m, tiles_n);
    return SLHIP_EINVAL;
  }
  g.tiles_m = (unsigned)tiles_m; g.tiles_n = (unsigned)tiles_n;
  const size_t lda = ta ? M : K, ldb = tb ? K : N;
  g.a_vec = aligned16(A) && lda % 4 == 0;
  g.b_vec = aligned16(B) && ldb % 4 == 0;

  // Split K when the tile grid alone leaves CUs idle.  Two workgroups fit a CU, so the chip runs
  // `slots` workgroups at a time; pick the split count whose last round of workgroups is the
  // fullest (ties: the smaller count, which writes fewer partial results).
  const size_t tiles = tiles_m * tiles_n;
  const size_t slots = (size_t)ctx->num_cu * 2;
  size_t splits = 1;
  if (tiles < slots && K >= 512) {
    size_t max_splits = K / 128;  // every split keeps >= 128 of K
    if (max_splits > 32) max_splits = 32;
    const size_t fit = ctx->workspace_bytes / (M * N * sizeof(float));
    if (max_splits > fit) max_splits = fit;
    double best = 0.0;
    for (size_t sp = 1; sp <= max_splits; ++sp) {
      const size_t wgs = tiles * sp;
      const size_t rounds = (wgs + slots - 1) / slots;
      const double eff = (double)wgs / (double)(rounds * slots);
      if (eff > best + 1e-9) { best = eff; splits = sp; }
    }
  }
  constexpr int BK = GEMM_BK;
  size_t k_chunk = (K + splits - 1) / splits;
  k_chunk = (k_chunk + BK - 1) / BK * BK;
  if (k_chunk == 0) k_chunk = BK;
  splits = (K + k_chunk - 1) / k_chunk;
  if (splits < 1) splits = 1;
  g.splits = (unsigned)splits;
  g.k_chunk = k_chunk;
  g.partial = (float*)ctx->workspace;

  dim3 grid((unsigned)tiles, (unsigned)splits);
#define SL_GEMM(TA_, TB_) hipLaunchKernelGGL((gemm_kernel<TA_, TB_, GEMM_BK>), grid, dim3(256), 0, ctx->stream, g)
  if (!ta && !tb) SL_GEMM(false, false);
  else if (!ta && tb) SL_GEMM(false, true);
  else if (ta && !tb) SL_GEMM(true, false);
  else SL_GEMM(true, true);
#undef SL_GEMM
  int32_t rc = post_launch();
  if (rc || splits == 1) return rc;

  const size_t mn = M * N;
  const int vec = (mn % 4 == 0) && (N % 4 == 0) && aligned16(C) && (!bias || aligned16(bias)) &&
                  (!pre_act || aligned16(pre_act));
  size_t blocks = ((vec ? mn / 4 : mn) + 255) / 256;
  const size_t cap = (size_t)ctx->num_cu * 16;
  if (blocks > cap) blocks = cap;
  hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, mn, N, (unsigned)splits,
                     (const float*)ctx->workspace, C, beta, bias, relu, pre_act, vec);
  return post_launch();
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
  return gemm_run(ctx, trans_a != 0, trans_b != 0, m, n, k, a, b, c, beta, nullptr, 0, nullptr);
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

SLHIP_API int32_t slhip_linear_fwd(slhip_ctx* ctx, size_t m, size_t k, size_t n, const float* x, const float* w,
                                   const float* bias, int32_t relu, float* pre_act, float* out) {
  size_t mk, kn, mn;
  SLHIP_REQUIRE(ctx && x && w && out, "null argument");
  SLHIP_REQUIRE(checked_len(m, k, &mk) && checked_len(k, n, &kn) && checked_len(m, n, &mn), "bad dims");
  if (overlaps(out, mn, x, mk) || overlaps(out, mn, w, kn)) {
    set_error("slhip_linear_fwd: out overlaps an input");
    return SLHIP_EALIAS;
  }
  return gemm_run(ctx, false, false, m, n, k, x, w, out, 0.0f, bias, relu != 0, pre_act);
}
