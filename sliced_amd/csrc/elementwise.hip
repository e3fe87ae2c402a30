// Streaming kernels: binary / unary elementwise ops and their gradients, the fused elementwise
// chain, bias broadcast (row op), broadcast gradients of the reductions, SGD, cce, onehot.
//
// All of them are HBM-bound: one pass, one streaming float4 access per thread and operand.
// Arithmetic is unfused f32 (the file is compiled with -ffp-contract=off) so each op rounds
// exactly like the reference's scalar Rust loops.
#include "common.hpp"

namespace slhip {

constexpr int EW_BLOCK = 64;  // one wave per block: measured best for pure streaming

// Generic elementwise driver: ONE float4 per thread, no loop, as many blocks as it takes.  On
// MI355X this shape (with streaming loads/stores) sustains 6.2-6.6 TB/s on a 4-in/1-out chain,
// against 4.0-5.5 TB/s for grid-stride loops of any unroll depth.
// F::apply(const float in[NIN], float io[NOUT]) computes one element: io[] holds the current
// value of each output on entry when F::READS_OUT is set.
template <int NIN, int NOUT, class F>
struct EwArgs {
  const float* in[NIN > 0 ? NIN : 1];
  float* out[NOUT];
  F f;
};

template <int NIN, int NOUT, class F, bool VEC>
__global__ __launch_bounds__(EW_BLOCK) void ew_kernel(size_t n, EwArgs<NIN, NOUT, F> a) {
  const size_t t = (size_t)blockIdx.x * EW_BLOCK + threadIdx.x;
  if (VEC) {
    const size_t n4 = n >> 2;
    if (t < n4) {
      float4 vin[NIN > 0 ? NIN : 1];
      float4 vout[NOUT];
#pragma unroll
      for (int j = 0; j < NIN; ++j) vin[j] = ld4s(a.in[j] + 4 * t);
      if (F::READS_OUT) {
#pragma unroll
        for (int j = 0; j < NOUT; ++j) vout[j] = ld4s(a.out[j] + 4 * t);
      }
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        float si[NIN > 0 ? NIN : 1], so[NOUT];
#pragma unroll
        for (int j = 0; j < NIN; ++j) si[j] = (&vin[j].x)[c];
#pragma unroll
        for (int j = 0; j < NOUT; ++j) so[j] = F::READS_OUT ? (&vout[j].x)[c] : 0.0f;
        a.f.apply(si, so);
#pragma unroll
        for (int j = 0; j < NOUT; ++j) (&vout[j].x)[c] = so[j];
      }
#pragma unroll
      for (int j = 0; j < NOUT; ++j) st4s(a.out[j] + 4 * t, vout[j]);
    }
    if (t >= (n & 3)) return;  // the first n%4 threads also take one tail element each
  } else if (t >= n) {
    return;
  }
  const size_t i = VEC ? ((n >> 2) << 2) + t : t;
  float si[NIN > 0 ? NIN : 1], so[NOUT];
#pragma unroll
  for (int j = 0; j < NIN; ++j) si[j] = a.in[j][i];
#pragma unroll
  for (int j = 0; j < NOUT; ++j) so[j] = F::READS_OUT ? a.out[j][i] : 0.0f;
  a.f.apply(si, so);
#pragma unroll
  for (int j = 0; j < NOUT; ++j) a.out[j][i] = so[j];
}

template <int NIN, int NOUT, class F>
int32_t ew_launch(slhip_ctx* ctx, size_t n, EwArgs<NIN, NOUT, F> a) {
  if (n == 0) return SLHIP_OK;
  const bool vec = true;  // dword-aligned vector accesses: any float* qualifies
  const size_t threads = vec ? ((n >> 2) > 3 ? (n >> 2) : 4) : n;
  const size_t blocks = (threads + EW_BLOCK - 1) / EW_BLOCK;
  if (blocks > 0x7fffffffu) {
    set_error("elementwise: %zu elements exceed one launch", n);
    return SLHIP_EINVAL;
  }
  if (vec)
    hipLaunchKernelGGL((ew_kernel<NIN, NOUT, F, true>), dim3((unsigned)blocks), dim3(EW_BLOCK), 0, ctx->stream, n, a);
  else
    hipLaunchKernelGGL((ew_kernel<NIN, NOUT, F, false>), dim3((unsigned)blocks), dim3(EW_BLOCK), 0, ctx->stream, n, a);
  return post_launch();
}

// ------------------------------------------------------------------ functors
template <int OP>
struct BinF {
  static constexpr bool READS_OUT = false;
  __device__ __forceinline__ void apply(const float* in, float* o) const {
    float a = in[0], b = in[1];
    o[0] = OP == SLHIP_ADD ? a + b : OP == SLHIP_SUB ? a - b : OP == SLHIP_MUL ? a * b : a / b;
  }
};

// in: l, r, g ; out: lg and/or rg (WHICH: 1 = lhs only, 2 = rhs only, 3 = both -> out[0]=lg, out[1]=rg)
template <int OP, int WHICH>
struct BinGradF {
  static constexpr bool READS_OUT = true;
  __device__ __forceinline__ void apply(const float* in, float* o) const {
    float l = in[0], r = in[1], g = in[2];
    float dl, dr;
    if (OP == SLHIP_ADD) { dl = 1.0f; dr = 1.0f; }
    else if (OP == SLHIP_SUB) { dl = 1.0f; dr = -1.0f; }
    else if (OP == SLHIP_MUL) { dl = r; dr = l; }
    else { dl = 1.0f / r; dr = -l / (r * r); }
    if (WHICH == 1) o[0] += dl * g;
    else if (WHICH == 2) o[0] += dr * g;
    else { o[0] += dl * g; o[1] += dr * g; }
  }
};

__device__ __forceinline__ float pow_ref(float x, float p) {
  // The exponents the tape actually uses are exact products / roots (correctly rounded, and
  // two orders of magnitude cheaper than the general routine, which would make the streaming
  // kernels ALU-bound).  Everything else goes through powf proper, which keeps integer
  // exponents of negative bases finite.
  if (p == 2.0f) return x * x;
  if (p == 1.0f) return x;
  // powf(-inf, 0.5) is +inf and powf(-0, 0.5) is +0 where the square root has NaN and -0
  if (p == 0.5f) return x == -__builtin_huge_valf() ? __builtin_huge_valf() : sqrtf(x) + 0.0f;
  return powf(x, p);
}

template <int OP>
struct UnF {
  static constexpr bool READS_OUT = false;
  float p, q;
  __device__ __forceinline__ void apply(const float* in, float* o) const {
    float x = in[0];
    switch (OP) {
      case SLHIP_SQUARE: o[0] = x * x; break;
      case SLHIP_POW: o[0] = pow_ref(x, p); break;
      case SLHIP_RELU: o[0] = (x >= 0.0f ? 1.0f : 0.0f) * x; break;  // -0.0 for x<0, as geq(0)*x
      case SLHIP_EXP: o[0] = expf(x); break;
      case SLHIP_CLIP: o[0] = fminf(fmaxf(x, p), q); break;
      case SLHIP_NEG_LN: o[0] = -logf(x); break;
      case SLHIP_SCALE: o[0] = x * p; break;
      case SLHIP_TANH: o[0] = tanhf(x); break;
      case SLHIP_SIGMOID: o[0] = 1.0f / (1.0f + expf(-x)); break;
      default: o[0] = (-x) / p; break;
    }
  }
};

// in: x, g ; out: x_grad (+=)
template <int OP>
struct UnGradF {
  static constexpr bool READS_OUT = true;
  float p;
  __device__ __forceinline__ void apply(const float* in, float* o) const {
    float x = in[0], g = in[1], d;
    switch (OP) {
      case SLHIP_SQUARE: d = x * 2.0f; break;
      case SLHIP_POW: d = pow_ref(x, p - 1.0f) * p; break;
      case SLHIP_RELU: d = x >= 0.0f ? 1.0f : 0.0f; break;
      case SLHIP_EXP: d = expf(x); break;
      case SLHIP_TANH: { const float t = tanhf(x); d = 1.0f - t * t; break; }
      case SLHIP_SIGMOID: { const float e = expf(-x); const float s = 1.0f + e; d = e / (s * s); break; }
      default: d = p; break;  // SLHIP_SCALE
    }
    o[0] += d * g;
  }
};

struct ChainF {  // ((a+b)*c - d) -> pow 2 -> square
  static constexpr bool READS_OUT = false;
  __device__ __forceinline__ void apply(const float* in, float* o) const {
    float t = (in[0] + in[1]) * in[2] - in[3];
    float u = pow_ref(t, 2.0f);
    o[0] = u * u;
  }
};

struct SgdF {  // p -= g * lr
  static constexpr bool READS_OUT = true;
  float lr;
  __device__ __forceinline__ void apply(const float* in, float* o) const { o[0] -= in[0] * lr; }
};

struct CceGradF {  // (-(t/p)) / rows ; in: p, t
  static constexpr bool READS_OUT = false;
  float rows;
  __device__ __forceinline__ void apply(const float* in, float* o) const { o[0] = (-(in[1] / in[0])) / rows; }
};

// ------------------------------------------------------------------ broadcast kernels
// MODE 0: out[r,c]  = lhs[r,c] + v[c]          (add_row / add_row_mut)
// MODE 1: xg[r,c]  += s * v[c]                  (sum_rows_grad s=1, mean_rows_grad s=cols/len)
// MODE 2: xg[r,c]  += v[r] (or v[r]/s)          (sum_cols_grad; mean_cols_grad with DIVCOLS)
// MODE 3: xg[r,c]  += (x[r,c]==v[c]) ? g[c] : 0 (max_rows_grad; v = out)
// One vector per thread over the flat (row, column-vector) index space; the matrix streams
// through once, the broadcast vector stays in cache.
template <int MODE, bool VEC, bool DIVCOLS, class IDX>
__global__ __launch_bounds__(EW_BLOCK) void bcast_kernel(size_t rows, size_t cols, const float* a,
                                                         const float* __restrict__ v, const float* __restrict__ g,
                                                         float* out, float s) {
  constexpr int V = VEC ? 4 : 1;
  const IDX colsv = (IDX)(cols / V);
  const size_t i = (size_t)blockIdx.x * EW_BLOCK + threadIdx.x;
  if (i >= rows * (size_t)colsv) return;
  const IDX r = (IDX)i / colsv;          // 32-bit division whenever the index space allows it
  const IDX cv = (IDX)i - r * colsv;
  const size_t c = (size_t)cv * V;
  const size_t off = (size_t)r * cols + c;
  float vv[4], o[4], av[4], gv[4];
  if (VEC) {
    float4 t;
    if (MODE == 0 || MODE == 3) { t = ld4s(a + off); av[0] = t.x; av[1] = t.y; av[2] = t.z; av[3] = t.w; }
    if (MODE != 0) { t = ld4s(out + off); o[0] = t.x; o[1] = t.y; o[2] = t.z; o[3] = t.w; }
    if (MODE == 2) { vv[0] = vv[1] = vv[2] = vv[3] = DIVCOLS ? v[r] / s : v[r]; }
    else { t = ld4g(v + c); vv[0] = t.x; vv[1] = t.y; vv[2] = t.z; vv[3] = t.w; }
    if (MODE == 3) { t = ld4g(g + c); gv[0] = t.x; gv[1] = t.y; gv[2] = t.z; gv[3] = t.w; }
  } else {
    if (MODE == 0 || MODE == 3) av[0] = a[off];
    if (MODE != 0) o[0] = out[off];
    vv[0] = MODE == 2 ? (DIVCOLS ? v[r] / s : v[r]) : v[c];
    if (MODE == 3) gv[0] = g[c];
  }
#pragma unroll
  for (int j = 0; j < V; ++j) {
    if (MODE == 0) o[j] = av[j] + vv[j];
    else if (MODE == 1) o[j] += s * vv[j];
    else if (MODE == 2) o[j] += vv[j];
    else if (av[j] == vv[j]) o[j] += gv[j];
  }
  if (VEC) st4s(out + off, make_float4(o[0], o[1], o[2], o[3]));
  else out[off] = o[0];
}

// Rows of odd length: the matrix is walked as one flat run of vectors, each element finds its
// own row and column (one division per thread, then increments).
template <int MODE, bool DIVCOLS, class IDX>
__global__ __launch_bounds__(EW_BLOCK) void bcast_flat_kernel(size_t len, size_t cols, const float* a,
                                                              const float* __restrict__ v, const float* __restrict__ g,
                                                              float* out, float s) {
  const size_t i = (size_t)blockIdx.x * EW_BLOCK + threadIdx.x;
  const size_t e0 = 4 * i;
  if (e0 >= len) return;
  IDX r = (IDX)e0 / (IDX)cols;
  IDX c = (IDX)e0 - r * (IDX)cols;
  const bool whole = e0 + 3 < len;
  float av[4] = {0.f, 0.f, 0.f, 0.f}, o[4] = {0.f, 0.f, 0.f, 0.f};
  if (whole) {
    float4 t;
    if (MODE == 0 || MODE == 3) { t = ld4s(a + e0); av[0] = t.x; av[1] = t.y; av[2] = t.z; av[3] = t.w; }
    if (MODE != 0) { t = ld4s(out + e0); o[0] = t.x; o[1] = t.y; o[2] = t.z; o[3] = t.w; }
  } else {
    for (size_t q = 0; e0 + q < len; ++q) {
      if (MODE == 0 || MODE == 3) av[q] = a[e0 + q];
      if (MODE != 0) o[q] = out[e0 + q];
    }
  }
  // the broadcast entries of the four elements: one vector load where they lie in one row (a thread
  // that gathers them one by one streams a matrix of odd row length at 4.0-4.6 TB/s)
  float vv[4] = {0.f, 0.f, 0.f, 0.f}, gv[4] = {0.f, 0.f, 0.f, 0.f};
  if (MODE != 2 && whole && (size_t)c + 3 < cols) {
    float4 t = ld4g(v + c);
    vv[0] = t.x; vv[1] = t.y; vv[2] = t.z; vv[3] = t.w;
    if (MODE == 3) { t = ld4g(g + c); gv[0] = t.x; gv[1] = t.y; gv[2] = t.z; gv[3] = t.w; }
  } else {
    IDX rq = r, cq = c;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (e0 + q < len) {
        vv[q] = MODE == 2 ? v[rq] : v[cq];
        if (MODE == 3) gv[q] = g[cq];
      }
      if (++cq == (IDX)cols) { cq = 0; ++rq; }
    }
  }
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    if (e0 + q < len) {
      if (MODE == 0) o[q] = av[q] + vv[q];
      else if (MODE == 1) o[q] += s * vv[q];
      else if (MODE == 2) o[q] += DIVCOLS ? vv[q] / s : vv[q];
      else if (av[q] == vv[q]) o[q] += gv[q];
    }
  }
  if (whole) st4s(out + e0, make_float4(o[0], o[1], o[2], o[3]));
  else
    for (size_t q = 0; e0 + q < len; ++q) out[e0 + q] = o[q];
}

template <int MODE, bool DIVCOLS = false>
int32_t bcast_launch(slhip_ctx* ctx, size_t rows, size_t cols, const float* a, const float* v, const float* g,
                     float* out, float s) {
  const bool vec = cols % 4 == 0;  // a thread's vector lies inside one row; alignment does not matter
  const size_t total = vec ? rows * (cols / 4) : (rows * cols + 3) / 4;
  const size_t blocks = (total + EW_BLOCK - 1) / EW_BLOCK;
  if (blocks > 0x7fffffffu) {
    set_error("broadcast op: %zu x %zu exceeds one launch", rows, cols);
    return SLHIP_EINVAL;
  }
  const bool small = rows * cols <= 0xffffffffu;  // 32-bit index arithmetic whenever the matrix allows it
  if (vec) {
#define SL_BC(IDXT)                                                                                                  \
  hipLaunchKernelGGL((bcast_kernel<MODE, true, DIVCOLS, IDXT>), dim3((unsigned)blocks), dim3(EW_BLOCK), 0, ctx->stream, \
                     rows, cols, a, v, g, out, s)
    if (small) SL_BC(uint32_t); else SL_BC(size_t);
#undef SL_BC
  } else {
#define SL_BF(IDXT)                                                                                                      \
  hipLaunchKernelGGL((bcast_flat_kernel<MODE, DIVCOLS, IDXT>), dim3((unsigned)blocks), dim3(EW_BLOCK), 0, ctx->stream, \
                     rows * cols, cols, a, v, g, out, s)
    if (small) SL_BF(uint32_t); else SL_BF(size_t);
#undef SL_BF
  }
  return post_launch();
}

// One vector of four outputs per thread, the matrix walked as one flat run (any class count): a
// thread finds the row and class of its first element with one division and steps from there.
// (One scalar store per thread wrote [13M x 10] at 2.1 TB/s.)
template <class IDX>
__global__ __launch_bounds__(256) void onehot_kernel(size_t n, size_t classes, const float* __restrict__ cls,
                                                     float* __restrict__ out) {
  const size_t len = n * classes;
  const size_t e0 = 4 * ((size_t)blockIdx.x * 256 + threadIdx.x);
  if (e0 >= len) return;
  IDX r = (IDX)e0 / (IDX)classes;
  IDX c = (IDX)e0 - r * (IDX)classes;
  float cur = cls[r];
  float o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    if (e0 + q < len) o[q] = ((size_t)cur == (size_t)c) ? 1.0f : 0.0f;
    if (++c == (IDX)classes) {
      c = 0;
      ++r;
      if ((size_t)r < n) cur = cls[r];
    }
  }
  if (e0 + 3 < len) st4s(out + e0, make_float4(o[0], o[1], o[2], o[3]));
  else
    for (size_t q = 0; e0 + q < len; ++q) out[e0 + q] = o[q];
}

}  // namespace slhip

using namespace slhip;

// ---------------------------------------------------------------------------- C ABI
SLHIP_API int32_t slhip_ew_binary(slhip_ctx* ctx, int32_t op, size_t n, const float* l, const float* r, float* out) {
  SLHIP_REQUIRE(ctx && l && r && out, "null argument");
  SLHIP_REQUIRE(n > 0, "empty buffer");
#define SL_BIN(OP)                                   \
  case OP: {                                         \
    EwArgs<2, 1, BinF<OP>> a{{l, r}, {out}, {}};     \
    return ew_launch(ctx, n, a);                     \
  }
  switch (op) {
    SL_BIN(SLHIP_ADD) SL_BIN(SLHIP_SUB) SL_BIN(SLHIP_MUL) SL_BIN(SLHIP_DIV)
    default: break;
  }
#undef SL_BIN
  set_error("slhip_ew_binary: unknown op %d", op);
  return SLHIP_EINVAL;
}

template <int OP>
static int32_t bin_grad(slhip_ctx* ctx, size_t n, const float* l, const float* r, float* lg, float* rg,
                        const float* g) {
  if (lg && rg) {
    EwArgs<3, 2, BinGradF<OP, 3>> a{{l, r, g}, {lg, rg}, {}};
    return ew_launch(ctx, n, a);
  } else if (lg) {
    EwArgs<3, 1, BinGradF<OP, 1>> a{{l, r, g}, {lg}, {}};
    return ew_launch(ctx, n, a);
  } else if (rg) {
    EwArgs<3, 1, BinGradF<OP, 2>> a{{l, r, g}, {rg}, {}};
    return ew_launch(ctx, n, a);
  }
  return SLHIP_OK;
}

SLHIP_API int32_t slhip_ew_binary_grad(slhip_ctx* ctx, int32_t op, size_t n, const float* l, const float* r,
                                       float* lg, float* rg, const float* g) {
  SLHIP_REQUIRE(ctx && l && r && g, "null argument");
  SLHIP_REQUIRE(n > 0, "empty buffer");
  if (lg && lg == rg) {
    set_error("slhip_ew_binary_grad: lhs_grad and rhs_grad alias");
    return SLHIP_EALIAS;
  }
  switch (op) {
    case SLHIP_ADD: return bin_grad<SLHIP_ADD>(ctx, n, l, r, lg, rg, g);
    case SLHIP_SUB: return bin_grad<SLHIP_SUB>(ctx, n, l, r, lg, rg, g);
    case SLHIP_MUL: return bin_grad<SLHIP_MUL>(ctx, n, l, r, lg, rg, g);
    case SLHIP_DIV: return bin_grad<SLHIP_DIV>(ctx, n, l, r, lg, rg, g);
    default: break;
  }
  set_error("slhip_ew_binary_grad: unknown op %d", op);
  return SLHIP_EINVAL;
}

SLHIP_API int32_t slhip_ew_unary(slhip_ctx* ctx, int32_t op, float p, float q, size_t n, const float* x, float* out) {
  SLHIP_REQUIRE(ctx && x && out, "null argument");
  SLHIP_REQUIRE(n > 0, "empty buffer");
#define SL_UN(OP)                                    \
  case OP: {                                         \
    EwArgs<1, 1, UnF<OP>> a{{x}, {out}, {p, q}};     \
    return ew_launch(ctx, n, a);                     \
  }
  switch (op) {
    SL_UN(SLHIP_SQUARE) SL_UN(SLHIP_POW) SL_UN(SLHIP_RELU) SL_UN(SLHIP_EXP) SL_UN(SLHIP_CLIP)
    SL_UN(SLHIP_NEG_LN) SL_UN(SLHIP_SCALE) SL_UN(SLHIP_NEG_DIV) SL_UN(SLHIP_TANH) SL_UN(SLHIP_SIGMOID)
    default: break;
  }
#undef SL_UN
  set_error("slhip_ew_unary: unknown op %d", op);
  return SLHIP_EINVAL;
}

SLHIP_API int32_t slhip_ew_unary_grad(slhip_ctx* ctx, int32_t op, float p, size_t n, const float* x, float* x_grad,
                                      const float* out_grad) {
  SLHIP_REQUIRE(ctx && x && x_grad && out_grad, "null argument");
  SLHIP_REQUIRE(n > 0, "empty buffer");
#define SL_UNG(OP)                                              \
  case OP: {                                                    \
    EwArgs<2, 1, UnGradF<OP>> a{{x, out_grad}, {x_grad}, {p}};  \
    return ew_launch(ctx, n, a);                                \
  }
  switch (op) {
    SL_UNG(SLHIP_SQUARE) SL_UNG(SLHIP_POW) SL_UNG(SLHIP_RELU) SL_UNG(SLHIP_EXP) SL_UNG(SLHIP_SCALE)
    SL_UNG(SLHIP_TANH) SL_UNG(SLHIP_SIGMOID)
    default: break;
  }
#undef SL_UNG
  set_error("slhip_ew_unary_grad: op %d has no gradient", op);
  return SLHIP_EINVAL;
}

SLHIP_API int32_t slhip_ew_chain(slhip_ctx* ctx, size_t n, const float* a, const float* b, const float* c,
                                 const float* d, float* out) {
  SLHIP_REQUIRE(ctx && a && b && c && d && out, "null argument");
  SLHIP_REQUIRE(n > 0, "empty buffer");
  EwArgs<4, 1, ChainF> args{{a, b, c, d}, {out}, {}};
  return ew_launch(ctx, n, args);
}

SLHIP_API int32_t slhip_sgd_step(slhip_ctx* ctx, size_t n, float* p, const float* g, float lr) {
  SLHIP_REQUIRE(ctx && p && g, "null argument");
  SLHIP_REQUIRE(n > 0, "empty buffer");
  EwArgs<1, 1, SgdF> a{{g}, {p}, {lr}};
  return ew_launch(ctx, n, a);
}

// Up to SGD_MULTI_MAX parameter tensors per launch; blockIdx.y picks the tensor.
constexpr int SGD_MULTI_MAX = 8;
struct SgdMultiArgs {
  float* p[SGD_MULTI_MAX];
  const float* g[SGD_MULTI_MAX];
  size_t n[SGD_MULTI_MAX];
  int vec[SGD_MULTI_MAX];
};

__global__ __launch_bounds__(256) void sgd_multi_kernel(SgdMultiArgs a, float lr) {
  const int t = blockIdx.y;
  float* __restrict__ p = a.p[t];
  const float* __restrict__ g = a.g[t];
  const size_t n = a.n[t];
  const size_t tid = (size_t)blockIdx.x * 256 + threadIdx.x, stride = (size_t)gridDim.x * 256;
  size_t done = 0;
  if (a.vec[t]) {
    const size_t n4 = n / 4;
    for (size_t i = tid; i < n4; i += stride) {
      float4 pv = ld4g(p + 4 * i);
      const float4 gv = ld4g(g + 4 * i);
      pv.x -= gv.x * lr; pv.y -= gv.y * lr; pv.z -= gv.z * lr; pv.w -= gv.w * lr;
      st4g(p + 4 * i, pv);
    }
    done = n4 * 4;
  }
  for (size_t i = done + tid; i < n; i += stride) p[i] -= g[i] * lr;
}

SLHIP_API int32_t slhip_sgd_step_multi(slhip_ctx* ctx, size_t count, float* const* params, const float* const* grads,
                                       const size_t* lens, float lr) {
  SLHIP_REQUIRE(ctx && params && grads && lens, "null argument");
  SLHIP_REQUIRE(count > 0, "no tensors");
  for (size_t i = 0; i < count; ++i) SLHIP_REQUIRE(params[i] && grads[i] && lens[i] > 0, "null or empty tensor");
  for (size_t first = 0; first < count; first += SGD_MULTI_MAX) {
    const size_t m = count - first < (size_t)SGD_MULTI_MAX ? count - first : (size_t)SGD_MULTI_MAX;
    SgdMultiArgs a;
    size_t longest = 0;
    for (size_t i = 0; i < (size_t)SGD_MULTI_MAX; ++i) {
      const size_t j = first + (i < m ? i : 0);  // unused slots repeat the first tensor; no block reads them
      a.p[i] = params[j]; a.g[i] = grads[j]; a.n[i] = lens[j];
      a.vec[i] = 1;
      if (i < m && lens[j] > longest) longest = lens[j];
    }
    size_t blocks = (longest / 4 + 255) / 256 + 1;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(sgd_multi_kernel, dim3((unsigned)blocks, (unsigned)m), dim3(256), 0, ctx->stream, a, lr);
    int32_t rc = post_launch();
    if (rc) return rc;
  }
  return SLHIP_OK;
}

SLHIP_API int32_t slhip_add_row(slhip_ctx* ctx, size_t rows, size_t cols, const float* lhs, const float* rhs,
                                float* out) {
  size_t len;
  SLHIP_REQUIRE(ctx && lhs && rhs && out, "null argument");
  SLHIP_REQUIRE(checked_len(rows, cols, &len), "bad dims");
  return bcast_launch<0>(ctx, rows, cols, lhs, rhs, nullptr, out, 0.0f);
}

SLHIP_API int32_t slhip_sum_rows_grad(slhip_ctx* ctx, size_t rows, size_t cols, float* x_grad, const float* out_grad) {
  size_t len;
  SLHIP_REQUIRE(ctx && x_grad && out_grad, "null argument");
  SLHIP_REQUIRE(checked_len(rows, cols, &len), "bad dims");
  return bcast_launch<1>(ctx, rows, cols, nullptr, out_grad, nullptr, x_grad, 1.0f);
}

SLHIP_API int32_t slhip_mean_rows_grad(slhip_ctx* ctx, size_t rows, size_t cols, float* x_grad, const float* out_grad) {
  size_t len;
  SLHIP_REQUIRE(ctx && x_grad && out_grad, "null argument");
  SLHIP_REQUIRE(checked_len(rows, cols, &len), "bad dims");
  return bcast_launch<1>(ctx, rows, cols, nullptr, out_grad, nullptr, x_grad, (float)cols / (float)len);
}

SLHIP_API int32_t slhip_sum_cols_grad(slhip_ctx* ctx, size_t rows, size_t cols, float* x_grad, const float* out_grad) {
  size_t len;
  SLHIP_REQUIRE(ctx && x_grad && out_grad, "null argument");
  SLHIP_REQUIRE(checked_len(rows, cols, &len), "bad dims");
  return bcast_launch<2>(ctx, rows, cols, nullptr, out_grad, nullptr, x_grad, 1.0f);
}

SLHIP_API int32_t slhip_mean_cols_grad(slhip_ctx* ctx, size_t rows, size_t cols, float* x_grad, const float* out_grad) {
  size_t len;
  SLHIP_REQUIRE(ctx && x_grad && out_grad, "null argument");
  SLHIP_REQUIRE(checked_len(rows, cols, &len), "bad dims");
  return bcast_launch<2, true>(ctx, rows, cols, nullptr, out_grad, nullptr, x_grad, (float)cols);
}

SLHIP_API int32_t slhip_max_rows_grad(slhip_ctx* ctx, size_t rows, size_t cols, const float* out, const float* x,
                                      float* x_grad, const float* out_grad) {
  size_t len;
  SLHIP_REQUIRE(ctx && out && x && x_grad && out_grad, "null argument");
  SLHIP_REQUIRE(checked_len(rows, cols, &len), "bad dims");
  return bcast_launch<3>(ctx, rows, cols, x, out, out_grad, x_grad, 0.0f);
}

SLHIP_API int32_t slhip_cce(slhip_ctx* ctx, size_t rows, size_t cols, const float* preds, const float* targets,
                            float* loss) {
  size_t len;
  SLHIP_REQUIRE(ctx && preds && targets && loss, "null argument");
  SLHIP_REQUIRE(checked_len(rows, cols, &len), "bad dims");
  return cce_rows_reduce(ctx, rows, cols, preds, targets, loss);
}

SLHIP_API int32_t slhip_cce_grad(slhip_ctx* ctx, size_t rows, size_t cols, const float* preds, const float* targets,
                                 float* grad) {
  size_t len;
  SLHIP_REQUIRE(ctx && preds && targets && grad, "null argument");
  SLHIP_REQUIRE(checked_len(rows, cols, &len), "bad dims");
  EwArgs<2, 1, CceGradF> a{{preds, targets}, {grad}, {(float)rows}};
  return ew_launch(ctx, len, a);
}

SLHIP_API int32_t slhip_onehot(slhip_ctx* ctx, size_t n, size_t classes, const float* cls, float* out) {
  size_t len;
  SLHIP_REQUIRE(ctx && cls && out, "null argument");
  SLHIP_REQUIRE(checked_len(n, classes, &len), "bad dims");
  SLHIP_REQUIRE(grid_fits((len + 3) / 4, 256), "too many elements for one launch");
  if (len <= 0xffffffffu)
    hipLaunchKernelGGL((onehot_kernel<uint32_t>), dim3(ceil_div((len + 3) / 4, 256)), dim3(256), 0, ctx->stream, n, classes, cls, out);
  else
    hipLaunchKernelGGL((onehot_kernel<size_t>), dim3(ceil_div((len + 3) / 4, 256)), dim3(256), 0, ctx->stream, n, classes, cls, out);
  return post_launch();
}
