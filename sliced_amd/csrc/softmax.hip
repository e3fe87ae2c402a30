// Row-wise softmax, forward and backward, as single-pass kernels: a row is loaded once into
// registers (float4 per lane), reduced with wave64 shuffles (plus LDS across waves for long
// rows), and written once.  Forward moves 8 B/element, backward 12 B/element (+4 when it
// accumulates) - the algorithmic minimum.
//
// The reference builds the forward from five passes (max_cols, sub_cols, exp, sum_cols,
// div_cols) and the backward from a per-sample Jacobian; the arithmetic per element is the
// same: e = exp(x - max); out = e / sum(e);  x_grad = s * (g - <s, g>).
#include <numeric>

#include "common.hpp"

namespace slhip {

// Reduce over the LANES threads that share a row (LANES <= 64: shuffles; else: whole block).
// Across waves: one barrier per reduction.  Every wave leaves its partial in its own slot of
// `smem` (a different 16-float slot group per call site, so no barrier is needed before the
// slots are written again) and every thread folds all the partials itself.
template <class Op, int LANES>
__device__ __forceinline__ float row_reduce(float v, float* smem) {
  if (LANES <= 64) return wave_reduce<Op, (LANES <= 64 ? LANES : 64)>(v);
  constexpr int NW = LANES / 64;
  v = wave_reduce<Op>(v);
  if ((threadIdx.x & 63) == 0) smem[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = smem[0];
#pragma unroll
  for (int w = 1; w < NW; ++w) r = Op::apply(r, smem[w]);
  return r;
}

// TAIL: the row length is not a multiple of 4 (VEC only): lane 0 also takes the up to 3 floats
// beyond the last whole vector.  A template parameter because even an untaken tail costs the
// whole-vector rows 10-15 % of their bandwidth.
//
// CCE: the categorical cross-entropy of every row against the targets tg rides along,
// loss_rows[r] = -ln sum_c clip(p, 1e-7, 1 - 1e-7) * tg (reference: Matrix::softmax followed by cce,
// examples/nn.rs:124-143); out may then be null (the probabilities are not stored).
__device__ __forceinline__ float cce_term(float p, float t) { return fminf(fmaxf(p, (float)1e-7), (float)(1.0 - 1e-7)) * t; }
// (512 lanes with sixteen vectors each: two rows a CU need four waves a SIMD, i.e. at most 128 VGPRs;
// the form with a tail came out at 3 waves otherwise - rows of 20001 floats 3.8 TB/s against 5.6 for
// rows of 20000)
template <bool VEC, int LANES, int ITEMS, bool TAIL, bool CCE>
__global__ __launch_bounds__(LANES <= 64 ? 256 : LANES, (LANES == 512 && ITEMS == 16) ? 4 : 1) void softmax_fwd_kernel(size_t rows, size_t cols,
                                                                                const float* __restrict__ x,
                                                                                float* __restrict__ out,
                                                                                const float* __restrict__ tg,
                                                                                float* __restrict__ loss_rows) {
  __shared__ float smem[32];
  constexpr int V = VEC ? 4 : 1;
  constexpr int RPB = LANES <= 64 ? 256 / LANES : 1;
  const size_t colsv = cols / V;
  const int lane = threadIdx.x % LANES;
  const size_t row = (size_t)blockIdx.x * RPB + threadIdx.x / LANES;
  const bool active = row < rows;
  const float NEG_INF = -__builtin_huge_valf();

  float v[ITEMS][V];
  float w[CCE ? ITEMS : 1][V];  // the targets of the same elements
  float m = NEG_INF;
  // every lane of the row holds ITEMS full vectors: unconditional loads, all in flight together
  const bool full = active && (size_t)LANES * ITEMS <= colsv;
  if (VEC && full) {
    float4 t[ITEMS], u[CCE ? ITEMS : 1];
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      t[j] = ld4s(x + row * cols + 4 * ((size_t)lane + (size_t)j * LANES));
      if (CCE) u[j] = ld4s(tg + row * cols + 4 * ((size_t)lane + (size_t)j * LANES));
    }
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      v[j][0] = t[j].x; v[j][V > 1 ? 1 : 0] = t[j].y; v[j][V > 1 ? 2 : 0] = t[j].z; v[j][V > 1 ? 3 : 0] = t[j].w;
      if (CCE) { w[j][0] = u[j].x; w[j][V > 1 ? 1 : 0] = u[j].y; w[j][V > 1 ? 2 : 0] = u[j].z; w[j][V > 1 ? 3 : 0] = u[j].w; }
    }
  } else {
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      const size_t c = (size_t)lane + (size_t)j * LANES;
      if (active && c < colsv) {
        if (VEC) {
          float4 t = ld4s(x + row * cols + 4 * c);
          v[j][0] = t.x; v[j][V > 1 ? 1 : 0] = t.y; v[j][V > 1 ? 2 : 0] = t.z; v[j][V > 1 ? 3 : 0] = t.w;
          if (CCE) {
            t = ld4s(tg + row * cols + 4 * c);
            w[j][0] = t.x; w[j][V > 1 ? 1 : 0] = t.y; w[j][V > 1 ? 2 : 0] = t.z; w[j][V > 1 ? 3 : 0] = t.w;
          }
        } else {
          v[j][0] = x[row * cols + c];
          if (CCE) w[j][0] = tg[row * cols + c];
        }
      } else {
#pragma unroll
        for (int q = 0; q < V; ++q) {
          v[j][q] = NEG_INF;
          if (CCE) w[j][q] = 0.0f;
        }
      }
    }
  }
  // a row of odd length ends in up to 3 floats beyond its last whole vector
  const int rem = TAIL ? (int)(cols & 3) : 0;
  // (from four lanes a row on, lane q takes the q-th of them: one float each, no loop)
  constexpr bool SPREAD = LANES >= 4;
  const bool tail = TAIL && active && (SPREAD ? lane < rem : (rem != 0 && lane == 0));
  const int tq0 = SPREAD ? lane : 0, tq1 = SPREAD ? lane + 1 : rem;  // this lane's share of the tail
  float tv[3] = {NEG_INF, NEG_INF, NEG_INF};
  if (tail)
    for (int q = tq0; q < tq1; ++q) tv[q - tq0] = x[row * cols + 4 * colsv + q];
#pragma unroll
  for (int j = 0; j < ITEMS; ++j)
#pragma unroll
    for (int q = 0; q < V; ++q) m = fmaxf(m, v[j][q]);
  if (TAIL) m = fmaxf(m, fmaxf(tv[0], fmaxf(tv[1], tv[2])));
  m = row_reduce<MaxOp, LANES>(m, smem);

  float s = 0.0f;
#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    const size_t c = (size_t)lane + (size_t)j * LANES;
    const bool in = active && c < colsv;
#pragma unroll
    for (int q = 0; q < V; ++q) {
      float e = in ? expf(v[j][q] - m) : 0.0f;
      v[j][q] = e;
      s += e;
    }
  }
  if (tail)
    for (int q = tq0; q < tq1; ++q) {
      tv[q - tq0] = expf(tv[q - tq0] - m);
      s += tv[q - tq0];
    }
  s = row_reduce<SumOp, LANES>(s, smem + 16);
  // e * (1 / sum) where the reference divides by the sum: at most 1.5 ulp from the quotient.  The
  // kernel is close to ALU-bound on the exponential and the division wherever lanes idle or rows end
  // in a scalar tail (+3 % on rows of 16384 floats, +5-7 % on rows of 257, 513 and 1030).
  const float inv = 1.0f / s;
  auto scale = [&](float e) { return e * inv; };
  if (CCE) {
    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < ITEMS; ++j)
#pragma unroll
      for (int q = 0; q < V; ++q) acc += cce_term(scale(v[j][q]), w[j][q]);  // (elements outside the row: e = 0, t = 0)
    if (tail)
      for (int q = tq0; q < tq1; ++q) acc += cce_term(scale(tv[q - tq0]), tg[row * cols + 4 * colsv + q]);
    acc = row_reduce<SumOp, LANES>(acc, smem);  // (every lane is past its reads of the first reduction)
    if (active && lane == 0) loss_rows[row] = -logf(acc);
    if (!out) return;
  }
  if (tail)
    for (int q = tq0; q < tq1; ++q) out[row * cols + 4 * colsv + q] = scale(tv[q - tq0]);

#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    const size_t c = (size_t)lane + (size_t)j * LANES;
    if (active && c < colsv) {
      if (VEC) st4s(out + row * cols + 4 * c, make_float4(scale(v[j][0]), scale(v[j][V > 1 ? 1 : 0]), scale(v[j][V > 1 ? 2 : 0]),
                                                        scale(v[j][V > 1 ? 3 : 0])));
      else out[row * cols + c] = scale(v[j][0]);
    }
  }
}

// What the backward kernels make of a row (s, g): the softmax gradient s * (g - <s, g>), or, with
// s = the probabilities and g = the targets, the gradient of the mean cross-entropy pushed through
// the softmax in closed form, (p * sum_c t - t) * (upstream / rows) (reference: cce_grad followed by
// softmax_grad, examples/nn.rs:145-152, which divides by p and yields inf * 0 when p underflows).
struct SoftmaxGradForm {
  __device__ __forceinline__ float term(float s, float g) const { return s * g; }
  __device__ __forceinline__ float k() const { return 0.0f; }
  __device__ __forceinline__ float result(float s, float g, float red, float) const { return s * (g - red); }
};
struct CceGradForm {
  const float* upstream;
  float rows;
  __device__ __forceinline__ float term(float, float g) const { return g; }
  __device__ __forceinline__ float k() const { return upstream[0] / rows; }
  __device__ __forceinline__ float result(float s, float g, float red, float kk) const { return (s * red - g) * kk; }
};

template <bool VEC, int LANES, int ITEMS, bool TAIL, class RG>
__global__ __launch_bounds__(LANES <= 64 ? 256 : LANES) void softmax_bwd_kernel(size_t rows, size_t cols,
                                                                                float* x_grad,
                                                                                const float* __restrict__ out,
                                                                                const float* out_grad, float beta, RG rg) {
  const float kk = rg.k();
  __shared__ float smem[16];
  constexpr int V = VEC ? 4 : 1;
  constexpr int RPB = LANES <= 64 ? 256 / LANES : 1;
  const size_t colsv = cols / V;
  const int lane = threadIdx.x % LANES;
  const size_t row = (size_t)blockIdx.x * RPB + threadIdx.x / LANES;
  const bool active = row < rows;

  float s[ITEMS][V], g[ITEMS][V];
  float dot = 0.0f;
  const bool full = active && (size_t)LANES * ITEMS <= colsv;
  if (VEC && full) {
    float4 a[ITEMS], b[ITEMS];
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      const size_t off = row * cols + 4 * ((size_t)lane + (size_t)j * LANES);
      a[j] = ld4s(out + off);
      b[j] = ld4s(out_grad + off);
    }
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      s[j][0] = a[j].x; s[j][V > 1 ? 1 : 0] = a[j].y; s[j][V > 1 ? 2 : 0] = a[j].z; s[j][V > 1 ? 3 : 0] = a[j].w;
      g[j][0] = b[j].x; g[j][V > 1 ? 1 : 0] = b[j].y; g[j][V > 1 ? 2 : 0] = b[j].z; g[j][V > 1 ? 3 : 0] = b[j].w;
    }
  } else {
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      const size_t c = (size_t)lane + (size_t)j * LANES;
      if (active && c < colsv) {
        if (VEC) {
          float4 a = ld4s(out + row * cols + 4 * c), b = ld4s(out_grad + row * cols + 4 * c);
          s[j][0] = a.x; s[j][V > 1 ? 1 : 0] = a.y; s[j][V > 1 ? 2 : 0] = a.z; s[j][V > 1 ? 3 : 0] = a.w;
          g[j][0] = b.x; g[j][V > 1 ? 1 : 0] = b.y; g[j][V > 1 ? 2 : 0] = b.z; g[j][V > 1 ? 3 : 0] = b.w;
        } else {
          s[j][0] = out[row * cols + c];
          g[j][0] = out_grad[row * cols + c];
        }
      } else {
#pragma unroll
        for (int q = 0; q < V; ++q) { s[j][q] = 0.0f; g[j][q] = 0.0f; }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < ITEMS; ++j)
#pragma unroll
    for (int q = 0; q < V; ++q) dot += rg.term(s[j][q], g[j][q]);
  // the up to 3 floats beyond the last whole vector of a row of odd length: lane q takes the q-th
  // (lane 0 all of them where a row has fewer than four lanes)
  const int rem = TAIL ? (int)(cols & 3) : 0;
  constexpr bool SPREAD = LANES >= 4;
  const bool tail = TAIL && active && (SPREAD ? lane < rem : (rem != 0 && lane == 0));
  const int tq0 = SPREAD ? lane : 0, tq1 = SPREAD ? lane + 1 : rem;
  float ts[3] = {0.f, 0.f, 0.f}, tg[3] = {0.f, 0.f, 0.f};
  if (tail)
    for (int q = tq0; q < tq1; ++q) {
      ts[q - tq0] = out[row * cols + 4 * colsv + q];
      tg[q - tq0] = out_grad[row * cols + 4 * colsv + q];
      dot += rg.term(ts[q - tq0], tg[q - tq0]);
    }
  dot = row_reduce<SumOp, LANES>(dot, smem);
  if (tail)
    for (int q = tq0; q < tq1; ++q) {
      float* p = x_grad + row * cols + 4 * colsv + q;
      const float r = rg.result(ts[q - tq0], tg[q - tq0], dot, kk);
      *p = beta != 0.0f ? beta * *p + r : r;
    }

#pragma unroll
  for (int j = 0; j < ITEMS; ++j) {
    const size_t c = (size_t)lane + (size_t)j * LANES;
    if (active && c < colsv) {
      float r[V];
#pragma unroll
      for (int q = 0; q < V; ++q) r[q] = rg.result(s[j][q], g[j][q], dot, kk);
      float* p = x_grad + row * cols + c * V;
      if (beta != 0.0f) {
        if (VEC) {
          float4 o = ld4s(p);
          r[0] = beta * o.x + r[0]; r[V > 1 ? 1 : 0] = beta * o.y + r[V > 1 ? 1 : 0];
          r[V > 1 ? 2 : 0] = beta * o.z + r[V > 1 ? 2 : 0]; r[V > 1 ? 3 : 0] = beta * o.w + r[V > 1 ? 3 : 0];
        } else {
          r[0] = beta * p[0] + r[0];
        }
      }
      if (VEC) st4s(p, make_float4(r[0], r[V > 1 ? 1 : 0], r[V > 1 ? 2 : 0], r[V > 1 ? 3 : 0]));
      else p[0] = r[0];
    }
  }
}

// Rows too long for registers: one block per row and two sweeps over global memory, float4 at
// a time with a scalar tail.  The first sweep keeps a running maximum and a sum of exponentials
// relative to it per thread (rescaled whenever the maximum moves); the block then combines the
// per-thread pairs, and the second sweep (which finds the row in L2 or the memory-side cache)
// writes exp(x - max) / sum.
__device__ __forceinline__ void online_add(float& m, float& s, float v) {
  if (v > m) {
    s = s * expf(m - v);  // m = -inf on the first element: s is 0 and stays 0
    m = v;
  }
  s += expf(v - m);
}
__global__ __launch_bounds__(1024) void softmax_fwd_stream_kernel(size_t cols, const float* __restrict__ x,
                                                                  float* __restrict__ out) {
  __shared__ float smem[16];
  const float* xr = x + (size_t)blockIdx.x * cols;
  float* o = out + (size_t)blockIdx.x * cols;
  const size_t nv = cols >> 2;
  float m = -__builtin_huge_valf(), s = 0.0f;
  // four vectors of a thread in flight per trip (one at a time left the sweep at 4.0-4.4 TB/s)
  for (size_t c0 = threadIdx.x; c0 < nv; c0 += 4096) {
    float4 t[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (c0 + 1024 * u < nv) t[u] = ld4g(xr + 4 * (c0 + 1024 * u));
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (c0 + 1024 * u >= nv) break;
      const float m4 = fmaxf(fmaxf(t[u].x, t[u].y), fmaxf(t[u].z, t[u].w));
      if (m4 > m) {
        s = s * expf(m - m4);
        m = m4;
      }
      s += (expf(t[u].x - m) + expf(t[u].y - m)) + (expf(t[u].z - m) + expf(t[u].w - m));
    }
  }
  for (size_t c = 4 * nv + threadIdx.x; c < cols; c += 1024) online_add(m, s, xr[c]);
  const float M = block_reduce<MaxOp>(m, smem);
  // threads that saw no element hold (m, s) = (-inf, 0): their term is 0, not exp(-inf + inf)
  const float S = block_reduce<SumOp>(s > 0.0f ? s * expf(m - M) : 0.0f, smem);
  for (size_t c0 = threadIdx.x; c0 < nv; c0 += 4096) {
    float4 t[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (c0 + 1024 * u < nv) t[u] = ld4g(xr + 4 * (c0 + 1024 * u));
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (c0 + 1024 * u < nv)
        st4s(o + 4 * (c0 + 1024 * u),
             make_float4(expf(t[u].x - M) / S, expf(t[u].y - M) / S, expf(t[u].z - M) / S, expf(t[u].w - M) / S));
  }
  for (size_t c = 4 * nv + threadIdx.x; c < cols; c += 1024) o[c] = expf(xr[c] - M) / S;
}

template <class RG>
__global__ __launch_bounds__(1024) void softmax_bwd_stream_kernel(size_t cols, float* x_grad,
                                                                  const float* __restrict__ out, const float* out_grad,
                                                                  float beta, RG rg) {
  __shared__ float smem[16];
  const float kk = rg.k();
  const size_t base = (size_t)blockIdx.x * cols;
  const float* sr = out + base;
  const float* gr = out_grad + base;
  float* xr = x_grad + base;
  const size_t nv = cols >> 2;
  float dot = 0.0f;
  for (size_t c0 = threadIdx.x; c0 < nv; c0 += 4096) {  // four vectors of each tensor in flight per trip
    float4 a[4], b[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (c0 + 1024 * u < nv) {
        a[u] = ld4g(sr + 4 * (c0 + 1024 * u));
        b[u] = ld4g(gr + 4 * (c0 + 1024 * u));
      }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (c0 + 1024 * u < nv)
        dot += (rg.term(a[u].x, b[u].x) + rg.term(a[u].y, b[u].y)) + (rg.term(a[u].z, b[u].z) + rg.term(a[u].w, b[u].w));
  }
  for (size_t c = 4 * nv + threadIdx.x; c < cols; c += 1024) dot += rg.term(sr[c], gr[c]);
  dot = block_reduce<SumOp>(dot, smem);
  for (size_t c0 = threadIdx.x; c0 < nv; c0 += 4096) {
    float4 a[4], b[4], p[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (c0 + 1024 * u < nv) {
        a[u] = ld4g(sr + 4 * (c0 + 1024 * u));
        b[u] = ld4g(gr + 4 * (c0 + 1024 * u));
        if (beta != 0.0f) p[u] = ld4g(xr + 4 * (c0 + 1024 * u));
      }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (c0 + 1024 * u < nv) {
        float4 r = make_float4(rg.result(a[u].x, b[u].x, dot, kk), rg.result(a[u].y, b[u].y, dot, kk),
                               rg.result(a[u].z, b[u].z, dot, kk), rg.result(a[u].w, b[u].w, dot, kk));
        if (beta != 0.0f) r = make_float4(beta * p[u].x + r.x, beta * p[u].y + r.y, beta * p[u].z + r.z, beta * p[u].w + r.w);
        st4s(xr + 4 * (c0 + 1024 * u), r);
      }
  }
  for (size_t c = 4 * nv + threadIdx.x; c < cols; c += 1024) {
    const float r = rg.result(sr[c], gr[c], dot, kk);
    xr[c] = beta != 0.0f ? beta * xr[c] + r : r;
  }
}

// Few rows, each far too long for a block (a softmax over one vector of 2^23 floats ran on one CU:
// 0.4 TB/s): the row is cut into segments of `seg` floats (a multiple of 4), one block each.  The
// first launch leaves every segment's running maximum and its sum of exponentials relative to it
// (backward: its share of <s, g>) in `stats`; the second combines the row's segments - every block
// for itself, all in the same order - and writes its own segment.
__global__ __launch_bounds__(1024) void softmax_fwd_seg_stats_kernel(size_t cols, size_t seg, const float* __restrict__ x,
                                                                     float* __restrict__ stats) {
  __shared__ float smem[16];
  const size_t beg = (size_t)blockIdx.x * seg, len = beg + seg <= cols ? seg : cols - beg;
  const float* xr = x + (size_t)blockIdx.y * cols + beg;
  const size_t nv = len >> 2;
  float m = -__builtin_huge_valf(), s = 0.0f;
  for (size_t c0 = threadIdx.x; c0 < nv; c0 += 4096) {
    float4 t[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (c0 + 1024 * u < nv) t[u] = ld4g(xr + 4 * (c0 + 1024 * u));
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (c0 + 1024 * u >= nv) break;
      const float m4 = fmaxf(fmaxf(t[u].x, t[u].y), fmaxf(t[u].z, t[u].w));
      if (m4 > m) {
        s = s * expf(m - m4);
        m = m4;
      }
      s += (expf(t[u].x - m) + expf(t[u].y - m)) + (expf(t[u].z - m) + expf(t[u].w - m));
    }
  }
  for (size_t c = 4 * nv + threadIdx.x; c < len; c += 1024) online_add(m, s, xr[c]);
  const float M = block_reduce<MaxOp>(m, smem);
  const float S = block_reduce<SumOp>(s > 0.0f ? s * expf(m - M) : 0.0f, smem);
  if (threadIdx.x == 0) {
    float* st = stats + 2 * ((size_t)blockIdx.y * gridDim.x + blockIdx.x);
    st[0] = M;
    st[1] = S;
  }
}

__global__ __launch_bounds__(1024) void softmax_fwd_seg_write_kernel(size_t cols, size_t seg, const float* __restrict__ x,
                                                                     float* __restrict__ out, const float* __restrict__ stats) {
  __shared__ float smem[16];
  const float* st = stats + 2 * (size_t)blockIdx.y * gridDim.x;
  float m = -__builtin_huge_valf();
  for (unsigned i = threadIdx.x; i < gridDim.x; i += 1024) m = fmaxf(m, st[2 * i]);
  const float M = block_reduce<MaxOp>(m, smem);
  float sum = 0.0f;
  for (unsigned i = threadIdx.x; i < gridDim.x; i += 1024) sum += st[2 * i + 1] > 0.0f ? st[2 * i + 1] * expf(st[2 * i] - M) : 0.0f;
  const float S = block_reduce<SumOp>(sum, smem);
  const size_t beg = (size_t)blockIdx.x * seg, len = beg + seg <= cols ? seg : cols - beg;
  const float* xr = x + (size_t)blockIdx.y * cols + beg;
  float* o = out + (size_t)blockIdx.y * cols + beg;
  const size_t nv = len >> 2;
  for (size_t c0 = threadIdx.x; c0 < nv; c0 += 4096) {
    float4 t[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (c0 + 1024 * u < nv) t[u] = ld4g(xr + 4 * (c0 + 1024 * u));
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (c0 + 1024 * u < nv)
        st4s(o + 4 * (c0 + 1024 * u),
             make_float4(expf(t[u].x - M) / S, expf(t[u].y - M) / S, expf(t[u].z - M) / S, expf(t[u].w - M) / S));
  }
  for (size_t c = 4 * nv + threadIdx.x; c < len; c += 1024) o[c] = expf(xr[c] - M) / S;
}

template <class RG>
__global__ __launch_bounds__(1024) void softmax_bwd_seg_stats_kernel(size_t cols, size_t seg, const float* __restrict__ out,
                                                                     const float* __restrict__ out_grad,
                                                                     float* __restrict__ stats, RG rg) {
  __shared__ float smem[16];
  const size_t beg = (size_t)blockIdx.x * seg, len = beg + seg <= cols ? seg : cols - beg;
  const size_t base = (size_t)blockIdx.y * cols + beg;
  const float* sr = out + base;
  const float* gr = out_grad + base;
  const size_t nv = len >> 2;
  float dot = 0.0f;
  for (size_t c0 = threadIdx.x; c0 < nv; c0 += 4096) {
    float4 a[4], b[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (c0 + 1024 * u < nv) {
        a[u] = ld4g(sr + 4 * (c0 + 1024 * u));
        b[u] = ld4g(gr + 4 * (c0 + 1024 * u));
      }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (c0 + 1024 * u < nv)
        dot += (rg.term(a[u].x, b[u].x) + rg.term(a[u].y, b[u].y)) + (rg.term(a[u].z, b[u].z) + rg.term(a[u].w, b[u].w));
  }
  for (size_t c = 4 * nv + threadIdx.x; c < len; c += 1024) dot += rg.term(sr[c], gr[c]);
  dot = block_reduce<SumOp>(dot, smem);
  if (threadIdx.x == 0) stats[(size_t)blockIdx.y * gridDim.x + blockIdx.x] = dot;
}

template <class RG>
__global__ __launch_bounds__(1024) void softmax_bwd_seg_write_kernel(size_t cols, size_t seg, float* x_grad,
                                                                     const float* __restrict__ out, const float* out_grad,
                                                                     float beta, const float* __restrict__ stats, RG rg) {
  __shared__ float smem[16];
  const float kk = rg.k();
  float part = 0.0f;
  for (unsigned i = threadIdx.x; i < gridDim.x; i += 1024) part += stats[(size_t)blockIdx.y * gridDim.x + i];
  const float dot = block_reduce<SumOp>(part, smem);
  const size_t beg = (size_t)blockIdx.x * seg, len = beg + seg <= cols ? seg : cols - beg;
  const size_t base = (size_t)blockIdx.y * cols + beg;
  const float* sr = out + base;
  const float* gr = out_grad + base;
  float* xr = x_grad + base;
  const size_t nv = len >> 2;
  for (size_t c0 = threadIdx.x; c0 < nv; c0 += 4096) {
    float4 a[4], b[4], p[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (c0 + 1024 * u < nv) {
        a[u] = ld4g(sr + 4 * (c0 + 1024 * u));
        b[u] = ld4g(gr + 4 * (c0 + 1024 * u));
        if (beta != 0.0f) p[u] = ld4g(xr + 4 * (c0 + 1024 * u));
      }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (c0 + 1024 * u < nv) {
        float4 r = make_float4(rg.result(a[u].x, b[u].x, dot, kk), rg.result(a[u].y, b[u].y, dot, kk),
                               rg.result(a[u].z, b[u].z, dot, kk), rg.result(a[u].w, b[u].w, dot, kk));
        if (beta != 0.0f) r = make_float4(beta * p[u].x + r.x, beta * p[u].y + r.y, beta * p[u].z + r.z, beta * p[u].w + r.w);
        st4s(xr + 4 * (c0 + 1024 * u), r);
      }
  }
  for (size_t c = 4 * nv + threadIdx.x; c < len; c += 1024) {
    const float r = rg.result(sr[c], gr[c], dot, kk);
    xr[c] = beta != 0.0f ? beta * xr[c] + r : r;
  }
}

// Short rows whose length is not a power of two (10, 100, 200 ... classes): with a few lanes per row
// every row starts at a different phase of the cache lines and the wave's loads scatter (2.2-4.7
// TB/s at 2^27 elements).  Here a workgroup streams a contiguous 16 KiB chunk of whole rows into LDS
// with full-width loads, L lanes per row (shuffles only) work on it in place, and the chunk is
// streamed out again.  The LDS index is skewed by one word per 32 (rows of even length would
// otherwise pile onto the same banks).
constexpr int SS_CHUNK = 4096;  // floats per workgroup and tensor
// sh = 5 for rows of even length, 31 (no skew) for odd ones, whose stride already visits every bank
__device__ __forceinline__ int ss_skew(int sh, int i) { return i + (i >> sh); }
__device__ __forceinline__ int ss_skew_shift(int cols) { return (cols & 1) ? 31 : 5; }

// Requests every vector of the chunk (of NB chunks at the same offsets) before the first one is
// used, then stores them into the skewed LDS buffers.
template <int NB>
__device__ __forceinline__ void ss_load(float* const (&buf)[NB], const float* const (&src)[NB], int len, int sh) {
  constexpr int NJ = SS_CHUNK / 1024;
  float4 v[NB][NJ];
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int i = 4 * threadIdx.x + 1024 * j;
      if (i + 3 < len) v[b][j] = ld4s(src[b] + i);
    }
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int i = 4 * threadIdx.x + 1024 * j;
      float* d = buf[b];
      if (i + 3 < len) {
        d[ss_skew(sh, i)] = v[b][j].x; d[ss_skew(sh, i + 1)] = v[b][j].y; d[ss_skew(sh, i + 2)] = v[b][j].z; d[ss_skew(sh, i + 3)] = v[b][j].w;
      } else {
        for (int e = i; e < len; ++e) d[ss_skew(sh, e)] = src[b][e];
      }
    }
}

template <int L, bool CCE>
__global__ __launch_bounds__(256) void softmax_fwd_short_kernel(size_t rows, int cols, int rpb, const float* __restrict__ x,
                                                                float* __restrict__ out, const float* __restrict__ tg,
                                                                float* __restrict__ loss_rows) {
  __shared__ float buf[SS_CHUNK + SS_CHUNK / 32 + 4];
  __shared__ float tbuf[CCE ? SS_CHUNK + SS_CHUNK / 32 + 4 : 1];  // the targets of the same rows
  const int sh = ss_skew_shift(cols);
  const size_t r0 = (size_t)blockIdx.x * rpb;
  const int nr = r0 + rpb <= rows ? rpb : (int)(rows - r0);
  const int len = nr * cols;
  if (CCE) {
    float* const bufs[2] = {buf, tbuf};
    const float* const srcs[2] = {x + r0 * cols, tg + r0 * cols};
    ss_load<2>(bufs, srcs, len, sh);
  } else {
    float* const bufs[1] = {buf};
    const float* const srcs[1] = {x + r0 * cols};
    ss_load<1>(bufs, srcs, len, sh);
  }
  __syncthreads();
  const int lane = threadIdx.x % L, group = threadIdx.x / L;
  for (int rb = 0; rb < nr; rb += 256 / L) {  // the same trip count for every thread: the shuffles need whole groups
    const int r = rb + group;
    const bool active = r < nr;
    const int base = r * cols;
    float m = -__builtin_huge_valf();
    if (active)
      for (int c = lane; c < cols; c += L) m = fmaxf(m, buf[ss_skew(sh, base + c)]);
    m = wave_reduce<MaxOp, L>(m);
    float sum = 0.0f;
    if (active)
      for (int c = lane; c < cols; c += L) {
        const float e = expf(buf[ss_skew(sh, base + c)] - m);
        buf[ss_skew(sh, base + c)] = e;
        sum += e;
      }
    sum = wave_reduce<SumOp, L>(sum);
    float acc = 0.0f;
    // e * (1 / sum), at most 1.5 ulp from the quotient e / sum: the kernel is bound by its arithmetic
    // (an exponential and a division per element, a lane or a few per row), and the division was a
    // quarter of it - rows of 100 floats 4.45 -> 5.4 TB/s, 33: 4.7 -> 5.4, 200: 4.4 -> 5.4, 255: 4.8 -> 5.7
    const float inv = 1.0f / sum;
    if (active)
      for (int c = lane; c < cols; c += L) {
        const float p = buf[ss_skew(sh, base + c)] * inv;
        buf[ss_skew(sh, base + c)] = p;
        if (CCE) acc += cce_term(p, tbuf[ss_skew(sh, base + c)]);
      }
    if (CCE) {
      acc = wave_reduce<SumOp, L>(acc);
      if (active && lane == 0) loss_rows[r0 + r] = -logf(acc);
    }
  }
  if (CCE && !out) return;
  __syncthreads();
  float* dst = out + r0 * cols;
  for (int i = 4 * threadIdx.x; i < len; i += 1024) {
    if (i + 3 < len) st4s(dst + i, make_float4(buf[ss_skew(sh, i)], buf[ss_skew(sh, i + 1)], buf[ss_skew(sh, i + 2)], buf[ss_skew(sh, i + 3)]));
    else
      for (int e = i; e < len; ++e) dst[e] = buf[ss_skew(sh, e)];
  }
}

template <int L, class RG>
__global__ __launch_bounds__(256) void softmax_bwd_short_kernel(size_t rows, int cols, int rpb, float* x_grad,
                                                                const float* __restrict__ out,
                                                                const float* __restrict__ out_grad, float beta, RG rg) {
  const float kk = rg.k();
  __shared__ float sb[SS_CHUNK + SS_CHUNK / 32 + 4];
  __shared__ float gb[SS_CHUNK + SS_CHUNK / 32 + 4];
  const int sh = ss_skew_shift(cols);
  const size_t r0 = (size_t)blockIdx.x * rpb;
  const int nr = r0 + rpb <= rows ? rpb : (int)(rows - r0);
  const int len = nr * cols;
  {
    float* const bufs[2] = {sb, gb};
    const float* const srcs[2] = {out + r0 * cols, out_grad + r0 * cols};
    ss_load<2>(bufs, srcs, len, sh);
  }
  __syncthreads();
  const int lane = threadIdx.x % L, group = threadIdx.x / L;
  for (int rb = 0; rb < nr; rb += 256 / L) {
    const int r = rb + group;
    const bool active = r < nr;
    const int base = r * cols;
    float dot = 0.0f;
    if (active)
      for (int c = lane; c < cols; c += L) dot += rg.term(sb[ss_skew(sh, base + c)], gb[ss_skew(sh, base + c)]);
    dot = wave_reduce<SumOp, L>(dot);
    if (active)
      for (int c = lane; c < cols; c += L)
        sb[ss_skew(sh, base + c)] = rg.result(sb[ss_skew(sh, base + c)], gb[ss_skew(sh, base + c)], dot, kk);
  }
  __syncthreads();
  float* dst = x_grad + r0 * cols;
  for (int i = 4 * threadIdx.x; i < len; i += 1024) {
    if (i + 3 < len) {
      float4 v = make_float4(sb[ss_skew(sh, i)], sb[ss_skew(sh, i + 1)], sb[ss_skew(sh, i + 2)], sb[ss_skew(sh, i + 3)]);
      if (beta != 0.0f) {
        const float4 o = ld4g(dst + i);
        v.x = beta * o.x + v.x; v.y = beta * o.y + v.y; v.z = beta * o.z + v.z; v.w = beta * o.w + v.w;
      }
      st4s(dst + i, v);  // (streaming, like every other softmax store: rows of 100 floats 5.6 -> 6.35 TB/s, 7: 5.7 -> 6.3, 10: 5.6 -> 5.8)
    } else {
      for (int e = i; e < len; ++e) dst[e] = beta != 0.0f ? beta * dst[e] + sb[ss_skew(sh, e)] : sb[ss_skew(sh, e)];
    }
  }
}

struct SoftmaxCfg {
  int lanes;  // 0 = streaming fallback
  int items;
};

static SoftmaxCfg pick_cfg(size_t colsv, bool fwd, bool long_rows) {
  if (colsv <= 256) {
    int lanes = 1;
    while ((size_t)lanes * 4 < colsv) lanes <<= 1;
    return {lanes, 4};
  }
  // forward rows of 257..448 vectors: one wave per row with eight vectors a lane (256 lanes a row
  // leave three quarters of them without a vector: rows of 1028 floats 3.9 -> 5.65 TB/s, 1280: 4.7 ->
  // 6.1, 1500: 5.3 -> 5.7; at 2000 floats the block per row is ahead again, and the backward pass
  // measured 3-7 % slower this way at every length)
  if (fwd && colsv <= 448) return {64, 8};
  if (colsv <= 1024) return {256, 4};
  // forward rows of 1025..2048 vectors: 512 lanes (with 1024 half the lanes idle through the two
  // reductions: 3.6-5.4 TB/s on rows of 4500-8192 floats against 5.6-5.9); the backward pass
  // measured the other way round (6.1-6.3 against 5.7-5.8)
  if (fwd && colsv <= 2048) return {512, 4};
  if (colsv <= 4096) return {1024, 4};
  // Rows of 16388..32768 floats still fit the registers of a block: 512 lanes with sixteen vectors each
  // forward (two rows a CU), 1024 lanes with eight vectors of each tensor backward.  Against the
  // two-sweep kernels below: rows of 20000 floats 4.5 -> 5.7 TB/s forward, 4.3 -> 6.0 backward; 32768:
  // 4.5 -> 5.8, 4.2 -> 6.0.  Forward rows of 40000..65536 floats take 1024 lanes with sixteen vectors,
  // one row a CU, which gains less (50257: 4.3 -> 4.55, 65536: 4.4 -> 4.8) and loses just above 32768,
  // where half the lanes idle (33333: 4.4 -> 4.1).
  if (long_rows) {
    if (fwd && colsv <= 8192) return {512, 16};
    if (fwd && colsv > 10000 && colsv <= 16384) return {1024, 16};
    if (!fwd && colsv <= 8192) return {1024, 8};
  }
  return {0, 0};
}

template <bool FWD, bool VEC, class RG = SoftmaxGradForm, bool CCE = false>
static int32_t softmax_dispatch(slhip_ctx* ctx, size_t rows, size_t cols, const float* x, float* out, float* x_grad,
                                const float* s, const float* g, float beta, RG rg = RG{}, const float* tg = nullptr,
                                float* loss_rows = nullptr) {
  // many short rows (measured at 2^27 elements, forward / backward TB/s, lanes-per-row kernel -> this
  // one: 10: 3.1 / 2.8 -> 5.8 / 6.1; 36: 2.2 / 2.9 -> 5.3 / 5.4; 100: 3.0 / 3.6 -> 4.8 / 5.2; 8: 3.3 / 4.0 ->
  // 5.9 / 6.1; 16: 1.4 / 1.8 -> 6.2 / 6.1; 32: 1.8 / 2.5 -> 5.6 / 6.2; 64: 4.9 / 5.2 -> 5.6 / 6.2; rows of 2 only
  // backward: 4.6 / 5.6 -> 4.0 / 6.1; 161: 4.5 / 4.35 -> 4.7 / 5.6; 200: 4.7 / 5.05 -> 4.8 / 5.8; 255: 4.1 / 4.2 -> 5.2 /
  // 5.0; at 128, 256 and from 257 on the lanes-per-row kernel is the faster one)
  if (cols >= (FWD ? 3 : 2) && cols <= 256 && (cols <= 64 || (cols & (cols - 1)) != 0) && rows >= 1024) {
    int rpb = SS_CHUNK / (int)cols;
    // chunks start on 128-byte boundaries of the tensors, or on 64-byte ones where a chunk holds too few
    // rows for that (rows of 129..255 floats of odd length: 16 of them); a 64-byte block that two
    // workgroups each write a part of costs the write side a sixth of its rate and more
    const int g32 = 32 / std::gcd((int)cols, 32), g16 = 16 / std::gcd((int)cols, 16);
    if (rpb >= 256) rpb -= rpb % 256;  // every thread of the row phase busy
    else if (rpb >= g32) rpb -= rpb % g32;
    else if (rpb >= g16) rpb -= rpb % g16;
    int lanes = 1;
    while (lanes < 64 && lanes * 2 * rpb <= 256) lanes <<= 1;  // groups of `lanes` lanes, at least one per row of the chunk
    const size_t blocks = (rows + rpb - 1) / rpb;
    SLHIP_REQUIRE(blocks <= 0x7fffffffu, "too many rows for one launch");
#define SL_SS(L)                                                                                                          \
  case L:                                                                                                                 \
    if (FWD)                                                                                                              \
      hipLaunchKernelGGL((softmax_fwd_short_kernel<L, CCE>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, rows,      \
                         (int)cols, rpb, x, out, tg, loss_rows);                                                          \
    else                                                                                                                  \
      hipLaunchKernelGGL((softmax_bwd_short_kernel<L, RG>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, rows,       \
                         (int)cols, rpb, x_grad, s, g, beta, rg);                                                         \
    break;
    switch (lanes) { SL_SS(1) SL_SS(2) SL_SS(4) SL_SS(8) SL_SS(16) SL_SS(32) SL_SS(64) }
#undef SL_SS
    return post_launch();
  }
  const size_t colsv = cols / (VEC ? 4 : 1);
  SoftmaxCfg cfg = pick_cfg(colsv, FWD, VEC && !CCE);
  SLHIP_REQUIRE(rows <= MAX_GRID, "too many rows for one launch");
  if (cfg.lanes == 0) {
    if (CCE) {  // rows too long for registers: the caller splits the work
      set_error("softmax with cross-entropy: rows of %zu floats do not fit the one-pass kernels", cols);
      return SLHIP_EINVAL;
    }
    // fewer rows than would fill the chip: segments of 64 Ki floats and more, four blocks per CU in all
    if (rows < (size_t)ctx->num_cu * 2 && cols >= (size_t(1) << 17)) {
      size_t nseg = ((size_t)ctx->num_cu * 4 + rows - 1) / rows;
      if (nseg > cols >> 16) nseg = cols >> 16;
      if (nseg > 65535) nseg = 65535;
      const size_t seg = ((cols + nseg - 1) / nseg + 3) & ~(size_t)3;
      nseg = (cols + seg - 1) / seg;
      if (nseg > 1 && rows * nseg * 2 * sizeof(float) <= ctx->workspace_bytes) {
        float* stats = (float*)ctx->workspace;
        const dim3 grid((unsigned)nseg, (unsigned)rows);
        if (FWD) {
          hipLaunchKernelGGL(softmax_fwd_seg_stats_kernel, grid, dim3(1024), 0, ctx->stream, cols, seg, x, stats);
          hipLaunchKernelGGL(softmax_fwd_seg_write_kernel, grid, dim3(1024), 0, ctx->stream, cols, seg, x, out, (const float*)stats);
        } else {
          hipLaunchKernelGGL((softmax_bwd_seg_stats_kernel<RG>), grid, dim3(1024), 0, ctx->stream, cols, seg, s, g, stats, rg);
          hipLaunchKernelGGL((softmax_bwd_seg_write_kernel<RG>), grid, dim3(1024), 0, ctx->stream, cols, seg, x_grad, s, g, beta,
                             (const float*)stats, rg);
        }
        return post_launch();
      }
    }
    if (FWD) hipLaunchKernelGGL(softmax_fwd_stream_kernel, dim3((unsigned)rows), dim3(1024), 0, ctx->stream, cols, x, out);
    else hipLaunchKernelGGL((softmax_bwd_stream_kernel<RG>), dim3((unsigned)rows), dim3(1024), 0, ctx->stream, cols, x_grad, s, g, beta, rg);
    return post_launch();
  }
#define SL_SM2(L, I, T)                                                                                              \
  do {                                                                                                               \
    constexpr int RPB = L <= 64 ? 256 / L : 1;                                                                       \
    constexpr int BLOCK = L <= 64 ? 256 : L;                                                                         \
    if (FWD)                                                                                                         \
      hipLaunchKernelGGL((softmax_fwd_kernel<VEC, L, I, T, CCE>), dim3(ceil_div(rows, RPB)), dim3(BLOCK), 0, ctx->stream, \
                         rows, cols, x, out, tg, loss_rows);                                                         \
    else                                                                                                             \
      hipLaunchKernelGGL((softmax_bwd_kernel<VEC, L, I, T, RG>), dim3(ceil_div(rows, RPB)), dim3(BLOCK), 0, ctx->stream, \
                         rows, cols, x_grad, s, g, beta, rg);                                                        \
  } while (0)
#define SL_SM(L, I)                                  \
  case (L) * 32 + (I):                               \
    if (VEC && (cols & 3)) SL_SM2(L, I, true);       \
    else SL_SM2(L, I, false);                        \
    break;
  // (the long-row forms hold 64 floats of the row per lane: not compiled for the scalar and the cross-entropy forms)
#define SL_SML(L, I)                                 \
  case (L) * 32 + (I):                               \
    if constexpr (VEC && !CCE) {                     \
      if (cols & 3) SL_SM2(L, I, true);              \
      else SL_SM2(L, I, false);                      \
    }                                                \
    break;
  switch (cfg.lanes * 32 + cfg.items) {
    SL_SM(1, 4) SL_SM(2, 4) SL_SM(4, 4) SL_SM(8, 4) SL_SM(16, 4) SL_SM(32, 4) SL_SM(64, 4) SL_SM(64, 8) SL_SM(256, 4) SL_SM(512, 4)
    SL_SM(1024, 4) SL_SML(512, 16) SL_SML(1024, 16) SL_SML(1024, 8)
  }
#undef SL_SML
#undef SL_SM
#undef SL_SM2
  return post_launch();
}

// The longest row the one-pass forward kernels hold in registers.
constexpr size_t SOFTMAX_ONE_PASS_COLS = 16384 + 3;

// probs = softmax(logits) (probs may be null) and loss_rows[r] = the cross-entropy of row r against
// targets, in one pass through the softmax forward kernels; rows beyond SOFTMAX_ONE_PASS_COLS are
// the caller's business.
int32_t softmax_cce_rows(slhip_ctx* ctx, size_t rows, size_t cols, const float* logits, const float* targets, float* probs,
                         float* loss_rows) {
  if (cols > SOFTMAX_ONE_PASS_COLS) {
    set_error("softmax with cross-entropy: rows of %zu floats do not fit the one-pass kernels", cols);
    return SLHIP_EINVAL;
  }
  return cols >= 4 ? softmax_dispatch<true, true, SoftmaxGradForm, true>(ctx, rows, cols, logits, probs, nullptr, nullptr,
                                                                        nullptr, 0.0f, SoftmaxGradForm{}, targets, loss_rows)
                   : softmax_dispatch<true, false, SoftmaxGradForm, true>(ctx, rows, cols, logits, probs, nullptr, nullptr,
                                                                         nullptr, 0.0f, SoftmaxGradForm{}, targets, loss_rows);
}

size_t softmax_one_pass_cols() { return SOFTMAX_ONE_PASS_COLS; }

// logits_grad = beta * logits_grad + (p * sum_c t - t) * (upstream / rows), row by row, through the
// softmax backward kernels.
int32_t softmax_cce_grad_rows(slhip_ctx* ctx, size_t rows, size_t cols, const float* probs, const float* targets,
                              float* logits_grad, float beta, const float* upstream_dev) {
  const CceGradForm rg{upstream_dev, (float)rows};
  return cols >= 4 ? softmax_dispatch<false, true, CceGradForm>(ctx, rows, cols, nullptr, nullptr, logits_grad, probs, targets,
                                                                beta, rg)
                   : softmax_dispatch<false, false, CceGradForm>(ctx, rows, cols, nullptr, nullptr, logits_grad, probs, targets,
                                                                 beta, rg);
}

}  // namespace slhip

using namespace slhip;

SLHIP_API int32_t slhip_softmax(slhip_ctx* ctx, size_t samples, size_t features, const float* x, float* out) {
  size_t len;
  SLHIP_REQUIRE(ctx && x && out, "null argument");
  SLHIP_REQUIRE(checked_len(samples, features, &len), "bad dims");
  SLHIP_REQUIRE(samples <= 0x7fffffffu, "too many rows for one launch");
  const bool vec = features >= 4;  // any row length: dword-aligned float4 accesses plus a scalar tail
  return vec ? softmax_dispatch<true, true>(ctx, samples, features, x, out, nullptr, nullptr, nullptr, 0.0f)
             : softmax_dispatch<true, false>(ctx, samples, features, x, out, nullptr, nullptr, nullptr, 0.0f);
}

SLHIP_API int32_t slhip_softmax_grad(slhip_ctx* ctx, size_t samples, size_t features, float* x_grad, const float* out,
                                     const float* out_grad, float beta) {
  size_t len;
  SLHIP_REQUIRE(ctx && x_grad && out && out_grad, "null argument");
  SLHIP_REQUIRE(checked_len(samples, features, &len), "bad dims");
  SLHIP_REQUIRE(samples <= 0x7fffffffu, "too many rows for one launch");
  const bool vec = features >= 4;  // any row length: dword-aligned float4 accesses plus a scalar tail
  return vec ? softmax_dispatch<false, true>(ctx, samples, features, nullptr, nullptr, x_grad, out, out_grad, beta)
             : softmax_dispatch<false, false>(ctx, samples, features, nullptr, nullptr, x_grad, out, out_grad, beta);
}
