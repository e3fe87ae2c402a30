// Row / column reductions (sum, max, mean), the scalar reductions, the bias gradient and the
// first-tie max gradient.  All HBM-bound: every input element is read exactly once with
// float4 loads; partial results of the two-stage forms live in the context workspace.
//
// Naming (kept from the reference): *_cols reduces along the contiguous axis (one value per
// row); *_rows reduces along the strided axis (one value per column).
#include <mutex>
#include <numeric>
#include <type_traits>

#include "common.hpp"

namespace slhip {

// How a finished value is written: out = v, or v / scale for the means (a true division, as the
// reference divides), optionally added to what out already holds.
struct Finalize {
  float scale;     // divisor of the means; unused otherwise
  int divide;      // 1: v = v / scale; 2: v = -ln v (the cross-entropy of a row)
  int accumulate;  // 1: out += v
};
__device__ __forceinline__ void finalize_store(float* p, float v, Finalize f) {
  if (f.divide == 2) v = -logf(v);
  else if (f.divide) v = v / f.scale;
  if (f.accumulate) v = *p + v;
  *p = v;
}

// What a reduction reads.  PlainSrc: the matrix itself.  BcGradSrc: the rhs-gradient terms of a
// broadcast op, dR(lhs[e], v) * g[e], v being the broadcast vector's entry for that element's row
// (reductions along the contiguous axis: col_op) or column (reductions along the strided axis:
// row_op); the kernels hand in v's entry, which they know from the row or column they work on.
struct PlainSrc {
  static constexpr bool HAS_V = false;
  static constexpr bool IS_PLAIN = true;
  const float* x;
  __device__ __forceinline__ float bvalue(size_t) const { return 0.0f; }
  __device__ __forceinline__ float4 vec(size_t e, float, float, float, float) const { return ld4s(x + e); }
  __device__ __forceinline__ float one(size_t e, float) const { return ld1s(x + e); }
};
template <int op>  // compile-time op code: the switch inside the load loops cost the two-matrix read a fifth of its rate
struct BcGradSrc {
  static constexpr bool HAS_V = true;
  static constexpr bool IS_PLAIN = false;
  const float* l;
  const float* g;
  const float* v;
  __device__ __forceinline__ float bvalue(size_t i) const { return v[i]; }
  __device__ __forceinline__ float4 vec(size_t e, float v0, float v1, float v2, float v3) const {
    const float4 a = ld4s(l + e), b = ld4s(g + e);
    return make_float4(bc_dr(op, a.x, v0) * b.x, bc_dr(op, a.y, v1) * b.y, bc_dr(op, a.z, v2) * b.z,
                       bc_dr(op, a.w, v3) * b.w);
  }
  __device__ __forceinline__ float one(size_t e, float vv) const { return bc_dr(op, ld1s(l + e), vv) * ld1s(g + e); }
};

// The terms of the categorical cross-entropy of a row: clip(p, 1e-7, 1 - 1e-7) * t
// (reference: examples/nn.rs:124-143).
struct CceSrc {
  static constexpr bool HAS_V = false;
  static constexpr bool IS_PLAIN = false;
  const float* p;
  const float* t;
  static __device__ __forceinline__ float term(float p, float t) {
    return fminf(fmaxf(p, (float)1e-7), (float)(1.0 - 1e-7)) * t;
  }
  __device__ __forceinline__ float bvalue(size_t) const { return 0.0f; }
  __device__ __forceinline__ float4 vec(size_t e, float, float, float, float) const {
    const float4 a = ld4s(p + e), b = ld4s(t + e);
    return make_float4(term(a.x, b.x), term(a.y, b.y), term(a.z, b.z), term(a.w, b.w));
  }
  __device__ __forceinline__ float one(size_t e, float) const { return term(ld1s(p + e), ld1s(t + e)); }
};

// ---------------------------------------------------------------------------------------
// Contiguous-axis reduction.  TPR lanes (power of two <= 64) or a whole block (TPR == 0) own one
// row segment; gridDim.y = number of segments a row is split into (partials when > 1).
// ---------------------------------------------------------------------------------------
template <class Op, bool VEC, int TPR, class Src>
__global__ __launch_bounds__(256) void rowreduce_kernel(size_t rows, size_t cols, Src src, float* __restrict__ out,
                                                        Finalize fin) {
  __shared__ float smem[8];
  constexpr int V = VEC ? 4 : 1;
  constexpr int LANES = TPR == 0 ? 256 : TPR;
  constexpr int ROWS_PER_BLOCK = TPR == 0 ? 1 : 256 / TPR;
  const size_t colsv = cols / V;
  const unsigned nseg = gridDim.y, seg = blockIdx.y;
  const size_t seg_len = (colsv + nseg - 1) / nseg;
  const size_t cbeg = (size_t)seg * seg_len;
  const size_t cend = cbeg + seg_len < colsv ? cbeg + seg_len : colsv;
  const int lane = TPR == 0 ? threadIdx.x : (threadIdx.x % LANES);
  const size_t row = (size_t)blockIdx.x * ROWS_PER_BLOCK + (TPR == 0 ? 0 : threadIdx.x / LANES);
  const bool active = row < rows;

  float a0 = Op::identity(), a1 = Op::identity(), a2 = Op::identity(), a3 = Op::identity();
  if (active) {
    const size_t xr = row * cols;
    const float vv = Src::HAS_V ? src.bvalue(row) : 0.0f;
    if (VEC) {
      // Four vectors a lane and trip, requested together, in one loop without a branch in it: a lane
      // whose trip holds fewer than four loads the row's last vector again instead and drops it.  (A
      // loop of whole trips with a tail that took the leftovers one by one waited for each of them,
      // and lanes of one wave that split between loop and tail ran both in turn: rows of 255 floats
      // 4.1 TB/s against 6.2 for rows of 257, whose 64 vectors are one whole trip for every lane;
      // tests around the loads instead of selects behind them cost max_cols 15-30 % on rows of 129,
      // 257, 513 and 1025.  Now 161: 4.2 -> 5.6, 200: 4.6 -> 6.7, 255: 5.2, 300: 5.2 -> 6.9, 500: 5.4 ->
      // 6.7, 1000: 5.5 -> 6.4, 16384: 6.8 -> 7.0.)
      const float id = Op::identity();
      const size_t last = cend - 1;
      for (size_t c = cbeg + lane; c < cend; c += 4 * LANES) {
        const size_t c1 = c + LANES, c2 = c + 2 * LANES, c3 = c + 3 * LANES;
        const bool h1 = c1 < cend, h2 = c2 < cend, h3 = c3 < cend;
        const float4 v0 = src.vec(xr + 4 * c, vv, vv, vv, vv), v1 = src.vec(xr + 4 * (h1 ? c1 : last), vv, vv, vv, vv),
                     v2 = src.vec(xr + 4 * (h2 ? c2 : last), vv, vv, vv, vv), v3 = src.vec(xr + 4 * (h3 ? c3 : last), vv, vv, vv, vv);
        a0 = Op::apply(a0, Op::apply(Op::apply(v0.x, v0.y), Op::apply(v0.z, v0.w)));
        a1 = Op::apply(a1, h1 ? Op::apply(Op::apply(v1.x, v1.y), Op::apply(v1.z, v1.w)) : id);
        a2 = Op::apply(a2, h2 ? Op::apply(Op::apply(v2.x, v2.y), Op::apply(v2.z, v2.w)) : id);
        a3 = Op::apply(a3, h3 ? Op::apply(Op::apply(v3.x, v3.y), Op::apply(v3.z, v3.w)) : id);
      }
      // a row of odd length ends in up to 3 floats beyond its last whole vector: lane q takes the q-th
      // (lane 0 all of them where a row has fewer than four lanes)
      if ((cols & 3) && seg == nseg - 1) {
        if (LANES >= 4) {
          if (lane < (int)(cols & 3)) a1 = Op::apply(a1, src.one(xr + 4 * colsv + lane, vv));
        } else if (lane == 0) {
          for (size_t e = 4 * colsv; e < cols; ++e) a1 = Op::apply(a1, src.one(xr + e, vv));
        }
      }
    } else {
      size_t c = cbeg + lane;
      for (; c + 3 * LANES < cend; c += 4 * LANES) {
        a0 = Op::apply(a0, src.one(xr + c, vv));
        a1 = Op::apply(a1, src.one(xr + c + LANES, vv));
        a2 = Op::apply(a2, src.one(xr + c + 2 * LANES, vv));
        a3 = Op::apply(a3, src.one(xr + c + 3 * LANES, vv));
      }
      for (; c < cend; c += LANES) a0 = Op::apply(a0, src.one(xr + c, vv));
    }
  }
  float v = Op::apply(Op::apply(a0, a1), Op::apply(a2, a3));
  if (TPR == 0) {
    v = block_reduce<Op>(v, smem);
    if (threadIdx.x == 0) {
      if (nseg > 1) out[row * nseg + seg] = v;
      else finalize_store(out + row, v, fin);
    }
  } else {
    v = wave_reduce<Op, (TPR > 0 ? TPR : 1)>(v);
    if (active && lane == 0) {
      if (nseg > 1) out[row * nseg + seg] = v;
      else finalize_store(out + row, v, fin);
    }
  }
}

// Contiguous-axis reduction of SHORT rows (up to 64 floats, or up to 128 when the length is not a
// power of two): with a few lanes per row every lane would start its loads at a different dword
// phase and the wave's loads would scatter (measured 2.1-3.2 TB/s for lengths 3, 10, 100; 3.3-4.0
// for 2, 16, 32 against 6.2-6.6 here).  Here a workgroup streams a contiguous
// chunk of whole rows into LDS with full-width vector loads, all of them requested before the
// first is used, then `tpr` lanes (a power of two) per row sum the row out of LDS.  The LDS index
// is skewed by one word per 32 so that threads striding by an even row length do not pile onto the
// same banks.  A chunk starts on a 128-byte boundary of the matrix.
constexpr int RS_CHUNK = 4096;  // floats per workgroup at most
// sh = 5 for rows of even length, 31 (no skew) for odd ones, whose stride already visits every bank
__device__ __forceinline__ int rs_skew(int sh, int i) { return i + (i >> sh); }
__device__ __forceinline__ int rs_skew_shift(int cols) { return (cols & 1) ? 31 : 5; }
template <class Op, class Src>
__global__ __launch_bounds__(256) void rowreduce_short_kernel(size_t rows, size_t cols, size_t rows_per_block, int tpr,
                                                              Src src, float* __restrict__ out, Finalize fin) {
  __shared__ float buf[RS_CHUNK + RS_CHUNK / 32 + 4];
  const int sh = rs_skew_shift((int)cols);
  const size_t r0 = (size_t)blockIdx.x * rows_per_block;
  const size_t nr = r0 + rows_per_block <= rows ? rows_per_block : rows - r0;
  const int len = (int)(nr * cols);  // <= RS_CHUNK
  const size_t e0 = r0 * cols;
  // the broadcast entry of local element i: the one of row r0 + i / cols
  auto bv = [&](int i) { return src.bvalue(r0 + (size_t)(i / (int)cols)); };
  float4 v[RS_CHUNK / 1024];
#pragma unroll
  for (int j = 0; j < RS_CHUNK / 1024; ++j) {
    const int i = 4 * threadIdx.x + 1024 * j;
    if (i + 3 < len) {
      float b[4] = {0.0f, 0.0f, 0.0f, 0.0f};
      if (Src::HAS_V) {
        int rl = i / (int)cols, c = i - rl * (int)cols;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          b[q] = src.bvalue(r0 + rl);
          if (++c == (int)cols) { c = 0; ++rl; }
        }
      }
      v[j] = src.vec(e0 + i, b[0], b[1], b[2], b[3]);
    }
  }
#pragma unroll
  for (int j = 0; j < RS_CHUNK / 1024; ++j) {
    const int i = 4 * threadIdx.x + 1024 * j;
    if (i + 3 < len) {
      buf[rs_skew(sh, i)] = v[j].x; buf[rs_skew(sh, i + 1)] = v[j].y; buf[rs_skew(sh, i + 2)] = v[j].z; buf[rs_skew(sh, i + 3)] = v[j].w;
    } else {
      for (int e = i; e < len; ++e) buf[rs_skew(sh, e)] = src.one(e0 + e, Src::HAS_V ? bv(e) : 0.0f);
    }
  }
  __syncthreads();
  const int lane = threadIdx.x & (tpr - 1), slot = threadIdx.x / tpr, slots = 256 / tpr;
  for (int rb = 0; rb < (int)nr; rb += slots) {  // the same trip count for every lane of the block
    const int r = rb + slot;
    float a0 = Op::identity(), a1 = a0;
    if (r < (int)nr) {
      const int base = r * (int)cols;
      int c = lane;
      for (; c + tpr < (int)cols; c += 2 * tpr) {
        a0 = Op::apply(a0, buf[rs_skew(sh, base + c)]);
        a1 = Op::apply(a1, buf[rs_skew(sh, base + c + tpr)]);
      }
      if (c < (int)cols) a0 = Op::apply(a0, buf[rs_skew(sh, base + c)]);
    }
    float s = Op::apply(a0, a1);
    for (int off = tpr >> 1; off > 0; off >>= 1) s = Op::apply(s, __shfl_xor(s, off, WAVE));
    if (r < (int)nr && lane == 0) finalize_store(out + r0 + r, s, fin);
  }
}

template <class Op, bool VEC, class Src>
static int32_t rowreduce_launch(slhip_ctx* ctx, size_t rows, size_t cols, Src x, float* out, unsigned nseg,
                                Finalize fin) {
  const size_t colsv = cols / (VEC ? 4 : 1);
  const size_t per_seg = (colsv + nseg - 1) / nseg;
  // lanes per row: about 4 vectors per lane, a whole block once a segment is long
  int tpr;
  if (per_seg >= 1024) tpr = 0;
  else {
    tpr = 1;
    while (tpr < 64 && (size_t)tpr * 4 < per_seg) tpr <<= 1;
  }
  SLHIP_REQUIRE(grid_fits(rows, tpr == 0 ? 1 : 256 / tpr), "too many rows for one launch");
#define SL_RR(T)                                                                                              \
  case T: {                                                                                                   \
    unsigned rpb = T == 0 ? 1 : 256 / (T == 0 ? 1 : T);                                                       \
    dim3 grid(ceil_div(rows, rpb), nseg);                                                                     \
    hipLaunchKernelGGL((rowreduce_kernel<Op, VEC, T, Src>), grid, dim3(256), 0, ctx->stream, rows, cols, x, out, fin); \
    break;                                                                                                    \
  }
  switch (tpr) {
    SL_RR(0) SL_RR(1) SL_RR(2) SL_RR(4) SL_RR(8) SL_RR(16) SL_RR(32) SL_RR(64)
  }
#undef SL_RR
  return post_launch();
}

// The sum (or mean) over an axis of length one: out[i] = 0 + x[i], the reference's fold from +0 -
// a copy but for -0, which it turns into +0.  One streaming vector per thread.
__global__ __launch_bounds__(64) void sum_of_one_kernel(size_t n, const float* __restrict__ x, float* __restrict__ out) {
  const size_t i = 4 * ((size_t)blockIdx.x * 64 + threadIdx.x);
  if (i + 3 < n) {
    float4 v = ld4s(x + i);
    v.x += 0.0f; v.y += 0.0f; v.z += 0.0f; v.w += 0.0f;
    st4s(out + i, v);
  } else {
    for (size_t e = i; e < n; ++e) out[e] = x[e] + 0.0f;
  }
}
static int32_t sum_of_one(slhip_ctx* ctx, size_t n, const float* x, float* out) {
  const size_t blocks = ((n + 3) / 4 + 63) / 64;
  SLHIP_REQUIRE(blocks <= 0x7fffffffu, "too many elements for one launch");
  hipLaunchKernelGGL(sum_of_one_kernel, dim3((unsigned)blocks), dim3(64), 0, ctx->stream, n, x, out);
  return post_launch();
}

// out[r] = reduce over the contiguous axis.
template <class Op, class Src>
static int32_t reduce_cols_src(slhip_ctx* ctx, size_t rows, size_t cols, Src x, float* out, Finalize fin) {
  // one column: every row is its own maximum, i.e. a plain copy (not so for a sum or a mean: the
  // reference's sum starts at +0, and 0 + -0 is +0 where a copy would leave -0)
  if constexpr (Src::IS_PLAIN && std::is_same<Op, MaxOp>::value)
    if (cols == 1 && !fin.accumulate) return slhip_memcpy_d2d(ctx, out, x.x, rows * sizeof(float));
  if constexpr (Src::IS_PLAIN && std::is_same<Op, SumOp>::value)
    if (cols == 1 && !fin.accumulate && fin.divide != 2 && x.x != out) return sum_of_one(ctx, rows, x.x, out);  // (a mean divides by 1)
  if (cols <= 128 && (cols <= 64 || (cols & (cols - 1)) != 0) && rows >= 1024) {  // many short rows
    // whole multiples of 256 rows while they fit (every lane of the second phase busy), else as many
    // rows as fit, rounded down so that every chunk starts on a 128-byte boundary
    size_t rpb = RS_CHUNK / cols;
    const size_t g32 = 32 / (size_t)std::gcd((unsigned long long)cols, 32ull);
    if (rpb >= 256) rpb -= rpb % 256;
    else if (rpb >= g32) rpb -= rpb % g32;
    int tpr = 1;  // lanes per row in the second phase
    while (tpr < 64 && rpb * (size_t)tpr * 2 <= 256 && (size_t)tpr * 2 <= cols) tpr <<= 1;
    const size_t blocks = (rows + rpb - 1) / rpb;
    SLHIP_REQUIRE(blocks <= 0x7fffffffu, "too many rows for one launch");
    hipLaunchKernelGGL((rowreduce_short_kernel<Op, Src>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, rows, cols, rpb, tpr, x, out, fin);
    return post_launch();
  }
  const bool vec = cols >= 4;  // any row length: dword-aligned float4 loads plus a scalar tail
  const size_t colsv = cols / (vec ? 4 : 1);
  // few long rows: split every row so the whole chip is busy
  unsigned nseg = 1;
  // (four workgroups per CU: 134 x 10^6 6.16 -> 6.28 TB/s, 16 x 2^23 6.30 -> 6.49, 300 x 400000 5.84 -> 6.51
  // against eight; with two the few-row shapes fall to 5.9)
  const size_t want_blocks = (size_t)ctx->num_cu * 4;
  if (rows < want_blocks && colsv >= 8192) {
    size_t s = (want_blocks + rows - 1) / rows;
    size_t max_s = colsv / 2048;  // each segment keeps >= 2048 vectors
    if (s > max_s) s = max_s;
    if (s > 1) nseg = (unsigned)s;
  }
  if (nseg == 1) return vec ? rowreduce_launch<Op, true, Src>(ctx, rows, cols, x, out, 1, fin)
                            : rowreduce_launch<Op, false, Src>(ctx, rows, cols, x, out, 1, fin);
  if (rows * nseg * sizeof(float) > ctx->workspace_bytes) {
    set_error("reduce over columns: %zu x %u partials exceed the workspace", rows, nseg);
    return SLHIP_EWORKSPACE;
  }
  float* part = (float*)ctx->workspace;
  Finalize none{1.0f, 0, 0};
  int32_t rc = vec ? rowreduce_launch<Op, true, Src>(ctx, rows, cols, x, part, nseg, none)
                   : rowreduce_launch<Op, false, Src>(ctx, rows, cols, x, part, nseg, none);
  if (rc) return rc;
  return rowreduce_launch<Op, false, PlainSrc>(ctx, rows, nseg, PlainSrc{part}, out, 1, fin);
}

// ---------------------------------------------------------------------------------------
// Strided-axis reduction, the streaming stages.  The matrix is read as ONE flat stream of float4,
// whatever the row length: T threads, 4T a multiple of cols; thread t reads the vectors t, t + T,
// t + 2T, ...  Component q of every vector it reads lies in the same column, (4t + q) mod cols, so
// the thread keeps four running values and writes them to partial[4t + q].  `partial` is then a
// (4T / cols) x cols matrix with the same column structure: the next stage reduces it the same
// way, until what is left is small enough for colreduce_final_kernel.  Rows of odd length, which a
// one-column-per-thread kernel with scalar loads reduced at 3.1-3.5 TB/s, stream at the same rate
// as rows that are a multiple of 4 long; one sweep of the grid reads one contiguous span of 16T bytes.
// ---------------------------------------------------------------------------------------
template <class Op, class Src>
__global__ __launch_bounds__(256) void colreduce_flat_kernel(size_t n, size_t T, size_t cols, Src src,
                                                             float* __restrict__ part) {
  const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= T) return;
  float b[4] = {0.0f, 0.0f, 0.0f, 0.0f};  // the broadcast entries of this thread's four columns
  if (Src::HAS_V) {
    size_t c = (4 * t) % cols;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      b[q] = src.bvalue(c);
      if (++c == cols) c = 0;
    }
  }
  const size_t nv = n >> 2;  // whole vectors of the stream
  const float id = Op::identity();
  float4 a0 = make_float4(id, id, id, id), a1 = a0, a2 = a0, a3 = a0;
#define SL_ACC(A, Q) A.x = Op::apply(A.x, Q.x); A.y = Op::apply(A.y, Q.y); A.z = Op::apply(A.z, Q.z); A.w = Op::apply(A.w, Q.w);
  size_t i = t;
  for (; i + 3 * T < nv; i += 4 * T) {
    float4 v0 = src.vec(4 * i, b[0], b[1], b[2], b[3]), v1 = src.vec(4 * (i + T), b[0], b[1], b[2], b[3]),
           v2 = src.vec(4 * (i + 2 * T), b[0], b[1], b[2], b[3]), v3 = src.vec(4 * (i + 3 * T), b[0], b[1], b[2], b[3]);
    SL_ACC(a0, v0) SL_ACC(a1, v1) SL_ACC(a2, v2) SL_ACC(a3, v3)
  }
  for (; i < nv; i += T) {
    float4 v0 = src.vec(4 * i, b[0], b[1], b[2], b[3]);
    SL_ACC(a0, v0)
  }
  SL_ACC(a0, a1) SL_ACC(a2, a3) SL_ACC(a0, a2)
#undef SL_ACC
  // the up to three floats behind the last whole vector belong to whoever owns their position
  for (size_t e = nv << 2; e < n; ++e) {
    const size_t pos = e % (4 * T);
    if (pos >> 2 == t) {
      const int q = (int)(pos & 3);
      const float v = src.one(e, b[q]);
      if (q == 0) a0.x = Op::apply(a0.x, v);
      else if (q == 1) a0.y = Op::apply(a0.y, v);
      else if (q == 2) a0.z = Op::apply(a0.z, v);
      else a0.w = Op::apply(a0.w, v);
    }
  }
  st4g(part + 4 * t, a0);
}

// Stage 2 (also the only stage for short matrices): a block owns CW adjacent columns, its
// 256/CW row-lanes stride over the rows and combine through LDS.
template <class Op, int CW, class Src>
__global__ __launch_bounds__(256) void colreduce_final_kernel(size_t rows, size_t cols, Src src, float* __restrict__ out,
                                                              Finalize fin) {
  constexpr int RL = 256 / CW;
  __shared__ float sm[256];
  const int cx = threadIdx.x % CW, ry = threadIdx.x / CW;
  const size_t c = (size_t)blockIdx.x * CW + cx;
  float a0 = Op::identity(), a1 = a0, a2 = a0, a3 = a0;
  if (c < cols) {
    const float vv = Src::HAS_V ? src.bvalue(c) : 0.0f;
    size_t r = ry;
    for (; r + 3 * RL < rows; r += 4 * RL) {  // four loads in flight per lane
      a0 = Op::apply(a0, src.one(r * cols + c, vv));
      a1 = Op::apply(a1, src.one((r + RL) * cols + c, vv));
      a2 = Op::apply(a2, src.one((r + 2 * RL) * cols + c, vv));
      a3 = Op::apply(a3, src.one((r + 3 * RL) * cols + c, vv));
    }
    for (; r < rows; r += RL) a0 = Op::apply(a0, src.one(r * cols + c, vv));
  }
  a0 = Op::apply(a0, a2);
  a1 = Op::apply(a1, a3);
  sm[threadIdx.x] = Op::apply(a0, a1);
  __syncthreads();
#pragma unroll
  for (int s = RL / 2; s > 0; s >>= 1) {
    if (ry < s) sm[threadIdx.x] = Op::apply(sm[threadIdx.x], sm[threadIdx.x + s * CW]);
    __syncthreads();
  }
  if (ry == 0 && c < cols) finalize_store(out + c, sm[cx], fin);
}

// Strided-axis reduction of a matrix of fewer than 8 rows (a single row that is added into `out`
// included): one thread per four adjacent columns, every row's vector requested before the first
// is used.  colreduce_final_kernel would leave three lanes in four idle on such a matrix and read
// it with scalar loads (measured 1.4 TB/s on [1 x 2^27] into an accumulating output).
constexpr int FEW_ROWS = 8;
template <class Op, class Src>
__global__ __launch_bounds__(256) void colreduce_fewrows_kernel(size_t rows, size_t cols, Src src, float* __restrict__ out,
                                                                Finalize fin) {
  const size_t c0 = 4 * ((size_t)blockIdx.x * 256 + threadIdx.x);
  if (c0 >= cols) return;
  float b[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  if (Src::HAS_V)
    for (int q = 0; q < 4 && c0 + q < cols; ++q) b[q] = src.bvalue(c0 + q);
  const float id = Op::identity();
  float a[4] = {id, id, id, id};
  if (c0 + 3 < cols) {
    float4 v[FEW_ROWS];
#pragma unroll
    for (int r = 0; r < FEW_ROWS; ++r)
      if ((size_t)r < rows) v[r] = src.vec((size_t)r * cols + c0, b[0], b[1], b[2], b[3]);
#pragma unroll
    for (int r = 0; r < FEW_ROWS; ++r)
      if ((size_t)r < rows) {
        a[0] = Op::apply(a[0], v[r].x); a[1] = Op::apply(a[1], v[r].y);
        a[2] = Op::apply(a[2], v[r].z); a[3] = Op::apply(a[3], v[r].w);
      }
    float4 o = make_float4(a[0], a[1], a[2], a[3]);
    if (fin.divide == 2) { o.x = -logf(o.x); o.y = -logf(o.y); o.z = -logf(o.z); o.w = -logf(o.w); }
    else if (fin.divide) { o.x = o.x / fin.scale; o.y = o.y / fin.scale; o.z = o.z / fin.scale; o.w = o.w / fin.scale; }
    if (fin.accumulate) {
      const float4 old = ld4g(out + c0);
      o.x = old.x + o.x; o.y = old.y + o.y; o.z = old.z + o.z; o.w = old.w + o.w;
    }
    st4g(out + c0, o);
  } else {
    for (int q = 0; c0 + q < cols; ++q) {
      for (size_t r = 0; r < rows; ++r) a[q] = Op::apply(a[q], src.one(r * cols + c0 + q, b[q]));
      finalize_store(out + c0 + q, a[q], fin);
    }
  }
}

template <class Op, class Src>
static int32_t colreduce_final_launch(slhip_ctx* ctx, size_t rows, size_t cols, Src x, float* out, Finalize fin) {
  // the widest column strip that still leaves every row-lane at most 16 rows
  int cw = 1;
  if (cols >= 64 && rows * 64 <= 4096) cw = 64;
  else if (cols >= 16 && rows * 16 <= 4096) cw = 16;
  else if (cols >= 4 && rows * 4 <= 4096) cw = 4;
  else if (rows > 4096) cw = cols >= 16 ? 16 : cols >= 4 ? 4 : 1;  // long inputs: coalescing matters more
  SLHIP_REQUIRE(grid_fits(cols, cw), "too many columns for one launch");
#define SL_CF(CW_)                                                                                                    \
  hipLaunchKernelGGL((colreduce_final_kernel<Op, CW_, Src>), dim3(ceil_div(cols, CW_)), dim3(256), 0, ctx->stream, rows, cols, \
                     x, out, fin)
  if (cw == 64) SL_CF(64);
  else if (cw == 16) SL_CF(16);
  else if (cw == 4) SL_CF(4);
  else SL_CF(1);
#undef SL_CF
  return post_launch();
}

// ---------------------------------------------------------------------------------------
// Whole-buffer reduction: per-block partials, then one block.
// ---------------------------------------------------------------------------------------
template <class Op, bool VEC, class Src>
__global__ __launch_bounds__(256) void fullreduce_kernel(size_t n, Src src, float* __restrict__ part) {
  __shared__ float smem[8];
  const float vv = Src::HAS_V ? src.bvalue(0) : 0.0f;  // a matrix of one column: one broadcast entry
  // every block streams ONE contiguous chunk (measured: 7.0-7.2 TB/s, against 5.7 TB/s when the
  // blocks interleave grid-stride fashion)
  float a0 = Op::identity(), a1 = a0, a2 = a0, a3 = a0;
  if (VEC) {
    const size_t n4 = n >> 2;
    const size_t chunk = (n4 + gridDim.x - 1) / gridDim.x;
    const size_t beg = (size_t)blockIdx.x * chunk;
    const size_t end = beg + chunk < n4 ? beg + chunk : n4;
    size_t i = beg + threadIdx.x;
    for (; i + 3 * 256 < end; i += 4 * 256) {
      float4 v0 = src.vec(4 * i, vv, vv, vv, vv), v1 = src.vec(4 * (i + 256), vv, vv, vv, vv),
             v2 = src.vec(4 * (i + 512), vv, vv, vv, vv), v3 = src.vec(4 * (i + 768), vv, vv, vv, vv);
      a0 = Op::apply(a0, Op::apply(Op::apply(v0.x, v0.y), Op::apply(v0.z, v0.w)));
      a1 = Op::apply(a1, Op::apply(Op::apply(v1.x, v1.y), Op::apply(v1.z, v1.w)));
      a2 = Op::apply(a2, Op::apply(Op::apply(v2.x, v2.y), Op::apply(v2.z, v2.w)));
      a3 = Op::apply(a3, Op::apply(Op::apply(v3.x, v3.y), Op::apply(v3.z, v3.w)));
    }
    for (; i < end; i += 256) {
      float4 v0 = src.vec(4 * i, vv, vv, vv, vv);
      a0 = Op::apply(a0, Op::apply(Op::apply(v0.x, v0.y), Op::apply(v0.z, v0.w)));
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) a1 = Op::apply(a1, src.one((n4 << 2) + threadIdx.x, vv));
  } else {
    const size_t chunk = (n + gridDim.x - 1) / gridDim.x;
    const size_t beg = (size_t)blockIdx.x * chunk;
    const size_t end = beg + chunk < n ? beg + chunk : n;
    for (size_t i = beg + threadIdx.x; i < end; i += 256) a0 = Op::apply(a0, src.one(i, vv));
  }
  float v = block_reduce<Op>(Op::apply(Op::apply(a0, a1), Op::apply(a2, a3)), smem);
  if (threadIdx.x == 0) part[blockIdx.x] = v;
}

template <class Op, class Src>
__global__ __launch_bounds__(1024) void fullreduce_final_kernel(size_t n, Src part, float* __restrict__ out,
                                                                Finalize fin) {
  __shared__ float smem[16];
  const float vv = Src::HAS_V ? part.bvalue(0) : 0.0f;
  float a = Op::identity();
  for (size_t i = threadIdx.x; i < n; i += 1024) a = Op::apply(a, part.one(i, vv));
  a = block_reduce<Op>(a, smem);
  if (threadIdx.x == 0) finalize_store(out, a, fin);
}

template <class Op, class Src>
static int32_t reduce_all_src(slhip_ctx* ctx, size_t n, Src x, float* out, Finalize fin, float* part) {
  const bool vec = true;
  size_t items = vec ? (n >> 2) + 1 : n;
  size_t blocks = (items + 256 * 16 - 1) / (256 * 16);
  // four workgroups per CU (measured on 2^28 / 2^26 / 2^24 floats: 6.93 / 6.21 / 4.89 TB/s; eight per
  // CU 6.50 / 5.92 / 4.63, two 6.26 / 6.05 / 4.35, one 3.86 / 3.66 / 3.05)
  size_t cap = (size_t)ctx->num_cu * 4;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  if (n <= 16384) {  // short buffers: the one-block kernel reads x itself
    hipLaunchKernelGGL((fullreduce_final_kernel<Op, Src>), dim3(1), dim3(1024), 0, ctx->stream, n, x, out, fin);
    return post_launch();
  }
  if (vec)
    hipLaunchKernelGGL((fullreduce_kernel<Op, true, Src>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, n, x, part);
  else
    hipLaunchKernelGGL((fullreduce_kernel<Op, false, Src>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, n, x, part);
  int32_t rc = post_launch();
  if (rc) return rc;
  hipLaunchKernelGGL((fullreduce_final_kernel<Op, PlainSrc>), dim3(1), dim3(1024), 0, ctx->stream, blocks, PlainSrc{part}, out,
                     fin);
  return post_launch();
}

// out[c] = reduce over the strided axis.  ws / ws_left: where the partial results of the streaming
// stages go (the context workspace, or the static scratch array), in floats.
template <class Op, class Src>
static int32_t reduce_rows_src(slhip_ctx* ctx, size_t rows, size_t cols, Src x, float* out, Finalize fin, float* ws,
                           size_t ws_left) {
  if (cols == 1) return reduce_all_src<Op, Src>(ctx, rows, x, out, fin, ws);  // at most 4 partials per CU
  // one row: the maximum over rows is that row itself (a sum starts at +0 and turns a -0 into +0)
  if constexpr (Src::IS_PLAIN && std::is_same<Op, MaxOp>::value)
    if (rows == 1 && !fin.accumulate) return slhip_memcpy_d2d(ctx, out, x.x, cols * sizeof(float));
  if constexpr (Src::IS_PLAIN && std::is_same<Op, SumOp>::value)
    if (rows == 1 && !fin.accumulate && fin.divide != 2 && x.x != out) return sum_of_one(ctx, cols, x.x, out);
  // Streaming stages until the matrix is short, then the one-kernel form.  Threads per stage:
  // about 512 per CU (measured optimum: 7.0 TB/s at 131072 threads on [16384 x 16384]; 5.4 TB/s at
  // four times as many), at least 16 vectors each, and a multiple of cols / gcd(cols, 4) so that
  // 4T is a multiple of cols.
  const size_t unit = cols / (cols % 4 == 0 ? 4 : cols % 2 == 0 ? 2 : 1);
  PlainSrc cur{nullptr};  // the partials of the stage before, once a stage has run
  bool first = true;
  size_t cur_rows = rows;
  // (the last stage is quick for up to 256 rows of any length - 16 rows per lane, 16 columns per
  // workgroup - and for small matrices of up to 4096 rows)
  while (cur_rows >= 8 && !((cur_rows <= 256 && cur_rows * cols <= (1u << 22)) || (cur_rows * cols <= (1u << 18) && cur_rows <= 4096))) {
    const size_t n = cur_rows * cols, nv = n >> 2;
    size_t T = (size_t)ctx->num_cu * 512;
    if (T > nv / 16) T = nv / 16;
    // A multiple of `unit`: the one below for a single stream (rows of 33333 floats: 3 x 33333 threads
    // 6.2 TB/s, 4 x 33333 - more than 512 per CU - 5.5), the nearest one for the two-matrix sources
    // of the first stage, which want more loads in flight (5.1 -> 6.1 TB/s on the same shape,
    // 3.8 -> 6.0 on rows of 66667)
    if (first && !Src::IS_PLAIN) {
      T = (T + unit / 2) / unit * unit;
      if (T > nv / 8 && T > unit) T -= unit;
    } else {
      T = T / unit * unit;
    }
    if (T < unit) T = unit;
    if (4 * T > ws_left || 8 * T > n) break;  // no room, or nothing gained: the last stage takes it as it is
    SLHIP_REQUIRE((T + 255) / 256 <= 0x7fffffffu, "matrix too wide for one launch");
    if (first)
      hipLaunchKernelGGL((colreduce_flat_kernel<Op, Src>), dim3((unsigned)((T + 255) / 256)), dim3(256), 0, ctx->stream, n, T, cols, x, ws);
    else
      hipLaunchKernelGGL((colreduce_flat_kernel<Op, PlainSrc>), dim3((unsigned)((T + 255) / 256)), dim3(256), 0, ctx->stream, n, T, cols, cur, ws);
    int32_t rc = post_launch();
    if (rc) return rc;
    first = false;
    cur.x = ws;
    cur_rows = 4 * T / cols;
    ws += 4 * T;
    ws_left -= 4 * T;
  }
  if (cur_rows < (size_t)FEW_ROWS && cols >= 4) {
    const size_t blocks = ((cols + 3) / 4 + 255) / 256;
    SLHIP_REQUIRE(blocks <= 0x7fffffffu, "matrix too wide for one launch");
    if (first)
      hipLaunchKernelGGL((colreduce_fewrows_kernel<Op, Src>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, cur_rows, cols, x,
                         out, fin);
    else
      hipLaunchKernelGGL((colreduce_fewrows_kernel<Op, PlainSrc>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, cur_rows,
                         cols, cur, out, fin);
    return post_launch();
  }
  if (first) return colreduce_final_launch<Op, Src>(ctx, cur_rows, cols, x, out, fin);
  return colreduce_final_launch<Op, PlainSrc>(ctx, cur_rows, cols, cur, out, fin);
}

template <class Op>
static int32_t reduce_rows(slhip_ctx* ctx, size_t rows, size_t cols, const float* x, float* out, Finalize fin) {
  return reduce_rows_src<Op, PlainSrc>(ctx, rows, cols, PlainSrc{x}, out, fin, (float*)ctx->workspace,
                                   ctx->workspace_bytes / sizeof(float));
}
template <class Op>
static int32_t reduce_cols(slhip_ctx* ctx, size_t rows, size_t cols, const float* x, float* out, Finalize fin) {
  return reduce_cols_src<Op, PlainSrc>(ctx, rows, cols, PlainSrc{x}, out, fin);
}
template <class Op>
static int32_t reduce_all(slhip_ctx* ctx, size_t n, const float* x, float* out, Finalize fin) {
  return reduce_all_src<Op, PlainSrc>(ctx, n, PlainSrc{x}, out, fin, (float*)ctx->workspace);
}

// ---------------------------------------------------------------------------------------
// Scratch memory for callers that cannot allocate (slhip_sum_rows_static): the partial results of
// the streaming stages in a file-scope device array instead of the context workspace.  Every GPU
// holds its own copy of the array at its own address; in host code the array's name is only a
// stand-in for the symbol, so the address is asked for once per device and everything below works
// with that pointer.  Nothing in it has to start at zero: each stage writes all the partials the
// next stage reads.
// ---------------------------------------------------------------------------------------
constexpr size_t STATIC_SCRATCH_FLOATS = size_t(1) << 20;  // 4 MiB per GPU, held until the process ends
static __device__ __align__(256) float static_scratch[STATIC_SCRATCH_FLOATS];
constexpr int STATIC_SCRATCH_MAX_DEVICES = 64;
static float* g_static_scratch[STATIC_SCRATCH_MAX_DEVICES];  // device address per ordinal, 0 = not asked yet
static std::mutex g_static_scratch_lock;                    // contexts may be created from several threads

int32_t static_scratch_resolve(int device, float** ptr) {
  if (device < 0 || device >= STATIC_SCRATCH_MAX_DEVICES) {
    set_error("device ordinal %d beyond the %d this library keeps scratch addresses for", device, STATIC_SCRATCH_MAX_DEVICES);
    return SLHIP_EINVAL;
  }
  std::lock_guard<std::mutex> hold(g_static_scratch_lock);
  if (!g_static_scratch[device]) {
    void* p = nullptr;
    SLHIP_CHECK_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(static_scratch)));
    if (!p) {
      set_error("hipGetSymbolAddress returned no address for the static scratch array");
      return SLHIP_EINVAL;
    }
    g_static_scratch[device] = (float*)p;
  }
  *ptr = g_static_scratch[device];
  return SLHIP_OK;
}

// ---------------------------------------------------------------------------------------
// max_cols_grad: the FIRST column equal to the row maximum receives out_grad[row].
// LANES lanes scan one row; the smallest matching index wins.
// ---------------------------------------------------------------------------------------
template <int TPR>
__global__ __launch_bounds__(256) void max_cols_grad_kernel(size_t rows, size_t cols, const float* __restrict__ out,
                                                            const float* __restrict__ x, float* __restrict__ x_grad,
                                                            const float* __restrict__ out_grad) {
  __shared__ unsigned long long smin;
  constexpr int LANES = TPR == 0 ? 256 : TPR;
  constexpr int RPB = TPR == 0 ? 1 : 256 / TPR;
  const int lane = TPR == 0 ? threadIdx.x : threadIdx.x % LANES;
  const size_t row = (size_t)blockIdx.x * RPB + (TPR == 0 ? 0 : threadIdx.x / LANES);
  const unsigned long long NONE = ~0ull;
  unsigned long long best = NONE;
  if (TPR == 0) {
    if (threadIdx.x == 0) smin = NONE;
    __syncthreads();
  }
  if (row < rows) {
    const float m = out[row];
    const float* xr = x + row * cols;
    // the whole row is streamed with float4 loads and no early exit (a loop that stops at the first
    // hit issues one dependent scalar load at a time: 1.4-3.3 TB/s); the smallest matching index wins
    const size_t colsv = cols >> 2;
    auto hit = [&](const float4& v, size_t c4) {
      unsigned long long h = NONE;
      if (v.w == m) h = 4 * c4 + 3;
      if (v.z == m) h = 4 * c4 + 2;
      if (v.y == m) h = 4 * c4 + 1;
      if (v.x == m) h = 4 * c4;
      return h;
    };
    size_t c = lane;
    for (; c + LANES < colsv; c += 2 * LANES) {
      const float4 v0 = ld4s(xr + 4 * c), v1 = ld4s(xr + 4 * (c + LANES));
      const unsigned long long h0 = hit(v0, c), h1 = hit(v1, c + LANES);
      best = h0 < best ? h0 : best;
      best = h1 < best ? h1 : best;
    }
    for (; c < colsv; c += LANES) {
      const unsigned long long h0 = hit(ld4s(xr + 4 * c), c);
      best = h0 < best ? h0 : best;
    }
    // the up to 3 floats behind the last whole vector: lane q takes the q-th (lane 0 all of them
    // where a row has fewer than four lanes)
    if (LANES >= 4) {
      const size_t e = (colsv << 2) + lane;
      if (e < cols && xr[e] == m && e < best) best = e;
    } else if (lane == 0) {
      for (size_t e = colsv << 2; e < cols; ++e)
        if (xr[e] == m && e < best) best = e;
    }
  }
  if (TPR == 0) {
    if (best != NONE) atomicMin(&smin, best);
    __syncthreads();
    if (threadIdx.x == 0 && row < rows && smin != NONE) x_grad[row * cols + smin] += out_grad[row];
  } else {
#pragma unroll
    for (int off = LANES / 2; off > 0; off >>= 1) {
      unsigned long long o = __shfl_xor(best, off, WAVE);
      best = o < best ? o : best;
    }
    if (row < rows && lane == 0 && best != NONE) x_grad[row * cols + best] += out_grad[row];
  }
}

// loss[r] = -ln sum_c clip(p[r, c]) * t[r, c]
int32_t cce_rows_reduce(slhip_ctx* ctx, size_t rows, size_t cols, const float* p, const float* t, float* loss) {
  return reduce_cols_src<SumOp, CceSrc>(ctx, rows, cols, CceSrc{p, t}, loss, Finalize{1.0f, 2, 0});
}

// rhs gradient of a broadcast op: v_grad[i] += sum of dR(lhs, v[i]) * g over row i (by_row: col_op)
// or over column i (row_op), through the same kernels as the plain sums.
int32_t bc_grad_rhs_reduce(slhip_ctx* ctx, bool by_row, int op, size_t rows, size_t cols, const float* lhs, const float* v,
                           const float* g, float* v_grad) {
  const Finalize add{1.0f, 0, 1};
#define SL_BG(OP)                                                                                                    \
  case OP: {                                                                                                         \
    const BcGradSrc<OP> src{lhs, g, v};                                                                              \
    if (by_row) return reduce_cols_src<SumOp, BcGradSrc<OP>>(ctx, rows, cols, src, v_grad, add);                     \
    return reduce_rows_src<SumOp, BcGradSrc<OP>>(ctx, rows, cols, src, v_grad, add, (float*)ctx->workspace,          \
                                                 ctx->workspace_bytes / sizeof(float));                              \
  }
  switch (op) {
    SL_BG(SLHIP_ADD) SL_BG(SLHIP_SUB) SL_BG(SLHIP_MUL) SL_BG(SLHIP_DIV)
  }
#undef SL_BG
  set_error("broadcast op grad: unknown op %d", op);
  return SLHIP_EINVAL;
}

// Few rows of great length: one workgroup per row would leave most of the chip idle (measured
// 1.9 TB/s on [134 x 10^6], 34 ms on [1 x 2^27]).  Every row is cut into segments, each workgroup
// scans one segment and lowers the row's slot to the smallest matching index it found, and a last
// kernel applies the slots.  The slots (one 64-bit word per row) live in the context workspace.
__global__ __launch_bounds__(256) void max_cols_grad_init_kernel(size_t rows, unsigned long long* __restrict__ slot) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < rows) slot[i] = ~0ull;
}
__global__ __launch_bounds__(256) void max_cols_grad_seg_kernel(size_t cols, size_t seg_vecs, const float* __restrict__ out,
                                                                const float* __restrict__ x, unsigned long long* slot) {
  __shared__ unsigned long long smin;
  const unsigned long long NONE = ~0ull;
  const size_t row = blockIdx.y;
  const float m = out[row];
  const float* xr = x + row * cols;
  const size_t colsv = cols >> 2;
  const size_t vbeg = (size_t)blockIdx.x * seg_vecs;
  const size_t vend = vbeg + seg_vecs < colsv ? vbeg + seg_vecs : colsv;
  if (threadIdx.x == 0) smin = NONE;
  __syncthreads();
  unsigned long long best = NONE;
  auto hit = [&](const float4& v, size_t c4) {
    unsigned long long h = NONE;
    if (v.w == m) h = 4 * c4 + 3;
    if (v.z == m) h = 4 * c4 + 2;
    if (v.y == m) h = 4 * c4 + 1;
    if (v.x == m) h = 4 * c4;
    return h;
  };
  size_t c = vbeg + threadIdx.x;
  for (; c + 3 * 256 < vend; c += 4 * 256) {
    const float4 v0 = ld4s(xr + 4 * c), v1 = ld4s(xr + 4 * (c + 256)), v2 = ld4s(xr + 4 * (c + 512)),
                 v3 = ld4s(xr + 4 * (c + 768));
    const unsigned long long h0 = hit(v0, c), h1 = hit(v1, c + 256), h2 = hit(v2, c + 512), h3 = hit(v3, c + 768);
    best = h0 < best ? h0 : best;
    best = h1 < best ? h1 : best;
    best = h2 < best ? h2 : best;
    best = h3 < best ? h3 : best;
  }
  for (; c < vend; c += 256) {
    const unsigned long long h0 = hit(ld4s(xr + 4 * c), c);
    best = h0 < best ? h0 : best;
  }
  // the up to three floats behind the row's last whole vector go with the last segment
  if (blockIdx.x == gridDim.x - 1 && threadIdx.x == 0)
    for (size_t e = colsv << 2; e < cols; ++e)
      if (xr[e] == m && e < best) best = e;
  if (best != NONE) atomicMin(&smin, best);
  __syncthreads();
  if (threadIdx.x == 0 && smin != NONE) atomicMin(slot + row, smin);
}
__global__ __launch_bounds__(256) void max_cols_grad_apply_kernel(size_t rows, size_t cols,
                                                                  const unsigned long long* __restrict__ slot,
                                                                  float* __restrict__ x_grad,
                                                                  const float* __restrict__ out_grad) {
  const size_t row = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (row < rows && slot[row] != ~0ull) x_grad[row * cols + slot[row]] += out_grad[row];
}

}  // namespace slhip

using namespace slhip;

#define SL_DIMS_OK()                                           \
  size_t len;                                                  \
  SLHIP_REQUIRE(ctx && x && out, "null argument");             \
  SLHIP_REQUIRE(checked_len(rows, cols, &len), "bad dims");    \
  (void)len;

SLHIP_API int32_t slhip_sum_cols(slhip_ctx* ctx, size_t rows, size_t cols, const float* x, float* out) {
  SL_DIMS_OK();
  return reduce_cols<SumOp>(ctx, rows, cols, x, out, Finalize{1.0f, 0, 0});
}
SLHIP_API int32_t slhip_max_cols(slhip_ctx* ctx, size_t rows, size_t cols, const float* x, float* out) {
  SL_DIMS_OK();
  return reduce_cols<MaxOp>(ctx, rows, cols, x, out, Finalize{1.0f, 0, 0});
}
SLHIP_API int32_t slhip_mean_cols(slhip_ctx* ctx, size_t rows, size_t cols, const float* x, float* out) {
  SL_DIMS_OK();
  return reduce_cols<SumOp>(ctx, rows, cols, x, out, Finalize{(float)cols, 1, 0});
}
SLHIP_API int32_t slhip_sum_rows(slhip_ctx* ctx, size_t rows, size_t cols, const float* x, float* out) {
  SL_DIMS_OK();
  return reduce_rows<SumOp>(ctx, rows, cols, x, out, Finalize{1.0f, 0, 0});
}
// The widest matrix whose streaming stages fit the static scratch array whatever its height: a stage
// keeps 4 partials for each of its T <= 512 * (number of CUs) threads, T a multiple of
// cols / gcd(cols, 4), and a stage runs only if it at least halves its input; with cols <= 131072 and
// 256 CUs the first stage needs at most 2^19 floats and every later one at most half of the one
// before, so all of them fit the 2^20 floats.
constexpr size_t STATIC_MAX_COLS = 131072;
SLHIP_API int32_t slhip_sum_rows_static(slhip_ctx* ctx, size_t rows, size_t cols, const float* x, float* out) {
  SL_DIMS_OK();
  if (cols > STATIC_MAX_COLS) {
    set_error("slhip_sum_rows_static: %zu columns; the static scratch serves at most %zu (use slhip_sum_rows)", cols,
              STATIC_MAX_COLS);
    return SLHIP_EWORKSPACE;
  }
  SLHIP_REQUIRE(ctx->static_scratch, "the context has no static scratch address");
  return reduce_rows_src<SumOp, PlainSrc>(ctx, rows, cols, PlainSrc{x}, out, Finalize{1.0f, 0, 0}, ctx->static_scratch,
                                          STATIC_SCRATCH_FLOATS);
}
SLHIP_API int32_t slhip_max_rows(slhip_ctx* ctx, size_t rows, size_t cols, const float* x, float* out) {
  SL_DIMS_OK();
  return reduce_rows<MaxOp>(ctx, rows, cols, x, out, Finalize{1.0f, 0, 0});
}
SLHIP_API int32_t slhip_mean_rows(slhip_ctx* ctx, size_t rows, size_t cols, const float* x, float* out) {
  SL_DIMS_OK();
  return reduce_rows<SumOp>(ctx, rows, cols, x, out, Finalize{(float)rows, 1, 0});
}

SLHIP_API int32_t slhip_sum(slhip_ctx* ctx, size_t n, const float* x, float* out) {
  SLHIP_REQUIRE(ctx && x && out, "null argument");
  SLHIP_REQUIRE(n > 0, "empty buffer");
  return reduce_all<SumOp>(ctx, n, x, out, Finalize{1.0f, 0, 0});
}
SLHIP_API int32_t slhip_max(slhip_ctx* ctx, size_t n, const float* x, float* out) {
  SLHIP_REQUIRE(ctx && x && out, "null argument");
  SLHIP_REQUIRE(n > 0, "empty buffer");
  return reduce_all<MaxOp>(ctx, n, x, out, Finalize{1.0f, 0, 0});
}
SLHIP_API int32_t slhip_mean(slhip_ctx* ctx, size_t n, const float* x, float* out) {
  SLHIP_REQUIRE(ctx && x && out, "null argument");
  SLHIP_REQUIRE(n > 0, "empty buffer");
  return reduce_all<SumOp>(ctx, n, x, out, Finalize{(float)n, 1, 0});
}

// rhs_grad[c] += sum over rows of out_grad[r, c]
SLHIP_API int32_t slhip_add_row_mut_grad(slhip_ctx* ctx, size_t rows, size_t cols, float* rhs_grad,
                                         const float* out_grad) {
  size_t len;
  SLHIP_REQUIRE(ctx && rhs_grad && out_grad, "null argument");
  SLHIP_REQUIRE(checked_len(rows, cols, &len), "bad dims");
  return reduce_rows<SumOp>(ctx, rows, cols, out_grad, rhs_grad, Finalize{1.0f, 0, 1});
}

SLHIP_API int32_t slhip_add_row_grad(slhip_ctx* ctx, size_t rows, size_t cols, float* lhs_grad, float* rhs_grad,
                                     const float* out_grad) {
  size_t len;
  SLHIP_REQUIRE(ctx && rhs_grad && out_grad, "null argument");
  SLHIP_REQUIRE(checked_len(rows, cols, &len), "bad dims");
  if (lhs_grad && lhs_grad != out_grad) {
    int32_t rc = slhip_memcpy_d2d(ctx, lhs_grad, out_grad, len * sizeof(float));
    if (rc) return rc;
  }
  return reduce_rows<SumOp>(ctx, rows, cols, out_grad, rhs_grad, Finalize{1.0f, 0, 1});
}

SLHIP_API int32_t slhip_max_cols_grad(slhip_ctx* ctx, size_t rows, size_t cols, const float* out, const float* x,
                                      float* x_grad, const float* out_grad) {
  size_t len;
  SLHIP_REQUIRE(ctx && out && x && x_grad && out_grad, "null argument");
  SLHIP_REQUIRE(checked_len(rows, cols, &len), "bad dims");
  // few long rows: several workgroups per row
  if (rows < (size_t)ctx->num_cu * 2 && cols >= 65536 && rows <= 65535 && rows * sizeof(unsigned long long) <= ctx->workspace_bytes) {
    const size_t colsv = cols >> 2;
    size_t nseg = ((size_t)ctx->num_cu * 8 + rows - 1) / rows;
    if (nseg > colsv / 4096) nseg = colsv / 4096;  // at least 4096 vectors per segment
    if (nseg < 1) nseg = 1;
    const size_t seg_vecs = (colsv + nseg - 1) / nseg;
    nseg = (colsv + seg_vecs - 1) / seg_vecs;
    unsigned long long* slot = (unsigned long long*)ctx->workspace;
    hipLaunchKernelGGL(max_cols_grad_init_kernel, dim3(ceil_div(rows, 256)), dim3(256), 0, ctx->stream, rows, slot);
    hipLaunchKernelGGL(max_cols_grad_seg_kernel, dim3((unsigned)nseg, (unsigned)rows), dim3(256), 0, ctx->stream, cols, seg_vecs,
                       out, x, slot);
    hipLaunchKernelGGL(max_cols_grad_apply_kernel, dim3(ceil_div(rows, 256)), dim3(256), 0, ctx->stream, rows, cols,
                       (const unsigned long long*)slot, x_grad, out_grad);
    return post_launch();
  }
  int tpr;
  if (cols >= 4096) tpr = 0;
  else {
    tpr = 1;
    while (tpr < 64 && (size_t)tpr * 8 < cols) tpr <<= 1;
  }
  SLHIP_REQUIRE(grid_fits(rows, tpr == 0 ? 1 : 256 / tpr), "too many rows for one launch");
#define SL_MCG(T)                                                                                          \
  case T: {                                                                                                \
    unsigned rpb = T == 0 ? 1 : 256 / (T == 0 ? 1 : T);                                                    \
    hipLaunchKernelGGL((max_cols_grad_kernel<T>), dim3(ceil_div(rows, rpb)), dim3(256), 0, ctx->stream,    \
                       rows, cols, out, x, x_grad, out_grad);                                              \
    break;                                                                                                 \
  }
  switch (tpr) {
    SL_MCG(0) SL_MCG(1) SL_MCG(2) SL_MCG(4) SL_MCG(8) SL_MCG(16) SL_MCG(32) SL_MCG(64)
  }
#undef SL_MCG
  return post_launch();
}
