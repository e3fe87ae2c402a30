// Matrix transpose through a padded LDS tile: out[c*rows + r] = x[r*cols + c].
//
// A 64x64 tile is read with float4 loads along the input rows, staged in LDS with a row pitch
// of 65 words (so that the column-wise read-back hits 64 different banks pairs instead of one),
// and written with float4 stores along the output rows.  8 B/element of HBM traffic, the
// algorithmic minimum.  beta selects `=` (0) or `+=` (1).
#include "common.hpp"

namespace slhip {

constexpr int TT = 64;  // tile edge

template <bool VEC, bool ACC>
__global__ __launch_bounds__(256) void transpose_kernel(size_t rows, size_t cols, const float* __restrict__ x,
                                                        float* out, unsigned tiles_c) {
  __shared__ float tile[TT][TT + 1];
  // tiles are numbered along the input columns first; consecutive blocks therefore write to
  // consecutive output rows
  const size_t tr = blockIdx.x / tiles_c, tc = blockIdx.x % tiles_c;
  const size_t r0 = tr * TT, c0 = tc * TT;
  const int t = threadIdx.x;

  if (VEC) {
    const int lx = t & 15, ly = t >> 4;  // 16 float4 per tile row, 16 rows per pass
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int rr = ly + 16 * p;
      const size_t r = r0 + rr, c = c0 + 4 * lx;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (r < rows && c < cols) v = ld4(x + r * cols + c);  // cols % 4 == 0: a vector is all in or all out
      tile[rr][4 * lx + 0] = v.x;
      tile[rr][4 * lx + 1] = v.y;
      tile[rr][4 * lx + 2] = v.z;
      tile[rr][4 * lx + 3] = v.w;
    }
    __syncthreads();
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int cc = ly + 16 * p;  // input column = output row
      const size_t oc = c0 + cc, orow0 = r0 + 4 * lx;
      if (oc < cols && orow0 < rows) {  // rows % 4 == 0 as well
        float4 v = make_float4(tile[4 * lx + 0][cc], tile[4 * lx + 1][cc], tile[4 * lx + 2][cc], tile[4 * lx + 3][cc]);
        float* p_out = out + oc * rows + orow0;
        if (ACC) {
          float4 o = ld4(p_out);
          v.x += o.x; v.y += o.y; v.z += o.z; v.w += o.w;
        }
        st4(p_out, v);
      }
    }
  } else {
    const int lx = t & 63, ly = t >> 6;  // 64 columns, 4 rows per pass
#pragma unroll 4
    for (int p = 0; p < 16; ++p) {
      const int rr = ly + 4 * p;
      const size_t r = r0 + rr, c = c0 + lx;
      tile[rr][lx] = (r < rows && c < cols) ? x[r * cols + c] : 0.0f;
    }
    __syncthreads();
#pragma unroll 4
    for (int p = 0; p < 16; ++p) {
      const int cc = ly + 4 * p;
      const size_t oc = c0 + cc, orow = r0 + lx;
      if (oc < cols && orow < rows) {
        float v = tile[lx][cc];
        float* p_out = out + oc * rows + orow;
        if (ACC) v += *p_out;
        *p_out = v;
      }
    }
  }
}

__global__ __launch_bounds__(256) void axpy_copy_kernel(size_t n, const float* __restrict__ x, float* out) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * 256;
  for (; i < n; i += stride) out[i] += x[i];
}

}  // namespace slhip

using namespace slhip;

SLHIP_API int32_t slhip_transpose(slhip_ctx* ctx, size_t rows, size_t cols, const float* x, float* out, float beta) {
  size_t len;
  SLHIP_REQUIRE(ctx && x && out, "null argument");
  SLHIP_REQUIRE(checked_len(rows, cols, &len), "bad dims");
  SLHIP_REQUIRE(beta == 0.0f || beta == 1.0f, "beta must be 0 (set) or 1 (accumulate)");
  if (x == out) {
    set_error("slhip_transpose: in-place transpose is not supported");
    return SLHIP_EALIAS;
  }
  const bool acc = beta != 0.0f;
  if (rows == 1 || cols == 1) {  // a vector: the transpose is the same sequence of values
    if (!acc) return slhip_memcpy_d2d(ctx, out, x, len * sizeof(float));
    unsigned grid = (unsigned)(len / 256 + 1 < (size_t)ctx->num_cu * 16 ? len / 256 + 1 : (size_t)ctx->num_cu * 16);
    hipLaunchKernelGGL(axpy_copy_kernel, dim3(grid), dim3(256), 0, ctx->stream, len, x, out);
    return post_launch();
  }
  const size_t tiles_r = (rows + TT - 1) / TT, tiles_c = (cols + TT - 1) / TT;
  SLHIP_REQUIRE(tiles_r * tiles_c <= 0x7fffffffu, "matrix too large for one launch");
  const unsigned grid = (unsigned)(tiles_r * tiles_c);
  const bool vec = (rows % 4 == 0) && (cols % 4 == 0) && aligned16(x) && aligned16(out);
#define SL_TR(V, A) \
  hipLaunchKernelGGL((transpose_kernel<V, A>), dim3(grid), dim3(256), 0, ctx->stream, rows, cols, x, out, (unsigned)tiles_c)
  if (vec) { if (acc) SL_TR(true, true); else SL_TR(true, false); }
  else { if (acc) SL_TR(false, true); else SL_TR(false, false); }
#undef SL_TR
  return post_launch();
}
