// Row / column broadcast ops with an op code, diagflat and the onehot gradient: the part of the
// reference's op surface beside the training hot path (reference: src/ops2/row_op, src/ops2/col_op,
// src/ops2/diagflat, src/ops2/onehot).  Plain streaming kernels; the
// reductions of the broadcast-side gradients run through the row / column reduction kernels.
#include "common.hpp"

namespace slhip {

__device__ __forceinline__ float bc_apply(int op, float a, float b) {
  switch (op) {
    case SLHIP_ADD: return a + b;
    case SLHIP_SUB: return a - b;
    case SLHIP_MUL: return a * b;
    default: return a / b;
  }
}
// Forward and lhs gradient.  The matrix is walked as one flat run of float4 (dword-aligned, so any
// row length and base address): a thread finds the row and column of its first element with one
// division and steps from there.  BY_ROW_INDEX: the broadcast vector is indexed by the row
// (col_op), else by the column (row_op).  GRAD: lhs_grad += dL(lhs, v) * g instead of out = f(lhs, v).
// IDX: 32-bit index arithmetic whenever the matrix allows it.
template <bool BY_ROW_INDEX, bool GRAD, class IDX>
__global__ __launch_bounds__(256) void bc_flat_kernel(int op, size_t len, size_t cols, const float* __restrict__ lhs,
                                                      const float* __restrict__ v, float* out,
                                                      const float* __restrict__ g) {
  const size_t e0 = 4 * ((size_t)blockIdx.x * 256 + threadIdx.x);
  if (e0 >= len) return;
  IDX r = (IDX)e0 / (IDX)cols;
  IDX c = (IDX)e0 - r * (IDX)cols;
  const bool whole = e0 + 3 < len;
  float l[4] = {0.f, 0.f, 0.f, 0.f}, gv[4] = {0.f, 0.f, 0.f, 0.f}, o[4] = {0.f, 0.f, 0.f, 0.f};
  if (whole) {
    float4 t = ld4s(lhs + e0);
    l[0] = t.x; l[1] = t.y; l[2] = t.z; l[3] = t.w;
    if (GRAD) {
      t = ld4s(g + e0); gv[0] = t.x; gv[1] = t.y; gv[2] = t.z; gv[3] = t.w;
      t = ld4g(out + e0); o[0] = t.x; o[1] = t.y; o[2] = t.z; o[3] = t.w;
    }
  } else {
    for (size_t q = 0; e0 + q < len; ++q) {
      l[q] = lhs[e0 + q];
      if (GRAD) { gv[q] = g[e0 + q]; o[q] = out[e0 + q]; }
    }
  }
  // the broadcast entries of the four elements: one load where they lie in one row
  float vv[4] = {0.f, 0.f, 0.f, 0.f};
  if (whole && (size_t)c + 3 < cols) {
    if (BY_ROW_INDEX) {
      vv[0] = vv[1] = vv[2] = vv[3] = v[r];
    } else {
      const float4 t = ld4g(v + c);
      vv[0] = t.x; vv[1] = t.y; vv[2] = t.z; vv[3] = t.w;
    }
  } else {
    IDX rq = r, cq = c;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (e0 + q < len) vv[q] = v[BY_ROW_INDEX ? rq : cq];
      if (++cq == (IDX)cols) { cq = 0; ++rq; }
    }
  }
#pragma unroll
  for (int q = 0; q < 4; ++q)
    if (e0 + q < len) o[q] = GRAD ? o[q] + bc_dl(op, l[q], vv[q]) * gv[q] : bc_apply(op, l[q], vv[q]);
  if (whole) st4g(out + e0, make_float4(o[0], o[1], o[2], o[3]));
  else
    for (size_t q = 0; e0 + q < len; ++q) out[e0 + q] = o[q];
}

template <bool BY_ROW_INDEX, bool GRAD>
static void bc_flat_launch(slhip_ctx* ctx, int op, size_t len, size_t cols, const float* lhs, const float* v, float* out,
                           const float* g) {
  const unsigned blocks = (unsigned)(((len + 3) / 4 + 255) / 256);
  if (len <= 0xffffffffu)
    hipLaunchKernelGGL((bc_flat_kernel<BY_ROW_INDEX, GRAD, uint32_t>), dim3(blocks), dim3(256), 0, ctx->stream, op, len, cols, lhs, v, out, g);
  else
    hipLaunchKernelGGL((bc_flat_kernel<BY_ROW_INDEX, GRAD, size_t>), dim3(blocks), dim3(256), 0, ctx->stream, op, len, cols, lhs, v, out, g);
}

// One vector of four outputs per thread over the flat n x n matrix (one scalar store per thread
// wrote it at 3.9-4.2 TB/s).
template <class IDX>
__global__ __launch_bounds__(256) void diagflat_kernel(size_t n, const float* __restrict__ x, float* __restrict__ out) {
  const size_t len = n * n;
  const size_t e0 = 4 * ((size_t)blockIdx.x * 256 + threadIdx.x);
  if (e0 >= len) return;
  IDX r = (IDX)e0 / (IDX)n;
  IDX c = (IDX)e0 - r * (IDX)n;
  float o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    if (e0 + q < len && r == c) o[q] = x[r];
    if (++c == (IDX)n) { c = 0; ++r; }
  }
  if (e0 + 3 < len) st4s(out + e0, make_float4(o[0], o[1], o[2], o[3]));
  else
    for (size_t q = 0; e0 + q < len; ++q) out[e0 + q] = o[q];
}
__global__ __launch_bounds__(256) void diagflat_grad_kernel(size_t n, float* __restrict__ x_grad,
                                                            const float* __restrict__ out_grad) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) x_grad[i] += out_grad[i * n + i];
}
__global__ __launch_bounds__(256) void onehot_grad_kernel(size_t n, size_t classes, const float* __restrict__ cls,
                                                          float* __restrict__ cls_grad, const float* __restrict__ out_grad) {
  const size_t r = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (r >= n) return;
  const size_t c = (size_t)cls[r];
  if (c < classes) cls_grad[r] += out_grad[r * classes + c];
}

static bool grid_for(size_t threads, unsigned* blocks) {
  const size_t b = (threads + 255) / 256;
  if (b == 0 || b > 0x7fffffffu) return false;
  *blocks = (unsigned)b;
  return true;
}

template <bool BY_ROW_INDEX>
static int32_t bc_forward(slhip_ctx* ctx, int32_t op, size_t rows, size_t cols, const float* lhs, const float* v,
                          float* out) {
  size_t len;
  unsigned blocks;
  if (!checked_len(rows, cols, &len) || !grid_for(len, &blocks)) {
    set_error("broadcast op: bad dims %zu x %zu", rows, cols);
    return SLHIP_EINVAL;
  }
  if (op < SLHIP_ADD || op > SLHIP_DIV) {
    set_error("broadcast op: unknown op %d", op);
    return SLHIP_EINVAL;
  }
  bc_flat_launch<BY_ROW_INDEX, false>(ctx, op, len, cols, lhs, v, out, nullptr);
  return post_launch();
}

template <bool BY_ROW_INDEX>
static int32_t bc_backward(slhip_ctx* ctx, int32_t op, size_t rows, size_t cols, const float* lhs, const float* v,
                           float* lhs_grad, float* v_grad, const float* g) {
  size_t len;
  unsigned blocks;
  if (!checked_len(rows, cols, &len) || !grid_for(len, &blocks)) {
    set_error("broadcast op grad: bad dims %zu x %zu", rows, cols);
    return SLHIP_EINVAL;
  }
  if (op < SLHIP_ADD || op > SLHIP_DIV) {
    set_error("broadcast op grad: unknown op %d", op);
    return SLHIP_EINVAL;
  }
  if (lhs_grad) {
    bc_flat_launch<BY_ROW_INDEX, true>(ctx, op, len, cols, lhs, v, lhs_grad, g);
    int32_t rc = post_launch();
    if (rc) return rc;
  }
  if (!v_grad) return SLHIP_OK;
  // v_grad[i] += sum over row i (col_op) or column i (row_op) of dR(lhs, v[i]) * g: the reductions'
  // own kernels, reading the two matrices in place of one
  return bc_grad_rhs_reduce(ctx, BY_ROW_INDEX, op, rows, cols, lhs, v, g, v_grad);
}

}  // namespace slhip

using namespace slhip;

SLHIP_API int32_t slhip_row_op(slhip_ctx* ctx, int32_t op, size_t rows, size_t cols, const float* lhs, const float* rhs,
                               float* out) {
  SLHIP_REQUIRE(ctx && lhs && rhs && out, "null argument");
  return bc_forward<false>(ctx, op, rows, cols, lhs, rhs, out);
}

SLHIP_API int32_t slhip_row_op_grad(slhip_ctx* ctx, int32_t op, size_t rows, size_t cols, const float* lhs,
                                    const float* rhs, float* lhs_grad, float* rhs_grad, const float* out_grad) {
  SLHIP_REQUIRE(ctx && lhs && rhs && out_grad, "null argument");
  return bc_backward<false>(ctx, op, rows, cols, lhs, rhs, lhs_grad, rhs_grad, out_grad);
}

SLHIP_API int32_t slhip_col_op(slhip_ctx* ctx, int32_t op, size_t rows, size_t cols, const float* lhs, const float* rhs,
                               float* out) {
  SLHIP_REQUIRE(ctx && lhs && rhs && out, "null argument");
  return bc_forward<true>(ctx, op, rows, cols, lhs, rhs, out);
}

SLHIP_API int32_t slhip_col_op_grad(slhip_ctx* ctx, int32_t op, size_t rows, size_t cols, const float* lhs,
                                    const float* rhs, float* lhs_grad, float* rhs_grad, const float* out_grad) {
  SLHIP_REQUIRE(ctx && lhs && rhs && out_grad, "null argument");
  return bc_backward<true>(ctx, op, rows, cols, lhs, rhs, lhs_grad, rhs_grad, out_grad);
}

SLHIP_API int32_t slhip_diagflat(slhip_ctx* ctx, size_t n, const float* x, float* out) {
  SLHIP_REQUIRE(ctx && x && out, "null argument");
  size_t len;
  unsigned blocks;
  SLHIP_REQUIRE(checked_len(n, n, &len) && grid_for((len + 3) / 4, &blocks), "bad length");
  if (len <= 0xffffffffu) hipLaunchKernelGGL((diagflat_kernel<uint32_t>), dim3(blocks), dim3(256), 0, ctx->stream, n, x, out);
  else hipLaunchKernelGGL((diagflat_kernel<size_t>), dim3(blocks), dim3(256), 0, ctx->stream, n, x, out);
  return post_launch();
}

SLHIP_API int32_t slhip_diagflat_grad(slhip_ctx* ctx, size_t n, float* x_grad, const float* out_grad) {
  SLHIP_REQUIRE(ctx && x_grad && out_grad, "null argument");
  size_t len;
  unsigned blocks;
  SLHIP_REQUIRE(checked_len(n, n, &len) && grid_for(n, &blocks), "bad length");
  hipLaunchKernelGGL(diagflat_grad_kernel, dim3(blocks), dim3(256), 0, ctx->stream, n, x_grad, out_grad);
  return post_launch();
}

SLHIP_API int32_t slhip_onehot_grad(slhip_ctx* ctx, size_t n, size_t classes, const float* cls, float* cls_grad,
                                    const float* out_grad) {
  SLHIP_REQUIRE(ctx && cls && cls_grad && out_grad, "null argument");
  size_t len;
  unsigned blocks;
  SLHIP_REQUIRE(checked_len(n, classes, &len) && grid_for(n, &blocks), "bad dims");
  hipLaunchKernelGGL(onehot_grad_kernel, dim3(blocks), dim3(256), 0, ctx->stream, n, classes, cls, cls_grad, out_grad);
  return post_launch();
}
