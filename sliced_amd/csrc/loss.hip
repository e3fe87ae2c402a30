// Fused losses of the two example training loops: each replaces a chain of reference ops by one
// forward and one backward kernel (the chains stay available op by op).
//
//   mean squared error      L = (sum_i (x_i - y_i)^2) * (1/n)
//       reference chain: sub, squared, sum_cols over one row, mul by the constant 1/n
//       (the tape of examples/sine_net.rs:150-156 with the sum taken on the device)
//       gradient: x_grad_i += ((x_i - y_i) * 2) * ((1/n) * upstream)   — the product the chain's
//       mul / sum_cols / square / sub gradient functions form, in their order
//   softmax cross-entropy    p = softmax(logits);  loss_r = -ln sum_c clip(p, 1e-7, 1-1e-7) * t
//       reference: Matrix::softmax + cce (examples/nn.rs:124-143)
//       gradient wrt the logits of mean_r loss_r, for the unclipped p the reference's cce_grad
//       uses (examples/nn.rs:145-152) pushed through softmax_grad in closed form:
//           p * (g - <p, g>) with g = -(t / p) / rows   ==   (p * sum_c t - t) / rows
//       which never divides by p (the chain yields inf * 0 when a probability underflows).
#include "common.hpp"

namespace slhip {

// ---------------------------------------------------------------- mean squared error
__global__ __launch_bounds__(256) void mse_partial_kernel(size_t n, const float* __restrict__ x,
                                                          const float* __restrict__ y, float* __restrict__ part,
                                                          size_t chunk, int vec, float inv_n, float* __restrict__ out) {
  __shared__ float smem[4];
  const size_t beg = (size_t)blockIdx.x * chunk, end = beg + chunk < n ? beg + chunk : n;
  float s = 0.0f;
  if (vec) {  // chunk is a multiple of 4 (always) and both pointers are 16-byte aligned
    for (size_t i = beg + 4 * (size_t)threadIdx.x; i + 3 < end; i += 1024) {
      const float4 a = ld4g(x + i), b = ld4g(y + i);
      const float d0 = a.x - b.x, d1 = a.y - b.y, d2 = a.z - b.z, d3 = a.w - b.w;
      s += (d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3);
    }
    const size_t tail = beg + ((end - beg) & ~(size_t)3);
    for (size_t i = tail + threadIdx.x; i < end; i += 256) {
      const float d = x[i] - y[i];
      s += d * d;
    }
  } else {
    for (size_t i = beg + threadIdx.x; i < end; i += 256) {
      const float d = x[i] - y[i];
      s += d * d;
    }
  }
  s = block_reduce<SumOp>(s, smem);
  if (threadIdx.x == 0) {
    if (gridDim.x == 1) out[0] = s * inv_n;  // a single block is its own final stage
    else part[blockIdx.x] = s;
  }
}

__global__ __launch_bounds__(64) void mse_final_kernel(unsigned nparts, const float* __restrict__ part, float inv_n,
                                                       float* __restrict__ out) {
  float s = 0.0f;
  for (unsigned i = threadIdx.x; i < nparts; i += 64) s += part[i];
  s = wave_reduce<SumOp>(s);
  if (threadIdx.x == 0) out[0] = s * inv_n;
}

__global__ __launch_bounds__(256) void mse_grad_kernel(size_t n, const float* __restrict__ x, const float* __restrict__ y,
                                                       float* __restrict__ x_grad, float inv_n,
                                                       const float* __restrict__ upstream) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const float gs = inv_n * upstream[0];
  x_grad[i] += ((x[i] - y[i]) * 2.0f) * gs;
}

// ---------------------------------------------------------------- softmax cross-entropy
// The fallback for rows too long for the one-pass softmax kernels when the caller wants no
// probabilities: L lanes per row, the row swept from global memory three times.
template <int L>
__global__ __launch_bounds__(256) void softmax_cce_kernel(size_t rows, size_t cols, const float* __restrict__ x,
                                                          const float* __restrict__ t, float* __restrict__ probs,
                                                          float* __restrict__ loss_rows) {
  const size_t r = (size_t)blockIdx.x * (256 / L) + threadIdx.x / L;
  const bool active = r < rows;
  const int lane = threadIdx.x % L;
  const float* xr = x + (active ? r : 0) * cols;
  const float* tr = t + (active ? r : 0) * cols;
  float m = -__builtin_huge_valf();
  if (active)
    for (size_t c = lane; c < cols; c += L) m = fmaxf(m, xr[c]);
  m = wave_reduce<MaxOp, L>(m);
  float s = 0.0f;
  if (active)
    for (size_t c = lane; c < cols; c += L) s += expf(xr[c] - m);
  s = wave_reduce<SumOp, L>(s);
  const float lo = (float)1e-7, hi = (float)(1.0 - 1e-7);
  float acc = 0.0f;
  if (active)
    for (size_t c = lane; c < cols; c += L) {
      const float p = expf(xr[c] - m) / s;
      if (probs) probs[r * cols + c] = p;
      acc += fminf(fmaxf(p, lo), hi) * tr[c];
    }
  acc = wave_reduce<SumOp, L>(acc);
  if (active && lane == 0) loss_rows[r] = -logf(acc);
}

}  // namespace slhip

using namespace slhip;

SLHIP_API int32_t slhip_mse(slhip_ctx* ctx, size_t n, const float* x, const float* y, float* loss_dev) {
  SLHIP_REQUIRE(ctx && x && y && loss_dev, "null argument");
  SLHIP_REQUIRE(n > 0, "empty buffer");
  // every block a contiguous chunk that is a multiple of 4 long; at most 1024 blocks
  size_t blocks = (n + 4095) / 4096;
  if (blocks > 1024) blocks = 1024;
  if (blocks * sizeof(float) > ctx->workspace_bytes) {
    set_error("slhip_mse: workspace too small");
    return SLHIP_EWORKSPACE;
  }
  const size_t chunk = ((n + blocks - 1) / blocks + 3) / 4 * 4;
  blocks = (n + chunk - 1) / chunk;
  const int vec = 1;
  float* part = (float*)ctx->workspace;
  hipLaunchKernelGGL(mse_partial_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, n, x, y, part, chunk, vec,
                     1.0f / (float)n, loss_dev);
  int32_t rc = post_launch();
  if (rc || blocks == 1) return rc;
  hipLaunchKernelGGL(mse_final_kernel, dim3(1), dim3(64), 0, ctx->stream, (unsigned)blocks, (const float*)part,
                     1.0f / (float)n, loss_dev);
  return post_launch();
}

SLHIP_API int32_t slhip_mse_grad(slhip_ctx* ctx, size_t n, const float* x, const float* y, float* x_grad,
                                 const float* upstream_dev) {
  SLHIP_REQUIRE(ctx && x && y && x_grad && upstream_dev, "null argument");
  SLHIP_REQUIRE(n > 0, "empty buffer");
  const size_t blocks = (n + 255) / 256;
  SLHIP_REQUIRE(blocks <= 0x7fffffffu, "buffer too long for one launch");
  hipLaunchKernelGGL(mse_grad_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, n, x, y, x_grad,
                     1.0f / (float)n, upstream_dev);
  return post_launch();
}

SLHIP_API int32_t slhip_softmax_cce(slhip_ctx* ctx, size_t rows, size_t cols, const float* logits, const float* targets,
                                    float* probs, float* loss_rows) {
  size_t len;
  SLHIP_REQUIRE(ctx && logits && targets && loss_rows, "null argument");
  SLHIP_REQUIRE(checked_len(rows, cols, &len), "bad dims");
  SLHIP_REQUIRE(rows <= 0x7fffffffu, "too many rows for one launch");
  // rows that fit the softmax kernels' registers or LDS chunks: one pass, 12 B per element
  if (cols <= softmax_one_pass_cols()) return softmax_cce_rows(ctx, rows, cols, logits, targets, probs, loss_rows);
  // longer rows: the streaming softmax, then the cross-entropy as a row reduction
  if (probs) {
    int32_t rc = slhip_softmax(ctx, rows, cols, logits, probs);
    if (rc) return rc;
    return slhip_cce(ctx, rows, cols, probs, targets, loss_rows);
  }
  // ... and without a buffer for the probabilities: one wave per row, three sweeps
  const size_t blocks = (rows + 3) / 4;
  hipLaunchKernelGGL((softmax_cce_kernel<64>), dim3((unsigned)blocks), dim3(256), 0, ctx->stream, rows, cols, logits, targets, probs,
                     loss_rows);
  return post_launch();
}

SLHIP_API int32_t slhip_softmax_cce_grad(slhip_ctx* ctx, size_t rows, size_t cols, const float* probs,
                                         const float* targets, float* logits_grad, float beta,
                                         const float* upstream_dev) {
  size_t len;
  SLHIP_REQUIRE(ctx && probs && targets && logits_grad && upstream_dev, "null argument");
  SLHIP_REQUIRE(checked_len(rows, cols, &len), "bad dims");
  SLHIP_REQUIRE(rows <= 0x7fffffffu, "too many rows for one launch");
  return softmax_cce_grad_rows(ctx, rows, cols, probs, targets, logits_grad, beta, upstream_dev);
}
