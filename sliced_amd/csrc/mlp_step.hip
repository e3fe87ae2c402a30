// One whole training step of a small three-layer perceptron in two launches.
//
//   x[batch x d_in] -> Linear(d_in, d_h) -> ReLU -> Linear(d_h, d_h) -> ReLU -> Linear(d_h, d_out)
//   loss = (sum over every output (out - y)^2) * 1/(batch * d_out), plain SGD
//
// the loop of examples/sine_net.rs:119-166 (Linear = gemm + add_row_mut, :32-40; Matrix::relu,
// src/matrix.rs:169-190; the loss tape sub, squared, sum, scale; SGD `value -= grad * lr`, :105-116).
// Issued op by op that step is ten launches of 4-12 us each for 26 MFLOP of arithmetic and 17 KB of
// parameters: all launch latency.  Here:
//
//   mlp3_rows_kernel   one wave per batch row (a wave loops when there are more rows than waves): lane j
//                      owns hidden unit j.  The d_h x d_h weight matrix sits in registers twice - lane j
//                      holds column j for the forward product and row j for the backward one - so both
//                      are 64 multiply-adds per lane with the other factor broadcast from a lane by
//                      v_readlane; no LDS traffic and no barrier in the row loop.  It leaves h1, h2 and
//                      the pre-activation gradients dz1, dz2, dout of its row in the context workspace.
//   mlp3_update_kernel one workgroup per row of the hidden weight matrix, plus three for the rest:
//                      every weight and bias gradient is a sum over the batch of a product of two of
//                      those per-row vectors, added up by sixteen waves over a sixteenth of the rows each
//                      and combined in wave order, then the SGD update in place (and the gradient
//                      itself, if the caller keeps gradient buffers).  The loss is summed the same way.
//
// Every sum has a fixed order: a step gives the same bits whenever it runs.  The values differ from
// the op-by-op sequence in rounding only (fused multiply-adds, a butterfly instead of a sequential sum
// over the hidden units); the per-step loss stays within 2e-6 relative of the oracle's loop over the
// 200 steps of the sine fit.
#include "common.hpp"

namespace slhip {

constexpr int MLP_H = 64;       // hidden units: one per lane
constexpr int MLP_IO = 8;       // most inputs and outputs per row

struct Mlp3Args {
  size_t batch;
  int d_in, d_h, d_out;
  const float* x;
  const float* y;
  float *w1, *b1, *w2, *b2, *w3, *b3;
  float *g_w1, *g_b1, *g_w2, *g_b2, *g_w3, *g_b3;  // may be null
  // per-row results of the first kernel, in the workspace: [batch][64] each, then [batch][8] each
  float *h1, *h2, *dz1, *dz2, *dout, *q;
  float lr, inv_n;
  float* loss;
};

__device__ __forceinline__ float relu_ref(float z) { return (z >= 0.0f ? 1.0f : 0.0f) * z; }
__device__ __forceinline__ float bcast_lane(float v, int k) { return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), k)); }

__global__ __launch_bounds__(256) void mlp3_rows_kernel(Mlp3Args a) {
  __shared__ float w2s[MLP_H * (MLP_H + 1)];  // pitch 65: a lane reading its row meets no other lane's bank
  const int lane = threadIdx.x & 63;
  const int H = a.d_h;
  for (int i = threadIdx.x; i < MLP_H * MLP_H; i += 256) {
    const int k = i >> 6, j = i & 63;
    w2s[k * (MLP_H + 1) + j] = (k < H && j < H) ? a.w2[k * H + j] : 0.0f;
  }
  __syncthreads();
  float w2c[MLP_H], w2r[MLP_H];  // column `lane` and row `lane` of the hidden weight matrix
#pragma unroll
  for (int k = 0; k < MLP_H; ++k) {
    w2c[k] = w2s[k * (MLP_H + 1) + lane];
    w2r[k] = w2s[lane * (MLP_H + 1) + k];
  }
  const bool live = lane < H;
  float w1[MLP_IO], w3[MLP_IO], b3[MLP_IO];
#pragma unroll
  for (int i = 0; i < MLP_IO; ++i) {
    w1[i] = (live && i < a.d_in) ? a.w1[i * H + lane] : 0.0f;
    w3[i] = (live && i < a.d_out) ? a.w3[lane * a.d_out + i] : 0.0f;
    b3[i] = i < a.d_out ? a.b3[i] : 0.0f;
  }
  const float b1 = live ? a.b1[lane] : 0.0f, b2 = live ? a.b2[lane] : 0.0f;

  const unsigned wave = __builtin_amdgcn_readfirstlane(blockIdx.x * 4 + (threadIdx.x >> 6));
  const unsigned waves = gridDim.x * 4;
  for (size_t r = wave; r < a.batch; r += waves) {
    // layer 1: z1 = x . W1 (the terms in order, as the product's k loop runs) + b1
    const float* xr = a.x + r * a.d_in;
    float z1 = xr[0] * w1[0];
#pragma unroll
    for (int i = 1; i < MLP_IO; ++i)
      if (i < a.d_in) z1 = z1 + xr[i] * w1[i];
    z1 = z1 + b1;
    const float h1 = live ? relu_ref(z1) : 0.0f;  // lanes past d_h stay out of every sum, whatever x holds
    // layer 2: z2[j] = sum_k h1[k] W2[k][j], k ascending
    float z2 = 0.0f;
#pragma unroll
    for (int k = 0; k < MLP_H; ++k) z2 = __builtin_fmaf(bcast_lane(h1, k), w2c[k], z2);
    z2 = z2 + b2;
    const float h2 = live ? relu_ref(z2) : 0.0f;
    // layer 3 and the loss: out[o] = sum_k h2[k] W3[k][o] + b3[o]; d = out - y; q = d^2
    // backward: L = (sum q) * inv_n seeded with one  ->  dout = (d * 2) * inv_n
    float dout[MLP_IO], qv[MLP_IO], dh2 = 0.0f;
#pragma unroll
    for (int o = 0; o < MLP_IO; ++o) {
      dout[o] = 0.0f;
      qv[o] = 0.0f;
      if (o < a.d_out) {
        const float out = wave_reduce<SumOp>(h2 * w3[o]) + b3[o];
        const float d = out - a.y[r * a.d_out + o];
        qv[o] = d * d;
        dout[o] = (d * 2.0f) * a.inv_n;
        dh2 = __builtin_fmaf(dout[o], w3[o], dh2);
      }
    }
    const float dz2 = (z2 >= 0.0f ? 1.0f : 0.0f) * dh2;
    // dh1[k] = sum_j dz2[j] W2[k][j]
    float dh1 = 0.0f;
#pragma unroll
    for (int j = 0; j < MLP_H; ++j) dh1 = __builtin_fmaf(bcast_lane(dz2, j), w2r[j], dh1);
    const float dz1 = (z1 >= 0.0f ? 1.0f : 0.0f) * dh1;
    a.h1[r * MLP_H + lane] = h1;
    a.h2[r * MLP_H + lane] = h2;
    a.dz1[r * MLP_H + lane] = dz1;
    a.dz2[r * MLP_H + lane] = dz2;
#pragma unroll
    for (int o = 0; o < MLP_IO; ++o)
      if (lane == o) {
        a.dout[r * MLP_IO + o] = dout[o];
        a.q[r * MLP_IO + o] = qv[o];
      }
  }
}

// sum over the batch rows of u[r] * v[r * 64 + lane] (u == nullptr: of v alone), the rows dealt out to
// the sixteen waves in contiguous sixteenths and the sixteen partial sums added in wave order; every
// thread returns the total.  `red` holds 16 x 64 floats.  The loop is a chain of trips to L2, so what
// counts is how many rows are in flight: sixteen per wave, sixteen waves.
constexpr int UPD_WAVES = 16;
__device__ __forceinline__ float batch_dot(const float* __restrict__ u, size_t ustride, const float* __restrict__ v, size_t vstride,
                                           size_t batch, float* red) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const size_t per = (batch + UPD_WAVES - 1) / UPD_WAVES, beg = (size_t)w * per, end = beg + per < batch ? beg + per : batch;
  float acc = 0.0f;
  size_t r = beg;
  for (; r + 16 <= end; r += 16) {
    float uv[16], vv[16];
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      uv[t] = u ? u[(r + t) * ustride] : 1.0f;
      vv[t] = v[(r + t) * vstride + lane];
    }
#pragma unroll
    for (int t = 0; t < 16; ++t) acc = u ? __builtin_fmaf(uv[t], vv[t], acc) : acc + vv[t];
  }
  for (; r < end; ++r) acc = u ? __builtin_fmaf(u[r * ustride], v[r * vstride + lane], acc) : acc + v[r * vstride + lane];
  __syncthreads();  // red may still be read from the call before
  red[w * 64 + lane] = acc;
  __syncthreads();
  float total = red[lane];
#pragma unroll
  for (int i = 1; i < UPD_WAVES; ++i) total += red[i * 64 + lane];
  return total;
}

__device__ __forceinline__ void sgd_store(float* p, float* g_out, size_t idx, float g, float lr) {
  if (g_out) g_out[idx] = g;
  p[idx] = p[idx] - g * lr;  // examples/sine_net.rs:105-116: value -= grad * lr
}

__global__ __launch_bounds__(64 * UPD_WAVES) void mlp3_update_kernel(Mlp3Args a) {
  __shared__ float red[64 * UPD_WAVES];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int H = a.d_h;
  const int b = blockIdx.x;
  if (b < H) {  // row b of the hidden weight matrix: dW2[b][j] = sum_r h1[r][b] dz2[r][j]
    const float g = batch_dot(a.h1 + b, MLP_H, a.dz2, MLP_H, a.batch, red);
    if (w == 0 && lane < H) sgd_store(a.w2, a.g_w2, (size_t)b * H + lane, g, a.lr);
    return;
  }
  if (b == H) {  // dW1[i][j] = sum_r x[r][i] dz1[r][j];  db1[j] = sum_r dz1[r][j]
    for (int i = 0; i < a.d_in; ++i) {
      const float g = batch_dot(a.x + i, a.d_in, a.dz1, MLP_H, a.batch, red);
      if (w == 0 && lane < H) sgd_store(a.w1, a.g_w1, (size_t)i * H + lane, g, a.lr);
    }
    const float g = batch_dot(nullptr, 0, a.dz1, MLP_H, a.batch, red);
    if (w == 0 && lane < H) sgd_store(a.b1, a.g_b1, lane, g, a.lr);
    return;
  }
  if (b == H + 1) {  // db2[j] = sum_r dz2[r][j]
    const float g = batch_dot(nullptr, 0, a.dz2, MLP_H, a.batch, red);
    if (w == 0 && lane < H) sgd_store(a.b2, a.g_b2, lane, g, a.lr);
    return;
  }
  // dW3[k][o] = sum_r h2[r][k] dout[r][o];  db3[o] = sum_r dout[r][o];  loss = (sum_r sum_o q[r][o]) * inv_n
  for (int o = 0; o < a.d_out; ++o) {
    const float g = batch_dot(a.dout + o, MLP_IO, a.h2, MLP_H, a.batch, red);
    if (w == 0 && lane < H) sgd_store(a.w3, a.g_w3, (size_t)lane * a.d_out + o, g, a.lr);
  }
  // (the [batch][8] arrays read as [batch / 8][64]: lane o + 8 t of row-group R holds row 8 R + t, output o;
  // entries past d_out are zero)
  const size_t groups = a.batch / 8;
  float gb = batch_dot(nullptr, 0, a.dout, MLP_H, groups, red);
  float ql = batch_dot(nullptr, 0, a.q, MLP_H, groups, red);
  for (size_t r = groups * 8; r < a.batch; ++r) {  // the last rows, when the batch is no multiple of 8
    if (lane < MLP_IO) {
      gb += a.dout[r * MLP_IO + lane];
      ql += a.q[r * MLP_IO + lane];
    }
  }
  if (w == 0) {
    // lanes o, o + 8, ..., o + 56 hold the eight row residues of output o
    float gsum = gb, qsum = ql;
#pragma unroll
    for (int off = 8; off < 64; off <<= 1) {
      gsum += __shfl_xor(gsum, off, 64);
      qsum += __shfl_xor(qsum, off, 64);
    }
    if (lane < a.d_out) sgd_store(a.b3, a.g_b3, lane, gsum, a.lr);
    // the outputs of a row, then one value
    float total = lane < MLP_IO ? qsum : 0.0f;
#pragma unroll
    for (int off = 1; off < 8; off <<= 1) total += __shfl_xor(total, off, 64);
    if (lane == 0) *a.loss = total * a.inv_n;
  }
}

}  // namespace slhip

using namespace slhip;

SLHIP_API int32_t slhip_mlp3_mse_step(slhip_ctx* ctx, size_t batch, size_t d_in, size_t d_h, size_t d_out, const float* x,
                                      const float* target, float* w1, float* b1, float* w2, float* b2, float* w3, float* b3,
                                      float* const* grads, float lr, float* loss_dev) {
  SLHIP_REQUIRE(ctx && x && target && w1 && b1 && w2 && b2 && w3 && b3 && loss_dev, "null argument");
  SLHIP_REQUIRE(batch > 0 && d_in > 0 && d_h > 0 && d_out > 0, "bad dims");
  if (d_h > (size_t)MLP_H || d_in > (size_t)MLP_IO || d_out > (size_t)MLP_IO) {
    set_error("slhip_mlp3_mse_step: %zu-%zu-%zu-%zu; the one-step kernels serve at most %d hidden units and %d inputs and outputs "
              "(run the layers op by op)", d_in, d_h, d_h, d_out, MLP_H, MLP_IO);
    return SLHIP_EINVAL;
  }
  const size_t per_row = 4 * (size_t)MLP_H + 2 * (size_t)MLP_IO;
  if (batch > ctx->workspace_bytes / sizeof(float) / per_row || batch > (size_t(1) << 30)) {
    set_error("slhip_mlp3_mse_step: a batch of %zu rows does not fit the workspace", batch);
    return SLHIP_EWORKSPACE;
  }
  Mlp3Args a;
  a.batch = batch; a.d_in = (int)d_in; a.d_h = (int)d_h; a.d_out = (int)d_out;
  a.x = x; a.y = target;
  a.w1 = w1; a.b1 = b1; a.w2 = w2; a.b2 = b2; a.w3 = w3; a.b3 = b3;
  a.g_w1 = grads ? grads[0] : nullptr; a.g_b1 = grads ? grads[1] : nullptr; a.g_w2 = grads ? grads[2] : nullptr;
  a.g_b2 = grads ? grads[3] : nullptr; a.g_w3 = grads ? grads[4] : nullptr; a.g_b3 = grads ? grads[5] : nullptr;
  float* ws = (float*)ctx->workspace;
  a.h1 = ws; a.h2 = ws + batch * MLP_H; a.dz1 = ws + 2 * batch * MLP_H; a.dz2 = ws + 3 * batch * MLP_H;
  a.dout = ws + 4 * batch * MLP_H; a.q = a.dout + batch * MLP_IO;
  a.lr = lr;
  a.inv_n = 1.0f / (float)(batch * d_out);
  a.loss = loss_dev;
  // one wave per row while the chip has waves to give (four per workgroup, up to eight workgroups a CU)
  size_t blocks = (batch + 3) / 4;
  const size_t cap = (size_t)ctx->num_cu * 8;
  if (blocks > cap) blocks = cap;
  hipLaunchKernelGGL(mlp3_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, a);
  int32_t rc = post_launch();
  if (rc) return rc;
  hipLaunchKernelGGL(mlp3_update_kernel, dim3((unsigned)(d_h + 3)), dim3(64 * UPD_WAVES), 0, ctx->stream, a);
  return post_launch();
}
