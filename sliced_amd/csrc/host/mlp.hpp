// The two training loops of the reference's examples, written against the Matrix / HIP device
// API exactly as the examples are written against Matrix / CPU:
//   Linear { weights, bias }   forward = gemm + add_row_mut          examples/sine_net.rs:8-48
//   SGD                         value -= grad * lr                     examples/sine_net.rs:80-117
//   sine fit (kind 0)           examples/sine_net.rs:119-166
//   classifier (kind 1)         examples/nn.rs:154-244, cce / cce_grad :124-152
// Everything stays on the device; per step the host reads back one float (the loss).
#pragma once
#include <chrono>

#include "sliced.hpp"

namespace sliced {

struct Linear {
  Matrix weights, bias;
  size_t in = 0, out = 0;
  Linear() = default;
  Linear(HIP& dev, size_t i, size_t o, const float* w, const float* b)
      : weights(dev.from(w, i * o), i, o), bias(dev.from(b, o), 1, o), in(i), out(o) {
    weights.require_grad();
    bias.require_grad();
  }
  // inputs.gemm(&weights); out.add_row_mut(&bias)
  Matrix forward(const Matrix& x) const {
    Matrix y = x.gemm(weights);
    y.add_row_mut(bias);
    return y;
  }
  // the same Linear (+ ReLU) as one fused kernel
  Matrix forward_fused(const Matrix& x, bool relu) const {
    return Matrix(x.device().linear(x.rows, in, out, x.data, weights.data, bias.data, relu), x.rows, out);
  }
};

struct SGD {
  float lr;
  void step(HIP& dev, Linear& l) const {
    dev.sgd_step(l.weights.data, lr);
    dev.sgd_step(l.bias.data, lr);
  }
  // every layer's parameters in one launch
  void step(HIP& dev, std::initializer_list<Linear*> layers) const {
    std::vector<Buffer> params;
    for (Linear* l : layers) {
      params.push_back(l->weights.data);
      params.push_back(l->bias.data);
    }
    dev.sgd_step(params, lr);
  }
};

struct MlpResult {
  double seconds = 0.0;  // wall time of the timed steps, device idle on both sides
  size_t graph_nodes = 0;  // kernels per recorded step (MLP_GRAPH only)
};

enum MlpMode {
  MLP_FUSED = 1,  // Linear (+ReLU) forward as one kernel, ReLU gradient inside the next layer's input-gradient GEMM
  MLP_GRAPH = 2,  // step 0 runs eagerly, step 1 is recorded, every later step replays the recording
  MLP_FUSED_LOSS = 4,  // the loss chain (MSE, or softmax + cross-entropy) as one forward and one backward kernel
  MLP_WHOLE_STEP = 8   // kind 0 with at most 64 hidden units: the whole step as two launches (HIP::mlp3_mse_step)
};

// kind 0: MSE on the tape (sub, square, sum_cols, mul by 1/n; seed 1).
// kind 1: softmax on the tape, cce / cce_grad off the tape, backward_with.
// `params` are six host arrays W1,b1,W2,b2,W3,b3 and receive the trained values back.
// Without MLP_GRAPH the host reads the loss back every step, as the examples do; with it the
// losses collect in a device array and are read once at the end (the lazy example reads
// `loss.replace()` after `dev.run()`, examples/sine_net.rs:209-212).
inline MlpResult mlp_train(HIP& dev, int kind, size_t batch, size_t d_in, size_t d_h, size_t d_out, const float* x_host,
                           const float* target_host, float* const params[6], float lr, size_t steps, size_t warmup,
                           float* losses, int mode) {
  const bool fused = (mode & MLP_FUSED) != 0, graph = (mode & MLP_GRAPH) != 0, fused_loss = (mode & MLP_FUSED_LOSS) != 0;
  Linear lin1(dev, d_in, d_h, params[0], params[1]);
  Linear lin2(dev, d_h, d_h, params[2], params[3]);
  Linear lin3(dev, d_h, d_out, params[4], params[5]);
  Matrix x(dev.from(x_host, batch * d_in), batch, d_in);
  Matrix y(dev.from(target_host, batch * d_out), batch, d_out);
  x.no_grad();
  y.no_grad();
  const size_t n_out = batch * d_out;
  const float inv = 1.0f / (float)n_out;
  Matrix c(dev.from(&inv, 1), 1, 1);
  c.no_grad();
  SGD sgd{lr};
  // loss pieces of kind 1 live outside the cache: they are not tape outputs
  Buffer loss_rows = kind == 1 ? dev.alloc(batch, true) : Buffer();
  Buffer seed = kind == 1 ? dev.alloc(n_out, true) : Buffer();
  Buffer loss_dev = dev.alloc(1, true);
  Buffer loss_log = graph ? dev.alloc(warmup + steps, true) : Buffer();

  // with the fused Linear the ReLU gradients ride in the next layer's input-gradient GEMM
  dev.policy.fuse_relu_grad = fused;
  dev.policy.relu_bits = fused;

  // One training step.  Reads the loss back unless `deferred`; then `loss_at` names the device
  // scalar that holds it (the same one every step: op outputs are cached by call position).
  Buffer loss_at = loss_dev;
  auto train_step = [&](bool deferred) -> float {
    dev.zero_grad();
    Matrix out;
    if (fused) {
      Matrix h1 = lin1.forward_fused(x, true);
      Matrix h2 = lin2.forward_fused(h1, true);
      out = lin3.forward_fused(h2, false);
    } else {
      Matrix h1 = lin1.forward(x).relu();
      Matrix h2 = lin2.forward(h1).relu();
      out = lin3.forward(h2);
    }
    float loss_val = 0.0f;
    if (fused_loss) {
      Buffer L = kind == 0 ? dev.mse_loss(out.data, y.data) : dev.softmax_cce_loss(batch, d_out, out.data, y.data);
      if (deferred) loss_at = L;
      else loss_val = L.read()[0];
      L.backward();
    } else if (kind == 0) {
      Matrix d = out.sub(y);
      Matrix q = d.squared();
      Matrix s = q.as_dims(1, n_out).sum_cols();  // one row: the sum over every element
      Matrix L = s.mul(c);
      if (deferred) loss_at = L.data;
      else loss_val = L.read()[0];
      L.backward();
    } else {
      Matrix p = out.softmax();
      check(slhip_cce(dev.ctx(), batch, d_out, p.data.ptr, y.data.ptr, loss_rows.ptr), "slhip_cce");
      if (deferred) dev.mean_to(loss_rows, loss_dev);
      else loss_val = dev.mean(loss_rows);
      check(slhip_cce_grad(dev.ctx(), batch, d_out, p.data.ptr, y.data.ptr, seed.ptr), "slhip_cce_grad");
      p.data.backward_with(seed);
    }
    if (fused) {
      sgd.step(dev, {&lin1, &lin2, &lin3});
    } else {
      sgd.step(dev, lin1);
      sgd.step(dev, lin2);
      sgd.step(dev, lin3);
    }
    return loss_val;
  };

  MlpResult res;
  Graph recorded;
  std::chrono::steady_clock::time_point t0;
  if (mode & MLP_WHOLE_STEP) {
    if (kind != 0) throw Error("the whole-step kernels serve the MSE loop only");
    const std::vector<Buffer> ps{lin1.weights.data, lin1.bias.data, lin2.weights.data, lin2.bias.data, lin3.weights.data, lin3.bias.data};
    Buffer log = dev.alloc(warmup + steps, true);
    for (size_t it = 0; it < warmup + steps; ++it) {
      if (it == warmup) {
        dev.sync();
        t0 = std::chrono::steady_clock::now();
      }
      dev.mlp3_mse_step(batch, d_in, d_h, d_out, x.data, y.data, ps, lr, log, it);  // the loss of step `it` lands in log[it]
    }
    dev.sync();
    res.seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    res.graph_nodes = 2;
    std::vector<float> all = log.read();
    for (size_t i = 0; i < steps; ++i) losses[i] = all[warmup + i];
    const Linear* ls[3] = {&lin1, &lin2, &lin3};
    for (int i = 0; i < 3; ++i) {
      std::vector<float> w = ls[i]->weights.read(), b = ls[i]->bias.read();
      for (size_t j = 0; j < w.size(); ++j) params[2 * i][j] = w[j];
      for (size_t j = 0; j < b.size(); ++j) params[2 * i + 1][j] = b[j];
    }
    return res;
  }
  for (size_t it : dev.range(warmup + steps)) {
    if (it == warmup) {
      dev.sync();
      t0 = std::chrono::steady_clock::now();
    }
    if (!graph) {
      const float loss_val = train_step(false);
      if (it >= warmup) losses[it - warmup] = loss_val;
      continue;
    }
    if (it == 0) {
      train_step(true);  // eagerly: fills the cache and the gradient map
    } else {
      if (!recorded.valid()) {
        recorded = dev.record([&] { train_step(true); });
        res.graph_nodes = recorded.nodes();
      }
      recorded.run();
    }
    dev.copy(loss_at, 0, loss_log, it, 1);
  }
  dev.sync();
  res.seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
  if (graph) {
    std::vector<float> log = loss_log.read();
    for (size_t i = 0; i < steps; ++i) losses[i] = log[warmup + i];
  }
  // warm-up steps train too: hand back what the timed steps ended with
  const Linear* ls[3] = {&lin1, &lin2, &lin3};
  for (int i = 0; i < 3; ++i) {
    std::vector<float> w = ls[i]->weights.read(), b = ls[i]->bias.read();
    for (size_t j = 0; j < w.size(); ++j) params[2 * i][j] = w[j];
    for (size_t j = 0; j < b.size(); ++j) params[2 * i + 1][j] = b[j];
  }
  return res;
}

}  // namespace sliced
