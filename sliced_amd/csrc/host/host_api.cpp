// C entry points of the host device layer (sliced.hpp / mlp.hpp), so that tests and the
// benchmark can drive the C++ tape from another language.  Buffers are named by their ids.
// Every function returns 0 on success and -1 on error; slh_last_error() gives the text.
#include <cstring>
#include <string>

#include "mlp.hpp"

using namespace sliced;

#define SLH_API extern "C" __attribute__((visibility("default")))

static thread_local std::string g_err = "no error";

template <class F>
static int guard(F&& f) {
  try {
    f();
    return 0;
  } catch (const std::exception& e) {
    g_err = e.what();
    return -1;
  }
}

SLH_API const char* slh_last_error(void) { return g_err.c_str(); }

SLH_API int slh_device_new(int ordinal, int cached, void** dev) {
  return guard([&] { *dev = new HIP(ordinal, cached != 0); });
}
SLH_API int slh_device_free(void* dev) {
  return guard([&] { delete (HIP*)dev; });
}
SLH_API int slh_set_grad_policy(void* dev, float gemm_beta, float softmax_beta, float transpose_beta) {
  return guard([&] {
    GradPolicy& p = ((HIP*)dev)->policy;
    p.gemm_beta = gemm_beta; p.softmax_beta = softmax_beta; p.transpose_beta = transpose_beta;
  });
}
SLH_API int slh_set_fuse_relu_grad(void* dev, int on) {
  return guard([&] { ((HIP*)dev)->policy.fuse_relu_grad = on != 0; });
}
SLH_API int slh_set_relu_bits(void* dev, int on) {
  return guard([&] { ((HIP*)dev)->policy.relu_bits = on != 0; });
}
// Elementwise ops are deferred and chains of them launched as one kernel (GradPolicy::fuse_elementwise).
SLH_API int slh_set_fuse_elementwise(void* dev, int on) {
  return guard([&] {
    HIP* d = (HIP*)dev;
    d->run();
    d->policy.fuse_elementwise = on != 0;
  });
}
SLH_API int slh_run(void* dev) {  // launches whatever is deferred: the lazy device's `run()`
  return guard([&] { ((HIP*)dev)->run(); });
}
SLH_API size_t slh_deferred(void* dev) { return ((HIP*)dev)->deferred(); }
SLH_API int slh_enable_tape(void* dev, int on) {
  return guard([&] { ((HIP*)dev)->enable_tape(on != 0); });
}
SLH_API int slh_device_ctx(void* dev, void** ctx) {  // the slhip context the device issues its ops on
  return guard([&] { *ctx = (void*)((HIP*)dev)->ctx(); });
}
// Records body-less helper for tests: begins / ends a recording around ops issued through this API.
SLH_API int slh_record_begin(void* dev) {
  return guard([&] {
    HIP* d = (HIP*)dev;
    d->run();
    check(slhip_graph_begin(d->ctx()), "slhip_graph_begin");
  });
}
SLH_API int slh_record_end(void* dev, size_t* nodes) {
  return guard([&] {
    HIP* d = (HIP*)dev;
    d->run();
    slhip_graph* g = nullptr;
    check(slhip_graph_end(d->ctx(), &g), "slhip_graph_end");
    check(slhip_graph_node_count(g, nodes), "slhip_graph_node_count");
    check(slhip_graph_launch(d->ctx(), g), "slhip_graph_launch");  // the recorded ops have not run yet: run them once
    check(slhip_sync(d->ctx()), "slhip_sync");
    slhip_graph_destroy(g);
  });
}
// The two elementwise chains of the reference's examples written against Matrix, method by method:
// which == 0: ((a + b) * c - d).pow(2).squared()      (the bandwidth suite's chain; a, b, c, d)
// which == 1: square(x) * x + (b + x) * b              (examples/chained_perf.rs:86-90; a = x, b = b)
SLH_API int slh_matrix_chain(void* dev, int which, size_t rows, size_t cols, uint64_t a, uint64_t b, uint64_t c,
                             uint64_t d, uint64_t* out) {
  return guard([&] {
    HIP* dv = (HIP*)dev;
    if (which == 0) {
      Matrix A(dv->lookup(a), rows, cols), B(dv->lookup(b), rows, cols), C(dv->lookup(c), rows, cols),
          D(dv->lookup(d), rows, cols);
      *out = A.add(B).mul(C).sub(D).pow(2.0f).squared().data.id;
    } else {
      Matrix X(dv->lookup(a), rows, cols), B(dv->lookup(b), rows, cols);
      Matrix squared = X.squared();
      Matrix add = B.add(X);
      Matrix mul_b = add.mul(B);
      Matrix mul = squared.mul(X);
      *out = mul.add(mul_b).data.id;
    }
  });
}
// Matrix::rand (src/matrix.rs:266-271) on a rows x cols view of the buffer
SLH_API int slh_matrix_rand(void* dev, uint64_t id, size_t rows, size_t cols, float lo, float hi, uint64_t seed, uint64_t tag) {
  return guard([&] {
    HIP* dv = (HIP*)dev;
    Matrix m(dv->lookup(id), rows, cols);
    m.rand(lo, hi, seed, tag);
  });
}
SLH_API int slh_buffer_from(void* dev, const float* host, size_t len, uint64_t* id) {
  return guard([&] { *id = ((HIP*)dev)->from(host, len).id; });
}
SLH_API int slh_buffer_zeros(void* dev, size_t len, uint64_t* id) {
  return guard([&] { *id = ((HIP*)dev)->alloc(len, true).id; });
}
SLH_API int slh_buffer_ptr(void* dev, uint64_t id, void** ptr) {  // the device address, for callers that fill it themselves
  return guard([&] { *ptr = (void*)((HIP*)dev)->lookup(id).ptr; });
}
SLH_API int slh_buffer_len(void* dev, uint64_t id, size_t* len) {
  return guard([&] { *len = ((HIP*)dev)->lookup(id).len; });
}
SLH_API int slh_buffer_read(void* dev, uint64_t id, float* host) {
  return guard([&] {
    std::vector<float> v = ((HIP*)dev)->lookup(id).read();
    std::memcpy(host, v.data(), v.size() * sizeof(float));
  });
}
SLH_API int slh_buffer_release(void* dev, uint64_t id) {
  return guard([&] { ((HIP*)dev)->release(id); });
}
SLH_API int slh_require_grad(void* dev, uint64_t id, int on) {
  return guard([&] { ((HIP*)dev)->set_requires_grad(id, on != 0); });
}
SLH_API int slh_grad(void* dev, uint64_t id, uint64_t* grad_id) {
  return guard([&] {
    HIP* d = (HIP*)dev;
    *grad_id = d->grad(d->lookup(id)).id;
  });
}
SLH_API int slh_has_grad(void* dev, uint64_t id) { return ((HIP*)dev)->has_grad(id) ? 1 : 0; }
SLH_API int slh_zero_grad(void* dev) {
  return guard([&] { ((HIP*)dev)->zero_grad(); });
}
SLH_API int slh_backward(void* dev, uint64_t id) {
  return guard([&] {
    HIP* d = (HIP*)dev;
    d->backward(d->lookup(id));
  });
}
SLH_API int slh_backward_with(void* dev, uint64_t id, uint64_t seed_id) {
  return guard([&] {
    HIP* d = (HIP*)dev;
    d->backward_with(d->lookup(id), d->lookup(seed_id));
  });
}
SLH_API int slh_begin_iteration(void* dev) {  // what `device.range` does at the top of every iteration
  return guard([&] { (void)((HIP*)dev)->range(0).begin(); });
}
SLH_API size_t slh_tape_len(void* dev) { return ((HIP*)dev)->tape_len(); }

// ---- ops (forward + tape registration) -------------------------------------------------------
SLH_API int slh_gemm(void* dev, size_t m, size_t k, size_t n, uint64_t lhs, uint64_t rhs, uint64_t* out) {
  return guard([&] {
    HIP* d = (HIP*)dev;
    *out = d->gemm(m, k, n, d->lookup(lhs), d->lookup(rhs)).id;
  });
}
SLH_API int slh_linear(void* dev, size_t m, size_t k, size_t n, uint64_t x, uint64_t w, uint64_t bias, int relu,
                       uint64_t* out) {
  return guard([&] {
    HIP* d = (HIP*)dev;
    *out = d->linear(m, k, n, d->lookup(x), d->lookup(w), d->lookup(bias), relu != 0).id;
  });
}
SLH_API int slh_add_row(void* dev, size_t rows, size_t cols, uint64_t lhs, uint64_t rhs, uint64_t* out) {
  return guard([&] {
    HIP* d = (HIP*)dev;
    *out = d->add_row(rows, cols, d->lookup(lhs), d->lookup(rhs)).id;
  });
}
SLH_API int slh_add_row_mut(void* dev, size_t rows, size_t cols, uint64_t lhs, uint64_t rhs) {
  return guard([&] {
    HIP* d = (HIP*)dev;
    d->add_row_mut(rows, cols, d->lookup(lhs), d->lookup(rhs));
  });
}
SLH_API int slh_binary(void* dev, int op, uint64_t lhs, uint64_t rhs, uint64_t* out) {
  return guard([&] {
    HIP* d = (HIP*)dev;
    *out = d->binary(op, d->lookup(lhs), d->lookup(rhs)).id;
  });
}
SLH_API int slh_unary(void* dev, int op, float p, float q, uint64_t x, int with_grad, uint64_t* out) {
  return guard([&] {
    HIP* d = (HIP*)dev;
    *out = d->unary(op, d->lookup(x), p, q, with_grad != 0).id;
  });
}
// by_row_index 0: row_op (rhs has one entry per column), 1: col_op (one per row); op = SLHIP_ADD..DIV
SLH_API int slh_bcast_op(void* dev, int by_row_index, int op, size_t rows, size_t cols, uint64_t lhs, uint64_t rhs,
                         uint64_t* out) {
  return guard([&] {
    HIP* d = (HIP*)dev;
    *out = d->bcast_op(by_row_index != 0, op, rows, cols, d->lookup(lhs), d->lookup(rhs)).id;
  });
}
SLH_API int slh_diagflat(void* dev, uint64_t x, uint64_t* out) {
  return guard([&] {
    HIP* d = (HIP*)dev;
    *out = d->diagflat(d->lookup(x)).id;
  });
}
SLH_API int slh_onehot(void* dev, size_t classes, uint64_t cls, uint64_t* out) {
  return guard([&] {
    HIP* d = (HIP*)dev;
    *out = d->onehot(classes, d->lookup(cls)).id;
  });
}
SLH_API int slh_mse_loss(void* dev, uint64_t x, uint64_t y, uint64_t* out) {
  return guard([&] {
    HIP* d = (HIP*)dev;
    *out = d->mse_loss(d->lookup(x), d->lookup(y)).id;
  });
}
SLH_API int slh_softmax_cce_loss(void* dev, size_t rows, size_t cols, uint64_t logits, uint64_t targets, uint64_t* out) {
  return guard([&] {
    HIP* d = (HIP*)dev;
    *out = d->softmax_cce_loss(rows, cols, d->lookup(logits), d->lookup(targets)).id;
  });
}
SLH_API int slh_transpose(void* dev, size_t rows, size_t cols, uint64_t x, uint64_t* out) {
  return guard([&] {
    HIP* d = (HIP*)dev;
    *out = d->transpose(rows, cols, d->lookup(x)).id;
  });
}
SLH_API int slh_softmax(void* dev, size_t samples, size_t features, uint64_t x, uint64_t* out) {
  return guard([&] {
    HIP* d = (HIP*)dev;
    *out = d->softmax(samples, features, d->lookup(x)).id;
  });
}
// kind: 0 sum_rows, 1 sum_cols, 2 max_rows, 3 max_cols, 4 mean_rows, 5 mean_cols
SLH_API int slh_reduce(void* dev, int kind, size_t rows, size_t cols, uint64_t x, uint64_t* out) {
  return guard([&] {
    HIP* d = (HIP*)dev;
    if (kind < 0 || kind > 5) throw Error("unknown reduction");
    *out = d->reduce((HIP::Red)kind, rows, cols, d->lookup(x)).id;
  });
}
SLH_API int slh_mean(void* dev, uint64_t x, float* out) {
  return guard([&] {
    HIP* d = (HIP*)dev;
    *out = d->mean(d->lookup(x));
  });
}
SLH_API int slh_sgd_step(void* dev, uint64_t p, float lr) {
  return guard([&] {
    HIP* d = (HIP*)dev;
    d->sgd_step(d->lookup(p), lr);
  });
}

// ---- training loops ----------------------------------------------------------------------------
// Three-layer MLP d_in -> d_h -> relu -> d_h -> relu -> d_out on a fresh device object.
// kind 0 = sine fit (MSE on the tape), 1 = classifier (softmax + cce).  W1..b3 are updated in
// place.  `warmup` untimed steps run first (they train too); seconds = wall time of `steps`.
// mode: bit 0 = fused Linear forward, bit 1 = record one step as a graph and replay it,
// bit 2 = fused loss kernels.
SLH_API int slh_mlp_train(int ordinal, int kind, size_t batch, size_t d_in, size_t d_h, size_t d_out, const float* x,
                          const float* target, float* W1, float* b1, float* W2, float* b2, float* W3, float* b3,
                          float lr, size_t steps, size_t warmup, int mode, float* losses, double* seconds,
                          size_t* graph_nodes) {
  return guard([&] {
    HIP dev(ordinal, true);
    float* params[6] = {W1, b1, W2, b2, W3, b3};
    MlpResult r = mlp_train(dev, kind, batch, d_in, d_h, d_out, x, target, params, lr, steps, warmup, losses, mode);
    if (seconds) *seconds = r.seconds;
    if (graph_nodes) *graph_nodes = r.graph_nodes;
  });
}
