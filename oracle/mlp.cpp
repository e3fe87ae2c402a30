// CPU oracle, part 2: the two training loops of the reference's examples, restated op by op
// with the oracle's slice functions in the order the autograd tape would run them.
//
// TEST INFRASTRUCTURE ONLY (see oracle.cpp).
//
// Loop shape: examples/sine_net.rs:135-164 and examples/nn.rs:184-237 —
//   zero_grad; Linear.forward = gemm + add_row_mut (examples/sine_net.rs:32-40); relu
//   (src/matrix.rs:169-190); loss; backward (tape closures in reverse); SGD step
//   (examples/sine_net.rs:105-116).
// Parity unpinned: the reference's weight init is an unseeded RNG (src/rawops/cpu/rand.rs:8),
// so no loss curve of the reference exists to compare with; parameters and data come from
// the caller, and the curve is pinned only through the per-op checks of the functions used.
#include <cstddef>
#include <cstring>
#include <vector>

extern "C" {
void orc_gemm(size_t m, size_t n, size_t k, const float* a, const float* b, float* c, float beta);
void orc_gemm_grad(size_t m, size_t k, size_t n, const float* lhs, const float* rhs, float* lhs_grad,
                   float* rhs_grad, const float* out_grad, float beta);
void orc_add_row(size_t rows, size_t cols, const float* lhs, const float* rhs, float* out);
void orc_add_row_mut_grad(size_t rows, size_t cols, float* rhs_grad, const float* out_grad);
void orc_unary(int op, float p, float q, size_t len, const float* x, float* out);
void orc_unary_grad(int op, float p, size_t len, const float* x, float* x_grad, const float* out_grad);
void orc_binary_ew(int op, size_t len, const float* l, const float* r, float* out);
void orc_binary_ew_grad(int op, size_t len, const float* l, const float* r, float* lg, float* rg,
                        const float* g);
void orc_sum_cols(size_t cols, size_t len, const float* x, float* out);
void orc_sum_cols_grad(size_t cols, size_t len, float* x_grad, const float* out_grad);
void orc_softmax(size_t samples, size_t features, const float* x, float* out);
void orc_softmax_grad(size_t samples, size_t features, float* x_grad, const float* out,
                      const float* out_grad, float beta);
void orc_cce(size_t rows, size_t cols, const float* preds, const float* targets, float* loss);
void orc_cce_grad(size_t rows, size_t cols, const float* preds, const float* targets, float* grad);
float orc_mean(size_t len, const float* x);
void orc_sgd_step(size_t n, float* p, const float* g, float lr);
}

namespace {
enum { SQUARE = 0, RELU = 2 };
enum { ADD = 0, SUB = 1, MUL = 2 };
typedef std::vector<float> V;
}  // namespace

// Three-layer MLP  d_in -> d_h -> relu -> d_h -> relu -> d_out.
//   kind 0 (sine fit): d = sub(o, y); q = square(d); s = sum_cols(q viewed as one row);
//          L = mul(s, [1/(batch*d_out)]); L.backward() (seed 1); loss value = L.
//   kind 1 (classifier): p = softmax(o); loss value = mean(cce(p, t));
//          p.backward_with(cce_grad(p, t, batch))   (examples/nn.rs:193,213-233).
// x is `no_grad` (examples/sine_net.rs:67, examples/nn.rs:170), so layer 1 gets no dX.
// Parameters are updated in place; losses[step] receives the loss of every step.
extern "C" __attribute__((visibility("default")))
int orc_mlp_train(int kind, size_t batch, size_t d_in, size_t d_h, size_t d_out, const float* x,
                  const float* target, float* W1, float* b1, float* W2, float* b2, float* W3,
                  float* b3, float lr, size_t steps, float* losses) {
  const size_t nh = batch * d_h, no = batch * d_out;
  V h1(nh), a1(nh), h2(nh), a2(nh), o(no);
  V gh1(nh), ga1(nh), gh2(nh), ga2(nh), go(no);
  V gW1(d_in * d_h), gb1(d_h), gW2(d_h * d_h), gb2(d_h), gW3(d_h * d_out), gb3(d_out);
  V d(no), q(no), gd(no), gq(no), gy(no), p(no), gp(no), lossv(batch);
  float s = 0.f, gs = 0.f, L = 0.f, c = 1.0f / (float)no, gc = 0.f;

  auto zero = [](V& v) { std::memset(v.data(), 0, v.size() * sizeof(float)); };

  for (size_t step = 0; step < steps; ++step) {
    // gradients_mut().zero_grad()
    zero(gh1); zero(ga1); zero(gh2); zero(ga2); zero(go);
    zero(gW1); zero(gb1); zero(gW2); zero(gb2); zero(gW3); zero(gb3);
    zero(gd); zero(gq); zero(gy); zero(gp);
    gs = 0.f; gc = 0.f;

    // forward
    orc_gemm(batch, d_h, d_in, x, W1, h1.data(), 0.f);
    orc_add_row(batch, d_h, h1.data(), b1, h1.data());
    orc_unary(RELU, 0, 0, nh, h1.data(), a1.data());
    orc_gemm(batch, d_h, d_h, a1.data(), W2, h2.data(), 0.f);
    orc_add_row(batch, d_h, h2.data(), b2, h2.data());
    orc_unary(RELU, 0, 0, nh, h2.data(), a2.data());
    orc_gemm(batch, d_out, d_h, a2.data(), W3, o.data(), 0.f);
    orc_add_row(batch, d_out, o.data(), b3, o.data());

    if (kind == 0) {
      orc_binary_ew(SUB, no, o.data(), target, d.data());
      orc_unary(SQUARE, 0, 0, no, d.data(), q.data());
      orc_sum_cols(no, no, q.data(), &s);
      orc_binary_ew(MUL, 1, &s, &c, &L);
      losses[step] = L;
      // backward(): seed 1, closures in reverse
      float gL = 1.0f;
      orc_binary_ew_grad(MUL, 1, &s, &c, &gs, &gc, &gL);
      orc_sum_cols_grad(no, no, gq.data(), &gs);
      orc_unary_grad(SQUARE, 0, no, d.data(), gd.data(), gq.data());
      orc_binary_ew_grad(SUB, no, o.data(), target, go.data(), gy.data(), gd.data());
    } else {
      orc_softmax(batch, d_out, o.data(), p.data());
      orc_cce(batch, d_out, p.data(), target, lossv.data());
      losses[step] = orc_mean(batch, lossv.data());
      orc_cce_grad(batch, d_out, p.data(), target, gp.data());   // backward_with(&grad)
      orc_softmax_grad(batch, d_out, go.data(), p.data(), gp.data(), 0.f);
    }

    // layer 3
    orc_add_row_mut_grad(batch, d_out, gb3.data(), go.data());
    orc_gemm_grad(batch, d_h, d_out, a2.data(), W3, ga2.data(), gW3.data(), go.data(), 0.f);
    // relu 2 (input buffer is h2 after the in-place bias add), layer 2
    orc_unary_grad(RELU, 0, nh, h2.data(), gh2.data(), ga2.data());
    orc_add_row_mut_grad(batch, d_h, gb2.data(), gh2.data());
    orc_gemm_grad(batch, d_h, d_h, a1.data(), W2, ga1.data(), gW2.data(), gh2.data(), 0.f);
    // relu 1, layer 1 (x does not require grad)
    orc_unary_grad(RELU, 0, nh, h1.data(), gh1.data(), ga1.data());
    orc_add_row_mut_grad(batch, d_h, gb1.data(), gh1.data());
    orc_gemm_grad(batch, d_in, d_h, x, W1, nullptr, gW1.data(), gh1.data(), 0.f);

    // sgd.step(lin_i.params())
    orc_sgd_step(d_in * d_h, W1, gW1.data(), lr); orc_sgd_step(d_h, b1, gb1.data(), lr);
    orc_sgd_step(d_h * d_h, W2, gW2.data(), lr);  orc_sgd_step(d_h, b2, gb2.data(), lr);
    orc_sgd_step(d_h * d_out, W3, gW3.data(), lr); orc_sgd_step(d_out, b3, gb3.data(), lr);
  }
  return 0;
}
