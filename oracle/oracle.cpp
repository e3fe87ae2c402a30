// CPU oracle for the sliced array-op hot path.
//
// THIS IS TEST INFRASTRUCTURE. It is a restatement, in plain C++, of the
// reference's CPU slice functions (Rust, `src/ops2/*/cpu*.rs`) and of the
// arithmetic they delegate to the absent `custos` crate (sgemm in three forms,
// apply_fn / add_unary_grad).  Only the test-suite, the smoke check and the
// CPU-baseline leg of the benchmark may load it; the shipped library never does.
//
// Faithfulness rules:
//   * every loop runs in the reference's element order; f32 arithmetic only,
//     compiled with -ffp-contract=off and without fast-math so nothing is fused
//     or reassociated (Rust never contracts a*b+c);
//   * OpenMP is used only across independent outputs (rows of a row-wise op,
//     column blocks of a column-wise op, rows of C in sgemm), so the threaded
//     result is bit-identical to the single-threaded one.  The whole-buffer
//     `sum`/`mean` stay strictly sequential.
//
// Pinning (which check nails which function) is listed next to each function:
//   GOLDEN  = literal vector transcribed from the reference's own tests
//   MATH    = closed form / invariant / brute force exercised by the tests
//   UNPINNED = nothing in the reference fixes it; stated explicitly.
//
// Parity unpinned (no reference test or fixture can distinguish the choice):
//   * orc_gemm_grad / orc_softmax_grad write with SET (BLAS beta = 0, inferred:
//     custos' GenericBlas is not in the tree and has no lock-file version);
//   * fmaxf semantics of `T::max` for NaN and signed zero;
//   * relu producing -0.0 for negative inputs (`geq(0) * x`);
//   * last-ulp behaviour of expf/powf/logf (platform libm behind Rust f32).
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <vector>
#include <algorithm>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API extern "C" __attribute__((visibility("default")))

static int g_threads = 1;

ORC_API void orc_set_threads(int n) {
  g_threads = n < 1 ? 1 : n;
#ifdef _OPENMP
  omp_set_num_threads(g_threads);
#endif
}
ORC_API int orc_get_threads() { return g_threads; }
ORC_API int orc_max_threads() {
#ifdef _OPENMP
  return omp_get_num_procs();
#else
  return 1;
#endif
}

// ---------------------------------------------------------------------------
// sum  (src/ops2/sum/cpu.rs, src/ops2/sum/grad/cpu.rs)
// ---------------------------------------------------------------------------

// `Sum::sum`  src/ops2/sum/cpu.rs:18-20 — `x.iter().copied().sum()`, sequential.
// MATH: sum of a constant, sum of integers (exact in f32).
ORC_API float orc_sum(size_t len, const float* x) {
  float acc = 0.0f;  // Iterator::sum::<f32> folds from 0.0 left to right
  for (size_t i = 0; i < len; ++i) acc += x[i];
  return acc;
}

// `slice_sum_rows`  src/ops2/sum/cpu.rs:66-76 — out[c] += x[r,c], r ascending.
// Accumulates into `out` (caller zeroes it, as custos `retrieve` does).
// GOLDEN: src/ops2/sum/cpu.rs:96-109 (via the identical slice_sum_rows2).
ORC_API void orc_sum_rows(size_t rows, size_t cols, const float* x, float* out) {
  const size_t CB = 1024;  // column blocks are independent outputs
#pragma omp parallel for schedule(static) if (cols >= 4 * CB && g_threads > 1)
  for (size_t c0 = 0; c0 < cols; c0 += CB) {
    size_t c1 = std::min(cols, c0 + CB);
    for (size_t r = 0; r < rows; ++r) {
      const float* row = x + r * cols;
      for (size_t c = c0; c < c1; ++c) out[c] += row[c];
    }
  }
}

// `slice_sum_rows2`  src/ops2/sum/cpu.rs:78-84 — same arithmetic, chunks(cols).
ORC_API void orc_sum_rows2(size_t cols, size_t len, const float* x, float* out) {
  orc_sum_rows(len / cols, cols, x, out);
}

// `slice_sum_cols`  src/ops2/sum/cpu.rs:86-90 — out[r] = sequential sum of row r.
// GOLDEN: src/ops2/sum/cpu.rs:110-123.
ORC_API void orc_sum_cols(size_t cols, size_t len, const float* x, float* out) {
  size_t rows = len / cols;
#pragma omp parallel for schedule(static) if (rows >= 64 && g_threads > 1)
  for (size_t r = 0; r < rows; ++r) {
    const float* row = x + r * cols;
    float acc = 0.0f;
    for (size_t c = 0; c < cols; ++c) acc += row[c];
    out[r] = acc;
  }
}

// `slice_sum_rows_grad`  src/ops2/sum/grad/cpu.rs:41-48 — x_grad[r,c] += out_grad[c].
// GOLDEN: src/ops2/sum/grad/cpu.rs:84-104.
ORC_API void orc_sum_rows_grad(size_t cols, size_t len, float* x_grad, const float* out_grad) {
  size_t rows = len / cols;
#pragma omp parallel for schedule(static) if (rows >= 64 && g_threads > 1)
  for (size_t r = 0; r < rows; ++r)
    for (size_t c = 0; c < cols; ++c) x_grad[r * cols + c] += out_grad[c];
}

// `slice_sum_cols_grad`  src/ops2/sum/grad/cpu.rs:50-56 — x_grad[r,c] += out_grad[r].
// GOLDEN: src/ops2/sum/grad/cpu.rs:62-82.
ORC_API void orc_sum_cols_grad(size_t cols, size_t len, float* x_grad, const float* out_grad) {
  size_t rows = len / cols;
#pragma omp parallel for schedule(static) if (rows >= 64 && g_threads > 1)
  for (size_t r = 0; r < rows; ++r)
    for (size_t c = 0; c < cols; ++c) x_grad[r * cols + c] += out_grad[r];
}

// ---------------------------------------------------------------------------
// max  (src/ops2/max/cpu.rs, src/ops2/max/grad/cpu.rs)
// ---------------------------------------------------------------------------

// `T::max` of custos' Number for f32 is taken to be f32::max == fmaxf (UNPINNED
// for NaN / signed zero; all reference vectors are finite, non-zero ties).
static inline float tmax(float a, float b) { return fmaxf(a, b); }

// `max`  src/ops2/max/cpu.rs:11-13 — reduce(T::max) left to right.
ORC_API float orc_max(size_t len, const float* x) {
  float m = x[0];
  for (size_t i = 1; i < len; ++i) m = tmax(m, x[i]);
  return m;
}

// `MaxRows::max_rows` + `max_rows`  src/ops2/max/cpu.rs:37-54 — out starts as row 0
// (`:41`), then out[c] = T::max(x[r,c], out[c]) for every row including row 0.
// GOLDEN: src/ops2/max/cpu.rs:86-108 (incl. the all-negative case).
ORC_API void orc_max_rows(size_t cols, size_t len, const float* x, float* out) {
  size_t rows = len / cols;
  const size_t CB = 1024;
#pragma omp parallel for schedule(static) if (cols >= 4 * CB && g_threads > 1)
  for (size_t c0 = 0; c0 < cols; c0 += CB) {
    size_t c1 = std::min(cols, c0 + CB);
    for (size_t c = c0; c < c1; ++c) out[c] = x[c];
    for (size_t r = 0; r < rows; ++r) {
      const float* row = x + r * cols;
      for (size_t c = c0; c < c1; ++c) out[c] = tmax(row[c], out[c]);
    }
  }
}

// `max_cols`  src/ops2/max/cpu.rs:76-80 — out[r] = reduce(T::max) over row r.
// GOLDEN: src/ops2/max/cpu.rs:110-120, tests/test_max_cols.rs:18.
ORC_API void orc_max_cols(size_t cols, size_t len, const float* x, float* out) {
  size_t rows = len / cols;
#pragma omp parallel for schedule(static) if (rows >= 64 && g_threads > 1)
  for (size_t r = 0; r < rows; ++r) out[r] = orc_max(cols, x + r * cols);
}

// `slice_max_rows_grad`  src/ops2/max/grad/cpu.rs:40-55 — EVERY row equal to the
// column max receives out_grad[c] (`+=`).
// GOLDEN: src/ops2/max/grad/cpu.rs:101-125, tests/test_max_rows.rs:26-33.
ORC_API void orc_max_rows_grad(size_t cols, size_t len, const float* out, const float* x,
                               float* x_grad, const float* out_grad) {
  size_t rows = len / cols;
#pragma omp parallel for schedule(static) if (rows >= 64 && g_threads > 1)
  for (size_t r = 0; r < rows; ++r)
    for (size_t c = 0; c < cols; ++c) {
      size_t i = r * cols + c;
      if (out[c] == x[i]) x_grad[i] += out_grad[c];
    }
}

// `slice_max_cols_grad`  src/ops2/max/grad/cpu.rs:57-69 — only the FIRST position
// equal to the row max receives out_grad[r] (`position`, `+=`).
// GOLDEN: src/ops2/max/grad/cpu.rs:75-99, tests/test_max_cols.rs:27-33.
// Returns -1 if some row holds no element equal to its max (the reference panics).
ORC_API int orc_max_cols_grad(size_t cols, size_t len, const float* out, const float* x,
                              float* x_grad, const float* out_grad) {
  size_t rows = len / cols;
  int bad = 0;
#pragma omp parallel for schedule(static) if (rows >= 64 && g_threads > 1)
  for (size_t r = 0; r < rows; ++r) {
    const float* row = x + r * cols;
    size_t pos = cols;
    for (size_t c = 0; c < cols; ++c)
      if (row[c] == out[r]) { pos = c; break; }
    if (pos == cols) { bad = 1; continue; }
    x_grad[r * cols + pos] += out_grad[r];
  }
  return bad ? -1 : 0;
}

// ---------------------------------------------------------------------------
// mean  (src/ops2/mean/cpu.rs, src/ops2/mean/grad/cpu.rs)
// ---------------------------------------------------------------------------

// `mean`  src/ops2/mean/cpu.rs:34-36 — sequential sum / T::from_usize(len).
// MATH: mean of a constant; equals orc_sum / len.
ORC_API float orc_mean(size_t len, const float* x) { return orc_sum(len, x) / (float)len; }

// `mean_rows`  src/ops2/mean/cpu.rs:38-43 — slice_sum_rows2 into out (caller zeroes),
// then out[c] /= rows.  GOLDEN: src/ops2/mean/cpu.rs:68-79.
ORC_API void orc_mean_rows(size_t cols, size_t len, const float* x, float* out) {
  orc_sum_rows2(cols, len, x, out);
  float d = (float)(len / cols);
  for (size_t c = 0; c < cols; ++c) out[c] /= d;
}

// `mean_cols`  src/ops2/mean/cpu.rs:45-49 — out[r] = (sequential row sum) / cols.
// GOLDEN: src/ops2/mean/cpu.rs:55-66.
ORC_API void orc_mean_cols(size_t cols, size_t len, const float* x, float* out) {
  orc_sum_cols(cols, len, x, out);
  size_t rows = len / cols;
  float d = (float)cols;
  for (size_t r = 0; r < rows; ++r) out[r] /= d;
}

// `mean_rows_grad`  src/ops2/mean/grad/cpu.rs:43-54 — x_grad[r,c] += (cols/len) * out_grad[c]
// with cols/len evaluated in T.  GOLDEN: src/ops2/mean/grad/cpu.rs:69-84, tests/test_mean.rs:26-31.
ORC_API void orc_mean_rows_grad(size_t cols, size_t len, float* x_grad, const float* out_grad) {
  size_t rows = len / cols;
  float f = (float)cols / (float)len;
  for (size_t r = 0; r < rows; ++r)
    for (size_t c = 0; c < cols; ++c) x_grad[r * cols + c] += f * out_grad[c];
}

// `mean_cols_grad`  src/ops2/mean/grad/cpu.rs:56-63 — x_grad[r,c] += out_grad[r] / cols.
// GOLDEN: src/ops2/mean/grad/cpu.rs:86-100.
ORC_API void orc_mean_cols_grad(size_t cols, size_t len, float* x_grad, const float* out_grad) {
  size_t rows = len / cols;
  for (size_t r = 0; r < rows; ++r) {
    float div = out_grad[r] / (float)cols;
    for (size_t c = 0; c < cols; ++c) x_grad[r * cols + c] += div;
  }
}

// ---------------------------------------------------------------------------
// row_op  (src/ops2/row_op/cpu.rs, src/ops2/row_op/grad/cpu.rs)
// ---------------------------------------------------------------------------

// `slice_row_op_mut` with `*out = lhs + rhs`  src/ops2/row_op/cpu.rs:81-90 (add_row), and
// `slice_row_op_lhs` with `*c += a`  :67-79 (add_row_mut) when out == lhs.
// GOLDEN: src/ops2/row_op/cpu.rs:103-115, tests/test_row_op.rs:22-26,61-65.
ORC_API void orc_add_row(size_t rows, size_t cols, const float* lhs, const float* rhs, float* out) {
#pragma omp parallel for schedule(static) if (rows >= 64 && g_threads > 1)
  for (size_t r = 0; r < rows; ++r)
    for (size_t c = 0; c < cols; ++c) out[r * cols + c] = lhs[r * cols + c] + rhs[c];
}

// `slice_add_row_op_grad`  src/ops2/row_op/grad/cpu.rs:54-64 — lhs_grad is OVERWRITTEN with
// out_grad (copy_from_slice), rhs_grad[c] += sum over rows (slice_sum_rows).
// GOLDEN: tests/test_row_op.rs:28-36.
ORC_API void orc_add_row_grad(size_t rows, size_t cols, float* lhs_grad, float* rhs_grad,
                              const float* out_grad) {
  if (lhs_grad != out_grad) std::memcpy(lhs_grad, out_grad, rows * cols * sizeof(float));
  orc_sum_rows(rows, cols, out_grad, rhs_grad);
}

// `add_row_mut_grad`  src/ops2/row_op/grad/cpu.rs:42-50 — rhs_grad[c] += Σ_r out_grad[r,c].
// GOLDEN: tests/test_row_op.rs:67-75.
ORC_API void orc_add_row_mut_grad(size_t rows, size_t cols, float* rhs_grad, const float* out_grad) {
  orc_sum_rows(rows, cols, out_grad, rhs_grad);
}

// `slice_row_op_grad_lhs/rhs` with the identity grad fn (a row-wise multiply)
// src/ops2/row_op/grad/cpu.rs:66-88.  GOLDEN: :94-111.
ORC_API void orc_mul_row_grad(size_t cols, size_t len, const float* lhs, const float* rhs,
                              float* lhs_grad, float* rhs_grad, const float* out_grad) {
  size_t rows = len / cols;
  for (size_t r = 0; r < rows; ++r)
    for (size_t c = 0; c < cols; ++c) lhs_grad[r * cols + c] += rhs[c] * out_grad[r * cols + c];
  for (size_t r = 0; r < rows; ++r)
    for (size_t c = 0; c < cols; ++c) rhs_grad[c] += lhs[r * cols + c] * out_grad[r * cols + c];
}

// ---------------------------------------------------------------------------
// col_op  (src/ops2/col_op/cpu.rs:40-50, src/ops2/col_op/mod.rs:33-57)
// op: 0 add, 1 sub, 2 mul, 3 div — out[r,c] = f(lhs[r,c], rhs[r]).
// GOLDEN: src/ops2/col_op/cpu.rs:56-72.
// ---------------------------------------------------------------------------
static inline float bin(int op, float a, float b) {
  switch (op) {
    case 0: return a + b;
    case 1: return a - b;
    case 2: return a * b;
    default: return a / b;
  }
}
ORC_API void orc_col_op(int op, size_t cols, size_t len, const float* lhs, const float* rhs, float* out) {
  size_t rows = len / cols;
#pragma omp parallel for schedule(static) if (rows >= 64 && g_threads > 1)
  for (size_t r = 0; r < rows; ++r)
    for (size_t c = 0; c < cols; ++c) out[r * cols + c] = bin(op, lhs[r * cols + c], rhs[r]);
}

// row_op / col_op gradients with a named op (src/ops2/row_op/grad/cpu.rs:66-88,
// src/ops2/col_op/grad/cpu.rs:41-88): lhs_grad += dL(lhs, rhs) * out_grad elementwise, the
// broadcast side accumulates dR(lhs, rhs) * out_grad over the other axis, one `+=` per element in
// row-major order.  dL / dR as the reference's tests write them: div -> 1/rhs and
// lhs / -(rhs*rhs) (src/ops2/col_op/grad/cpu.rs:115,146).
// GOLDEN: src/ops2/col_op/grad/cpu.rs:97-161; src/ops2/row_op/grad/cpu.rs:94-111 (mul).
static inline float bin_dl(int op, float l, float r) {
  switch (op) {
    case 0: case 1: return 1.0f;
    case 2: return r;
    default: return 1.0f / r;
  }
}
static inline float bin_dr(int op, float l, float r) {
  switch (op) {
    case 0: return 1.0f;
    case 1: return -1.0f;
    case 2: return l;
    default: return l / (-(r * r));
  }
}
// by_row_index = 1: col_op (rhs has one entry per row); 0: row_op (one entry per column).
ORC_API void orc_bcast_op_grad(int by_row_index, int op, size_t cols, size_t len, const float* lhs, const float* rhs,
                               float* lhs_grad, float* rhs_grad, const float* out_grad) {
  size_t rows = len / cols;
  if (lhs_grad)
    for (size_t r = 0; r < rows; ++r)
      for (size_t c = 0; c < cols; ++c) {
        const size_t i = r * cols + c;
        lhs_grad[i] += bin_dl(op, lhs[i], rhs[by_row_index ? r : c]) * out_grad[i];
      }
  if (rhs_grad)
    for (size_t r = 0; r < rows; ++r)
      for (size_t c = 0; c < cols; ++c) {
        const size_t i = r * cols + c, j = by_row_index ? r : c;
        rhs_grad[j] += bin_dr(op, lhs[i], rhs[j]) * out_grad[i];
      }
}
// row_op forward with a named op (src/ops2/row_op/cpu.rs:67-80)
ORC_API void orc_row_op(int op, size_t cols, size_t len, const float* lhs, const float* rhs, float* out) {
  size_t rows = len / cols;
  for (size_t r = 0; r < rows; ++r)
    for (size_t c = 0; c < cols; ++c) out[r * cols + c] = bin(op, lhs[r * cols + c], rhs[c]);
}

// ---------------------------------------------------------------------------
// binary_ew  (src/ops2/binary_ew/cpu_stack.rs:42-55, grad/cpu_stack.rs:40-88)
// ---------------------------------------------------------------------------

// `slice_binary_ew`: out[i] = f(l[i], r[i]).  GOLDEN: src/ops2/binary_ew/cpu_stack.rs:63-72,
// tests/test_{add,sub,mul}.rs:13.
ORC_API void orc_binary_ew(int op, size_t len, const float* l, const float* r, float* out) {
#pragma omp parallel for schedule(static) if (len >= (1u << 16) && g_threads > 1)
  for (size_t i = 0; i < len; ++i) out[i] = bin(op, l[i], r[i]);
}

// `slice_binary_grad` with the grad closures of BinaryOpsMayGrad (src/ops.rs:115-171):
// add (1, 1); sub (1, -1); mul (rhs, lhs); div (1/r, -l/r²) (div has no MayGrad wrapper in
// the reference; the quotient rule is supplied for completeness, MATH-pinned by finite
// differences).  Both sides always accumulate: g_l += dL * g ; g_r += dR * g.
// GOLDEN: tests/test_add.rs:19-23, test_sub.rs:19-23, test_mul.rs:19-23.
ORC_API void orc_binary_ew_grad(int op, size_t len, const float* l, const float* r, float* lg,
                                float* rg, const float* g) {
#pragma omp parallel for schedule(static) if (len >= (1u << 16) && g_threads > 1)
  for (size_t i = 0; i < len; ++i) {
    float dl, dr;
    switch (op) {
      case 0: dl = 1.0f; dr = 1.0f; break;
      case 1: dl = 1.0f; dr = -1.0f; break;
      case 2: dl = r[i]; dr = l[i]; break;
      default: dl = 1.0f / r[i]; dr = -l[i] / (r[i] * r[i]); break;
    }
    if (lg) lg[i] += dl * g[i];
    if (rg) rg[i] += dr * g[i];
  }
}

// `slice_add_ew_grad`  src/ops2/binary_ew/grad/cpu_stack.rs:80-88.
ORC_API void orc_add_ew_grad(size_t len, float* lg, float* rg, const float* g) {
  for (size_t i = 0; i < len; ++i) { lg[i] += g[i]; rg[i] += g[i]; }
}

// ---------------------------------------------------------------------------
// unary apply_fn / add_unary_grad (custos; call sites src/ops.rs:36-41,65-72,423,438,
// src/matrix.rs:181-187, examples/nn.rs:137,151).
//   op 0 square : x*x            grad 2x            (x.mul(T::two()))
//   op 1 pow    : powf(x,p)      grad powf(x,p-1)*p
//   op 2 relu   : (x>=0 ? 1:0)*x grad (x>=0 ? 1:0)
//   op 3 exp    : expf(x)        grad expf(x)
//   op 4 clip   : min(max(x,p),q) (no grad in the reference)
//   op 5 neg_ln : -(ln x)         (cce, examples/nn.rs:137; no grad)
//   op 6 scale  : x*p             (helper: -(v)/rows of cce_grad is op 7)
//   op 7 neg_div: (-x)/p          (examples/nn.rs:151)
//   op 8 tanh   : tanhf(x)        grad 1 - tanh(x)^2             (src/matrix.rs:206-227)
//   op 9 sigmoid: 1/(1+exp(-x))   grad exp(-x)/(1+exp(-x))^2     (src/matrix.rs:231-258)
// GOLDEN: tests/test_square.rs:12,19; tests/test_pow.rs:15,20; tests/matrix/relu.rs:12,20;
// tests/matrix/tanh.rs:12-31.  sigmoid has no vector in the reference: pinned by the closed form
// against an f64 evaluation and by a finite difference (tests/test_oracle_math.py).
// ---------------------------------------------------------------------------
static inline float un(int op, float x, float p, float q) {
  switch (op) {
    case 0: return x * x;
    case 1: return powf(x, p);
    case 2: return (x >= 0.0f ? 1.0f : 0.0f) * x;
    case 3: return expf(x);
    case 4: return fminf(fmaxf(x, p), q);
    case 5: return -logf(x);
    case 6: return x * p;
    case 8: return tanhf(x);
    case 9: return 1.0f / (1.0f + expf(-x));
    default: return (-x) / p;
  }
}
static inline float un_grad(int op, float x, float p) {
  switch (op) {
    case 0: return x * 2.0f;
    case 1: return powf(x, p - 1.0f) * p;
    case 2: return x >= 0.0f ? 1.0f : 0.0f;
    case 3: return expf(x);
    case 6: return p;
    case 8: { const float t = tanhf(x); return 1.0f - t * t; }
    case 9: { const float e = expf(-x); const float d = 1.0f + e; return e / (d * d); }
    default: return 0.0f;
  }
}
ORC_API void orc_unary(int op, float p, float q, size_t len, const float* x, float* out) {
#pragma omp parallel for schedule(static) if (len >= (1u << 16) && g_threads > 1)
  for (size_t i = 0; i < len; ++i) out[i] = un(op, x[i], p, q);
}
// x_grad[i] += f'(x[i]) * out_grad[i]
ORC_API void orc_unary_grad(int op, float p, size_t len, const float* x, float* x_grad,
                            const float* out_grad) {
#pragma omp parallel for schedule(static) if (len >= (1u << 16) && g_threads > 1)
  for (size_t i = 0; i < len; ++i) x_grad[i] += un_grad(op, x[i], p) * out_grad[i];
}

// ---------------------------------------------------------------------------
// transpose  (src/ops2/transpose/cpu.rs:10-25) — b[c*rows + r] = a[r*cols + c].
// The second, unconditional `b[idx] = row.clone()` (`:23`) makes the CPU function SET even
// when instantiated with `Assign`; `assign` = 1 restates the OpenCL `+=` behaviour instead.
// GOLDEN: src/ops2/transpose/cpu.rs:76-85, tests/test_transpose.rs:13.
// ---------------------------------------------------------------------------
ORC_API void orc_transpose(size_t rows, size_t cols, const float* a, float* b, int assign) {
  const size_t T = 32;
#pragma omp parallel for schedule(static) if (rows >= 4 * T && g_threads > 1)
  for (size_t r0 = 0; r0 < rows; r0 += T)
    for (size_t c0 = 0; c0 < cols; c0 += T)
      for (size_t r = r0; r < std::min(rows, r0 + T); ++r)
        for (size_t c = c0; c < std::min(cols, c0 + T); ++c) {
          if (assign) b[c * rows + r] += a[r * cols + c];
          else b[c * rows + r] = a[r * cols + c];
        }
}

// ---------------------------------------------------------------------------
// sgemm in the three GenericBlas forms (custos, absent; call sites
// src/ops2/gemm/cpu_stack.rs:39, src/ops2/gemm/grad/cpu_stack.rs:36,39; argument
// convention pinned by tests/test_trans_gemm.rs:27,32,62,66,96,101).
//   gemm (m,n,k,a,b,c): c[m×n]  = a[m×k] · b[k×n]
//   gemmT(m,n,k,a,b,c): c[m×n]  = a[m×k] · bᵀ,  b stored n×k
//   Tgemm(m,n,k,a,b,c): c[m×n]  = aᵀ · b,       a stored k×m
// Each c[i,j] is the f32 sum over k ascending of a[i,k]*b[k,j], products rounded to f32
// before the add.  The transposed forms materialise the transpose first, which is how the
// reference's own tests define them (Tgemm(a,b) == gemm(transpose(a), b), asserted exactly).
// beta = 0 overwrites c, beta = 1 accumulates into it (`Assign` of the OpenCL path).
// GOLDEN: tests/test_gemm.rs:28-31,38,41.  MATH: f64-accumulated triple loop below.
// ---------------------------------------------------------------------------
static void sgemm_nn(size_t m, size_t n, size_t k, const float* a, const float* b, float* c, float beta) {
  // Cache blocking only: for every (i,j) the k index still ascends monotonically, so the
  // rounding sequence is that of the plain triple loop.
  const size_t IB = 16, KB = 256, JB = 512;
#pragma omp parallel for schedule(dynamic, 1) if (m >= 2 * IB && g_threads > 1)
  for (size_t i0 = 0; i0 < m; i0 += IB) {
    size_t i1 = std::min(m, i0 + IB);
    std::vector<float> accv((i1 - i0) * n, 0.0f);
    for (size_t j0 = 0; j0 < n; j0 += JB) {
      size_t j1 = std::min(n, j0 + JB);
      for (size_t k0 = 0; k0 < k; k0 += KB) {
        size_t k1 = std::min(k, k0 + KB);
        for (size_t i = i0; i < i1; ++i) {
          float* acc = accv.data() + (i - i0) * n;
          for (size_t kk = k0; kk < k1; ++kk) {
            float av = a[i * k + kk];
            const float* brow = b + kk * n;
            for (size_t j = j0; j < j1; ++j) acc[j] += av * brow[j];
          }
        }
      }
    }
    for (size_t i = i0; i < i1; ++i) {
      const float* acc = accv.data() + (i - i0) * n;
      float* crow = c + i * n;
      if (beta == 0.0f) for (size_t j = 0; j < n; ++j) crow[j] = acc[j];
      else for (size_t j = 0; j < n; ++j) crow[j] = beta * crow[j] + acc[j];
    }
  }
}

ORC_API void orc_gemm(size_t m, size_t n, size_t k, const float* a, const float* b, float* c, float beta) {
  sgemm_nn(m, n, k, a, b, c, beta);
}
ORC_API void orc_gemmT(size_t m, size_t n, size_t k, const float* a, const float* b, float* c, float beta) {
  std::vector<float> bt(k * n);
  orc_transpose(n, k, b, bt.data(), 0);  // b is n×k -> bt is k×n
  sgemm_nn(m, n, k, a, bt.data(), c, beta);
}
ORC_API void orc_Tgemm(size_t m, size_t n, size_t k, const float* a, const float* b, float* c, float beta) {
  std::vector<float> at(k * m);
  orc_transpose(k, m, a, at.data(), 0);  // a is k×m -> at is m×k
  sgemm_nn(m, n, k, at.data(), b, c, beta);
}

// f64-accumulated truth for error budgeting: c64[i,j] = Σ_k (double)a·(double)b.
// ta/tb follow the BLAS meaning (operand stored transposed).
ORC_API void orc_gemm_f64(int ta, int tb, size_t m, size_t n, size_t k, const float* a, const float* b,
                          double* c) {
#pragma omp parallel for schedule(dynamic, 4) if (m >= 8 && g_threads > 1)
  for (size_t i = 0; i < m; ++i) {
    double* crow = c + i * n;
    for (size_t j = 0; j < n; ++j) crow[j] = 0.0;
    for (size_t kk = 0; kk < k; ++kk) {
      double av = ta ? a[kk * m + i] : a[i * k + kk];
      if (!tb) {
        const float* brow = b + kk * n;
        for (size_t j = 0; j < n; ++j) crow[j] += av * (double)brow[j];
      } else {
        for (size_t j = 0; j < n; ++j) crow[j] += av * (double)b[j * k + kk];
      }
    }
  }
}

// `GemmGrad::gemm_grad`  src/ops2/gemm/grad/cpu_stack.rs:24-41 with the trait's (m,k,n):
//   lhs[m×k], rhs[k×n], out_grad[m×n];
//   if lhs requires grad: lhs_grad = gemmT(m,k,n, out_grad, rhs)   (= G·rhsᵀ)
//   if rhs requires grad: rhs_grad = Tgemm(k,n,m, lhs, out_grad)   (= lhsᵀ·G)
// A null grad pointer stands for `requires_grad() == false`.  `beta` 0 = SET (CPU, inferred),
// 1 = accumulate (OpenCL `Assign`, src/ops2/gemm/grad/opencl.rs:20,33).
// GOLDEN: tests/test_gemm.rs:35-41 (zero-initialised grads, so beta is not distinguished).
ORC_API void orc_gemm_grad(size_t m, size_t k, size_t n, const float* lhs, const float* rhs,
                           float* lhs_grad, float* rhs_grad, const float* out_grad, float beta) {
  if (lhs_grad) orc_gemmT(m, k, n, out_grad, rhs, lhs_grad, beta);
  if (rhs_grad) orc_Tgemm(k, n, m, lhs, out_grad, rhs_grad, beta);
}

// ---------------------------------------------------------------------------
// softmax  (src/ops2/softmax/cpu.rs:11-16): max_cols -> sub_cols -> exp -> sum_cols -> div_cols,
// every stage materialised in f32 exactly as the five reference passes do.
// GOLDEN: src/ops2/softmax/cpu.rs:24-35.  MATH: rows sum to 1; shift invariance.
// ---------------------------------------------------------------------------
ORC_API void orc_softmax(size_t samples, size_t features, const float* x, float* out) {
#pragma omp parallel for schedule(static) if (samples >= 64 && g_threads > 1)
  for (size_t r = 0; r < samples; ++r) {
    const float* row = x + r * features;
    float* o = out + r * features;
    float m = orc_max(features, row);                              // max_cols
    for (size_t c = 0; c < features; ++c) o[c] = row[c] - m;       // sub_cols
    for (size_t c = 0; c < features; ++c) o[c] = expf(o[c]);       // exp
    float s = 0.0f;
    for (size_t c = 0; c < features; ++c) s += o[c];               // sum_cols (sequential)
    for (size_t c = 0; c < features; ++c) o[c] = o[c] / s;         // div_cols
  }
}

// `diagflat`  src/ops2/diagflat/cpu.rs:42-46.  GOLDEN: :54-77.
ORC_API void orc_diagflat(size_t n, const float* x, float* out) {
  for (size_t i = 0; i < n; ++i) out[n * i + i] = x[i];
}

// `SoftmaxGrad::softmax_grad`, literal form  src/ops2/softmax/grad/cpu.rs:24-61: per sample,
//   J = diagflat(s) - gemm(F,1,F, s, transpose(F,1,s))      (F×F)
//   x_grad_row = gemm(F,1,F, J, g)                          (SET: BLAS beta = 0, inferred)
// O(samples·F²); used on small inputs to pin the closed form below.
// GOLDEN: src/ops2/softmax/grad/cpu.rs:82-95; tests/matrix/softmax.rs:9-17.
ORC_API void orc_softmax_grad_jacobian(size_t samples, size_t features, float* x_grad,
                                       const float* out, const float* out_grad) {
  size_t F = features;
  std::vector<float> diag(F * F), outer(F * F), J(F * F);
  for (size_t r = 0; r < samples; ++r) {
    const float* s = out + r * F;
    const float* g = out_grad + r * F;
    std::fill(diag.begin(), diag.end(), 0.0f);
    orc_diagflat(F, s, diag.data());
    sgemm_nn(F, F, 1, s, s, outer.data(), 0.0f);  // s[F×1] · sᵀ[1×F]
    for (size_t i = 0; i < F * F; ++i) J[i] = diag[i] - outer[i];
    sgemm_nn(F, 1, F, J.data(), g, x_grad + r * F, 0.0f);
  }
}

// Closed form of the same product: x_grad[r,c] = s·(g − <s,g>), <s,g> summed in f32 left to
// right.  MATH: equals the Jacobian form up to rounding (tested on small F); a constant
// upstream gradient gives 0.  beta 0 = SET, 1 = accumulate.
ORC_API void orc_softmax_grad(size_t samples, size_t features, float* x_grad, const float* out,
                              const float* out_grad, float beta) {
#pragma omp parallel for schedule(static) if (samples >= 64 && g_threads > 1)
  for (size_t r = 0; r < samples; ++r) {
    const float* s = out + r * features;
    const float* g = out_grad + r * features;
    float* xg = x_grad + r * features;
    float dot = 0.0f;
    for (size_t c = 0; c < features; ++c) dot += s[c] * g[c];
    for (size_t c = 0; c < features; ++c) {
      float v = s[c] * (g[c] - dot);
      xg[c] = beta == 0.0f ? v : beta * xg[c] + v;
    }
  }
}

// ---------------------------------------------------------------------------
// onehot  (src/ops2/onehot/cpu.rs:40-44) — onehot[row*hc + class] = 1.
// GOLDEN: src/ops2/onehot/cpu.rs:52-73 and the doc-test :26-37.
// ---------------------------------------------------------------------------
ORC_API void orc_onehot(size_t highest_class, size_t n, const float* classes, float* onehot) {
  for (size_t r = 0; r < n; ++r) onehot[r * highest_class + (size_t)classes[r]] = 1.0f;
}
// onehot_grad  src/ops2/onehot/grad/cpu.rs:3-12.  GOLDEN: :18-38.
ORC_API void orc_onehot_grad(size_t highest_class, size_t n, const float* classes, float* classes_grad,
                             const float* out_grad) {
  for (size_t r = 0; r < n; ++r) classes_grad[r] += out_grad[r * highest_class + (size_t)classes[r]];
}
// diagflat_grad  src/ops2/diagflat/grad/cpu.rs:34-38.  GOLDEN: :44-60.
ORC_API void orc_diagflat_grad(size_t n, float* x_grad, const float* out_grad) {
  for (size_t i = 0; i < n; ++i) x_grad[i] += out_grad[n * i + i];
}

// ---------------------------------------------------------------------------
// Loss helpers of the classifier example (examples/nn.rs:124-152), off the tape.
//   cce      : loss[r] = -ln( Σ_c clip(p[r,c], 1e-7, 1-1e-7) * t[r,c] )
//   cce_grad : grad[r,c] = (-(t[r,c] / p[r,c])) / rows        (unclipped p, as written)
// MATH: for a one-hot t the loss is -ln p[target].
// ---------------------------------------------------------------------------
ORC_API void orc_cce(size_t rows, size_t cols, const float* preds, const float* targets, float* loss) {
  const float lo = (float)1e-7, hi = (float)(1.0 - 1e-7);
  for (size_t r = 0; r < rows; ++r) {
    float s = 0.0f;
    for (size_t c = 0; c < cols; ++c) s += fminf(fmaxf(preds[r * cols + c], lo), hi) * targets[r * cols + c];
    loss[r] = -logf(s);
  }
}
ORC_API void orc_cce_grad(size_t rows, size_t cols, const float* preds, const float* targets, float* grad) {
  float fr = (float)rows;
  for (size_t i = 0; i < rows * cols; ++i) grad[i] = (-(targets[i] / preds[i])) / fr;
}

// SGD step of the examples (examples/sine_net.rs:105-116): value -= grad * lr.
ORC_API void orc_sgd_step(size_t n, float* p, const float* g, float lr) {
  for (size_t i = 0; i < n; ++i) p[i] -= g[i] * lr;
}
