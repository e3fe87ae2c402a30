/* sliced_hip.h — C ABI of the MI355X (gfx950) backend for sliced's array-op hot path.
 *
 * These are the entry points a `HIP<Mods>` device in the reference's host language would bind
 * (one per method of the op traits under src/ops2/ of the reference, plus the runtime calls
 * its custos-style device layer needs).  Plain pointers and sizes only.
 *
 * Conventions
 *   - every function returns 0 on success, a SLHIP_E* code or a positive hipError_t otherwise;
 *     slhip_last_error_string() describes the last failure on the calling thread;
 *   - all matrices are f32, row-major, contiguous (len = rows * cols), as in the reference;
 *   - data pointers are DEVICE pointers; a context owns one in-order HIP stream and every op
 *     is asynchronous on it.  Only slhip_memcpy_h2d, slhip_memcpy_d2h, slhip_free, slhip_sync and
 *     slhip_event_elapsed_ms wait;
 *   - a context is used from one host thread at a time (the reference's devices are
 *     single-threaded, RefCell-style);
 *   - the library never allocates inside an op call: partial results of the two-stage
 *     reductions and of split-K GEMM live in a workspace that slhip_init allocates once;
 *   - no aliasing between inputs and outputs unless a comment allows it;
 *   - pointers need only the 4-byte alignment of a float: views at odd offsets into an
 *     allocation and rows of odd length stay on the vector paths.
 *
 * Naming trap kept from the reference: *_rows reduces OVER the rows (output length = cols),
 * *_cols reduces OVER the columns (output length = rows).
 */
#ifndef SLICED_HIP_H
#define SLICED_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct slhip_ctx slhip_ctx;
typedef struct slhip_event slhip_event;
typedef struct slhip_graph slhip_graph;

enum {
  SLHIP_OK = 0,
  SLHIP_EINVAL = -1,     /* null pointer, zero/overflowing dims, unknown op code */
  SLHIP_ENODEVICE = -2,  /* no HIP device / wrong architecture */
  SLHIP_EWORKSPACE = -3, /* request does not fit the context workspace */
  SLHIP_EALIAS = -4,     /* forbidden overlap of operands */
  SLHIP_ECAPTURE = -5    /* call not allowed while the context records a graph (or none is recording) */
};

/* BinaryElementWise op codes (reference: src/ops2/binary_ew/mod.rs:55-100). */
enum { SLHIP_ADD = 0, SLHIP_SUB = 1, SLHIP_MUL = 2, SLHIP_DIV = 3 };

/* apply_fn / add_unary_grad op codes (reference call sites: src/ops.rs:36-41 square,
 * :65-72 pow, :423 clip, :438 exp; src/matrix.rs:181-187 relu; examples/nn.rs:137 -ln,
 * :151 neg-div). p and q are the scalar parameters: pow exponent, clip bounds, scale factor. */
enum {
  SLHIP_SQUARE = 0,
  SLHIP_POW = 1,
  SLHIP_RELU = 2,
  SLHIP_EXP = 3,
  SLHIP_CLIP = 4,
  SLHIP_NEG_LN = 5,
  SLHIP_SCALE = 6,
  SLHIP_NEG_DIV = 7,
  SLHIP_TANH = 8,   /* src/matrix.rs:206-227: tanh x, gradient 1 - tanh(x)^2 */
  SLHIP_SIGMOID = 9 /* src/matrix.rs:231-258: 1/(1+exp(-x)), gradient exp(-x)/(1+exp(-x))^2 */
};

/* ---------------------------------------------------------------- runtime ----------
 * Replaces what the reference gets from custos' device layer (not in its tree): Alloc,
 * WriteBuf/Read, ClearBuf and the in-order queue (usage: src/ops2/gemm/cpu_stack.rs:35-43
 * retrieve + add_op; examples/sine_net.rs:124 device construction). */
int32_t slhip_init(int32_t device_ordinal, slhip_ctx** ctx);
/* Same, but ops run on a stream the caller owns (e.g. a framework's current stream). */
int32_t slhip_init_on_stream(int32_t device_ordinal, void* hip_stream, slhip_ctx** ctx);
int32_t slhip_destroy(slhip_ctx* ctx);
const char* slhip_last_error_string(void);
int32_t slhip_device_name(slhip_ctx* ctx, char* buf, size_t buflen);
int32_t slhip_stream(slhip_ctx* ctx, void** hip_stream);
size_t slhip_workspace_bytes(slhip_ctx* ctx);
/* The device address of the context's workspace (slhip_workspace_bytes long), where two-stage
 * reductions and split products keep their partial results between launches.  Its contents mean
 * nothing between calls; a caller may use it as scratch of its own while no op of this context is
 * in flight.  No counterpart in the reference, whose devices hand out scratch through retrieve(). */
int32_t slhip_workspace(slhip_ctx* ctx, void** dptr);

int32_t slhip_malloc(slhip_ctx* ctx, size_t bytes, void** dptr);
int32_t slhip_free(slhip_ctx* ctx, void* dptr);
int32_t slhip_memcpy_h2d(slhip_ctx* ctx, void* dst_dev, const void* src_host, size_t bytes);
int32_t slhip_memcpy_d2h(slhip_ctx* ctx, void* dst_host, const void* src_dev, size_t bytes); /* waits */
int32_t slhip_memcpy_d2d(slhip_ctx* ctx, void* dst_dev, const void* src_dev, size_t bytes);
int32_t slhip_memset(slhip_ctx* ctx, void* dptr, int32_t byte_value, size_t bytes);
int32_t slhip_fill(slhip_ctx* ctx, size_t n, float value, float* x);
int32_t slhip_sync(slhip_ctx* ctx);

/* HIP events on the context's stream, for timing kernels where they run. */
int32_t slhip_event_create(slhip_ctx* ctx, slhip_event** ev);
int32_t slhip_event_record(slhip_ctx* ctx, slhip_event* ev);
int32_t slhip_event_elapsed_ms(slhip_event* start, slhip_event* stop, float* ms); /* waits for stop */
int32_t slhip_event_destroy(slhip_event* ev);

/* Record once, replay many: between slhip_graph_begin and slhip_graph_end every op issued on
 * the context is recorded into a HIP graph instead of being run; slhip_graph_launch replays
 * the whole recording as one launch.  This is the device-side form of the reference's lazy
 * mode (`Autograd<Lazy<Base>>` + `dev.run()`, examples/sine_net.rs:178-220), where ops are
 * recorded on the first pass and re-run each epoch.  Pointers and sizes are baked into the
 * recording: every buffer it names must stay allocated until slhip_graph_destroy.  While
 * recording, the calls that wait or touch the allocator (slhip_malloc, slhip_free,
 * slhip_memcpy_h2d, slhip_memcpy_d2h, slhip_sync, slhip_event_record, slhip_memset with a
 * non-zero byte) return SLHIP_ECAPTURE and end nothing; the recording contains kernel nodes
 * only (device-to-device copies and zero fills are recorded as kernels, never as
 * memcpy/memset nodes). */
int32_t slhip_graph_begin(slhip_ctx* ctx);
int32_t slhip_graph_end(slhip_ctx* ctx, slhip_graph** graph);
int32_t slhip_graph_launch(slhip_ctx* ctx, slhip_graph* graph);
int32_t slhip_graph_node_count(slhip_graph* graph, size_t* nodes);
int32_t slhip_graph_destroy(slhip_graph* graph);

/* Seeded counter-based uniform fill: x[i] = lo + (hi-lo) * u(seed, tag, i), u a 24-bit
 * fraction from splitmix64((seed ^ (tag << 40)) + i).  Replaces RandOp::rand
 * (src/rawops/cpu/rand.rs:7-12), whose generator is unseeded. */
int32_t slhip_rand_uniform(slhip_ctx* ctx, uint64_t seed, uint64_t tag, float lo, float hi, size_t n,
                           float* x);

/* ---------------------------------------------------------------- GEMM -------------
 * C[m×n] = op(A)·op(B) + beta·C.  trans_a: A is stored k×m; trans_b: B is stored n×k.
 * Replaces GenericBlas::{gemm, gemmT, Tgemm} as called at src/ops2/gemm/cpu_stack.rs:39 and
 * src/ops2/gemm/grad/cpu_stack.rs:36,39:
 *     gemm (m,n,k,a,b,c) = slhip_sgemm(ctx,0,0,m,n,k,a,b,c,0)
 *     gemmT(m,n,k,a,b,c) = slhip_sgemm(ctx,0,1,m,n,k,a,b,c,0)
 *     Tgemm(m,n,k,a,b,c) = slhip_sgemm(ctx,1,0,m,n,k,a,b,c,0)
 * beta = 0 is `Set`, beta = 1 is `Assign` (src/assign_or_set.rs; src/ops2/gemm/opencl.rs:138-139).
 * C must not overlap A or B. */
int32_t slhip_sgemm(slhip_ctx* ctx, int32_t trans_a, int32_t trans_b, size_t m, size_t n, size_t k,
                    const float* a, const float* b, float* c, float beta);
/* C = beta·C + (op(A)·op(B)) ⊙ (pre >= 0), pre shaped like C: the input gradient of a Linear layer
 * and the ReLU gradient of the layer before it in one kernel, for tapes that chain them -
 * GemmGrad's lhs_grad (src/ops2/gemm/grad/cpu_stack.rs:36) followed by relu's grad closure
 * `x.grad += (x >= 0) * out.grad` (src/matrix.rs:169-190).  With beta = 1 and C the zeroed gradient
 * of `pre` the result has the bits of the two-op sequence.  C must not overlap A, B or pre. */
int32_t slhip_sgemm_relu_mask(slhip_ctx* ctx, int32_t trans_a, int32_t trans_b, size_t m, size_t n, size_t k,
                              const float* a, const float* b, const float* pre, float* c, float beta);
/* How the tiled kernel treats a tile grid that does not fill the chip's last round of
 * workgroups.  SLHIP_TAIL_AUTO (the default) lets a cost model choose between running it as it
 * is, splitting K for every tile, and spreading the k range of the last round's tiles evenly over
 * one more round of workgroups; SLHIP_TAIL_WHOLE never spreads, SLHIP_TAIL_SPREAD spreads
 * whenever the shape allows it.  All three give the same result up to summation order, and each
 * is deterministic.  A tuning and testing knob: no counterpart in the reference. */
enum { SLHIP_TAIL_AUTO = 0, SLHIP_TAIL_WHOLE = 1, SLHIP_TAIL_SPREAD = 2 };
int32_t slhip_gemm_tail_policy(slhip_ctx* ctx, int32_t policy);
/* The tile of C that one workgroup of the tiled kernel computes.  SLHIP_TILE_AUTO (the default)
 * chooses by a cost model (64 x 64, unsplit, for products of a few hundred such tiles and a
 * moderate K; 128 x 128 otherwise, on eight waves, two workgroups to a CU); the others force a
 * tile for every product that takes the tiled kernel (SLHIP_TILE_128X128: the four-wave form of
 * that tile; SLHIP_TILE_128X128_WIDE: the eight-wave form, which has no doubly transposed instance
 * and then falls back to four waves).  Same results up to the summation order of k splits; a tuning and
 * testing knob with no counterpart in the reference. */
enum { SLHIP_TILE_AUTO = 0, SLHIP_TILE_128X128 = 1, SLHIP_TILE_64X64 = 3, SLHIP_TILE_128X128_WIDE = 4 };
int32_t slhip_gemm_tile_policy(slhip_ctx* ctx, int32_t policy);
/* Writes into buf (len bytes, NUL-terminated) which kernel and plan the last product issued on this
 * context ran as: kernel template, tile, waves per workgroup, k splits.  For logs and benchmark
 * records; no counterpart in the reference. */
int32_t slhip_gemm_plan_describe(slhip_ctx* ctx, char* buf, size_t len);

/* Gemm::gemm (src/ops2/gemm/mod.rs:21-32), trait argument order (m, k, n). */
int32_t slhip_gemm(slhip_ctx* ctx, size_t m, size_t k, size_t n, const float* lhs, const float* rhs,
                   float* out);

/* GemmGrad::gemm_grad (src/ops2/gemm/grad.rs:15-29; CPU body src/ops2/gemm/grad/cpu_stack.rs:24-41):
 * lhs_grad[m×k] = out_grad·rhsᵀ, rhs_grad[k×n] = lhsᵀ·out_grad.  A NULL grad pointer means the
 * operand does not require a gradient and that product is skipped.  beta 0 = SET (CPU
 * behaviour), 1 = accumulate (OpenCL behaviour, src/ops2/gemm/grad/opencl.rs:20,33). */
int32_t slhip_gemm_grad(slhip_ctx* ctx, size_t m, size_t k, size_t n, const float* lhs, const float* rhs,
                        float* lhs_grad, float* rhs_grad, const float* out_grad, float beta);

/* Linear forward of the examples (examples/sine_net.rs:32-40: gemm + add_row_mut, optionally
 * followed by Matrix::relu, src/matrix.rs:169-190) in one kernel: out = relu?(x[m×k]·w[k×n] + bias[n]).
 * pre_act (may be NULL) receives the value before relu, which the relu gradient needs. */
int32_t slhip_linear_fwd(slhip_ctx* ctx, size_t m, size_t k, size_t n, const float* x, const float* w,
                         const float* bias, int32_t relu, float* pre_act, float* out);
/* The whole backward pass of that Linear layer, out_grad[m×n] given - the closures that gemm
 * (GemmGrad, src/ops2/gemm/grad/cpu_stack.rs:36,39) and add_row_mut (add_row_mut_grad,
 * src/ops2/row_op/grad/cpu.rs:42-50) leave on the tape, and optionally the ReLU closure of the layer
 * before (src/matrix.rs:169-190):
 *     x_grad[m×k]  = beta·x_grad + (out_grad·wᵀ) ⊙ (relu_pre >= 0)     (relu_pre NULL: no mask)
 *     w_grad[k×n]  = beta·w_grad + xᵀ·out_grad
 *     bias_grad[n] += Σ_r out_grad[r,·]
 * x_grad, w_grad and bias_grad may each be NULL (that result is skipped).  Layers of up to 2^25
 * flop whose operands stay below 2^18 elements run as ONE launch (such steps are bound by launch
 * latency); every other shape runs the same kernels as slhip_add_row_mut_grad, slhip_sgemm /
 * slhip_sgemm_relu_mask and slhip_sgemm called one after the other.  x_grad and w_grad have the bits
 * of those calls either way; bias_grad is summed in another order in the single launch.  No
 * gradient may overlap an input. */
int32_t slhip_linear_grad(slhip_ctx* ctx, size_t m, size_t k, size_t n, const float* x, const float* w, float* x_grad,
                          const float* relu_pre, float* w_grad, float* bias_grad, const float* out_grad, float beta);

/* ---------------------------------------------------------------- reductions -------
 * SumRows/SumCols (src/ops2/sum/mod.rs:19-25), MaxRows/MaxCols (src/ops2/max/mod.rs:20-26),
 * MeanRows/MeanCols/Mean (src/ops2/mean/mod.rs:15-45), Sum/Max scalars
 * (src/ops2/sum/cpu.rs:18-20, src/ops2/max/cpu.rs:23-25).  `out` is overwritten. */
int32_t slhip_sum_rows(slhip_ctx* ctx, size_t rows, size_t cols, const float* x, float* out /*cols*/);
int32_t slhip_sum_cols(slhip_ctx* ctx, size_t rows, size_t cols, const float* x, float* out /*rows*/);
int32_t slhip_max_rows(slhip_ctx* ctx, size_t rows, size_t cols, const float* x, float* out /*cols*/);
int32_t slhip_max_cols(slhip_ctx* ctx, size_t rows, size_t cols, const float* x, float* out /*rows*/);
int32_t slhip_mean_rows(slhip_ctx* ctx, size_t rows, size_t cols, const float* x, float* out /*cols*/);
int32_t slhip_mean_cols(slhip_ctx* ctx, size_t rows, size_t cols, const float* x, float* out /*rows*/);
/* slhip_sum_rows for callers that cannot allocate device memory, or may not have a library do it
 * on their behalf: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  It has no counterpart in the reference.  Same kernels, same result bits as
 * slhip_sum_rows; the partial sums of its streaming stages live in a file-scope device array of
 * 4 MiB that every GPU the library runs on holds until the process ends, instead of the context
 * workspace.  The call itself allocates and frees nothing.  Limit: cols <= 131072 (any number of
 * rows); wider matrices return SLHIP_EWORKSPACE.  All calls on one GPU share that GPU's array:
 * calls that overlap in time on one GPU (two contexts, two streams) race; calls on one context
 * are ordered by its stream.  The array needs no clearing between calls. */
int32_t slhip_sum_rows_static(slhip_ctx* ctx, size_t rows, size_t cols, const float* x, float* out /*cols*/);
int32_t slhip_sum(slhip_ctx* ctx, size_t len, const float* x, float* out_dev /*1*/);
int32_t slhip_max(slhip_ctx* ctx, size_t len, const float* x, float* out_dev /*1*/);
int32_t slhip_mean(slhip_ctx* ctx, size_t len, const float* x, float* out_dev /*1*/);

/* Backward traits (src/ops2/sum/grad.rs, src/ops2/max/grad.rs, src/ops2/mean/grad.rs); every
 * one accumulates into x_grad (`+=`), as the CPU bodies do.
 *   sum_rows_grad : x_grad[r,c] += out_grad[c]            (src/ops2/sum/grad/cpu.rs:41-48)
 *   sum_cols_grad : x_grad[r,c] += out_grad[r]            (:50-56)
 *   max_rows_grad : every r with x[r,c] == out[c] gets out_grad[c]   (src/ops2/max/grad/cpu.rs:40-55)
 *   max_cols_grad : only the FIRST c with x[r,c] == out[r] gets out_grad[r]   (:57-69)
 *   mean_rows_grad: x_grad[r,c] += (cols/len)·out_grad[c] (src/ops2/mean/grad/cpu.rs:43-54)
 *   mean_cols_grad: x_grad[r,c] += out_grad[r]/cols       (:56-63) */
int32_t slhip_sum_rows_grad(slhip_ctx* ctx, size_t rows, size_t cols, float* x_grad, const float* out_grad);
int32_t slhip_sum_cols_grad(slhip_ctx* ctx, size_t rows, size_t cols, float* x_grad, const float* out_grad);
int32_t slhip_max_rows_grad(slhip_ctx* ctx, size_t rows, size_t cols, const float* out, const float* x,
                            float* x_grad, const float* out_grad);
int32_t slhip_max_cols_grad(slhip_ctx* ctx, size_t rows, size_t cols, const float* out, const float* x,
                            float* x_grad, const float* out_grad);
int32_t slhip_mean_rows_grad(slhip_ctx* ctx, size_t rows, size_t cols, float* x_grad, const float* out_grad);
int32_t slhip_mean_cols_grad(slhip_ctx* ctx, size_t rows, size_t cols, float* x_grad, const float* out_grad);

/* ---------------------------------------------------------------- softmax ----------
 * Softmax::softmax(samples, features, x) (src/ops2/softmax/mod.rs:16-18; CPU body
 * src/ops2/softmax/cpu.rs:11-16 = max_cols, sub_cols, exp, sum_cols, div_cols) as ONE pass.
 * SoftmaxGrad::softmax_grad (src/ops2/softmax/grad.rs:15-24; CPU body
 * src/ops2/softmax/grad/cpu.rs:24-61 builds the Jacobian per sample): x_grad = s·(g − <s,g>),
 * beta 0 = SET (CPU behaviour), 1 = accumulate. out may alias x; x_grad may alias out_grad. */
int32_t slhip_softmax(slhip_ctx* ctx, size_t samples, size_t features, const float* x, float* out);
int32_t slhip_softmax_grad(slhip_ctx* ctx, size_t samples, size_t features, float* x_grad,
                           const float* out, const float* out_grad, float beta);

/* ---------------------------------------------------------------- transpose --------
 * Transpose::transpose(rows, cols, x) (src/ops2/transpose/mod.rs:17-21; slice_transpose
 * src/ops2/transpose/cpu.rs:10-25): out[c·rows + r] = x[r·cols + c].  beta 0 = `Set`, 1 = `Assign`
 * (+=, the OpenCL transpose_grad, src/ops2/transpose/grad/opencl.rs:21).  TranposeGrad is
 * slhip_transpose(ctx, cols, rows, out_grad, x_grad, beta) (src/ops.rs:210-217). */
int32_t slhip_transpose(slhip_ctx* ctx, size_t rows, size_t cols, const float* x, float* out, float beta);

/* ---------------------------------------------------------------- row op (bias) ----
 * RowOp::{add_row, add_row_mut} (src/ops2/row_op/mod.rs:17-47): out[r,c] = lhs[r,c] + rhs[c];
 * out == lhs is the in-place add_row_mut.
 * RowOpGrad::add_row_grad (src/ops2/row_op/grad/cpu.rs:54-64): lhs_grad is OVERWRITTEN with
 * out_grad (skipped when NULL or the same pointer), rhs_grad[c] += Σ_r out_grad[r,c].
 * RowOpGrad::add_row_mut_grad (:42-50): rhs_grad[c] += Σ_r out_grad[r,c]. */
int32_t slhip_add_row(slhip_ctx* ctx, size_t rows, size_t cols, const float* lhs, const float* rhs, float* out);
int32_t slhip_add_row_grad(slhip_ctx* ctx, size_t rows, size_t cols, float* lhs_grad, float* rhs_grad,
                           const float* out_grad);
int32_t slhip_add_row_mut_grad(slhip_ctx* ctx, size_t rows, size_t cols, float* rhs_grad, const float* out_grad);

/* RowOp::row_op with a named op (src/ops2/row_op/mod.rs:17-30, slice_row_op
 * src/ops2/row_op/cpu.rs:67-80): out[r,c] = f(lhs[r,c], rhs[c]), f = SLHIP_ADD..SLHIP_DIV, and
 * its gradients (slice_row_op_grad_lhs / _rhs, src/ops2/row_op/grad/cpu.rs:66-88):
 *     lhs_grad[r,c] += df/dlhs * out_grad[r,c]      rhs_grad[c] += sum_r df/drhs * out_grad[r,c]
 * ColOp::col_op (src/ops2/col_op/mod.rs:20-57, slice_col_op src/ops2/col_op/cpu.rs:40-50) is the
 * same with the vector indexed by the row: out[r,c] = f(lhs[r,c], rhs[r]); sub_cols = SLHIP_SUB,
 * div_cols = SLHIP_DIV; gradients as slice_col_op_grad_lhs / _rhs
 * (src/ops2/col_op/grad/cpu.rs:41-88).  Either gradient pointer may be NULL (skipped). */
int32_t slhip_row_op(slhip_ctx* ctx, int32_t op, size_t rows, size_t cols, const float* lhs, const float* rhs,
                     float* out);
int32_t slhip_row_op_grad(slhip_ctx* ctx, int32_t op, size_t rows, size_t cols, const float* lhs, const float* rhs,
                          float* lhs_grad, float* rhs_grad, const float* out_grad);
int32_t slhip_col_op(slhip_ctx* ctx, int32_t op, size_t rows, size_t cols, const float* lhs, const float* rhs,
                     float* out);
int32_t slhip_col_op_grad(slhip_ctx* ctx, int32_t op, size_t rows, size_t cols, const float* lhs, const float* rhs,
                          float* lhs_grad, float* rhs_grad, const float* out_grad);

/* ---------------------------------------------------------------- elementwise ------
 * BinaryElementWise::{add,sub,mul,div} (src/ops2/binary_ew/mod.rs:55-100) and
 * BinaryElementWiseGrad with the closures of BinaryOpsMayGrad (src/ops.rs:115-171;
 * slice_binary_grad src/ops2/binary_ew/grad/cpu_stack.rs:40-60): lg += dL·g, rg += dR·g.
 * A NULL lg or rg skips that side.  out may alias l or r. */
int32_t slhip_ew_binary(slhip_ctx* ctx, int32_t op, size_t n, const float* l, const float* r, float* out);
int32_t slhip_ew_binary_grad(slhip_ctx* ctx, int32_t op, size_t n, const float* l, const float* r, float* lg,
                             float* rg, const float* g);
/* apply_fn / add_unary_grad: out[i] = f(x[i]); x_grad[i] += f'(x[i])·out_grad[i]. out may alias x. */
int32_t slhip_ew_unary(slhip_ctx* ctx, int32_t op, float p, float q, size_t n, const float* x, float* out);
int32_t slhip_ew_unary_grad(slhip_ctx* ctx, int32_t op, float p, size_t n, const float* x, float* x_grad,
                            const float* out_grad);
/* The chain of the elementwise workload, ((a+b)*c − d) -> pow 2 -> square, fused into one pass
 * (same ops as examples/chained_perf.rs:86-90 chains: add, mul, sub, pow, square). */
int32_t slhip_ew_chain(slhip_ctx* ctx, size_t n, const float* a, const float* b, const float* c,
                       const float* d, float* out);

/* A chain of elementwise ops as ONE pass: what the tape's blanket wrappers (BinaryOpsMayGrad,
 * SquareMayGrad, PowMayGrad ..., src/ops.rs:20-187) produce when they are chained, e.g.
 * examples/chained_perf.rs:86-90 (square, add, mul, mul, add), with the intermediates kept in
 * registers.  A program has up to SLHIP_EW_MAX_OPS instructions over up to SLHIP_EW_MAX_INPUTS
 * input buffers of n floats.  Register j < 4 is input j; register 4 + i is the result of
 * instruction i; an instruction reads registers below its own; the program's result is that of
 * its last instruction.  op is a binary code (SLHIP_ADD .. SLHIP_DIV, reads src0 and src1) or
 * SLHIP_EW_UNARY | a unary code (reads src0; p and q as in slhip_ew_unary).  Results have the bits
 * of the same ops run one after the other through slhip_ew_binary / slhip_ew_unary.
 * slhip_ew_program_grad: input_grads[j] += d result / d input j * out_grad for every non-null
 * entry, the intermediates recomputed, every instruction's terms added in the order the
 * single-op gradient calls would add them (last instruction first, lhs before rhs).  An
 * instruction flagged SLHIP_EW_NOGRAD passes no gradient on (exp and clip have no gradient
 * function in the reference, src/ops.rs:394-408,419-425).  out may alias an input; the
 * gradients must be distinct buffers. */
enum { SLHIP_EW_MAX_INPUTS = 4, SLHIP_EW_MAX_OPS = 8 };
enum { SLHIP_EW_UNARY = 0x10 };  /* or-ed into slhip_ew_insn.op */
enum { SLHIP_EW_NOGRAD = 0x1 };  /* slhip_ew_insn.flags */
typedef struct slhip_ew_insn {
  uint8_t op, src0, src1, flags;
  float p, q;
} slhip_ew_insn;
int32_t slhip_ew_program(slhip_ctx* ctx, size_t n, size_t n_inputs, const float* const* inputs, size_t n_ops,
                         const slhip_ew_insn* prog, float* out);
int32_t slhip_ew_program_grad(slhip_ctx* ctx, size_t n, size_t n_inputs, const float* const* inputs,
                              float* const* input_grads, size_t n_ops, const slhip_ew_insn* prog,
                              const float* out_grad);

/* ---------------------------------------------------------------- training helpers -
 * Host loops of the examples that a device-resident training loop needs as kernels.
 *   sgd_step : p[i] -= g[i]·lr                       (examples/sine_net.rs:105-116)
 *   cce      : loss[r] = −ln Σ_c clip(p,1e-7,1−1e-7)·t (examples/nn.rs:124-138)
 *   cce_grad : grad = (−(t/p))/rows                  (examples/nn.rs:140-152)
 *   onehot   : out[r·classes + (size_t)cls[r]] = 1, rest 0 (src/ops2/onehot/cpu.rs:40-44) */
int32_t slhip_sgd_step(slhip_ctx* ctx, size_t n, float* p, const float* g, float lr);
/* The same update for `count` parameter tensors in one launch per 8 tensors (the examples call
 * the step once per layer, examples/sine_net.rs:157-159).  params, grads and lens are HOST
 * arrays of `count` device pointers / lengths. */
int32_t slhip_sgd_step_multi(slhip_ctx* ctx, size_t count, float* const* params, const float* const* grads,
                             const size_t* lens, float lr);
int32_t slhip_cce(slhip_ctx* ctx, size_t rows, size_t cols, const float* preds, const float* targets, float* loss);
int32_t slhip_cce_grad(slhip_ctx* ctx, size_t rows, size_t cols, const float* preds, const float* targets,
                       float* grad);
int32_t slhip_onehot(slhip_ctx* ctx, size_t n, size_t classes, const float* cls, float* out);

/* The ReLU mask of a fused Linear as one bit per element, packed 32 columns to a word, row-major
 * [m][ceil(n / 32)] (bit c % 32 of word c / 32 of a row = pre-activation >= 0).  The backward pass
 * of the reference needs the pre-activations only for that comparison (relu gradient
 * src/matrix.rs:190-199; examples/sine_net.rs:32-40 chains gemm -> add_row_mut -> relu), so the
 * pair below moves 1/32 of the bytes slhip_linear_fwd's pre_act and slhip_sgemm_relu_mask's pre do.
 * slhip_linear_fwd_bits : out = relu(x·w + bias), bits = (x·w + bias >= 0); bias may be NULL.
 * slhip_sgemm_relu_bits : c = beta*c + (op(a)·op(b)) * bit — what slhip_sgemm_relu_mask computes
 *   from the float pre-activations, same values.
 * slhip_relu_grad_bits  : x_grad += bit * out_grad, for a ReLU output that feeds something else
 *   than a fused Linear.
 * The two products run one workgroup per 128 x 128 tile of the result without splitting K. */
int32_t slhip_linear_fwd_bits(slhip_ctx* ctx, size_t m, size_t k, size_t n, const float* x, const float* w,
                              const float* bias, uint32_t* bits, float* out);
int32_t slhip_sgemm_relu_bits(slhip_ctx* ctx, int32_t trans_a, int32_t trans_b, size_t m, size_t n, size_t k,
                              const float* a, const float* b, const uint32_t* bits, float* c, float beta);
int32_t slhip_relu_grad_bits(slhip_ctx* ctx, size_t rows, size_t cols, const uint32_t* bits, float* x_grad,
                             const float* out_grad);

/* Fused losses of the two example loops; every reference op they stand for stays available.
 * slhip_mse: loss_dev[0] = (sum_i (x_i - y_i)^2) * (1/n) — the chain sub, squared, sum_cols over one
 *   row, mul by the constant 1/n (loss tape of examples/sine_net.rs:150-156 summed on the device).
 * slhip_mse_grad: x_grad_i += ((x_i - y_i) * 2) * ((1/n) * upstream_dev[0]) — what the chain's
 *   gradient functions (src/ops.rs:118-128, :595-611, :38-41, :137-147) produce for x.
 * slhip_softmax_cce: probs = softmax(logits) (may be NULL), loss_rows[r] = -ln sum_c
 *   clip(p, 1e-7, 1-1e-7) * t — Matrix::softmax (src/matrix.rs:368-378) + cce (examples/nn.rs:124-143).
 * slhip_softmax_cce_grad: logits_grad = beta*logits_grad + (p * sum_c t - t) * (upstream_dev[0] / rows):
 *   cce_grad (examples/nn.rs:145-152) pushed through softmax_grad (src/ops2/softmax/grad/cpu.rs:8-62)
 *   in closed form, for the loss mean_r loss_rows[r]. */
int32_t slhip_mse(slhip_ctx* ctx, size_t n, const float* x, const float* y, float* loss_dev /*1*/);
int32_t slhip_mse_grad(slhip_ctx* ctx, size_t n, const float* x, const float* y, float* x_grad,
                       const float* upstream_dev /*1*/);
int32_t slhip_softmax_cce(slhip_ctx* ctx, size_t rows, size_t cols, const float* logits, const float* targets,
                          float* probs, float* loss_rows /*rows*/);
int32_t slhip_softmax_cce_grad(slhip_ctx* ctx, size_t rows, size_t cols, const float* probs, const float* targets,
                               float* logits_grad, float beta, const float* upstream_dev /*1*/);
/* One whole training step of the sine-fit loop (examples/sine_net.rs:119-166) in two launches:
 * x[batch×d_in] → Linear(d_in,d_h) → ReLU → Linear(d_h,d_h) → ReLU → Linear(d_h,d_out) (Linear = gemm +
 * add_row_mut, :32-40; Matrix::relu, src/matrix.rs:169-190), loss_dev[0] = (Σ (out − target)²)·1/(batch·d_out)
 * (the loss tape sub, squared, sum, scale of :150-156), backward with seed one, and SGD
 * `value -= grad * lr` (:105-116) on all six parameter tensors in place.  grads (may be NULL) names
 * six device arrays W1,b1,W2,b2,W3,b3-shaped that receive the step's gradients (SET), for callers
 * that keep gradient buffers.  d_h ≤ 64, d_in ≤ 8 and d_out ≤ 8 (larger layers: the ops one by one);
 * the per-row intermediates live in the context workspace (272 floats per row).  Same values as the
 * op sequence up to rounding (fused multiply-adds, tree sums over the hidden units); every sum has
 * a fixed order, so a step is reproducible bit for bit. */
int32_t slhip_mlp3_mse_step(slhip_ctx* ctx, size_t batch, size_t d_in, size_t d_h, size_t d_out, const float* x,
                            const float* target, float* w1, float* b1, float* w2, float* b2, float* w3, float* b3,
                            float* const* grads, float lr, float* loss_dev /*1*/);
/* onehot_grad (src/ops2/onehot/grad/cpu.rs:3-12): cls_grad[r] += out_grad[r*classes + cls[r]]. */
int32_t slhip_onehot_grad(slhip_ctx* ctx, size_t n, size_t classes, const float* cls, float* cls_grad,
                          const float* out_grad);
/* diagflat (src/ops2/diagflat/cpu.rs:42-46): out[n×n] = diag(x), every other entry zero;
 * diagflat_grad (src/ops2/diagflat/grad/cpu.rs:34-38): x_grad[i] += out_grad[i*n + i]. */
int32_t slhip_diagflat(slhip_ctx* ctx, size_t n, const float* x, float* out);
int32_t slhip_diagflat_grad(slhip_ctx* ctx, size_t n, float* x_grad, const float* out_grad);

#ifdef __cplusplus
}
#endif
#endif /* SLICED_HIP_H */
