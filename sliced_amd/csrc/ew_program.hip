// Elementwise programs: a chain (tree, DAG) of up to 8 binary / unary elementwise ops over up to 4
// input buffers evaluated in ONE pass, and its gradient in one pass as well.  This is what the
// host tape launches where it finds elementwise ops chained through intermediates that nothing
// else reads: the intermediates never make the round trip through HBM (the chain
// ((a+b)*c-d) -> pow 2 -> square moves 20 B per element this way and 52 B op by op).
//
// The program is data, not code: a kernel argument of at most 8 instructions.  In the C ABI's
// form register j < 4 is input j and register 4 + i the result of instruction i.  Every lane of
// every wave runs the same program, so decoding it is scalar work: the op code selects a uniform
// branch, the cheap ops first.  What is NOT uniform-friendly is a register file in VGPRs: a
// register number that is only known at run time turns every operand fetch into a chain of
// selects or an indexed move per component (measured: 245 issue cycles per wave and instruction,
// 0.105 ms per instruction on 2^28 elements, whichever of the two the compiler picked).  So the
// register file lives in LDS, one float4 per lane and register, [register][lane]: a run-time
// register number is just part of the address, an operand fetch is one ds_read_b128, a result one
// ds_write_b128, consecutive lanes touch consecutive 16-byte slots (no bank conflicts) and no lane
// touches another lane's slots (no barriers).  One wave per block; 1 KiB of LDS per register, so
// the host renumbers the program onto as few registers as its liveness allows (an intermediate
// dies at its single reader) to keep many waves per CU in flight.
//
// Arithmetic is the unfused f32 arithmetic of the single-op kernels (elementwise.hip; this file
// is compiled with -ffp-contract=off too), instruction by instruction, so a fused chain gives the
// bits of the same ops run one by one.  The gradient pass recomputes the intermediates, seeds the
// result's adjoint with out_grad, walks the instructions backwards adding lhs term then rhs term
// (the order of slice_binary_grad, src/ops2/binary_ew/grad/cpu_stack.rs:55-58) and finally stores
// every input gradient - which started from its value in memory - once.
#include "common.hpp"

namespace slhip {

constexpr int EWP_IN = SLHIP_EW_MAX_INPUTS;   // 4
constexpr int EWP_OPS = SLHIP_EW_MAX_OPS;     // 8
constexpr int EWP_REGS = EWP_IN + EWP_OPS;    // registers of the C ABI's numbering

// An instruction as the kernels read it, 16 bytes = one scalar load: the ABI's fields, the register
// its result goes to and, for the gradient pass, where the adjoints of its result and operands
// live in the adjoint file (inputs in 0..3, intermediates renumbered by lifetime) and which of
// them nothing has written yet when the instruction's turn comes (ADJ_*: they count as zero and
// are not read).
struct __attribute__((aligned(16))) EwpInsn {
  uint8_t op, src0, src1, dst;
  uint8_t adj_dst, adj_s0, adj_s1, adj_flags;
  float p, q;
};
enum { ADJ_S0_FIRST = 1, ADJ_S1_FIRST = 2, ADJ_DST_UNSET = 4 };

struct EwProgArgs {
  const float* in[EWP_IN];
  float* grad[EWP_IN];  // gradient pass: gradient of input j, or null
  float* out;           // forward: the result
  const float* g;       // gradient pass: gradient of the result
  int n_in, n_ops;
  int n_regs;           // registers in use (the value file's size in LDS)
  unsigned nograd;      // bit i: instruction i passes no gradient on
  int n_adj;            // adjoint slots in use (gradient pass)
  int seed_slot;        // where out_grad goes; -1: the last instruction passes no gradient on
  EwpInsn insn[EWP_OPS];
};

__device__ __forceinline__ float ewp_pow(float x, float p) {  // as pow_ref of the single-op kernels
  if (p == 2.0f) return x * x;
  if (p == 1.0f) return x;
  // powf(-inf, 0.5) is +inf and powf(-0, 0.5) is +0 where the square root has NaN and -0
  if (p == 0.5f) return x == -__builtin_huge_valf() ? __builtin_huge_valf() : sqrtf(x) + 0.0f;
  return powf(x, p);
}

constexpr int U_ = SLHIP_EW_UNARY;

// W = 4: one float4 per lane; W = 1: one float (the tail elements).  slot(k) = this lane's copy of
// register k.
template <int W>
struct EwpLane {
  float* file;  // LDS, [register][64 lanes][4 floats]
  int lane;
  __device__ __forceinline__ float* slot(int k) const { return file + (k * 64 + lane) * 4; }
  __device__ __forceinline__ void get(int k, float (&v)[W]) const {
    if (W == 4) {
      const float4 t = ld4(slot(k));
      v[0] = t.x; v[1 % W] = t.y; v[2 % W] = t.z; v[3 % W] = t.w;
    } else {
      v[0] = *slot(k);
    }
  }
  __device__ __forceinline__ void put(int k, const float (&v)[W]) const {
    if (W == 4) st4(slot(k), make_float4(v[0], v[1 % W], v[2 % W], v[3 % W]));
    else *slot(k) = v[0];
  }
};

#define EWP_EACH(expr)                   \
  _Pragma("unroll") for (int c = 0; c < W; ++c) { expr; }
#define EWP_EACH_ROLLED(expr)            \
  _Pragma("unroll 1") for (int c = 0; c < W; ++c) { expr; }

// Runs the program; on return v holds the last instruction's result (which has no slot).
template <int W>
__device__ __forceinline__ void ewp_forward(const EwProgArgs& a, const EwpLane<W>& r, float (&v)[W]) {
  EwpInsn next = a.insn[0];
#pragma unroll 1
  for (int i = 0; i < a.n_ops; ++i) {
    const EwpInsn in = next;
    next = a.insn[i + 1 < a.n_ops ? i + 1 : i];  // in flight while this instruction runs
    const int op = in.op;
    float x[W];
    r.get(in.src0, x);
    if (!(op & U_)) {
      float y[W];
      r.get(in.src1, y);
      if (op == SLHIP_ADD) { EWP_EACH(v[c] = x[c] + y[c]) }
      else if (op == SLHIP_MUL) { EWP_EACH(v[c] = x[c] * y[c]) }
      else if (op == SLHIP_SUB) { EWP_EACH(v[c] = x[c] - y[c]) }
      else { EWP_EACH(v[c] = x[c] / y[c]) }
    } else if (op == (U_ | SLHIP_SQUARE) || (op == (U_ | SLHIP_POW) && in.p == 2.0f)) { EWP_EACH(v[c] = x[c] * x[c]) }
    else if (op == (U_ | SLHIP_RELU)) { EWP_EACH(v[c] = (x[c] >= 0.0f ? 1.0f : 0.0f) * x[c]) }
    else if (op == (U_ | SLHIP_SCALE)) { EWP_EACH(v[c] = x[c] * in.p) }
    else if (op == (U_ | SLHIP_CLIP)) { EWP_EACH(v[c] = fminf(fmaxf(x[c], in.p), in.q)) }
    else if (op == (U_ | SLHIP_NEG_DIV)) { EWP_EACH(v[c] = (-x[c]) / in.p) }
    // the long routines: rolled over the components, one copy of each in the kernel
    else if (op == (U_ | SLHIP_POW)) { EWP_EACH_ROLLED(v[c] = ewp_pow(x[c], in.p)) }
    else if (op == (U_ | SLHIP_EXP)) { EWP_EACH_ROLLED(v[c] = expf(x[c])) }
    else if (op == (U_ | SLHIP_TANH)) { EWP_EACH_ROLLED(v[c] = tanhf(x[c])) }
    else if (op == (U_ | SLHIP_SIGMOID)) { EWP_EACH_ROLLED(v[c] = 1.0f / (1.0f + expf(-x[c]))) }
    else { EWP_EACH_ROLLED(v[c] = -logf(x[c])) }  // SLHIP_NEG_LN
    if (i + 1 < a.n_ops) r.put(in.dst, v);  // the last result stays in v
  }
}

__device__ __forceinline__ float ewp_unary_d(int code, float x, float p) {
  switch (code) {
    case SLHIP_SQUARE: return x * 2.0f;
    case SLHIP_POW: return ewp_pow(x, p - 1.0f) * p;
    case SLHIP_RELU: return x >= 0.0f ? 1.0f : 0.0f;
    case SLHIP_EXP: return expf(x);
    case SLHIP_TANH: { const float t = tanhf(x); return 1.0f - t * t; }
    case SLHIP_SIGMOID: { const float e = expf(-x); const float s = 1.0f + e; return e / (s * s); }
    default: return p;  // SLHIP_SCALE
  }
}

// adj: the adjoint file (same shape as the value file); slots 0..3 hold the current input
// gradients (or zero) on entry and the updated ones on exit.  The adjoint of an intermediate
// starts from zero, as its zeroed gradient buffer does when the ops run one by one: the first term
// is added to 0.0f, not stored as it is.
template <int W>
__device__ __forceinline__ void ewp_backward(const EwProgArgs& a, const EwpLane<W>& r, const EwpLane<W>& adj,
                                             const float (&g)[W]) {
  if (a.seed_slot < 0) return;
  adj.put(a.seed_slot, g);
  EwpInsn next = a.insn[a.n_ops - 1];
#pragma unroll 1
  for (int i = a.n_ops - 1; i >= 0; --i) {  // last instruction first
    const EwpInsn in = next;
    next = a.insn[i > 0 ? i - 1 : 0];  // in flight while this instruction runs
    if ((a.nograd >> i) & 1u) continue;
    const int op = in.op, fl = in.adj_flags;
    float x[W], go[W], s0[W];
    r.get(in.src0, x);
    if (fl & ADJ_DST_UNSET) { EWP_EACH(go[c] = 0.0f) }
    else adj.get(in.adj_dst, go);
    if (fl & ADJ_S0_FIRST) { EWP_EACH(s0[c] = 0.0f) }
    else adj.get(in.adj_s0, s0);
    if (op & U_) {
      if (op == (U_ | SLHIP_SQUARE)) { EWP_EACH(s0[c] = s0[c] + (x[c] * 2.0f) * go[c]) }
      else if (op == (U_ | SLHIP_RELU)) { EWP_EACH(s0[c] = s0[c] + (x[c] >= 0.0f ? 1.0f : 0.0f) * go[c]) }
      else if (op == (U_ | SLHIP_SCALE)) { EWP_EACH(s0[c] = s0[c] + in.p * go[c]) }
      else { EWP_EACH_ROLLED(s0[c] = s0[c] + ewp_unary_d(op & 0xf, x[c], in.p) * go[c]) }
      adj.put(in.adj_s0, s0);
    } else {
      float y[W], tl[W], tr[W];
      r.get(in.src1, y);
      if (op == SLHIP_ADD) { EWP_EACH(tl[c] = 1.0f * go[c]; tr[c] = 1.0f * go[c]) }
      else if (op == SLHIP_SUB) { EWP_EACH(tl[c] = 1.0f * go[c]; tr[c] = -1.0f * go[c]) }
      else if (op == SLHIP_MUL) { EWP_EACH(tl[c] = y[c] * go[c]; tr[c] = x[c] * go[c]) }
      else { EWP_EACH(tl[c] = (1.0f / y[c]) * go[c]; tr[c] = (-x[c] / (y[c] * y[c])) * go[c]) }
      // lhs term first, then the rhs term (they may land in the same slot: x op x)
      EWP_EACH(s0[c] = s0[c] + tl[c])
      adj.put(in.adj_s0, s0);
      float s1[W];
      if (fl & ADJ_S1_FIRST) { EWP_EACH(s1[c] = 0.0f) }
      else adj.get(in.adj_s1, s1);
      EWP_EACH(s1[c] = s1[c] + tr[c])
      adj.put(in.adj_s1, s1);
    }
  }
}

// One float4 per lane, one wave per block, no loop: the launch shape of every streaming kernel
// here.  The first n % 4 lanes of the grid also take one tail element each.
// Dynamic LDS: n_regs KiB (forward) or (n_regs + n_adj) KiB (gradient).
template <bool GRAD>
__global__ __launch_bounds__(64) void ew_program_kernel(size_t n, EwProgArgs a) {
  extern __shared__ __attribute__((aligned(16))) float ewp_lds[];
  const size_t t = (size_t)blockIdx.x * 64 + threadIdx.x;
  const size_t n4 = n >> 2;
  const int lane = threadIdx.x;
  if (t < n4) {
    const EwpLane<4> r{ewp_lds, lane};
    const EwpLane<4> adj{ewp_lds + a.n_regs * 256, lane};
    float4 v[EWP_IN], gv[EWP_IN], gup;
#pragma unroll
    for (int j = 0; j < EWP_IN; ++j)
      if (j < a.n_in) v[j] = ld4s(a.in[j] + 4 * t);
    if (GRAD) {
      gup = ld4s(a.g + 4 * t);
#pragma unroll
      for (int j = 0; j < EWP_IN; ++j)
        if (j < a.n_in && a.grad[j]) gv[j] = ld4s(a.grad[j] + 4 * t);
    }
#pragma unroll
    for (int j = 0; j < EWP_IN; ++j)
      if (j < a.n_in) st4(r.slot(j), v[j]);
    float res[4];
    ewp_forward<4>(a, r, res);
    if (!GRAD) {
      st4s(a.out + 4 * t, make_float4(res[0], res[1], res[2], res[3]));
    } else {
#pragma unroll
      for (int j = 0; j < EWP_IN; ++j)
        if (j < a.n_in) st4(adj.slot(j), a.grad[j] ? gv[j] : make_float4(0.f, 0.f, 0.f, 0.f));
      const float g4[4] = {gup.x, gup.y, gup.z, gup.w};
      ewp_backward<4>(a, r, adj, g4);
#pragma unroll
      for (int j = 0; j < EWP_IN; ++j)
        if (j < a.n_in && a.grad[j]) st4s(a.grad[j] + 4 * t, ld4(adj.slot(j)));
    }
  }
  if (t >= (n & 3)) return;
  const size_t i = (n4 << 2) + t;
  const EwpLane<1> r{ewp_lds, lane};
  const EwpLane<1> adj{ewp_lds + a.n_regs * 256, lane};
  for (int j = 0; j < a.n_in; ++j) *r.slot(j) = a.in[j][i];
  float res[1];
  ewp_forward<1>(a, r, res);
  if (!GRAD) {
    a.out[i] = res[0];
  } else {
    for (int j = 0; j < a.n_in; ++j) *adj.slot(j) = a.grad[j] ? a.grad[j][i] : 0.0f;
    const float g1[1] = {a.g[i]};
    ewp_backward<1>(a, r, adj, g1);
    for (int j = 0; j < a.n_in; ++j)
      if (a.grad[j]) a.grad[j][i] = *adj.slot(j);
  }
}

static bool unary_has_grad(int op) {
  return op == SLHIP_SQUARE || op == SLHIP_POW || op == SLHIP_RELU || op == SLHIP_EXP || op == SLHIP_SCALE ||
         op == SLHIP_TANH || op == SLHIP_SIGMOID;
}

// Shared validation; fills `a` except for out / g / grad.
static int32_t ewp_prepare(const char* who, size_t n, size_t n_inputs, const float* const* inputs, size_t n_ops,
                           const slhip_ew_insn* prog, bool grad, EwProgArgs* a) {
  if (n == 0 || n_inputs == 0 || n_inputs > (size_t)EWP_IN || n_ops == 0 || n_ops > (size_t)EWP_OPS || !inputs || !prog) {
    set_error("%s: needs 1..%d inputs, 1..%d instructions and a non-empty buffer", who, EWP_IN, EWP_OPS);
    return SLHIP_EINVAL;
  }
  for (size_t j = 0; j < (size_t)EWP_IN; ++j) {
    a->in[j] = j < n_inputs ? inputs[j] : nullptr;
    a->grad[j] = nullptr;
    if (j < n_inputs && !inputs[j]) {
      set_error("%s: input %zu is null", who, j);
      return SLHIP_EINVAL;
    }
  }
  for (size_t i = 0; i < n_ops; ++i) {
    const slhip_ew_insn in = prog[i];
    const bool unary = (in.op & SLHIP_EW_UNARY) != 0;
    const int code = unary ? (in.op & 0xf) : in.op;
    const bool op_ok = unary ? code <= SLHIP_SIGMOID : code <= SLHIP_DIV;
    auto src_ok = [&](unsigned s) { return s < n_inputs || (s >= (unsigned)EWP_IN && s < (unsigned)EWP_IN + i); };
    if (!op_ok || (in.op & ~(SLHIP_EW_UNARY | 0xf)) || !src_ok(in.src0) || (!unary && !src_ok(in.src1))) {
      set_error("%s: instruction %zu is malformed (op %u, sources %u and %u)", who, i, (unsigned)in.op, (unsigned)in.src0,
                (unsigned)in.src1);
      return SLHIP_EINVAL;
    }
    if (grad && unary && !(in.flags & SLHIP_EW_NOGRAD) && !unary_has_grad(code)) {
      set_error("%s: instruction %zu: unary op %d has no gradient (flag it SLHIP_EW_NOGRAD)", who, i, code);
      return SLHIP_EINVAL;
    }
    a->insn[i] = EwpInsn{in.op, in.src0, unary ? in.src0 : in.src1, (uint8_t)(EWP_IN + i), 0, 0, 0, 0, in.p, in.q};
    if (in.flags & SLHIP_EW_NOGRAD) a->nograd |= 1u << i;
  }
  for (size_t i = n_ops; i < (size_t)EWP_OPS; ++i) a->insn[i] = EwpInsn{0, 0, 0, 0, 0, 0, 0, 0, 0.0f, 0.0f};
  a->n_in = (int)n_inputs;
  a->n_ops = (int)n_ops;
  a->n_regs = EWP_IN + (int)n_ops;
  return SLHIP_OK;
}

// Renumbers the values onto as few registers as their lifetimes allow: a value's register is free
// again after the last instruction that reads it (an input's too), and an instruction may write
// the register of an operand that dies there.  The last instruction's result stays in VGPRs and
// gets no register.  For the gradient pass (`grad`) a value that a backward step reads - the
// operands of mul and div, the operand of every unary op but scale - keeps its register to the
// end; what add, sub and scale read on the way back is not used, so it may be anything.
// Waves per CU follow from the KiB of LDS per wave: the gradient pass of ((a+b)*c-d) -> pow 2 ->
// square went from 15 KiB and 5.3 TB/s to 10 KiB; 5, 10 and 20 KiB more measured 4.5, 3.6, 2.6 TB/s.
static void ewp_pack_registers(EwProgArgs* a, bool grad) {
  int last_use[EWP_REGS];
  bool keep[EWP_REGS];
  for (int k = 0; k < EWP_REGS; ++k) {
    last_use[k] = -1;
    keep[k] = false;
  }
  for (int i = 0; i < a->n_ops; ++i) {
    const EwpInsn& in = a->insn[i];
    last_use[in.src0] = i;
    last_use[in.src1] = i;
    if (!grad || ((a->nograd >> i) & 1u)) continue;
    if (in.op & SLHIP_EW_UNARY) {
      if ((in.op & 0xf) != SLHIP_SCALE) keep[in.src0] = true;
    } else if (in.op == SLHIP_MUL || in.op == SLHIP_DIV) {
      keep[in.src0] = keep[in.src1] = true;
    }
  }
  int phys[EWP_REGS];
  bool busy[EWP_REGS];
  for (int k = 0; k < EWP_REGS; ++k) {
    phys[k] = k;
    busy[k] = k < a->n_in;  // the kernel puts input j into register j
  }
  int top = a->n_in;
  for (int i = 0; i < a->n_ops; ++i) {
    EwpInsn& in = a->insn[i];
    const int s0 = in.src0, s1 = in.src1;
    in.src0 = (uint8_t)phys[s0];
    in.src1 = (uint8_t)phys[s1];
    if (last_use[s0] == i && !keep[s0]) busy[phys[s0]] = false;
    if (last_use[s1] == i && !keep[s1]) busy[phys[s1]] = false;
    if (i + 1 == a->n_ops) {  // never stored
      in.dst = 0;
      break;
    }
    int d = 0;
    while (busy[d]) ++d;  // at most 4 inputs and 7 stored intermediates: one of 0..11 is free
    busy[d] = last_use[EWP_IN + i] >= 0;  // a result nobody reads does not hold its register
    phys[EWP_IN + i] = d;
    in.dst = (uint8_t)d;
    if (d + 1 > top) top = d + 1;
  }
  a->n_regs = top > 0 ? top : 1;
}

// Gradient pass: gives every intermediate's adjoint a slot for as long as it lives - from the
// backward step of the reader that comes last in the program (the first one the backward walk
// meets) to the intermediate's own step - and notes which adjoints a step finds untouched.
static void ewp_plan_adjoints(EwProgArgs* a) {
  int slot[EWP_REGS];
  bool touched[EWP_REGS], busy[EWP_REGS];
  for (int k = 0; k < EWP_REGS; ++k) {
    slot[k] = k < EWP_IN ? k : -1;
    touched[k] = k < EWP_IN;  // the inputs' slots hold their gradients from the start
    busy[k] = k < EWP_IN;
  }
  int top = EWP_IN;
  auto grab = [&](int reg) {
    if (slot[reg] >= 0) return;
    int d = EWP_IN;
    while (busy[d]) ++d;
    busy[d] = true;
    slot[reg] = d;
    if (d + 1 > top) top = d + 1;
  };
  const int last = EWP_IN + a->n_ops - 1;
  grab(last);
  touched[last] = true;  // seeded with out_grad
  a->seed_slot = ((a->nograd >> (a->n_ops - 1)) & 1u) ? -1 : slot[last];
  for (int i = a->n_ops - 1; i >= 0; --i) {
    const int dst = EWP_IN + i;
    const int s0 = a->insn[i].src0, s1 = a->insn[i].src1;  // (still the ABI's numbering)
    int fl = 0;
    if ((a->nograd >> i) & 1u) {
      if (slot[dst] >= EWP_IN) busy[slot[dst]] = false;
      continue;
    }
    if (!touched[dst]) fl |= ADJ_DST_UNSET;
    grab(dst);
    grab(s0);
    if (!touched[s0]) fl |= ADJ_S0_FIRST;
    touched[s0] = true;
    const bool unary = (a->insn[i].op & SLHIP_EW_UNARY) != 0;
    if (!unary) {
      grab(s1);
      if (!touched[s1]) fl |= ADJ_S1_FIRST;
      touched[s1] = true;
    }
    a->insn[i].adj_dst = (uint8_t)slot[dst];
    a->insn[i].adj_s0 = (uint8_t)slot[s0];
    a->insn[i].adj_s1 = (uint8_t)slot[unary ? s0 : s1];
    a->insn[i].adj_flags = (uint8_t)fl;
    busy[slot[dst]] = false;  // the result's adjoint has been passed on
  }
  a->n_adj = top;
}

static int32_t ewp_launch(slhip_ctx* ctx, size_t n, EwProgArgs a, bool grad) {
  const size_t threads = (n >> 2) > 3 ? (n >> 2) : 4;
  if (!grid_fits(threads, 64)) {
    set_error("elementwise program: %zu elements exceed one launch", n);
    return SLHIP_EINVAL;
  }
  const dim3 grid(ceil_div(threads, 64));
  if (grad) {
    ewp_plan_adjoints(&a);  // on the ABI's numbering, which the packing below replaces
    ewp_pack_registers(&a, true);
    const size_t lds = (size_t)(a.n_regs + a.n_adj) * 1024;
    hipLaunchKernelGGL(ew_program_kernel<true>, grid, dim3(64), lds, ctx->stream, n, a);
  } else {
    ewp_pack_registers(&a, false);
    hipLaunchKernelGGL(ew_program_kernel<false>, grid, dim3(64), (size_t)a.n_regs * 1024, ctx->stream, n, a);
  }
  return post_launch();
}

}  // namespace slhip

using namespace slhip;

SLHIP_API int32_t slhip_ew_program(slhip_ctx* ctx, size_t n, size_t n_inputs, const float* const* inputs, size_t n_ops,
                                   const slhip_ew_insn* prog, float* out) {
  SLHIP_REQUIRE(ctx && out, "null argument");
  EwProgArgs a{};
  int32_t rc = ewp_prepare("slhip_ew_program", n, n_inputs, inputs, n_ops, prog, false, &a);
  if (rc) return rc;
  a.out = out;
  a.g = nullptr;
  return ewp_launch(ctx, n, a, false);
}

SLHIP_API int32_t slhip_ew_program_grad(slhip_ctx* ctx, size_t n, size_t n_inputs, const float* const* inputs,
                                        float* const* input_grads, size_t n_ops, const slhip_ew_insn* prog,
                                        const float* out_grad) {
  SLHIP_REQUIRE(ctx && out_grad && input_grads, "null argument");
  EwProgArgs a{};
  int32_t rc = ewp_prepare("slhip_ew_program_grad", n, n_inputs, inputs, n_ops, prog, true, &a);
  if (rc) return rc;
  bool any = false;
  for (size_t j = 0; j < n_inputs; ++j) {
    a.grad[j] = input_grads[j];
    any = any || input_grads[j];
    for (size_t k = 0; k < j; ++k)
      if (input_grads[j] && input_grads[j] == input_grads[k]) {
        set_error("slhip_ew_program_grad: the gradients of inputs %zu and %zu alias", k, j);
        return SLHIP_EALIAS;
      }
  }
  if (!any) return SLHIP_OK;
  a.out = nullptr;
  a.g = out_grad;
  return ewp_launch(ctx, n, a, true);
}
