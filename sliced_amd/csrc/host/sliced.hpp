// Host-side device layer above the C ABI: the part of the reference's `custos` device model that
// its array-op path relies on, re-stated for a HIP device.
//
//   HIP            device: one slhip context (one in-order stream), the buffer registry, the
//                  gradient map, the autograd tape and the call-position cache
//                  (reference usage: `CPU::<Autograd<Cached<Base>>>::new()`, examples/sine_net.rs:124)
//   Buffer         {id, device pointer, len, requires_grad}; copies share the allocation
//   Matrix         {Buffer, rows, cols} with one method per op (reference: src/matrix.rs:21-25,98-378)
//
// Semantics taken from how the reference uses custos (the crate itself is not in its tree):
//   * retrieve(len) hands out a ZEROED buffer (slice_sum_rows2 accumulates into it,
//     src/ops2/sum/cpu.rs:78-84); in cached mode the same call position of the next
//     `range` iteration gets the same allocation again (examples/sine_net.rs:135);
//   * every forward op pushes a closure on the tape (`add_grad_fn`, src/ops.rs:38 ...); the
//     closure looks gradients up by buffer id: grad() reads, grad_mut() creates zeroed;
//   * backward() seeds the output gradient with ones (tests/test_add.rs:17-23) and runs the
//     closures in reverse; backward_with(g) seeds with g (examples/nn.rs:233); the tape is
//     cleared afterwards;
//   * every gradient accumulates (`+=`) except gemm_grad, softmax_grad, transpose_grad and the
//     lhs side of add_row_grad, which overwrite, as the reference's CPU device does
//     (src/ops2/gemm/grad/cpu_stack.rs:36-39, src/ops2/softmax/grad/cpu.rs:53-60,
//     src/ops2/transpose/cpu.rs:22-23, src/ops2/row_op/grad/cpu.rs:61).
//
// Nothing here computes: every op is one call into libsliced_hip.so.
#pragma once
#include <cstdint>
#include <cstdio>
#include <algorithm>
#include <functional>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "sliced_hip.h"

namespace sliced {

struct Error : std::runtime_error {
  using std::runtime_error::runtime_error;
};

inline void check(int32_t rc, const char* what) {
  if (rc != 0) throw Error(std::string(what) + " failed (" + std::to_string(rc) + "): " + slhip_last_error_string());
}

class HIP;

// A recorded op sequence (see HIP::record): run() replays it as one launch.
class HIP;
class Graph {
 public:
  Graph() = default;
  Graph(HIP* dev, slhip_ctx* ctx, slhip_graph* g, std::vector<uint64_t> seeds)
      : dev_(dev), ctx_(ctx), g_(g), seeds_(std::move(seeds)) {}
  Graph(Graph&& o) noexcept : dev_(o.dev_), ctx_(o.ctx_), g_(o.g_), seeds_(std::move(o.seeds_)) { o.g_ = nullptr; }
  Graph& operator=(Graph&& o) noexcept {
    if (this != &o) {
      slhip_graph_destroy(g_);
      dev_ = o.dev_; ctx_ = o.ctx_; g_ = o.g_; seeds_ = std::move(o.seeds_);
      o.g_ = nullptr;
    }
    return *this;
  }
  Graph(const Graph&) = delete;
  Graph& operator=(const Graph&) = delete;
  ~Graph() { slhip_graph_destroy(g_); }
  bool valid() const { return g_ != nullptr; }
  inline void run() const;
  size_t nodes() const {
    size_t n = 0;
    check(slhip_graph_node_count(g_, &n), "slhip_graph_node_count");
    return n;
  }

 private:
  HIP* dev_ = nullptr;
  slhip_ctx* ctx_ = nullptr;
  slhip_graph* g_ = nullptr;
  std::vector<uint64_t> seeds_;  // seed gradients whose fill with ones backward() left out of the recording
};

struct Buffer {
  HIP* dev = nullptr;
  uint64_t id = 0;
  float* ptr = nullptr;
  size_t len = 0;
  bool requires_grad = true;  // custos buffers take part in autograd unless `no_grad()` was called
  bool pooled = false;        // lives in the gradient pool, not in an allocation of its own

  bool valid() const { return ptr != nullptr; }
  inline std::vector<float> read() const;
  inline void write(const float* host, size_t n) const;
  inline Buffer grad() const;  // throws if no gradient was ever written for this buffer
  inline void backward() const;
  inline void backward_with(const Buffer& g) const;
};

// How gemm_grad / softmax_grad / transpose_grad write: 0 = overwrite (the reference's CPU
// device), 1 = accumulate (its OpenCL device, src/ops2/gemm/grad/opencl.rs:20,33).
struct GradPolicy {
  float gemm_beta = 0.0f;
  float softmax_beta = 0.0f;
  float transpose_beta = 0.0f;
  // A fused Linear whose input is the ReLU output of another fused Linear writes its input gradient
  // already multiplied by that ReLU's gradient, (g·Wᵀ) ⊙ (pre >= 0), straight into pre's gradient:
  // one kernel instead of GEMM + elementwise pass, equal values (a zero may change its sign).  Off by
  // default: it is only the sequence the tape would run when that ReLU output feeds nothing else.
  bool fuse_relu_grad = false;
  // With fuse_relu_grad: a fused Linear + ReLU whose output has 2^22 elements or more keeps the
  // ReLU mask as one bit per element (slhip_linear_fwd_bits) instead of the pre-activations, and
  // the consumer's input-gradient GEMM reads those bits (slhip_sgemm_relu_bits): 1/32 of the bytes
  // both ways, equal values.  The pre-activation buffer then only names the gradient.
  bool relu_bits = false;
  // Elementwise ops (binary, unary) are not launched when they are issued but when something
  // needs their result; by then the tape knows which intermediates of a chain nothing else reads
  // and launches each such chain as ONE kernel (slhip_ew_program), its backward as one kernel too
  // (slhip_ew_program_grad, which recomputes the intermediates) - the device-side form of what the
  // reference's lazy devices do with an op queue (`Autograd<Lazy<Base>>`, examples/sine_net.rs:178).
  // Values and leaf gradients have the bits of the op-by-op sequence.  What differs: the gradient
  // BUFFER of an intermediate that was fused away is never written (reading it throws), and an
  // intermediate that is read later is computed then, from what its inputs hold at that time.
  // Off by default, like every other departure from the reference's eager CPU device.
  bool fuse_elementwise = false;
};

class HIP {
 public:
  GradPolicy policy;

  explicit HIP(int ordinal = 0, bool cached = true) : cached_(cached) { check(slhip_init(ordinal, &ctx_), "slhip_init"); }
  ~HIP() {
    for (auto& kv : allocs_)
      if (!kv.second.pooled) slhip_free(ctx_, kv.second.ptr);
    for (auto& sl : slabs_) slhip_free(ctx_, sl.base);
    slhip_destroy(ctx_);
  }
  HIP(const HIP&) = delete;
  HIP& operator=(const HIP&) = delete;

  slhip_ctx* ctx() const { return ctx_; }
  void sync() {
    run();
    check(slhip_sync(ctx_), "slhip_sync");
  }

  // ---- buffers ---------------------------------------------------------------------------
  Buffer alloc(size_t len, bool zero = true) {
    if (len == 0) throw Error("zero-length buffer");
    Buffer b;
    b.dev = this;
    b.id = next_id_++;
    b.len = len;
    check(slhip_malloc(ctx_, len * sizeof(float), (void**)&b.ptr), "slhip_malloc");
    if (zero) check(slhip_memset(ctx_, b.ptr, 0, len * sizeof(float)), "slhip_memset");
    allocs_[b.id] = b;
    return b;
  }
  Buffer from(const float* host, size_t len) {
    Buffer b = alloc(len, false);
    check(slhip_memcpy_h2d(ctx_, b.ptr, host, len * sizeof(float)), "slhip_memcpy_h2d");
    return b;
  }
  Buffer from(const std::vector<float>& v) { return from(v.data(), v.size()); }
  Buffer lookup(uint64_t id) const {
    auto it = allocs_.find(id);
    if (it == allocs_.end()) throw Error("unknown buffer id " + std::to_string(id));
    return it->second;
  }
  void set_requires_grad(uint64_t id, bool v) {
    auto it = allocs_.find(id);
    if (it == allocs_.end()) throw Error("unknown buffer id");
    it->second.requires_grad = v;
  }
  void release(uint64_t id) {
    if (pending_.count(id) || !pending_order_.empty()) run();
    // intermediates that a fused chain kept in registers and that are computed from this buffer
    // get their values now, while it still holds what they were computed from
    if (!virtual_.empty()) {
      std::vector<uint64_t> readers;
      for (auto& kv : virtual_)
        if (kv.second.a == id || (!kv.second.unary && kv.second.b == id)) readers.push_back(kv.first);
      for (uint64_t r : readers) materialise(r);
    }
    virtual_.erase(id);
    auto it = allocs_.find(id);
    if (it == allocs_.end()) return;
    if (!it->second.pooled) check(slhip_free(ctx_, it->second.ptr), "slhip_free");  // pool memory stays with the pool
    allocs_.erase(it);
    auto g = grads_.find(id);
    if (g != grads_.end()) {  // the gradient lives and dies with its buffer
      const uint64_t gid = g->second.id;
      grads_.erase(g);
      stale_.erase(gid);
      ones_.erase(gid);
      lazy_.erase(gid);
      release(gid);
    }
  }

  // Output buffer of an op.  Cached mode: position `cursor_` of this iteration; the buffer is
  // zeroed only when the op accumulates into it (`zero`), every other op overwrites all of it.
  Buffer retrieve(size_t len, bool zero = false) {
    if (!cached_) return alloc(len, zero);
    if (cursor_ < cache_.size() && cache_[cursor_].len == len) {
      Buffer b = cache_[cursor_++];
      if (pending_.count(b.id)) run();  // last iteration's deferred op into this very buffer
      virtual_.erase(b.id);             // whatever it stood for, the op at hand overwrites it
      if (zero) check(slhip_memset(ctx_, b.ptr, 0, len * sizeof(float)), "slhip_memset");
      return b;
    }
    // first iteration, or the op sequence changed: (re)build the cache from here on
    for (size_t i = cursor_; i < cache_.size(); ++i) release(cache_[i].id);
    cache_.resize(cursor_);
    Buffer b = alloc(len, zero);
    cache_.push_back(b);
    ++cursor_;
    return b;
  }

  // `for epoch in device.range(0..n)`: every iteration starts at cache position 0.
  struct Range {
    HIP* dev;
    size_t n;
    struct It {
      HIP* dev;
      size_t i;
      size_t operator*() const { return i; }
      bool operator!=(const It& o) const { return i != o.i; }
      // what one iteration deferred runs before the next hands the same buffers out again
      It& operator++() { ++i; dev->run(); dev->cursor_ = 0; return *this; }
    };
    It begin() { dev->run(); dev->cursor_ = 0; return {dev, 0}; }
    It end() { return {dev, n}; }
  };
  Range range(size_t n) { return Range{this, n}; }

  // Record once, replay many — the reference's lazy device (`Autograd<Lazy<Base>>`, `dev.run()`,
  // examples/sine_net.rs:178-220) as a HIP graph.  body() issues ops as usual (forward, backward,
  // optimiser step); none of them runs, all of them land in the returned Graph.  body() must not
  // allocate or read back: run the same sequence eagerly once before, so that the cache and the
  // gradient map already hold every buffer it names, and keep those buffers alive while the
  // Graph is in use.
  template <class F>
  Graph record(F&& body) {
    run();  // what was deferred before the recording belongs before it
    check(slhip_graph_begin(ctx_), "slhip_graph_begin");
    slhip_graph* g = nullptr;
    recording_ = true;
    recorded_seeds_.clear();
    try {
      body();
      run();  // deferred elementwise ops of the body are part of the recording
    } catch (...) {
      recording_ = false;
      slhip_graph_end(ctx_, &g);
      slhip_graph_destroy(g);
      clear_tape();
      throw;
    }
    recording_ = false;
    check(slhip_graph_end(ctx_, &g), "slhip_graph_end");
    return Graph(this, ctx_, g, std::move(recorded_seeds_));
  }
  // What a replay relies on without recording it: the host-side bookkeeping of zero_grad() and
  // backward() ran when the step was recorded, not now.  Every fill that is pending on the host
  // runs here, and every seed gradient whose fill the recording left out holds its ones again.
  // In a loop that replays the same recording this finds nothing to do from the second replay on.
  void before_replay(const std::vector<uint64_t>& seeds) {
    run();
    for (uint64_t id : seeds) {
      auto it = allocs_.find(id);
      if (it == allocs_.end()) continue;
      stale_.erase(id);
      if (!ones_.count(id)) {
        check(slhip_fill(ctx_, it->second.len, 1.0f, it->second.ptr), "slhip_fill");
        ones_.insert(id);
      }
    }
    const std::vector<uint64_t> pending(stale_.begin(), stale_.end());
    for (uint64_t id : pending) {
      auto it = allocs_.find(id);
      if (it != allocs_.end()) settle(it->second);
    }
    stale_.clear();
  }

  // ---- deferred elementwise ops (GradPolicy::fuse_elementwise) ------------------------------
  // Launches everything that is deferred (the lazy device's `dev.run()`, examples/sine_net.rs:205).
  // Every op that is not elementwise, every read-back, backward() and record() call it themselves.
  void run() {
    if (pending_order_.empty() || flushing_) return;
    flushing_ = true;
    std::vector<uint64_t> order;
    order.swap(pending_order_);
    try {
      // group roots first, in the order they were issued: nodes that end a chain or have several
      // readers; a root's group pulls in the single-reader nodes below it
      for (uint64_t id : order) {
        auto it = pending_.find(id);
        if (it != pending_.end() && it->second.readers != 1) emit_group(id);
      }
      for (uint64_t id : order)
        if (pending_.count(id)) emit_group(id);
    } catch (...) {
      // the ops that did not launch have left placeholder closures on the tape: a backward pass over
      // it would silently skip them, so the tape goes with them
      flushing_ = false;
      clear_tape();
      throw;
    }
    pending_.clear();
    flushing_ = false;
  }
  // Makes b's memory hold b's value: launches what is deferred, and computes b now if it was an
  // intermediate that a fused chain kept in registers.
  void ready(const Buffer& b) {
    run();
    if (!virtual_.empty() && virtual_.count(b.id)) materialise(b.id);
  }
  size_t deferred() const { return pending_order_.size(); }

  // ---- autograd --------------------------------------------------------------------------
  void add_grad_fn(std::function<void()> f) { if (tape_enabled_) tape_.push_back(std::move(f)); }
  void enable_tape(bool on) { tape_enabled_ = on; }
  size_t tape_len() const { return tape_.size(); }

  bool has_grad(uint64_t id) const { return grads_.count(id) != 0; }
  // Gradient of `b` for reading (throws if none was ever written).
  Buffer grad(const Buffer& b) {
    auto it = grads_.find(b.id);
    if (it == grads_.end()) throw Error("buffer " + std::to_string(b.id) + " has no gradient");
    settle(it->second);
    return it->second;
  }
  // Gradient of `b` for an op that accumulates into it: created zeroed if absent.
  Buffer grad_mut(const Buffer& b) {
    Buffer g = grad_slot(b);
    settle(g);
    ones_.erase(g.id);
    return g;
  }
  // Gradient of `b` for an op that writes it: `overwrite` = the op sets every element without
  // reading any, so a pending zero fill of this gradient is dropped instead of run.
  Buffer grad_out(const Buffer& b, bool overwrite) {
    if (!overwrite) return grad_mut(b);
    Buffer g = grad_slot(b);
    stale_.erase(g.id);
    ones_.erase(g.id);
    return g;
  }
  // All gradients live side by side in a few large slabs, so that zeroing them is one fill per
  // slab instead of one per gradient (17 launches per step for the three-layer MLP otherwise).
  // Gradients of LAZY_ZERO_MIN floats and more have slabs of their own and are only marked: the
  // fill runs when the gradient is next read or accumulated into, and not at all when an op
  // overwrites it first - the activation gradients of a fused step, 64 MiB each for the classifier
  // with batch 8192, are all written that way (41 us of fills a step otherwise).
  void zero_grad() {
    run();
    for (auto& sl : slabs_)
      if (!sl.lazy && sl.used) check(slhip_memset(ctx_, sl.base, 0, sl.used * sizeof(float)), "slhip_memset");
    for (auto& kv : grads_) {
      if (lazy_.count(kv.second.id)) stale_.insert(kv.second.id);
      else ones_.erase(kv.second.id);
    }
  }
  void drop_pending_zero(const Buffer& g) {  // the caller overwrites all of g
    stale_.erase(g.id);
    ones_.erase(g.id);
  }
  // Runs the zero fill that zero_grad() left pending for this buffer, if any.
  void settle(const Buffer& g) {
    if (!stale_.empty() && stale_.erase(g.id)) {
      check(slhip_memset(ctx_, g.ptr, 0, g.len * sizeof(float)), "slhip_memset");
      ones_.erase(g.id);
    }
  }
  // After a backward pass, finished or failed, the device holds no tape: a closure that throws
  // (a released buffer, a refused launch) must not leave the rest behind for the next pass to replay.
  // (virtual_ stays: an intermediate that a chain kept in registers can still be asked for after
  // the backward pass, and is computed then)
  void clear_tape() {
    tape_.clear();
    relu_pre_.clear();
    relu_bits_.clear();
    relu_grad_done_.clear();
    relu_uses_.clear();
    pending_.clear();
    pending_order_.clear();
  }
  void run_tape() {
    try {
      for (size_t i = tape_.size(); i-- > 0;) tape_[i]();
    } catch (...) {
      clear_tape();
      throw;
    }
    clear_tape();
  }
  // Seeds out's gradient with ones and runs the tape.  A seed gradient that backward() itself created
  // lives with the deferred-zero gradients: while nothing else has written it since the last
  // backward(), it still holds the ones, zero_grad() has only marked it, and the fill is skipped
  // (one kernel less in every training step, recorded or not).
  void backward(const Buffer& out) {
    run();
    const bool fresh = !has_grad(out.id);
    Buffer g = grad_slot(out, /*lazy=*/fresh);
    const bool still_ones = ones_.count(g.id) != 0;
    stale_.erase(g.id);
    if (!still_ones) check(slhip_fill(ctx_, g.len, 1.0f, g.ptr), "slhip_fill");
    else if (recording_) recorded_seeds_.push_back(g.id);
    ones_.insert(g.id);
    run_tape();
  }
  void backward_with(const Buffer& out, const Buffer& seed) {
    if (seed.len != out.len) throw Error("backward_with: seed length differs");
    run();
    ready(seed);
    Buffer g = grad_out(out, true);
    check(slhip_memcpy_d2d(ctx_, g.ptr, seed.ptr, g.len * sizeof(float)), "slhip_memcpy_d2d");
    run_tape();
  }

  // ---- ops: forward + tape registration (reference: the *MayGrad impls in src/ops.rs) ------
  // GemmMayGrad::gemm  src/ops.rs:250-289
  Buffer gemm(size_t m, size_t k, size_t n, const Buffer& lhs, const Buffer& rhs) {
    expect(lhs, m * k, "gemm lhs"); expect(rhs, k * n, "gemm rhs");
    used(lhs, rhs);
    Buffer out = retrieve(m * n);
    check(slhip_gemm(ctx_, m, k, n, lhs.ptr, rhs.ptr, out.ptr), "slhip_gemm");
    uint64_t li = lhs.id, ri = rhs.id, oi = out.id;
    add_grad_fn([=] {
      Buffer l = lookup(li), r = lookup(ri), o = lookup(oi);
      const bool set = policy.gemm_beta == 0.0f;
      float* lg = l.requires_grad ? grad_out(l, set).ptr : nullptr;
      float* rg = r.requires_grad ? grad_out(r, set).ptr : nullptr;
      check(slhip_gemm_grad(ctx_, m, k, n, l.ptr, r.ptr, lg, rg, grad(o).ptr, policy.gemm_beta), "slhip_gemm_grad");
    });
    return out;
  }

  // Linear forward fused into the GEMM epilogue: relu?(x·w + bias) in one kernel.  On the tape
  // it is the same three closures the unfused sequence gemm -> add_row_mut -> relu leaves
  // (examples/sine_net.rs:32-40, src/matrix.rs:169-190), merged into one.
  Buffer linear(size_t m, size_t k, size_t n, const Buffer& x, const Buffer& w, const Buffer& bias, bool relu) {
    expect(x, m * k, "linear x"); expect(w, k * n, "linear w"); expect(bias, n, "linear bias");
    used(x, w, bias);
    Buffer pre = relu ? retrieve(m * n) : Buffer();
    Buffer out = retrieve(m * n);
    // (layers narrower than 64 outputs keep the float mask: the bit kernels' tile path starts there)
    const bool as_bits = relu && policy.fuse_relu_grad && policy.relu_bits && m * n >= (size_t(1) << 22) && n >= 64 && k > 16;
    Buffer mask = as_bits ? retrieve(m * ((n + 31) / 32)) : Buffer();
    if (as_bits)
      check(slhip_linear_fwd_bits(ctx_, m, k, n, x.ptr, w.ptr, bias.ptr, (uint32_t*)mask.ptr, out.ptr), "slhip_linear_fwd_bits");
    else
      check(slhip_linear_fwd(ctx_, m, k, n, x.ptr, w.ptr, bias.ptr, relu ? 1 : 0, relu ? pre.ptr : nullptr, out.ptr),
            "slhip_linear_fwd");
    uint64_t xi = x.id, wi = w.id, bi = bias.id, oi = out.id, pi = relu ? pre.id : 0, mi = as_bits ? mask.id : 0;
    if (relu && tape_enabled_) relu_pre_[oi] = pi;  // entries live until run_tape()
    if (as_bits && tape_enabled_) relu_bits_[oi] = mi;
    add_grad_fn([=] {
      Buffer xb = lookup(xi), wb = lookup(wi), bb = lookup(bi), o = lookup(oi);
      Buffer g;
      if (relu) {  // relu grad: pre.grad += (pre >= 0) * out.grad
        Buffer p = lookup(pi);
        Buffer pg = grad_mut(p);
        relu_pre_.erase(oi);
        relu_bits_.erase(oi);
        if (!relu_grad_done_.erase(oi)) {  // else the consumer's backward has written pre.grad already
          if (mi) check(slhip_relu_grad_bits(ctx_, m, n, (const uint32_t*)lookup(mi).ptr, pg.ptr, grad(o).ptr), "relu grad");
          else check(slhip_ew_unary_grad(ctx_, SLHIP_RELU, 0.0f, p.len, p.ptr, pg.ptr, grad(o).ptr), "relu grad");
        }
        g = pg;
      } else {
        g = grad(o);
      }
      float* bg = grad_mut(bb).ptr;
      const bool set = policy.gemm_beta == 0.0f;
      auto producer = relu_pre_.find(xi);
      auto uses = relu_uses_.find(xi);
      // only when this Linear is the ReLU output's single reader: any other consumer adds its own
      // term to x.grad, which the producer's ReLU gradient then has to pick up the unfused way
      const bool into_pre = policy.fuse_relu_grad && xb.requires_grad && producer != relu_pre_.end() &&
                            uses != relu_uses_.end() && uses->second == 1;
      float* xg = xb.requires_grad && !into_pre ? grad_out(xb, set).ptr : nullptr;
      float* wg = wb.requires_grad ? grad_out(wb, set).ptr : nullptr;
      auto packed = into_pre ? relu_bits_.find(xi) : relu_bits_.end();
      if (into_pre && packed != relu_bits_.end()) {
        // x is the ReLU output of a fused Linear that is still on the tape, its mask one bit an element
        Buffer xp = lookup(producer->second);
        check(slhip_add_row_mut_grad(ctx_, m, n, bg, g.ptr), "bias grad");
        check(slhip_sgemm_relu_bits(ctx_, 0, 1, m, k, n, g.ptr, wb.ptr, (const uint32_t*)lookup(packed->second).ptr,
                                    grad_out(xp, set).ptr, policy.gemm_beta),
              "slhip_sgemm_relu_bits");
        relu_grad_done_.insert(xi);
        check(slhip_gemm_grad(ctx_, m, k, n, xb.ptr, wb.ptr, nullptr, wg, g.ptr, policy.gemm_beta), "slhip_gemm_grad");
        return;
      }
      const float* pre = nullptr;
      if (into_pre) {
        // the same with the float pre-activations as the mask.  x.grad goes to pre.grad, written the
        // way gemm_grad writes x.grad (policy.gemm_beta; SET by default): pre.grad is zero at this
        // point, and `0 + v` differs from `v` only in the sign of a zero
        Buffer xp = lookup(producer->second);
        pre = xp.ptr;
        xg = grad_out(xp, set).ptr;
        relu_grad_done_.insert(xi);
      }
      // bias, input and weight gradient: one launch for small layers, else the three kernels in turn
      check(slhip_linear_grad(ctx_, m, k, n, xb.ptr, wb.ptr, xg, pre, wg, bg, g.ptr, policy.gemm_beta), "slhip_linear_grad");
    });
    return out;
  }

  // RowOpMayGrad::add_row  src/ops.rs:323-356
  Buffer add_row(size_t rows, size_t cols, const Buffer& lhs, const Buffer& rhs) {
    expect(lhs, rows * cols, "add_row lhs"); expect(rhs, cols, "add_row rhs");
    used(lhs, rhs);
    Buffer out = retrieve(rows * cols);
    check(slhip_add_row(ctx_, rows, cols, lhs.ptr, rhs.ptr, out.ptr), "slhip_add_row");
    uint64_t li = lhs.id, ri = rhs.id, oi = out.id;
    add_grad_fn([=] {
      Buffer l = lookup(li), r = lookup(ri), o = lookup(oi);
      check(slhip_add_row_grad(ctx_, rows, cols, grad_mut(l).ptr, grad_mut(r).ptr, grad(o).ptr), "slhip_add_row_grad");
    });
    return out;
  }
  // RowOpMayGrad::add_row_mut  src/ops.rs:358-374 — in place; lhs keeps its id and gradient
  void add_row_mut(size_t rows, size_t cols, const Buffer& lhs, const Buffer& rhs) {
    expect(lhs, rows * cols, "add_row_mut lhs"); expect(rhs, cols, "add_row_mut rhs");
    used(lhs, rhs);
    check(slhip_add_row(ctx_, rows, cols, lhs.ptr, rhs.ptr, lhs.ptr), "slhip_add_row");
    uint64_t li = lhs.id, ri = rhs.id;
    add_grad_fn([=] {
      Buffer l = lookup(li), r = lookup(ri);
      check(slhip_add_row_mut_grad(ctx_, rows, cols, grad_mut(r).ptr, grad(l).ptr), "slhip_add_row_mut_grad");
    });
  }

  // RowOp::row_op / ColOp::col_op with a named op (src/ops2/row_op/mod.rs:17-30,
  // src/ops2/col_op/mod.rs:20-57) and their gradients (RowOpGrad / ColOpGrad::row_op_grad,
  // src/ops2/row_op/grad.rs:12-41, src/ops2/col_op/grad.rs:12-27): both sides accumulate.
  Buffer bcast_op(bool by_row_index, int op, size_t rows, size_t cols, const Buffer& lhs, const Buffer& rhs) {
    expect(lhs, rows * cols, "row/col op lhs"); expect(rhs, by_row_index ? rows : cols, "row/col op rhs");
    used(lhs, rhs);
    Buffer out = retrieve(rows * cols);
    check((by_row_index ? slhip_col_op : slhip_row_op)(ctx_, op, rows, cols, lhs.ptr, rhs.ptr, out.ptr), "row/col op");
    uint64_t li = lhs.id, ri = rhs.id, oi = out.id;
    add_grad_fn([=] {
      Buffer l = lookup(li), r = lookup(ri), o = lookup(oi);
      check((by_row_index ? slhip_col_op_grad : slhip_row_op_grad)(ctx_, op, rows, cols, l.ptr, r.ptr, grad_mut(l).ptr,
                                                                   grad_mut(r).ptr, grad(o).ptr),
            "row/col op grad");
    });
    return out;
  }
  Buffer row_op(int op, size_t rows, size_t cols, const Buffer& l, const Buffer& r) { return bcast_op(false, op, rows, cols, l, r); }
  Buffer col_op(int op, size_t rows, size_t cols, const Buffer& l, const Buffer& r) { return bcast_op(true, op, rows, cols, l, r); }
  Buffer sub_cols(size_t rows, size_t cols, const Buffer& l, const Buffer& r) { return col_op(SLHIP_SUB, rows, cols, l, r); }
  Buffer div_cols(size_t rows, size_t cols, const Buffer& l, const Buffer& r) { return col_op(SLHIP_DIV, rows, cols, l, r); }

  // Diagflat::diagflat + DiagflatGrad (src/ops2/diagflat/mod.rs, grad/cpu.rs:34-38)
  Buffer diagflat(const Buffer& x) {
    used(x);
    Buffer out = retrieve(x.len * x.len);
    check(slhip_diagflat(ctx_, x.len, x.ptr, out.ptr), "slhip_diagflat");
    uint64_t xi = x.id, oi = out.id;
    add_grad_fn([=] {
      Buffer xb = lookup(xi), o = lookup(oi);
      check(slhip_diagflat_grad(ctx_, xb.len, grad_mut(xb).ptr, grad(o).ptr), "slhip_diagflat_grad");
    });
    return out;
  }

  // Onehot::onehot + onehot_grad (src/ops2/onehot/cpu.rs:40-44, grad/cpu.rs:3-12)
  Buffer onehot(size_t classes, const Buffer& cls) {
    used(cls);
    Buffer out = retrieve(cls.len * classes);
    check(slhip_onehot(ctx_, cls.len, classes, cls.ptr, out.ptr), "slhip_onehot");
    uint64_t ci = cls.id, oi = out.id;
    add_grad_fn([=] {
      Buffer c = lookup(ci), o = lookup(oi);
      check(slhip_onehot_grad(ctx_, c.len, classes, c.ptr, grad_mut(c).ptr, grad(o).ptr), "slhip_onehot_grad");
    });
    return out;
  }

  // BinaryOpsMayGrad::{add,sub,mul}  src/ops.rs:115-171
  Buffer binary(int op, const Buffer& lhs, const Buffer& rhs) {
    if (lhs.len != rhs.len) throw Error("binary op: lengths differ");
    if (op < SLHIP_ADD || op > SLHIP_DIV) throw Error("binary op: unknown op code");
    if (policy.fuse_elementwise) return defer(EwNode{0, lhs.id, rhs.id, op, false, 0.0f, 0.0f, true, lhs.len}, lhs, rhs);
    used(lhs, rhs);
    Buffer out = retrieve(lhs.len);
    check(slhip_ew_binary(ctx_, op, lhs.len, lhs.ptr, rhs.ptr, out.ptr), "slhip_ew_binary");
    uint64_t li = lhs.id, ri = rhs.id, oi = out.id;
    add_grad_fn([=] {
      Buffer l = lookup(li), r = lookup(ri), o = lookup(oi);
      // the reference touches both gradients whatever requires_grad says (src/ops.rs:118-128)
      float* lg = grad_mut(l).ptr;
      float* rg = grad_mut(r).ptr;
      if (lg == rg) {
        // x op x: slice_binary_grad adds the lhs term, then the rhs term, into the one gradient
        // (src/ops2/binary_ew/grad/cpu_stack.rs:55-58); two one-sided calls keep that order
        check(slhip_ew_binary_grad(ctx_, op, l.len, l.ptr, r.ptr, lg, nullptr, grad(o).ptr), "slhip_ew_binary_grad");
        check(slhip_ew_binary_grad(ctx_, op, l.len, l.ptr, r.ptr, nullptr, rg, grad(o).ptr), "slhip_ew_binary_grad");
      } else {
        check(slhip_ew_binary_grad(ctx_, op, l.len, l.ptr, r.ptr, lg, rg, grad(o).ptr), "slhip_ew_binary_grad");
      }
    });
    return out;
  }
  Buffer add(const Buffer& l, const Buffer& r) { return binary(SLHIP_ADD, l, r); }
  Buffer sub(const Buffer& l, const Buffer& r) { return binary(SLHIP_SUB, l, r); }
  Buffer mul(const Buffer& l, const Buffer& r) { return binary(SLHIP_MUL, l, r); }

  // apply_fn + add_unary_grad: square (src/ops.rs:25-45), pow (:64-77), relu (src/matrix.rs:169-190)
  Buffer unary(int op, const Buffer& x, float p = 0.0f, float q = 0.0f, bool with_grad = true) {
    if (op < SLHIP_SQUARE || op > SLHIP_SIGMOID) throw Error("unary op: unknown op code");
    if (policy.fuse_elementwise) return defer(EwNode{0, x.id, 0, op, true, p, q, with_grad, x.len}, x, x);
    used(x);
    Buffer out = retrieve(x.len);
    check(slhip_ew_unary(ctx_, op, p, q, x.len, x.ptr, out.ptr), "slhip_ew_unary");
    if (with_grad) {
      uint64_t xi = x.id, oi = out.id;
      add_grad_fn([=] {
        Buffer xb = lookup(xi), o = lookup(oi);
        check(slhip_ew_unary_grad(ctx_, op, p, xb.len, xb.ptr, grad_mut(xb).ptr, grad(o).ptr), "slhip_ew_unary_grad");
      });
    }
    return out;
  }
  Buffer square(const Buffer& x) { return unary(SLHIP_SQUARE, x); }
  Buffer pow(const Buffer& x, float rhs) { return unary(SLHIP_POW, x, rhs); }
  Buffer relu(const Buffer& x) { return unary(SLHIP_RELU, x); }
  Buffer tanh(const Buffer& x) { return unary(SLHIP_TANH, x); }        // src/matrix.rs:206-227
  Buffer sigmoid(const Buffer& x) { return unary(SLHIP_SIGMOID, x); }  // src/matrix.rs:231-258
  Buffer exp(const Buffer& x) { return unary(SLHIP_EXP, x, 0, 0, false); }                        // src/ops.rs:435-440
  Buffer clip(const Buffer& x, float lo, float hi) { return unary(SLHIP_CLIP, x, lo, hi, false); }  // src/ops.rs:419-425

  // TransposeMayGrad::transpose  src/ops.rs:207-220
  Buffer transpose(size_t rows, size_t cols, const Buffer& x) {
    expect(x, rows * cols, "transpose");
    used(x);
    Buffer out = retrieve(x.len);
    check(slhip_transpose(ctx_, rows, cols, x.ptr, out.ptr, 0.0f), "slhip_transpose");
    uint64_t xi = x.id, oi = out.id;
    add_grad_fn([=] {
      Buffer xb = lookup(xi), o = lookup(oi);
      check(slhip_transpose(ctx_, cols, rows, grad(o).ptr, grad_out(xb, policy.transpose_beta == 0.0f).ptr, policy.transpose_beta), "transpose_grad");
    });
    return out;
  }

  // SoftmaxMayGrad::softmax  src/ops.rs:751-778
  Buffer softmax(size_t samples, size_t features, const Buffer& x) {
    expect(x, samples * features, "softmax");
    used(x);
    Buffer out = retrieve(x.len);
    check(slhip_softmax(ctx_, samples, features, x.ptr, out.ptr), "slhip_softmax");
    uint64_t xi = x.id, oi = out.id;
    add_grad_fn([=] {
      Buffer xb = lookup(xi), o = lookup(oi);
      check(slhip_softmax_grad(ctx_, samples, features, grad_out(xb, policy.softmax_beta == 0.0f).ptr, o.ptr, grad(o).ptr, policy.softmax_beta),
            "slhip_softmax_grad");
    });
    return out;
  }

  // Reductions with gradients: SumColsMayGrad (src/ops.rs:592-611), SumRows (forward + the slice
  // gradient; the reference's own wrapper is `unimplemented!()`, src/ops.rs:553-567),
  // MaxCols/MaxRows (:471-491, :515-534), MeanCols/MeanRows (:635-651, :675-684).
  enum Red { SUM_ROWS, SUM_COLS, MAX_ROWS, MAX_COLS, MEAN_ROWS, MEAN_COLS };
  Buffer reduce(Red kind, size_t rows, size_t cols, const Buffer& x) {
    expect(x, rows * cols, "reduction");
    used(x);
    const bool over_rows = kind == SUM_ROWS || kind == MAX_ROWS || kind == MEAN_ROWS;
    Buffer out = retrieve(over_rows ? cols : rows);
    typedef int32_t (*Fwd)(slhip_ctx*, size_t, size_t, const float*, float*);
    static const Fwd fwd[] = {slhip_sum_rows, slhip_sum_cols, slhip_max_rows, slhip_max_cols, slhip_mean_rows,
                              slhip_mean_cols};
    check(fwd[kind](ctx_, rows, cols, x.ptr, out.ptr), "reduction");
    uint64_t xi = x.id, oi = out.id;
    add_grad_fn([=] {
      Buffer xb = lookup(xi), o = lookup(oi);
      float* xg = grad_mut(xb).ptr;
      const float* og = grad(o).ptr;
      switch (kind) {
        case SUM_ROWS: check(slhip_sum_rows_grad(ctx_, rows, cols, xg, og), "sum_rows_grad"); break;
        case SUM_COLS: check(slhip_sum_cols_grad(ctx_, rows, cols, xg, og), "sum_cols_grad"); break;
        case MAX_ROWS: check(slhip_max_rows_grad(ctx_, rows, cols, o.ptr, xb.ptr, xg, og), "max_rows_grad"); break;
        case MAX_COLS: check(slhip_max_cols_grad(ctx_, rows, cols, o.ptr, xb.ptr, xg, og), "max_cols_grad"); break;
        case MEAN_ROWS: check(slhip_mean_rows_grad(ctx_, rows, cols, xg, og), "mean_rows_grad"); break;
        case MEAN_COLS: check(slhip_mean_cols_grad(ctx_, rows, cols, xg, og), "mean_cols_grad"); break;
      }
    });
    return out;
  }

  // Fused losses (one forward and one backward kernel each instead of an op chain); the result is
  // a one-element buffer on the tape, so `loss.backward()` works as for any other op.
  // mean squared error == sub, squared, sum_cols over one row, mul by 1/n
  Buffer mse_loss(const Buffer& x, const Buffer& y) {
    if (x.len != y.len) throw Error("mse_loss: lengths differ");
    used(x, y);
    Buffer out = retrieve(1);
    check(slhip_mse(ctx_, x.len, x.ptr, y.ptr, out.ptr), "slhip_mse");
    uint64_t xi = x.id, yi = y.id, oi = out.id;
    add_grad_fn([=] {
      Buffer xb = lookup(xi), yb = lookup(yi), o = lookup(oi);
      check(slhip_mse_grad(ctx_, xb.len, xb.ptr, yb.ptr, grad_mut(xb).ptr, grad(o).ptr), "slhip_mse_grad");
    });
    return out;
  }
  // mean over the rows of the cross-entropy of softmax(logits) against `targets`
  // == softmax on the tape + cce / cce_grad + backward_with of examples/nn.rs:124-152,229-233
  Buffer softmax_cce_loss(size_t rows, size_t cols, const Buffer& logits, const Buffer& targets) {
    expect(logits, rows * cols, "softmax_cce logits"); expect(targets, rows * cols, "softmax_cce targets");
    used(logits, targets);
    Buffer probs = retrieve(rows * cols);
    Buffer per_row = retrieve(rows);
    Buffer out = retrieve(1);
    check(slhip_softmax_cce(ctx_, rows, cols, logits.ptr, targets.ptr, probs.ptr, per_row.ptr), "slhip_softmax_cce");
    check(slhip_mean(ctx_, rows, per_row.ptr, out.ptr), "slhip_mean");
    uint64_t li = logits.id, ti = targets.id, pi = probs.id, oi = out.id;
    add_grad_fn([=] {
      Buffer l = lookup(li), t = lookup(ti), p = lookup(pi), o = lookup(oi);
      check(slhip_softmax_cce_grad(ctx_, rows, cols, p.ptr, t.ptr, grad_out(l, policy.softmax_beta == 0.0f).ptr, policy.softmax_beta, grad(o).ptr),
            "slhip_softmax_cce_grad");
    });
    return out;
  }

  // Mean::mean  src/ops2/mean/mod.rs:15-17 — a host scalar, not on the tape
  float mean(const Buffer& x) {
    ready(x);
    Buffer s = scalar_scratch();
    check(slhip_mean(ctx_, x.len, x.ptr, s.ptr), "slhip_mean");
    float v;
    check(slhip_memcpy_d2h(ctx_, &v, s.ptr, sizeof(float)), "slhip_memcpy_d2h");
    return v;
  }

  // The same reduction left on the device (for recorded sequences, which cannot read back)
  void mean_to(const Buffer& x, const Buffer& out) {
    expect(out, 1, "mean_to out");
    ready(x);
    ready(out);
    check(slhip_mean(ctx_, x.len, x.ptr, out.ptr), "slhip_mean");
  }
  void copy(const Buffer& src, size_t src_off, const Buffer& dst, size_t dst_off, size_t n) {
    if (src_off + n > src.len || dst_off + n > dst.len) throw Error("copy: range outside the buffer");
    ready(src);
    ready(dst);
    check(slhip_memcpy_d2d(ctx_, dst.ptr + dst_off, src.ptr + src_off, n * sizeof(float)), "slhip_memcpy_d2d");
  }

  // One whole training step of the sine-fit loop (examples/sine_net.rs:119-166) as two launches:
  // forward through three Linear layers with ReLU between them, the MSE loss into loss[loss_at],
  // backward, and SGD on the six parameter buffers (W1, b1, W2, b2, W3, b3) in place.  Nothing goes
  // on the tape; the parameters' gradient buffers receive this step's gradients (overwritten), so
  // `.grad()` reads what the op-by-op step would have left there.
  void mlp3_mse_step(size_t batch, size_t d_in, size_t d_h, size_t d_out, const Buffer& x, const Buffer& y,
                     const std::vector<Buffer>& params, float lr, const Buffer& loss, size_t loss_at = 0) {
    if (params.size() != 6) throw Error("mlp3_mse_step: six parameter buffers expected");
    expect(x, batch * d_in, "mlp3_mse_step x"); expect(y, batch * d_out, "mlp3_mse_step y");
    const size_t lens[6] = {d_in * d_h, d_h, d_h * d_h, d_h, d_h * d_out, d_out};
    if (loss_at >= loss.len) throw Error("mlp3_mse_step: loss slot outside the buffer");
    run();
    ready(x); ready(y); ready(loss);
    float* g[6];
    for (int i = 0; i < 6; ++i) {
      expect(params[i], lens[i], "mlp3_mse_step parameter");
      ready(params[i]);
      g[i] = grad_out(params[i], true).ptr;
    }
    check(slhip_mlp3_mse_step(ctx_, batch, d_in, d_h, d_out, x.ptr, y.ptr, params[0].ptr, params[1].ptr, params[2].ptr,
                              params[3].ptr, params[4].ptr, params[5].ptr, g, lr, loss.ptr + loss_at),
          "slhip_mlp3_mse_step");
  }

  // RandOp::rand (src/rawops/cpu/rand.rs:7-12) on the device: x[i] = lo + (hi - lo) * u_i
  void rand(const Buffer& x, float lo, float hi, uint64_t seed, uint64_t tag) {
    ready(x);
    drop_pending_zero(x);
    check(slhip_rand_uniform(ctx_, seed, tag, lo, hi, x.len, x.ptr), "slhip_rand_uniform");
  }

  // SGD of the examples (examples/sine_net.rs:105-116): value -= grad * lr, on the device
  void sgd_step(const Buffer& p, float lr) {
    ready(p);
    check(slhip_sgd_step(ctx_, p.len, p.ptr, grad(p).ptr, lr), "slhip_sgd_step");
  }
  // the same for a whole parameter list in one launch
  void sgd_step(const std::vector<Buffer>& params, float lr) {
    std::vector<float*> p;
    std::vector<const float*> g;
    std::vector<size_t> n;
    run();
    for (const Buffer& b : params) {
      p.push_back(b.ptr);
      g.push_back(grad(b).ptr);
      n.push_back(b.len);
    }
    check(slhip_sgd_step_multi(ctx_, p.size(), p.data(), g.data(), n.data(), lr), "slhip_sgd_step_multi");
  }

 private:
  // Every op's forward reports the buffers it reads.  What is counted: the consumers of a fused
  // Linear's ReLU output, because GradPolicy::fuse_relu_grad may skip that output's own gradient
  // only while exactly one op (the next fused Linear) reads it.
  void used(const Buffer& b) {
    ready(b);
    count_use(b);
  }
  void count_use(const Buffer& b) {
    if (!tape_enabled_ || relu_pre_.empty()) return;
    if (relu_pre_.count(b.id)) ++relu_uses_[b.id];
  }
  template <class... Rest>
  void used(const Buffer& b, const Rest&... rest) { used(b); used(rest...); }
  // One deferred elementwise op.  ids, not pointers: the closures resolve buffers when they run.
  struct EwNode {
    uint64_t out, a, b;  // b = 0 for a unary op
    int op;
    bool unary;
    float p, q;
    bool with_grad;
    size_t len;
    size_t tape_slot = SIZE_MAX;  // where its gradient closure goes on the tape, if anywhere
    unsigned readers = 0;         // deferred ops that read `out` so far
    uint64_t seq = 0;             // order of issue
  };
  Buffer defer(EwNode n, const Buffer& lhs, const Buffer& rhs) {
    count_use(lhs);
    if (!n.unary) count_use(rhs);
    // an input that an earlier chain kept in registers is computed now: it has a second reader
    if (!virtual_.empty()) {
      if (virtual_.count(n.a)) materialise(n.a);
      if (!n.unary && virtual_.count(n.b)) materialise(n.b);
    }
    Buffer out = retrieve(n.len);
    n.out = out.id;
    n.seq = ++ew_seq_;
    if (tape_enabled_ && n.with_grad) {
      n.tape_slot = tape_.size();
      tape_.push_back([] {});
    }
    auto reads = [&](uint64_t id) {
      auto it = pending_.find(id);
      if (it != pending_.end()) ++it->second.readers;
    };
    reads(n.a);
    if (!n.unary) reads(n.b);
    pending_[n.out] = n;
    pending_order_.push_back(n.out);
    if (pending_order_.size() >= 1024) run();  // bounds the host-side bookkeeping of very long chains
    return out;
  }
  void launch_single(const EwNode& n) {
    Buffer a = lookup(n.a), o = lookup(n.out);
    if (n.unary) check(slhip_ew_unary(ctx_, n.op, n.p, n.q, n.len, a.ptr, o.ptr), "slhip_ew_unary");
    else check(slhip_ew_binary(ctx_, n.op, n.len, a.ptr, lookup(n.b).ptr, o.ptr), "slhip_ew_binary");
  }
  // The gradient step of one elementwise op, as the op-by-op tape runs it.
  void single_grad(const EwNode& n) {
    Buffer a = lookup(n.a), o = lookup(n.out);
    if (n.unary) {
      check(slhip_ew_unary_grad(ctx_, n.op, n.p, n.len, a.ptr, grad_mut(a).ptr, grad(o).ptr), "slhip_ew_unary_grad");
      return;
    }
    Buffer b = lookup(n.b);
    // the reference touches both gradients whatever requires_grad says (src/ops.rs:118-128)
    float* lg = grad_mut(a).ptr;
    float* rg = grad_mut(b).ptr;
    if (lg == rg) {
      // x op x: slice_binary_grad adds the lhs term, then the rhs term, into the one gradient
      // (src/ops2/binary_ew/grad/cpu_stack.rs:55-58); two one-sided calls keep that order
      check(slhip_ew_binary_grad(ctx_, n.op, n.len, a.ptr, b.ptr, lg, nullptr, grad(o).ptr), "slhip_ew_binary_grad");
      check(slhip_ew_binary_grad(ctx_, n.op, n.len, a.ptr, b.ptr, nullptr, rg, grad(o).ptr), "slhip_ew_binary_grad");
    } else {
      check(slhip_ew_binary_grad(ctx_, n.op, n.len, a.ptr, b.ptr, lg, rg, grad(o).ptr), "slhip_ew_binary_grad");
    }
  }
  // Computes a fused-away intermediate into its buffer after all (somebody reads it).
  void materialise(uint64_t id) {
    auto it = virtual_.find(id);
    if (it == virtual_.end()) return;
    const EwNode n = it->second;
    virtual_.erase(it);
    materialise(n.a);
    if (!n.unary) materialise(n.b);
    launch_single(n);
  }
  // Launches the chain that ends in `root`: the root and, below it, every deferred op whose result
  // only this chain reads, as long as the program stays within 8 instructions and 4 inputs.
  void emit_group(uint64_t root) {
    std::vector<uint64_t> ops{root}, leaves;
    std::function<bool(uint64_t)> expand = [&](uint64_t id) -> bool {
      const EwNode n = pending_.at(id);
      const uint64_t srcs[2] = {n.a, n.unary ? 0 : n.b};
      for (uint64_t src : srcs) {
        if (!src || std::find(ops.begin(), ops.end(), src) != ops.end()) continue;
        auto it = pending_.find(src);
        if (it != pending_.end() && it->second.readers == 1 && ops.size() < SLHIP_EW_MAX_OPS) {
          const std::vector<uint64_t> ops_before = ops, leaves_before = leaves;
          ops.push_back(src);
          if (expand(src)) continue;
          ops = ops_before;        // does not fit: src is computed on its own and read as an input
          leaves = leaves_before;
        }
        if (std::find(leaves.begin(), leaves.end(), src) == leaves.end()) {
          if (leaves.size() == SLHIP_EW_MAX_INPUTS) return false;
          leaves.push_back(src);
        }
      }
      return true;
    };
    if (!expand(root)) {
      const EwNode n = pending_.at(root);
      ops.assign(1, root);
      leaves.assign(1, n.a);
      if (!n.unary && n.b != n.a) leaves.push_back(n.b);
    }
    for (uint64_t leaf : leaves)
      if (pending_.count(leaf)) emit_group(leaf);  // an input that is itself deferred comes first
    std::vector<EwNode> group;
    for (uint64_t id : ops) group.push_back(pending_.at(id));
    std::sort(group.begin(), group.end(), [](const EwNode& x, const EwNode& y) { return x.seq < y.seq; });
    for (uint64_t id : ops) pending_.erase(id);
    const EwNode last = group.back();  // the root: issued after everything it reads
    if (group.size() == 1) {
      launch_single(last);
      if (last.tape_slot != SIZE_MAX) tape_[last.tape_slot] = [this, last] { single_grad(last); };
      return;
    }
    // registers: input j -> j, instruction i -> 4 + i
    std::vector<slhip_ew_insn> prog;
    auto reg_of = [&](uint64_t id) -> uint8_t {
      for (size_t j = 0; j < leaves.size(); ++j)
        if (leaves[j] == id) return (uint8_t)j;
      for (size_t i = 0; i < group.size(); ++i)
        if (group[i].out == id) return (uint8_t)(SLHIP_EW_MAX_INPUTS + i);
      throw Error("elementwise fusion: operand outside its group");
    };
    for (const EwNode& n : group) {
      slhip_ew_insn in;
      in.op = (uint8_t)(n.unary ? (SLHIP_EW_UNARY | n.op) : n.op);
      in.src0 = reg_of(n.a);
      in.src1 = n.unary ? in.src0 : reg_of(n.b);
      // an op issued while the tape was off has no gradient step, as on the op-by-op tape
      in.flags = n.with_grad && n.tape_slot != SIZE_MAX ? 0 : SLHIP_EW_NOGRAD;
      in.p = n.p;
      in.q = n.q;
      prog.push_back(in);
    }
    std::vector<const float*> in_ptrs;
    for (uint64_t leaf : leaves) in_ptrs.push_back(lookup(leaf).ptr);
    check(slhip_ew_program(ctx_, last.len, in_ptrs.size(), in_ptrs.data(), prog.size(), prog.data(), lookup(last.out).ptr),
          "slhip_ew_program");
    for (size_t i = 0; i + 1 < group.size(); ++i) virtual_[group[i].out] = group[i];
    if (last.tape_slot == SIZE_MAX) {
      // The root carries no gradient (exp, clip, or issued with the tape off), so nothing flows into
      // the chain from above; a later reader of an intermediate may still leave a gradient for it.
      // Each intermediate keeps its own gradient step at its own place on the tape, as issued op by
      // op: it computes what it reads (a fused-away intermediate) first.
      for (size_t i = 0; i + 1 < group.size(); ++i) {
        const EwNode n = group[i];
        if (n.tape_slot == SIZE_MAX) continue;
        tape_[n.tape_slot] = [this, n] {
          materialise(n.a);
          if (!n.unary) materialise(n.b);
          single_grad(n);
        };
      }
      return;
    }
    tape_[last.tape_slot] = [this, group, leaves, prog] {
      const EwNode& root_node = group.back();
      // Another op has read an intermediate after all and left a gradient for it: that term has to
      // flow on through the intermediate's own gradient step, so the chain runs backwards op by op.
      bool touched = false;
      for (size_t i = 0; i + 1 < group.size(); ++i) touched = touched || has_grad(group[i].out);
      if (touched) {
        for (size_t i = 0; i + 1 < group.size(); ++i) materialise(group[i].out);
        for (size_t i = group.size(); i-- > 0;)
          if (group[i].with_grad && group[i].tape_slot != SIZE_MAX && has_grad(group[i].out)) single_grad(group[i]);
        return;
      }
      std::vector<const float*> ins;
      std::vector<float*> grads;
      for (uint64_t leaf : leaves) {
        Buffer l = lookup(leaf);
        ins.push_back(l.ptr);
        grads.push_back(grad_mut(l).ptr);
      }
      check(slhip_ew_program_grad(ctx_, root_node.len, ins.size(), ins.data(), grads.data(), prog.size(), prog.data(),
                                  grad(lookup(root_node.out)).ptr),
            "slhip_ew_program_grad");
    };
  }

  static void expect(const Buffer& b, size_t len, const char* what) {
    if (!b.valid() || b.len != len)
      throw Error(std::string(what) + ": buffer length " + std::to_string(b.len) + " != " + std::to_string(len));
  }
  // Gradient pool: bump allocation in 256-byte granules out of slabs that double in size
  // (16 MiB first, 1 GiB at most, or whatever one gradient needs).  A slab is zeroed once when it
  // is created; memory of released gradients is not handed out again.
  struct Slab {
    float* base;
    size_t cap, used;
    bool lazy;  // holds the large gradients, which zero_grad() marks instead of filling
  };
  static constexpr size_t LAZY_ZERO_MIN = size_t(1) << 20;
  Buffer pool_alloc(size_t len, bool force_lazy = false) {
    const size_t need = (len + 63) / 64 * 64;
    const bool lazy = force_lazy || len >= LAZY_ZERO_MIN;
    Slab* cur = nullptr;
    size_t last_cap = 0;
    for (auto& sl : slabs_)
      if (sl.lazy == lazy) { cur = &sl; last_cap = sl.cap; }
    if (!cur || cur->used + need > cur->cap) {
      size_t cap = last_cap ? last_cap * 2 : (size_t(1) << 22);
      if (cap > (size_t(1) << 28)) cap = size_t(1) << 28;
      if (cap < need) cap = need;
      Slab sl{nullptr, cap, 0, lazy};
      check(slhip_malloc(ctx_, cap * sizeof(float), (void**)&sl.base), "slhip_malloc");
      check(slhip_memset(ctx_, sl.base, 0, cap * sizeof(float)), "slhip_memset");
      slabs_.push_back(sl);
      cur = &slabs_.back();
    }
    Buffer b;
    b.dev = this;
    b.id = next_id_++;
    b.len = len;
    b.ptr = cur->base + cur->used;
    b.requires_grad = false;
    b.pooled = true;
    cur->used += need;
    allocs_[b.id] = b;
    if (lazy) lazy_.insert(b.id);
    return b;
  }
  Buffer grad_slot(const Buffer& b, bool lazy = false) {
    auto it = grads_.find(b.id);
    if (it != grads_.end()) return it->second;
    Buffer g = pool_alloc(b.len, lazy);  // out of a slab that was zeroed when it was created
    grads_[b.id] = g;
    return g;
  }
  Buffer scalar_scratch() {
    if (!scratch_.valid()) scratch_ = alloc(1, true);
    return scratch_;
  }

  slhip_ctx* ctx_ = nullptr;
  bool cached_;
  uint64_t next_id_ = 1;
  std::unordered_map<uint64_t, Buffer> allocs_;
  std::unordered_map<uint64_t, Buffer> grads_;
  std::vector<Slab> slabs_;
  std::vector<std::function<void()>> tape_;
  std::unordered_map<uint64_t, uint64_t> relu_pre_;   // ReLU output of a fused Linear on the tape -> its pre-activation
  bool recording_ = false;                            // inside record(): ops land in a graph
  std::vector<uint64_t> recorded_seeds_;              // seed gradients the current recording relies on
  std::unordered_set<uint64_t> lazy_;                 // gradients in the slabs that zero_grad() marks instead of filling
  std::unordered_set<uint64_t> ones_;                 // gradients known to hold nothing but 1.0 (backward()'s seed)
  std::unordered_set<uint64_t> stale_;                // large gradients with a zero fill pending since zero_grad()
  std::unordered_map<uint64_t, uint64_t> relu_bits_;  // ... -> its packed mask, where the forward kept bits instead
  std::unordered_set<uint64_t> relu_grad_done_;       // ReLU outputs whose pre-activation gradient a consumer has written
  std::unordered_map<uint64_t, unsigned> relu_uses_;  // ReLU output of a fused Linear on the tape -> ops that read it so far
  std::unordered_map<uint64_t, EwNode> pending_;      // deferred elementwise ops by the buffer they will write
  std::vector<uint64_t> pending_order_;               // ... in the order they were issued
  std::unordered_map<uint64_t, EwNode> virtual_;      // intermediates a launched chain kept in registers: how to compute them
  uint64_t ew_seq_ = 0;
  bool flushing_ = false;
  bool tape_enabled_ = true;
  std::vector<Buffer> cache_;
  size_t cursor_ = 0;
  Buffer scratch_;
};

inline std::vector<float> Buffer::read() const {
  std::vector<float> v(len);
  dev->ready(*this);
  dev->settle(*this);
  check(slhip_memcpy_d2h(dev->ctx(), v.data(), ptr, len * sizeof(float)), "slhip_memcpy_d2h");
  return v;
}
inline void Buffer::write(const float* host, size_t n) const {
  if (n != len) throw Error("write: length differs");
  dev->ready(*this);
  dev->drop_pending_zero(*this);
  check(slhip_memcpy_h2d(dev->ctx(), ptr, host, len * sizeof(float)), "slhip_memcpy_h2d");
}
inline void Graph::run() const {
  dev_->before_replay(seeds_);
  check(slhip_graph_launch(ctx_, g_), "slhip_graph_launch");
}
inline Buffer Buffer::grad() const { return dev->grad(*this); }
inline void Buffer::backward() const { dev->backward(*this); }
inline void Buffer::backward_with(const Buffer& g) const { dev->backward_with(*this, g); }

// ---------------------------------------------------------------------------------------------
// Matrix: {Buffer, rows, cols} with a method per op (src/matrix.rs).
// ---------------------------------------------------------------------------------------------
class Matrix {
 public:
  Buffer data;
  size_t rows = 0, cols = 0;

  Matrix() = default;
  Matrix(Buffer b, size_t r, size_t c) : data(b), rows(r), cols(c) {
    if (b.len != r * c) throw Error("Matrix: buffer length != rows*cols");  // src/matrix/impl_from.rs:7-10
  }
  Matrix(HIP& dev, size_t r, size_t c) : data(dev.alloc(r * c, true)), rows(r), cols(c) {}
  Matrix(HIP& dev, size_t r, size_t c, const std::vector<float>& v) : Matrix(dev.from(v), r, c) {}

  HIP& device() const { return *data.dev; }
  Matrix require_grad() { data.requires_grad = true; data.dev->set_requires_grad(data.id, true); return *this; }
  Matrix no_grad() { data.requires_grad = false; data.dev->set_requires_grad(data.id, false); return *this; }
  std::vector<float> read() const { return data.read(); }
  Matrix grad() const { return Matrix(data.grad(), rows, cols); }
  void backward() const { data.backward(); }
  void backward_with(const Matrix& g) const { data.backward_with(g.data); }

  // Matrix::rand (src/matrix.rs:266-271 -> RandOp::rand, src/rawops/cpu/rand.rs:7-12): every element
  // uniform in [lo, hi).  The reference draws from an unseeded generator; here the stream is
  // counter-based and named by (seed, tag), so a run can be repeated and checked on the host.
  void rand(float lo, float hi, uint64_t seed = 0x51CED, uint64_t tag = 0) { device().rand(data, lo, hi, seed, tag); }

  Matrix T() const { return Matrix(device().transpose(rows, cols, data), cols, rows); }                         // :98-107
  Matrix gemm(const Matrix& rhs) const { return Matrix(device().gemm(rows, cols, rhs.cols, data, rhs.data), rows, rhs.cols); }  // :111-122
  Matrix add(const Matrix& rhs) const { return Matrix(device().add(data, rhs.data), rows, cols); }              // :127-132
  Matrix sub(const Matrix& rhs) const { return Matrix(device().sub(data, rhs.data), rows, cols); }              // :409-417
  Matrix mul(const Matrix& rhs) const { return Matrix(device().mul(data, rhs.data), rows, cols); }              // :137-142
  Matrix add_row(const Matrix& rhs) const { return Matrix(device().add_row(rows, cols, data, rhs.data), rows, cols); }  // :146-156
  void add_row_mut(const Matrix& rhs) { device().add_row_mut(rows, cols, data, rhs.data); }                     // :160-165
  Matrix relu() const { return Matrix(device().relu(data), rows, cols); }                                       // :169-190
  Matrix squared() const { return Matrix(device().square(data), rows, cols); }                                  // :275-288
  Matrix pow(float rhs) const { return Matrix(device().pow(data, rhs), rows, cols); }                           // :292-297
  Matrix softmax() const { return Matrix(device().softmax(rows, cols, data), rows, cols); }                     // :368-378
  Matrix tanh() const { return Matrix(device().tanh(data), rows, cols); }                                       // :206-227
  Matrix sigmoid() const { return Matrix(device().sigmoid(data), rows, cols); }                                 // :231-258
  Matrix l2_norm_cols() const { return squared().sum_cols().pow(0.5f); }                                        // :337-355
  Matrix diagflat() const { return Matrix(device().diagflat(data), data.len, data.len); }                       // :359-364
  Matrix sum_cols() const { return Matrix(device().reduce(HIP::SUM_COLS, rows, cols, data), rows, 1); }         // :329-334
  // The reference's Matrix::max_rows / max_cols wrap the reduced buffer as (rows, cols) and trip
  // its own length assert unless one dimension is 1 (src/matrix.rs:301-325); here the result
  // carries its true shape.
  Matrix max_rows() const { return Matrix(device().reduce(HIP::MAX_ROWS, rows, cols, data), 1, cols); }
  Matrix max_cols() const { return Matrix(device().reduce(HIP::MAX_COLS, rows, cols, data), rows, 1); }
  Matrix as_dims(size_t r, size_t c) const { return Matrix(data, r, c); }                                       // :383-390
};

}  // namespace sliced
