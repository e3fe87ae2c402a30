// Shared definitions of the gfx950 backend: context, error plumbing, launch helpers and the
// wave64 reduction primitives used by every bandwidth kernel.
#pragma once
#include <hip/hip_runtime.h>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstring>

#include "../../include/sliced_hip.h"

#define SLHIP_API extern "C" __attribute__((visibility("default")))

struct slhip_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  bool owns_stream = false;
  void* workspace = nullptr;     // partials of two-stage reductions and split-K GEMM
  size_t workspace_bytes = 0;
  int num_cu = 256;
  char name[64] = {0};
  bool capturing = false;        // between slhip_graph_begin and slhip_graph_end
  int gemm_tail = 0;             // SLHIP_TAIL_*: how the tiled GEMM treats a partly filled last round
  int gemm_tile = 0;             // SLHIP_TILE_*: tile of C per workgroup of the tiled GEMM
  float* static_scratch = nullptr;  // this device's copy of the file-scope scratch array of reduce.hip
  // what the last product on this context ran as (slhip_gemm_plan_describe); set by gemm_run
  struct GemmPlan {
    int kind = 0;  // 0 none, 1 wave-per-tile, 2 tiled four waves, 3 tiled eight waves, 4 spread tail, 5 tall A, 6 skinny
    bool ta = false, tb = false, only_fast = false, small_tile = false;
    unsigned splits = 1, waves = 4;
  } last_gemm;
  // A product issued as its transpose (gemm_run): where the combine of the inner product's k shares may
  // write the result, transposed, instead of leaving it to a transpose launch of its own.
  float* swap_c = nullptr;   // the caller's C (N' x M' row-major for an inner M' x N' product), or null
  float swap_beta = 0.0f;
  bool swap_done = false;    // a combine has written swap_c
};

struct slhip_event {
  hipEvent_t ev;
};

struct slhip_graph {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  size_t nodes = 0;
};

namespace slhip {

constexpr int WAVE = 64;
constexpr size_t DEFAULT_WORKSPACE_BYTES = size_t(256) << 20;

void set_error(const char* fmt, ...);
// reduce.hip: resolves the device address of the file-scope scratch array for `device`, which must
// be the current device.  Called once per context by slhip_init.
int32_t static_scratch_resolve(int device, float** ptr);
int32_t hip_fail(hipError_t e, const char* what);

#define SLHIP_CHECK_HIP(expr)                                   \
  do {                                                          \
    hipError_t _e = (expr);                                     \
    if (_e != hipSuccess) return slhip::hip_fail(_e, #expr);    \
  } while (0)

#define SLHIP_NOT_CAPTURING(ctx)                                                        \
  do {                                                                                 \
    if ((ctx)->capturing) {                                                            \
      slhip::set_error("%s: not allowed while the context records a graph", __func__); \
      return SLHIP_ECAPTURE;                                                           \
    }                                                                                  \
  } while (0)

#define SLHIP_REQUIRE(cond, msg)                                \
  do {                                                          \
    if (!(cond)) {                                              \
      slhip::set_error("%s: %s", __func__, msg);                \
      return SLHIP_EINVAL;                                      \
    }                                                           \
  } while (0)

// rows*cols with overflow check; false on overflow or zero.
inline bool checked_len(size_t rows, size_t cols, size_t* len) {
  if (rows == 0 || cols == 0) return false;
  if (rows > SIZE_MAX / cols) return false;
  *len = rows * cols;
  return *len <= (SIZE_MAX / sizeof(float));
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int32_t post_launch() {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return hip_fail(e, "kernel launch");
  return SLHIP_OK;
}

// Blocks for `a` items at `b` per block.  The count is computed in size_t; launch sites check
// grid_fits() first, because a count cast to unsigned would wrap and cover part of the data.
constexpr size_t MAX_GRID = 0x7fffffffu;
inline bool grid_fits(size_t a, size_t b) { return (a + b - 1) / b <= MAX_GRID; }
inline unsigned ceil_div(size_t a, size_t b) { return (unsigned)((a + b - 1) / b); }

// ------------------------------------------------------------------ device helpers
struct SumOp {
  static __device__ __forceinline__ float identity() { return 0.0f; }
  static __device__ __forceinline__ float apply(float a, float b) { return a + b; }
};
// fmaxf returns its other operand when one is NaN, so NaN is its neutral element and -inf is not:
// a row of nothing but NaN has NaN as its maximum (src/ops2/max/cpu.rs:11-13 folds `T::max` from the
// row's first element), which an accumulator that starts at -inf would turn into -inf.
struct MaxOp {
  static __device__ __forceinline__ float identity() { return __builtin_nanf(""); }
  static __device__ __forceinline__ float apply(float a, float b) { return fmaxf(a, b); }
};

// Butterfly reduction over `width` adjacent lanes (power of two, <= 64) of a wave64.
template <class Op, int width = WAVE>
__device__ __forceinline__ float wave_reduce(float v) {
#pragma unroll
  for (int off = width / 2; off > 0; off >>= 1) v = Op::apply(v, __shfl_xor(v, off, WAVE));
  return v;
}

// Block-wide reduction; every thread receives the result. `smem` holds >= blockDim.x/64 floats.
template <class Op>
__device__ __forceinline__ float block_reduce(float v, float* smem) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int wid = threadIdx.x >> 6;
  const int nw = (blockDim.x + WAVE - 1) >> 6;
  v = wave_reduce<Op>(v);
  if (nw == 1) return v;
  __syncthreads();  // smem may still be read from a previous call
  if (lane == 0) smem[wid] = v;
  __syncthreads();
  float r = lane < nw ? smem[lane] : Op::identity();
  r = wave_reduce<Op>(r);
  return r;
}

// 16-byte aligned vector access: LDS, and global memory whose alignment the caller has checked.
__device__ __forceinline__ float4 ld4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ void st4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }

// Global-memory vector access that only needs the 4-byte alignment every float* has: gfx950
// serves dwordx4 loads and stores at any dword address (measured on a 1 GiB copy: 6.7 TB/s
// aligned, 6.4 with the source one float off, 5.3 with both off, against 2.4 TB/s for scalar
// accesses), so views at odd offsets and rows of odd length keep the vector paths.
typedef float slhip_f4 __attribute__((ext_vector_type(4), aligned(4)));
__device__ __forceinline__ float4 ld4g(const float* p) {
  slhip_f4 t = *reinterpret_cast<const slhip_f4*>(p);
  return make_float4(t.x, t.y, t.z, t.w);
}
__device__ __forceinline__ void st4g(float* p, float4 v) {
  slhip_f4 t = {v.x, v.y, v.z, v.w};
  *reinterpret_cast<slhip_f4*>(p) = t;
}
// Streaming (non-temporal) forms for data that is touched once per kernel: measured on
// MI355X they raise read bandwidth from about 6.2 to 7.1 TB/s and copy bandwidth by 5-8 %.
__device__ __forceinline__ float4 ld4s(const float* p) {
  slhip_f4 t = __builtin_nontemporal_load(reinterpret_cast<const slhip_f4*>(p));
  return make_float4(t.x, t.y, t.z, t.w);
}
__device__ __forceinline__ void st4s(float* p, float4 v) {
  slhip_f4 t = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(t, reinterpret_cast<slhip_f4*>(p));
}
__device__ __forceinline__ float ld1s(const float* p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void st1s(float* p, float v) { __builtin_nontemporal_store(v, p); }

// d f(l, r) / d l   and   d f(l, r) / d r, as the reference's tests write them
// (src/ops2/col_op/grad/cpu.rs:115,146: 1/rhs and lhs / -(rhs*rhs) for div)
__device__ __forceinline__ float bc_dl(int op, float /*l*/, float r) {
  switch (op) {
    case SLHIP_ADD: return 1.0f;
    case SLHIP_SUB: return 1.0f;
    case SLHIP_MUL: return r;
    default: return 1.0f / r;
  }
}
__device__ __forceinline__ float bc_dr(int op, float l, float r) {
  switch (op) {
    case SLHIP_ADD: return 1.0f;
    case SLHIP_SUB: return -1.0f;
    case SLHIP_MUL: return l;
    default: return l / (-(r * r));
  }
}

// v_grad[i] += the rhs-gradient terms of a broadcast op summed over row i (by_row) or column i
// (defined with the reductions, whose kernels it runs).
int32_t bc_grad_rhs_reduce(slhip_ctx* ctx, bool by_row, int op, size_t rows, size_t cols, const float* lhs, const float* v,
                           const float* g, float* v_grad);

// loss[r] = -ln sum_c clip(p[r, c], 1e-7, 1 - 1e-7) * t[r, c], through the contiguous-axis
// reduction kernels (defined with them).
int32_t cce_rows_reduce(slhip_ctx* ctx, size_t rows, size_t cols, const float* p, const float* t, float* loss);

// logits_grad = beta * logits_grad + (probs * sum_c targets - targets) * (upstream / rows), through
// the softmax backward kernels (defined with them).
int32_t softmax_cce_grad_rows(slhip_ctx* ctx, size_t rows, size_t cols, const float* probs, const float* targets,
                              float* logits_grad, float beta, const float* upstream_dev);

// probs = softmax(logits) (probs may be null), loss_rows[r] = -ln sum_c clip(probs) * targets, in
// one pass through the softmax forward kernels; rows of more than softmax_one_pass_cols() floats
// are refused (defined with those kernels).
int32_t softmax_cce_rows(slhip_ctx* ctx, size_t rows, size_t cols, const float* logits, const float* targets, float* probs,
                         float* loss_rows);
size_t softmax_one_pass_cols();

}  // namespace slhip
