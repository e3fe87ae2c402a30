// Runtime part of the C ABI: context, memory, events, fills, the seeded generator.
#include <cstdarg>

#include "common.hpp"

namespace slhip {

static thread_local char g_err[512] = "no error";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int32_t hip_fail(hipError_t e, const char* what) {
  set_error("%s failed: %s (%d)", what, hipGetErrorString(e), (int)e);
  (void)hipGetLastError();  // clear the sticky launch error so later calls report their own
  return (int32_t)e > 0 ? (int32_t)e : SLHIP_EINVAL;
}

__global__ void fill_kernel(size_t n, float v, float* __restrict__ x) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) x[i] = v;
}

// Device copy, one streaming float4 per thread (6.7 TB/s on MI355X against about 5 TB/s for the
// runtime's own device-to-device copy).
__global__ __launch_bounds__(64) void copy4_kernel(size_t n4, const float* __restrict__ src, float* __restrict__ dst) {
  const size_t i = (size_t)blockIdx.x * 64 + threadIdx.x;
  if (i < n4) st4s(dst + 4 * i, ld4s(src + 4 * i));
}

// Whatever the vector copy cannot take (tails, small or unaligned copies), as words or bytes.
template <class T>
__global__ void copy_kernel(size_t n, const T* __restrict__ src, T* __restrict__ dst) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) dst[i] = src[i];
}

__device__ __forceinline__ uint64_t splitmix64(uint64_t s) {
  uint64_t z = s + 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

__global__ void rand_uniform_kernel(uint64_t base, float lo, float span, size_t n, float* __restrict__ x) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    uint32_t r = (uint32_t)(splitmix64(base + i) >> 40);
    float u = (float)r * 5.9604644775390625e-08f;  // 2^-24, exact
    x[i] = __fadd_rn(lo, __fmul_rn(span, u));      // two separately rounded operations
  }
}

static int32_t make_ctx(int32_t ordinal, hipStream_t external, bool use_external, slhip_ctx** out) {
  if (!out) {
    set_error("slhip_init: ctx is NULL");
    return SLHIP_EINVAL;
  }
  *out = nullptr;
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count == 0) {
    (void)hipGetLastError();
    set_error("slhip_init: no HIP device visible");
    return SLHIP_ENODEVICE;
  }
  if (ordinal < 0 || ordinal >= count) {
    set_error("slhip_init: device ordinal %d out of range (have %d)", ordinal, count);
    return SLHIP_EINVAL;
  }
  SLHIP_CHECK_HIP(hipSetDevice(ordinal));
  hipDeviceProp_t prop;
  SLHIP_CHECK_HIP(hipGetDeviceProperties(&prop, ordinal));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
    set_error("slhip_init: device %d is %s; this library carries gfx950 code only", ordinal, prop.gcnArchName);
    return SLHIP_ENODEVICE;
  }
  slhip_ctx* c = new slhip_ctx();
  c->device = ordinal;
  c->num_cu = prop.multiProcessorCount;
  snprintf(c->name, sizeof(c->name), "%s (%s)", prop.name, prop.gcnArchName);
  if (use_external) {
    c->stream = external;
    c->owns_stream = false;
  } else {
    e = hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking);
    if (e != hipSuccess) {
      delete c;
      return hip_fail(e, "hipStreamCreate");
    }
    c->owns_stream = true;
  }
  e = hipMalloc(&c->workspace, DEFAULT_WORKSPACE_BYTES);
  if (e != hipSuccess) {
    if (c->owns_stream) (void)hipStreamDestroy(c->stream);
    delete c;
    return hip_fail(e, "hipMalloc(workspace)");
  }
  c->workspace_bytes = DEFAULT_WORKSPACE_BYTES;
  // the device is current (hipSetDevice above): every GPU holds its own copy of the static scratch
  // array at its own address
  const int32_t rc = static_scratch_resolve(ordinal, &c->static_scratch);
  if (rc != SLHIP_OK) {
    (void)hipFree(c->workspace);
    if (c->owns_stream) (void)hipStreamDestroy(c->stream);
    delete c;
    return rc;
  }
  *out = c;
  return SLHIP_OK;
}

}  // namespace slhip

using namespace slhip;

SLHIP_API const char* slhip_last_error_string(void) { return g_err; }

SLHIP_API int32_t slhip_init(int32_t ordinal, slhip_ctx** ctx) { return make_ctx(ordinal, nullptr, false, ctx); }

SLHIP_API int32_t slhip_init_on_stream(int32_t ordinal, void* stream, slhip_ctx** ctx) {
  return make_ctx(ordinal, (hipStream_t)stream, true, ctx);
}

SLHIP_API int32_t slhip_destroy(slhip_ctx* ctx) {
  if (!ctx) return SLHIP_OK;
  (void)hipSetDevice(ctx->device);
  if (ctx->capturing) {  // abandon an unfinished recording so that the stream can be waited on
    hipGraph_t g = nullptr;
    (void)hipStreamEndCapture(ctx->stream, &g);
    if (g) (void)hipGraphDestroy(g);
    (void)hipGetLastError();
  }
  (void)hipStreamSynchronize(ctx->stream);
  if (ctx->workspace) (void)hipFree(ctx->workspace);
  if (ctx->owns_stream) (void)hipStreamDestroy(ctx->stream);
  delete ctx;
  return SLHIP_OK;
}

SLHIP_API int32_t slhip_device_name(slhip_ctx* ctx, char* buf, size_t buflen) {
  SLHIP_REQUIRE(ctx && buf && buflen > 0, "null argument");
  snprintf(buf, buflen, "%s", ctx->name);
  return SLHIP_OK;
}

SLHIP_API int32_t slhip_stream(slhip_ctx* ctx, void** s) {
  SLHIP_REQUIRE(ctx && s, "null argument");
  *s = (void*)ctx->stream;
  return SLHIP_OK;
}

SLHIP_API size_t slhip_workspace_bytes(slhip_ctx* ctx) { return ctx ? ctx->workspace_bytes : 0; }
SLHIP_API int32_t slhip_workspace(slhip_ctx* ctx, void** dptr) {
  SLHIP_REQUIRE(ctx && dptr, "null argument");
  *dptr = ctx->workspace;
  return SLHIP_OK;
}

SLHIP_API int32_t slhip_malloc(slhip_ctx* ctx, size_t bytes, void** dptr) {
  SLHIP_REQUIRE(ctx && dptr, "null argument");
  SLHIP_REQUIRE(bytes > 0, "zero-byte allocation");
  SLHIP_NOT_CAPTURING(ctx);
  *dptr = nullptr;
  SLHIP_CHECK_HIP(hipMalloc(dptr, bytes));
  return SLHIP_OK;
}

SLHIP_API int32_t slhip_free(slhip_ctx* ctx, void* dptr) {
  SLHIP_REQUIRE(ctx, "null context");
  if (!dptr) return SLHIP_OK;
  SLHIP_NOT_CAPTURING(ctx);
  SLHIP_CHECK_HIP(hipStreamSynchronize(ctx->stream));
  SLHIP_CHECK_HIP(hipFree(dptr));
  return SLHIP_OK;
}

SLHIP_API int32_t slhip_memcpy_h2d(slhip_ctx* ctx, void* dst, const void* src, size_t bytes) {
  SLHIP_REQUIRE(ctx && dst && src, "null argument");
  if (bytes == 0) return SLHIP_OK;
  SLHIP_NOT_CAPTURING(ctx);
  SLHIP_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx->stream));
  // pageable host memory: the source may be reused by the caller as soon as we return
  SLHIP_CHECK_HIP(hipStreamSynchronize(ctx->stream));
  return SLHIP_OK;
}

SLHIP_API int32_t slhip_memcpy_d2h(slhip_ctx* ctx, void* dst, const void* src, size_t bytes) {
  SLHIP_REQUIRE(ctx && dst && src, "null argument");
  if (bytes == 0) return SLHIP_OK;
  SLHIP_NOT_CAPTURING(ctx);
  SLHIP_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx->stream));
  SLHIP_CHECK_HIP(hipStreamSynchronize(ctx->stream));
  return SLHIP_OK;
}

// Device-to-device copies are kernels, never runtime copies: faster for large buffers, and a
// recording (slhip_graph_begin) then holds kernel nodes only.
SLHIP_API int32_t slhip_memcpy_d2d(slhip_ctx* ctx, void* dst, const void* src, size_t bytes) {
  SLHIP_REQUIRE(ctx && dst && src, "null argument");
  if (bytes == 0 || dst == src) return SLHIP_OK;
  size_t done = 0;
  if (bytes >= 4096 && (((uintptr_t)dst | (uintptr_t)src) & 3) == 0) {
    const size_t n4 = bytes / 16;
    SLHIP_REQUIRE((n4 + 63) / 64 <= 0x7fffffffu, "copy too large for one launch");
    hipLaunchKernelGGL(copy4_kernel, dim3((unsigned)((n4 + 63) / 64)), dim3(64), 0, ctx->stream, n4,
                       (const float*)src, (float*)dst);
    int32_t rc = post_launch();
    if (rc) return rc;
    done = n4 * 16;
    if (done == bytes) return SLHIP_OK;
  }
  const char* s = (const char*)src + done;
  char* d = (char*)dst + done;
  const size_t rest = bytes - done;
  if ((rest & 3) == 0 && (((uintptr_t)s | (uintptr_t)d) & 3) == 0) {
    const size_t n = rest / 4;
    unsigned grid = (unsigned)(n / 256 + 1 < 8192 ? n / 256 + 1 : 8192);
    hipLaunchKernelGGL(copy_kernel<uint32_t>, dim3(grid), dim3(256), 0, ctx->stream, n, (const uint32_t*)s, (uint32_t*)d);
  } else {
    unsigned grid = (unsigned)(rest / 256 + 1 < 8192 ? rest / 256 + 1 : 8192);
    hipLaunchKernelGGL(copy_kernel<uint8_t>, dim3(grid), dim3(256), 0, ctx->stream, rest, (const uint8_t*)s, (uint8_t*)d);
  }
  return post_launch();
}

SLHIP_API int32_t slhip_memset(slhip_ctx* ctx, void* dptr, int32_t value, size_t bytes) {
  SLHIP_REQUIRE(ctx && dptr, "null argument");
  if (bytes == 0) return SLHIP_OK;
  if (value == 0 && (bytes & 3) == 0 && ((uintptr_t)dptr & 3) == 0) {
    // a fill kernel rather than a memset node: safe for callers that capture the stream
    size_t n = bytes / 4;
    unsigned grid = (unsigned)(n / 256 + 1 < 4096 ? n / 256 + 1 : 4096);
    hipLaunchKernelGGL(fill_kernel, dim3(grid), dim3(256), 0, ctx->stream, n, 0.0f, (float*)dptr);
    return post_launch();
  }
  SLHIP_NOT_CAPTURING(ctx);  // a memset node: kept out of recordings
  SLHIP_CHECK_HIP(hipMemsetAsync(dptr, value, bytes, ctx->stream));
  return SLHIP_OK;
}

SLHIP_API int32_t slhip_fill(slhip_ctx* ctx, size_t n, float value, float* x) {
  SLHIP_REQUIRE(ctx && x, "null argument");
  if (n == 0) return SLHIP_OK;
  unsigned grid = (unsigned)(n / 256 + 1 < 8192 ? n / 256 + 1 : 8192);
  hipLaunchKernelGGL(fill_kernel, dim3(grid), dim3(256), 0, ctx->stream, n, value, x);
  return post_launch();
}

SLHIP_API int32_t slhip_sync(slhip_ctx* ctx) {
  SLHIP_REQUIRE(ctx, "null context");
  SLHIP_NOT_CAPTURING(ctx);
  SLHIP_CHECK_HIP(hipStreamSynchronize(ctx->stream));
  return SLHIP_OK;
}

SLHIP_API int32_t slhip_event_create(slhip_ctx* ctx, slhip_event** ev) {
  SLHIP_REQUIRE(ctx && ev, "null argument");
  slhip_event* e = new slhip_event();
  hipError_t r = hipEventCreate(&e->ev);
  if (r != hipSuccess) {
    delete e;
    return hip_fail(r, "hipEventCreate");
  }
  *ev = e;
  return SLHIP_OK;
}

SLHIP_API int32_t slhip_event_record(slhip_ctx* ctx, slhip_event* ev) {
  SLHIP_REQUIRE(ctx && ev, "null argument");
  SLHIP_NOT_CAPTURING(ctx);
  SLHIP_CHECK_HIP(hipEventRecord(ev->ev, ctx->stream));
  return SLHIP_OK;
}

SLHIP_API int32_t slhip_event_elapsed_ms(slhip_event* a, slhip_event* b, float* ms) {
  SLHIP_REQUIRE(a && b && ms, "null argument");
  SLHIP_CHECK_HIP(hipEventSynchronize(b->ev));
  SLHIP_CHECK_HIP(hipEventElapsedTime(ms, a->ev, b->ev));
  return SLHIP_OK;
}

SLHIP_API int32_t slhip_event_destroy(slhip_event* ev) {
  if (!ev) return SLHIP_OK;
  (void)hipEventDestroy(ev->ev);
  delete ev;
  return SLHIP_OK;
}

SLHIP_API int32_t slhip_graph_begin(slhip_ctx* ctx) {
  SLHIP_REQUIRE(ctx, "null context");
  SLHIP_NOT_CAPTURING(ctx);
  // relaxed mode: other threads of the process (a framework's allocator, say) stay unrestricted;
  // this library refuses its own waiting and allocating calls while `capturing` is set
  SLHIP_CHECK_HIP(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed));
  ctx->capturing = true;
  return SLHIP_OK;
}

SLHIP_API int32_t slhip_graph_end(slhip_ctx* ctx, slhip_graph** graph) {
  SLHIP_REQUIRE(ctx && graph, "null argument");
  *graph = nullptr;
  if (!ctx->capturing) {
    set_error("slhip_graph_end: the context is not recording");
    return SLHIP_ECAPTURE;
  }
  ctx->capturing = false;
  hipGraph_t g = nullptr;
  hipError_t e = hipStreamEndCapture(ctx->stream, &g);
  if (e != hipSuccess || !g) {
    if (g) (void)hipGraphDestroy(g);
    return hip_fail(e != hipSuccess ? e : hipErrorUnknown, "hipStreamEndCapture");
  }
  slhip_graph* out = new slhip_graph();
  out->graph = g;
  e = hipGraphGetNodes(g, nullptr, &out->nodes);
  if (e == hipSuccess) e = hipGraphInstantiate(&out->exec, g, nullptr, nullptr, 0);
  if (e != hipSuccess) {
    (void)hipGraphDestroy(g);
    delete out;
    return hip_fail(e, "hipGraphInstantiate");
  }
  *graph = out;
  return SLHIP_OK;
}

SLHIP_API int32_t slhip_graph_launch(slhip_ctx* ctx, slhip_graph* graph) {
  SLHIP_REQUIRE(ctx && graph && graph->exec, "null argument");
  SLHIP_NOT_CAPTURING(ctx);
  SLHIP_CHECK_HIP(hipGraphLaunch(graph->exec, ctx->stream));
  return SLHIP_OK;
}

SLHIP_API int32_t slhip_graph_node_count(slhip_graph* graph, size_t* nodes) {
  SLHIP_REQUIRE(graph && nodes, "null argument");
  *nodes = graph->nodes;
  return SLHIP_OK;
}

SLHIP_API int32_t slhip_graph_destroy(slhip_graph* graph) {
  if (!graph) return SLHIP_OK;
  if (graph->exec) (void)hipGraphExecDestroy(graph->exec);
  if (graph->graph) (void)hipGraphDestroy(graph->graph);
  delete graph;
  return SLHIP_OK;
}

SLHIP_API int32_t slhip_rand_uniform(slhip_ctx* ctx, uint64_t seed, uint64_t tag, float lo, float hi, size_t n,
                                     float* x) {
  SLHIP_REQUIRE(ctx && x, "null argument");
  if (n == 0) return SLHIP_OK;
  uint64_t base = seed ^ (tag << 40);
  unsigned grid = (unsigned)(n / 256 + 1 < 16384 ? n / 256 + 1 : 16384);
  hipLaunchKernelGGL(rand_uniform_kernel, dim3(grid), dim3(256), 0, ctx->stream, base, lo, hi - lo, n, x);
  return post_launch();
}
