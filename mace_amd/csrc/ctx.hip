// Context, arena, timers, scalar host helpers and the host-pointer staging wrappers.
#include <math.h>
#include <stdarg.h>
#include <string.h>

#include <mutex>
#include <new>

#include "common.h"

int mh_fail(mace_hip_ctx *ctx, int code, const char *fmt, ...) {
  if (ctx) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(ctx->err, sizeof(ctx->err), fmt, ap);
    va_end(ap);
  }
  return code;
}

// Scratch for the entry point that allocates nothing: one array per GPU, part of the code
// object, held from the first use of the library on that GPU until the process ends.  Host
// code never uses the array's name as an address; it asks the runtime for this device's copy
// (mh_static_scratch) and passes that pointer on.
static __device__ __align__(256) unsigned char scratch[MACE_HIP_NOALLOC_SCRATCH_BYTES];
constexpr int MH_MAX_DEVICES = 64;
static void *g_scratch_ptr[MH_MAX_DEVICES];
static std::mutex g_scratch_mutex;   // contexts may be created from several threads at once

// Address of `scratch` on `device` (which must be the current device), looked up once.
static hipError_t mh_static_scratch(int device, void **ptr) {
  if (device < 0 || device >= MH_MAX_DEVICES) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[device]) {
    void *p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    g_scratch_ptr[device] = p;
  }
  *ptr = g_scratch_ptr[device];
  return hipSuccess;
}

int mh_arena_reserve(mace_hip_ctx *ctx, size_t bytes) {
  // headroom for the per-slice alignment
  const size_t need = ctx->arena_used + bytes + 16 * 256;
  if (need <= ctx->arena_bytes) return MACE_HIP_SUCCESS;
  if (ctx->plan_only) {
    // nothing is ever read or written through a plan-only context's arena: addresses only
    ctx->arena = (char *)(uintptr_t)0x100000000ull;
    ctx->arena_bytes = mh_align_up(need + need / 4, 1 << 20);
    return MACE_HIP_SUCCESS;
  }
  if (ctx->no_alloc)
    return mh_fail(ctx, MACE_HIP_INVALID_ARGS,
                   "this call needs %zu bytes of scratch; the allocation-free entry point has %zu",
                   need, ctx->arena_bytes);
  if (ctx->fail_allocs > 0) {
    --ctx->fail_allocs;
    return mh_fail(ctx, MACE_HIP_OUT_OF_RESOURCES, "arena allocation of %zu bytes failed (mock)",
                   need);
  }
  if (ctx->capturing)
    return mh_fail(ctx, MACE_HIP_INVALID_ARGS,
                   "this call needs %zu bytes of scratch, more than the context holds; run it once "
                   "before capturing it into a graph", need);
  if (ctx->arena_used != 0)
    return mh_fail(ctx, MACE_HIP_RUNTIME_ERROR, "arena grown while slices are live");
  MH_HIP(ctx, hipStreamSynchronize(ctx->stream));
  if (ctx->arena) {
    // An instantiated graph captured from this context replays with the old arena's addresses:
    // while one exists the old arena stays allocated (retired) and only new calls move on.
    if (ctx->live_graphs > 0) ctx->retired.push_back(ctx->arena);
    else MH_HIP(ctx, hipFree(ctx->arena));
    ctx->arena = nullptr;
    ctx->arena_bytes = 0;
  }
  const size_t want = mh_align_up(need + need / 4, 1 << 20);
  void *p = nullptr;
  hipError_t e = hipMalloc(&p, want);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return mh_fail(ctx, MACE_HIP_OUT_OF_RESOURCES, "hipMalloc(%zu) failed: %s", want,
                   hipGetErrorString(e));
  }
  ctx->arena = (char *)p;
  ctx->arena_bytes = want;
  return MACE_HIP_SUCCESS;
}

void *mh_arena_take(mace_hip_ctx *ctx, size_t bytes) {
  const size_t at = mh_align_up(ctx->arena_used, 256);
  if (at + bytes > ctx->arena_bytes) return nullptr;   // reserve() was too small: a bug
  ctx->arena_used = at + bytes;
  return ctx->arena + at;
}

namespace {
__global__ __launch_bounds__(256) void mh_fill_bytes_kernel(uint8_t *dst, uint8_t value, size_t bytes) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < bytes; i += (size_t)gridDim.x * 256)
    dst[i] = value;
}
}  // namespace

int mh_fill_bytes(mace_hip_ctx *ctx, void *dst, uint8_t value, size_t bytes) {
  if (bytes == 0) return MACE_HIP_SUCCESS;
  const size_t blocks = (bytes + 255) / 256;
  mh_plan_aux(ctx, MACE_HIP_AUX_FILL);
  MH_KLAUNCH(ctx, mh_fill_bytes_kernel, dim3((unsigned)(blocks < 4096 ? blocks : 4096)), dim3(256), 0,
             ctx->stream, (uint8_t *)dst, value, bytes);
  MH_LAUNCH_CHECK(ctx);
  return MACE_HIP_SUCCESS;
}

// Entry points that move data or need a stream have nothing to do on a plan-only context.
#define MH_NEEDS_GPU(ctx)                                                                       \
  do {                                                                                          \
    if ((ctx)->plan_only)                                                                       \
      return mh_fail((ctx), MACE_HIP_UNSUPPORTED, "%s needs a GPU: this is a plan-only context", \
                     __func__);                                                                 \
  } while (0)

// Entry points that wait for the stream (or copy from or to host memory) cannot be recorded into
// a graph; while one is being captured from this context they are refused before they touch the
// runtime, so the capture itself stays valid.
#define MH_NOT_CAPTURING(ctx)                                                                  \
  do {                                                                                         \
    if ((ctx)->capturing)                                                                      \
      return mh_fail((ctx), MACE_HIP_INVALID_ARGS,                                             \
                     "%s waits for the stream: not possible while a graph is being captured", \
                     __func__);                                                                \
  } while (0)

static void mh_free_retired(mace_hip_ctx *ctx) {
  for (void *p : ctx->retired) (void)hipFree(p);
  ctx->retired.clear();
}

extern "C" {

int mace_hip_ctx_create(int device, mace_hip_ctx **out) {
  if (!out) return MACE_HIP_INVALID_ARGS;
  *out = nullptr;
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || device < 0 || device >= count) {
    (void)hipGetLastError();
    return MACE_HIP_RUNTIME_ERROR;
  }
  mace_hip_ctx *ctx = new (std::nothrow) mace_hip_ctx();
  if (!ctx) return MACE_HIP_OUT_OF_RESOURCES;
  ctx->device = device;
  hipDeviceProp_t prop;
  if (hipSetDevice(device) != hipSuccess || hipGetDeviceProperties(&prop, device) != hipSuccess ||
      hipStreamCreate(&ctx->own_stream) != hipSuccess ||
      hipEventCreate(&ctx->ev_start) != hipSuccess ||
      hipEventCreate(&ctx->ev_stop) != hipSuccess) {
    (void)hipGetLastError();
    delete ctx;
    return MACE_HIP_RUNTIME_ERROR;
  }
  void *sp = nullptr;
  if (mh_static_scratch(device, &sp) != hipSuccess) {
    (void)hipGetLastError();
    (void)hipStreamDestroy(ctx->own_stream);
    (void)hipEventDestroy(ctx->ev_start);
    (void)hipEventDestroy(ctx->ev_stop);
    delete ctx;
    return MACE_HIP_RUNTIME_ERROR;
  }
  ctx->static_scratch = (char *)sp;
  // (staging through pinned memory is an optimisation: without the buffer, copies go direct)
  void *pin = nullptr;
  if (hipHostMalloc(&pin, MH_PINNED_BYTES, hipHostMallocDefault) == hipSuccess) {
    ctx->pinned = (char *)pin;
    ctx->pinned_bytes = MH_PINNED_BYTES;
  } else {
    (void)hipGetLastError();
  }
  // so that raising a kernel's LDS limit or asking for its occupancy never reallocates (host
  // memory either: the allocation-free entry point allocates nothing at all)
  ctx->big_lds_kernels.reserve(128);
  ctx->occupancy.reserve(256);
  ctx->stream = ctx->own_stream;
  ctx->cu_count = prop.multiProcessorCount;
  ctx->lds_bytes = (int)prop.sharedMemPerBlock;
  snprintf(ctx->arch, sizeof(ctx->arch), "%s", prop.gcnArchName);
  if (strncmp(ctx->arch, "gfx950", 6) != 0) {
    // the code objects in this library exist for gfx950 only
    (void)hipStreamDestroy(ctx->own_stream);
    (void)hipEventDestroy(ctx->ev_start);
    (void)hipEventDestroy(ctx->ev_stop);
    delete ctx;
    return MACE_HIP_UNSUPPORTED;
  }
  *out = ctx;
  return MACE_HIP_SUCCESS;
}

int mace_hip_ctx_destroy(mace_hip_ctx *ctx) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  if (ctx->plan_only) {
    delete ctx;
    return MACE_HIP_SUCCESS;
  }
  (void)hipSetDevice(ctx->device);
  (void)hipStreamSynchronize(ctx->stream);
  if (ctx->arena) (void)hipFree(ctx->arena);
  for (mh_weight &w : ctx->weights) mh_weight_drop_panels(&w, true, nullptr);
  for (mh_host_weight &w : ctx->host_weights) (void)hipFree(w.dev);
  if (ctx->pinned) (void)hipHostFree(ctx->pinned);
  mh_free_retired(ctx);
  (void)hipEventDestroy(ctx->ev_start);
  (void)hipEventDestroy(ctx->ev_stop);
  for (hipEvent_t e : ctx->prof_ev) (void)hipEventDestroy(e);
  (void)hipStreamDestroy(ctx->own_stream);
  delete ctx;
  return MACE_HIP_SUCCESS;
}

int mace_hip_weight_register(mace_hip_ctx *ctx, const void *device_ptr, size_t bytes) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_CHECK(ctx, device_ptr && bytes > 0, "null or empty weight");
  for (mh_weight &w : ctx->weights)
    if (w.ptr == device_ptr) {   // registered again: whatever was derived from it is stale
      if (!ctx->plan_only) MH_HIP(ctx, hipStreamSynchronize(ctx->stream));
      mh_weight_drop_panels(&w, !ctx->plan_only, ctx->live_graphs > 0 ? &ctx->retired : nullptr);
      w.bytes = bytes;
      return MACE_HIP_SUCCESS;
    }
  ctx->weights.push_back(mh_weight{device_ptr, bytes, {}});
  return MACE_HIP_SUCCESS;
}

int mace_hip_weight_unregister(mace_hip_ctx *ctx, const void *device_ptr) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_NOT_CAPTURING(ctx);
  for (size_t i = 0; i < ctx->weights.size(); ++i)
    if (ctx->weights[i].ptr == device_ptr) {
      // kernels may still read the panels; so may a captured graph, until it is destroyed
      if (!ctx->plan_only) MH_HIP(ctx, hipStreamSynchronize(ctx->stream));
      mh_weight_drop_panels(&ctx->weights[i], !ctx->plan_only,
                            ctx->live_graphs > 0 ? &ctx->retired : nullptr);
      ctx->weights.erase(ctx->weights.begin() + (long)i);
      return MACE_HIP_SUCCESS;
    }
  return mh_fail(ctx, MACE_HIP_INVALID_ARGS, "weight %p is not registered", device_ptr);
}

int mace_hip_host_weight_register(mace_hip_ctx *ctx, const void *host_ptr, size_t bytes) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  MH_CHECK(ctx, host_ptr && bytes > 0, "null or empty weight");
  MH_CHECK(ctx, !ctx->capturing, "a capture is in progress on this context");
  mh_host_weight *w = nullptr;
  for (mh_host_weight &e : ctx->host_weights)
    if (e.host == host_ptr) w = &e;
  if (w && w->bytes != bytes) {   // same address, another size: start over
    MH_RETURN_IF_ERROR(mace_hip_host_weight_unregister(ctx, host_ptr));
    w = nullptr;
  }
  if (!w) {
    void *dev = nullptr;
    const hipError_t e = hipMalloc(&dev, bytes);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      return mh_fail(ctx, MACE_HIP_OUT_OF_RESOURCES, "hipMalloc(%zu) failed: %s", bytes,
                     hipGetErrorString(e));
    }
    ctx->host_weights.push_back(mh_host_weight{host_ptr, bytes, dev});
    w = &ctx->host_weights.back();
  }
  // (registered again: the caller has changed the weight; the copy and whatever the uint8 GEMM
  // derived from it are refreshed)
  MH_HIP(ctx, hipMemcpyAsync(w->dev, host_ptr, bytes, hipMemcpyHostToDevice, ctx->stream));
  MH_HIP(ctx, hipStreamSynchronize(ctx->stream));
  ++ctx->host_weight_uploads;
  return mace_hip_weight_register(ctx, w->dev, bytes);
}

int mace_hip_host_weight_unregister(mace_hip_ctx *ctx, const void *host_ptr) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  MH_NOT_CAPTURING(ctx);
  for (size_t i = 0; i < ctx->host_weights.size(); ++i)
    if (ctx->host_weights[i].host == host_ptr) {
      void *dev = ctx->host_weights[i].dev;
      (void)mace_hip_weight_unregister(ctx, dev);   // synchronizes the stream
      if (ctx->live_graphs > 0) ctx->retired.push_back(dev);
      else (void)hipFree(dev);
      ctx->host_weights.erase(ctx->host_weights.begin() + (long)i);
      return MACE_HIP_SUCCESS;
    }
  return mh_fail(ctx, MACE_HIP_INVALID_ARGS, "host weight %p is not registered", host_ptr);
}

int mace_hip_host_weight_stats(mace_hip_ctx *ctx, int64_t *uploads, int64_t *hits) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  if (uploads) *uploads = ctx->host_weight_uploads;
  if (hits) *hits = ctx->host_weight_hits;
  return MACE_HIP_SUCCESS;
}

int mace_hip_weight_cache_stats(mace_hip_ctx *ctx, int64_t *builds, int64_t *hits) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  if (builds) *builds = ctx->weight_builds;
  if (hits) *hits = ctx->weight_hits;
  return MACE_HIP_SUCCESS;
}

int mace_hip_ctx_set_stream(mace_hip_ctx *ctx, void *hip_stream) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  MH_NOT_CAPTURING(ctx);
  MH_HIP(ctx, hipStreamSynchronize(ctx->stream));
  ctx->stream = hip_stream ? (hipStream_t)hip_stream : ctx->own_stream;
  return MACE_HIP_SUCCESS;
}

int mace_hip_sync(mace_hip_ctx *ctx) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  MH_NOT_CAPTURING(ctx);
  MH_HIP(ctx, hipStreamSynchronize(ctx->stream));
  return MACE_HIP_SUCCESS;
}

const char *mace_hip_last_error(const mace_hip_ctx *ctx) { return ctx ? ctx->err : ""; }

int mace_hip_device_info(mace_hip_ctx *ctx, char *arch, size_t arch_len, int *cu_count,
                         int *lds_bytes) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  if (arch && arch_len) snprintf(arch, arch_len, "%s", ctx->arch);
  if (cu_count) *cu_count = ctx->cu_count;
  if (lds_bytes) *lds_bytes = ctx->lds_bytes;
  return MACE_HIP_SUCCESS;
}

int mace_hip_timer_start(mace_hip_ctx *ctx) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  MH_HIP(ctx, hipEventRecord(ctx->ev_start, ctx->stream));
  return MACE_HIP_SUCCESS;
}

int mace_hip_timer_stop(mace_hip_ctx *ctx, float *elapsed_ms) {
  if (!ctx || !elapsed_ms) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  MH_NOT_CAPTURING(ctx);
  MH_HIP(ctx, hipEventRecord(ctx->ev_stop, ctx->stream));
  MH_HIP(ctx, hipEventSynchronize(ctx->ev_stop));
  MH_HIP(ctx, hipEventElapsedTime(elapsed_ms, ctx->ev_start, ctx->ev_stop));
  return MACE_HIP_SUCCESS;
}

int mace_hip_profile_enable(mace_hip_ctx *ctx, int on) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  if (on && ctx->prof_ev.empty()) {
    ctx->prof_ev.reserve(2 * MH_PROF_RING);
    for (int i = 0; i < 2 * MH_PROF_RING; ++i) {
      hipEvent_t e = nullptr;
      MH_HIP(ctx, hipEventCreate(&e));
      ctx->prof_ev.push_back(e);
    }
  }
  ctx->prof_on = on ? 1 : 0;
  if (on) ctx->prof_count = 0;   // switching off keeps the recorded launches readable
  return MACE_HIP_SUCCESS;
}

int mace_hip_profile_kernel_count(mace_hip_ctx *ctx, int *count) {
  if (!ctx || !count) return MACE_HIP_INVALID_ARGS;
  *count = ctx->prof_count;
  return MACE_HIP_SUCCESS;
}

int mace_hip_profile_kernel_ms(mace_hip_ctx *ctx, int index, float *elapsed_ms) {
  if (!ctx || !elapsed_ms) return MACE_HIP_INVALID_ARGS;
  MH_CHECK(ctx, index >= 0 && index < ctx->prof_count,
           "no timed launch with this index since profiling was enabled");
  MH_CHECK(ctx, index >= ctx->prof_count - MH_PROF_RING,
           "the stopwatch keeps only the most recent launches; this one has been overwritten");
  const int slot = index % MH_PROF_RING;
  MH_HIP(ctx, hipEventSynchronize(ctx->prof_ev[2 * slot + 1]));
  MH_HIP(ctx, hipEventElapsedTime(elapsed_ms, ctx->prof_ev[2 * slot], ctx->prof_ev[2 * slot + 1]));
  return MACE_HIP_SUCCESS;
}

int mace_hip_profile_last_kernel_ms(mace_hip_ctx *ctx, float *elapsed_ms) {
  if (!ctx || !elapsed_ms) return MACE_HIP_INVALID_ARGS;
  MH_CHECK(ctx, ctx->prof_count > 0, "no kernel has been timed since profiling was enabled");
  return mace_hip_profile_kernel_ms(ctx, ctx->prof_count - 1, elapsed_ms);
}

// ---- HIP graphs ---------------------------------------------------------------------------------

struct mace_hip_graph {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
};

int mace_hip_graph_capture_begin(mace_hip_ctx *ctx) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  MH_CHECK(ctx, !ctx->capturing, "a capture is already in progress on this context");
  MH_HIP(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
  ctx->capturing = true;
  return MACE_HIP_SUCCESS;
}

int mace_hip_graph_capture_end(mace_hip_ctx *ctx, mace_hip_graph **out) {
  if (!ctx || !out) return MACE_HIP_INVALID_ARGS;
  *out = nullptr;
  MH_CHECK(ctx, ctx->capturing, "no capture in progress on this context");
  ctx->capturing = false;
  hipGraph_t g = nullptr;
  // (ends the capture also when a call in between has invalidated it: the error comes back here)
  MH_HIP(ctx, hipStreamEndCapture(ctx->stream, &g));
  mace_hip_graph *h = new (std::nothrow) mace_hip_graph();
  if (!h) { (void)hipGraphDestroy(g); return MACE_HIP_OUT_OF_RESOURCES; }
  h->graph = g;
  const hipError_t e = hipGraphInstantiate(&h->exec, g, nullptr, nullptr, 0);
  if (e != hipSuccess) {
    (void)hipGraphDestroy(g);
    delete h;
    MH_HIP(ctx, e);
  }
  *out = h;
  ++ctx->live_graphs;
  return MACE_HIP_SUCCESS;
}

int mace_hip_graph_launch(mace_hip_ctx *ctx, mace_hip_graph *graph) {
  if (!ctx || !graph || !graph->exec) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  MH_CHECK(ctx, !ctx->capturing, "a capture is in progress on this context");
  MH_HIP(ctx, hipGraphLaunch(graph->exec, ctx->stream));
  return MACE_HIP_SUCCESS;
}

int mace_hip_graph_destroy(mace_hip_ctx *ctx, mace_hip_graph *graph) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  if (!graph) return MACE_HIP_SUCCESS;
  MH_HIP(ctx, hipStreamSynchronize(ctx->stream));   // a launch of it may still be running
  if (graph->exec) (void)hipGraphExecDestroy(graph->exec);
  if (graph->graph) (void)hipGraphDestroy(graph->graph);
  delete graph;
  // memory that was kept only because a graph might still replay with its address
  if (ctx->live_graphs > 0 && --ctx->live_graphs == 0) mh_free_retired(ctx);
  return MACE_HIP_SUCCESS;
}

int mace_hip_ctx_set_kernel_mask(mace_hip_ctx *ctx, int mask) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  ctx->kernel_mask = mask;
  return MACE_HIP_SUCCESS;
}

int mace_hip_ctx_fail_next_allocs(mace_hip_ctx *ctx, int n) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  ctx->fail_allocs = n;
  return MACE_HIP_SUCCESS;
}

int mace_hip_malloc(mace_hip_ctx *ctx, size_t bytes, void **dev_ptr) {
  if (!ctx || !dev_ptr) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  *dev_ptr = nullptr;
  if (bytes == 0) return MACE_HIP_SUCCESS;
  hipError_t e = hipMalloc(dev_ptr, bytes);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return mh_fail(ctx, MACE_HIP_OUT_OF_RESOURCES, "hipMalloc(%zu) failed: %s", bytes,
                   hipGetErrorString(e));
  }
  return MACE_HIP_SUCCESS;
}

int mace_hip_free(mace_hip_ctx *ctx, void *dev_ptr) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  MH_NOT_CAPTURING(ctx);
  if (!dev_ptr) return MACE_HIP_SUCCESS;
  MH_HIP(ctx, hipStreamSynchronize(ctx->stream));
  MH_HIP(ctx, hipFree(dev_ptr));
  return MACE_HIP_SUCCESS;
}

int mace_hip_memcpy_h2d(mace_hip_ctx *ctx, void *dst, const void *src, size_t bytes) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  MH_NOT_CAPTURING(ctx);
  if (bytes == 0) return MACE_HIP_SUCCESS;
  MH_HIP(ctx, hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx->stream));
  MH_HIP(ctx, hipStreamSynchronize(ctx->stream));
  return MACE_HIP_SUCCESS;
}

int mace_hip_memcpy_d2h(mace_hip_ctx *ctx, void *dst, const void *src, size_t bytes) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  MH_NOT_CAPTURING(ctx);
  if (bytes == 0) return MACE_HIP_SUCCESS;
  MH_HIP(ctx, hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx->stream));
  MH_HIP(ctx, hipStreamSynchronize(ctx->stream));
  return MACE_HIP_SUCCESS;
}

// ---- quantisation scalars -----------------------------------------------------------------

void mace_hip_quantize_multiplier(double multiplier, int32_t *quantized_multiplier,
                                  int *exponent) {
  int e = 0;
  const double q = frexp(multiplier, &e);
  int64_t qint = (int64_t)roundl((long double)(q * (double)(1ll << 31)));
  if (qint == (1ll << 31)) {
    qint /= 2;
    ++e;
  }
  *quantized_multiplier = (int32_t)qint;
  *exponent = e;
}

int mace_hip_get_output_multiplier_and_shift(float lhs_scale, float rhs_scale,
                                             float output_scale,
                                             int32_t *quantized_multiplier,
                                             int *right_shift) {
  volatile float prod = lhs_scale * rhs_scale;      // binary32, left to right
  volatile float real = prod / output_scale;
  const float r = real;
  if (!(r > 0.f && r < 1.f)) return MACE_HIP_INVALID_ARGS;
  int e = 0;
  mace_hip_quantize_multiplier((double)r, quantized_multiplier, &e);
  *right_shift = -e;
  return *right_shift >= 0 ? MACE_HIP_SUCCESS : MACE_HIP_INVALID_ARGS;
}

uint8_t mace_hip_quantize_u8(float value, float scale, int32_t zero_point) {
  volatile float q = value / scale;
  volatile float s = q + (float)zero_point;
  return mh_saturate_u8(mh_roundf(s));
}

uint8_t mace_hip_requant_fixed_u8(int32_t acc, int32_t multiplier, int right_shift,
                                  int32_t offset_after_shift, int clamp_min, int clamp_max) {
  RequantFixed q;
  if (!mh_make_requant(multiplier, right_shift, offset_after_shift, clamp_min, clamp_max, &q))
    return 0;
  return (uint8_t)mh_requant_fixed(acc, q);
}

int mace_hip_requant_table_u8(int32_t acc, int32_t multiplier, int right_shift,
                              int32_t offset_after_shift, int clamp_min, int clamp_max,
                              uint8_t *out) {
  RequantFixed q;
  if (!out || clamp_min < 0 || clamp_max > 255 || clamp_min > clamp_max ||
      !mh_make_requant(multiplier, right_shift, offset_after_shift, clamp_min, clamp_max, &q))
    return -1;
  if (!q.table) {
    *out = (uint8_t)mh_requant_fixed(acc, q);
    return 0;
  }
  int32_t tab[MH_REQUANT_TABLE_MAX];
  for (int j = 0; j <= q.n + 1; ++j) tab[j] = mh_requant_table_entry(q, j);
  *out = (uint8_t)(q.lo + mh_requant_step(acc, q, tab));
  return 1;
}

uint8_t mace_hip_requant_float_u8(int32_t acc, float multiplier, int32_t out_zp, int mode) {
  return mh_requant_float(acc, multiplier, out_zp, mode == MACE_HIP_REQUANT_NEON);
}

// ---- host-pointer staging --------------------------------------------------------------------

namespace {

inline bool nonneg(int64_t a, int64_t b, int64_t c, int64_t d) {
  return a >= 0 && b >= 0 && c >= 0 && d >= 0;
}

// scratch the device-pointer call itself takes from the arena (generous upper bounds:
// packed copies of both operands plus the correction vectors)
inline size_t q8_gemm_scratch(int64_t batch, int64_t rows, int64_t depth, int64_t cols) {
  const size_t kp = mh_align_up((size_t)depth, 64) + 64;
  return (size_t)batch * ((size_t)rows + (size_t)cols) * (kp + 8) + (1 << 16);
}

}  // namespace

int mace_hip_gemm_f32_host(mace_hip_ctx *ctx, const float *lhs, const float *rhs,
                           int64_t batch, int64_t rows, int64_t cols, int64_t depth,
                           int lhs_major, int rhs_major, int out_major, int lhs_batched,
                           int rhs_batched, float *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  MH_NOT_CAPTURING(ctx);
  MH_CHECK(ctx, nonneg(batch, rows, cols, depth), "negative dimension");
  const size_t lb = sizeof(float) * (lhs_batched ? batch : 1) * rows * depth;
  const size_t rb = sizeof(float) * (rhs_batched ? batch : 1) * depth * cols;
  const size_t ob = sizeof(float) * batch * rows * cols;
  MH_RETURN_IF_ERROR(mh_arena_reserve(ctx, lb + rb + ob + mh_f32_ksplit_bytes(ctx, batch, rows, cols, depth) + 4096));
  Stage st(ctx);
  void *dl, *dr, *dout;
  MH_RETURN_IF_ERROR(st.in(lhs, lb, &dl));
  MH_RETURN_IF_ERROR(st.in(rhs, rb, &dr));
  MH_RETURN_IF_ERROR(st.out(ob, &dout));
  MH_RETURN_IF_ERROR(mace_hip_gemm_f32(ctx, (const float *)dl, (const float *)dr, batch, rows,
                                       cols, depth, lhs_major, rhs_major, out_major,
                                       lhs_batched, rhs_batched, (float *)dout));
  return st.back(out, dout, ob);
}

int mace_hip_gemv_f32_host(mace_hip_ctx *ctx, const float *lhs, const float *rhs,
                           const float *bias, int64_t batch, int64_t height, int64_t width,
                           int lhs_batched, int rhs_batched, float *out) {
  return mace_hip_gemv_f32_act_host(ctx, lhs, rhs, bias, batch, height, width, lhs_batched,
                                    rhs_batched, MACE_HIP_ACT_NOOP, 0.f, out);
}

int mace_hip_gemv_f32_act_host(mace_hip_ctx *ctx, const float *lhs, const float *rhs,
                               const float *bias, int64_t batch, int64_t height, int64_t width,
                               int lhs_batched, int rhs_batched, int activation, float max_limit,
                               float *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  MH_NOT_CAPTURING(ctx);
  MH_CHECK(ctx, nonneg(batch, height, width, 0), "negative dimension");
  const size_t lb = sizeof(float) * (lhs_batched ? batch : 1) * height * width;
  const size_t rb = sizeof(float) * (rhs_batched ? batch : 1) * width;
  const size_t bb = bias ? sizeof(float) * height : 0;
  const size_t ob = sizeof(float) * batch * height;
  MH_RETURN_IF_ERROR(mh_arena_reserve(ctx, lb + rb + bb + ob));
  Stage st(ctx);
  void *dl, *dr, *db, *dout;
  MH_RETURN_IF_ERROR(st.in(lhs, lb, &dl));
  MH_RETURN_IF_ERROR(st.in(rhs, rb, &dr));
  MH_RETURN_IF_ERROR(st.in(bias, bb, &db));
  MH_RETURN_IF_ERROR(st.out(ob, &dout));
  MH_RETURN_IF_ERROR(mace_hip_gemv_f32_act(ctx, (const float *)dl, (const float *)dr,
                                           (const float *)db, batch, height, width, lhs_batched,
                                           rhs_batched, activation, max_limit, (float *)dout));
  return st.back(out, dout, ob);
}

int mace_hip_conv1x1_f32_nchw_host(mace_hip_ctx *ctx, const float *input,
                                   const float *filter, const float *bias, int64_t n,
                                   int64_t cin, int64_t hw, int64_t cout, int activation,
                                   float max_limit, float *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  MH_NOT_CAPTURING(ctx);
  MH_CHECK(ctx, nonneg(n, cin, hw, cout), "negative dimension");
  const size_t ib = sizeof(float) * n * cin * hw;
  const size_t fb = sizeof(float) * cout * cin;
  const size_t bb = bias ? sizeof(float) * cout : 0;
  const size_t ob = sizeof(float) * n * cout * hw;
  MH_RETURN_IF_ERROR(mh_arena_reserve(ctx, ib + fb + bb + ob + mh_f32_ksplit_bytes(ctx, n, cout, hw, cin) + 4096));
  Stage st(ctx);
  void *di, *df, *db, *dout;
  MH_RETURN_IF_ERROR(st.in(input, ib, &di));
  MH_RETURN_IF_ERROR(st.in(filter, fb, &df));
  MH_RETURN_IF_ERROR(st.in(bias, bb, &db));
  MH_RETURN_IF_ERROR(st.out(ob, &dout));
  MH_RETURN_IF_ERROR(mace_hip_conv1x1_f32_nchw(ctx, (const float *)di, (const float *)df,
                                               (const float *)db, n, cin, hw, cout,
                                               activation, max_limit, (float *)dout));
  return st.back(out, dout, ob);
}

int mace_hip_matmul_f32_host(mace_hip_ctx *ctx, const float *lhs, const float *rhs,
                             const float *bias, int64_t batch, int64_t lhs_rows, int64_t lhs_cols,
                             int64_t rhs_rows, int64_t rhs_cols, int transpose_lhs,
                             int transpose_rhs, int lhs_batched, int rhs_batched, float *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  MH_NOT_CAPTURING(ctx);
  MH_CHECK(ctx, nonneg(batch, lhs_rows, lhs_cols, 0) && nonneg(rhs_rows, rhs_cols, 0, 0),
           "negative dimension");
  const int64_t rows = transpose_lhs ? lhs_cols : lhs_rows;
  const int64_t cols = transpose_rhs ? rhs_rows : rhs_cols;
  const size_t lb = sizeof(float) * (lhs_batched ? batch : 1) * lhs_rows * lhs_cols;
  const size_t rb = sizeof(float) * (rhs_batched ? batch : 1) * rhs_rows * rhs_cols;
  const size_t bb = bias ? sizeof(float) * cols : 0;
  const size_t ob = sizeof(float) * batch * rows * cols;
  MH_RETURN_IF_ERROR(mh_arena_reserve(ctx, lb + rb + bb + ob +
                                           mh_f32_ksplit_bytes(ctx, batch, rows, cols, transpose_lhs ? lhs_rows : lhs_cols) + 4096));
  Stage st(ctx);
  void *dl, *dr, *db, *dout;
  MH_RETURN_IF_ERROR(st.in(lhs, lb, &dl));
  MH_RETURN_IF_ERROR(st.in(rhs, rb, &dr));
  MH_RETURN_IF_ERROR(st.in(bias, bb, &db));
  MH_RETURN_IF_ERROR(st.out(ob, &dout));
  MH_RETURN_IF_ERROR(mace_hip_matmul_f32(ctx, (const float *)dl, (const float *)dr,
                                         (const float *)db, batch, lhs_rows, lhs_cols, rhs_rows,
                                         rhs_cols, transpose_lhs, transpose_rhs, lhs_batched,
                                         rhs_batched, (float *)dout));
  return st.back(out, dout, ob);
}

int mace_hip_conv2d_f32_nchw_host(mace_hip_ctx *ctx, const float *input, const float *filter,
                                  const float *bias, int64_t n, int64_t cin, int64_t in_h,
                                  int64_t in_w, int64_t cout, int64_t k_h, int64_t k_w,
                                  int stride_h, int stride_w, int dilation_h, int dilation_w,
                                  int pad_h, int pad_w, int activation, float max_limit,
                                  float *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  MH_NOT_CAPTURING(ctx);
  MH_CHECK(ctx, nonneg(n, cin, in_h, in_w) && nonneg(cout, k_h, k_w, 0) && pad_h >= 0 && pad_w >= 0,
           "negative dimension");
  if (k_h != 1 || k_w != 1 || stride_h != 1 || stride_w != 1 || dilation_h != 1 || dilation_w != 1)
    return mh_fail(ctx, MACE_HIP_UNSUPPORTED,
                   "only 1x1 filters at stride 1, dilation 1 run on the GPU");
  const int64_t ohw = (in_h + pad_h) * (in_w + pad_w);
  const size_t ib = sizeof(float) * n * cin * in_h * in_w;
  const size_t fb = sizeof(float) * cout * cin;
  const size_t bb = bias ? sizeof(float) * cout : 0;
  const size_t ob = sizeof(float) * n * cout * ohw;
  MH_RETURN_IF_ERROR(mh_arena_reserve(ctx, ib + fb + bb + ob + sizeof(float) * n * cin * ohw +
                                           mh_f32_ksplit_bytes(ctx, n, cout, ohw, cin) + 8192));
  Stage st(ctx);
  void *di, *df, *db, *dout;
  MH_RETURN_IF_ERROR(st.in(input, ib, &di));
  MH_RETURN_IF_ERROR(st.in(filter, fb, &df));
  MH_RETURN_IF_ERROR(st.in(bias, bb, &db));
  MH_RETURN_IF_ERROR(st.out(ob, &dout));
  MH_RETURN_IF_ERROR(mace_hip_conv2d_f32_nchw(ctx, (const float *)di, (const float *)df,
                                              (const float *)db, n, cin, in_h, in_w, cout, k_h, k_w,
                                              stride_h, stride_w, dilation_h, dilation_w, pad_h,
                                              pad_w, activation, max_limit, (float *)dout));
  return st.back(out, dout, ob);
}

int mace_hip_gemv_q8_u8_host(mace_hip_ctx *ctx, const uint8_t *lhs, const uint8_t *rhs,
                             const int32_t *bias, int64_t batch, int64_t height,
                             int64_t width, int lhs_batched, int rhs_batched, int32_t lhs_zp,
                             int32_t rhs_zp, float lhs_scale, float rhs_scale,
                             float out_scale, int32_t out_zp, int requant_mode,
                             uint8_t *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  MH_NOT_CAPTURING(ctx);
  MH_CHECK(ctx, nonneg(batch, height, width, 0), "negative dimension");
  const size_t lb = (size_t)(lhs_batched ? batch : 1) * height * width;
  const size_t rb = (size_t)(rhs_batched ? batch : 1) * width;
  const size_t bb = bias ? sizeof(int32_t) * height : 0;
  const size_t ob = (size_t)batch * height;
  MH_RETURN_IF_ERROR(mh_arena_reserve(ctx, lb + rb + bb + ob));
  Stage st(ctx);
  void *dl, *dr, *db, *dout;
  MH_RETURN_IF_ERROR(st.in(lhs, lb, &dl));
  MH_RETURN_IF_ERROR(st.in(rhs, rb, &dr));
  MH_RETURN_IF_ERROR(st.in(bias, bb, &db));
  MH_RETURN_IF_ERROR(st.out(ob, &dout));
  MH_RETURN_IF_ERROR(mace_hip_gemv_q8_u8(ctx, (const uint8_t *)dl, (const uint8_t *)dr,
                                         (const int32_t *)db, batch, height, width,
                                         lhs_batched, rhs_batched, lhs_zp, rhs_zp, lhs_scale,
                                         rhs_scale, out_scale, out_zp, requant_mode,
                                         (uint8_t *)dout));
  return st.back(out, dout, ob);
}

int mace_hip_gemv_q8_i32_host(mace_hip_ctx *ctx, const uint8_t *lhs, const uint8_t *rhs,
                              const int32_t *bias, int64_t batch, int64_t height,
                              int64_t width, int lhs_batched, int rhs_batched,
                              int32_t lhs_zp, int32_t rhs_zp, int32_t *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  MH_NOT_CAPTURING(ctx);
  MH_CHECK(ctx, nonneg(batch, height, width, 0), "negative dimension");
  const size_t lb = (size_t)(lhs_batched ? batch : 1) * height * width;
  const size_t rb = (size_t)(rhs_batched ? batch : 1) * width;
  const size_t bb = bias ? sizeof(int32_t) * height : 0;
  const size_t ob = sizeof(int32_t) * batch * height;
  MH_RETURN_IF_ERROR(mh_arena_reserve(ctx, lb + rb + bb + ob));
  Stage st(ctx);
  void *dl, *dr, *db, *dout;
  MH_RETURN_IF_ERROR(st.in(lhs, lb, &dl));
  MH_RETURN_IF_ERROR(st.in(rhs, rb, &dr));
  MH_RETURN_IF_ERROR(st.in(bias, bb, &db));
  MH_RETURN_IF_ERROR(st.out(ob, &dout));
  MH_RETURN_IF_ERROR(mace_hip_gemv_q8_i32(ctx, (const uint8_t *)dl, (const uint8_t *)dr,
                                          (const int32_t *)db, batch, height, width,
                                          lhs_batched, rhs_batched, lhs_zp, rhs_zp,
                                          (int32_t *)dout));
  return st.back(out, dout, ob);
}

int mace_hip_gemm_q8_i32_host(mace_hip_ctx *ctx, const uint8_t *lhs, int lhs_order,
                              const uint8_t *rhs, int rhs_order, int32_t *out,
                              int out_order, int64_t batch, int64_t rows, int64_t depth,
                              int64_t cols, int lhs_batched, int rhs_batched,
                              int32_t lhs_offset, int32_t rhs_offset) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  MH_NOT_CAPTURING(ctx);
  MH_CHECK(ctx, nonneg(batch, rows, depth, cols), "negative dimension");
  const size_t lb = (size_t)(lhs_batched ? batch : 1) * rows * depth;
  const size_t rb = (size_t)(rhs_batched ? batch : 1) * depth * cols;
  const size_t ob = sizeof(int32_t) * batch * rows * cols;
  MH_RETURN_IF_ERROR(
      mh_arena_reserve(ctx, lb + rb + ob + q8_gemm_scratch(batch, rows, depth, cols)));
  Stage st(ctx);
  void *dl, *dr, *dout;
  MH_RETURN_IF_ERROR(st.in(lhs, lb, &dl));
  MH_RETURN_IF_ERROR(st.in(rhs, rb, &dr));
  MH_RETURN_IF_ERROR(st.out(ob, &dout));
  MH_RETURN_IF_ERROR(mace_hip_gemm_q8_i32(ctx, (const uint8_t *)dl, lhs_order,
                                          (const uint8_t *)dr, rhs_order, (int32_t *)dout,
                                          out_order, batch, rows, depth, cols, lhs_batched,
                                          rhs_batched, lhs_offset, rhs_offset));
  return st.back(out, dout, ob);
}

int mace_hip_gemm_q8_u8_host(mace_hip_ctx *ctx, const uint8_t *lhs, int lhs_order,
                             const uint8_t *rhs, int rhs_order, uint8_t *out, int out_order,
                             int64_t batch, int64_t rows, int64_t depth, int64_t cols,
                             int lhs_batched, int rhs_batched, int32_t lhs_offset,
                             int32_t rhs_offset, const int32_t *bias, int32_t multiplier,
                             int right_shift, int32_t offset_after_shift, int clamp_min,
                             int clamp_max) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  MH_NOT_CAPTURING(ctx);
  MH_CHECK(ctx, nonneg(batch, rows, depth, cols), "negative dimension");
  const size_t lb = (size_t)(lhs_batched ? batch : 1) * rows * depth;
  const size_t rb = (size_t)(rhs_batched ? batch : 1) * depth * cols;
  const size_t bb = bias ? sizeof(int32_t) * rows : 0;
  const size_t ob = (size_t)batch * rows * cols;
  MH_RETURN_IF_ERROR(
      mh_arena_reserve(ctx, lb + rb + bb + ob + q8_gemm_scratch(batch, rows, depth, cols)));
  Stage st(ctx);
  void *dl, *dr, *db, *dout;
  MH_RETURN_IF_ERROR(st.in(lhs, lb, &dl));
  MH_RETURN_IF_ERROR(st.in(rhs, rb, &dr));
  MH_RETURN_IF_ERROR(st.in(bias, bb, &db));
  MH_RETURN_IF_ERROR(st.out(ob, &dout));
  MH_RETURN_IF_ERROR(mace_hip_gemm_q8_u8(ctx, (const uint8_t *)dl, lhs_order,
                                         (const uint8_t *)dr, rhs_order, (uint8_t *)dout,
                                         out_order, batch, rows, depth, cols, lhs_batched,
                                         rhs_batched, lhs_offset, rhs_offset,
                                         (const int32_t *)db, multiplier, right_shift,
                                         offset_after_shift, clamp_min, clamp_max));
  return st.back(out, dout, ob);
}

int mace_hip_gemm_q8_u8_noalloc(mace_hip_ctx *ctx, const uint8_t *lhs, int lhs_order,
                                const uint8_t *rhs, int rhs_order, uint8_t *out, int out_order,
                                int64_t batch, int64_t rows, int64_t depth, int64_t cols,
                                int lhs_batched, int rhs_batched, int32_t lhs_offset,
                                int32_t rhs_offset, const int32_t *bias, int32_t multiplier,
                                int right_shift, int32_t offset_after_shift, int clamp_min,
                                int clamp_max) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  PlanScope plan_scope(ctx);
  MH_CHECK(ctx, ctx->arena_used == 0 && !ctx->no_alloc, "another call is in progress on this context");
  // For the length of this call the arena is this GPU's static array: the repacked panels and
  // the correction vectors go there, the kernels are the ones mace_hip_gemm_q8_u8 launches.
  // Everything taken from it is written before it is read (the panel sums that a repack adds up
  // with atomics are cleared by a kernel first), so what the previous call left does not matter.
  char *const saved_arena = ctx->arena;
  const size_t saved_bytes = ctx->arena_bytes;
  ctx->arena = ctx->static_scratch;
  ctx->arena_bytes = MACE_HIP_NOALLOC_SCRATCH_BYTES;
  ctx->no_alloc = true;
  Q8GemmEpilogue ep{bias, multiplier, right_shift, offset_after_shift, clamp_min, clamp_max};
  const int rc = mh_q8_gemm(ctx, lhs, lhs_order, rhs, rhs_order, out, out_order, true, batch, rows,
                            depth, cols, lhs_batched, rhs_batched, lhs_offset, rhs_offset, ep);
  ctx->no_alloc = false;
  ctx->arena = saved_arena;
  ctx->arena_bytes = saved_bytes;
  ctx->arena_used = 0;
  return rc;
}

int mace_hip_conv1x1_q8_nhwc_host(mace_hip_ctx *ctx, const uint8_t *input,
                                  const uint8_t *filter, const int32_t *bias, int64_t n,
                                  int64_t h, int64_t w, int64_t cin, int64_t cout,
                                  float input_scale, int32_t input_zp, float filter_scale,
                                  int32_t filter_zp, float bias_scale, float out_scale,
                                  int32_t out_zp, int clamp_min, int clamp_max,
                                  uint8_t *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  MH_NOT_CAPTURING(ctx);
  MH_CHECK(ctx, nonneg(n, h, w, 0) && nonneg(cin, cout, 0, 0), "negative dimension");
  const int64_t pix = n * h * w;
  const size_t ib = (size_t)pix * cin, fb = (size_t)cout * cin;
  const size_t bb = bias ? sizeof(int32_t) * cout : 0;
  const size_t ob = (size_t)pix * cout;
  MH_RETURN_IF_ERROR(mh_arena_reserve(
      ctx, ib + fb + bb + ob + q8_gemm_scratch(1, cout, cin, pix) + sizeof(int32_t) * cout));
  Stage st(ctx);
  void *di, *df, *db, *dout;
  MH_RETURN_IF_ERROR(st.in(input, ib, &di));
  MH_RETURN_IF_ERROR(st.in(filter, fb, &df));
  MH_RETURN_IF_ERROR(st.in(bias, bb, &db));
  MH_RETURN_IF_ERROR(st.out(ob, &dout));
  MH_RETURN_IF_ERROR(mace_hip_conv1x1_q8_nhwc(
      ctx, (const uint8_t *)di, (const uint8_t *)df, (const int32_t *)db, n, h, w, cin, cout,
      input_scale, input_zp, filter_scale, filter_zp, bias_scale, out_scale, out_zp,
      clamp_min, clamp_max, (uint8_t *)dout));
  return st.back(out, dout, ob);
}

int mace_hip_conv2d_q8_nhwc_host(mace_hip_ctx *ctx, const uint8_t *input, const uint8_t *filter,
                                 const int32_t *bias, int64_t n, int64_t in_h, int64_t in_w,
                                 int64_t cin, int64_t cout, int64_t k_h, int64_t k_w,
                                 int stride_h, int stride_w, int pad_h, int pad_w,
                                 float input_scale, int32_t input_zp, float filter_scale,
                                 int32_t filter_zp, float bias_scale, float out_scale,
                                 int32_t out_zp, int clamp_min, int clamp_max, uint8_t *out) {
  if (!ctx) return MACE_HIP_INVALID_ARGS;
  MH_NEEDS_GPU(ctx);
  MH_NOT_CAPTURING(ctx);
  MH_CHECK(ctx, nonneg(n, in_h, in_w, 0) && nonneg(cin, cout, 0, 0), "negative dimension");
  MH_CHECK(ctx, k_h >= 1 && k_w >= 1 && stride_h >= 1 && stride_w >= 1 && pad_h >= 0 &&
                    pad_w >= 0, "filter / stride < 1 or negative padding");
  const int64_t num_h = in_h + pad_h - k_h, num_w = in_w + pad_w - k_w;
  MH_CHECK(ctx, num_h >= -stride_h && num_w >= -stride_w, "filter larger than the padded input");
  const int64_t out_h = (num_h >= 0 ? num_h / stride_h : -1) + 1;
  const int64_t out_w = (num_w >= 0 ? num_w / stride_w : -1) + 1;
  const int64_t columns = n * out_h * out_w, depth = k_h * k_w * cin;
  const size_t ib = (size_t)n * in_h * in_w * cin, fb = (size_t)cout * depth;
  const size_t bb = bias ? sizeof(int32_t) * cout : 0;
  const size_t ob = (size_t)columns * cout;
  // staged tensors + the im2col matrix + what the GEMM takes for itself
  MH_RETURN_IF_ERROR(mh_arena_reserve(
      ctx, ib + fb + bb + ob + (size_t)columns * (mh_align_up((size_t)depth + 1, 64) + 8) +
               q8_gemm_scratch(1, cout, depth, 0) + sizeof(int32_t) * (4 * cout + columns) +
               (1 << 17)));
  Stage st(ctx);
  void *di, *df, *db, *dout;
  MH_RETURN_IF_ERROR(st.in(input, ib, &di));
  MH_RETURN_IF_ERROR(st.in(filter, fb, &df));
  MH_RETURN_IF_ERROR(st.in(bias, bb, &db));
  MH_RETURN_IF_ERROR(st.out(ob, &dout));
  MH_RETURN_IF_ERROR(mace_hip_conv2d_q8_nhwc(
      ctx, (const uint8_t *)di, (const uint8_t *)df, (const int32_t *)db, n, in_h, in_w, cin,
      cout, k_h, k_w, stride_h, stride_w, pad_h, pad_w, input_scale, input_zp, filter_scale,
      filter_zp, bias_scale, out_scale, out_zp, clamp_min, clamp_max, (uint8_t *)dout));
  return st.back(out, dout, ob);
}

}  // extern "C"
