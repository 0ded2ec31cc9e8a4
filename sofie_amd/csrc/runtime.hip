// Context, memory and timing entry points of libsofie_hip.so.
#include <stdarg.h>

#include <mutex>
#include <vector>

#include "common.h"

// Scratch memory of the no-allocation entry point (sofie_hip_qgemm_s8_noalloc): a fixed array in the code object,
// one copy per GPU the library is loaded on, held until the process ends. In host code the array's name is only
// a handle for hipGetSymbolAddress: the device address is looked up once per device in sofie_hip_create and kept
// in g_scratch_addr; kernels get that address as an ordinary argument.
static __device__ __align__(256) unsigned char scratch[SOFIE_HIP_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_addr[kMaxDevices] = {};
// One event per device, made with the array's address (so nothing is created at call time): recorded behind the last
// kernel of every no-allocation call and waited for in front of the first kernel of the next one, whatever context
// and stream that call runs on. Calls from different contexts then use the array one after the other.
hipEvent_t g_scratch_free[kMaxDevices] = {};

// With `device` current: the address of this device's copy of `scratch` (looked up at the first call).
hipError_t scratch_address(int device, void **addr)
{
   *addr = nullptr;
   if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
   std::lock_guard<std::mutex> lock(g_scratch_mutex);
   if (!g_scratch_addr[device]) {
      void *p = nullptr;
      hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
      if (e != hipSuccess) return e;
      g_scratch_addr[device] = p;
      if (hipEventCreateWithFlags(&g_scratch_free[device], hipEventDisableTiming) != hipSuccess) {
         (void)hipGetLastError();
         g_scratch_free[device] = nullptr;
      }
   }
   *addr = g_scratch_addr[device];
   return hipSuccess;
}

// Kernels listed by SOFIE_LARGE_LDS (static initialisers of the kernel translation units, so the list lives in a
// function and exists whenever one of them runs) and the devices on which their limit has been raised.
std::vector<const void *> &large_lds_kernels()
{
   static std::vector<const void *> v;
   return v;
}
std::mutex g_lds_mutex;
bool g_lds_done[kMaxDevices] = {};

// With `device` current: raise the dynamic-LDS limit of every listed kernel to what the LDS holds beside the kernel's
// own static arrays, once per device. A kernel whose limit cannot be raised is reported once on stderr and left as it
// is: its launches with more than the default then fail with the runtime's message.
void raise_lds_limits(int device)
{
   if (device < 0 || device >= kMaxDevices) return;
   std::lock_guard<std::mutex> lock(g_lds_mutex);
   if (g_lds_done[device]) return;
   g_lds_done[device] = true;
   for (const void *f : large_lds_kernels()) {
      hipFuncAttributes attr{};
      int limit = sofie::kMaxDynamicLds;
      if (hipFuncGetAttributes(&attr, f) == hipSuccess) limit -= (int)attr.sharedSizeBytes;
      else (void)hipGetLastError();
      const hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, limit);
      if (e != hipSuccess) {
         (void)hipGetLastError();
         fprintf(stderr, "libsofie_hip: dynamic LDS limit of %d bytes refused for a kernel: %s\n", limit, hipGetErrorString(e));
      }
   }
}
}  // namespace

namespace sofie {

// Around the kernels of a no-allocation call: the stream waits for the event of the call that used the array last, and
// records it again behind its own kernels. Both under the lock, so that two threads' calls take turns in one order.
// (Not while the stream is being captured: an event of another stream has no place in the recording; a recorded
// no-allocation call is ordered only against the calls of its own stream.)
void scratch_turn_begin(sofie_hip_ctx *ctx)
{
   g_scratch_mutex.lock();
   hipEvent_t ev = (ctx->device >= 0 && ctx->device < kMaxDevices) ? g_scratch_free[ctx->device] : nullptr;
   if (ev && !ctx->capturing && hipStreamWaitEvent(ctx->stream, ev, 0) != hipSuccess) (void)hipGetLastError();
}

void scratch_turn_end(sofie_hip_ctx *ctx)
{
   hipEvent_t ev = (ctx->device >= 0 && ctx->device < kMaxDevices) ? g_scratch_free[ctx->device] : nullptr;
   if (ev && !ctx->capturing && hipEventRecord(ev, ctx->stream) != hipSuccess) (void)hipGetLastError();
   g_scratch_mutex.unlock();
}

void list_large_lds_kernel(const void *func)
{
   std::lock_guard<std::mutex> lock(g_lds_mutex);
   large_lds_kernels().push_back(func);
}

int set_error(sofie_hip_ctx *ctx, int code, const char *fmt, ...)
{
   if (ctx) {
      va_list ap;
      va_start(ap, fmt);
      vsnprintf(ctx->err, sizeof(ctx->err), fmt, ap);
      va_end(ap);
   }
   return code;
}

unsigned long long layout_key(const int *values, int n)
{
   unsigned long long h = 1469598103934665603ull;      // FNV-1a over the bytes of the values
   for (int i = 0; i < n; ++i)
      for (int b = 0; b < 4; ++b) {
         h ^= (unsigned long long)(((unsigned)values[i] >> (8 * b)) & 0xffu);
         h *= 1099511628211ull;
      }
   return h;
}

int packed_weights(sofie_hip_ctx *ctx, const void *w, unsigned long long key, size_t bytes, void **ptr, bool *fresh)
{
   *fresh = true;
   if (ctx->constant_weights && !ctx->no_alloc) {
      for (int i = 0; i < ctx->packed_len; ++i) {
         const sofie_hip_ctx::PackedWeights &e = ctx->packed[i];
         if (e.w == w && e.key == key && e.bytes == bytes) {
            *ptr = e.packed;
            *fresh = false;
            return SOFIE_HIP_OK;
         }
      }
      // a new tensor: a buffer of its own, unless a graph is being recorded (nothing may allocate then) or the table is full
      if (!ctx->capturing && ctx->packed_len < SOFIE_HIP_PACKED_MAX) {
         if (!ctx->packed) ctx->packed = new sofie_hip_ctx::PackedWeights[SOFIE_HIP_PACKED_MAX];
         void *buf = nullptr;
         if (hipMalloc(&buf, bytes) == hipSuccess) {
            ctx->packed[ctx->packed_len++] = {w, key, bytes, buf};
            *ptr = buf;
            return SOFIE_HIP_OK;
         }
         (void)hipGetLastError();
      }
   }
   return workspace(ctx, bytes, ptr);
}

int workspace(sofie_hip_ctx *ctx, size_t bytes, void **ptr)
{
   if (ctx->no_alloc) {   // inside the no-allocation entry point: the fixed array or nothing
      if (!ctx->static_scratch)
         return set_error(ctx, SOFIE_HIP_EHIP, "the fixed scratch array of this device could not be located when the context was created");
      if (bytes > (size_t)SOFIE_HIP_NOALLOC_SCRATCH_BYTES)
         return set_error(ctx, SOFIE_HIP_EINVAL, "this shape needs %zu bytes of scratch memory; the no-allocation entry "
                          "point holds %zu: use sofie_hip_qgemm_s8", bytes, (size_t)SOFIE_HIP_NOALLOC_SCRATCH_BYTES);
      *ptr = ctx->static_scratch;
      return SOFIE_HIP_OK;
   }
   if (bytes > ctx->workspace_bytes) {
      if (ctx->capturing)
         return set_error(ctx, SOFIE_HIP_EINVAL, "the scratch buffer would grow to %zu bytes while a graph is captured: "
                          "run the same calls once before capturing", bytes);
      // a recorded graph keeps the address of the buffer it was recorded with: freeing it would leave the next
      // replay reading and writing freed device memory
      if (ctx->live_graphs > 0)
         return set_error(ctx, SOFIE_HIP_EINVAL, "the scratch buffer would grow to %zu bytes while %d recorded graph(s) of "
                          "this context still use the present one: destroy them first", bytes, ctx->live_graphs);
      // the old buffer may still be read by kernels in flight on the stream
      if (ctx->workspace) {
         SOFIE_HIP_CALL(ctx, hipStreamSynchronize(ctx->stream));
         SOFIE_HIP_CALL(ctx, hipFree(ctx->workspace));
         ctx->workspace = nullptr;
         ctx->workspace_bytes = 0;
      }
      size_t want = bytes + (bytes >> 2);
      if (hipMalloc(&ctx->workspace, want) != hipSuccess) {
         (void)hipGetLastError();
         return set_error(ctx, SOFIE_HIP_ENOMEM, "workspace of %zu bytes", want);
      }
      ctx->workspace_bytes = want;
   }
   *ptr = ctx->workspace;
   return SOFIE_HIP_OK;
}

int check_launch(sofie_hip_ctx *ctx, const char *what)
{
   hipError_t e = hipGetLastError();
   if (e != hipSuccess)
      return set_error(ctx, SOFIE_HIP_EHIP, "launch of %s failed: %s", what, hipGetErrorString(e));
   if (ctx->tracing) {
      ++ctx->trace_seen;
      if (ctx->trace_len <= SOFIE_HIP_TRACE_MAX) {
         hipEvent_t ev = nullptr;
         if (hipEventCreate(&ev) == hipSuccess && hipEventRecord(ev, ctx->stream) == hipSuccess) {
            ctx->trace[ctx->trace_len].what = what;
            ctx->trace[ctx->trace_len].done = ev;
            ++ctx->trace_len;
         } else {
            (void)hipGetLastError();
            if (ev) (void)hipEventDestroy(ev);
         }
      }
   }
   return SOFIE_HIP_OK;
}

}  // namespace sofie

static void drop_trace(sofie_hip_ctx *ctx)
{
   for (int i = 0; i < ctx->trace_len; ++i) (void)hipEventDestroy(ctx->trace[i].done);
   delete[] ctx->trace;
   ctx->trace = nullptr;
   ctx->trace_len = 0;
   ctx->tracing = false;
}

extern "C" {

int sofie_hip_version(void) { return 1; }

int sofie_hip_create(sofie_hip_ctx **out, int device, void *stream)
{
   if (!out) return SOFIE_HIP_EINVAL;
   *out = nullptr;
   int count = 0;
   if (hipGetDeviceCount(&count) != hipSuccess || device < 0 || device >= count) return SOFIE_HIP_EHIP;
   if (hipSetDevice(device) != hipSuccess) return SOFIE_HIP_EHIP;
   sofie_hip_ctx *ctx = new sofie_hip_ctx();
   ctx->device = device;
   {
      int cus = 0;
      if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && cus > 0)
         ctx->num_cus = cus;
   }
   raise_lds_limits(device);
   if (hipError_t e = scratch_address(device, &ctx->static_scratch); e != hipSuccess) {
      // only the no-allocation entry point needs it: that call then fails with this message
      (void)hipGetLastError();
      ctx->static_scratch = nullptr;
   }
   if (stream) {
      ctx->stream = static_cast<hipStream_t>(stream);
   } else {
      if (hipStreamCreate(&ctx->stream) != hipSuccess) { delete ctx; return SOFIE_HIP_EHIP; }
      ctx->owns_stream = true;
   }
   if (hipEventCreate(&ctx->ev_start) != hipSuccess || hipEventCreate(&ctx->ev_stop) != hipSuccess) {
      if (ctx->owns_stream) (void)hipStreamDestroy(ctx->stream);
      delete ctx;
      return SOFIE_HIP_EHIP;
   }
   *out = ctx;
   return SOFIE_HIP_OK;
}

int sofie_hip_destroy(sofie_hip_ctx *ctx)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   if (ctx->capturing) {   // an open recording is given up: a capturing stream cannot be waited for
      hipGraph_t dropped = nullptr;
      (void)hipStreamEndCapture(ctx->stream, &dropped);
      if (dropped) (void)hipGraphDestroy(dropped);
      (void)hipGetLastError();
      ctx->capturing = false;
   }
   (void)hipStreamSynchronize(ctx->stream);
   if (ctx->trace) drop_trace(ctx);
   if (ctx->workspace) (void)hipFree(ctx->workspace);
   for (int i = 0; i < ctx->packed_len; ++i) (void)hipFree(ctx->packed[i].packed);
   delete[] ctx->packed;
   (void)hipEventDestroy(ctx->ev_start);
   (void)hipEventDestroy(ctx->ev_stop);
   if (ctx->owns_stream) (void)hipStreamDestroy(ctx->stream);
   delete ctx;
   return SOFIE_HIP_OK;
}

int sofie_hip_constant_weights(sofie_hip_ctx *ctx, int on)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, !ctx->capturing, "not allowed between capture_begin and capture_end");
   // a recorded graph may hold the address of a kept copy
   SOFIE_REQUIRE(ctx, on || ctx->live_graphs == 0 || ctx->packed_len == 0, "recorded graphs of this context may still use the kept copies: destroy them first");
   ctx->constant_weights = on != 0;
   if (!on && ctx->packed_len > 0) {
      SOFIE_HIP_CALL(ctx, hipStreamSynchronize(ctx->stream));      // kernels in flight may still read them
      for (int i = 0; i < ctx->packed_len; ++i) (void)hipFree(ctx->packed[i].packed);
      ctx->packed_len = 0;
   }
   return SOFIE_HIP_OK;
}

const char *sofie_hip_last_error(const sofie_hip_ctx *ctx) { return ctx ? ctx->err : "null context"; }

int sofie_hip_malloc(sofie_hip_ctx *ctx, void **dptr, size_t bytes)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, !ctx->capturing, "not allowed between capture_begin and capture_end");
   SOFIE_REQUIRE(ctx, dptr != nullptr, "null result pointer");
   *dptr = nullptr;
   if (bytes == 0) return SOFIE_HIP_OK;
   if (hipMalloc(dptr, bytes) != hipSuccess) {
      (void)hipGetLastError();
      return sofie::set_error(ctx, SOFIE_HIP_ENOMEM, "sofie_hip_malloc: %zu bytes", bytes);
   }
   return SOFIE_HIP_OK;
}

int sofie_hip_free(sofie_hip_ctx *ctx, void *dptr)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, !ctx->capturing, "not allowed between capture_begin and capture_end");
   if (!dptr) return SOFIE_HIP_OK;
   SOFIE_HIP_CALL(ctx, hipStreamSynchronize(ctx->stream));
   SOFIE_HIP_CALL(ctx, hipFree(dptr));
   return SOFIE_HIP_OK;
}

int sofie_hip_host_malloc(sofie_hip_ctx *ctx, void **hptr, size_t bytes)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, !ctx->capturing, "not allowed between capture_begin and capture_end");
   SOFIE_REQUIRE(ctx, hptr != nullptr, "null result pointer");
   *hptr = nullptr;
   if (bytes == 0) return SOFIE_HIP_OK;
   if (hipHostMalloc(hptr, bytes, hipHostMallocDefault) != hipSuccess) {
      (void)hipGetLastError();
      *hptr = nullptr;
      return sofie::set_error(ctx, SOFIE_HIP_ENOMEM, "sofie_hip_host_malloc: %zu bytes of page-locked memory", bytes);
   }
   return SOFIE_HIP_OK;
}

int sofie_hip_host_free(sofie_hip_ctx *ctx, void *hptr)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   if (!hptr) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, !ctx->capturing, "not allowed between capture_begin and capture_end");
   SOFIE_HIP_CALL(ctx, hipStreamSynchronize(ctx->stream));   // a copy from or into the buffer may still run
   SOFIE_HIP_CALL(ctx, hipHostFree(hptr));
   return SOFIE_HIP_OK;
}

int sofie_hip_upload(sofie_hip_ctx *ctx, void *dst, const void *src, size_t bytes)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, !ctx->capturing, "not allowed between capture_begin and capture_end");
   if (bytes == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, dst && src, "null pointer");
   SOFIE_HIP_CALL(ctx, hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx->stream));
   SOFIE_HIP_CALL(ctx, hipStreamSynchronize(ctx->stream));
   return SOFIE_HIP_OK;
}

int sofie_hip_download(sofie_hip_ctx *ctx, void *dst, const void *src, size_t bytes)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, !ctx->capturing, "not allowed between capture_begin and capture_end");
   if (bytes == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, dst && src, "null pointer");
   SOFIE_HIP_CALL(ctx, hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx->stream));
   SOFIE_HIP_CALL(ctx, hipStreamSynchronize(ctx->stream));
   return SOFIE_HIP_OK;
}

int sofie_hip_copy(sofie_hip_ctx *ctx, void *dst, const void *src, size_t bytes)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   if (bytes == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, dst && src, "null pointer");
   SOFIE_HIP_CALL(ctx, hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, ctx->stream));
   return SOFIE_HIP_OK;
}

int sofie_hip_memset(sofie_hip_ctx *ctx, void *dptr, int value, size_t bytes)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, !ctx->capturing, "not allowed between capture_begin and capture_end");
   if (bytes == 0) return SOFIE_HIP_OK;
   SOFIE_REQUIRE(ctx, dptr != nullptr, "null pointer");
   SOFIE_HIP_CALL(ctx, hipMemsetAsync(dptr, value, bytes, ctx->stream));
   return SOFIE_HIP_OK;
}

int sofie_hip_sync(sofie_hip_ctx *ctx)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, !ctx->capturing, "not allowed between capture_begin and capture_end");
   SOFIE_HIP_CALL(ctx, hipStreamSynchronize(ctx->stream));
   return SOFIE_HIP_OK;
}

// ---- HIP graphs: a fixed sequence of calls recorded once and replayed with one launch -----------------------
struct sofie_hip_graph {
   hipGraph_t graph = nullptr;
   hipGraphExec_t exec = nullptr;
};

int sofie_hip_capture_begin(sofie_hip_ctx *ctx)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, !ctx->capturing, "a capture is already open on this context");
   SOFIE_REQUIRE(ctx, !ctx->tracing, "a trace is open on this context: events cannot be recorded into a graph");
   SOFIE_HIP_CALL(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed));
   ctx->capturing = true;
   return SOFIE_HIP_OK;
}

int sofie_hip_capture_end(sofie_hip_ctx *ctx, sofie_hip_graph **out)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, ctx->capturing, "no capture is open on this context");
   ctx->capturing = false;
   hipGraph_t graph = nullptr;
   SOFIE_HIP_CALL(ctx, hipStreamEndCapture(ctx->stream, &graph));
   if (!out) {   // the caller gives the recording up (an error in between)
      if (graph) (void)hipGraphDestroy(graph);
      return SOFIE_HIP_OK;
   }
   *out = nullptr;
   SOFIE_REQUIRE(ctx, graph != nullptr, "the capture recorded nothing");
   hipGraphExec_t exec = nullptr;
   if (hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0) != hipSuccess) {
      (void)hipGetLastError();
      (void)hipGraphDestroy(graph);
      return sofie::set_error(ctx, SOFIE_HIP_EHIP, "hipGraphInstantiate failed");
   }
   sofie_hip_graph *g = new sofie_hip_graph();
   g->graph = graph;
   g->exec = exec;
   *out = g;
   ++ctx->live_graphs;
   return SOFIE_HIP_OK;
}

int sofie_hip_graph_launch(sofie_hip_ctx *ctx, sofie_hip_graph *g)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, g && g->exec, "null graph");
   SOFIE_REQUIRE(ctx, !ctx->capturing, "a capture is open on this context");
   SOFIE_HIP_CALL(ctx, hipGraphLaunch(g->exec, ctx->stream));
   return SOFIE_HIP_OK;
}

int sofie_hip_graph_destroy(sofie_hip_ctx *ctx, sofie_hip_graph *g)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, !ctx->capturing, "not allowed between capture_begin and capture_end");
   if (!g) return SOFIE_HIP_OK;
   (void)hipStreamSynchronize(ctx->stream);
   if (g->exec) (void)hipGraphExecDestroy(g->exec);
   if (g->graph) (void)hipGraphDestroy(g->graph);
   delete g;
   if (ctx->live_graphs > 0) --ctx->live_graphs;
   return SOFIE_HIP_OK;
}

int sofie_hip_trace_begin(sofie_hip_ctx *ctx)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, !ctx->capturing, "not allowed between capture_begin and capture_end");
   SOFIE_REQUIRE(ctx, !ctx->tracing, "a trace is already open on this context");
   ctx->trace = new sofie_hip_ctx::TracePoint[SOFIE_HIP_TRACE_MAX + 1];
   ctx->trace_len = 0;
   ctx->trace_seen = 0;
   hipEvent_t ev = nullptr;
   if (hipEventCreate(&ev) != hipSuccess || hipEventRecord(ev, ctx->stream) != hipSuccess) {
      (void)hipGetLastError();
      if (ev) (void)hipEventDestroy(ev);
      drop_trace(ctx);
      return sofie::set_error(ctx, SOFIE_HIP_EHIP, "sofie_hip_trace_begin: the start event could not be recorded");
   }
   ctx->trace[0].what = "";
   ctx->trace[0].done = ev;
   ctx->trace_len = 1;
   ctx->tracing = true;
   return SOFIE_HIP_OK;
}

int sofie_hip_trace_end(sofie_hip_ctx *ctx, char *text, size_t capacity, int *launches)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, ctx->tracing, "no trace is open on this context");
   SOFIE_REQUIRE(ctx, !ctx->capturing, "not allowed between capture_begin and capture_end");
   ctx->tracing = false;
   if (launches) *launches = ctx->trace_seen;
   if (text && capacity) text[0] = 0;
   hipError_t e = hipStreamSynchronize(ctx->stream);
   size_t used = 0;
   for (int i = 1; i < ctx->trace_len && e == hipSuccess; ++i) {
      float ms = 0.0f;
      e = hipEventElapsedTime(&ms, ctx->trace[i - 1].done, ctx->trace[i].done);
      if (e != hipSuccess || !text || used + 1 >= capacity) continue;
      const int n = snprintf(text + used, capacity - used, "%s %.3f\n", ctx->trace[i].what, ms * 1e3);
      if (n < 0 || (size_t)n >= capacity - used) {
         text[used] = 0;       // the line does not fit: the text ends in front of it
         used = capacity;
      } else {
         used += (size_t)n;
      }
   }
   drop_trace(ctx);
   if (e != hipSuccess) return sofie::set_error(ctx, SOFIE_HIP_EHIP, "sofie_hip_trace_end: %s", hipGetErrorString(e));
   return SOFIE_HIP_OK;
}

int sofie_hip_timer_start(sofie_hip_ctx *ctx)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, !ctx->capturing, "not allowed between capture_begin and capture_end");
   SOFIE_HIP_CALL(ctx, hipEventRecord(ctx->ev_start, ctx->stream));
   return SOFIE_HIP_OK;
}

int sofie_hip_timer_stop(sofie_hip_ctx *ctx, float *ms)
{
   if (!ctx) return SOFIE_HIP_EINVAL;
   SOFIE_REQUIRE(ctx, !ctx->capturing, "not allowed between capture_begin and capture_end");
   SOFIE_REQUIRE(ctx, ms != nullptr, "null result pointer");
   SOFIE_HIP_CALL(ctx, hipEventRecord(ctx->ev_stop, ctx->stream));
   SOFIE_HIP_CALL(ctx, hipEventSynchronize(ctx->ev_stop));
   SOFIE_HIP_CALL(ctx, hipEventElapsedTime(ms, ctx->ev_start, ctx->ev_stop));
   return SOFIE_HIP_OK;
}

}  // extern "C"
