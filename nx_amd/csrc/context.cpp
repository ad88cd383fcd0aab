// Context, device buffers and transfers of libhipnx (host code only, no kernels).
//
// The buffer life-cycle follows what the reference's device backends expose to Elixir:
// explicit, idempotent deallocation that reports :ok / :already_deallocated
// (torchx/c_src/torchx_nif_util.h:66-111, torchx/test/torchx/device_test.exs:30-37) and a
// use-after-free that is an error, not a crash (exla/test/exla/backend_test.exs:48-50).
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <system_error>
#include <thread>

#include "internal.h"

namespace hipnx {

static thread_local char g_err[512] = "";

int set_error(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof g_err, fmt, ap);
  va_end(ap);
  return code;
}

int hip_fail(hipError_t e, const char *what) {
  (void)hipGetLastError();  // clear the sticky error so later calls report their own
  return set_error(e == hipErrorOutOfMemory ? HIPNX_ENOMEM : HIPNX_EHIP, "HIP error %d (%s) in %s",
                   (int)e, hipGetErrorString(e), what);
}

int check_buf(const hipnx_ctx *ctx, const hipnx_buf *b, uint64_t need_bytes, const char *name) {
  if (!b) return set_error(HIPNX_EINVAL, "%s: null buffer handle", name);
  if (b->freed.load()) return set_error(HIPNX_EFREED, "%s: buffer has been deallocated", name);
  if (b->ctx != ctx) return set_error(HIPNX_EINVAL, "%s: buffer belongs to another context", name);
  if (b->bytes < need_bytes)
    return set_error(HIPNX_EINVAL, "%s: buffer holds %zu bytes, the shape needs %llu", name, b->bytes,
                     (unsigned long long)need_bytes);
  return HIPNX_OK;
}

Enter::Enter(hipnx_ctx *ctx) : status(HIPNX_OK) {
  if (!ctx) {
    status = set_error(HIPNX_EINVAL, "null context");
    return;
  }
  lk = std::unique_lock<std::mutex>(ctx->mu);
  hipError_t e = hipSetDevice(ctx->device);
  if (e != hipSuccess) status = hip_fail(e, "hipSetDevice");
}

static uint64_t pool_cap_bytes() {
  static uint64_t cap = [] {
    const char *s = getenv("HIPNX_POOL_MAX_MB");
    uint64_t mb = s ? strtoull(s, nullptr, 10) : 32768ull;
    return mb << 20;
  }();
  return cap;
}

static size_t round_capacity(size_t bytes) {
  if (bytes == 0) bytes = 1;
  if (bytes <= (1u << 20)) return (bytes + 255) & ~size_t(255);
  return (bytes + ((1u << 20) - 1)) & ~size_t((1u << 20) - 1);
}

// Both run with the context mutex held.
int pool_alloc(hipnx_ctx *ctx, size_t bytes, void **ptr_out, size_t *cap_out) {
  size_t cap = round_capacity(bytes);
  void *ptr = nullptr;
  if (ctx->capture) {  // blocks released earlier in this capture come first: they already belong to the graph
    auto own = ctx->capture->parked.lower_bound(cap);
    if (own != ctx->capture->parked.end() && own->first <= cap + cap / 4) {
      *ptr_out = own->second;
      *cap_out = own->first;
      ctx->live += own->first;
      if (ctx->live > ctx->peak) ctx->peak = ctx->live;
      ctx->capture->parked.erase(own);
      return HIPNX_OK;
    }
  }
  auto it = ctx->pool.lower_bound(cap);
  if (it != ctx->pool.end() && it->first <= cap + cap / 4) {
    ptr = it->second;
    cap = it->first;
    ctx->pooled -= cap;
    ctx->pool.erase(it);
  } else {
    hipError_t e = hipMalloc(&ptr, cap);
    if (e != hipSuccess && !ctx->pool.empty() && !ctx->capture) {
      // give cached blocks back and retry once
      (void)hipGetLastError();
      (void)hipStreamSynchronize(ctx->stream);
      int refused = 0;
      hipError_t first_refusal = hipSuccess;
      for (auto &kv : ctx->pool) {
        const hipError_t f = hipFree(kv.second);
        if (f != hipSuccess) {
          if (!refused++) first_refusal = f;
          (void)hipGetLastError();
        }
      }
      const size_t handed_back = ctx->pool.size();
      ctx->pool.clear();
      ctx->pooled = 0;
      e = hipMalloc(&ptr, cap);
      // hipFree returns before the driver has the memory back (observed: a third of a second after freeing 30 GiB): give
      // it up to a second, as long as what it reports free is short of the request
      for (int spin = 0; e == hipErrorOutOfMemory && handed_back > 0 && spin < 50; spin++) {
        (void)hipGetLastError();
        std::this_thread::sleep_for(std::chrono::milliseconds(20));
        e = hipMalloc(&ptr, cap);
      }
      if (e != hipSuccess) {
        (void)hipGetLastError();
        return set_error(e == hipErrorOutOfMemory ? HIPNX_ENOMEM : HIPNX_EHIP,
                         "HIP error %d (%s) in hipMalloc of %zu bytes, after %zu pooled blocks went back to the device (hipFree refused %d of them, first with error %d)",
                         (int)e, hipGetErrorString(e), cap, handed_back, refused, (int)first_refusal);
      }
    }
    if (e != hipSuccess) return hip_fail(e, "hipMalloc");
  }
  ctx->live += cap;
  if (ctx->live > ctx->peak) ctx->peak = ctx->live;
  if (ctx->capture) {
    ctx->capture->owned.emplace_back(ptr, cap);
    ctx->graph_blocks[ptr] = ctx->capture;
  }
  *ptr_out = ptr;
  *cap_out = cap;
  return HIPNX_OK;
}

int pool_free(hipnx_ctx *ctx, void *ptr, size_t cap) {
  ctx->live -= cap;
  auto owner = ctx->graph_blocks.find(ptr);
  if (owner != ctx->graph_blocks.end()) {  // stays with its graph, whenever it is released
    owner->second->parked.emplace(cap, ptr);
    return HIPNX_OK;
  }
  if (ctx->pooled + cap <= pool_cap_bytes() || ctx->capture) {
    // reuse without a device wait is safe: all work of this context is ordered on one stream
    ctx->pool.emplace(cap, ptr);
    ctx->pooled += cap;
    return HIPNX_OK;
  }
  HIPNX_HIP(hipStreamSynchronize(ctx->stream));
  HIPNX_HIP(hipFree(ptr));
  return HIPNX_OK;
}

// codes: HIPNX_RAISE_* of elementwise_ops.cuh (kept in step by value)
int deferred_error(hipnx_ctx *ctx) {
  volatile unsigned long long *word = (volatile unsigned long long *)((char *)ctx->flag_host + 16);
  const unsigned long long w = *word;
  if (w == 0) return HIPNX_OK;
  *word = 0;
  const int code = (int)(w >> 56);
  long long operand = (long long)(w << 8) >> 8;  // sign-extend the low 56 bits
  switch (code) {
    case 1: return set_error(HIPNX_ERAISED, "ArithmeticError: bad argument in arithmetic expression (raised late: an earlier quotient / remainder on this context divided by zero)");
    case 2: return set_error(HIPNX_ERAISED, "ArgumentError: cannot left shift by %lld (raised late: an earlier left_shift on this context)", operand);
    case 3: return set_error(HIPNX_ERAISED, "ArgumentError: cannot right shift by %lld (raised late: an earlier right_shift on this context)", operand);
    case 4: return set_error(HIPNX_ERAISED, "ArithmeticError: bad argument in arithmetic expression (raised late: an earlier integer pow on this context had the negative exponent %lld)", operand);
    case 5: return set_error(HIPNX_ERAISED, "ArgumentError: errors were found at the given arguments: not a number (raised late: an earlier float remainder on this context met a non-finite element)");
    case 6: return set_error(HIPNX_ERAISED, "ArgumentError: index %lld is out of bounds (raised late: an earlier gather / take on this context with the deferred bounds policy)", operand);
  }
  return set_error(HIPNX_ERAISED, "an earlier kernel on this context recorded error code %d", code);
}

}  // namespace hipnx

using namespace hipnx;

extern "C" {

int hipnx_last_error(char *dst, size_t cap) {
  if (!dst || cap == 0) return HIPNX_EINVAL;
  snprintf(dst, cap, "%s", g_err);
  return HIPNX_OK;
}

int hipnx_device_count(int *count) {
  if (!count) return set_error(HIPNX_EINVAL, "null count");
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    n = 0;
  }
  *count = n;
  return HIPNX_OK;
}

int hipnx_ctx_create(int device, hipnx_ctx **out) {
  if (!out) return set_error(HIPNX_EINVAL, "null out");
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess || n == 0) {
    (void)hipGetLastError();
    return set_error(HIPNX_EHIP, "no HIP device available");
  }
  if (device < 0 || device >= n) return set_error(HIPNX_EINVAL, "device %d out of range (0..%d)", device, n - 1);
  HIPNX_HIP(hipSetDevice(device));
  hipnx_ctx *ctx = new hipnx_ctx;
  ctx->device = device;
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, device) == hipSuccess) ctx->num_cus = prop.multiProcessorCount;
  hipError_t e1 = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
  hipError_t e2 = hipEventCreate(&ctx->ev_start);
  hipError_t e3 = hipEventCreate(&ctx->ev_stop);
  hipError_t e4 = hipMalloc(&ctx->flag, 256);
  hipError_t e5 = hipHostMalloc(&ctx->flag_host, 256, hipHostMallocMapped);
  if (e5 == hipSuccess) {
    std::memset(ctx->flag_host, 0, 256);
    e5 = hipHostGetDevicePointer(&ctx->flag_host_dev, ctx->flag_host, 0);
  }
  if (e4 == hipSuccess) e4 = hipMemset(ctx->flag, 0xFF, 256);  // gather bounds word: all-ones = no bad index
  if (e1 != hipSuccess || e2 != hipSuccess || e3 != hipSuccess || e4 != hipSuccess || e5 != hipSuccess) {
    hipnx_ctx_destroy(ctx);
    return hip_fail(e1 != hipSuccess ? e1 : e2 != hipSuccess ? e2 : e3 != hipSuccess ? e3 : e4 != hipSuccess ? e4 : e5,
                    "context set-up");
  }
  if (int st = reduce_static_init(ctx)) {
    hipnx_ctx_destroy(ctx);
    return st;
  }
  *out = ctx;
  return HIPNX_OK;
}

int hipnx_ctx_destroy(hipnx_ctx *ctx) {
  if (!ctx) return set_error(HIPNX_EINVAL, "null context");
  (void)hipSetDevice(ctx->device);
  if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
  for (hipnx_graph *g : ctx->graphs) {  // handles to them are dead from here on, like buffer handles
    if (g->exec) (void)hipGraphExecDestroy(g->exec);
    if (g->graph) (void)hipGraphDestroy(g->graph);
    for (auto &kv : g->parked) (void)hipFree(kv.second);
    delete g;
  }
  ctx->graphs.clear();
  for (auto &kv : ctx->fused_kernels) (void)hipModuleUnload(kv.second.module);
  ctx->fused_kernels.clear();
  for (auto &kv : ctx->pool) (void)hipFree(kv.second);
  ctx->pool.clear();
  if (ctx->flag) (void)hipFree(ctx->flag);
  if (ctx->flag_host) (void)hipHostFree(ctx->flag_host);
  for (int i = 0; i < 4; i++) {
    if (ctx->stage[i]) (void)hipHostFree(ctx->stage[i]);
    if (ctx->stage_ev[i]) (void)hipEventDestroy(ctx->stage_ev[i]);
  }
  if (ctx->ev_start) (void)hipEventDestroy(ctx->ev_start);
  if (ctx->ev_stop) (void)hipEventDestroy(ctx->ev_stop);
  for (hipEvent_t m : ctx->marks)
    if (m) (void)hipEventDestroy(m);
  if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
  delete ctx;
  return HIPNX_OK;
}

int hipnx_sync(hipnx_ctx *ctx) {
  Enter in(ctx);
  if (in.status) return in.status;
  HIPNX_NOT_CAPTURING(ctx, "sync");
  HIPNX_HIP(hipStreamSynchronize(ctx->stream));
  return deferred_error(ctx);
}

int hipnx_mem_stats(hipnx_ctx *ctx, uint64_t *live, uint64_t *peak, uint64_t *pooled) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (live) *live = ctx->live;
  if (peak) *peak = ctx->peak;
  if (pooled) *pooled = ctx->pooled;
  return HIPNX_OK;
}

int hipnx_trim(hipnx_ctx *ctx) {
  Enter in(ctx);
  if (in.status) return in.status;
  HIPNX_NOT_CAPTURING(ctx, "trim");
  HIPNX_HIP(hipStreamSynchronize(ctx->stream));
  for (auto &kv : ctx->pool) (void)hipFree(kv.second);
  ctx->pool.clear();
  ctx->pooled = 0;
  return HIPNX_OK;
}

int hipnx_timer_start(hipnx_ctx *ctx) {
  Enter in(ctx);
  if (in.status) return in.status;
  HIPNX_NOT_CAPTURING(ctx, "timer");
  HIPNX_HIP(hipEventRecord(ctx->ev_start, ctx->stream));
  return HIPNX_OK;
}

int hipnx_timer_stop(hipnx_ctx *ctx, float *elapsed_ms) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (!elapsed_ms) return set_error(HIPNX_EINVAL, "null elapsed_ms");
  HIPNX_NOT_CAPTURING(ctx, "timer");
  HIPNX_HIP(hipEventRecord(ctx->ev_stop, ctx->stream));
  HIPNX_HIP(hipEventSynchronize(ctx->ev_stop));
  HIPNX_HIP(hipEventElapsedTime(elapsed_ms, ctx->ev_start, ctx->ev_stop));
  return deferred_error(ctx);
}

int hipnx_timer_mark(hipnx_ctx *ctx, int index) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (index < 0 || index > 65535) return set_error(HIPNX_EINVAL, "timer mark %d out of range (0..65535)", index);
  HIPNX_NOT_CAPTURING(ctx, "timer");
  if ((size_t)index >= ctx->marks.size()) ctx->marks.resize((size_t)index + 1, nullptr);
  if (!ctx->marks[index]) HIPNX_HIP(hipEventCreate(&ctx->marks[index]));
  HIPNX_HIP(hipEventRecord(ctx->marks[index], ctx->stream));
  return HIPNX_OK;
}

int hipnx_timer_between(hipnx_ctx *ctx, int from, int to, float *elapsed_ms) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (!elapsed_ms) return set_error(HIPNX_EINVAL, "null elapsed_ms");
  const int n = (int)ctx->marks.size();
  if (from < 0 || to < 0 || from >= n || to >= n || !ctx->marks[from] || !ctx->marks[to])
    return set_error(HIPNX_EINVAL, "timer marks %d / %d were never recorded", from, to);
  HIPNX_NOT_CAPTURING(ctx, "timer");
  HIPNX_HIP(hipEventSynchronize(ctx->marks[to]));
  HIPNX_HIP(hipEventElapsedTime(elapsed_ms, ctx->marks[from], ctx->marks[to]));
  return deferred_error(ctx);
}

// ---- captured graphs -------------------------------------------------------------------------

static void release_graph(hipnx_ctx *ctx, hipnx_graph *g) {
  for (auto &blk : g->owned) ctx->graph_blocks.erase(blk.first);
  for (auto &kv : g->parked) {  // blocks still held by buffers go to the pool when those are freed
    ctx->pool.emplace(kv.first, kv.second);
    ctx->pooled += kv.first;
  }
  for (size_t i = 0; i < ctx->graphs.size(); i++)
    if (ctx->graphs[i] == g) { ctx->graphs.erase(ctx->graphs.begin() + i); break; }
  if (g->exec) (void)hipGraphExecDestroy(g->exec);
  if (g->graph) (void)hipGraphDestroy(g->graph);
  delete g;
}

int hipnx_capture_begin(hipnx_ctx *ctx) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (ctx->capture) return set_error(HIPNX_EINVAL, "capture_begin: the context is already capturing");
  hipnx_graph *g = new hipnx_graph;
  g->ctx = ctx;
  // relaxed: a pool miss may still call hipMalloc (run the sequence once before capturing it and there is none)
  hipError_t e = hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed);
  if (e != hipSuccess) {
    delete g;
    return hip_fail(e, "hipStreamBeginCapture");
  }
  ctx->capture = g;
  ctx->graphs.push_back(g);
  return HIPNX_OK;
}

int hipnx_capture_end(hipnx_ctx *ctx, hipnx_graph **out) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (!ctx->capture) return set_error(HIPNX_EINVAL, "capture_end: the context is not capturing");
  hipnx_graph *g = ctx->capture;
  ctx->capture = nullptr;
  hipError_t e = hipStreamEndCapture(ctx->stream, &g->graph);
  if (e == hipSuccess) e = hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0);
  if (e != hipSuccess || !out) {
    release_graph(ctx, g);
    if (out) *out = nullptr;
    return e != hipSuccess ? hip_fail(e, "ending the capture") : set_error(HIPNX_EINVAL, "capture_end: null out");
  }
  *out = g;
  return HIPNX_OK;
}

int hipnx_graph_launch(hipnx_graph *g) {
  if (!g) return set_error(HIPNX_EINVAL, "null graph");
  hipnx_ctx *ctx = g->ctx;
  Enter in(ctx);
  if (in.status) return in.status;
  if (ctx->capture) return set_error(HIPNX_EINVAL, "graph_launch: the context is capturing");
  HIPNX_HIP(hipGraphLaunch(g->exec, ctx->stream));
  return HIPNX_OK;
}

int hipnx_graph_destroy(hipnx_graph *g) {
  if (!g) return set_error(HIPNX_EINVAL, "null graph");
  hipnx_ctx *ctx = g->ctx;
  Enter in(ctx);
  if (in.status) return in.status;
  if (ctx->capture == g) return set_error(HIPNX_EINVAL, "graph_destroy: this graph is still being captured");
  if (!ctx->capture) HIPNX_HIP(hipStreamSynchronize(ctx->stream));  // a replay may be in flight
  release_graph(ctx, g);
  return HIPNX_OK;
}

int hipnx_buf_alloc(hipnx_ctx *ctx, size_t bytes, hipnx_buf **out) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (!out) return set_error(HIPNX_EINVAL, "null out");
  void *ptr = nullptr;
  size_t cap = 0;
  if (int st = pool_alloc(ctx, bytes, &ptr, &cap)) return st;
  hipnx_buf *b = new hipnx_buf;
  b->ctx = ctx;
  b->ptr = ptr;
  b->bytes = bytes;
  b->capacity = cap;
  *out = b;
  return HIPNX_OK;
}

int hipnx_buf_free(hipnx_buf *buf) {
  if (!buf) return set_error(HIPNX_EINVAL, "null buffer handle");
  int expected = 0;
  if (!buf->freed.compare_exchange_strong(expected, 1)) return HIPNX_ALREADY_FREED;
  hipnx_ctx *ctx = buf->ctx;
  Enter in(ctx);
  if (in.status) return in.status;
  int st = HIPNX_OK;
  if (buf->ipc) {  // work that uses the mapping may still be running: wait, then close it
    (void)hipStreamSynchronize(ctx->stream);
    if (hipIpcCloseMemHandle(buf->ptr) != hipSuccess) (void)hipGetLastError();
  } else if (!buf->borrowed) {
    st = pool_free(ctx, buf->ptr, buf->capacity);
  }
  buf->ptr = nullptr;
  return st;
}

int hipnx_buf_wrap(hipnx_ctx *ctx, void *device_ptr, size_t bytes, hipnx_buf **out) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (!out || !device_ptr) return set_error(HIPNX_EINVAL, "buf_wrap: null argument");
  hipPointerAttribute_t attr;
  hipError_t e = hipPointerGetAttributes(&attr, device_ptr);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return set_error(HIPNX_EINVAL, "buf_wrap: %p is not a pointer this process can use on a device", device_ptr);
  }
  if (attr.type != hipMemoryTypeDevice || attr.device != ctx->device)
    return set_error(HIPNX_EINVAL, "buf_wrap: %p is not device memory of device %d", device_ptr, ctx->device);
  hipnx_buf *b = new hipnx_buf;
  b->ctx = ctx;
  b->ptr = device_ptr;
  b->bytes = bytes;
  b->capacity = bytes;
  b->borrowed = true;
  *out = b;
  return HIPNX_OK;
}

int hipnx_buf_ipc_export(hipnx_ctx *ctx, const hipnx_buf *buf, void *handle_out) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (!handle_out) return set_error(HIPNX_EINVAL, "ipc_export: null handle");
  if (int st = check_buf(ctx, buf, 0, "ipc_export")) return st;
  HIPNX_NOT_CAPTURING(ctx, "ipc_export");
  if (buf->borrowed) return set_error(HIPNX_EUNSUPPORTED, "ipc_export: the buffer wraps memory it does not own");
  if (buf->capacity >= (1ull << 31)) return set_error(HIPNX_EUNSUPPORTED, "ipc_export: allocations of 2 GiB or more are not shared");
  static_assert(sizeof(hipIpcMemHandle_t) == HIPNX_IPC_HANDLE_BYTES, "handle size of the public header");
  hipIpcMemHandle_t h;
  buf->index_bound = 0;  // another process may write here from now on
  HIPNX_HIP(hipIpcGetMemHandle(&h, buf->ptr));
  HIPNX_HIP(hipStreamSynchronize(ctx->stream));  // the other process sees what has been written so far
  std::memcpy(handle_out, &h, sizeof h);
  return deferred_error(ctx);
}

int hipnx_buf_ipc_import(hipnx_ctx *ctx, const void *handle, size_t bytes, hipnx_buf **out) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (!handle || !out) return set_error(HIPNX_EINVAL, "ipc_import: null argument");
  if (bytes >= (1ull << 31)) return set_error(HIPNX_EUNSUPPORTED, "ipc_import: allocations of 2 GiB or more are not shared");
  hipIpcMemHandle_t h;
  std::memcpy(&h, handle, sizeof h);
  void *ptr = nullptr;
  HIPNX_HIP(hipIpcOpenMemHandle(&ptr, h, hipIpcMemLazyEnablePeerAccess));
  hipnx_buf *b = new hipnx_buf;
  b->ctx = ctx;
  b->ptr = ptr;
  b->bytes = bytes;
  b->capacity = bytes;
  b->borrowed = true;
  b->ipc = true;
  *out = b;
  return HIPNX_OK;
}

int hipnx_buf_destroy(hipnx_buf *buf) {
  if (!buf) return set_error(HIPNX_EINVAL, "null buffer handle");
  int st = hipnx_buf_free(buf);
  delete buf;
  return st == HIPNX_ALREADY_FREED ? HIPNX_OK : st;
}

int hipnx_buf_size(const hipnx_buf *buf, size_t *bytes) {
  if (!buf || !bytes) return set_error(HIPNX_EINVAL, "null argument");
  if (buf->freed.load()) return set_error(HIPNX_EFREED, "buffer has been deallocated");
  *bytes = buf->bytes;
  return HIPNX_OK;
}

void *hipnx_buf_device_ptr(const hipnx_buf *buf) {
  if (!buf || buf->freed.load()) return nullptr;
  buf->index_bound = 0;  // the address leaves the library: what is written through it is not seen here
  return buf->ptr;
}

int hipnx_buf_index_bound(const hipnx_buf *buf, int64_t *bound) {
  if (!buf || !bound) return set_error(HIPNX_EINVAL, "null argument");
  if (buf->freed.load()) return set_error(HIPNX_EFREED, "buffer has been deallocated");
  *bound = buf->index_bound;
  return HIPNX_OK;
}

// Host memory of callers is pageable (an Erlang binary, a numpy array).  The runtime's own path for it costs 35 us for
// 64 KiB and delivers 17 GB/s device-to-host on large copies, against 10 us and 57 GB/s for pinned memory, so transfers
// go through pinned staging buffers of the context: a thread copies (28-30 GB/s) while the link fills or drains its
// other buffer.  A lane is two buffers; copies of 32 MiB and more are halved between the calling thread on lane 0 and
// a second thread on lane 1, since one thread's copy is what limits a lane.
static constexpr size_t STAGE_BYTES = 4u << 20;        // one staging buffer
static constexpr size_t TWO_LANES_MIN = 32u << 20;
static constexpr size_t PINNED_CHECK_MIN = 256u << 10;  // from here on it pays to ask whether the host memory is pinned already

static bool is_pinned(const void *p) {
  hipPointerAttribute_t at;
  const bool yes = hipPointerGetAttributes(&at, p) == hipSuccess && at.type == hipMemoryTypeHost;
  (void)hipGetLastError();  // "not a registered pointer" is the expected answer
  return yes;
}

#define STAGE_TRY(call)               \
  do {                                \
    hipError_t e__ = (call);          \
    if (e__ != hipSuccess) return e__; \
  } while (0)

// makes staging buffer `i` exist and waits for the transfer that last used it
static hipError_t stage_ready(hipnx_ctx *ctx, int i) {
  if (!ctx->stage[i]) STAGE_TRY(hipHostMalloc(&ctx->stage[i], STAGE_BYTES, hipHostMallocDefault));
  if (!ctx->stage_ev[i]) STAGE_TRY(hipEventCreateWithFlags(&ctx->stage_ev[i], hipEventDisableTiming));
  if (ctx->stage_busy[i]) {
    STAGE_TRY(hipEventSynchronize(ctx->stage_ev[i]));
    ctx->stage_busy[i] = false;
  }
  return hipSuccess;
}

// host -> device through lane `lane`, `chunk` bytes at a time; returns with the last transfers in flight
static hipError_t upload_range(hipnx_ctx *ctx, int lane, char *dev, const char *src, size_t bytes, size_t chunk) {
  STAGE_TRY(hipSetDevice(ctx->device));
  for (size_t done = 0; done < bytes; done += chunk) {
    const size_t n = bytes - done < chunk ? bytes - done : chunk;
    const int i = 2 * lane + ctx->stage_next[lane];
    ctx->stage_next[lane] ^= 1;
    STAGE_TRY(stage_ready(ctx, i));
    std::memcpy(ctx->stage[i], src + done, n);
    STAGE_TRY(hipMemcpyAsync(dev + done, ctx->stage[i], n, hipMemcpyHostToDevice, ctx->stream));
    STAGE_TRY(hipEventRecord(ctx->stage_ev[i], ctx->stream));
    ctx->stage_busy[i] = true;
  }
  return hipSuccess;
}

// device -> host through lane `lane`: piece k is on the link while piece k - 1 is copied out
static hipError_t download_range(hipnx_ctx *ctx, int lane, char *dst, const char *dev, size_t bytes, size_t chunk) {
  STAGE_TRY(hipSetDevice(ctx->device));
  const size_t chunks = (bytes + chunk - 1) / chunk;
  auto len = [&](size_t k) { return k + 1 < chunks ? chunk : bytes - k * chunk; };
  for (size_t k = 0; k <= chunks; k++) {
    if (k < chunks) {  // (piece k - 2 has left this buffer in the pass before)
      const int i = 2 * lane + (int)(k & 1);
      STAGE_TRY(stage_ready(ctx, i));
      STAGE_TRY(hipMemcpyAsync(ctx->stage[i], dev + k * chunk, len(k), hipMemcpyDeviceToHost, ctx->stream));
      STAGE_TRY(hipEventRecord(ctx->stage_ev[i], ctx->stream));
    }
    if (k >= 1) {
      const int i = 2 * lane + (int)((k - 1) & 1);
      STAGE_TRY(hipEventSynchronize(ctx->stage_ev[i]));
      std::memcpy(dst + (k - 1) * chunk, ctx->stage[i], len(k - 1));
    }
  }
  return hipSuccess;
}
#undef STAGE_TRY

// the two halves of a large copy on the two lanes; `half` is a multiple of the staging size
// pieces of a copy on one lane: a quarter of it, 512 KiB ... 4 MiB (a piece costs ~15 us beside its bytes)
static size_t piece_size(size_t bytes) {
  const size_t q = (bytes / 4 + 4095) & ~(size_t)4095;
  return q < (512u << 10) ? (512u << 10) : q > STAGE_BYTES ? STAGE_BYTES : q;
}

static hipError_t on_two_lanes(size_t bytes, const std::function<hipError_t(int, size_t, size_t)> &range) {
  const size_t half = (bytes / 2 + STAGE_BYTES - 1) / STAGE_BYTES * STAGE_BYTES;
  hipError_t second = hipSuccess;
  std::thread helper;
  try {
    helper = std::thread([&] { second = range(1, half, bytes - half); });
  } catch (const std::system_error &) {  // no thread to be had: the calling thread does both halves
    const hipError_t first = range(0, (size_t)0, half);
    return first != hipSuccess ? first : range(0, half, bytes - half);
  }
  const hipError_t first = range(0, (size_t)0, half);
  helper.join();
  return first != hipSuccess ? first : second;
}

int hipnx_h2d(hipnx_ctx *ctx, hipnx_buf *dst, size_t dst_offset, const void *src, size_t bytes) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (int st = check_buf(ctx, dst, (uint64_t)dst_offset + bytes, "h2d dst")) return st;
  HIPNX_NOT_CAPTURING(ctx, "h2d");
  if (bytes == 0) return HIPNX_OK;
  if (!src) return set_error(HIPNX_EINVAL, "h2d: null source");
  char *to = (char *)dst->ptr + dst_offset;
  if (bytes > PINNED_CHECK_MIN && is_pinned(src)) {  // pinned already: straight over the link
    HIPNX_HIP(hipMemcpyAsync(to, src, bytes, hipMemcpyHostToDevice, ctx->stream));
    HIPNX_HIP(hipStreamSynchronize(ctx->stream));
    return HIPNX_OK;
  }
  // The source (caller-owned: it must be consumed on return) is copied into staging buffers and the transfers out
  // of them are left in flight: the call returns without waiting for the device.
  if (bytes >= TWO_LANES_MIN) {
    HIPNX_HIP(on_two_lanes(bytes, [&](int lane, size_t at, size_t n) {
      return upload_range(ctx, lane, to + at, (const char *)src + at, n, STAGE_BYTES);
    }));
    return HIPNX_OK;
  }
  HIPNX_HIP(upload_range(ctx, 0, to, (const char *)src, bytes, piece_size(bytes)));
  return HIPNX_OK;
}

int hipnx_d2h(hipnx_ctx *ctx, const hipnx_buf *src, size_t src_offset, void *dst, size_t bytes) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (int st = check_buf(ctx, src, (uint64_t)src_offset + bytes, "d2h src")) return st;
  HIPNX_NOT_CAPTURING(ctx, "d2h");
  if (bytes == 0) {
    HIPNX_HIP(hipStreamSynchronize(ctx->stream));
    return deferred_error(ctx);
  }
  if (!dst) return set_error(HIPNX_EINVAL, "d2h: null destination");
  const char *from = (const char *)src->ptr + src_offset;
  if (bytes > PINNED_CHECK_MIN && is_pinned(dst)) {  // a destination that is pinned already takes the transfer directly
    HIPNX_HIP(hipMemcpyAsync(dst, from, bytes, hipMemcpyDeviceToHost, ctx->stream));
    HIPNX_HIP(hipStreamSynchronize(ctx->stream));
    return deferred_error(ctx);
  }
  if (bytes >= TWO_LANES_MIN) {
    HIPNX_HIP(on_two_lanes(bytes, [&](int lane, size_t at, size_t n) {
      return download_range(ctx, lane, (char *)dst + at, from + at, n, STAGE_BYTES);
    }));
    return deferred_error(ctx);
  }
  HIPNX_HIP(download_range(ctx, 0, (char *)dst, from, bytes, bytes <= (1u << 20) ? bytes : piece_size(bytes)));
  return deferred_error(ctx);  // the bytes have been delivered either way
}

int hipnx_d2d(hipnx_ctx *ctx, hipnx_buf *dst, size_t dst_offset, const hipnx_buf *src, size_t src_offset,
              size_t bytes) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (int st = check_buf(ctx, dst, (uint64_t)dst_offset + bytes, "d2d dst")) return st;
  if (int st = check_buf(ctx, src, (uint64_t)src_offset + bytes, "d2d src")) return st;
  if (bytes == 0) return HIPNX_OK;
  HIPNX_HIP(hipMemcpyAsync((char *)dst->ptr + dst_offset, (const char *)src->ptr + src_offset, bytes,
                           hipMemcpyDeviceToDevice, ctx->stream));
  return HIPNX_OK;
}

}  // extern "C"
