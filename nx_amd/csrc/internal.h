// Host-side internals of libhipnx: context, buffer handles, argument checks.
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <map>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/hipnx.h"

struct hipnx_ctx;

// A captured sequence of this context's work (stream capture -> executable graph) together with
// the device blocks it runs in.  Every block handed out while capturing belongs to the graph until
// the graph is destroyed: a replay writes to the same addresses, so none of them may reach the
// shared pool (and another owner) in between.
struct hipnx_graph {
  hipnx_ctx *ctx = nullptr;
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  std::vector<std::pair<void *, size_t>> owned;  // every block allocated during the capture
  std::multimap<size_t, void *> parked;          // owned blocks that no buffer holds right now
};

struct hipnx_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  hipEvent_t ev_start = nullptr, ev_stop = nullptr;
  std::vector<hipEvent_t> marks;  // lap marks of the stopwatch, created on first use
  std::mutex mu;  // serialises enqueueing and the pool
  // size-bucketed cache of freed device blocks; reuse is safe without a device wait because
  // every kernel of this context runs on the one stream, in order
  std::multimap<size_t, void *> pool;
  uint64_t live = 0, peak = 0, pooled = 0;
  int num_cus = 256;
  void *flag = nullptr;       // 32-byte device scratch for the gather bounds report
  void *flag_host = nullptr;  // pinned host word, mapped into the device: non-zero once a kernel saw a bad index
  void *flag_host_dev = nullptr;  // its device address
  // pinned staging buffers for host transfers (created on first use), two per lane: the link fills or drains one while
  // a thread copies the other; large copies run on both lanes (buffers 0-1: the calling thread, 2-3: a helper thread).
  // `stage_busy[i]`: an upload out of buffer i may still be in flight (its end is `stage_ev[i]`)
  void *stage[4] = {nullptr, nullptr, nullptr, nullptr};
  hipEvent_t stage_ev[4] = {nullptr, nullptr, nullptr, nullptr};
  bool stage_busy[4] = {false, false, false, false};
  int stage_next[2] = {0, 0};  // per lane: the buffer its next upload piece takes
  void *reduce_scratch = nullptr;  // this device's address of the static partial-result array of reduce.hip
  hipnx_graph *capture = nullptr;                        // non-null while the stream is capturing
  std::unordered_map<void *, hipnx_graph *> graph_blocks;  // block -> the live graph that owns it
  std::vector<hipnx_graph *> graphs;                     // live graphs of this context
  // fused groups compiled at run time for one program each: program bytes -> loaded kernel
  int fused_mode = 0;  // 0 = the interpreting kernels, 1 = compile each distinct program once
  // compiled fused groups, keyed by what each is specialised on; at most fused_cache_max are kept (the least
  // recently launched quarter is unloaded when the table is full; kernels recorded into a graph stay)
  struct FusedKernel {
    hipModule_t module;
    hipFunction_t function;
    uint64_t last_use;
    bool in_graph;
  };
  size_t fused_cache_max = 512;  // hipnx_fused_set_cache_limit
  std::unordered_map<std::string, FusedKernel> fused_kernels;
  uint64_t fused_clock = 0;
};

struct hipnx_buf {
  hipnx_ctx *ctx = nullptr;
  void *ptr = nullptr;
  size_t bytes = 0;     // what the caller asked for
  size_t capacity = 0;  // what the pool block holds
  std::atomic<int> freed{0};
  bool borrowed = false;  // wraps memory owned by someone else: never returned to the pool
  bool ipc = false;       // borrowed through an IPC handle of another process: closed on release
  // What the library knows about the VALUES it last wrote here: the first index_bytes bytes hold indices of type
  // index_dt that all lie in [0, index_bound) -- set by hipnx_argreduce on its result (an index along an axis of
  // that length), cleared whenever the buffer is handed to an entry point as an output or its address leaves the
  // library.  gather / take use it to skip the wait of the raising bounds policy for indices that cannot be out
  // of range.  0 = nothing known.
  mutable int64_t index_bound = 0;
  uint64_t index_bytes = 0;
  int index_dt = -1;
};

namespace hipnx {

int set_error(int code, const char *fmt, ...);
int hip_fail(hipError_t e, const char *what);

#define HIPNX_HIP(call)                                         \
  do {                                                          \
    hipError_t e__ = (call);                                    \
    if (e__ != hipSuccess) return hipnx::hip_fail(e__, #call);  \
  } while (0)

// hipFuncAttributeMaxDynamicSharedMemorySize is a property of a kernel ON A DEVICE.  Expanded where a kernel
// that needs more than 64 KiB of LDS is launched (so the static below belongs to that kernel's launch site):
// sets the attribute once per device (a bit per device index; devices beyond 63 set it on every launch), with
// the context's device current -- the entry point's scope has selected it.
#define HIPNX_ALLOW_DYNAMIC_LDS(ctx, kern, bytes)                                                              \
  do {                                                                                                         \
    static std::atomic<uint64_t> done__{0};                                                                    \
    const uint64_t bit__ = (ctx)->device >= 0 && (ctx)->device < 64 ? 1ull << (ctx)->device : 0;               \
    if (!bit__ || !(done__.load(std::memory_order_acquire) & bit__)) {                                         \
      HIPNX_HIP(hipFuncSetAttribute((const void *)(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (bytes))); \
      if (bit__) done__.fetch_or(bit__, std::memory_order_release);                                            \
    }                                                                                                          \
  } while (0)

inline int dtype_size(int dt) {
  static const int sz[HIPNX_NTYPES] = {1, 2, 4, 8, 1, 2, 4, 8, 2, 2, 4, 8};
  return (dt >= 0 && dt < HIPNX_NTYPES) ? sz[dt] : -1;
}
inline bool is_float(int dt) { return dt >= HIPNX_F16; }
// output type of as_type and dot: the twelve element types and the round-to-nearest-even bf16 encoding
inline int out_dtype_size(int dt) { return dt == HIPNX_BF16_RNE ? 2 : dtype_size(dt); }
inline bool is_unsigned(int dt) { return dt >= 0 && dt <= HIPNX_U64; }
inline bool is_wide(int dt) {  // not exactly representable in f32
  return dt == HIPNX_U32 || dt == HIPNX_U64 || dt == HIPNX_S32 || dt == HIPNX_S64 || dt == HIPNX_F64;
}

// operand checks shared by every entry point: live handle, same context, enough bytes
int check_buf(const hipnx_ctx *ctx, const hipnx_buf *b, uint64_t need_bytes, const char *name);
// the same for a buffer an entry point is about to write (outputs are the non-const handles of the C ABI): what was
// known about its values is forgotten
inline int check_buf(const hipnx_ctx *ctx, hipnx_buf *b, uint64_t need_bytes, const char *name) {
  const int st = check_buf(ctx, static_cast<const hipnx_buf *>(b), need_bytes, name);
  if (st == HIPNX_OK) b->index_bound = 0;  // (only a live handle of this context is written to)
  return st;
}

// pooled device memory; both expect the context mutex to be held (i.e. inside an Enter scope)
int pool_alloc(hipnx_ctx *ctx, size_t bytes, void **ptr_out, size_t *cap_out);
int pool_free(hipnx_ctx *ctx, void *ptr, size_t cap);

// The deferred error word: 8 bytes of the context's pinned, device-mapped host block (offset 16; the
// first word belongs to the gather bounds report).  Kernels that meet operands the reference raises
// for store (code << 56 | operand) there; deferred_error() is called by every entry point that has
// just waited for the stream and turns a recorded case into HIPNX_ERAISED (once; the word is re-armed).
inline unsigned long long *deferred_error_word(const hipnx_ctx *ctx) {
  return (unsigned long long *)((char *)ctx->flag_host_dev + 16);
}
int deferred_error(hipnx_ctx *ctx);

// looks up this device's address of the static scratch array of hipnx_reduce_static (the device of
// `ctx` must be current); defined beside the array in reduce.hip
int reduce_static_init(hipnx_ctx *ctx);

// entry points that wait for the device cannot run while the stream is capturing
#define HIPNX_NOT_CAPTURING(ctx, what)                                                                 \
  do {                                                                                                 \
    if ((ctx)->capture)                                                                                \
      return hipnx::set_error(HIPNX_EUNSUPPORTED, "%s waits for the device: not possible while capturing", what); \
  } while (0)

// RAII: select the device and take the context mutex for the duration of an entry point
struct Enter {
  std::unique_lock<std::mutex> lk;
  int status;
  explicit Enter(hipnx_ctx *ctx);
};

}  // namespace hipnx
