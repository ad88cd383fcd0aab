/*
 * hipnx.h -- C ABI of libhipnx, the MI355X (gfx950) device library underneath HipNx.Backend.
 *
 * This is the drop-in boundary for the eager tensor path of Nx: every entry point is what a NIF
 * for one `Nx.Backend` callback (reference: nx/lib/nx/backend.ex:46-144) binds.  The structural
 * model is the reference's Torchx NIF (torchx/c_src/torchx.cpp, one native function per
 * callback) with LibTorch replaced by hand-written HIP kernels.
 *
 * Conventions
 *  - Plain C: opaque handles, pointers and sizes only.
 *  - Every function returns an int status (HIPNX_OK = 0).  On failure a message is kept per
 *    calling thread and can be fetched with hipnx_last_error().  Nothing aborts the process.
 *  - A context owns one device and one HIP stream.  Compute entry points only enqueue work on
 *    that stream and return; hipnx_d2h() and hipnx_sync() wait.  Contexts may be used from any
 *    thread (NIFs run on arbitrary dirty-scheduler threads): each entry selects the device and
 *    serialises enqueueing with a short mutex.
 *  - Device buffers are flat, untyped byte ranges.  Shape, element type and strides always come
 *    from the caller (the `Nx.Tensor` struct), never from the handle -- `Nx.reshape`, `rename`,
 *    `vectorize` rewrite them without calling the backend (nx/lib/nx.ex:5354-5405, 3058-3060).
 *  - Inputs are immutable; every op writes a buffer the caller allocated for `out`.
 *  - Before any launch the host side checks that every operand buffer is live and large enough
 *    for the shape it is claimed to hold.
 */
#ifndef HIPNX_H
#define HIPNX_H
#ifndef __HIPCC_RTC__ /* the run-time compiler brings its own fixed-width types and has no C headers */
#include <stddef.h>
#include <stdint.h>
#endif
#ifdef __cplusplus
extern "C" {
#endif

typedef struct hipnx_ctx hipnx_ctx;
typedef struct hipnx_buf hipnx_buf;
typedef struct hipnx_graph hipnx_graph;

/* status codes */
enum {
  HIPNX_OK = 0,
  HIPNX_ALREADY_FREED = 1, /* hipnx_buf_free on a freed buffer (-> :already_deallocated) */
  HIPNX_EINVAL = 2,        /* malformed call: bad code, rank, size mismatch (-> ArgumentError) */
  HIPNX_EFREED = 3,        /* an operand buffer was deallocated before use */
  HIPNX_ENOMEM = 4,        /* device allocation failed */
  HIPNX_EHIP = 5,          /* a HIP runtime call failed */
  HIPNX_EINDEX = 6,        /* gather/take index out of bounds (-> ArgumentError, reference text) */
  HIPNX_EUNSUPPORTED = 7,  /* type combination not implemented natively */
  HIPNX_ERAISED = 8        /* a kernel issued EARLIER on this context met operands the reference raises for
                            * (integer quotient / remainder by zero, a negative shift count, a negative
                            * integer exponent, float remainder by zero or of a non-finite value:
                            * binary_backend.ex:711-750; a deferred gather index).  Kernels cannot raise:
                            * they record the first case in a pinned host word and write 0 (or skip the
                            * slice); the next call that waits for the device -- hipnx_sync, hipnx_d2h,
                            * hipnx_timer_stop / between, a raising gather -- returns this status once with
                            * the reference's exception text ("ArithmeticError: ..." / "ArgumentError: ...")
                            * and re-arms the word.  The data of that call is still delivered. */
};

/* element types, Nx.Type tuples {:u,8} .. {:f,64} (nx/lib/nx/type.ex:27-48) */
enum {
  HIPNX_U8 = 0, HIPNX_U16 = 1, HIPNX_U32 = 2, HIPNX_U64 = 3,
  HIPNX_S8 = 4, HIPNX_S16 = 5, HIPNX_S32 = 6, HIPNX_S64 = 7,
  HIPNX_F16 = 8, HIPNX_BF16 = 9, HIPNX_F32 = 10, HIPNX_F64 = 11, HIPNX_NTYPES = 12,
  /* OUTPUT ONLY, accepted as out_dt by hipnx_as_type and hipnx_dot: bf16 encoded with round-to-nearest-even,
   * as Torchx and EXLA do (torchx/test/torchx/nx_test.exs:380-394 expects 1/5 -> 0.2001953125), instead of
   * Nx.BinaryBackend's truncation (shared.ex:136-152).  The buffer holds ordinary bf16. */
  HIPNX_BF16_RNE = 12
};

/* element-wise binary callbacks, in the order of nx/lib/nx/binary_backend.ex:649-653 */
enum {
  HIPNX_ADD = 0, HIPNX_SUBTRACT, HIPNX_MULTIPLY, HIPNX_DIVIDE, HIPNX_POW, HIPNX_REMAINDER,
  HIPNX_ATAN2, HIPNX_MIN, HIPNX_MAX, HIPNX_QUOTIENT, HIPNX_BITWISE_AND, HIPNX_BITWISE_OR,
  HIPNX_BITWISE_XOR, HIPNX_LEFT_SHIFT, HIPNX_RIGHT_SHIFT, HIPNX_EQUAL, HIPNX_NOT_EQUAL,
  HIPNX_GREATER, HIPNX_LESS, HIPNX_GREATER_EQUAL, HIPNX_LESS_EQUAL, HIPNX_LOGICAL_AND,
  HIPNX_LOGICAL_OR, HIPNX_LOGICAL_XOR, HIPNX_NBINARY
};

/* element-wise unary callbacks: the 23 math functions of nx/lib/nx/shared.ex:311-376 in that
 * order, then nx/lib/nx/backend.ex:125-132 */
enum {
  HIPNX_EXP = 0, HIPNX_EXPM1, HIPNX_LOG, HIPNX_LOG1P, HIPNX_SIGMOID, HIPNX_COS, HIPNX_SIN,
  HIPNX_TAN, HIPNX_COSH, HIPNX_SINH, HIPNX_TANH, HIPNX_ACOS, HIPNX_ASIN, HIPNX_ATAN,
  HIPNX_ACOSH, HIPNX_ASINH, HIPNX_ATANH, HIPNX_SQRT, HIPNX_RSQRT, HIPNX_CBRT, HIPNX_ERF,
  HIPNX_ERFC, HIPNX_ERF_INV, HIPNX_ABS, HIPNX_BITWISE_NOT, HIPNX_CEIL, HIPNX_FLOOR,
  HIPNX_NEGATE, HIPNX_ROUND, HIPNX_SIGN, HIPNX_CLZ, HIPNX_POPCOUNT, HIPNX_IS_NAN,
  HIPNX_IS_INFINITY, HIPNX_NUNARY
};

enum { HIPNX_RED_SUM = 0, HIPNX_RED_MAX = 1, HIPNX_RED_MIN = 2, HIPNX_RED_PRODUCT = 3, HIPNX_RED_ALL = 4, HIPNX_RED_ANY = 5 };
enum { HIPNX_ARGMAX = 0, HIPNX_ARGMIN = 1 };
enum { HIPNX_TIE_LOW = 0, HIPNX_TIE_HIGH = 1 };

/* operand layouts of hipnx_dot: which of the two non-batch axes is contiguous */
enum {
  HIPNX_K_INNER = 0, /* [batch, M or N, K]: the contracted axis is the last (unit stride) */
  HIPNX_K_OUTER = 1  /* [batch, K, M or N]: the contracted axis comes first */
};

/* out-of-bounds index policy of hipnx_gather */
enum {
  HIPNX_OOB_RAISE = 0, /* Nx.BinaryBackend: raise (binary_backend.ex:1949-1952); waits for the kernel */
  HIPNX_OOB_CLAMP = 1, /* EXLA / Torchx behaviour: clamp into range; stays asynchronous */
  HIPNX_OOB_DEFER = 2  /* raise, but late: the kernel records the first bad index it meets and the next
                        * waiting call on the context (hipnx_sync, hipnx_d2h, ...) fails with HIPNX_ERAISED;
                        * the slices of bad tuples are left unwritten; stays asynchronous */
};

/* ---- context, errors ---------------------------------------------------------------------
 * replaces: backend `init/1` + per-backend client/device selection
 * (nx/lib/nx/backend.ex:46; torchx/lib/torchx/backend.ex:49-52; exla/lib/exla/client.ex:20-55) */
int hipnx_device_count(int *count);
int hipnx_ctx_create(int device, hipnx_ctx **out);
int hipnx_ctx_destroy(hipnx_ctx *ctx);
int hipnx_sync(hipnx_ctx *ctx);
/* copies the calling thread's last error message (NUL-terminated, truncated to cap) */
int hipnx_last_error(char *dst, size_t cap);
/* live / peak / pooled device bytes of this context (cf. EXLA client memory statistics,
 * exla/c_src/exla/exla_client.cc:597-631) */
int hipnx_mem_stats(hipnx_ctx *ctx, uint64_t *live, uint64_t *peak, uint64_t *pooled);
/* returns pooled (cached, unused) device memory to the driver */
int hipnx_trim(hipnx_ctx *ctx);

/* HIP-event stopwatch on the context's stream (device-side timing for benchmarks) */
int hipnx_timer_start(hipnx_ctx *ctx);
int hipnx_timer_stop(hipnx_ctx *ctx, float *elapsed_ms);
/* lap marks of the same stopwatch: `mark` records event number `index` (0 .. 65535) on the stream
 * and returns at once; `between` waits for mark `to` and gives the device time from mark `from` to
 * it.  One mark per step gives per-step times (median, minimum) without a host wait per step. */
int hipnx_timer_mark(hipnx_ctx *ctx, int index);
int hipnx_timer_between(hipnx_ctx *ctx, int from, int to, float *elapsed_ms);

/* ---- buffers -------------------------------------------------------------------------------
 * replaces: from_binary / to_binary / backend_copy / backend_transfer / backend_deallocate
 * (nx/lib/nx/backend.ex:50-57; torchx/c_src/torchx.cpp:100-185 from_blob, to_blob,
 * delete_tensor; exla/c_src/exla/exla.cc:439-475) */
int hipnx_buf_alloc(hipnx_ctx *ctx, size_t bytes, hipnx_buf **out);
/* explicit deallocation; idempotent: HIPNX_OK the first time, HIPNX_ALREADY_FREED afterwards.
 * The handle itself stays valid until hipnx_buf_destroy (the BEAM resource destructor). */
int hipnx_buf_free(hipnx_buf *buf);
/* releases the handle (and the device memory if still live) */
int hipnx_buf_destroy(hipnx_buf *buf);
int hipnx_buf_size(const hipnx_buf *buf, size_t *bytes);
/* replaces: to_pointer/2 with mode :local (nx/lib/nx/backend.ex:66; exla/lib/exla/backend.ex:86-131,
 * exla/c_src/exla/exla.cc:327-385): the raw device address of a live buffer; NULL once freed */
void *hipnx_buf_device_ptr(const hipnx_buf *buf);
/* replaces: nothing in the reference (its backends check or clamp every index, nx/lib/nx/binary_backend.ex:1949-1952,
 * exla/test/exla/defn/expr_test.exs:3478-3481).  0, or the length L of the axis along which hipnx_argreduce last
 * wrote this buffer's values, every one of them in [0, L): such a buffer used as the indices of hipnx_take /
 * hipnx_gather (one index per slice, same index type) along an axis of at least L entries cannot hold a bad index,
 * and the HIPNX_OOB_RAISE policy then does not wait for the kernel (a violation, impossible by construction, would
 * still be recorded and raised by the next wait).  The knowledge is dropped when the buffer is written again (any
 * entry point that takes it as an output) or its address leaves the library (hipnx_buf_device_ptr, ipc_export). */
int hipnx_buf_index_bound(const hipnx_buf *buf, int64_t *bound);
/* replaces: from_pointer/5 for a :local pointer (nx/lib/nx/backend.ex:59-65;
 * exla/lib/exla/backend.ex:133-181, exla/c_src/exla/exla.cc:387-437): a handle over `bytes` of
 * device memory of this context's device that someone else owns.  Freeing or destroying the
 * handle never frees the memory; the owner keeps it alive while the handle is used. */
int hipnx_buf_wrap(hipnx_ctx *ctx, void *device_ptr, size_t bytes, hipnx_buf **out);
/* replaces: to_pointer/2 with mode :ipc and from_pointer/5 for an :ipc pointer (nx/lib/nx/pointer.ex:8-15;
 * exla/lib/exla/backend.ex:85-181; exla/c_src/exla/exla_cuda.cc:11-52 -- cudaIpcGetMemHandle /
 * cudaIpcOpenMemHandle there, hipIpcGetMemHandle / hipIpcOpenMemHandle here).  `export` waits for the
 * work enqueued so far and writes the HIPNX_IPC_HANDLE_BYTES bytes another PROCESS on the same machine
 * opens with `import` (on the device with the same index); the buffer must own its memory (not a
 * wrapped or imported one) and hold less than 2 GiB.  `import` gives a handle over the exporter's
 * memory; destroying it closes the mapping and never frees the memory, which the exporter keeps alive
 * while the importer uses it.  Opening a handle in the process that exported it is an error of the
 * HIP runtime and is reported as such.  What an importer writes through the handle (hipnx_h2d, a
 * kernel's output) is in flight on ITS context's stream when the call returns: the exporter may read it
 * only after the writing process has called hipnx_sync (and told the exporter so). */
#define HIPNX_IPC_HANDLE_BYTES 64
int hipnx_buf_ipc_export(hipnx_ctx *ctx, const hipnx_buf *buf, void *handle_out);
int hipnx_buf_ipc_import(hipnx_ctx *ctx, const void *handle, size_t bytes, hipnx_buf **out);
/* `src` is consumed on return (it may be an Erlang binary): the bytes are copied into pinned staging buffers of the
 * context (from 32 MiB on by the calling thread and a helper thread, half each) and the transfers out of them are left
 * in flight on the stream, so the call does not wait for the device.  Uploads from memory that is pinned already go
 * straight over the link and wait.  Later work on the context is ordered after the upload either way. */
int hipnx_h2d(hipnx_ctx *ctx, hipnx_buf *dst, size_t dst_offset, const void *src, size_t bytes);
/* waits for all work enqueued so far, then copies: through the context's pinned staging buffers (the link fills one
 * while a thread empties the other; from 32 MiB on two threads, half each) unless `dst` is pinned memory itself */
int hipnx_d2h(hipnx_ctx *ctx, const hipnx_buf *src, size_t src_offset, void *dst, size_t bytes);
int hipnx_d2d(hipnx_ctx *ctx, hipnx_buf *dst, size_t dst_offset, const hipnx_buf *src,
              size_t src_offset, size_t bytes);
/* replaces: constant/3 (nx/lib/nx/backend.ex:49): n copies of one element (elem_bytes <= 8) */
int hipnx_fill(hipnx_ctx *ctx, hipnx_buf *dst, int elem_bytes, const void *elem, int64_t n);

/* ---- element-wise --------------------------------------------------------------------------
 * replaces: the 24 binary callbacks (nx/lib/nx/backend.ex:115-123; oracle
 * nx/lib/nx/binary_backend.ex:649-823; torchx/c_src/torchx.cpp:737-769).
 * out[i] = op(l[bcast i], r[bcast i]) over the row-major index space `out_dims[rank]`;
 * strides are in elements, 0 marks a broadcast axis (numpy-style, nx/lib/nx/shape.ex:316-376).
 * Known difference from the reference: with one operand u64 and the other a signed integer the pair is computed as s64,
 * so u64 values of 2^63 and more read as negative in the comparisons, min, max, quotient, remainder and right_shift
 * (add, subtract, multiply, bitwise and left_shift wrap to the same bits as the reference's unbounded integers). */
int hipnx_binary(hipnx_ctx *ctx, int op, int l_dt, int r_dt, int out_dt, int rank,
                 const int64_t *out_dims, const int64_t *l_strides, const int64_t *r_strides,
                 const hipnx_buf *l, const hipnx_buf *r, hipnx_buf *out);

/* replaces: the unary callbacks (nx/lib/nx/backend.ex:125-132; oracle binary_backend.ex:827-1005;
 * torchx/c_src/torchx.cpp:777-828) */
int hipnx_unary(hipnx_ctx *ctx, int op, int in_dt, int out_dt, int64_t n, const hipnx_buf *in,
                hipnx_buf *out);

/* replaces: as_type/2 (nx/lib/nx/backend.ex:68; oracle binary_backend.ex:2031-2076).
 * float->bf16 truncates, float->int truncates toward zero then wraps, NaN->0, +-Inf->max/min. */
int hipnx_as_type(hipnx_ctx *ctx, int in_dt, int out_dt, int64_t n, const hipnx_buf *in,
                  hipnx_buf *out);

/* ---- reductions ----------------------------------------------------------------------------
 * replaces: sum / product / reduce_max / reduce_min / all / any (nx/lib/nx/backend.ex:87-92; oracle
 * binary_backend.ex:1293-1375; all / any: 1 unless / if an element differs from 0, u8 output).  The input is viewed as [outer, red, inner] (the caller
 * collapses axes, transposing first when the reduced axes are not adjacent); out is
 * [outer, inner]. */
int hipnx_reduce(hipnx_ctx *ctx, int op, int in_dt, int out_dt, int64_t outer, int64_t red,
                 int64_t inner, const hipnx_buf *in, hipnx_buf *out);

/* No counterpart in the reference: hipnx_reduce for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  Same
 * arguments and kernels; the partial results of a split reduction go
 * to a static device array of HIPNX_REDUCE_STATIC_SCRATCH_BYTES (held by every GPU the library runs
 * on until the process ends) instead of a pool block, and the call performs no hipMalloc / hipFree.
 * Results are those of hipnx_reduce bit for bit, with one exception: for a few columns under a long
 * axis (inner > 1, inner * element size < 1024 bytes, red >= 4096) hipnx_reduce folds rows into the
 * columns and reduces in two steps through a pool block, which this entry point does not -- integer
 * results and selections (max, min, all, any) are still identical, float sums and products are
 * accumulated in another order and agree within the accumulation bound (red * 2^-53 * sum|x| before the
 * one rounding to the output type).
 * A shape whose partials do not fit fails with HIPNX_EUNSUPPORTED and launches nothing.  All calls
 * on one GPU share that array: calls that overlap on one GPU (two contexts, i.e. two streams) race. */
#define HIPNX_REDUCE_STATIC_SCRATCH_BYTES (1u << 20)
int hipnx_reduce_static(hipnx_ctx *ctx, int op, int in_dt, int out_dt, int64_t outer, int64_t red,
                        int64_t inner, const hipnx_buf *in, hipnx_buf *out);

/* replaces: argmax / argmin (nx/lib/nx/backend.ex:93-94; oracle binary_backend.ex:1393-1431).
 * Same view.  tie LOW = first index of the extreme, HIGH = last; any NaN wins and the last
 * NaN's index is returned.  out_dt is an integer type.  An axis of 2^31 positions or more is searched in
 * chunks (outer == 1: the flattened tensor, or the first axis); under more than one outer index such an axis
 * is refused with HIPNX_EUNSUPPORTED. */
int hipnx_argreduce(hipnx_ctx *ctx, int op, int tie, int in_dt, int out_dt, int64_t outer,
                    int64_t red, int64_t inner, const hipnx_buf *in, hipnx_buf *out);

/* ---- contraction ---------------------------------------------------------------------------
 * replaces: dot/7 (nx/lib/nx/backend.ex:77; oracle binary_backend.ex:476-599, 2362-2385;
 * torchx/c_src/torchx.cpp:844-890 tensordot).
 * out[b, m, n] = sum_k l[b, m, k] * r[b, n, k]; l is [batch, M, K] (HIPNX_K_INNER) or
 * [batch, K, M] (HIPNX_K_OUTER), r is [batch, N, K] or [batch, K, N]; out is [batch, M, N] in
 * out_dt (f32 accumulation for f16/bf16/f32 operands, exact s32 for s8, f64 accumulation on the matrix cores for
 * f64 operands whose K is a multiple of 16 and whose result has 256 elements or more, then one encode; other f64
 * shapes, wider integers and mixed operand types accumulate in f64 / wrapping 64-bit integers over k in order, as do
 * a handful of outputs over a long K -- the dot of two vectors -- whose segments of K are summed in f64).
 * out_dt may be HIPNX_BF16_RNE (bf16 rounded to nearest even).  Any batch count is taken (beyond 65535 items in
 * several launches).  The call may take workspace from the context's pool and return it before it ends: a re-laid
 * operand whose K-outer rows are not whole 16-byte blocks, one-slab zero-extended copies of the last part of K when K
 * is not a whole number of 128-byte slabs (copies of both operands where their rows are not whole 16-byte blocks
 * either), the partial results of a contraction whose K is split over several work-groups per tile or output. */
int hipnx_dot(hipnx_ctx *ctx, int l_dt, int r_dt, int out_dt, int64_t batch, int64_t M, int64_t N,
              int64_t K, int l_layout, int r_layout, const hipnx_buf *l, const hipnx_buf *r,
              hipnx_buf *out);

/* replaces: the three callbacks of a quantised linear layer in one -- dot/7 with an s32 result, as_type/2
 * to f32 and multiply/3 by the scales (nx/lib/nx/backend.ex:77, 68, 115), i.e.
 * Nx.multiply(Nx.as_type(Nx.dot(x, w), :f32), scales) on s8 operands.  out[b, m, n] (f32) =
 * (float)(sum_k l[b, m, k] * r[b, n, k] as s32) * scale, where scale (f32) is scale[n]
 * (HIPNX_SCALE_PER_COLUMN), scale[m] (PER_ROW, batch = 1) or scale[0] (ONE): the conversion and the product
 * are done on the accumulators and round exactly as the separate kernels do, so the result is
 * bit-identical to the three calls.  s8 x s8 on the matrix-core kernels only (K <= 65536, K a multiple of
 * 128); anything else is HIPNX_EUNSUPPORTED: make the three calls. */
enum { HIPNX_SCALE_NONE = 0, HIPNX_SCALE_PER_COLUMN = 1, HIPNX_SCALE_PER_ROW = 2, HIPNX_SCALE_ONE = 3 };
int hipnx_dot_scaled(hipnx_ctx *ctx, int l_dt, int r_dt, int64_t batch, int64_t M, int64_t N, int64_t K,
                     int l_layout, int r_layout, const hipnx_buf *l, const hipnx_buf *r, int scale_mode,
                     const hipnx_buf *scale, hipnx_buf *out);

/* ---- data movement -------------------------------------------------------------------------
 * replaces: transpose/3 (nx/lib/nx/backend.ex:73; oracle binary_backend.ex:280-319) */
int hipnx_transpose(hipnx_ctx *ctx, int elem_bytes, int rank, const int64_t *in_dims,
                    const int *perm, const hipnx_buf *in, hipnx_buf *out);

/* replaces: broadcast/4 (nx/lib/nx/backend.ex:72; oracle binary_backend.ex:215-276);
 * in_strides in elements per output axis, 0 = broadcast */
int hipnx_broadcast(hipnx_ctx *ctx, int elem_bytes, int rank, const int64_t *out_dims,
                    const int64_t *in_strides, const hipnx_buf *in, hipnx_buf *out);

/* replaces: gather/4 and block(%Nx.Block.Take{}) (nx/lib/nx/backend.ex:81,144; oracle
 * binary_backend.ex:1902-1959; nx/lib/nx.ex:14807-14819).  The tensor `t_dims[rank]` has its
 * indexed axes leading; each of the n_tuples index tuples (idx is [n_tuples, depth], integer
 * type idx_dt) addresses the first `depth` axes and the trailing slice is copied.  `take` along
 * axis 0 is depth = 1. */
int hipnx_gather(hipnx_ctx *ctx, int elem_bytes, int rank, const int64_t *t_dims, int idx_dt,
                 int64_t n_tuples, int depth, int oob_policy, const hipnx_buf *t,
                 const hipnx_buf *idx, hipnx_buf *out);

/* replaces: block(%Nx.Block.Take{axis}) for any axis (nx/lib/nx/backend.ex:144; nx/lib/nx/block.ex:57-59;
 * nx/lib/nx.ex:14807-14819, whose default is gather + transpose).  The tensor is viewed as
 * [outer, axis_len, inner]; out[o, j, :] = t[o, idx[j], :] for the n_idx indices of integer type idx_dt,
 * out is [outer, n_idx, inner].  `msg_dims[rank]` is the shape an out-of-range index is reported against:
 * the tensor's with the taken axis moved to the front, as the reference's transposing default reports it. */
int hipnx_take(hipnx_ctx *ctx, int elem_bytes, int64_t outer, int64_t axis_len, int64_t inner, int idx_dt,
               int64_t n_idx, int oob_policy, int rank, const int64_t *msg_dims, const hipnx_buf *t,
               const hipnx_buf *idx, hipnx_buf *out);

/* ---- callbacks one step off the hot path (callers: Nx.LinAlg, Nx.Random, grad code) ----------
 * replaces: select/4 (nx/lib/nx/backend.ex:84; oracle binary_backend.ex:604-648).
 * out[i] = pred[i] != 0 ? on_true[i] : on_false[i]; the three operands are broadcast to out_dims
 * by per-axis strides in elements (0 = repeat), values are converted to out_dt. */
int hipnx_select(hipnx_ctx *ctx, int pred_dt, int true_dt, int false_dt, int out_dt, int rank,
                 const int64_t *out_dims, const int64_t *pred_strides, const int64_t *true_strides,
                 const int64_t *false_strides, const hipnx_buf *pred, const hipnx_buf *on_true,
                 const hipnx_buf *on_false, hipnx_buf *out);

/* replaces: clip/4 (nx/lib/nx/backend.ex:78; oracle binary_backend.ex:1788-1811); min and max
 * are one-element buffers of their own types, read on the device */
int hipnx_clip(hipnx_ctx *ctx, int in_dt, int min_dt, int max_dt, int out_dt, int64_t n,
               const hipnx_buf *in, const hipnx_buf *min, const hipnx_buf *max, hipnx_buf *out);

/* replaces: concatenate/3 and stack/3 of operands that already have the output's type (nx/lib/nx/backend.ex:82-83;
 * oracle binary_backend.ex:1962-1986) in one launch per 64 operands instead of one copy per operand.  Part p is
 * [outer, extents[p], inner] elements of `elem_bytes`, out is [outer, sum of extents, inner]. */
int hipnx_concat(hipnx_ctx *ctx, int elem_bytes, int n_parts, const hipnx_buf *const *parts, const int64_t *extents,
                 int64_t outer, int64_t inner, hipnx_buf *out);
/* replaces: slice/5, concatenate/3, stack/3, pad/4, reverse/3, put_slice/4 (nx/lib/nx/backend.ex:79,82-83,
 * 74-75,80; oracle binary_backend.ex:1813-1863, 1962-2030, 326-431, 434-474, 1865-1900) -- one copy over the index space `dims` with
 * element strides and offsets on both sides: a slice reads strided and writes dense, a
 * concatenation writes each operand into its window of the output, a pad writes the elements
 * that survive the cropping at their spread-out positions in an output filled with the pad
 * value (hipnx_broadcast with zero strides), a reverse reads an axis backwards (negative input
 * stride, the offset on its last element), a put_slice writes the slice into its window of a copy */
int hipnx_strided_copy(hipnx_ctx *ctx, int elem_bytes, int rank, const int64_t *dims,
                       const int64_t *in_strides, int64_t in_offset, const int64_t *out_strides,
                       int64_t out_offset, const hipnx_buf *in, hipnx_buf *out);

/* replaces: iota/3 (nx/lib/nx/backend.ex:51; oracle binary_backend.ex:49-87):
 * out[i] = (i / inner) % dim; the flat iota is dim = n, inner = 1 */
int hipnx_iota(hipnx_ctx *ctx, int out_dt, int64_t n, int64_t dim, int64_t inner, hipnx_buf *out);

/* replaces: eye/2 (nx/lib/nx/backend.ex:50; oracle binary_backend.ex:90-110): n elements of
 * stacked rows x cols identity matrices */
int hipnx_eye(hipnx_ctx *ctx, int out_dt, int64_t n, int64_t rows, int64_t cols, hipnx_buf *out);

/* replaces: the write of an integer result at a sub-byte width, `<<x::size(bits)>>` keeping the low
 * bits (nx/lib/nx/shared.ex:190-194), for tensors of u2 / u4 / s2 / s4 held one element per byte as
 * the reference's device backends hold them (exla/lib/exla/device_buffer.ex:24-34,
 * torchx/lib/torchx/backend.ex:428-434): every byte of buf keeps its low `bits` bits (2 or 4), zero- or
 * sign-extended to the byte.  In place: meant for the fresh output of a callback that computed at 8 bits */
int hipnx_narrow_int(hipnx_ctx *ctx, hipnx_buf *buf, int64_t n, int bits, int is_signed);

/* replaces: the callback composition behind threefry2x32/2 of Nx.Random (nx/lib/nx/random.ex:214-285;
 * about 110 element-wise callbacks per call) with one kernel producing the same words: out[n] u32 is
 * the Threefry-2x32-20 stream of key (u32[2]) over the counters 0 .. n-1, in the reference's
 * order (pairs (i, ceil(n/2) + i), first words then second words, an odd n padded by one zero
 * counter whose output is dropped).  Not a Nx.Backend callback: a binding calls it from its
 * own random module when the key lives on the device. */
int hipnx_threefry2x32(hipnx_ctx *ctx, const hipnx_buf *key, int64_t n, hipnx_buf *out);

/* ---- fused element-wise chains ----------------------------------------------------------------
 * replaces: a group of element-wise callbacks that the reference's evaluator issues one by one
 * (nx/lib/nx/defn/evaluator.ex:363-388; the callbacks of nx/lib/nx/backend.ex:115-133) by one pass
 * over memory.  The group is a program for an accumulator machine: the accumulator holds the
 * value computed last, an instruction combines it with one other operand and rounds the result
 * to `dt`, the type the node has in the graph, so the final value is what the separate kernels
 * would have produced.
 *   SET     acc = other
 *   UNARY   acc = op(acc)                 op: HIPNX_EXP ... (not the integer-only ones)
 *   BINARY  acc = op(acc, other)          op: HIPNX_ADD ... (not the integer-only ones);
 *                                         flags bit 0: acc is the right operand, op(other, acc)
 *   SELECT  acc = acc != 0 ? other : other2
 *   AS_TYPE acc = acc (rounded to dt)
 * `other` is (src, arg, imm): input number arg (converted to f32; its element (row, col) is at
 * row * row_stride + col * col_stride), the constant imm, or saved slot arg; `other2` likewise
 * with (src2, arg2, imm2).  flags bits 4..7: slot + 1 in which the result is also saved (0: none).
 * The result of the last instruction is the output.  Types: bf16 / f16 / f32 values, u8 truth
 * values; inputs of at most 4 bytes per element.  The index space is [rows, cols]; col strides
 * are 1 or 0; cols, and with more than one row the row strides of dense inputs, are multiples
 * of 8 (otherwise HIPNX_EUNSUPPORTED: run the nodes one by one) -- except that with rows = 1 a compiled
 * kernel (HIPNX_FUSED_COMPILED) takes any cols: its last vector is partial.
 * reduce_op: -1, or HIPNX_RED_SUM / MAX / MIN to reduce the result along its rows without storing it
 * (sum/4, reduce_max/4, reduce_min/4 over the last axis, nx/lib/nx/backend.ex:89-92): `out` then has
 * `rows` elements, and equals the separate reduction kernel applied to the stored result (a few very long rows are
 * cut into segments by that kernel's own rule, their partial results kept in pool workspace and folded by its
 * second kernel: the same order of additions). */
enum { HIPNX_FUSED_SET = 0, HIPNX_FUSED_UNARY, HIPNX_FUSED_BINARY, HIPNX_FUSED_SELECT, HIPNX_FUSED_AS_TYPE,
       HIPNX_FUSED_BITCAST, HIPNX_FUSED_ROW_REDUCE, HIPNX_FUSED_ROW_STAT };
/* flags bit 1: the instruction works on 32-bit integers (dt u32 / s32) kept as raw bits -- a SET loads the
 * words of a 4-byte input, or the bits of imm, unconverted; a UNARY / BINARY computes like the integer
 * class of the separate kernels (wrapping at 32 bits); an AS_TYPE converts the integer of type `op` (an
 * element-type code) to the float dt; BITCAST (nx/lib/nx/backend.ex:69) relabels the bits.  These need
 * HIPNX_FUSED_COMPILED: the interpreting kernels return HIPNX_EUNSUPPORTED for them. */
enum { HIPNX_FUSED_FLAG_SWAP = 1, HIPNX_FUSED_FLAG_INT = 2, HIPNX_FUSED_FLAG_RESULT = 1 /* on a ROW_STAT */ };
enum { HIPNX_FUSED_SRC_CONST = 0, HIPNX_FUSED_SRC_INPUT, HIPNX_FUSED_SRC_SAVED, HIPNX_FUSED_SRC_ROWSTAT,
       HIPNX_FUSED_SRC_CARRY };
/* Stages over the same rows.  HIPNX_FUSED_ROW_REDUCE reduces the accumulator along the row (op =
 * HIPNX_RED_SUM / MAX / MIN, exactly as the reduction of the separate entry point would, the result stored
 * in type dt) and leaves that one value per row in the accumulator; the instructions that follow work on
 * it (a sum divided by the row length, an rsqrt of a variance, ...; operands are constants or earlier row
 * statistics) until HIPNX_FUSED_ROW_STAT ends the stage: the accumulator becomes row statistic number `arg`
 * (counted from 0 in program order), which later instructions read with source HIPNX_FUSED_SRC_ROWSTAT.
 * The next stage starts with a SET and empty slots; the last stage's value is the result.  Softmax over
 * rows is three stages of one program, a layer normalisation three as well.  In a stage that follows a
 * reducing one, source HIPNX_FUSED_SRC_CARRY is the value that stage reduced, element for element (it stays
 * in the lanes' registers): the softmax's division reads the exponentials its sum was taken over.  A ROW_STAT with flags bit 0
 * (HIPNX_FUSED_FLAG_RESULT) ends the program instead: that one value per row is the result (`out` has
 * `rows` elements) -- a log-sum-exp is two such stages.  Rows of more than 4096 elements
 * take a block each, as in the separate reduction; values are carried in registers for rows of up to 32768 elements
 * (HIPNX_EUNSUPPORTED for a program that reads them over longer rows, and for stages over the few very long rows
 * that the separate reduction cuts into segments: fewer than 8 rows per compute unit, 32768 elements or more each).
 * reduce_op = -1, HIPNX_FUSED_COMPILED only (HIPNX_EUNSUPPORTED otherwise). */
enum { HIPNX_FUSED_SAVED = 3, HIPNX_FUSED_MAX_INSTR = 32, HIPNX_FUSED_MAX_INPUTS = 8, HIPNX_FUSED_STATS = 3 };
typedef struct {
  uint8_t kind, op, src, arg;
  uint8_t src2, arg2, flags, dt;
  union { float imm; uint32_t imm_bits; };
  union { float imm2; uint32_t imm2_bits; };
} hipnx_fused_instr; /* 16 bytes: the interpreter fetches an instruction with one scalar load */
int hipnx_fused_elementwise(hipnx_ctx *ctx, int n_instr, const hipnx_fused_instr *prog, int n_inputs,
                            const hipnx_buf *const *inputs, const int *in_dts, const int64_t *in_row_strides,
                            const int *in_col_strides, int64_t rows, int64_t cols, int reduce_op, int out_dt,
                            hipnx_buf *out);

/* How hipnx_fused_elementwise runs a program on this context.  HIPNX_FUSED_INTERPRETED (the default):
 * one pair of kernels decodes any program, instruction by instruction.  HIPNX_FUSED_COMPILED: each
 * distinct program (instructions, input types and column strides, result type, reduction) is written
 * out over the same device functions, compiled for the device once by the run-time compiler (a few
 * hundred milliseconds) and kept with the context -- the role exla/lib/exla/defn.ex's compilation
 * cache plays for a whole function, here for one element-wise group.  Results are bit-identical in
 * both modes.  A program first met while the context is capturing runs interpreted in that capture.
 * A program's constants are part of what it is compiled for: one whose constant changes from call to
 * call compiles again for each value.  The context keeps at most 512 programs (another limit, at least
 * 4: hipnx_fused_set_cache_limit); when that many are held, the next new one first waits for the stream
 * and unloads the least recently launched quarter (those recorded into a graph stay).
 * hipnx_fused_compiled_count reports how many the context holds. */
enum { HIPNX_FUSED_INTERPRETED = 0, HIPNX_FUSED_COMPILED = 1 };
int hipnx_fused_set_mode(hipnx_ctx *ctx, int mode);
int hipnx_fused_set_cache_limit(hipnx_ctx *ctx, int programs);
int hipnx_fused_compiled_count(hipnx_ctx *ctx, int *count);

/* ---- captured sequences ---------------------------------------------------------------------
 * The reference's evaluator (nx/lib/nx/defn/evaluator.ex:363-388) issues one callback per node
 * on every call of a compiled function; the XLA-based backend compiles the function instead
 * (exla/lib/exla/defn.ex).  This is the device-side middle: between capture_begin and
 * capture_end the entry points of the context record their kernels instead of running them,
 * capture_end turns the record into an executable graph, graph_launch replays it on the
 * context's stream with one submission.  Every device block handed out while capturing stays
 * with the graph until graph_destroy (a replay writes to the same addresses), so buffers
 * allocated during the capture -- the results among them -- are overwritten by each replay.
 * Entry points that wait for the device (h2d, d2h, sync, trim, the timer, gather with
 * HIPNX_OOB_RAISE) return HIPNX_EUNSUPPORTED while capturing.  Run the sequence once before
 * capturing it: kernel attributes are set and the pool holds its block sizes after that.  One
 * thread drives a capture; graphs must be destroyed before their context. */
int hipnx_capture_begin(hipnx_ctx *ctx);
int hipnx_capture_end(hipnx_ctx *ctx, hipnx_graph **out);
int hipnx_graph_launch(hipnx_graph *graph);
int hipnx_graph_destroy(hipnx_graph *graph);

#ifdef __cplusplus
}
#endif
#endif
