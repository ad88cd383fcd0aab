/*
 * hipnx_nif.c -- erl_nif shim over libhipnx (include/hipnx.h): plain C, one NIF per C-ABI entry
 * point, no logic of its own.
 *
 * Follows the conventions of the reference's native backends:
 *  - module loaded from priv/ by `:erlang.load_nif/2` in HipNx.NIF (torchx/lib/torchx/nif.ex:3-16);
 *  - every NIF returns {:ok, term} | {:error, charlist} (torchx/lib/torchx.ex:476-491);
 *  - transfers and compute run on dirty IO schedulers (exla/c_src/exla/exla.cc:445,453,475);
 *  - a device buffer is a resource whose destructor releases it, explicit deallocation is
 *    idempotent and reported as :ok | :already_deallocated (torchx/c_src/torchx_nif_util.h:66-111).
 *
 * NOT BUILT IN THIS REPOSITORY'S CONTAINER: it needs erl_nif.h (ERTS), which is absent there.
 * Build: cc -shared -fPIC -I$ERTS_INCLUDE_DIR -I../../../include hipnx_nif.c -L../../lib -lhipnx
 */
#include <erl_nif.h>
#include <string.h>

#include "hipnx.h"

static ErlNifResourceType *CTX_TYPE, *BUF_TYPE;
typedef struct { hipnx_ctx *ctx; } ctx_res;
typedef struct { hipnx_buf *buf; } buf_res;

static void ctx_dtor(ErlNifEnv *env, void *obj) { (void)env; /* contexts live for the VM's life */ (void)obj; }
static void buf_dtor(ErlNifEnv *env, void *obj) {
  (void)env;
  buf_res *b = (buf_res *)obj;
  if (b->buf) hipnx_buf_destroy(b->buf);
}

static ERL_NIF_TERM ok(ErlNifEnv *env, ERL_NIF_TERM t) { return enif_make_tuple2(env, enif_make_atom(env, "ok"), t); }
static ERL_NIF_TERM error_from_status(ErlNifEnv *env, int status) {
  char msg[512];
  hipnx_last_error(msg, sizeof msg);
  /* {:error, {status, charlist}}: the Elixir side raises ArgumentError for EINVAL / EINDEX */
  return enif_make_tuple2(env, enif_make_atom(env, "error"),
                          enif_make_tuple2(env, enif_make_int(env, status), enif_make_string(env, msg, ERL_NIF_LATIN1)));
}
#define CHECK(call) do { int st__ = (call); if (st__ != HIPNX_OK) return error_from_status(env, st__); } while (0)
#define GET_CTX(i, v) ctx_res *v##_r; if (!enif_get_resource(env, argv[i], CTX_TYPE, (void **)&v##_r)) return enif_make_badarg(env); hipnx_ctx *v = v##_r->ctx
#define GET_BUF(i, v) buf_res *v##_r; if (!enif_get_resource(env, argv[i], BUF_TYPE, (void **)&v##_r)) return enif_make_badarg(env); hipnx_buf *v = v##_r->buf
#define GET_INT(i, v) int v; if (!enif_get_int(env, argv[i], &v)) return enif_make_badarg(env)
#define GET_I64(i, v) ErlNifSInt64 v; if (!enif_get_int64(env, argv[i], &v)) return enif_make_badarg(env)

static int get_i64_list(ErlNifEnv *env, ERL_NIF_TERM list, int64_t *dst, int max, int *n) {
  unsigned len;
  if (!enif_get_list_length(env, list, &len) || (int)len > max) return 0;
  ERL_NIF_TERM head, tail = list;
  for (unsigned i = 0; i < len; i++) {
    ErlNifSInt64 v;
    if (!enif_get_list_cell(env, tail, &head, &tail) || !enif_get_int64(env, head, &v)) return 0;
    dst[i] = v;
  }
  *n = (int)len;
  return 1;
}

static ERL_NIF_TERM make_buf(ErlNifEnv *env, hipnx_buf *buf) {
  buf_res *r = (buf_res *)enif_alloc_resource(BUF_TYPE, sizeof(buf_res));
  r->buf = buf;
  ERL_NIF_TERM t = enif_make_resource(env, r);
  enif_release_resource(r);
  return t;
}

/* ctx_create(device) */
static ERL_NIF_TERM nif_ctx_create(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_INT(0, device);
  hipnx_ctx *ctx;
  CHECK(hipnx_ctx_create(device, &ctx));
  ctx_res *r = (ctx_res *)enif_alloc_resource(CTX_TYPE, sizeof(ctx_res));
  r->ctx = ctx;
  ERL_NIF_TERM t = enif_make_resource(env, r);
  enif_release_resource(r);
  return ok(env, t);
}

static ERL_NIF_TERM nif_device_count(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc; (void)argv;
  int n = 0;
  CHECK(hipnx_device_count(&n));
  return ok(env, enif_make_int(env, n));
}

/* from_binary(ctx, binary, nbytes): H2D of an Erlang binary (from_binary/3, constant via fill) */
static ERL_NIF_TERM nif_from_binary(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx);
  ErlNifBinary bin;
  if (!enif_inspect_binary(env, argv[1], &bin)) return enif_make_badarg(env);
  GET_I64(2, need);
  if ((ErlNifSInt64)bin.size < need) {
    return enif_make_tuple2(env, enif_make_atom(env, "error"),
                            enif_make_tuple2(env, enif_make_int(env, HIPNX_EINVAL),
                                             enif_make_string(env, "binary size is too small for the requested shape", ERL_NIF_LATIN1)));
  }
  hipnx_buf *buf;
  CHECK(hipnx_buf_alloc(ctx, (size_t)need, &buf));
  int st = hipnx_h2d(ctx, buf, 0, bin.data, (size_t)need);
  if (st != HIPNX_OK) { hipnx_buf_destroy(buf); return error_from_status(env, st); }
  return ok(env, make_buf(env, buf));
}

/* to_binary(ctx, buf, nbytes) */
static ERL_NIF_TERM nif_to_binary(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx); GET_BUF(1, buf); GET_I64(2, nbytes);
  ERL_NIF_TERM term;
  unsigned char *dst = enif_make_new_binary(env, (size_t)nbytes, &term);
  CHECK(hipnx_d2h(ctx, buf, 0, dst, (size_t)nbytes));
  return ok(env, term);
}

static ERL_NIF_TERM nif_alloc(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx); GET_I64(1, nbytes);
  hipnx_buf *buf;
  CHECK(hipnx_buf_alloc(ctx, (size_t)nbytes, &buf));
  return ok(env, make_buf(env, buf));
}

/* deallocate(buf) -> :ok | :already_deallocated */
static ERL_NIF_TERM nif_deallocate(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_BUF(0, buf);
  int st = hipnx_buf_free(buf);
  if (st == HIPNX_OK) return enif_make_atom(env, "ok");
  if (st == HIPNX_ALREADY_FREED) return enif_make_atom(env, "already_deallocated");
  return error_from_status(env, st);
}

static ERL_NIF_TERM nif_copy(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx); GET_BUF(1, src); GET_I64(2, nbytes);
  hipnx_buf *dst;
  CHECK(hipnx_buf_alloc(ctx, (size_t)nbytes, &dst));
  int st = hipnx_d2d(ctx, dst, 0, src, 0, (size_t)nbytes);
  if (st != HIPNX_OK) { hipnx_buf_destroy(dst); return error_from_status(env, st); }
  return ok(env, make_buf(env, dst));
}

/* fill(ctx, elem_binary, count) */
static ERL_NIF_TERM nif_fill(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx);
  ErlNifBinary elem;
  if (!enif_inspect_binary(env, argv[1], &elem)) return enif_make_badarg(env);
  GET_I64(2, n);
  hipnx_buf *buf;
  CHECK(hipnx_buf_alloc(ctx, (size_t)n * elem.size, &buf));
  int st = hipnx_fill(ctx, buf, (int)elem.size, elem.data, n);
  if (st != HIPNX_OK) { hipnx_buf_destroy(buf); return error_from_status(env, st); }
  return ok(env, make_buf(env, buf));
}

/* binary(ctx, op, l_dt, r_dt, out_dt, out_dims, l_strides, r_strides, l, r, out_bytes) */
static ERL_NIF_TERM nif_binary(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx); GET_INT(1, op); GET_INT(2, ldt); GET_INT(3, rdt); GET_INT(4, odt);
  int64_t dims[64], ls[64], rs[64];
  int rank, n1, n2;
  if (!get_i64_list(env, argv[5], dims, 64, &rank) || !get_i64_list(env, argv[6], ls, 64, &n1) ||
      !get_i64_list(env, argv[7], rs, 64, &n2) || n1 != rank || n2 != rank) return enif_make_badarg(env);
  GET_BUF(8, l); GET_BUF(9, r); GET_I64(10, out_bytes);
  hipnx_buf *out;
  CHECK(hipnx_buf_alloc(ctx, (size_t)out_bytes, &out));
  int st = hipnx_binary(ctx, op, ldt, rdt, odt, rank, dims, ls, rs, l, r, out);
  if (st != HIPNX_OK) { hipnx_buf_destroy(out); return error_from_status(env, st); }
  return ok(env, make_buf(env, out));
}

/* unary(ctx, op, in_dt, out_dt, n, in, out_bytes); op = -1 selects as_type */
static ERL_NIF_TERM nif_unary(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx); GET_INT(1, op); GET_INT(2, idt); GET_INT(3, odt); GET_I64(4, n); GET_BUF(5, in); GET_I64(6, out_bytes);
  hipnx_buf *out;
  CHECK(hipnx_buf_alloc(ctx, (size_t)out_bytes, &out));
  int st = op < 0 ? hipnx_as_type(ctx, idt, odt, n, in, out) : hipnx_unary(ctx, op, idt, odt, n, in, out);
  if (st != HIPNX_OK) { hipnx_buf_destroy(out); return error_from_status(env, st); }
  return ok(env, make_buf(env, out));
}

/* reduce(ctx, op, in_dt, out_dt, outer, red, inner, in, out_bytes) */
static ERL_NIF_TERM nif_reduce(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx); GET_INT(1, op); GET_INT(2, idt); GET_INT(3, odt); GET_I64(4, outer); GET_I64(5, red); GET_I64(6, inner);
  GET_BUF(7, in); GET_I64(8, out_bytes);
  hipnx_buf *out;
  CHECK(hipnx_buf_alloc(ctx, (size_t)out_bytes, &out));
  int st = hipnx_reduce(ctx, op, idt, odt, outer, red, inner, in, out);
  if (st != HIPNX_OK) { hipnx_buf_destroy(out); return error_from_status(env, st); }
  return ok(env, make_buf(env, out));
}

/* argreduce(ctx, op, tie, in_dt, out_dt, outer, red, inner, in, out_bytes) */
static ERL_NIF_TERM nif_argreduce(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx); GET_INT(1, op); GET_INT(2, tie); GET_INT(3, idt); GET_INT(4, odt); GET_I64(5, outer); GET_I64(6, red);
  GET_I64(7, inner); GET_BUF(8, in); GET_I64(9, out_bytes);
  hipnx_buf *out;
  CHECK(hipnx_buf_alloc(ctx, (size_t)out_bytes, &out));
  int st = hipnx_argreduce(ctx, op, tie, idt, odt, outer, red, inner, in, out);
  if (st != HIPNX_OK) { hipnx_buf_destroy(out); return error_from_status(env, st); }
  return ok(env, make_buf(env, out));
}

/* dot(ctx, l_dt, r_dt, out_dt, batch, m, n, k, l_layout, r_layout, l, r, out_bytes) */
static ERL_NIF_TERM nif_dot(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx); GET_INT(1, ldt); GET_INT(2, rdt); GET_INT(3, odt); GET_I64(4, batch); GET_I64(5, m); GET_I64(6, n);
  GET_I64(7, k); GET_INT(8, ll); GET_INT(9, rl); GET_BUF(10, l); GET_BUF(11, r); GET_I64(12, out_bytes);
  hipnx_buf *out;
  CHECK(hipnx_buf_alloc(ctx, (size_t)out_bytes, &out));
  int st = hipnx_dot(ctx, ldt, rdt, odt, batch, m, n, k, ll, rl, l, r, out);
  if (st != HIPNX_OK) { hipnx_buf_destroy(out); return error_from_status(env, st); }
  return ok(env, make_buf(env, out));
}

/* transpose(ctx, elem_bytes, in_dims, perm, in, out_bytes) */
static ERL_NIF_TERM nif_transpose(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx); GET_INT(1, esz);
  int64_t dims[64], perm64[64];
  int perm[64], rank, n1;
  if (!get_i64_list(env, argv[2], dims, 64, &rank) || !get_i64_list(env, argv[3], perm64, 64, &n1) || n1 != rank)
    return enif_make_badarg(env);
  for (int i = 0; i < rank; i++) perm[i] = (int)perm64[i];
  GET_BUF(4, in); GET_I64(5, out_bytes);
  hipnx_buf *out;
  CHECK(hipnx_buf_alloc(ctx, (size_t)out_bytes, &out));
  int st = hipnx_transpose(ctx, esz, rank, dims, perm, in, out);
  if (st != HIPNX_OK) { hipnx_buf_destroy(out); return error_from_status(env, st); }
  return ok(env, make_buf(env, out));
}

/* broadcast(ctx, elem_bytes, out_dims, in_strides, in, out_bytes) */
static ERL_NIF_TERM nif_broadcast(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx); GET_INT(1, esz);
  int64_t dims[64], strides[64];
  int rank, n1;
  if (!get_i64_list(env, argv[2], dims, 64, &rank) || !get_i64_list(env, argv[3], strides, 64, &n1) || n1 != rank)
    return enif_make_badarg(env);
  GET_BUF(4, in); GET_I64(5, out_bytes);
  hipnx_buf *out;
  CHECK(hipnx_buf_alloc(ctx, (size_t)out_bytes, &out));
  int st = hipnx_broadcast(ctx, esz, rank, dims, strides, in, out);
  if (st != HIPNX_OK) { hipnx_buf_destroy(out); return error_from_status(env, st); }
  return ok(env, make_buf(env, out));
}

/* gather(ctx, elem_bytes, t_dims, idx_dt, n_tuples, depth, oob_policy, t, idx, out_bytes) */
static ERL_NIF_TERM nif_gather(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx); GET_INT(1, esz);
  int64_t dims[64];
  int rank;
  if (!get_i64_list(env, argv[2], dims, 64, &rank)) return enif_make_badarg(env);
  GET_INT(3, idt); GET_I64(4, n_tuples); GET_INT(5, depth); GET_INT(6, policy); GET_BUF(7, t); GET_BUF(8, idx); GET_I64(9, out_bytes);
  hipnx_buf *out;
  CHECK(hipnx_buf_alloc(ctx, (size_t)out_bytes, &out));
  int st = hipnx_gather(ctx, esz, rank, dims, idt, n_tuples, depth, policy, t, idx, out);
  if (st != HIPNX_OK) { hipnx_buf_destroy(out); return error_from_status(env, st); }
  return ok(env, make_buf(env, out));
}

/* take(ctx, elem_bytes, outer, axis_len, inner, idx_dt, n_idx, oob_policy, msg_dims, t, idx, out_bytes) */
static ERL_NIF_TERM nif_take(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx); GET_INT(1, esz); GET_I64(2, outer); GET_I64(3, axis_len); GET_I64(4, inner); GET_INT(5, idt); GET_I64(6, n_idx);
  GET_INT(7, policy);
  int64_t dims[64];
  int rank;
  if (!get_i64_list(env, argv[8], dims, 64, &rank)) return enif_make_badarg(env);
  GET_BUF(9, t); GET_BUF(10, idx); GET_I64(11, out_bytes);
  hipnx_buf *out;
  CHECK(hipnx_buf_alloc(ctx, (size_t)out_bytes, &out));
  int st = hipnx_take(ctx, esz, outer, axis_len, inner, idt, n_idx, policy, rank, dims, t, idx, out);
  if (st != HIPNX_OK) { hipnx_buf_destroy(out); return error_from_status(env, st); }
  return ok(env, make_buf(env, out));
}

/* select(ctx, pred_dt, true_dt, false_dt, out_dt, out_dims, pred_strides, true_strides, false_strides, pred, on_true, on_false, out_bytes) */
static ERL_NIF_TERM nif_select(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx); GET_INT(1, pdt); GET_INT(2, tdt); GET_INT(3, fdt); GET_INT(4, odt);
  int64_t dims[64], ps[64], ts[64], fs[64];
  int rank, n1, n2, n3;
  if (!get_i64_list(env, argv[5], dims, 64, &rank) || !get_i64_list(env, argv[6], ps, 64, &n1) ||
      !get_i64_list(env, argv[7], ts, 64, &n2) || !get_i64_list(env, argv[8], fs, 64, &n3) || n1 != rank || n2 != rank ||
      n3 != rank)
    return enif_make_badarg(env);
  GET_BUF(9, pred); GET_BUF(10, on_true); GET_BUF(11, on_false); GET_I64(12, out_bytes);
  hipnx_buf *out;
  CHECK(hipnx_buf_alloc(ctx, (size_t)out_bytes, &out));
  int st = hipnx_select(ctx, pdt, tdt, fdt, odt, rank, dims, ps, ts, fs, pred, on_true, on_false, out);
  if (st != HIPNX_OK) { hipnx_buf_destroy(out); return error_from_status(env, st); }
  return ok(env, make_buf(env, out));
}

/* clip(ctx, in_dt, min_dt, max_dt, out_dt, n, in, min, max, out_bytes) */
static ERL_NIF_TERM nif_clip(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx); GET_INT(1, idt); GET_INT(2, mndt); GET_INT(3, mxdt); GET_INT(4, odt); GET_I64(5, n);
  GET_BUF(6, in); GET_BUF(7, mn); GET_BUF(8, mx); GET_I64(9, out_bytes);
  hipnx_buf *out;
  CHECK(hipnx_buf_alloc(ctx, (size_t)out_bytes, &out));
  int st = hipnx_clip(ctx, idt, mndt, mxdt, odt, n, in, mn, mx, out);
  if (st != HIPNX_OK) { hipnx_buf_destroy(out); return error_from_status(env, st); }
  return ok(env, make_buf(env, out));
}

/* strided_copy(ctx, elem_bytes, dims, in_strides, in_offset, out_strides, out_offset, in, out | out_bytes):
 * the last argument is either a buffer to write into (a concatenation fills one output window
 * by window; buffers are only ever written before they are published as a tensor) or the size
 * of a fresh one */
static ERL_NIF_TERM nif_strided_copy(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx); GET_INT(1, esz);
  int64_t dims[64], is[64], os[64];
  int rank, n1, n2;
  if (!get_i64_list(env, argv[2], dims, 64, &rank) || !get_i64_list(env, argv[3], is, 64, &n1) ||
      !get_i64_list(env, argv[5], os, 64, &n2) || n1 != rank || n2 != rank)
    return enif_make_badarg(env);
  GET_I64(4, in_off); GET_I64(6, out_off); GET_BUF(7, in);
  buf_res *dst;
  if (enif_get_resource(env, argv[8], BUF_TYPE, (void **)&dst)) {
    CHECK(hipnx_strided_copy(ctx, esz, rank, dims, is, in_off, os, out_off, in, dst->buf));
    return ok(env, argv[8]);
  }
  GET_I64(8, out_bytes);
  hipnx_buf *out;
  CHECK(hipnx_buf_alloc(ctx, (size_t)out_bytes, &out));
  int st = hipnx_strided_copy(ctx, esz, rank, dims, is, in_off, os, out_off, in, out);
  if (st != HIPNX_OK) { hipnx_buf_destroy(out); return error_from_status(env, st); }
  return ok(env, make_buf(env, out));
}

/* iota(ctx, out_dt, n, dim, inner, out_bytes) */
static ERL_NIF_TERM nif_iota(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx); GET_INT(1, odt); GET_I64(2, n); GET_I64(3, dim); GET_I64(4, inner); GET_I64(5, out_bytes);
  hipnx_buf *out;
  CHECK(hipnx_buf_alloc(ctx, (size_t)out_bytes, &out));
  int st = hipnx_iota(ctx, odt, n, dim, inner, out);
  if (st != HIPNX_OK) { hipnx_buf_destroy(out); return error_from_status(env, st); }
  return ok(env, make_buf(env, out));
}

/* eye(ctx, out_dt, n, rows, cols, out_bytes) */
static ERL_NIF_TERM nif_eye(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx); GET_INT(1, odt); GET_I64(2, n); GET_I64(3, rows); GET_I64(4, cols); GET_I64(5, out_bytes);
  hipnx_buf *out;
  CHECK(hipnx_buf_alloc(ctx, (size_t)out_bytes, &out));
  int st = hipnx_eye(ctx, odt, n, rows, cols, out);
  if (st != HIPNX_OK) { hipnx_buf_destroy(out); return error_from_status(env, st); }
  return ok(env, make_buf(env, out));
}

/* threefry2x32(ctx, key, n, out_bytes) */
static ERL_NIF_TERM nif_threefry2x32(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx); GET_BUF(1, key); GET_I64(2, n); GET_I64(3, out_bytes);
  hipnx_buf *out;
  CHECK(hipnx_buf_alloc(ctx, (size_t)out_bytes, &out));
  int st = hipnx_threefry2x32(ctx, key, n, out);
  if (st != HIPNX_OK) { hipnx_buf_destroy(out); return error_from_status(env, st); }
  return ok(env, make_buf(env, out));
}

/* narrow_int(ctx, buf, n, bits, signed): in place on a callback's fresh output; returns the same buffer */
static ERL_NIF_TERM nif_narrow_int(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx); GET_BUF(1, buf); GET_I64(2, n); GET_INT(3, bits); GET_INT(4, is_signed);
  CHECK(hipnx_narrow_int(ctx, buf, n, bits, is_signed));
  return ok(env, argv[1]);
}

/* device_ptr(buf) -> {:ok, address}: the :local pointer of to_pointer/2 */
static ERL_NIF_TERM nif_device_ptr(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_BUF(0, buf);
  void *p = hipnx_buf_device_ptr(buf);
  if (!p) return error_from_status(env, HIPNX_EFREED);
  return ok(env, enif_make_uint64(env, (ErlNifUInt64)(uintptr_t)p));
}

/* wrap(ctx, address, nbytes): from_pointer/5 for a :local pointer; the memory stays with its owner */
static ERL_NIF_TERM nif_wrap(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx);
  ErlNifUInt64 address;
  if (!enif_get_uint64(env, argv[1], &address)) return enif_make_badarg(env);
  GET_I64(2, nbytes);
  hipnx_buf *buf;
  CHECK(hipnx_buf_wrap(ctx, (void *)(uintptr_t)address, (size_t)nbytes, &buf));
  return ok(env, make_buf(env, buf));
}

/* ipc_export(ctx, buf) -> {:ok, handle_binary}: the :ipc pointer of to_pointer/2 (64 bytes another OS
 * process opens with ipc_import) */
static ERL_NIF_TERM nif_ipc_export(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx); GET_BUF(1, buf);
  ERL_NIF_TERM term;
  unsigned char *dst = enif_make_new_binary(env, HIPNX_IPC_HANDLE_BYTES, &term);
  CHECK(hipnx_buf_ipc_export(ctx, buf, dst));
  return ok(env, term);
}

/* ipc_import(ctx, handle_binary, nbytes): from_pointer/5 for an :ipc pointer; the memory stays with the
 * exporting process, destroying the buffer closes the mapping */
static ERL_NIF_TERM nif_ipc_import(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx);
  ErlNifBinary handle;
  if (!enif_inspect_binary(env, argv[1], &handle) || handle.size != HIPNX_IPC_HANDLE_BYTES) return enif_make_badarg(env);
  GET_I64(2, nbytes);
  hipnx_buf *buf;
  CHECK(hipnx_buf_ipc_import(ctx, handle.data, (size_t)nbytes, &buf));
  return ok(env, make_buf(env, buf));
}

static ERL_NIF_TERM nif_sync(ErlNifEnv *env, int argc, const ERL_NIF_TERM argv[]) {
  (void)argc;
  GET_CTX(0, ctx);
  CHECK(hipnx_sync(ctx));
  return enif_make_atom(env, "ok");
}

static int on_load(ErlNifEnv *env, void **priv, ERL_NIF_TERM info) {
  (void)priv; (void)info;
  CTX_TYPE = enif_open_resource_type(env, NULL, "hipnx_ctx", ctx_dtor, ERL_NIF_RT_CREATE, NULL);
  BUF_TYPE = enif_open_resource_type(env, NULL, "hipnx_buf", buf_dtor, ERL_NIF_RT_CREATE, NULL);
  return (CTX_TYPE && BUF_TYPE) ? 0 : 1;
}

#define IO ERL_NIF_DIRTY_JOB_IO_BOUND
static ErlNifFunc funcs[] = {
    {"device_count", 0, nif_device_count, 0},   {"ctx_create", 1, nif_ctx_create, IO},
    {"from_binary", 3, nif_from_binary, IO},    {"to_binary", 3, nif_to_binary, IO},
    {"alloc", 2, nif_alloc, IO},                {"deallocate", 1, nif_deallocate, IO},
    {"copy", 3, nif_copy, IO},                  {"fill", 3, nif_fill, IO},
    {"binary", 11, nif_binary, IO},             {"unary", 7, nif_unary, IO},
    {"reduce", 9, nif_reduce, IO},              {"argreduce", 10, nif_argreduce, IO},
    {"dot", 13, nif_dot, IO},                   {"transpose", 6, nif_transpose, IO},
    {"broadcast", 6, nif_broadcast, IO},        {"gather", 10, nif_gather, IO},
    {"select", 13, nif_select, IO},             {"clip", 10, nif_clip, IO},
    {"strided_copy", 9, nif_strided_copy, IO},  {"iota", 6, nif_iota, IO},
    {"narrow_int", 5, nif_narrow_int, IO},      {"device_ptr", 1, nif_device_ptr, 0},
    {"wrap", 3, nif_wrap, 0},                   {"ipc_export", 2, nif_ipc_export, IO},
    {"ipc_import", 3, nif_ipc_import, IO},
    {"take", 12, nif_take, IO},
    {"eye", 6, nif_eye, IO},                    {"threefry2x32", 4, nif_threefry2x32, IO},
    {"sync", 1, nif_sync, IO}};

ERL_NIF_INIT(Elixir.HipNx.NIF, funcs, on_load, NULL, NULL, NULL)
