// argmax / argmin (a translation unit of its own: see reduce.hip)
#include "reduce_kernels.cuh"

namespace hipnx {

template <int OP, int TIE>
static int argreduce_op(hipnx_ctx *ctx, int idt, int odt, int64_t outer, int64_t red, int64_t inner, const void *in,
                        void *out) {
  if (is_float(idt) && idt != HIPNX_F64)
    return run_reduce<ArgReducer<float, OP, TIE, false>, float>(ctx, false, idt, odt, outer, red, inner, in, out);
  if (is_float(idt)) return run_reduce<ArgReducer<double, OP, TIE, false>, double>(ctx, false, idt, odt, outer, red, inner, in, out);
  if (idt == HIPNX_U64) return run_reduce<ArgReducer<int64_t, OP, TIE, true>, int64_t>(ctx, false, idt, odt, outer, red, inner, in, out);
  return run_reduce<ArgReducer<int64_t, OP, TIE, false>, int64_t>(ctx, false, idt, odt, outer, red, inner, in, out);
}

// An axis of 2^31 positions or more (the kernels above keep a position in 32 bits) under outer == 1: the axis is cut
// into chunks of 2^30 positions -- each a dense [1, length, inner] view of its own -- whose positions go to a workspace
// as s64; this kernel then walks the chunks of one output in order, reads the value each chunk found, and keeps the
// better pair by the reducer's own rules (NaN beats numbers and the later NaN wins; ties by tie_break).
constexpr int64_t ARG_CHUNK = (int64_t)1 << 30;

template <typename CT, int OP, int TIE, bool UNS>
__global__ void __launch_bounds__(256)
arg_chunks_combine_kernel(const void *__restrict__ in, int idt, const int64_t *__restrict__ found, void *__restrict__ out, int odt,
                          int64_t inner, int chunks) {
  typedef ArgReducer<CT, OP, TIE, UNS> R;
  for (int64_t j = (int64_t)blockIdx.x * 256 + threadIdx.x; j < inner; j += (int64_t)gridDim.x * 256) {
    int64_t best_i = found[j];
    CT best_v = load_one<CT>(in, idt, best_i * inner + j);
    for (int c = 1; c < chunks; c++) {
      const int64_t i = (int64_t)c * ARG_CHUNK + found[(int64_t)c * inner + j];  // (later than every position before it)
      const CT v = load_one<CT>(in, idt, i * inner + j);
      bool take;
      if (R::FP && (v != v || best_v != best_v)) take = v != v;  // a NaN beats a number, the later of two NaNs wins
      else take = TIE == HIPNX_TIE_LOW ? R::better(v, best_v) : R::better_or_equal(v, best_v);
      if (take) best_v = v, best_i = i;
    }
    store_one<int64_t>(out, odt, j, best_i);
  }
}

template <int OP, int TIE>
static int argreduce_chunked(hipnx_ctx *ctx, int idt, int odt, int64_t red, int64_t inner, const void *in, void *out) {
  const int chunks = (int)((red + ARG_CHUNK - 1) / ARG_CHUNK);
  void *ws = nullptr;
  size_t ws_cap = 0;
  if (int st = pool_alloc(ctx, (size_t)chunks * inner * 8, &ws, &ws_cap)) return st;
  int st = HIPNX_OK;
  for (int c = 0; c < chunks && st == HIPNX_OK; c++) {
    const int64_t first = (int64_t)c * ARG_CHUNK, len = red - first < ARG_CHUNK ? red - first : ARG_CHUNK;
    st = argreduce_op<OP, TIE>(ctx, idt, HIPNX_S64, 1, len, inner, (const unsigned char *)in + first * inner * dtype_size(idt),
                               (int64_t *)ws + (int64_t)c * inner);
  }
  if (st == HIPNX_OK) {
    const dim3 grid((unsigned)std::min<int64_t>((inner + 255) / 256, 65535)), block(256);
    const int64_t *found = (const int64_t *)ws;
    if (is_float(idt) && idt != HIPNX_F64)
      hipLaunchKernelGGL((arg_chunks_combine_kernel<float, OP, TIE, false>), grid, block, 0, ctx->stream, in, idt, found, out, odt, inner, chunks);
    else if (is_float(idt))
      hipLaunchKernelGGL((arg_chunks_combine_kernel<double, OP, TIE, false>), grid, block, 0, ctx->stream, in, idt, found, out, odt, inner, chunks);
    else if (idt == HIPNX_U64)
      hipLaunchKernelGGL((arg_chunks_combine_kernel<int64_t, OP, TIE, true>), grid, block, 0, ctx->stream, in, idt, found, out, odt, inner, chunks);
    else
      hipLaunchKernelGGL((arg_chunks_combine_kernel<int64_t, OP, TIE, false>), grid, block, 0, ctx->stream, in, idt, found, out, odt, inner, chunks);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) st = hip_fail(e, "argreduce chunk combine launch");
  }
  pool_free(ctx, ws, ws_cap);  // later work is ordered on the same stream
  return st;
}

}  // namespace hipnx

using namespace hipnx;

static int check_view(int64_t outer, int64_t red, int64_t inner) {
  if (outer < 0 || red < 0 || inner < 0) return set_error(HIPNX_EINVAL, "reduce: negative extent");
  return HIPNX_OK;
}

extern "C" int hipnx_argreduce(hipnx_ctx *ctx, int op, int tie, int in_dt, int out_dt, int64_t outer, int64_t red,
                               int64_t inner, const hipnx_buf *inb, hipnx_buf *out) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (op < 0 || op > HIPNX_ARGMIN || tie < 0 || tie > HIPNX_TIE_HIGH)
    return set_error(HIPNX_EINVAL, "argreduce: unknown op / tie_break");
  if (dtype_size(in_dt) < 0 || dtype_size(out_dt) < 0 || is_float(out_dt))
    return set_error(HIPNX_EINVAL, "argreduce: bad element type (the output must be an integer type)");
  if (int st = check_view(outer, red, inner)) return st;
  if (red == 0 && outer * inner > 0) return set_error(HIPNX_EINVAL, "argreduce: empty axis");
  const bool chunked = red > 0x7FFFFFFF;
  if (chunked && outer != 1)
    return set_error(HIPNX_EUNSUPPORTED, "argreduce: more than 2^31 - 1 elements along the reduced axis under more than one outer index");
  if (int st = check_buf(ctx, inb, (uint64_t)outer * red * inner * dtype_size(in_dt), "argreduce in")) return st;
  if (int st = check_buf(ctx, out, (uint64_t)outer * inner * dtype_size(out_dt), "argreduce out")) return st;
  if (outer * inner == 0) return HIPNX_OK;
  const void *ip = inb->ptr;
  void *op_ = out->ptr;
  int st;
  if (chunked) {
    if (op == HIPNX_ARGMAX)
      st = tie == HIPNX_TIE_LOW ? argreduce_chunked<HIPNX_ARGMAX, HIPNX_TIE_LOW>(ctx, in_dt, out_dt, red, inner, ip, op_)
                                : argreduce_chunked<HIPNX_ARGMAX, HIPNX_TIE_HIGH>(ctx, in_dt, out_dt, red, inner, ip, op_);
    else
      st = tie == HIPNX_TIE_LOW ? argreduce_chunked<HIPNX_ARGMIN, HIPNX_TIE_LOW>(ctx, in_dt, out_dt, red, inner, ip, op_)
                                : argreduce_chunked<HIPNX_ARGMIN, HIPNX_TIE_HIGH>(ctx, in_dt, out_dt, red, inner, ip, op_);
  } else if (op == HIPNX_ARGMAX)
    st = tie == HIPNX_TIE_LOW ? argreduce_op<HIPNX_ARGMAX, HIPNX_TIE_LOW>(ctx, in_dt, out_dt, outer, red, inner, ip, op_)
                              : argreduce_op<HIPNX_ARGMAX, HIPNX_TIE_HIGH>(ctx, in_dt, out_dt, outer, red, inner, ip, op_);
  else
    st = tie == HIPNX_TIE_LOW ? argreduce_op<HIPNX_ARGMIN, HIPNX_TIE_LOW>(ctx, in_dt, out_dt, outer, red, inner, ip, op_)
                              : argreduce_op<HIPNX_ARGMIN, HIPNX_TIE_HIGH>(ctx, in_dt, out_dt, outer, red, inner, ip, op_);
  // every value written is an index along the reduced axis: in [0, red) unless the output type is too narrow
  // to hold red - 1 (the index is then written wrapped, shared.ex:190-194, and nothing is claimed)
  const int bits = 8 * dtype_size(out_dt) - (is_unsigned(out_dt) ? 0 : 1);
  if (st == HIPNX_OK && !out->borrowed && (bits >= 63 || red - 1 < ((int64_t)1 << bits))) {
    out->index_bound = red;
    out->index_bytes = (uint64_t)outer * inner * dtype_size(out_dt);
    out->index_dt = out_dt;
  }
  return st;
}
