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
  if (red > 0x7FFFFFFF) return set_error(HIPNX_EUNSUPPORTED, "argreduce: more than 2^31 - 1 elements along the reduced axis");
  if (int st = check_buf(ctx, inb, (uint64_t)outer * red * inner * dtype_size(in_dt), "argreduce in")) return st;
  if (int st = check_buf(ctx, out, (uint64_t)outer * inner * dtype_size(out_dt), "argreduce out")) return st;
  if (outer * inner == 0) return HIPNX_OK;
  const void *ip = inb->ptr;
  void *op_ = out->ptr;
  int st;
  if (op == HIPNX_ARGMAX)
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
