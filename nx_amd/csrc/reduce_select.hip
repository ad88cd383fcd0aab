// reduce_max / reduce_min / all / any (a translation unit of its own: see reduce.hip)
#include "reduce_kernels.cuh"

namespace hipnx {

template <int OP>
static int reduce_op(hipnx_ctx *ctx, bool static_ws, int idt, int odt, int64_t outer, int64_t red, int64_t inner, const void *in,
                     void *out) {
  // selection (max / min) is exact in the element's own precision: f32 covers f32, bf16 and f16
  if (is_float(idt) && idt != HIPNX_F64 && (OP == HIPNX_RED_MAX || OP == HIPNX_RED_MIN || OP == HIPNX_RED_ALL || OP == HIPNX_RED_ANY))
    return run_reduce<PlainReducer<float, OP, false>, float>(ctx, static_ws, idt, odt, outer, red, inner, in, out);
  if (is_float(idt)) return run_reduce<PlainReducer<double, OP, false>, double>(ctx, static_ws, idt, odt, outer, red, inner, in, out);
  if (idt == HIPNX_U64 && (OP == HIPNX_RED_MAX || OP == HIPNX_RED_MIN))
    return run_reduce<PlainReducer<int64_t, OP, true>, int64_t>(ctx, static_ws, idt, odt, outer, red, inner, in, out);
  return run_reduce<PlainReducer<int64_t, OP, false>, int64_t>(ctx, static_ws, idt, odt, outer, red, inner, in, out);
}


int reduce_select(hipnx_ctx *ctx, bool static_ws, int op, int idt, int odt, int64_t outer, int64_t red, int64_t inner,
                  const void *in, void *out) {
  switch (op) {
    case HIPNX_RED_MAX: return reduce_op<HIPNX_RED_MAX>(ctx, static_ws, idt, odt, outer, red, inner, in, out);
    case HIPNX_RED_MIN: return reduce_op<HIPNX_RED_MIN>(ctx, static_ws, idt, odt, outer, red, inner, in, out);
    case HIPNX_RED_ALL: return reduce_op<HIPNX_RED_ALL>(ctx, static_ws, idt, odt, outer, red, inner, in, out);
    default: return reduce_op<HIPNX_RED_ANY>(ctx, static_ws, idt, odt, outer, red, inner, in, out);
  }
}

}  // namespace hipnx
