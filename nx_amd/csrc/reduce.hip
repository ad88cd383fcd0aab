// Axis reductions: the entry points of sum / product / reduce_max / reduce_min / all / any (kernels and their
// launcher: reduce_kernels.cuh).  The operations are compiled in two units (this one: sum and product; the
// selections in reduce_select.hip) so that the build runs in parallel.
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


// max / min / all / any: reduce_select.hip
int reduce_select(hipnx_ctx *ctx, bool static_ws, int op, int idt, int odt, int64_t outer, int64_t red, int64_t inner,
                  const void *in, void *out);

}  // namespace hipnx

using namespace hipnx;


static int check_view(int64_t outer, int64_t red, int64_t inner) {
  if (outer < 0 || red < 0 || inner < 0) return set_error(HIPNX_EINVAL, "reduce: negative extent");
  return HIPNX_OK;
}

static int reduce_dispatch(hipnx_ctx *ctx, int op, int in_dt, int out_dt, int64_t outer, int64_t red, int64_t inner, const void *in,
                           void *out) {
  switch (op) {
    case HIPNX_RED_SUM: return reduce_op<HIPNX_RED_SUM>(ctx, false, in_dt, out_dt, outer, red, inner, in, out);
    case HIPNX_RED_PRODUCT: return reduce_op<HIPNX_RED_PRODUCT>(ctx, false, in_dt, out_dt, outer, red, inner, in, out);
    default: return reduce_select(ctx, false, op, in_dt, out_dt, outer, red, inner, in, out);
  }
}

static int reduce_entry(hipnx_ctx *ctx, bool static_ws, int op, int in_dt, int out_dt, int64_t outer, int64_t red,
                        int64_t inner, const hipnx_buf *inb, hipnx_buf *out) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (op < 0 || op > HIPNX_RED_ANY) return set_error(HIPNX_EINVAL, "reduce: unknown op %d", op);
  if (dtype_size(in_dt) < 0 || dtype_size(out_dt) < 0) return set_error(HIPNX_EINVAL, "reduce: unknown element type");
  if (int st = check_view(outer, red, inner)) return st;
  if ((op == HIPNX_RED_MAX || op == HIPNX_RED_MIN) && red == 0 && outer * inner > 0)
    return set_error(HIPNX_EINVAL, "reduce: max/min over an empty axis");
  if (int st = check_buf(ctx, inb, (uint64_t)outer * red * inner * dtype_size(in_dt), "reduce in")) return st;
  if (int st = check_buf(ctx, out, (uint64_t)outer * inner * dtype_size(out_dt), "reduce out")) return st;
  if (outer * inner == 0) return HIPNX_OK;
  // A few columns under a long reduced axis ([N, 3] summed over N) give the column kernel a handful of lanes per
  // segment and its second pass a handful of outputs with a thousand partial results each (f32 [33M, 2]: 7.9 ms,
  // 0.03 TB/s).  With g rows folded into the columns the tensor is also [outer, red / g, g * inner]: reducing that
  // view first leaves [outer, g, inner] (sums and products in f64 / 64-bit integers, so the result is still rounded
  // once; selections in the element's own type), and a second, small reduction finishes.  A single slab (outer = 1)
  // takes any g -- the red mod g rows left over are reduced on their own into one more row for the second step --
  // several slabs need a divisor of the axis.
  const int esize = dtype_size(in_dt);
  if (!static_ws && inner > 1 && inner * esize < 1024 && red >= 4096) {
    int64_t g = 4096 / inner < red / 32 ? 4096 / inner : red / 32;
    if (outer == 1) g &= ~(int64_t)7;  // whole vectors in the folded rows
    else while (g >= 16 && red % g != 0) g--;
    if (g >= 16) {
      const int64_t q = red / g, left = red - q * g;
      const bool arith = op == HIPNX_RED_SUM || op == HIPNX_RED_PRODUCT;
      const int mid_dt = !arith ? (op == HIPNX_RED_MAX || op == HIPNX_RED_MIN ? in_dt : out_dt)
                         : is_float(in_dt) ? HIPNX_F64 : is_unsigned(in_dt) ? HIPNX_U64 : HIPNX_S64;
      const int msize = dtype_size(mid_dt);
      void *mid = nullptr;
      size_t cap = 0;
      if (int st = pool_alloc(ctx, (size_t)(outer * (g + 1) * inner) * msize, &mid, &cap)) return st;
      int st = reduce_dispatch(ctx, op, in_dt, mid_dt, outer, q, g * inner, inb->ptr, mid);
      if (st == HIPNX_OK && left)
        st = reduce_dispatch(ctx, op, in_dt, mid_dt, 1, left, inner, (const char *)inb->ptr + (size_t)(q * g * inner) * esize,
                             (char *)mid + (size_t)(g * inner) * msize);
      if (st == HIPNX_OK) st = reduce_dispatch(ctx, op, mid_dt, out_dt, outer, g + (left ? 1 : 0), inner, mid, out->ptr);
      pool_free(ctx, mid, cap);  // later work on the stream is ordered behind the launches
      return st;
    }
  }
  if (static_ws) {
    switch (op) {
      case HIPNX_RED_SUM: return reduce_op<HIPNX_RED_SUM>(ctx, true, in_dt, out_dt, outer, red, inner, inb->ptr, out->ptr);
      case HIPNX_RED_PRODUCT: return reduce_op<HIPNX_RED_PRODUCT>(ctx, true, in_dt, out_dt, outer, red, inner, inb->ptr, out->ptr);
      default: return reduce_select(ctx, true, op, in_dt, out_dt, outer, red, inner, inb->ptr, out->ptr);
    }
  }
  return reduce_dispatch(ctx, op, in_dt, out_dt, outer, red, inner, inb->ptr, out->ptr);
}

extern "C" int hipnx_reduce(hipnx_ctx *ctx, int op, int in_dt, int out_dt, int64_t outer, int64_t red,
                            int64_t inner, const hipnx_buf *inb, hipnx_buf *out) {
  return reduce_entry(ctx, false, op, in_dt, out_dt, outer, red, inner, inb, out);
}

// ---- the reduction that allocates nothing ------------------------------------------------------
// The partial results of a split reduction (few rows x a long axis, or few columns under a long
// axis) go to this array instead of a pool block.  In host code its name is only a stand-in for the
// symbol: the device address is looked up once per context (hipnx_ctx_create calls
// reduce_static_init with the device current; every device holds its own copy at its own address)
// and only that address is ever handed to a kernel.  Nothing in it has to start at zero -- every
// partial a combine kernel reads was written by the launch before it -- so a call leaves the last
// call's partials behind and clears nothing.
static __device__ __align__(256) unsigned char scratch[HIPNX_REDUCE_STATIC_SCRATCH_BYTES];

int hipnx::reduce_static_init(hipnx_ctx *ctx) {
  void *ptr = nullptr;
  HIPNX_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
  ctx->reduce_scratch = ptr;
  return HIPNX_OK;
}

extern "C" int hipnx_reduce_static(hipnx_ctx *ctx, int op, int in_dt, int out_dt, int64_t outer, int64_t red,
                                   int64_t inner, const hipnx_buf *inb, hipnx_buf *out) {
  return reduce_entry(ctx, true, op, in_dt, out_dt, outer, red, inner, inb, out);
}

