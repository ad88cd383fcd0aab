// A chain of element-wise callbacks in one pass over memory.
//
// The reference's evaluator issues one callback per node (nx/lib/nx/defn/evaluator.ex:363-388), so
// `sum(exp((a + b) * 0.5))` moves every intermediate through HBM: 32 bytes per element where the
// inputs and the result are 12.  Here a group of element-wise nodes with one result runs as a
// small program on an accumulator machine, interpreted per lane over a vector of eight elements
// at a time:
//   * the accumulator holds the value computed last; an instruction combines it with one other
//     operand -- an input (loaded from memory where it is used, converted to f32, broadcast by a
//     row / column stride), a constant, or one of three saved values -- and may save its result;
//   * every instruction rounds its result to the type its node has in the graph (bf16 by
//     truncation, f16 to nearest), so the value carried on is exactly what the separate kernels
//     would have stored and re-loaded: results are bit-identical to node-by-node evaluation.
// Decoding an instruction is scalar work (wave-uniform branches on the opcode).
// An earlier form with a general register file (in VGPRs behind switches, then in LDS) spent more
// time decoding and copying than computing.
//
// Scope: operands and results in bf16 / f16 / f32 (the f32 compute class of elementwise_ops.cuh),
// u8 truth values between comparisons / logical ops and select, and integer inputs of at most
// 32 bits feeding an as_type (exact in f32 after one rounding, as the as_type kernel does it).
// Programs with 32-bit integer instructions or bitcasts (flags bit 1, HIPNX_FUSED_BITCAST) exist only
// compiled (fused_rtc.hip); the kernels here refuse them.
// Bound by HBM: bytes(inputs) + bytes(out).
#include "fused_ops.cuh"
#include "internal.h"
#include "reduce_kernels.cuh"

namespace hipnx {

// The kernel comes in two sizes.  The registers a kernel needs are those of its hungriest path, and
// the rarely used functions (pow, atan2, remainder, the trigonometric and hyperbolic families, erf,
// cbrt) need twice what exp or tanh do: a program without them runs in the light instantiation,
// at twice the waves per SIMD.
constexpr bool unary_light(int op) {
  return op == HIPNX_EXP || op == HIPNX_LOG || op == HIPNX_SIGMOID || op == HIPNX_TANH || op == HIPNX_SQRT ||
         op == HIPNX_RSQRT || op == HIPNX_ABS || op == HIPNX_NEGATE || op == HIPNX_SIGN || op == HIPNX_CEIL ||
         op == HIPNX_FLOOR || op == HIPNX_ROUND || op == HIPNX_IS_NAN || op == HIPNX_IS_INFINITY;
}
constexpr bool binary_light(int op) { return op != HIPNX_POW && op != HIPNX_ATAN2 && op != HIPNX_REMAINDER; }

template <bool FULL, int... OPS>
__device__ __forceinline__ void unary_all(std::integer_sequence<int, OPS...>, int op, Vecs &x) {
  (void)(((FULL || unary_light(OPS)) && op == OPS ? (unary_vecs<OPS>(x), true) : false) || ...);
}

template <bool FULL, int... OPS>
__device__ __forceinline__ void binary_all(std::integer_sequence<int, OPS...>, int op, Vecs &x, const Vecs &y, bool swap) {
  (void)(((FULL || binary_light(OPS)) && op == OPS ? (binary_vecs<OPS>(x, y, swap), true) : false) || ...);
}

// saved slots are numbered by wave-uniform run-time values: a switch keeps them in registers (the
// empty asm differs from case to case so that the cases are not merged into one access through a
// selected address, which would move the slots to scratch memory)
__device__ __forceinline__ void read_saved(const Saved &S, int slot, Vecs &dst) {
  switch (slot) {
    case 1: copy_vecs(dst, S.s[1]); asm volatile("; saved 1"); break;
    case 2: copy_vecs(dst, S.s[2]); asm volatile("; saved 2"); break;
    default: copy_vecs(dst, S.s[0]); asm volatile("; saved 0"); break;
  }
}

__device__ __forceinline__ void write_saved(Saved &S, int slot, const Vecs &src) {
  switch (slot) {
    case 1: copy_vecs(S.s[1], src); asm volatile("; save 1"); break;
    case 2: copy_vecs(S.s[2], src); asm volatile("; save 2"); break;
    default: copy_vecs(S.s[0], src); asm volatile("; save 0"); break;
  }
}

__device__ __forceinline__ void fetch(KernArgs a, const Saved &S, int src, int arg, float imm, const int64_t (&row)[FV],
                                      const int64_t (&col)[FV], Vecs &dst) {
  switch (src) {
    case HIPNX_FUSED_SRC_INPUT: load_input_as(a, arg, a->in_dt[arg], a->in_cs[arg], row, col, dst); break;
    case HIPNX_FUSED_SRC_SAVED: read_saved(S, arg, dst); break;
    default:
#pragma unroll
      for (int u = 0; u < FV; u++)
#pragma unroll
        for (int e = 0; e < FE; e++) dst[u][e] = imm;
      break;
  }
}

// the program for the lane's vector at (row, col); the result is left in `acc`
template <bool FULL>
__device__ __forceinline__ void run_program(KernArgs a, int n_instr, const int64_t (&row)[FV], const int64_t (&col)[FV], Vecs &acc) {
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  typedef const __attribute__((address_space(4))) u32x4 *InstrWords;
  Vecs y, z;
  Saved S;
  u32x4 next = *(InstrWords)&a->ins[0];
  for (int pc = 0; pc < n_instr; pc++) {
    // one 16-byte scalar load per instruction, requested one instruction ahead
    const u32x4 q = next;
    if (pc + 1 < n_instr) next = *(InstrWords)&a->ins[pc + 1];
    const int kind = q.x & 0xFF, op = (q.x >> 8) & 0xFF, src = (q.x >> 16) & 0xFF, arg = q.x >> 24;
    const int src2 = q.y & 0xFF, arg2 = (q.y >> 8) & 0xFF, flags = (q.y >> 16) & 0xFF, dt = q.y >> 24;
    switch (kind) {
      case HIPNX_FUSED_SET:
        fetch(a, S, src, arg, __uint_as_float(q.z), row, col, acc);
        break;
      case HIPNX_FUSED_UNARY:
        unary_all<FULL>(std::make_integer_sequence<int, HIPNX_NUNARY>{}, op, acc);
        break;
      case HIPNX_FUSED_BINARY:
        fetch(a, S, src, arg, __uint_as_float(q.z), row, col, y);
        binary_all<FULL>(std::make_integer_sequence<int, HIPNX_NBINARY>{}, op, acc, y, (flags & 1) != 0);
        break;
      case HIPNX_FUSED_SELECT:
        fetch(a, S, src, arg, __uint_as_float(q.z), row, col, y);
        fetch(a, S, src2, arg2, __uint_as_float(q.w), row, col, z);
#pragma unroll
        for (int u = 0; u < FV; u++)
#pragma unroll
          for (int e = 0; e < FE; e++) acc[u][e] = acc[u][e] != 0.0f ? y[u][e] : z[u][e];  // NaN is true
        break;
      default:  // HIPNX_FUSED_AS_TYPE: the rounding below is the conversion
        break;
    }
    if (dt == HIPNX_BF16 || dt == HIPNX_F16) {
#pragma unroll
      for (int u = 0; u < FV; u++)
#pragma unroll
        for (int e = 0; e < FE; e++) acc[u][e] = round_to(acc[u][e], dt);
    }
    if (flags >> 4) write_saved(S, (flags >> 4) - 1, acc);
  }
}

template <bool FULL>
struct RunInterpreted {
  static __device__ __forceinline__ void run(KernArgs a, const int64_t (&row)[FV], const int64_t (&col)[FV], Vecs &acc, int = FE) {
    run_program<FULL>(a, a->n_instr, row, col, acc);  // (whole vectors only: the host sees to it)
  }
  static __device__ __forceinline__ int out_dt(KernArgs a) { return a->out_dt; }
  static constexpr bool raw_out = false;
};

template <bool FULL>
__global__ void __launch_bounds__(FBLOCK) fused_elementwise_kernel(FusedArgs by_value) {
  (void)by_value;
  fused_elementwise_body<RunInterpreted<FULL>>();
}

template <typename R, typename CT, int TPR>
__global__ void __launch_bounds__(FBLOCK) fused_reduce_rows_kernel(FusedArgs by_value) {
  (void)by_value;
  fused_reduce_rows_body<RunInterpreted<false>, R, CT, TPR>();
}

template <typename R, typename CT>
static void launch_fused_reduce(const hipnx_ctx *ctx, const FusedArgs &a) {
  if (a.cols <= 4096) {
    const int rpb = FBLOCK / WAVE;
    hipLaunchKernelGGL((fused_reduce_rows_kernel<R, CT, WAVE>), dim3((unsigned)((a.rows + rpb - 1) / rpb)), dim3(FBLOCK), 0, ctx->stream, a);
  } else {
    hipLaunchKernelGGL((fused_reduce_rows_kernel<R, CT, FBLOCK>), dim3((unsigned)(a.rows * a.nseg)), dim3(FBLOCK), 0, ctx->stream, a);
  }
}

// the second kernel of a reduction whose rows were cut into segments: the separate reduction's own
static void launch_fused_combine(const hipnx_ctx *ctx, const FusedArgs &a, int reduce_op) {
  const dim3 grid((unsigned)((a.rows + BLOCK / WAVE - 1) / (BLOCK / WAVE))), block(BLOCK);
  if (reduce_op == HIPNX_RED_SUM)
    hipLaunchKernelGGL((combine_partials_kernel<PlainReducer<double, HIPNX_RED_SUM, false>>), grid, block, 0, ctx->stream,
                       (const double *)a.partial, a.out, a.out_dt, a.rows, a.nseg);
  else if (reduce_op == HIPNX_RED_MAX)
    hipLaunchKernelGGL((combine_partials_kernel<PlainReducer<float, HIPNX_RED_MAX, false>>), grid, block, 0, ctx->stream,
                       (const float *)a.partial, a.out, a.out_dt, a.rows, a.nseg);
  else
    hipLaunchKernelGGL((combine_partials_kernel<PlainReducer<float, HIPNX_RED_MIN, false>>), grid, block, 0, ctx->stream,
                       (const float *)a.partial, a.out, a.out_dt, a.rows, a.nseg);
}

static bool narrow(int dt) { return dt == HIPNX_BF16 || dt == HIPNX_F16 || dt == HIPNX_F32; }

// fused_rtc.hip
int fused_launch_compiled(hipnx_ctx *ctx, const FusedArgs &a, int reduce_op, bool block_per_row, unsigned grid, bool *done);

}  // namespace hipnx

using namespace hipnx;

extern "C" int hipnx_fused_elementwise(hipnx_ctx *ctx, int n_instr, const hipnx_fused_instr *prog, int n_inputs,
                                       const hipnx_buf *const *inputs, const int *in_dts, const int64_t *in_row_strides,
                                       const int *in_col_strides, int64_t rows, int64_t cols, int reduce_op, int out_dt,
                                       hipnx_buf *out) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (n_instr < 1 || n_instr > HIPNX_FUSED_MAX_INSTR || !prog)
    return set_error(HIPNX_EINVAL, "fused: 1 .. %d instructions", HIPNX_FUSED_MAX_INSTR);
  if (n_inputs < 0 || n_inputs > HIPNX_FUSED_MAX_INPUTS || (n_inputs > 0 && (!inputs || !in_dts || !in_row_strides || !in_col_strides)))
    return set_error(HIPNX_EINVAL, "fused: 0 .. %d inputs", HIPNX_FUSED_MAX_INPUTS);
  if (rows < 0 || cols < 0) return set_error(HIPNX_EINVAL, "fused: negative extent");
  const bool int_out = out_dt == HIPNX_U32 || out_dt == HIPNX_S32;
  if (!narrow(out_dt) && out_dt != HIPNX_U8 && !int_out) return set_error(HIPNX_EUNSUPPORTED, "fused: result type %d", out_dt);
  if (reduce_op != -1 && reduce_op != HIPNX_RED_SUM && reduce_op != HIPNX_RED_MAX && reduce_op != HIPNX_RED_MIN)
    return set_error(HIPNX_EUNSUPPORTED, "fused: reduction %d (sum, max and min along the rows are built)", reduce_op);
  FusedArgs a{};
  a.n_instr = n_instr;
  a.n_inputs = n_inputs;
  unsigned saved = 0;  // slots that hold a value so far
  unsigned raw_inputs = 0;  // inputs whose words are loaded unconverted
  bool have_acc = false, full = false, needs_compiled = false;
  int n_stats = 0;       // row statistics kept so far (HIPNX_FUSED_ROW_STAT)
  bool on_stat = false;  // between a stage's reduction and its ROW_STAT
  bool row_result = false;  // the program ends in a ROW_STAT that is the result: one value per row
  bool uses_carry = false;  // some instruction reads the previous stage's element values
  auto int32 = [](int dt) { return dt == HIPNX_U32 || dt == HIPNX_S32; };
  auto source_ok = [&](int src, int arg, const char **why) {
    if (src == HIPNX_FUSED_SRC_INPUT && arg >= n_inputs) { *why = "reads an input that is not there"; return false; }
    if (src == HIPNX_FUSED_SRC_SAVED && (arg >= HIPNX_FUSED_SAVED || !(saved >> arg & 1))) { *why = "reads an empty slot"; return false; }
    if (src == HIPNX_FUSED_SRC_ROWSTAT) {
      if (arg >= n_stats) { *why = "reads a row statistic that no stage has produced yet"; return false; }
      return true;
    }
    if (src == HIPNX_FUSED_SRC_CARRY) {
      if (n_stats < 1 || on_stat) { *why = "reads the previous stage's values where there are none"; return false; }
      uses_carry = true;
      return true;
    }
    if (src != HIPNX_FUSED_SRC_INPUT && src != HIPNX_FUSED_SRC_SAVED && src != HIPNX_FUSED_SRC_CONST) { *why = "has an unknown operand source"; return false; }
    return true;
  };
  for (int i = 0; i < n_instr; i++) {
    const hipnx_fused_instr &q = prog[i];
    const char *why = nullptr;
    const bool ints = (q.flags & HIPNX_FUSED_FLAG_INT) != 0;
    needs_compiled |= ints || q.kind == HIPNX_FUSED_BITCAST;
    if (ints && q.kind != HIPNX_FUSED_AS_TYPE && q.kind != HIPNX_FUSED_SET && !int32(q.dt))
      return set_error(HIPNX_EINVAL, "fused: integer instruction %d has result type %d", i, q.dt);
    if (!narrow(q.dt) && q.dt != HIPNX_U8 && !((ints || q.kind == HIPNX_FUSED_BITCAST) && int32(q.dt)))
      return set_error(HIPNX_EUNSUPPORTED, "fused: instruction %d has result type %d", i, q.dt);
    if (q.kind != HIPNX_FUSED_SET && !have_acc) return set_error(HIPNX_EINVAL, "fused: instruction %d uses the accumulator before anything set it", i);
    switch (q.kind) {
      case HIPNX_FUSED_SET:
        if (!source_ok(q.src, q.arg, &why)) return set_error(HIPNX_EINVAL, "fused: instruction %d %s", i, why);
        if (ints && q.src == HIPNX_FUSED_SRC_INPUT) raw_inputs |= 1u << q.arg;
        break;
      case HIPNX_FUSED_UNARY:
        if (ints) {
          if (q.op != HIPNX_NEGATE && q.op != HIPNX_BITWISE_NOT) return set_error(HIPNX_EUNSUPPORTED, "fused: integer unary op %d", q.op);
          break;
        }
        if (q.op >= HIPNX_NUNARY || q.op == HIPNX_BITWISE_NOT || q.op == HIPNX_CLZ || q.op == HIPNX_POPCOUNT)
          return set_error(HIPNX_EUNSUPPORTED, "fused: unary op %d", q.op);
        full |= !unary_light(q.op);
        break;
      case HIPNX_FUSED_BINARY:
        if (!source_ok(q.src, q.arg, &why)) return set_error(HIPNX_EINVAL, "fused: instruction %d %s", i, why);
        if (ints) {
          if (q.op != HIPNX_ADD && q.op != HIPNX_SUBTRACT && q.op != HIPNX_MULTIPLY && q.op != HIPNX_MIN && q.op != HIPNX_MAX &&
              q.op != HIPNX_BITWISE_AND && q.op != HIPNX_BITWISE_OR && q.op != HIPNX_BITWISE_XOR &&
              q.op != HIPNX_LEFT_SHIFT && q.op != HIPNX_RIGHT_SHIFT)
            return set_error(HIPNX_EUNSUPPORTED, "fused: integer binary op %d", q.op);
          if (q.src == HIPNX_FUSED_SRC_INPUT) raw_inputs |= 1u << q.arg;
          break;
        }
        if (q.op >= HIPNX_NBINARY || binary_int_only(q.op)) return set_error(HIPNX_EUNSUPPORTED, "fused: binary op %d", q.op);
        full |= !binary_light(q.op);
        break;
      case HIPNX_FUSED_BITCAST: break;
      case HIPNX_FUSED_ROW_REDUCE:
        if (q.op != HIPNX_RED_SUM && q.op != HIPNX_RED_MAX && q.op != HIPNX_RED_MIN) return set_error(HIPNX_EUNSUPPORTED, "fused: stage reduction %d", q.op);
        if (on_stat || !narrow(q.dt) || i == 0 || !narrow(prog[i - 1].dt))
          return set_error(HIPNX_EINVAL, "fused: instruction %d reduces a non-float value, or a row statistic", i);
        if (q.flags) return set_error(HIPNX_EINVAL, "fused: instruction %d: a stage reduction takes no flags", i);
        on_stat = true;  // until the ROW_STAT that keeps it, instructions work on one value per row
        needs_compiled = true;
        break;
      case HIPNX_FUSED_ROW_STAT:
        if (q.flags == HIPNX_FUSED_FLAG_RESULT) {  // the value per row is the result: nothing follows
          if (!on_stat || i != n_instr - 1 || !narrow(prog[i - 1].dt) || q.dt != out_dt)
            return set_error(HIPNX_EINVAL, "fused: instruction %d: a row result ends the program, after a stage reduction, in the result's type", i);
          row_result = true;
          break;
        }
        if (!on_stat || n_stats >= HIPNX_FUSED_STATS || q.arg != n_stats || i == n_instr - 1 || !narrow(prog[i - 1].dt))
          return set_error(HIPNX_EINVAL, "fused: instruction %d keeps row statistic %d: at most %d, in order, after a stage reduction, and a last stage follows", i, q.arg, HIPNX_FUSED_STATS);
        if (q.flags) return set_error(HIPNX_EINVAL, "fused: instruction %d: keeping a row statistic takes no flags but the result mark", i);
        break;
      case HIPNX_FUSED_SELECT:
        if (!source_ok(q.src, q.arg, &why) || !source_ok(q.src2, q.arg2, &why))
          return set_error(HIPNX_EINVAL, "fused: instruction %d %s", i, why);
        break;
      case HIPNX_FUSED_AS_TYPE:
        if (ints && (!int32(q.op) || !narrow(q.dt))) return set_error(HIPNX_EINVAL, "fused: instruction %d converts type %d to %d", i, q.op, q.dt);
        break;
      default: return set_error(HIPNX_EINVAL, "fused: instruction %d has kind %d", i, q.kind);
    }
    if (on_stat && q.kind != HIPNX_FUSED_ROW_REDUCE && q.kind != HIPNX_FUSED_ROW_STAT) {
      // work on the statistic: nothing is loaded per element here, and nothing is set aside
      const bool reads_input = (q.kind == HIPNX_FUSED_BINARY || q.kind == HIPNX_FUSED_SELECT || q.kind == HIPNX_FUSED_SET) &&
                               (q.src == HIPNX_FUSED_SRC_INPUT || q.src == HIPNX_FUSED_SRC_SAVED ||
                                (q.kind == HIPNX_FUSED_SELECT && (q.src2 == HIPNX_FUSED_SRC_INPUT || q.src2 == HIPNX_FUSED_SRC_SAVED)));
      if (reads_input || q.kind == HIPNX_FUSED_SET || (q.flags >> 4) || ints)
        return set_error(HIPNX_EINVAL, "fused: instruction %d works on a row statistic with something other than constants and earlier statistics", i);
    }
    have_acc = q.kind != HIPNX_FUSED_ROW_STAT;  // the next stage starts from nothing
    if (q.kind == HIPNX_FUSED_ROW_STAT) { saved = 0; on_stat = false; n_stats++; }  // (a row result counts as a stage too)
    if (q.flags >> 4) {
      if ((q.flags >> 4) > HIPNX_FUSED_SAVED) return set_error(HIPNX_EINVAL, "fused: instruction %d saves to slot %d", i, (q.flags >> 4) - 1);
      saved |= 1u << ((q.flags >> 4) - 1);
    }
    a.ins[i] = q;
  }
  if (int_out != int32(prog[n_instr - 1].dt)) return set_error(HIPNX_EINVAL, "fused: result type %d after a program that ends in type %d", out_dt, prog[n_instr - 1].dt);
  if (needs_compiled && ctx->fused_mode != HIPNX_FUSED_COMPILED)
    return set_error(HIPNX_EUNSUPPORTED, "fused: 32-bit integer instructions and stages need the compiled mode");
  if (on_stat) return set_error(HIPNX_EINVAL, "fused: the program ends inside a stage's work on its statistic");
  if (n_stats && (reduce_op != -1 || cols == 0))
    return set_error(HIPNX_EUNSUPPORTED, "fused: stages take non-empty rows and no reduction of the result");
  // a few very long rows are split into segments by the separate reduction, whose order the stages follow: not here
  if (n_stats) {
    int would_be = 1;
    int64_t of_length = cols;
    plan_row_segments(ctx, rows, cols, &would_be, &of_length);
    if (would_be > 1) return set_error(HIPNX_EUNSUPPORTED, "fused: stages over rows that the reduction would split");
  }
  if (uses_carry && cols > 16 * (cols > 4096 ? 256 : 64) * 8)
    return set_error(HIPNX_EUNSUPPORTED, "fused: rows too long to keep a stage's values in registers");
  const int64_t n = rows * cols;
  if (cols % 8 != 0) {
    // a flat index space (one row) may end in a partial vector -- in a compiled kernel, which handles it
    if (rows != 1 || reduce_op != -1 || n_stats || ctx->fused_mode != HIPNX_FUSED_COMPILED)
      return set_error(HIPNX_EUNSUPPORTED, "fused: the row length is not a multiple of 8");
    needs_compiled = true;
  }
  for (int k = 0; k < n_inputs; k++) {
    const int dt = in_dts[k];
    const int sz = dtype_size(dt);
    if (sz < 0 || sz > 4) return set_error(HIPNX_EUNSUPPORTED, "fused: input %d has type %d", k, dt);
    if ((raw_inputs >> k & 1) && sz != 4) return set_error(HIPNX_EINVAL, "fused: input %d of type %d is read as 32-bit words", k, dt);
    if (in_row_strides[k] < 0 || (in_col_strides[k] != 0 && in_col_strides[k] != 1))
      return set_error(HIPNX_EINVAL, "fused: input %d has strides (%lld, %d)", k, (long long)in_row_strides[k], in_col_strides[k]);
    // rows of an operand read with vector loads must start on a vector boundary
    if (in_col_strides[k] == 1 && rows > 1 && in_row_strides[k] % 8 != 0)
      return set_error(HIPNX_EUNSUPPORTED, "fused: rows of input %d are not vector-aligned", k);
    const uint64_t extent = n == 0 ? 0 : (uint64_t)((rows - 1) * in_row_strides[k] + (cols - 1) * in_col_strides[k] + 1);
    if (int st = check_buf(ctx, inputs[k], extent * sz, "fused input")) return st;
    a.in[k] = inputs[k]->ptr;
    a.in_dt[k] = dt;
    a.in_rs[k] = in_row_strides[k];
    a.in_cs[k] = in_col_strides[k];
  }
  if (reduce_op != -1) {
    // the interpreting reduction kernels exist in the light instantiation only (registers); a compiled one holds just its own program
    if (full && ctx->fused_mode != HIPNX_FUSED_COMPILED)
      return set_error(HIPNX_EUNSUPPORTED, "fused: a reduction after a program with pow, atan2, remainder, trigonometric or erf functions");
    if (!narrow(prog[n_instr - 1].dt) || !narrow(out_dt)) return set_error(HIPNX_EUNSUPPORTED, "fused: a reduction of a non-float value");
    if (cols == 0) return set_error(HIPNX_EUNSUPPORTED, "fused: a reduction over an empty axis");
  }
  if (int st = check_buf(ctx, out, (uint64_t)(reduce_op == -1 && !row_result ? n : rows) * dtype_size(out_dt), "fused out")) return st;
  if (n == 0) return HIPNX_OK;
  a.out = out->ptr;
  a.out_dt = out_dt;
  a.rows = rows;
  a.cols = cols;
  a.vecs_per_row = (cols + FE - 1) / FE;
  a.nvec = rows * a.vecs_per_row;
  a.nseg = 1;
  a.seg_len = cols;
  // a few very long rows are cut into segments as the separate reduction cuts them, so that the sums add in its order
  void *partials = nullptr;
  size_t partials_cap = 0;
  if (reduce_op != -1) {
    plan_row_segments(ctx, rows, cols, &a.nseg, &a.seg_len);
    if (a.nseg > 1) {
      if (int st = pool_alloc(ctx, (size_t)(rows * a.nseg) * sizeof(double), &partials, &partials_cap)) return st;
      a.partial = partials;
    }
  }
  // (the pool hands the memory to later work on this stream only: it may go back right after the launches)
  struct Release {
    hipnx_ctx *ctx; void *&p; size_t &cap;
    ~Release() { if (p) pool_free(ctx, p, cap); }
  } release{ctx, partials, partials_cap};
  if (ctx->fused_mode == HIPNX_FUSED_COMPILED) {
    // the same grids as the interpreting kernels below
    const bool block_per_row = (reduce_op != -1 || n_stats) && a.cols > 4096;
    int64_t grid = n_stats ? (block_per_row ? a.rows : (a.rows + FBLOCK / WAVE - 1) / (FBLOCK / WAVE))  // a wave or a block per row
                   : reduce_op == -1 ? (a.nvec + (int64_t)FBLOCK * FV - 1) / ((int64_t)FBLOCK * FV)
                   : block_per_row ? a.rows * a.nseg : (a.rows + FBLOCK / WAVE - 1) / (FBLOCK / WAVE);
    // a launch may hold at most 2^32 - 1 lanes: the element-wise kernel loops over what a capped grid leaves, the row
    // kernels take one row (or wave of rows) per work-group and leave larger inputs to the separate callbacks
    const int64_t max_grid = ((1ll << 32) - 1) / FBLOCK;
    if (grid > max_grid) {
      if (n_stats || reduce_op != -1) return set_error(HIPNX_EUNSUPPORTED, "fused: more rows than one launch holds");
      grid = max_grid;
    }
    bool done = false;
    if (int st = fused_launch_compiled(ctx, a, reduce_op, block_per_row, (unsigned)grid, &done)) return st;
    if (done) {
      if (a.nseg > 1) {
        launch_fused_combine(ctx, a, reduce_op);
        HIPNX_HIP(hipGetLastError());
      }
      return HIPNX_OK;
    }
  }
  if (needs_compiled || (full && reduce_op != -1))
    return set_error(HIPNX_EUNSUPPORTED, "fused: a program that exists only compiled, first met while capturing");
  if (reduce_op != -1 && a.rows * a.nseg > ((1ll << 32) - 1) / FBLOCK) return set_error(HIPNX_EUNSUPPORTED, "fused: more rows than one launch holds");
  if (reduce_op == HIPNX_RED_SUM) launch_fused_reduce<PlainReducer<double, HIPNX_RED_SUM, false>, double>(ctx, a);
  else if (reduce_op == HIPNX_RED_MAX) launch_fused_reduce<PlainReducer<float, HIPNX_RED_MAX, false>, float>(ctx, a);
  else if (reduce_op == HIPNX_RED_MIN) launch_fused_reduce<PlainReducer<float, HIPNX_RED_MIN, false>, float>(ctx, a);
  if (reduce_op != -1) {
    if (a.nseg > 1) launch_fused_combine(ctx, a, reduce_op);
    HIPNX_HIP(hipGetLastError());
    return HIPNX_OK;
  }
  int64_t blocks = (a.nvec + (int64_t)FBLOCK * FV - 1) / ((int64_t)FBLOCK * FV);
  if (blocks > ((1ll << 32) - 1) / FBLOCK) blocks = ((1ll << 32) - 1) / FBLOCK;
  if (full) hipLaunchKernelGGL((fused_elementwise_kernel<true>), dim3((unsigned)blocks), dim3(FBLOCK), 0, ctx->stream, a);
  else hipLaunchKernelGGL((fused_elementwise_kernel<false>), dim3((unsigned)blocks), dim3(FBLOCK), 0, ctx->stream, a);
  HIPNX_HIP(hipGetLastError());
  return HIPNX_OK;
}
