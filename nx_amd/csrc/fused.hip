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
// Bound by HBM: bytes(inputs) + bytes(out).
#include "elementwise_ops.cuh"
#include "internal.h"
#include "reduce_ops.cuh"

namespace hipnx {

constexpr int FBLOCK = 256;
constexpr int FE = 8;  // elements per vector: two 16-byte accesses of f32, one of a 2-byte type
constexpr int FV = 1;  // vectors per lane and trip (more were measured: the registers they take cost more in
                       // waves per SIMD than the shared decoding saves: 276 / 303 / 402 us for 1 / 2 / 4)

static_assert(sizeof(hipnx_fused_instr) == 16, "an instruction is one 16-byte scalar load");

struct FusedArgs {
  int n_instr, n_inputs;
  int64_t pad_to_16;
  hipnx_fused_instr ins[HIPNX_FUSED_MAX_INSTR];
  const void *in[HIPNX_FUSED_MAX_INPUTS];
  int in_dt[HIPNX_FUSED_MAX_INPUTS];
  int64_t in_rs[HIPNX_FUSED_MAX_INPUTS];  // element stride between rows (0 = the same row for all)
  int in_cs[HIPNX_FUSED_MAX_INPUTS];      // element stride along a row: 1, or 0 = one value per row
  void *out;
  int out_dt, unused;
  int64_t rows, cols, vecs_per_row, nvec;
};

// The argument block is read where the launch put it (the kernel-argument segment, constant address
// space) with wave-uniform indices: indexing the by-value copy would move it to per-lane scratch.
typedef const __attribute__((address_space(4))) FusedArgs *KernArgs;
typedef float Vecs[FV][FE];

// what a store to `dt` followed by a load would give back
__device__ __forceinline__ float round_to(float x, int dt) {
  switch (dt) {
    case HIPNX_BF16: return bf16_bits_to_f32(f32_to_bf16_bits_trunc(x));
    case HIPNX_F16: return (float)bits_f16(f32_to_f16_bits(x));
    default: return x;  // f32, and u8 truth values (0 / 1)
  }
}

// one uniform dispatch per instruction, the loops over the vectors inside each case
template <int OP>
__device__ __forceinline__ void unary_vecs(Vecs &x) {
#pragma unroll
  for (int u = 0; u < FV; u++)
#pragma unroll
    for (int e = 0; e < FE; e++) x[u][e] = unary_apply<OP, float>(x[u][e], 32);
}

template <int OP>
__device__ __forceinline__ void binary_vecs(Vecs &x, const Vecs &y, bool swap) {
#pragma unroll
  for (int u = 0; u < FV; u++)
#pragma unroll
    for (int e = 0; e < FE; e++)
      x[u][e] = swap ? binary_apply<OP, float, false>(y[u][e], x[u][e]) : binary_apply<OP, float, false>(x[u][e], y[u][e]);
}

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

__device__ __forceinline__ float element_to_f32(uint32_t bits, int dt) {
  switch (dt) {
    case HIPNX_U8: case HIPNX_U16: case HIPNX_U32: return (float)bits;
    case HIPNX_S8: return (float)(int32_t)(int8_t)bits;
    case HIPNX_S16: return (float)(int32_t)(int16_t)bits;
    case HIPNX_S32: return (float)(int32_t)bits;
    case HIPNX_F16: return (float)bits_f16((uint16_t)bits);
    case HIPNX_BF16: return bf16_bits_to_f32((uint16_t)bits);
    default: return __uint_as_float(bits);
  }
}

// input k for the lane's FV vectors: all loads are requested, then converted
__device__ __forceinline__ void load_input(KernArgs a, int k, const int64_t (&row)[FV], const int64_t (&col)[FV], Vecs &dst) {
  const int dt = a->in_dt[k], cs = a->in_cs[k];
  const int esz = (dt == HIPNX_U8 || dt == HIPNX_S8) ? 1 : (dt == HIPNX_U32 || dt == HIPNX_S32 || dt == HIPNX_F32) ? 4 : 2;
  const char *base = (const char *)a->in[k];
  const int64_t rs = a->in_rs[k];
  uint32_t w[FV][FE];  // raw words: 8 for 4-byte elements, 4 for 2-byte ones, 2 for bytes, 1 for a broadcast value
#pragma unroll
  for (int u = 0; u < FV; u++) {
    const char *p = base + (row[u] * rs + col[u] * cs) * esz;
    if (cs == 0) {
      w[u][0] = esz == 4 ? *reinterpret_cast<const uint32_t *>(p)
                : esz == 2 ? (uint32_t)*reinterpret_cast<const uint16_t *>(p)
                           : (uint32_t)*reinterpret_cast<const uint8_t *>(p);
    } else if (esz == 4) {
      const uint4 lo = *reinterpret_cast<const uint4 *>(p), hi = *reinterpret_cast<const uint4 *>(p + 16);
      w[u][0] = lo.x; w[u][1] = lo.y; w[u][2] = lo.z; w[u][3] = lo.w;
      w[u][4] = hi.x; w[u][5] = hi.y; w[u][6] = hi.z; w[u][7] = hi.w;
    } else if (esz == 2) {
      const uint4 lo = *reinterpret_cast<const uint4 *>(p);
      w[u][0] = lo.x; w[u][1] = lo.y; w[u][2] = lo.z; w[u][3] = lo.w;
    } else {
      const uint2 lo = *reinterpret_cast<const uint2 *>(p);
      w[u][0] = lo.x; w[u][1] = lo.y;
    }
  }
#pragma unroll
  for (int u = 0; u < FV; u++) {
    if (cs == 0) {
      const float v = element_to_f32(w[u][0], dt);
#pragma unroll
      for (int e = 0; e < FE; e++) dst[u][e] = v;
    } else if (esz == 4) {
      if (dt == HIPNX_F32) {
#pragma unroll
        for (int e = 0; e < FE; e++) dst[u][e] = __uint_as_float(w[u][e]);
      } else {
#pragma unroll
        for (int e = 0; e < FE; e++) dst[u][e] = element_to_f32(w[u][e], dt);
      }
    } else if (esz == 2) {
#pragma unroll
      for (int e = 0; e < FE; e++) dst[u][e] = element_to_f32((w[u][e / 2] >> (16 * (e & 1))) & 0xFFFFu, dt);
    } else {
#pragma unroll
      for (int e = 0; e < FE; e++) dst[u][e] = element_to_f32((w[u][e / 4] >> (8 * (e & 3))) & 0xFFu, dt);
    }
  }
}

__device__ __forceinline__ void copy_vecs(Vecs &dst, const Vecs &src) {
#pragma unroll
  for (int u = 0; u < FV; u++)
#pragma unroll
    for (int e = 0; e < FE; e++) dst[u][e] = src[u][e];
}

struct Saved {
  Vecs s[HIPNX_FUSED_SAVED];
};

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
    case HIPNX_FUSED_SRC_INPUT: load_input(a, arg, row, col, dst); break;
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
__global__ void __launch_bounds__(FBLOCK) fused_elementwise_kernel(FusedArgs by_value) {
  (void)by_value;
  KernArgs a = (KernArgs)__builtin_amdgcn_kernarg_segment_ptr();
  const int64_t nvec = a->nvec, vecs_per_row = a->vecs_per_row, cols = a->cols;
  const int n_instr = a->n_instr;
  const int64_t stride = (int64_t)gridDim.x * FBLOCK;
  for (int64_t v0 = (int64_t)blockIdx.x * FBLOCK + threadIdx.x; v0 < nvec; v0 += stride * FV) {
    int64_t row[FV], col[FV];
    bool live[FV];
#pragma unroll
    for (int u = 0; u < FV; u++) {
      int64_t v = v0 + u * stride;
      live[u] = v < nvec;
      if (!live[u]) v = v0;  // a vector past the end repeats the lane's first one and is not stored
      row[u] = 0;
      col[u] = v * FE;
      if (vecs_per_row != nvec) {  // more than one row
        row[u] = nvec <= 0xFFFFFFFFll ? (int64_t)((uint32_t)v / (uint32_t)vecs_per_row) : v / vecs_per_row;
        col[u] = (v - row[u] * vecs_per_row) * FE;
      }
    }
    Vecs acc;
    run_program<FULL>(a, n_instr, row, col, acc);
    void *out = (void *)a->out;
    const int odt = a->out_dt;
#pragma unroll
    for (int u = 0; u < FV; u++)
      if (live[u]) store_vec<float, FE>(out, odt, row[u] * cols + col[u], acc[u]);
  }
}

// The group's result reduced along its rows without ever being stored: TPR lanes per row walk it
// in the order of reduce_rows_kernel (lane l takes the vectors l, l + TPR, ... and folds their
// elements in turn, then lanes combine by wave shuffles and the block's waves through LDS) with the
// same reducer policy, so the value equals what the element-wise group followed by the separate
// reduction kernel gives, bit for bit.
template <typename R, typename CT, int TPR>
__global__ void __launch_bounds__(FBLOCK) fused_reduce_rows_kernel(FusedArgs by_value) {
  (void)by_value;
  static_assert(FV == 1, "one vector per lane and step");
  KernArgs a = (KernArgs)__builtin_amdgcn_kernarg_segment_ptr();
  constexpr int RPB = FBLOCK / TPR;
  const int sub = threadIdx.x / TPR, lane = threadIdx.x % TPR;
  const int64_t rows = a->rows, red = a->cols;
  const int n_instr = a->n_instr;
  const int64_t r = (int64_t)blockIdx.x * RPB + sub;
  typename R::acc_t acc = R::init();
  if (r < rows) {
    const int64_t step = (int64_t)TPR * FE;
    for (int64_t k = (int64_t)lane * FE; k < red; k += step) {
      const int64_t row[FV] = {r}, col[FV] = {k};
      Vecs x;
      run_program<false>(a, n_instr, row, col, x);
#pragma unroll
      for (int e = 0; e < FE; e++) acc = R::accumulate(acc, (CT)x[0][e], k + e);
    }
  }
  acc = wave_reduce<R>(acc);
  if constexpr (TPR > WAVE) {
    __shared__ typename R::acc_t sm[FBLOCK / WAVE];
    if (threadIdx.x % WAVE == 0) sm[threadIdx.x / WAVE] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
      for (int w = 1; w < FBLOCK / WAVE; w++) acc = R::combine(acc, sm[w]);
    }
  }
  if (lane == 0 && r < rows) finalize((void *)a->out, a->out_dt, r, acc);
}

template <typename R, typename CT>
static void launch_fused_reduce(const hipnx_ctx *ctx, const FusedArgs &a) {
  if (a.cols <= 4096) {
    const int rpb = FBLOCK / WAVE;
    hipLaunchKernelGGL((fused_reduce_rows_kernel<R, CT, WAVE>), dim3((unsigned)((a.rows + rpb - 1) / rpb)), dim3(FBLOCK), 0, ctx->stream, a);
  } else {
    hipLaunchKernelGGL((fused_reduce_rows_kernel<R, CT, FBLOCK>), dim3((unsigned)a.rows), dim3(FBLOCK), 0, ctx->stream, a);
  }
}

static bool narrow(int dt) { return dt == HIPNX_BF16 || dt == HIPNX_F16 || dt == HIPNX_F32; }

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
  if (!narrow(out_dt) && out_dt != HIPNX_U8) return set_error(HIPNX_EUNSUPPORTED, "fused: result type %d", out_dt);
  if (reduce_op != -1 && reduce_op != HIPNX_RED_SUM && reduce_op != HIPNX_RED_MAX && reduce_op != HIPNX_RED_MIN)
    return set_error(HIPNX_EUNSUPPORTED, "fused: reduction %d (sum, max and min along the rows are built)", reduce_op);
  FusedArgs a{};
  a.n_instr = n_instr;
  a.n_inputs = n_inputs;
  unsigned saved = 0;  // slots that hold a value so far
  bool have_acc = false, full = false;
  auto source_ok = [&](int src, int arg, const char **why) {
    if (src == HIPNX_FUSED_SRC_INPUT && arg >= n_inputs) { *why = "reads an input that is not there"; return false; }
    if (src == HIPNX_FUSED_SRC_SAVED && (arg >= HIPNX_FUSED_SAVED || !(saved >> arg & 1))) { *why = "reads an empty slot"; return false; }
    if (src != HIPNX_FUSED_SRC_INPUT && src != HIPNX_FUSED_SRC_SAVED && src != HIPNX_FUSED_SRC_CONST) { *why = "has an unknown operand source"; return false; }
    return true;
  };
  for (int i = 0; i < n_instr; i++) {
    const hipnx_fused_instr &q = prog[i];
    const char *why = nullptr;
    if (!narrow(q.dt) && q.dt != HIPNX_U8) return set_error(HIPNX_EUNSUPPORTED, "fused: instruction %d has result type %d", i, q.dt);
    if (q.kind != HIPNX_FUSED_SET && !have_acc) return set_error(HIPNX_EINVAL, "fused: instruction %d uses the accumulator before anything set it", i);
    switch (q.kind) {
      case HIPNX_FUSED_SET:
        if (!source_ok(q.src, q.arg, &why)) return set_error(HIPNX_EINVAL, "fused: instruction %d %s", i, why);
        break;
      case HIPNX_FUSED_UNARY:
        if (q.op >= HIPNX_NUNARY || q.op == HIPNX_BITWISE_NOT || q.op == HIPNX_CLZ || q.op == HIPNX_POPCOUNT)
          return set_error(HIPNX_EUNSUPPORTED, "fused: unary op %d", q.op);
        full |= !unary_light(q.op);
        break;
      case HIPNX_FUSED_BINARY:
        if (q.op >= HIPNX_NBINARY || binary_int_only(q.op)) return set_error(HIPNX_EUNSUPPORTED, "fused: binary op %d", q.op);
        if (!source_ok(q.src, q.arg, &why)) return set_error(HIPNX_EINVAL, "fused: instruction %d %s", i, why);
        full |= !binary_light(q.op);
        break;
      case HIPNX_FUSED_SELECT:
        if (!source_ok(q.src, q.arg, &why) || !source_ok(q.src2, q.arg2, &why))
          return set_error(HIPNX_EINVAL, "fused: instruction %d %s", i, why);
        break;
      case HIPNX_FUSED_AS_TYPE: break;
      default: return set_error(HIPNX_EINVAL, "fused: instruction %d has kind %d", i, q.kind);
    }
    have_acc = true;
    if (q.flags >> 4) {
      if ((q.flags >> 4) > HIPNX_FUSED_SAVED) return set_error(HIPNX_EINVAL, "fused: instruction %d saves to slot %d", i, (q.flags >> 4) - 1);
      saved |= 1u << ((q.flags >> 4) - 1);
    }
    a.ins[i] = q;
  }
  const int64_t n = rows * cols;
  if (cols % 8 != 0) return set_error(HIPNX_EUNSUPPORTED, "fused: the row length is not a multiple of 8");
  for (int k = 0; k < n_inputs; k++) {
    const int dt = in_dts[k];
    const int sz = dtype_size(dt);
    if (sz < 0 || sz > 4) return set_error(HIPNX_EUNSUPPORTED, "fused: input %d has type %d", k, dt);
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
    if (full) return set_error(HIPNX_EUNSUPPORTED, "fused: a reduction after a program with pow, atan2, remainder, trigonometric or erf functions");
    if (!narrow(prog[n_instr - 1].dt) || !narrow(out_dt)) return set_error(HIPNX_EUNSUPPORTED, "fused: a reduction of a non-float value");
    if (cols == 0) return set_error(HIPNX_EUNSUPPORTED, "fused: a reduction over an empty axis");
    // a few very long rows are split into segments by the separate reduction: not here
    if (rows < (int64_t)ctx->num_cus * 8 && cols >= 2 * 16384) return set_error(HIPNX_EUNSUPPORTED, "fused: rows that the reduction would split");
  }
  if (int st = check_buf(ctx, out, (uint64_t)(reduce_op == -1 ? n : rows) * dtype_size(out_dt), "fused out")) return st;
  if (n == 0) return HIPNX_OK;
  a.out = out->ptr;
  a.out_dt = out_dt;
  a.rows = rows;
  a.cols = cols;
  a.vecs_per_row = cols / FE;
  a.nvec = rows * a.vecs_per_row;
  if (reduce_op == HIPNX_RED_SUM) launch_fused_reduce<PlainReducer<double, HIPNX_RED_SUM, false>, double>(ctx, a);
  else if (reduce_op == HIPNX_RED_MAX) launch_fused_reduce<PlainReducer<float, HIPNX_RED_MAX, false>, float>(ctx, a);
  else if (reduce_op == HIPNX_RED_MIN) launch_fused_reduce<PlainReducer<float, HIPNX_RED_MIN, false>, float>(ctx, a);
  if (reduce_op != -1) {
    HIPNX_HIP(hipGetLastError());
    return HIPNX_OK;
  }
  int64_t blocks = (a.nvec + (int64_t)FBLOCK * FV - 1) / ((int64_t)FBLOCK * FV);
  if (blocks > (1ll << 30)) blocks = 1ll << 30;
  if (full) hipLaunchKernelGGL((fused_elementwise_kernel<true>), dim3((unsigned)blocks), dim3(FBLOCK), 0, ctx->stream, a);
  else hipLaunchKernelGGL((fused_elementwise_kernel<false>), dim3((unsigned)blocks), dim3(FBLOCK), 0, ctx->stream, a);
  HIPNX_HIP(hipGetLastError());
  return HIPNX_OK;
}
