// A chain of element-wise callbacks in one pass over memory.
//
// The reference's evaluator issues one callback per node (nx/lib/nx/defn/evaluator.ex:363-388), so
// `sum(exp((a + b) * 0.5))` moves every intermediate through HBM: 32 bytes per element where the
// inputs and the result are 12.  Here a group of element-wise nodes with one result runs as a
// small register program, interpreted per vector of 4 elements: the operands start out in the
// first registers (converted to f32, broadcast by a row / column stride), CONST splats a number, the
// rest are the callbacks themselves.  Every instruction rounds its result to the type its node has in the
// graph (bf16 by truncation, f16 to nearest), so the value in the register is exactly what the
// unfused kernels would have stored and re-loaded: results are bit-identical to the node-by-node
// evaluation on this device.
//
// Scope: operands and results in bf16 / f16 / f32 (the f32 compute class of elementwise_ops.cuh),
// u8 truth values between comparisons / logical ops and select, and integer operands of at most
// 32 bits feeding an as_type (exact in f32 after one rounding, as the as_type kernel does it).
// The interpreter's opcode switches are wave-uniform scalar branches; the program is a kernel
// argument.  Bound by HBM: bytes(inputs) + bytes(out).
#include "elementwise_ops.cuh"
#include "internal.h"

namespace hipnx {

constexpr int FBLOCK = 256;
constexpr int FE = 4;  // elements per lane per step: one 16-byte LDS access per register

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
  int out_dt, out_reg;
  int64_t rows, cols, vecs_per_row, nvec;
};

// The register file of a lane lives in LDS: register r of lane t is the float4 at [r][t].  The
// register numbers of an instruction are wave-uniform run-time values: in LDS that is an address,
// one 16-byte access per operand; in VGPRs it is a switch per operand and, worse, a file of 64
// live registers carried around an interpreter loop full of branches (measured: 1077 vector
// instructions per wave for add, multiply, exp -- more than the three separate kernels together).
// Lanes only ever touch their own slots: no barriers.
typedef float v4f32 __attribute__((ext_vector_type(4)));

// what a store to `dt` followed by a load would give back
__device__ __forceinline__ float round_to(float x, int dt) {
  switch (dt) {
    case HIPNX_BF16: return bf16_bits_to_f32(f32_to_bf16_bits_trunc(x));
    case HIPNX_F16: return (float)bits_f16(f32_to_f16_bits(x));
    default: return x;  // f32, and u8 truth values (0 / 1)
  }
}

// one uniform dispatch per instruction, the loop over the vector inside each case
template <int OP>
__device__ __forceinline__ void unary_vec(float (&x)[FE]) {
#pragma unroll
  for (int e = 0; e < FE; e++) x[e] = unary_apply<OP, float>(x[e], 32);
}

template <int OP>
__device__ __forceinline__ void binary_vec(float (&x)[FE], const float (&y)[FE]) {
#pragma unroll
  for (int e = 0; e < FE; e++) x[e] = binary_apply<OP, float, false>(x[e], y[e]);
}

template <int... OPS>
__device__ __forceinline__ void unary_all(std::integer_sequence<int, OPS...>, int op, float (&x)[FE]) {
  (void)((op == OPS ? (unary_vec<OPS>(x), true) : false) || ...);
}

template <int... OPS>
__device__ __forceinline__ void binary_all(std::integer_sequence<int, OPS...>, int op, float (&x)[FE], const float (&y)[FE]) {
  (void)((op == OPS ? (binary_vec<OPS>(x, y), true) : false) || ...);
}

// The argument block is read where the launch put it (the kernel-argument segment, constant address
// space) with wave-uniform indices: indexing the by-value copy would move it to per-lane scratch.
typedef const __attribute__((address_space(4))) FusedArgs *KernArgs;

__device__ __forceinline__ int elem_size(int dt) {
  return (dt == HIPNX_U8 || dt == HIPNX_S8) ? 1 : (dt == HIPNX_U32 || dt == HIPNX_S32 || dt == HIPNX_F32) ? 4 : 2;
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

// raw bytes of input K for this lane's vector (16 / 8 / 4 bytes by element size, or one element
// when the input has one value per row), issued without waiting
template <int K>
__device__ __forceinline__ uint4 issue_load(KernArgs a, int64_t row, int64_t col) {
  const int dt = a->in_dt[K], cs = a->in_cs[K], esz = elem_size(dt);
  const char *p = (const char *)a->in[K] + (row * a->in_rs[K] + col * cs) * esz;
  uint4 w = {0, 0, 0, 0};
  if (cs == 0 || esz == 1) {
    w.x = (cs != 0 || esz == 4) ? *reinterpret_cast<const uint32_t *>(p)
          : esz == 2           ? (uint32_t)*reinterpret_cast<const uint16_t *>(p)
                               : (uint32_t)*reinterpret_cast<const uint8_t *>(p);
  } else if (esz == 4) {
    w = *reinterpret_cast<const uint4 *>(p);
  } else {
    const uint2 h = *reinterpret_cast<const uint2 *>(p);
    w.x = h.x; w.y = h.y;
  }
  return w;
}

template <int K>
__device__ __forceinline__ v4f32 convert_load(KernArgs a, uint4 w) {
  const int dt = a->in_dt[K], cs = a->in_cs[K], esz = elem_size(dt);
  v4f32 r;
  if (cs == 0) {
    const float v = element_to_f32(w.x, dt);
    r = {v, v, v, v};
  } else if (esz == 4) {
    r = {element_to_f32(w.x, dt), element_to_f32(w.y, dt), element_to_f32(w.z, dt), element_to_f32(w.w, dt)};
  } else if (esz == 2) {
    r = {element_to_f32(w.x & 0xFFFFu, dt), element_to_f32(w.x >> 16, dt), element_to_f32(w.y & 0xFFFFu, dt), element_to_f32(w.y >> 16, dt)};
  } else {
    r = {element_to_f32(w.x & 0xFFu, dt), element_to_f32((w.x >> 8) & 0xFFu, dt), element_to_f32((w.x >> 16) & 0xFFu, dt), element_to_f32(w.x >> 24, dt)};
  }
  return r;
}

// Inputs occupy registers 0 .. n_inputs-1 from the start.  A lane works on U vectors per trip and
// issues the loads of all of them (every input of every vector) before the first conversion.
// NIN is the most inputs this instantiation preloads.
template <int NIN, int U>
__global__ void __launch_bounds__(FBLOCK) fused_elementwise_kernel(FusedArgs by_value) {
  (void)by_value;
  __shared__ v4f32 file[HIPNX_FUSED_REGS][FBLOCK];
  KernArgs a = (KernArgs)__builtin_amdgcn_kernarg_segment_ptr();
  const int64_t nvec = a->nvec, vecs_per_row = a->vecs_per_row, cols = a->cols;
  const int n_instr = a->n_instr, n_in = a->n_inputs, t = threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * FBLOCK;
  for (int64_t v0 = (int64_t)blockIdx.x * FBLOCK + t; v0 < nvec; v0 += stride * U) {
    int64_t row[U], col[U];
    uint4 raw[U][NIN];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int64_t v = v0 + u * stride;
      row[u] = 0;
      col[u] = v * FE;
      if (vecs_per_row != nvec) {  // more than one row
        row[u] = nvec <= 0xFFFFFFFFll ? (int64_t)((uint32_t)v / (uint32_t)vecs_per_row) : v / vecs_per_row;
        col[u] = (v - row[u] * vecs_per_row) * FE;
      }
      if (v < nvec) {
#define HIPNX_IN(K) if constexpr (K < NIN) { if (K < n_in) raw[u][K] = issue_load<K>(a, row[u], col[u]); }
        HIPNX_IN(0) HIPNX_IN(1) HIPNX_IN(2) HIPNX_IN(3) HIPNX_IN(4) HIPNX_IN(5) HIPNX_IN(6)
#undef HIPNX_IN
      }
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      if (v0 + u * stride >= nvec) break;
#define HIPNX_IN(K) if constexpr (K < NIN) { if (K < n_in) file[K][t] = convert_load<K>(a, raw[u][K]); }
      HIPNX_IN(0) HIPNX_IN(1) HIPNX_IN(2) HIPNX_IN(3) HIPNX_IN(4) HIPNX_IN(5) HIPNX_IN(6)
#undef HIPNX_IN
      float x[FE], y[FE], z[FE];
      auto get = [&](int r, float (&dst)[FE]) {
        const v4f32 q = file[r][t];
        dst[0] = q.x; dst[1] = q.y; dst[2] = q.z; dst[3] = q.w;
      };
      typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
      typedef const __attribute__((address_space(4))) u32x4 *InstrWords;
      u32x4 next = *(InstrWords)&a->ins[0];
      for (int pc = 0; pc < n_instr; pc++) {
        // one 16-byte scalar load per instruction, requested one instruction ahead
        const u32x4 q = next;
        if (pc + 1 < n_instr) next = *(InstrWords)&a->ins[pc + 1];
        const int kind = q.x & 0xFF, op = (q.x >> 8) & 0xFF, dst = (q.x >> 16) & 0xFF, ra = q.x >> 24;
        const int rb = q.y & 0xFF, rc = (q.y >> 8) & 0xFF, dt = (q.y >> 16) & 0xFF;
        switch (kind) {
          case HIPNX_FUSED_CONST: {
            const float imm = __uint_as_float(q.z);
#pragma unroll
            for (int e = 0; e < FE; e++) x[e] = imm;
            break;
          }
          case HIPNX_FUSED_UNARY:
            get(ra, x);
            unary_all(std::make_integer_sequence<int, HIPNX_NUNARY>{}, op, x);
            break;
          case HIPNX_FUSED_BINARY:
            get(ra, x);
            get(rb, y);
            binary_all(std::make_integer_sequence<int, HIPNX_NBINARY>{}, op, x, y);
            break;
          case HIPNX_FUSED_SELECT:
            get(ra, x);
            get(rb, y);
            get(rc, z);
#pragma unroll
            for (int e = 0; e < FE; e++) x[e] = x[e] != 0.0f ? y[e] : z[e];  // NaN is true
            break;
          default:  // HIPNX_FUSED_AS_TYPE: the rounding below is the conversion
            get(ra, x);
            break;
        }
        if (dt == HIPNX_BF16 || dt == HIPNX_F16) {
#pragma unroll
          for (int e = 0; e < FE; e++) x[e] = round_to(x[e], dt);
        }
        file[dst][t] = v4f32{x[0], x[1], x[2], x[3]};
      }
      get(a->out_reg, x);
      store_vec<float, FE>((void *)a->out, a->out_dt, row[u] * cols + col[u], x);
    }
  }
}

static bool narrow(int dt) { return dt == HIPNX_BF16 || dt == HIPNX_F16 || dt == HIPNX_F32; }

}  // namespace hipnx

using namespace hipnx;

extern "C" int hipnx_fused_elementwise(hipnx_ctx *ctx, int n_instr, const hipnx_fused_instr *prog, int n_inputs,
                                       const hipnx_buf *const *inputs, const int *in_dts, const int64_t *in_row_strides,
                                       const int *in_col_strides, int64_t rows, int64_t cols, int out_reg, int out_dt,
                                       hipnx_buf *out) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (n_instr < 1 || n_instr > HIPNX_FUSED_MAX_INSTR || !prog)
    return set_error(HIPNX_EINVAL, "fused: 1 .. %d instructions", HIPNX_FUSED_MAX_INSTR);
  if (n_inputs < 0 || n_inputs > HIPNX_FUSED_MAX_INPUTS || (n_inputs > 0 && (!inputs || !in_dts || !in_row_strides || !in_col_strides)))
    return set_error(HIPNX_EINVAL, "fused: 0 .. %d inputs (each holds a register, one is left for results)", HIPNX_FUSED_MAX_INPUTS);
  if (rows < 0 || cols < 0) return set_error(HIPNX_EINVAL, "fused: negative extent");
  if (out_reg < 0 || out_reg >= HIPNX_FUSED_REGS) return set_error(HIPNX_EINVAL, "fused: bad result register");
  if (!narrow(out_dt) && out_dt != HIPNX_U8) return set_error(HIPNX_EUNSUPPORTED, "fused: result type %d", out_dt);
  FusedArgs a{};
  a.n_instr = n_instr;
  a.n_inputs = n_inputs;
  unsigned written = (1u << n_inputs) - 1;  // input k starts out in register k
  for (int i = 0; i < n_instr; i++) {
    const hipnx_fused_instr &q = prog[i];
    auto reads = [&](int r) { return r >= 0 && r < HIPNX_FUSED_REGS && (written >> r & 1); };
    if (q.dst >= HIPNX_FUSED_REGS) return set_error(HIPNX_EINVAL, "fused: instruction %d writes register %d", i, q.dst);
    if (!narrow(q.dt) && q.dt != HIPNX_U8) return set_error(HIPNX_EUNSUPPORTED, "fused: instruction %d has result type %d", i, q.dt);
    switch (q.kind) {
      case HIPNX_FUSED_CONST: break;
      case HIPNX_FUSED_UNARY:
        if (q.op >= HIPNX_NUNARY || q.op == HIPNX_BITWISE_NOT || q.op == HIPNX_CLZ || q.op == HIPNX_POPCOUNT)
          return set_error(HIPNX_EUNSUPPORTED, "fused: unary op %d", q.op);
        if (!reads(q.a)) return set_error(HIPNX_EINVAL, "fused: instruction %d reads an unwritten register", i);
        break;
      case HIPNX_FUSED_BINARY:
        if (q.op >= HIPNX_NBINARY || binary_int_only(q.op)) return set_error(HIPNX_EUNSUPPORTED, "fused: binary op %d", q.op);
        if (!reads(q.a) || !reads(q.b)) return set_error(HIPNX_EINVAL, "fused: instruction %d reads an unwritten register", i);
        break;
      case HIPNX_FUSED_SELECT:
        if (!reads(q.a) || !reads(q.b) || !reads(q.c)) return set_error(HIPNX_EINVAL, "fused: instruction %d reads an unwritten register", i);
        break;
      case HIPNX_FUSED_AS_TYPE:
        if (!reads(q.a)) return set_error(HIPNX_EINVAL, "fused: instruction %d reads an unwritten register", i);
        break;
      default: return set_error(HIPNX_EINVAL, "fused: instruction %d has kind %d", i, q.kind);
    }
    written |= 1u << q.dst;
    a.ins[i] = q;
  }
  if (!(written >> out_reg & 1)) return set_error(HIPNX_EINVAL, "fused: the result register is never written");
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
  if (int st = check_buf(ctx, out, (uint64_t)n * dtype_size(out_dt), "fused out")) return st;
  if (n == 0) return HIPNX_OK;
  a.out = out->ptr;
  a.out_dt = out_dt;
  a.out_reg = out_reg;
  a.rows = rows;
  a.cols = cols;
  a.vecs_per_row = (cols + FE - 1) / FE;
  a.nvec = rows * a.vecs_per_row;
  // vectors per lane and trip.  More than one (with all their loads issued first) was measured and is
  // slower (418 vs 326 us on add, multiply, exp over 8192^2 f32): the kernel is bound by the
  // interpreter's scalar work and waits, not by the bytes in flight.
  const int u = 1;
  int64_t blocks = (a.nvec + (int64_t)FBLOCK * u - 1) / ((int64_t)FBLOCK * u);
  if (blocks > (1ll << 30)) blocks = 1ll << 30;
  dim3 grid((unsigned)blocks), block(FBLOCK);
  if (u == 4) hipLaunchKernelGGL((fused_elementwise_kernel<2, 4>), grid, block, 0, ctx->stream, a);
  else if (u == 2) hipLaunchKernelGGL((fused_elementwise_kernel<4, 2>), grid, block, 0, ctx->stream, a);
  else hipLaunchKernelGGL((fused_elementwise_kernel<7, 1>), grid, block, 0, ctx->stream, a);
  HIPNX_HIP(hipGetLastError());
  return HIPNX_OK;
}
