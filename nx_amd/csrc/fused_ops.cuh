// The device side of the fused element-wise groups, shared by the interpreting kernels of
// fused.hip and by the kernels compiled at run time for one program (fused_rtc.cpp): the lane's
// vectors, the loads with their conversions, the rounding after every instruction, the kernel
// bodies, and the program as compile-time constants.  Both forms call the same functions in the
// same order on the same values, which is what makes their results bit-identical.
// This header is also given to the run-time compiler, which has no host headers: keep it to
// device code.
#pragma once
#include "elementwise_ops.cuh"
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
  // a reduction of the result along rows that are cut into segments (nseg > 1): segment `seg` of a row covers the
  // columns [seg * seg_len, min(cols, (seg + 1) * seg_len)) and leaves its raw accumulator in partial[row * nseg + seg]
  int64_t seg_len;
  void *partial;
  int nseg, unused2;
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

// input k (element type dt, column stride cs) for the lane's FV vectors: all loads are requested,
// then converted
__device__ __forceinline__ void load_input_as(KernArgs a, int k, int dt, int cs, const int64_t (&row)[FV],
                                              const int64_t (&col)[FV], Vecs &dst) {
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

// the last, partial vector of a flat index space: only its first `valid` elements exist in memory
__device__ __forceinline__ void load_input_tail(KernArgs a, int k, int dt, int cs, const int64_t (&row)[FV],
                                                const int64_t (&col)[FV], int valid, Vecs &dst) {
  if (cs == 0) {
    load_input_as(a, k, dt, cs, row, col, dst);
    return;
  }
  const int esz = (dt == HIPNX_U8 || dt == HIPNX_S8) ? 1 : (dt == HIPNX_U32 || dt == HIPNX_S32 || dt == HIPNX_F32) ? 4 : 2;
  const char *p = (const char *)a->in[k] + (row[0] * a->in_rs[k] + col[0]) * esz;
#pragma unroll
  for (int e = 0; e < FE; e++) {
    uint32_t w = 0;
    if (e < valid)
      w = esz == 4 ? *reinterpret_cast<const uint32_t *>(p + 4 * e)
          : esz == 2 ? (uint32_t)*reinterpret_cast<const uint16_t *>(p + 2 * e)
                     : (uint32_t)*reinterpret_cast<const uint8_t *>(p + e);
    dst[0][e] = element_to_f32(w, dt);
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


// ---- the program as compile-time constants ------------------------------------------------------
// P holds the program one field per array (kind[], op[], src[], arg[], src2[], arg2[], flags[],
// dt[], imm[] and imm2[] as f32 bit patterns), the inputs' element types and column strides, and
// the result type.  Every branch the interpreter takes on an instruction field is taken by the
// compiler here.
typedef float RowStats[HIPNX_FUSED_STATS];  // results of the row reductions of earlier stages (fused_row_stages_body)

template <typename P, int SRC, int ARG, unsigned IMM, bool RAW>
__device__ __forceinline__ void fetch_static(KernArgs a, const Saved &S, const RowStats &stats, const int64_t (&row)[FV],
                                             const int64_t (&col)[FV], int valid, const float (*carry)[FE], Vecs &dst) {
  if constexpr (SRC == HIPNX_FUSED_SRC_CARRY) {  // what the previous stage reduced, at this vector
#pragma unroll
    for (int e = 0; e < FE; e++) dst[0][e] = (*carry)[e];
  } else if constexpr (SRC == HIPNX_FUSED_SRC_ROWSTAT) {
#pragma unroll
    for (int u = 0; u < FV; u++)
#pragma unroll
      for (int e = 0; e < FE; e++) dst[u][e] = stats[ARG];
  } else if constexpr (SRC == HIPNX_FUSED_SRC_INPUT) {
    // RAW: the words of a 4-byte input as they are (what the f32 path does with its bits)
    if (valid == FE) load_input_as(a, ARG, RAW ? (int)HIPNX_F32 : P::in_dt[ARG], P::in_cs[ARG], row, col, dst);
    else load_input_tail(a, ARG, RAW ? (int)HIPNX_F32 : P::in_dt[ARG], P::in_cs[ARG], row, col, valid, dst);
  } else if constexpr (SRC == HIPNX_FUSED_SRC_SAVED) {
    copy_vecs(dst, S.s[ARG]);
  } else {
#pragma unroll
    for (int u = 0; u < FV; u++)
#pragma unroll
      for (int e = 0; e < FE; e++) dst[u][e] = __uint_as_float(IMM);
  }
}

// 32-bit integers travel through the lane's vectors as raw bits; an operation on them widens to
// the 64-bit integer class of the separate kernels and keeps the low word, as their stores do
template <int OP, bool UNS>
__device__ __forceinline__ float int_binary(float x, float y, bool swap) {
  const uint32_t a = __float_as_uint(swap ? y : x), b = __float_as_uint(swap ? x : y);
  const int64_t wa = UNS ? (int64_t)a : (int64_t)(int32_t)a, wb = UNS ? (int64_t)b : (int64_t)(int32_t)b;
  return __uint_as_float((uint32_t)binary_apply<OP, int64_t, UNS>(wa, wb));
}

template <int OP, bool UNS>
__device__ __forceinline__ float int_unary(float x) {
  const uint32_t a = __float_as_uint(x);
  return __uint_as_float((uint32_t)unary_apply<OP, int64_t>(UNS ? (int64_t)a : (int64_t)(int32_t)a, 32));
}

// A program that relabels bits or computes on integers can look at the bits of a float it made.  The separate kernels
// store every NaN they compute as the one quiet NaN (0x7FC00000), so such a program does the same after each float
// instruction; bits that only pass through (an input, a BITCAST) stay as they are, there as here.
template <typename P>
constexpr bool bits_are_observed() {
  for (int i = 0; i < P::n_instr; i++)
    if (P::kind[i] == HIPNX_FUSED_BITCAST || (P::flags[i] & HIPNX_FUSED_FLAG_INT) != 0) return true;
  return false;
}
// the result is the bits of the last instruction when that is a BITCAST to f32 (any NaN pattern leaves as it came)
template <typename P>
constexpr bool result_is_relabelled_bits() {
  return P::out_dt == HIPNX_U32 || P::out_dt == HIPNX_S32 || (P::out_dt == HIPNX_F32 && P::kind[P::n_instr - 1] == HIPNX_FUSED_BITCAST);
}

// Where integer bits become a float (a BITCAST, a conversion of a computed integer) the compiler is made to forget how
// the bits were computed.  Knowing it, this compiler (a) takes an integer with few significant bits for exactly
// convertible to f16 whatever its size and drops the rounding to f16 -- (x << 24) as f16 then stays finite -- and (b) turns
// an arithmetic shift by 24 whose result a float instruction reads into that instruction's byte select, which cannot
// sign-extend: the bits of -3 relabelled as f32 (a NaN) minus 1.0 came out as -1.0.
__device__ __forceinline__ void forget_provenance(float &x) { asm volatile("" : "+v"(x)); }

// instructions PC .. END-1
template <typename P, int PC, int END>
__device__ __forceinline__ void static_steps(KernArgs a, const int64_t (&row)[FV], const int64_t (&col)[FV], Vecs &acc, Saved &S,
                                             const RowStats &stats, int valid = FE, const float (*carry)[FE] = nullptr) {
  if constexpr (PC < END) {
    constexpr int kind = P::kind[PC], op = P::op[PC], src = P::src[PC], arg = P::arg[PC];
    constexpr int src2 = P::src2[PC], arg2 = P::arg2[PC], flags = P::flags[PC], dt = P::dt[PC];
    constexpr unsigned imm = P::imm[PC], imm2 = P::imm2[PC];
    constexpr bool ints = (flags & HIPNX_FUSED_FLAG_INT) != 0, uns = dt == HIPNX_U32;
    if constexpr (kind == HIPNX_FUSED_SET) {
      fetch_static<P, src, arg, imm, ints>(a, S, stats, row, col, valid, carry, acc);
    } else if constexpr (kind == HIPNX_FUSED_UNARY) {
      if constexpr (ints) {
#pragma unroll
        for (int u = 0; u < FV; u++)
#pragma unroll
          for (int e = 0; e < FE; e++) acc[u][e] = int_unary<op, uns>(acc[u][e]);
      } else {
        unary_vecs<op>(acc);
      }
    } else if constexpr (kind == HIPNX_FUSED_BINARY) {
      Vecs y;
      fetch_static<P, src, arg, imm, ints>(a, S, stats, row, col, valid, carry, y);
      if constexpr (ints) {
#pragma unroll
        for (int u = 0; u < FV; u++)
#pragma unroll
          for (int e = 0; e < FE; e++) acc[u][e] = int_binary<op, uns>(acc[u][e], y[u][e], (flags & 1) != 0);
      } else {
        binary_vecs<op>(acc, y, (flags & 1) != 0);
      }
    } else if constexpr (kind == HIPNX_FUSED_SELECT) {
      Vecs y, z;
      fetch_static<P, src, arg, imm, false>(a, S, stats, row, col, valid, carry, y);
      fetch_static<P, src2, arg2, imm2, false>(a, S, stats, row, col, valid, carry, z);
#pragma unroll
      for (int u = 0; u < FV; u++)
#pragma unroll
        for (int e = 0; e < FE; e++) acc[u][e] = acc[u][e] != 0.0f ? y[u][e] : z[u][e];  // NaN is true
    } else if constexpr (kind == HIPNX_FUSED_AS_TYPE && ints) {  // the integer of type `op`, held as bits, to a float
#pragma unroll
      for (int u = 0; u < FV; u++)
#pragma unroll
        for (int e = 0; e < FE; e++) {
          forget_provenance(acc[u][e]);
          acc[u][e] = element_to_f32(__float_as_uint(acc[u][e]), op);
        }
    } else if constexpr (kind == HIPNX_FUSED_BITCAST) {  // changes nothing in the registers
#pragma unroll
      for (int u = 0; u < FV; u++)
#pragma unroll
        for (int e = 0; e < FE; e++) forget_provenance(acc[u][e]);
    }  // a float AS_TYPE is the rounding below
    constexpr bool computed = kind == HIPNX_FUSED_UNARY || kind == HIPNX_FUSED_BINARY || kind == HIPNX_FUSED_SELECT || kind == HIPNX_FUSED_AS_TYPE ||
                              (kind == HIPNX_FUSED_SET && (src == HIPNX_FUSED_SRC_ROWSTAT || src == HIPNX_FUSED_SRC_CARRY));
    if constexpr (dt == HIPNX_F32 && computed && bits_are_observed<P>()) {
#pragma unroll
      for (int u = 0; u < FV; u++)
#pragma unroll
        for (int e = 0; e < FE; e++) {  // (tested on the bits: a float comparison that selects between floats is folded away)
          const uint32_t b = __float_as_uint(acc[u][e]);
          acc[u][e] = __uint_as_float((b & 0x7FFFFFFFu) > 0x7F800000u ? 0x7FC00000u : b);
        }
    }
    if constexpr (dt == HIPNX_BF16 || dt == HIPNX_F16) {
#pragma unroll
      for (int u = 0; u < FV; u++)
#pragma unroll
        for (int e = 0; e < FE; e++) acc[u][e] = round_to(acc[u][e], dt);
    }
    if constexpr ((flags >> 4) != 0) copy_vecs(S.s[(flags >> 4) - 1], acc);
    static_steps<P, PC + 1, END>(a, row, col, acc, S, stats, valid, carry);
  }
}

template <typename P>
struct RunStatic {
  static __device__ __forceinline__ void run(KernArgs a, const int64_t (&row)[FV], const int64_t (&col)[FV], Vecs &acc, int valid = FE) {
    Saved S;
    const RowStats none = {};
    static_steps<P, 0, P::n_instr>(a, row, col, acc, S, none, valid);
  }
  // a u32 / s32 result leaves as the bits it is held as
  static __device__ __forceinline__ int out_dt(KernArgs) { return P::out_dt; }
  static constexpr bool raw_out = result_is_relabelled_bits<P>();
};

// ---- kernel bodies: RUN is RunStatic<P> or the interpreter of fused.hip ---------------------------
template <typename RUN>
__device__ __forceinline__ void fused_elementwise_body() {
  KernArgs a = (KernArgs)__builtin_amdgcn_kernarg_segment_ptr();
  const int64_t nvec = a->nvec, vecs_per_row = a->vecs_per_row, cols = a->cols;
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
    static_assert(FV == 1, "the partial last vector is written for one vector per lane");
    // a flat index space need not be a whole number of vectors: the last one is partial
    const int64_t left = a->rows * cols - (row[0] * cols + col[0]);
    const int valid = left < FE ? (int)left : FE;
    Vecs acc;
    if (valid == FE) RUN::run(a, row, col, acc);
    else RUN::run(a, row, col, acc, valid);
    void *out = (void *)a->out;
    const int odt = RUN::out_dt(a);
#pragma unroll
    for (int u = 0; u < FV; u++) {
      if (!live[u]) continue;
      const int64_t at = row[u] * cols + col[u];
      if (valid < FE) {
        for (int e = 0; e < valid; e++) {
          if constexpr (RUN::raw_out) ((uint32_t *)out)[at + e] = __float_as_uint(acc[u][e]);
          else store_one<float>(out, odt, at + e, acc[u][e]);
        }
      } else if constexpr (RUN::raw_out) {
        uint4 *p = reinterpret_cast<uint4 *>((uint32_t *)out + at);
        p[0] = make_uint4(__float_as_uint(acc[u][0]), __float_as_uint(acc[u][1]), __float_as_uint(acc[u][2]), __float_as_uint(acc[u][3]));
        p[1] = make_uint4(__float_as_uint(acc[u][4]), __float_as_uint(acc[u][5]), __float_as_uint(acc[u][6]), __float_as_uint(acc[u][7]));
      } else {
        store_vec<float, FE>(out, odt, at, acc[u]);
      }
    }
  }
}

// The group's result reduced along its rows without ever being stored: TPR lanes per row walk it
// in the order of reduce_rows_kernel (lane l takes the vectors l, l + TPR, ... and folds their
// elements in turn, then lanes combine by wave shuffles and the block's waves through LDS) with the
// same reducer policy, so the value equals what the element-wise group followed by the separate
// reduction kernel gives, bit for bit.  A few very long rows are cut into segments exactly as that
// kernel cuts them (plan_row_segments), a work-group each, and the same second kernel folds them.
template <typename RUN, typename R, typename CT, int TPR>
__device__ __forceinline__ void fused_reduce_rows_body() {
  static_assert(FV == 1, "one vector per lane and step");
  KernArgs a = (KernArgs)__builtin_amdgcn_kernarg_segment_ptr();
  constexpr int RPB = FBLOCK / TPR;
  const int sub = threadIdx.x / TPR, lane = threadIdx.x % TPR;
  const int64_t rows = a->rows, red = a->cols;
  const int nseg = a->nseg;
  const int64_t unit = (int64_t)blockIdx.x * RPB + sub;  // (row, segment): whole rows unless nseg > 1
  const int64_t r = nseg > 1 ? unit / nseg : unit;
  const int seg = nseg > 1 ? (int)(unit - r * nseg) : 0;
  const int64_t k0 = nseg > 1 ? (int64_t)seg * a->seg_len : 0;
  const int64_t k1 = nseg > 1 && k0 + a->seg_len < red ? k0 + a->seg_len : red;
  typename R::acc_t acc = R::init();
  if (r < rows) {
    const int64_t step = (int64_t)TPR * FE;
    for (int64_t k = k0 + (int64_t)lane * FE; k < k1; k += step) {
      const int64_t row[FV] = {r}, col[FV] = {k};
      Vecs x;
      RUN::run(a, row, col, x);
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
  if (lane == 0 && r < rows) {
    if (nseg > 1) ((typename R::acc_t *)a->partial)[r * nseg + seg] = acc;
    else finalize((void *)a->out, a->out_dt, r, acc);
  }
}

// ---- several stages over the same rows in one kernel ------------------------------------------------
// A program with HIPNX_FUSED_ROW_REDUCE markers is a sequence of stages: each stage but the last
// ends in a reduction of its value along the row, and later stages read that row statistic as an
// operand (softmax: the row maximum, then the sum of the exponentials, then the division).  One wave
// takes a row through all stages; a stage walks the row exactly as fused_reduce_rows_body does with
// TPR = WAVE (same lanes, same order, same reducer), and a statistic is carried on as the value a
// store to its type and a load would give -- so the result equals the separate kernels', bit for bit.
// The row is read again by every stage, from the caches: one wave has just read it.
template <typename CT>
__device__ __forceinline__ float as_stored(CT v, int dt) {
  switch (dt) {
    case HIPNX_BF16: return bf16_bits_to_f32(conv<CT>::to_bf16(v));
    case HIPNX_F16: return (float)bits_f16(conv<CT>::to_f16(v));
    default: return __uint_as_float(conv<CT>::to_f32(v));
  }
}

// The walk of a row: lane l takes the vectors l, l + WAVE, ... -- at most P::nv of them when the program
// carries element values from one stage to the next (their registers are indexed by the trip), any
// number otherwise.
template <typename P, typename F>
__device__ __forceinline__ void for_each_vector(int lane, int64_t cols, F &&body) {
  if constexpr (P::nv > 0) {
#pragma unroll
    for (int it = 0; it < P::nv; it++) {
      const int64_t k = ((int64_t)lane + (int64_t)it * P::tpr) * FE;
      if (k < cols) body(k, it);
    }
  } else {
    for (int64_t k = (int64_t)lane * FE; k < cols; k += (int64_t)P::tpr * FE) body(k, 0);
  }
}

// the reduction of a stage over the P::tpr lanes of a row, left in every lane: within a wave by the
// butterfly, across the waves of a block through LDS in the order of fused_reduce_rows_body
template <typename P, typename R>
__device__ __forceinline__ typename R::acc_t row_reduce(typename R::acc_t acc) {
  acc = wave_reduce<R>(acc);
  if constexpr (P::tpr > WAVE) {
    __shared__ typename R::acc_t sm[FBLOCK / WAVE];
    __syncthreads();  // the previous stage's readers are done with sm
    if (threadIdx.x % WAVE == 0) sm[threadIdx.x / WAVE] = acc;
    __syncthreads();
    acc = sm[0];
#pragma unroll
    for (int w = 1; w < FBLOCK / WAVE; w++) acc = R::combine(acc, sm[w]);
  }
  return acc;
}

template <typename P, int SEG, typename CARRY>
__device__ __forceinline__ void row_stage(KernArgs a, int64_t r, int lane, RowStats &stats, CARRY &carry) {
  // stage SEG: instructions [begin, red) on the row's elements, the reduction at `red`, instructions
  // (red, save) on the statistic, which is kept at `save`; the last stage is [begin, n_instr)
  constexpr int begin = SEG == 0 ? 0 : P::seg_save[SEG - 1] + 1;
  constexpr int red = P::seg_red[SEG], save = P::seg_save[SEG];
  const int64_t cols = a->cols;
  if constexpr (red < 0) {  // the last stage: its value is the result
    void *out = (void *)a->out;
    for_each_vector<P>(lane, cols, [&](int64_t k, int it) {
      const int64_t row[FV] = {r}, col[FV] = {k};
      Vecs x;
      Saved S;
      static_steps<P, begin, P::n_instr>(a, row, col, x, S, stats, FE, &carry[it]);
      if constexpr (result_is_relabelled_bits<P>()) {
        uint4 *p = reinterpret_cast<uint4 *>((uint32_t *)out + r * cols + k);
        p[0] = make_uint4(__float_as_uint(x[0][0]), __float_as_uint(x[0][1]), __float_as_uint(x[0][2]), __float_as_uint(x[0][3]));
        p[1] = make_uint4(__float_as_uint(x[0][4]), __float_as_uint(x[0][5]), __float_as_uint(x[0][6]), __float_as_uint(x[0][7]));
      } else {
        store_vec<float, FE>(out, P::out_dt, r * cols + k, x[0]);
      }
    });
  } else {
    constexpr int op = P::op[red];
    typedef typename std::conditional<op == HIPNX_RED_SUM, double, float>::type CT;
    typedef PlainReducer<CT, op, false> R;
    typename R::acc_t acc = R::init();
    for_each_vector<P>(lane, cols, [&](int64_t k, int it) {
      const int64_t row[FV] = {r}, col[FV] = {k};
      Vecs x;
      Saved S;
      static_steps<P, begin, red>(a, row, col, x, S, stats, FE, &carry[it]);
#pragma unroll
      for (int e = 0; e < FE; e++) acc = R::accumulate(acc, (CT)x[0][e], k + e);
      if constexpr (P::nv > 0) {  // kept for the next stage (after this stage's own reads of the previous one's)
#pragma unroll
        for (int e = 0; e < FE; e++) carry[it][e] = x[0][e];
      }
    });
    acc = row_reduce<P, R>(acc);  // the same value in every lane of the row
    // the work on the statistic: the same instructions on a vector that holds it eight times
    const int64_t row[FV] = {r}, col[FV] = {0};
    Vecs x;
    Saved S;
#pragma unroll
    for (int e = 0; e < FE; e++) x[0][e] = as_stored<CT>(acc, P::dt[red]);
    static_steps<P, red + 1, save>(a, row, col, x, S, stats);
    if constexpr ((P::flags[save] & HIPNX_FUSED_FLAG_RESULT) != 0) {  // this one value per row is the result
      if (lane == 0) store_one<float>((void *)a->out, P::out_dt, r, x[0][0]);  // lane 0 of the row
    } else {
      stats[P::arg[save]] = x[0][0];
      row_stage<P, SEG + 1>(a, r, lane, stats, carry);
    }
  }
}

template <typename P>
__device__ __forceinline__ void fused_row_stages_body() {
  static_assert(FV == 1, "one vector per lane and step");
  KernArgs a = (KernArgs)__builtin_amdgcn_kernarg_segment_ptr();
  // P::tpr lanes per row: a wave (rows of at most 4096 elements) or the whole block, as the separate reduction has it
  const int64_t r = (int64_t)blockIdx.x * (FBLOCK / P::tpr) + threadIdx.x / P::tpr;
  if (r >= a->rows) return;  // (a whole wave, or with a block per row nobody: no barrier is left waiting)
  RowStats stats = {};
  float carry[P::nv > 0 ? P::nv : 1][FE];  // (indexed by compile-time trip numbers only: registers)
  row_stage<P, 0>(a, r, threadIdx.x % P::tpr, stats, carry);
}

}  // namespace hipnx
