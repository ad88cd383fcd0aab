// Broadcasting element-wise binary / unary kernels and as_type: HBM streaming kernels.
//
// Each lane owns E = 8 consecutive output elements and moves them with 16-byte accesses.  A
// binary op first has its index space collapsed on the host (unit axes dropped, axes merged
// where both operands stay contiguous or both broadcast); whatever collapses to [rows, cols]
// with per-operand strides (row stride, column stride in {0, 1}) -- same shape, scalar operand,
// trailing row vector, keep-dims column -- runs on the vector kernel, the rest on a generic
// rank-N kernel.  Algorithmic traffic is exactly bytes(l) + bytes(r) + bytes(out).
#include <type_traits>

#include "elementwise_ops.cuh"
#include "internal.h"

namespace hipnx {

constexpr int E = 8;
// A lane's vector when the element types are known at compile time: 16 bytes of the WIDEST type involved -- 8 elements of
// 1 or 2 bytes, 4 of 4 bytes, 2 of 8 bytes.  One 16-byte access per lane with the lanes side by side is what streams
// fastest here: a wave instruction then covers whole cache lines, where two adjacent 16-byte accesses per lane (eight
// f32) make every instruction touch twice the lines it fills (f32 multiply: 8.4 M elements 11.3 -> 9.4 us, 268 M
// elements 5.8 -> 6.2 TB/s; bf16 -> f32 conversion of 8.4 M elements 9.6 -> 7.6 us).  The narrower side of a
// conversion or comparison moves 8, 4 or 2 bytes per lane, still lanes side by side.
constexpr int fixed_type_bytes(int dt) {
  return dt < 0 ? 0
         : (dt == HIPNX_U8 || dt == HIPNX_S8) ? 1
         : (dt == HIPNX_U16 || dt == HIPNX_S16 || dt == HIPNX_F16 || dt == HIPNX_BF16 || dt == HIPNX_BF16_RNE) ? 2
         : (dt == HIPNX_U32 || dt == HIPNX_S32 || dt == HIPNX_F32) ? 4 : 8;
}
constexpr int vec_elems(int fix_in, int fix_out) {
  const int a = fixed_type_bytes(fix_in), b = fixed_type_bytes(fix_out), w = a > b ? a : b;
  return w == 8 ? 2 : w == 4 ? 4 : 8;  // (types known at run time only: 8 elements)
}
constexpr int BLOCK = 256;
constexpr int MAXR = 8;

struct NdIndex {
  int rank;
  int64_t dims[MAXR], ls[MAXR], rs[MAXR];
};

// Division of an index below 2^31 by an invariant divisor below 2^31 as one multiplication: the 64-bit
// division the compiler emits costs every wave some hundred scalar and vector instructions, more than the
// rest of an 8-element vector's work.
struct FastDiv32 {
  uint32_t mul, shr;
};
static FastDiv32 make_fastdiv(uint32_t d) {
  uint32_t shr = 0;
  while ((1ull << shr) < d) shr++;
  return FastDiv32{(uint32_t)(((1ull << 32) * ((1ull << shr) - d)) / d + 1), shr};
}
__device__ __forceinline__ uint32_t fastdiv(uint32_t n, FastDiv32 f) { return (__umulhi(n, f.mul) + n) >> f.shr; }

// how a vector index splits into (row, column); the FLAT modes cut the flat output into vectors that may run across
// row ends (rows whose length is not a whole number of vectors) and count `vecs_per_row` as the element count
enum { ROWS_ONE = 0, ROWS_FAST = 1, ROWS_WIDE = 2, ROWS_FLAT = 3, ROWS_FLAT_WIDE = 4 };

// Rows that are themselves two or three collapsed axes with their own strides per operand (a mask [b, 1, 1, s]
// against scores [b, h, s, s] collapses to [b, h * s | s]: the mask's row offset is b's index times s, not a
// multiple of the row number).  n = 0 or 1: a row's offset is row * stride, as without this; else the row
// number is taken apart from the innermost of its axes outwards (d[k] = extent, fd[k] its reciprocal, k >= 1).
struct RowAxes {
  int n;
  uint32_t d[3];
  FastDiv32 fd[3];
  int64_t ls[3], rs[3];
};

// FIX >= 0: both operands and the result have this element type, known when the kernel is compiled -- the
// three run-time type switches (and the scalar bookkeeping the compiler builds around them, ~200 scalar
// instructions per wave) fold away.  bf16 add on 16384^2: 388 -> 263 us (4.1 -> 6.1 TB/s), negate and exp 280 -> 175 us.
// (FIXO: the result's type when it differs -- u8 for comparisons and logical operations.)
template <int OP, typename CT, bool UNS, int FIX = -1, int FIXO = FIX>
__global__ void __launch_bounds__(BLOCK)
binary_vec_kernel(const void *__restrict__ l, const void *__restrict__ r, void *__restrict__ out, int ldt_, int rdt_,
                  int odt_, int64_t cols, int64_t vecs_per_row, int64_t nvec, int64_t ls0, int ls1, int64_t rs0,
                  int rs1, unsigned long long *__restrict__ err, int rows_mode, FastDiv32 fd, RowAxes ax) {
  constexpr bool RAISES = binary_can_raise(OP, is_fp<CT>::value);
  constexpr int E = vec_elems(FIX, FIXO);  // (vecs_per_row and nvec are counted in these by the launcher)
  const int ldt = FIX >= 0 ? FIX : ldt_, rdt = FIX >= 0 ? FIX : rdt_, odt = FIX >= 0 ? FIXO : odt_;
  for (int64_t v = (int64_t)blockIdx.x * BLOCK + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * BLOCK) {
    int64_t row, col;
    if (rows_mode >= ROWS_FLAT) {
      // [rows, cols] with cols not a whole number of vectors (x[N, 3] * w[3], x[N, 5] + b[N, 1]): a lane takes E
      // consecutive outputs anyway -- an operand as dense as the output is one vector load, a broadcast one is read
      // element by element (from a row or a column that the cache holds) -- instead of one output per lane with
      // its index divisions (1.5 TB/s whatever the element type)
      const int64_t total = vecs_per_row, f0 = v * E;
      if (rows_mode == ROWS_FLAT) {
        const uint32_t q = fastdiv((uint32_t)f0, fd);
        row = q;
        col = (int64_t)((uint32_t)f0 - q * (uint32_t)cols);
      } else {
        row = f0 / cols;
        col = f0 - row * cols;
      }
      const int nel = f0 + E <= total ? E : (int)(total - f0);
      // (with rows of several axes, ls0 / rs0 only say whether the operand is as dense as the output: cols if so)
      const bool l_dense = ls1 == 1 && ls0 == cols && nel == E, r_dense = rs1 == 1 && rs0 == cols && nel == E;
      int64_t lrow = 0, rrow = 0;
      auto row_offsets = [&]() {  // where row `row` begins in each operand
        if (ax.n <= 1) {
          lrow = row * ls0;
          rrow = row * rs0;
        } else {
          uint32_t rem = (uint32_t)row;
          lrow = 0;
          rrow = 0;
          for (int k = ax.n - 1; k >= 1; k--) {
            const uint32_t q = fastdiv(rem, ax.fd[k]), i = rem - q * ax.d[k];
            lrow += (int64_t)i * ax.ls[k];
            rrow += (int64_t)i * ax.rs[k];
            rem = q;
          }
          lrow += (int64_t)rem * ax.ls[0];
          rrow += (int64_t)rem * ax.rs[0];
        }
      };
      row_offsets();
      CT a[E], b[E], c[E];
      if (l_dense) load_vec<CT, E>(l, ldt, f0, a);
      if (r_dense) load_vec<CT, E>(r, rdt, f0, b);
#pragma unroll
      for (int i = 0; i < E; i++) {
        if (i < nel) {
          if (!l_dense) a[i] = load_one<CT>(l, ldt, lrow + col * ls1);
          if (!r_dense) b[i] = load_one<CT>(r, rdt, rrow + col * rs1);
        } else {
          a[i] = (CT)1;
          b[i] = (CT)1;
        }
        if (++col == cols) {
          col = 0;
          row++;
          if (i + 1 < nel) row_offsets();
        }
      }
#pragma unroll
      for (int i = 0; i < E; i++) c[i] = binary_apply<OP, CT, UNS>(a[i], b[i]);
      if constexpr (RAISES) {
        long long operand = 0;
#pragma unroll
        for (int i = 0; i < E; i++)
          if (int code = binary_raises<OP, CT, UNS>(a[i], b[i], &operand)) report_raise(err, code, operand);
      }
      if (nel == E) store_vec<CT, E>(out, odt, f0, c);
      else
        for (int i = 0; i < nel; i++) store_one<CT>(out, odt, f0 + i, c[i]);
      continue;
    }
    if (rows_mode == ROWS_ONE) {
      row = 0;
      col = v * E;
    } else if (rows_mode == ROWS_FAST) {
      const uint32_t q = fastdiv((uint32_t)v, fd);
      row = q;
      col = (int64_t)((uint32_t)v - q * (uint32_t)vecs_per_row) * E;
    } else {
      row = v / vecs_per_row;
      col = (v - row * vecs_per_row) * E;
    }
    int64_t lo, ro;
    const int64_t oo = row * cols + col;
    if (ax.n <= 1) {
      lo = row * ls0 + col * ls1;
      ro = row * rs0 + col * rs1;
    } else {
      uint32_t rem = (uint32_t)row;  // (the launcher takes this form only with fewer than 2^31 rows)
      lo = col * ls1;
      ro = col * rs1;
      for (int k = ax.n - 1; k >= 1; k--) {
        const uint32_t q = fastdiv(rem, ax.fd[k]), i = rem - q * ax.d[k];
        lo += (int64_t)i * ax.ls[k];
        ro += (int64_t)i * ax.rs[k];
        rem = q;
      }
      lo += (int64_t)rem * ax.ls[0];
      ro += (int64_t)rem * ax.rs[0];
    }
    CT a[E], b[E], c[E];
    if (col + E <= cols) {
      if (ls1) load_vec<CT, E>(l, ldt, lo, a);
      else {
        CT s = load_one<CT>(l, ldt, lo);
#pragma unroll
        for (int i = 0; i < E; i++) a[i] = s;
      }
      if (rs1) load_vec<CT, E>(r, rdt, ro, b);
      else {
        CT s = load_one<CT>(r, rdt, ro);
#pragma unroll
        for (int i = 0; i < E; i++) b[i] = s;
      }
#pragma unroll
      for (int i = 0; i < E; i++) c[i] = binary_apply<OP, CT, UNS>(a[i], b[i]);
      if constexpr (RAISES) {
        long long operand = 0;
#pragma unroll
        for (int i = 0; i < E; i++)
          if (int code = binary_raises<OP, CT, UNS>(a[i], b[i], &operand)) report_raise(err, code, operand);
      }
      store_vec<CT, E>(out, odt, oo, c);
    } else {  // ragged tail of a row
      for (int i = 0; col + i < cols; i++) {
        CT x = load_one<CT>(l, ldt, lo + i * ls1), y = load_one<CT>(r, rdt, ro + i * rs1);
        if constexpr (RAISES) {
          long long operand = 0;
          if (int code = binary_raises<OP, CT, UNS>(x, y, &operand)) report_raise(err, code, operand);
        }
        store_one<CT>(out, odt, oo + i, binary_apply<OP, CT, UNS>(x, y));
      }
    }
  }
}

// The common case of the above as a kernel of its own: element types known when it is compiled, an operation that
// cannot raise, rows that are whole vectors and one stride pair per operand -- [rows, cols] against itself, a row
// [cols], one value per row or one value.  Every wave of the general kernel spends some 0.4 us on eleven scalar
// loads of its arguments and the branches that choose its path before it asks for data; a wave lives for about
// 2.5 us, and at 4 to 64 MiB the grid is few waves deep, so that time shows: 8.4 M f32 elements, x * scalar
// 11.7 -> 10.6 us, x - value per row 10.7 -> 9.7 us, x + y 16.1 -> 14.7 us.
//   LM / RM: how an operand is met: 0 one value (read through the scalar cache: one address asked for by every
//   wave at once is a hot spot in the vector path), 1 one value per row, 2 whole vectors (row * s0 + col).
//   U vectors per lane, lanes side by side (v, v + 256, ...), every load issued before the first result is formed:
//   two for x + y of 1 to 64 MiB a side (32 MiB: 15.3 -> 14.7 us); beyond the last-level cache one streams faster
//   (1 GiB a side: 534 against 562 us).
//   NT: the tensors are far larger than the last-level cache and every access carries the non-temporal hint (a
//   template parameter, not an argument: where a branch chooses between a hinted and a plain access the compiler
//   merges the two and drops the hint).
template <int OP, typename CT, bool UNS, int FIX, int FIXO, int LM, int RM, int U, bool NT = false>
__global__ void __launch_bounds__(BLOCK)
binary_rows_kernel(const void *__restrict__ l, const void *__restrict__ r, void *__restrict__ out, uint32_t nvec,
                   uint32_t vecs_per_row, FastDiv32 fd, int64_t ls0, int64_t rs0) {
  constexpr int E = vec_elems(FIX, FIXO);
  const uint32_t v0 = blockIdx.x * (uint32_t)(BLOCK * U) + threadIdx.x;
  CT a[U][E], b[U][E];
  CT l_one = (CT)0, r_one = (CT)0;
  if constexpr (LM == 0) l_one = load_one<CT>(l, FIX, 0);
  if constexpr (RM == 0) r_one = load_one<CT>(r, FIX, 0);
#pragma unroll
  for (int u = 0; u < U; u++) {
    const uint32_t v = v0 + u * BLOCK;
    if (v < nvec) {
      const uint32_t row = fastdiv(v, fd), col = (v - row * vecs_per_row) * E;
      if constexpr (LM == 2) load_vec<CT, E, true, NT>(l, FIX, (int64_t)row * ls0 + col, a[u]);
      else {
        const CT s = LM == 0 ? l_one : load_one<CT>(l, FIX, (int64_t)row * ls0);
#pragma unroll
        for (int i = 0; i < E; i++) a[u][i] = s;
      }
      if constexpr (RM == 2) load_vec<CT, E, true, NT>(r, FIX, (int64_t)row * rs0 + col, b[u]);
      else {
        const CT s = RM == 0 ? r_one : load_one<CT>(r, FIX, (int64_t)row * rs0);
#pragma unroll
        for (int i = 0; i < E; i++) b[u][i] = s;
      }
    }
  }
#pragma unroll
  for (int u = 0; u < U; u++) {
    const uint32_t v = v0 + u * BLOCK;
    if (v < nvec) {
      CT c[E];
#pragma unroll
      for (int i = 0; i < E; i++) c[i] = binary_apply<OP, CT, UNS>(a[u][i], b[u][i]);
      store_vec<CT, E, NT>(out, FIXO, (int64_t)v * E, c);
    }
  }
}

template <typename CT, bool UNS>
__device__ __forceinline__ CT binary_switch(int op, CT a, CT b) {
  switch (op) {
#define C(O) case O: return binary_apply<O, CT, UNS>(a, b);
    C(0) C(1) C(2) C(3) C(4) C(5) C(6) C(7) C(8) C(9) C(10) C(11) C(12) C(13) C(14) C(15) C(16) C(17) C(18) C(19)
    C(20) C(21) C(22) C(23)
#undef C
  }
  return (CT)0;
}

template <typename CT, bool UNS>
__device__ __forceinline__ int binary_raises_switch(int op, CT a, CT b, long long *operand) {
  switch (op) {
    case HIPNX_QUOTIENT: return binary_raises<HIPNX_QUOTIENT, CT, UNS>(a, b, operand);
    case HIPNX_REMAINDER: return binary_raises<HIPNX_REMAINDER, CT, UNS>(a, b, operand);
    case HIPNX_LEFT_SHIFT: return binary_raises<HIPNX_LEFT_SHIFT, CT, UNS>(a, b, operand);
    case HIPNX_RIGHT_SHIFT: return binary_raises<HIPNX_RIGHT_SHIFT, CT, UNS>(a, b, operand);
    case HIPNX_POW: return binary_raises<HIPNX_POW, CT, UNS>(a, b, operand);
  }
  return HIPNX_RAISE_NONE;
}

// any rank, any strides: one element per lane per step
template <typename CT, bool UNS>
__global__ void __launch_bounds__(BLOCK)
binary_nd_kernel(const void *__restrict__ l, const void *__restrict__ r, void *__restrict__ out, int op, int ldt,
                 int rdt, int odt, int64_t n, NdIndex ix, unsigned long long *__restrict__ err) {
  const bool raises = binary_can_raise(op, is_fp<CT>::value);
  for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < n; i += (int64_t)gridDim.x * BLOCK) {
    int64_t rem = i, lo = 0, ro = 0;
    for (int a = ix.rank - 1; a >= 0; a--) {
      int64_t q = rem / ix.dims[a], c = rem - q * ix.dims[a];
      rem = q;
      lo += c * ix.ls[a];
      ro += c * ix.rs[a];
    }
    CT x = load_one<CT>(l, ldt, lo), y = load_one<CT>(r, rdt, ro);
    if (raises) {
      long long operand = 0;
      if (int code = binary_raises_switch<CT, UNS>(op, x, y, &operand)) report_raise(err, code, operand);
    }
    store_one<CT>(out, odt, i, binary_switch<CT, UNS>(op, x, y));
  }
}

template <int OP, typename CT, int FIX = -1, bool NT = false>  // FIX: the one element type of input and result, as above; NT: as above
__global__ void __launch_bounds__(BLOCK)
unary_vec_kernel(const void *__restrict__ in, void *__restrict__ out, int idt_, int odt_, int bits, int64_t n) {
  const int idt = FIX >= 0 ? FIX : idt_, odt = FIX >= 0 ? FIX : odt_;
  constexpr int E = vec_elems(FIX, FIX);
  int64_t nvec = (n + E - 1) / E;
  for (int64_t v = (int64_t)blockIdx.x * BLOCK + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * BLOCK) {
    int64_t o = v * E;
    if (o + E <= n) {
      CT a[E], c[E];
      load_vec<CT, E, true, NT>(in, idt, o, a);
#pragma unroll
      for (int i = 0; i < E; i++) c[i] = unary_apply<OP, CT>(a[i], bits);
      store_vec<CT, E, NT>(out, odt, o, c);
    } else {
      for (int i = 0; o + i < n; i++)
        store_one<CT>(out, odt, o + i, unary_apply<OP, CT>(load_one<CT>(in, idt, o + i), bits));
    }
  }
}

// as_type: CT is the decode type of the input; float -> integer goes through the wrap rule.
// FIXI / FIXO >= 0: input and result type known when the kernel is compiled.
template <typename CT, int FIXI = -1, int FIXO = -1, bool NT = false>
__global__ void __launch_bounds__(BLOCK)
as_type_kernel(const void *__restrict__ in, void *__restrict__ out, int idt_, int odt_, int64_t n, int64_t tmax,
               int64_t tmin) {
  const int idt = FIXI >= 0 ? FIXI : idt_, odt = FIXO >= 0 ? FIXO : odt_;
  constexpr int E = vec_elems(FIXI, FIXO);
  const bool to_int = odt < HIPNX_F16;
  int64_t nvec = (n + E - 1) / E;
  for (int64_t v = (int64_t)blockIdx.x * BLOCK + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * BLOCK) {
    int64_t o = v * E;
    if (o + E <= n) {
      CT a[E];
      load_vec<CT, E, true, NT>(in, idt, o, a);
      if constexpr (is_fp<CT>::value) {
        if (to_int) {
          int64_t c[E];
#pragma unroll
          for (int i = 0; i < E; i++) c[i] = float_to_int_wrap((double)a[i], tmax, tmin);
          store_vec<int64_t, E, NT>(out, odt, o, c);
          continue;
        }
      }
      store_vec<CT, E, NT>(out, odt, o, a);
    } else {
      for (int i = 0; o + i < n; i++) {
        CT x = load_one<CT>(in, idt, o + i);
        if constexpr (is_fp<CT>::value) {
          if (to_int) {
            store_one<int64_t>(out, odt, o + i, float_to_int_wrap((double)x, tmax, tmin));
            continue;
          }
        }
        store_one<CT>(out, odt, o + i, x);
      }
    }
  }
}

// ---- host side ------------------------------------------------------------------------------

enum { CLS_F32 = 0, CLS_F64 = 1, CLS_I64 = 2, CLS_U64 = 3 };

// Whether a launch over `n` elements moves tensors far larger than the 256 MB last-level cache (the widest of the
// element types decides): its loads and stores then carry the non-temporal hint.  Smaller tensors are better left in
// the cache for the callback that reads them next.
static int streams_past_cache(int64_t n, int dt_a, int dt_b = -1, int dt_c = -1) {
  int widest = dtype_size(dt_a);
  if (dt_b >= 0 && dtype_size(dt_b) > widest) widest = dtype_size(dt_b);
  if (dt_c >= 0 && dtype_size(dt_c) > widest) widest = dtype_size(dt_c);
  return n * widest >= (256ll << 20);
}

static int grid_for(const hipnx_ctx *ctx, int64_t work_items) {
  int64_t blocks = (work_items + BLOCK - 1) / BLOCK;
  // one 8-element vector per lane: on this part a grid that covers the whole tensor streams
  // faster than a resident grid looping over it (5.8 vs 5.1 TB/s on a 1 GiB add)
  (void)ctx;
  int64_t cap = ((1ll << 32) - 1) / BLOCK;  // a launch may hold at most 2^32 - 1 lanes: the kernels loop over the rest
  if (blocks < 1) blocks = 1;
  return (int)(blocks < cap ? blocks : cap);
}

struct BinArgs {
  const void *l, *r;
  void *out;
  int ldt, rdt, odt;
  int64_t cols, vecs_per_row, nvec, ls0, rs0;
  int ls1, rs1;
  unsigned long long *err;  // the context's deferred error word (device address of the pinned host word)
  RowAxes ax;
  int64_t flat_total;  // > 0: the FLAT modes over this many outputs (rows * cols)
  int stream;          // the tensors are far larger than the last-level cache: loads and stores carry the non-temporal hint
};

template <int OP, typename CT, bool UNS, int FIX, int FIXO = FIX>
static void launch_bvec_fix(const hipnx_ctx *ctx, const BinArgs &a_) {
  BinArgs a = a_;
  constexpr int EV = vec_elems(FIX, FIXO);
  if (EV != E) {  // the caller counted vectors of E elements
    const int64_t rows = a.nvec / a.vecs_per_row;
    a.vecs_per_row = (a.cols + EV - 1) / EV;
    a.nvec = rows * a.vecs_per_row;
  }
  int mode = a.vecs_per_row >= a.nvec ? ROWS_ONE : a.nvec < (1ll << 31) ? ROWS_FAST : ROWS_WIDE;
  FastDiv32 fd = mode == ROWS_FAST ? make_fastdiv((uint32_t)a.vecs_per_row) : FastDiv32{0, 0};
  if (a.flat_total > 0) {
    a.vecs_per_row = a.flat_total;
    a.nvec = (a.flat_total + EV - 1) / EV;
    mode = a.flat_total < (1ll << 31) ? ROWS_FLAT : ROWS_FLAT_WIDE;
    if (mode == ROWS_FLAT) fd = make_fastdiv((uint32_t)a.cols);
  }
  if constexpr (FIX >= 0 && !binary_can_raise(OP, is_fp<CT>::value)) {
    if (a.flat_total <= 0 && a.ax.n <= 1 && a.cols % EV == 0 && a.nvec < (1ll << 31)) {
      const bool one_row = mode == ROWS_ONE;
      const uint32_t nvec = (uint32_t)a.nvec, vpr = one_row ? nvec : (uint32_t)a.vecs_per_row;
      const FastDiv32 fdr = make_fastdiv(vpr);
      // how each operand is met (an operand of one row has no row stride to speak of)
      const int64_t l0 = one_row ? 0 : a.ls0, r0 = one_row ? 0 : a.rs0;
      const int lm = a.ls1 ? 2 : l0 ? 1 : 0, rm = a.rs1 ? 2 : r0 ? 1 : 0;
#define HIPNX_ROWS(LM, RM, U)                                                                                           \
  do {                                                                                                                  \
    const dim3 g((unsigned)((a.nvec + BLOCK * U - 1) / (BLOCK * U)));                                                    \
    if (U == 1 && a.stream)                                                                                             \
      hipLaunchKernelGGL((binary_rows_kernel<OP, CT, UNS, FIX, FIXO, LM, RM, 1, true>), g, dim3(BLOCK), 0, ctx->stream, \
                         a.l, a.r, a.out, nvec, vpr, fdr, l0, r0);                                                      \
    else                                                                                                                \
      hipLaunchKernelGGL((binary_rows_kernel<OP, CT, UNS, FIX, FIXO, LM, RM, U>), g, dim3(BLOCK), 0, ctx->stream, a.l,  \
                         a.r, a.out, nvec, vpr, fdr, l0, r0);                                                           \
  } while (0)
      // (two streams in and one out, each beyond 128 MiB: the general kernel is as fast, and with the three buffers
      // half a GiB apart this one lost 7 % -- bf16 x + y of 2^28 elements 260 against 279 us)
      const int how = lm == 2 && rm == 2 && a.nvec > (1 << 23) && !a.stream ? -1 : lm * 3 + rm;
      if (how == 8 && a.nvec >= (1 << 16) && a.nvec <= (1 << 22)) HIPNX_ROWS(2, 2, 2);  // (1 to 64 MiB a side)
      else if (how == 8) HIPNX_ROWS(2, 2, 1);
      else if (how == 7) HIPNX_ROWS(2, 1, 1);
      else if (how == 6) HIPNX_ROWS(2, 0, 1);
      else if (how == 5) HIPNX_ROWS(1, 2, 1);
      else if (how == 2) HIPNX_ROWS(0, 2, 1);
#undef HIPNX_ROWS
      if (how == 2 || how >= 5) return;
    }
  }
  hipLaunchKernelGGL((binary_vec_kernel<OP, CT, UNS, FIX, FIXO>), dim3(grid_for(ctx, a.nvec)), dim3(BLOCK), 0, ctx->stream, a.l,
                     a.r, a.out, a.ldt, a.rdt, a.odt, a.cols, a.vecs_per_row, a.nvec, a.ls0, a.ls1, a.rs0, a.rs1, a.err,
                     mode, fd, a.ax);
}

// the kernel compiled for one element type throughout, where there is one: the types of most tensor arithmetic
template <int OP, typename CT, bool UNS>
static void launch_bvec(const hipnx_ctx *ctx, const BinArgs &a) {
  if (a.ldt == a.rdt && a.ldt == a.odt) {
    if constexpr (std::is_same<CT, float>::value) {
      if (a.odt == HIPNX_F32) return launch_bvec_fix<OP, CT, UNS, HIPNX_F32>(ctx, a);
      if (a.odt == HIPNX_BF16) return launch_bvec_fix<OP, CT, UNS, HIPNX_BF16>(ctx, a);
      if (a.odt == HIPNX_F16) return launch_bvec_fix<OP, CT, UNS, HIPNX_F16>(ctx, a);
    } else if constexpr (std::is_same<CT, double>::value) {
      if (a.odt == HIPNX_F64) return launch_bvec_fix<OP, CT, UNS, HIPNX_F64>(ctx, a);
    } else if constexpr (!UNS) {
      if (a.odt == HIPNX_S32) return launch_bvec_fix<OP, CT, UNS, HIPNX_S32>(ctx, a);
      if (a.odt == HIPNX_S64) return launch_bvec_fix<OP, CT, UNS, HIPNX_S64>(ctx, a);
    }
  }
  if (a.ldt == a.rdt && a.odt == HIPNX_U8) {  // what comparisons and logical operations produce
    if constexpr (std::is_same<CT, float>::value) {
      if (a.ldt == HIPNX_F32) return launch_bvec_fix<OP, CT, UNS, HIPNX_F32, HIPNX_U8>(ctx, a);
      if (a.ldt == HIPNX_BF16) return launch_bvec_fix<OP, CT, UNS, HIPNX_BF16, HIPNX_U8>(ctx, a);
      if (a.ldt == HIPNX_F16) return launch_bvec_fix<OP, CT, UNS, HIPNX_F16, HIPNX_U8>(ctx, a);
    } else if constexpr (std::is_same<CT, int64_t>::value && !UNS) {
      if (a.ldt == HIPNX_S32) return launch_bvec_fix<OP, CT, UNS, HIPNX_S32, HIPNX_U8>(ctx, a);
      if (a.ldt == HIPNX_U8) return launch_bvec_fix<OP, CT, UNS, HIPNX_U8, HIPNX_U8>(ctx, a);
    }
  }
  launch_bvec_fix<OP, CT, UNS, -1>(ctx, a);
}

template <int OP>
static int launch_bvec_cls(const hipnx_ctx *ctx, int cls, const BinArgs &a) {
  if constexpr (!binary_int_only(OP)) {
    if (cls == CLS_F32) { launch_bvec<OP, float, false>(ctx, a); return HIPNX_OK; }
    if (cls == CLS_F64) { launch_bvec<OP, double, false>(ctx, a); return HIPNX_OK; }
  }
  if constexpr (!binary_float_only(OP)) {
    if (cls == CLS_I64) { launch_bvec<OP, int64_t, false>(ctx, a); return HIPNX_OK; }
    if (cls == CLS_U64) {
      if constexpr (binary_sign_matters(OP)) launch_bvec<OP, int64_t, true>(ctx, a);
      else launch_bvec<OP, int64_t, false>(ctx, a);
      return HIPNX_OK;
    }
  }
  return set_error(HIPNX_EINVAL, "binary op %d is not defined for these operand types", OP);
}

template <int... OPS>
static int launch_bvec_op(std::integer_sequence<int, OPS...>, const hipnx_ctx *ctx, int op, int cls,
                          const BinArgs &a) {
  int st = HIPNX_EINVAL;
  (void)((op == OPS ? (st = launch_bvec_cls<OPS>(ctx, cls, a), true) : false) || ...);
  return st;
}

static int binary_class(int op, int l_dt, int r_dt, int out_dt) {
  bool any_float = is_float(l_dt) || is_float(r_dt) || is_float(out_dt);
  if (any_float) {
    bool wide = is_wide(l_dt) || is_wide(r_dt) || out_dt == HIPNX_F64;
    return wide ? CLS_F64 : CLS_F32;
  }
  bool uns = is_unsigned(l_dt) && is_unsigned(r_dt) && (l_dt == HIPNX_U64 || r_dt == HIPNX_U64);
  return uns ? CLS_U64 : CLS_I64;
}

}  // namespace hipnx

using namespace hipnx;

extern "C" int hipnx_binary(hipnx_ctx *ctx, int op, int l_dt, int r_dt, int out_dt, int rank,
                            const int64_t *out_dims, const int64_t *l_strides, const int64_t *r_strides,
                            const hipnx_buf *l, const hipnx_buf *r, hipnx_buf *out) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (op < 0 || op >= HIPNX_NBINARY) return set_error(HIPNX_EINVAL, "binary: unknown op %d", op);
  if (dtype_size(l_dt) < 0 || dtype_size(r_dt) < 0 || dtype_size(out_dt) < 0)
    return set_error(HIPNX_EINVAL, "binary: unknown element type");
  if (rank < 0 || rank > 64 || (rank > 0 && (!out_dims || !l_strides || !r_strides)))
    return set_error(HIPNX_EINVAL, "binary: bad rank / null shape");
  // extent of each operand = 1 + sum (dim-1)*stride
  int64_t n = 1, l_ext = 1, r_ext = 1;
  for (int a = 0; a < rank; a++) {
    if (out_dims[a] < 0 || l_strides[a] < 0 || r_strides[a] < 0)
      return set_error(HIPNX_EINVAL, "binary: negative dimension or stride");
    n *= out_dims[a];
  }
  if (n > 0)
    for (int a = 0; a < rank; a++) {
      l_ext += (out_dims[a] - 1) * l_strides[a];
      r_ext += (out_dims[a] - 1) * r_strides[a];
    }
  if (int st = check_buf(ctx, l, n > 0 ? (uint64_t)l_ext * dtype_size(l_dt) : 0, "binary lhs")) return st;
  if (int st = check_buf(ctx, r, n > 0 ? (uint64_t)r_ext * dtype_size(r_dt) : 0, "binary rhs")) return st;
  if (int st = check_buf(ctx, out, (uint64_t)n * dtype_size(out_dt), "binary out")) return st;
  if (n == 0) return HIPNX_OK;

  bool any_float_in = is_float(l_dt) || is_float(r_dt);
  if (binary_int_only(op) && (any_float_in || is_float(out_dt)))
    return set_error(HIPNX_EINVAL, "binary: op %d needs integer operands", op);
  int cls = binary_class(op, l_dt, r_dt, out_dt);

  // collapse: drop unit axes, merge neighbours that stay contiguous (or broadcast) in both operands
  NdIndex ix;
  ix.rank = 0;
  int64_t dims[64], ls[64], rs[64];
  int m = 0;
  for (int a = 0; a < rank; a++) {
    if (out_dims[a] == 1) continue;
    int64_t d = out_dims[a], s1 = l_strides[a], s2 = r_strides[a];
    if (m > 0 && ls[m - 1] == s1 * d && rs[m - 1] == s2 * d) {
      dims[m - 1] *= d;
      ls[m - 1] = s1;
      rs[m - 1] = s2;
    } else {
      dims[m] = d; ls[m] = s1; rs[m] = s2;
      m++;
    }
  }
  if (m == 0) { dims[0] = 1; ls[0] = 0; rs[0] = 0; m = 1; }

  bool vec_ok = false;
  BinArgs a{};
  if (m == 3 || m == 4) {
    // two or three outer axes and a dense (or broadcast) inner one: the vector kernel with the row number taken apart
    const int64_t cols = dims[m - 1], l1 = ls[m - 1], r1 = rs[m - 1];
    int64_t rows = 1;
    bool aligned = cols % E == 0;
    for (int q = 0; q < m - 1; q++) {
      rows *= dims[q];
      aligned = aligned && (l1 == 0 || ls[q] % E == 0) && (r1 == 0 || rs[q] % E == 0);
    }
    if ((l1 == 0 || l1 == 1) && (r1 == 0 || r1 == 1) && !aligned && rows < (1ll << 31) && cols < (1ll << 31)) {
      // rows of several axes whose length (or an operand's row starts) is off the vector grid -- a mask
      // [b, 1, 1, 197] against scores [b, h, 197, 197] -- as vectors of the flat output
      vec_ok = true;
      a.l = l->ptr; a.r = r->ptr; a.out = out->ptr;
      a.ldt = l_dt; a.rdt = r_dt; a.odt = out_dt;
      a.cols = cols;
      a.vecs_per_row = 1; a.nvec = 1;  // (set by the launcher from flat_total)
      a.ls1 = (int)l1; a.rs1 = (int)r1;
      a.err = deferred_error_word(ctx);
      a.flat_total = n;
      a.ax.n = m - 1;
      bool l_dense = l1 == 1, r_dense = r1 == 1;
      int64_t run = cols;
      for (int q = m - 2; q >= 0; q--) {
        a.ax.d[q] = (uint32_t)dims[q];
        a.ax.fd[q] = make_fastdiv((uint32_t)dims[q]);
        a.ax.ls[q] = ls[q];
        a.ax.rs[q] = rs[q];
        l_dense = l_dense && ls[q] == run;
        r_dense = r_dense && rs[q] == run;
        run *= dims[q];
      }
      a.ls0 = l_dense ? cols : 0;
      a.rs0 = r_dense ? cols : 0;
    } else if ((l1 == 0 || l1 == 1) && (r1 == 0 || r1 == 1) && aligned && rows * ((cols + 3) / 4) < (1ll << 31)) {
      vec_ok = true;
      a.l = l->ptr; a.r = r->ptr; a.out = out->ptr;
      a.ldt = l_dt; a.rdt = r_dt; a.odt = out_dt;
      a.cols = cols;
      a.vecs_per_row = (cols + E - 1) / E;
      a.nvec = rows * a.vecs_per_row;
      a.ls0 = 0; a.rs0 = 0; a.ls1 = (int)l1; a.rs1 = (int)r1;
      a.err = deferred_error_word(ctx);
      a.ax.n = m - 1;
      for (int q = 0; q < m - 1; q++) {
        a.ax.d[q] = (uint32_t)dims[q];
        a.ax.fd[q] = make_fastdiv((uint32_t)dims[q]);
        a.ax.ls[q] = ls[q];
        a.ax.rs[q] = rs[q];
      }
    }
  }
  if (m <= 2) {
    int64_t rows = m == 2 ? dims[0] : 1, cols = dims[m - 1];
    int64_t l0 = m == 2 ? ls[0] : 0, r0 = m == 2 ? rs[0] : 0, l1 = ls[m - 1], r1 = rs[m - 1];
    bool aligned = rows == 1 || (cols % E == 0 && l0 % E == 0 && r0 % E == 0) ||
                   (cols % E == 0 && (l1 == 0 || l0 % E == 0) && (r1 == 0 || r0 % E == 0));
    if ((l1 == 0 || l1 == 1) && (r1 == 0 || r1 == 1) && aligned) {
      vec_ok = true;
      a.l = l->ptr; a.r = r->ptr; a.out = out->ptr;
      a.ldt = l_dt; a.rdt = r_dt; a.odt = out_dt;
      a.cols = cols;
      a.vecs_per_row = (cols + E - 1) / E;
      a.nvec = rows * a.vecs_per_row;
      a.ls0 = l0; a.rs0 = r0; a.ls1 = (int)l1; a.rs1 = (int)r1;
      a.err = deferred_error_word(ctx);
    } else if (m == 2 && (l1 == 0 || l1 == 1) && (r1 == 0 || r1 == 1) && cols < (1ll << 31)) {
      // rows that are not whole vectors: vectors of the flat output
      vec_ok = true;
      a.l = l->ptr; a.r = r->ptr; a.out = out->ptr;
      a.ldt = l_dt; a.rdt = r_dt; a.odt = out_dt;
      a.cols = cols;
      a.vecs_per_row = 1; a.nvec = 1;  // (set by the launcher from flat_total)
      a.ls0 = l0; a.rs0 = r0; a.ls1 = (int)l1; a.rs1 = (int)r1;
      a.err = deferred_error_word(ctx);
      a.flat_total = n;
    }
  }
  if (vec_ok) {
    a.stream = streams_past_cache(n, out_dt, l_dt, r_dt);
    int st = launch_bvec_op(std::make_integer_sequence<int, HIPNX_NBINARY>{}, ctx, op, cls, a);
    if (st) return st;
  } else {
    if (m > MAXR) return set_error(HIPNX_EUNSUPPORTED, "binary: more than %d non-collapsible axes", MAXR);
    if (binary_float_only(op) && cls >= CLS_I64) return set_error(HIPNX_EINVAL, "binary: op %d yields a float", op);
    ix.rank = m;
    for (int q = 0; q < m; q++) { ix.dims[q] = dims[q]; ix.ls[q] = ls[q]; ix.rs[q] = rs[q]; }
    dim3 grid(grid_for(ctx, n)), block(BLOCK);
    switch (cls) {
      case CLS_F32:
        hipLaunchKernelGGL((binary_nd_kernel<float, false>), grid, block, 0, ctx->stream, l->ptr, r->ptr, out->ptr, op,
                           l_dt, r_dt, out_dt, n, ix, deferred_error_word(ctx));
        break;
      case CLS_F64:
        hipLaunchKernelGGL((binary_nd_kernel<double, false>), grid, block, 0, ctx->stream, l->ptr, r->ptr, out->ptr, op,
                           l_dt, r_dt, out_dt, n, ix, deferred_error_word(ctx));
        break;
      case CLS_I64:
        hipLaunchKernelGGL((binary_nd_kernel<int64_t, false>), grid, block, 0, ctx->stream, l->ptr, r->ptr, out->ptr,
                           op, l_dt, r_dt, out_dt, n, ix, deferred_error_word(ctx));
        break;
      default:
        hipLaunchKernelGGL((binary_nd_kernel<int64_t, true>), grid, block, 0, ctx->stream, l->ptr, r->ptr, out->ptr, op,
                           l_dt, r_dt, out_dt, n, ix, deferred_error_word(ctx));
        break;
    }
  }
  HIPNX_HIP(hipGetLastError());
  return HIPNX_OK;
}

namespace hipnx {

template <int OP, typename CT, int FIX>
static void launch_uvec_fix(const hipnx_ctx *ctx, const void *in, void *out, int idt, int odt, int bits, int64_t n) {
  const dim3 grid(grid_for(ctx, (n + vec_elems(FIX, FIX) - 1) / vec_elems(FIX, FIX)));
  if (FIX >= 0 && streams_past_cache(n, idt, odt))
    hipLaunchKernelGGL((unary_vec_kernel<OP, CT, FIX, (FIX >= 0)>), grid, dim3(BLOCK), 0, ctx->stream, in, out, idt, odt, bits, n);
  else
    hipLaunchKernelGGL((unary_vec_kernel<OP, CT, FIX>), grid, dim3(BLOCK), 0, ctx->stream, in, out, idt, odt, bits, n);
}

template <int OP, typename CT>
static void launch_uvec(const hipnx_ctx *ctx, const void *in, void *out, int idt, int odt, int bits, int64_t n) {
  if (idt == odt) {
    if constexpr (std::is_same<CT, float>::value) {
      if (odt == HIPNX_F32) return launch_uvec_fix<OP, CT, HIPNX_F32>(ctx, in, out, idt, odt, bits, n);
      if (odt == HIPNX_BF16) return launch_uvec_fix<OP, CT, HIPNX_BF16>(ctx, in, out, idt, odt, bits, n);
      if (odt == HIPNX_F16) return launch_uvec_fix<OP, CT, HIPNX_F16>(ctx, in, out, idt, odt, bits, n);
    } else if constexpr (std::is_same<CT, double>::value) {
      if (odt == HIPNX_F64) return launch_uvec_fix<OP, CT, HIPNX_F64>(ctx, in, out, idt, odt, bits, n);
    } else {
      if (odt == HIPNX_S32) return launch_uvec_fix<OP, CT, HIPNX_S32>(ctx, in, out, idt, odt, bits, n);
      if (odt == HIPNX_S64) return launch_uvec_fix<OP, CT, HIPNX_S64>(ctx, in, out, idt, odt, bits, n);
    }
  }
  launch_uvec_fix<OP, CT, -1>(ctx, in, out, idt, odt, bits, n);
}

template <int OP>
static int launch_uvec_cls(const hipnx_ctx *ctx, int cls, const void *in, void *out, int idt, int odt, int bits,
                           int64_t n) {
  if constexpr (!unary_int_only(OP)) {
    if (cls == CLS_F32) { launch_uvec<OP, float>(ctx, in, out, idt, odt, bits, n); return HIPNX_OK; }
    if (cls == CLS_F64) { launch_uvec<OP, double>(ctx, in, out, idt, odt, bits, n); return HIPNX_OK; }
  }
  if constexpr (!unary_is_math(OP)) {
    if (cls >= CLS_I64) { launch_uvec<OP, int64_t>(ctx, in, out, idt, odt, bits, n); return HIPNX_OK; }
  }
  return set_error(HIPNX_EINVAL, "unary op %d is not defined for this operand type", OP);
}

template <int... OPS>
static int launch_uvec_op(std::integer_sequence<int, OPS...>, const hipnx_ctx *ctx, int op, int cls, const void *in,
                          void *out, int idt, int odt, int bits, int64_t n) {
  int st = HIPNX_EINVAL;
  (void)((op == OPS ? (st = launch_uvec_cls<OPS>(ctx, cls, in, out, idt, odt, bits, n), true) : false) || ...);
  return st;
}

}  // namespace hipnx

extern "C" int hipnx_unary(hipnx_ctx *ctx, int op, int in_dt, int out_dt, int64_t n, const hipnx_buf *inb,
                           hipnx_buf *out) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (op < 0 || op >= HIPNX_NUNARY) return set_error(HIPNX_EINVAL, "unary: unknown op %d", op);
  if (dtype_size(in_dt) < 0 || dtype_size(out_dt) < 0 || n < 0)
    return set_error(HIPNX_EINVAL, "unary: unknown element type or negative size");
  if (int st = check_buf(ctx, inb, (uint64_t)n * dtype_size(in_dt), "unary in")) return st;
  if (int st = check_buf(ctx, out, (uint64_t)n * dtype_size(out_dt), "unary out")) return st;
  if (n == 0) return HIPNX_OK;
  int cls;
  if (is_float(in_dt) || is_float(out_dt)) cls = (is_wide(in_dt) || out_dt == HIPNX_F64) ? CLS_F64 : CLS_F32;
  else cls = CLS_I64;
  if (unary_int_only(op) && cls < CLS_I64) return set_error(HIPNX_EINVAL, "unary: op %d needs an integer operand", op);
  int st = launch_uvec_op(std::make_integer_sequence<int, HIPNX_NUNARY>{}, ctx, op, cls, inb->ptr, out->ptr, in_dt,
                          out_dt, 8 * dtype_size(in_dt), n);
  if (st) return st;
  HIPNX_HIP(hipGetLastError());
  return HIPNX_OK;
}

extern "C" int hipnx_as_type(hipnx_ctx *ctx, int in_dt, int out_dt, int64_t n, const hipnx_buf *inb,
                             hipnx_buf *out) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (dtype_size(in_dt) < 0 || out_dtype_size(out_dt) < 0 || n < 0)
    return set_error(HIPNX_EINVAL, "as_type: unknown element type or negative size");
  if (int st = check_buf(ctx, inb, (uint64_t)n * dtype_size(in_dt), "as_type in")) return st;
  if (int st = check_buf(ctx, out, (uint64_t)n * out_dtype_size(out_dt), "as_type out")) return st;
  if (n == 0) return HIPNX_OK;
  static const int64_t tmax[8] = {0xFF, 0xFFFF, 0xFFFFFFFFll, -1ll /* u64 max */, 0x7F, 0x7FFF, 0x7FFFFFFFll,
                                  0x7FFFFFFFFFFFFFFFll};
  static const int64_t tmin[8] = {0, 0, 0, 0, -0x80, -0x8000, -0x80000000ll, (int64_t)0x8000000000000000ull};
  int64_t mx = out_dt < HIPNX_F16 ? tmax[out_dt] : 0, mn = out_dt < HIPNX_F16 ? tmin[out_dt] : 0;
  dim3 grid(grid_for(ctx, (n + E - 1) / E)), block(BLOCK);
#define HIPNX_AS(CT, I, O)                                                                                                        \
  do {                                                                                                                            \
    const dim3 g(grid_for(ctx, (n + vec_elems(I, O) - 1) / vec_elems(I, O)));                                                      \
    if (I >= 0 && streams_past_cache(n, in_dt, out_dt))                                                                           \
      hipLaunchKernelGGL((as_type_kernel<CT, I, O, (I >= 0)>), g, block, 0, ctx->stream, inb->ptr, out->ptr, in_dt, out_dt, n, mx, mn); \
    else                                                                                                                          \
      hipLaunchKernelGGL((as_type_kernel<CT, I, O>), g, block, 0, ctx->stream, inb->ptr, out->ptr, in_dt, out_dt, n, mx, mn);      \
  } while (0)
  // the conversions of mixed-precision work, compiled for their two types
  if (in_dt == HIPNX_F32 && out_dt == HIPNX_BF16) HIPNX_AS(float, HIPNX_F32, HIPNX_BF16);
  else if (in_dt == HIPNX_BF16 && out_dt == HIPNX_F32) HIPNX_AS(float, HIPNX_BF16, HIPNX_F32);
  else if (in_dt == HIPNX_F32 && out_dt == HIPNX_BF16_RNE) HIPNX_AS(float, HIPNX_F32, HIPNX_BF16_RNE);
  else if (in_dt == HIPNX_F16 && out_dt == HIPNX_F32) HIPNX_AS(float, HIPNX_F16, HIPNX_F32);
  else if (in_dt == HIPNX_F32 && out_dt == HIPNX_F16) HIPNX_AS(double, HIPNX_F32, HIPNX_F16);
  else if (in_dt == HIPNX_S32 && out_dt == HIPNX_F32) HIPNX_AS(double, HIPNX_S32, HIPNX_F32);
  else if (in_dt == HIPNX_U8 && out_dt == HIPNX_F32) HIPNX_AS(double, HIPNX_U8, HIPNX_F32);
  else if (in_dt == HIPNX_F32 && out_dt == HIPNX_F64) HIPNX_AS(double, HIPNX_F32, HIPNX_F64);
  else if (in_dt == HIPNX_F64 && out_dt == HIPNX_F32) HIPNX_AS(double, HIPNX_F64, HIPNX_F32);
  else if (!is_float(in_dt) && !is_float(out_dt))  // integer -> integer: keep the low bits
    HIPNX_AS(int64_t, -1, -1);
  else if (!is_float(in_dt) || in_dt == HIPNX_F64 || out_dt == HIPNX_F64 || out_dt == HIPNX_F16)
    // integer -> float decodes to f64 (exact below 2^53, u64 read as unsigned), then one rounding
    HIPNX_AS(double, -1, -1);
  else
    HIPNX_AS(float, -1, -1);
#undef HIPNX_AS
  HIPNX_HIP(hipGetLastError());
  return HIPNX_OK;
}
