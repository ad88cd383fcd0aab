// Callbacks one step off the hot path, native so that chains stay on the device:
// select, clip, slice / concatenate / stack (one strided copy), iota, eye.
// Reference semantics: nx/lib/nx/binary_backend.ex:49-112 (iota, eye), 604-648 (select),
// 1788-1811 (clip), 1813-1863 (slice), 1962-2030 (stack, concatenate).
#include <cstring>

#include "dtypes.cuh"
#include "internal.h"

namespace hipnx {

constexpr int BLOCK = 256;
constexpr int MAXR = 8;
constexpr int E = 8;  // elements per lane per step of the vector kernels

static bool narrow_float(int dt) { return dt == HIPNX_BF16 || dt == HIPNX_F16 || dt == HIPNX_F32; }

// elements per lane of the select kernel compiled for one element type: 16 bytes of a 4-byte type, else 8
constexpr int select_elems(int fix) { return fix == HIPNX_F32 || fix == HIPNX_S32 || fix == HIPNX_U32 ? 4 : 8; }

static int grid_for(int64_t items) {
  int64_t blocks = (items + BLOCK - 1) / BLOCK;
  if (blocks < 1) blocks = 1;
  const int64_t cap = ((1ll << 32) - 1) / BLOCK;  // a launch may hold at most 2^32 - 1 lanes: the kernels loop over the rest
  return (int)(blocks < cap ? blocks : cap);
}

// ---- select ---------------------------------------------------------------------------------
// out[i] = pred[i] != 0 ? on_true[i] : on_false[i], each operand broadcast by strides (0 = repeat).
// CT: double when the output is a float type, int64 otherwise (both value operands are integers
// then; u64 travels as its bit pattern and the store keeps the low bits).
struct Sel {
  int rank;
  int64_t dims[MAXR], ps[MAXR], ts[MAXR], fs[MAXR];
};

template <typename CT>
__device__ __forceinline__ bool truthy(const void *p, int dt, int64_t i) {
  if (dt >= HIPNX_F16) {
    const double v = load_one<double>(p, dt, i);
    return v != 0;  // NaN is true, as in the reference (as_boolean: everything but 0)
  }
  return load_one<int64_t>(p, dt, i) != 0;
}

template <typename CT>
__global__ void __launch_bounds__(BLOCK)
select_nd_kernel(const void *__restrict__ p, const void *__restrict__ t, const void *__restrict__ f, void *__restrict__ out,
                 int pdt, int tdt, int fdt, int odt, int64_t n, Sel s) {
  for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < n; i += (int64_t)gridDim.x * BLOCK) {
    int64_t rem = i, po = 0, to = 0, fo = 0;
    for (int a = s.rank - 1; a >= 0; a--) {
      const int64_t q = rem / s.dims[a], c = rem - q * s.dims[a];
      po += c * s.ps[a]; to += c * s.ts[a]; fo += c * s.fs[a];
      rem = q;
    }
    const CT v = truthy<CT>(p, pdt, po) ? load_one<CT>(t, tdt, to) : load_one<CT>(f, fdt, fo);
    store_one<CT>(out, odt, i, v);
  }
}

// all three operands dense (step 1) or a single element (step 0).  FIX >= 0: a u8 predicate and this
// element type for both values and the result, known when the kernel is compiled (the run-time type
// switches of the vector loads and the store fold away).
template <typename CT, int FIX = -1, bool NT = false>
__global__ void __launch_bounds__(BLOCK)
select_vec_kernel(const void *__restrict__ p, const void *__restrict__ t, const void *__restrict__ f, void *__restrict__ out,
                  int pdt_, int tdt_, int fdt_, int odt_, int64_t n, int pstep, int tstep, int fstep) {
  constexpr int E = select_elems(FIX);
  const int pdt = FIX >= 0 ? HIPNX_U8 : pdt_, tdt = FIX >= 0 ? FIX : tdt_, fdt = FIX >= 0 ? FIX : fdt_, odt = FIX >= 0 ? FIX : odt_;
  const int64_t nvec = (n + E - 1) / E;
  for (int64_t v = (int64_t)blockIdx.x * BLOCK + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * BLOCK) {
    const int64_t i0 = v * E;
    if (i0 + E <= n) {
      CT a[E], b[E], c[E];
      bool pt[E];
      if (!pstep) {
        const bool one = truthy<CT>(p, pdt, 0);
#pragma unroll
        for (int e = 0; e < E; e++) pt[e] = one;
      } else if (pdt == HIPNX_U8 || pdt == HIPNX_S8) {  // what comparisons and logical ops produce
        if constexpr (E == 8) {
          const uint2 w = *reinterpret_cast<const uint2 *>(static_cast<const unsigned char *>(p) + i0);
#pragma unroll
          for (int e = 0; e < E; e++) pt[e] = (((e < 4 ? w.x : w.y) >> (8 * (e & 3))) & 0xFF) != 0;
        } else {
          const uint32_t w = *reinterpret_cast<const uint32_t *>(static_cast<const unsigned char *>(p) + i0);
#pragma unroll
          for (int e = 0; e < E; e++) pt[e] = ((w >> (8 * e)) & 0xFF) != 0;
        }
      } else if (pdt >= HIPNX_F16) {
        double pd[E];
        load_vec<double, E>(p, pdt, i0, pd);
#pragma unroll
        for (int e = 0; e < E; e++) pt[e] = pd[e] != 0;
      } else {
        int64_t pi[E];
        load_vec<int64_t, E>(p, pdt, i0, pi);
#pragma unroll
        for (int e = 0; e < E; e++) pt[e] = pi[e] != 0;
      }
      // (an operand that is one element for all -- a number -- keeps its own type also in the typed form)
      if (tstep) load_vec<CT, E, true, NT>(t, tdt, i0, a);
      else { const CT x = load_one<CT>(t, tdt_, 0);
#pragma unroll
        for (int e = 0; e < E; e++) a[e] = x; }
      if (fstep) load_vec<CT, E, true, NT>(f, fdt, i0, b);
      else { const CT x = load_one<CT>(f, fdt_, 0);
#pragma unroll
        for (int e = 0; e < E; e++) b[e] = x; }
#pragma unroll
      for (int e = 0; e < E; e++) c[e] = pt[e] ? a[e] : b[e];
      store_vec<CT, E, NT>(out, odt, i0, c);
    } else {
      for (int64_t i = i0; i < n; i++) {
        const CT x = truthy<CT>(p, pdt, i * pstep) ? load_one<CT>(t, tstep ? tdt : tdt_, i * tstep) : load_one<CT>(f, fstep ? fdt : fdt_, i * fstep);
        store_one<CT>(out, odt, i, x);
      }
    }
  }
}

// ---- clip -----------------------------------------------------------------------------------
// c = x > min ? x : min;  out = c < max ? c : max  (so a NaN element becomes min, a NaN bound wins
// the way the reference's comparisons make it: binary_backend.ex:1794-1806)
// Integers are compared as the unbounded numbers the reference decodes them to: a value is the
// 64 bits plus whether they came from a u64 (then a set top bit means 2^63 or more, above every
// signed value).
struct Wide {
  int64_t bits;
  bool uns;
};
__device__ inline bool wide_gt(Wide a, Wide b) {
  const bool a_huge = a.uns && a.bits < 0, b_huge = b.uns && b.bits < 0;
  if (a_huge || b_huge) return a_huge && (!b_huge || (uint64_t)a.bits > (uint64_t)b.bits);
  return a.bits > b.bits;
}
template <typename CT>
__device__ inline CT clip_one(CT x, CT lo, CT hi, bool xu, bool lou, bool hiu) {
  if constexpr (std::is_same<CT, int64_t>::value) {
    const Wide X{x, xu}, LO{lo, lou}, HI{hi, hiu};
    const Wide c = wide_gt(X, LO) ? X : LO;
    return wide_gt(HI, c) ? c.bits : HI.bits;
  } else {
    const CT c = x > lo ? x : lo;  // element_greater(x, min) == 1 ? x : min   (NaN compares false)
    return c < hi ? c : hi;        // element_less(clipped, max) == 1 ? clipped : max
  }
}

// elements per lane where the element type is known at compile time: 16 bytes of a 4-byte type (one access per lane,
// lanes side by side: a wave instruction covers whole lines), else the 8 of the general form
constexpr int fixed_elems(int fix) { return fix == HIPNX_F32 || fix == HIPNX_S32 || fix == HIPNX_U32 ? 4 : 8; }

// FIX >= 0: the element type of input and result, known at compile time; NT: tensors far larger than the last-level
// cache, every access with the non-temporal hint
template <typename CT, int FIX = -1, bool NT = false>
__global__ void __launch_bounds__(BLOCK)
clip_kernel(const void *__restrict__ in, const void *__restrict__ mn, const void *__restrict__ mx, void *__restrict__ out,
            int idt_, int mndt, int mxdt, int odt_, int64_t n) {
  constexpr int E = fixed_elems(FIX);
  const int idt = FIX >= 0 ? FIX : idt_, odt = FIX >= 0 ? FIX : odt_;
  // (bounds of the tensor's own type, the usual case, are two scalar loads issued together; decoding a bound of any
  // type is a chain of branches and waits that every wave would walk before it asks for its data)
  CT lo, hi;
  if (FIX >= 0 && mndt == FIX && mxdt == FIX) {
    lo = load_one<CT>(mn, FIX, 0);
    hi = load_one<CT>(mx, FIX, 0);
  } else {
    lo = load_one<CT>(mn, mndt, 0);
    hi = load_one<CT>(mx, mxdt, 0);
  }
  const bool xu = idt == HIPNX_U64, lou = mndt == HIPNX_U64, hiu = mxdt == HIPNX_U64;
  const int64_t nvec = (n + E - 1) / E;
  for (int64_t v = (int64_t)blockIdx.x * BLOCK + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * BLOCK) {
    const int64_t i0 = v * E;
    if (i0 + E <= n) {
      CT x[E];
      load_vec<CT, E, true, NT>(in, idt, i0, x);
#pragma unroll
      for (int e = 0; e < E; e++) x[e] = clip_one<CT>(x[e], lo, hi, xu, lou, hiu);
      store_vec<CT, E, NT>(out, odt, i0, x);
    } else {
      for (int64_t i = i0; i < n; i++) store_one<CT>(out, odt, i, clip_one<CT>(load_one<CT>(in, idt, i), lo, hi, xu, lou, hiu));
    }
  }
}

// ---- strided copy: out[out_off + sum c_a * os_a] = in[in_off + sum c_a * is_a] -------------
struct Copy {
  int rank;
  int64_t dims[MAXR], is[MAXR], os[MAXR];
};

template <typename T>
__global__ void __launch_bounds__(BLOCK)
copy_nd_kernel(const T *__restrict__ in, T *__restrict__ out, int64_t n, Copy c) {
  for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < n; i += (int64_t)gridDim.x * BLOCK) {
    int64_t rem = i, io = 0, oo = 0;
    for (int a = c.rank - 1; a >= 0; a--) {
      const int64_t q = rem / c.dims[a], k = rem - q * c.dims[a];
      io += k * c.is[a]; oo += k * c.os[a];
      rem = q;
    }
    out[oo] = in[io];
  }
}

// The innermost axis dense on the output side and dense or reversed on the input side, but not on 16-byte
// boundaries (a slice that starts at an odd column, a padded copy, a reverse): a lane still moves V = 16 /
// sizeof(T) elements at once -- the hardware takes 16-byte accesses at element alignment -- and only the last,
// partial vector of a row goes by element.  `c.dims[rank - 1]` counts vectors (the row's elements rounded up),
// `row_len` elements.  One element per lane is bound by instructions: 1.4 TB/s on a bf16 slice of 16384^2.
template <typename T>
struct __attribute__((packed, aligned(sizeof(T)))) run_vec {
  T e[16 / sizeof(T)];
};
template <typename T>
__global__ void __launch_bounds__(BLOCK)
copy_runs_kernel(const T *__restrict__ in, T *__restrict__ out, int64_t nvec, Copy c, int64_t row_len, int reversed) {
  constexpr int V = 16 / sizeof(T);
  for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * BLOCK) {
    int64_t rem = i, io = 0, oo = 0, col = 0;
    for (int a = c.rank - 1; a >= 0; a--) {
      int64_t q, k;
      if (rem < (1ll << 31) && c.dims[a] < (1ll << 31)) { q = (uint32_t)rem / (uint32_t)c.dims[a]; k = (uint32_t)rem - (uint32_t)q * (uint32_t)c.dims[a]; }
      else { q = rem / c.dims[a]; k = rem - q * c.dims[a]; }
      if (a == c.rank - 1) col = k * V;
      else { io += k * c.is[a]; oo += k * c.os[a]; }
      rem = q;
    }
    const T *src = in + io + (reversed ? -col : col);
    T *dst = out + oo + col;
    if (col + V <= row_len) {
      run_vec<T> v;
      if (!reversed) v = *reinterpret_cast<const run_vec<T> *>(src);
      else {
        const run_vec<T> w = *reinterpret_cast<const run_vec<T> *>(src - (V - 1));
#pragma unroll
        for (int k = 0; k < V; k++) v.e[k] = w.e[V - 1 - k];
      }
      *reinterpret_cast<run_vec<T> *>(dst) = v;
    } else {
      for (int k = 0; col + k < row_len; k++) dst[k] = reversed ? src[-k] : src[k];
    }
  }
}

// ---- iota / eye -----------------------------------------------------------------------------
// mode 0: out[i] = (i / inner) % dim (iota along an axis; the flat iota is inner = 1, dim = n)
// mode 1: out[i] = 1 where (i / inner) % dim == i % inner  (eye: dim = rows, inner = columns)
// IT is the type the coordinates are counted in: 32-bit when the tensor has fewer than 2^31 elements
// (so the integer -> float conversion is one instruction and exact-or-nearest-even like the
// reference's integer written as a float, nx/lib/nx/binary_backend.ex:49-75), 64-bit otherwise.
// ODT >= 0: the result's element type, known when the kernel is compiled; EV elements per lane (4 for an
// 8-byte type: 32 bytes per lane -- with 8 each of a lane's four stores would land in a quarter of a line).
template <typename CT, typename IT, int ODT = -1, int EV = 8>
__global__ void __launch_bounds__(BLOCK)
iota_kernel(void *__restrict__ out, int odt_, int64_t n, int64_t dim_, int64_t inner_, int mode) {
  constexpr int E = EV;
  const int odt = ODT >= 0 ? ODT : odt_;
  const int64_t nvec = (n + E - 1) / E;
  const IT dim = (IT)dim_, inner = (IT)inner_;
  for (int64_t v = (int64_t)blockIdx.x * BLOCK + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * BLOCK) {
    const int64_t i0 = v * E;
    CT x[E];
    // one division per vector, then count along: c = i % inner, r = (i / inner) % dim
    IT q, c;
    if (sizeof(IT) == 4) { q = (IT)((uint32_t)i0 / (uint32_t)inner); c = (IT)((uint32_t)i0 - (uint32_t)q * (uint32_t)inner); }
    else { q = (IT)(i0 / inner); c = (IT)(i0 - q * inner); }
    IT r = q < dim ? q : q % dim;
#pragma unroll
    for (int e = 0; e < E; e++) {
      x[e] = mode == 0 ? (CT)r : (CT)(r == c ? 1 : 0);
      if (++c == inner) { c = 0; if (++r == dim) r = 0; }
    }
    if (i0 + E <= n) store_vec<CT, E>(out, odt, i0, x);
    else
      for (int e = 0; i0 + e < n; e++) store_one<CT>(out, odt, i0 + e, x[e]);
  }
}

// ---- sub-byte integers held one per byte: keep the low bits of each byte ------------------------
__global__ void __launch_bounds__(BLOCK)
narrow_int_kernel(unsigned char *__restrict__ p, int64_t n, int bits, int is_signed) {
  const int sh = 8 - bits;
  const int64_t nvec = n / 16;
  for (int64_t v = (int64_t)blockIdx.x * BLOCK + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * BLOCK) {
    raw_vec<16> r = *reinterpret_cast<raw_vec<16> *>(p + v * 16);
#pragma unroll
    for (int i = 0; i < 16; i++)
      r.b[i] = is_signed ? (unsigned char)((signed char)(r.b[i] << sh) >> sh) : (unsigned char)(r.b[i] & (0xFF >> sh));
    *reinterpret_cast<raw_vec<16> *>(p + v * 16) = r;
  }
  if (blockIdx.x == 0 && threadIdx.x < n - nvec * 16) {
    const int64_t i = nvec * 16 + threadIdx.x;
    p[i] = is_signed ? (unsigned char)((signed char)(p[i] << sh) >> sh) : (unsigned char)(p[i] & (0xFF >> sh));
  }
}

}  // namespace hipnx

using namespace hipnx;

extern "C" int hipnx_narrow_int(hipnx_ctx *ctx, hipnx_buf *buf, int64_t n, int bits, int is_signed) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (bits != 2 && bits != 4) return set_error(HIPNX_EINVAL, "narrow_int: %d bits (2 or 4)", bits);
  if (n < 0) return set_error(HIPNX_EINVAL, "narrow_int: negative size");
  if (int st = check_buf(ctx, buf, (uint64_t)n, "narrow_int")) return st;
  if (n == 0) return HIPNX_OK;
  if ((uintptr_t)buf->ptr % 16) return set_error(HIPNX_EINVAL, "narrow_int: buffer not 16-byte aligned");
  hipLaunchKernelGGL(narrow_int_kernel, dim3(grid_for(n / 16 + 1)), dim3(BLOCK), 0, ctx->stream,
                     (unsigned char *)buf->ptr, n, bits, is_signed);
  HIPNX_HIP(hipGetLastError());
  return HIPNX_OK;
}

extern "C" int hipnx_select(hipnx_ctx *ctx, int pred_dt, int true_dt, int false_dt, int out_dt, int rank,
                            const int64_t *out_dims, const int64_t *pred_strides, const int64_t *true_strides,
                            const int64_t *false_strides, const hipnx_buf *pred, const hipnx_buf *on_true,
                            const hipnx_buf *on_false, hipnx_buf *out) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (dtype_size(pred_dt) < 0 || dtype_size(true_dt) < 0 || dtype_size(false_dt) < 0 || dtype_size(out_dt) < 0)
    return set_error(HIPNX_EINVAL, "select: unknown element type");
  if (rank < 0 || rank > 64 || (rank > 0 && (!out_dims || !pred_strides || !true_strides || !false_strides)))
    return set_error(HIPNX_EINVAL, "select: bad rank");
  if (!is_float(out_dt) && (is_float(true_dt) || is_float(false_dt)))
    return set_error(HIPNX_EINVAL, "select: float operands with an integer output");
  int64_t n = 1, pe = 1, te = 1, fe = 1;
  for (int a = 0; a < rank; a++) {
    if (out_dims[a] < 0 || pred_strides[a] < 0 || true_strides[a] < 0 || false_strides[a] < 0)
      return set_error(HIPNX_EINVAL, "select: negative dimension or stride");
    n *= out_dims[a];
  }
  if (n > 0)
    for (int a = 0; a < rank; a++) {
      pe += (out_dims[a] - 1) * pred_strides[a]; te += (out_dims[a] - 1) * true_strides[a]; fe += (out_dims[a] - 1) * false_strides[a];
    }
  if (int st = check_buf(ctx, pred, n > 0 ? (uint64_t)pe * dtype_size(pred_dt) : 0, "select pred")) return st;
  if (int st = check_buf(ctx, on_true, n > 0 ? (uint64_t)te * dtype_size(true_dt) : 0, "select on_true")) return st;
  if (int st = check_buf(ctx, on_false, n > 0 ? (uint64_t)fe * dtype_size(false_dt) : 0, "select on_false")) return st;
  if (int st = check_buf(ctx, out, (uint64_t)n * dtype_size(out_dt), "select out")) return st;
  if (n == 0) return HIPNX_OK;
  // collapse: drop extent-1 axes, merge neighbours that are contiguous for all three operands
  Sel s;
  int m = 0;
  for (int a = 0; a < rank; a++) {
    const int64_t d = out_dims[a];
    if (d == 1) continue;
    if (m > 0 && s.ps[m - 1] == pred_strides[a] * d && s.ts[m - 1] == true_strides[a] * d && s.fs[m - 1] == false_strides[a] * d) {
      s.dims[m - 1] *= d; s.ps[m - 1] = pred_strides[a]; s.ts[m - 1] = true_strides[a]; s.fs[m - 1] = false_strides[a];
    } else {
      if (m == MAXR) return set_error(HIPNX_EUNSUPPORTED, "select: more than %d non-collapsible axes", MAXR);
      s.dims[m] = d; s.ps[m] = pred_strides[a]; s.ts[m] = true_strides[a]; s.fs[m] = false_strides[a]; m++;
    }
  }
  if (m == 0) { s.dims[0] = 1; s.ps[0] = s.ts[0] = s.fs[0] = 0; m = 1; }
  s.rank = m;
  const bool fl = is_float(out_dt);
  // values only pass through: f32 arithmetic holds every bf16 / f16 / f32 exactly
  const bool narrow = narrow_float(true_dt) && narrow_float(false_dt) && narrow_float(out_dt);
  if (m == 1 && s.ps[0] <= 1 && s.ts[0] <= 1 && s.fs[0] <= 1) {
    const dim3 block(BLOCK);
    const bool past_cache = n * (int64_t)dtype_size(out_dt) >= (256ll << 20);
#define HIPNX_SELECT(CT, FIX)                                                                                                       \
  do {                                                                                                                              \
    const dim3 grid(grid_for((n + select_elems(FIX) - 1) / select_elems(FIX)));                                                      \
    if (FIX >= 0 && past_cache)                                                                                                     \
      hipLaunchKernelGGL((select_vec_kernel<CT, FIX, (FIX >= 0)>), grid, block, 0, ctx->stream, pred->ptr, on_true->ptr, on_false->ptr, out->ptr, \
                         pred_dt, true_dt, false_dt, out_dt, n, (int)s.ps[0], (int)s.ts[0], (int)s.fs[0]);                          \
    else                                                                                                                            \
      hipLaunchKernelGGL((select_vec_kernel<CT, FIX>), grid, block, 0, ctx->stream, pred->ptr, on_true->ptr, on_false->ptr, out->ptr, \
                         pred_dt, true_dt, false_dt, out_dt, n, (int)s.ps[0], (int)s.ts[0], (int)s.fs[0]);                          \
  } while (0)
    // one element type throughout, where a lone element (a number) may have another one that the kernel's
    // arithmetic type holds exactly: select(mask, scores_bf16, -1.0e9) arrives with an f32 number
    auto fits = [&](int dt, int64_t step) {
      if (dt == out_dt) return true;
      if (step != 0) return false;
      return is_float(out_dt) ? narrow_float(dt) && narrow_float(out_dt) : !is_float(dt);
    };
    const bool one_type = pred_dt == HIPNX_U8 && fits(true_dt, s.ts[0]) && fits(false_dt, s.fs[0]) && (s.ts[0] != 0 || s.fs[0] != 0 || true_dt == false_dt);
    if (one_type && out_dt == HIPNX_F32) HIPNX_SELECT(float, HIPNX_F32);
    else if (one_type && out_dt == HIPNX_BF16) HIPNX_SELECT(float, HIPNX_BF16);
    else if (one_type && out_dt == HIPNX_F16) HIPNX_SELECT(float, HIPNX_F16);
    else if (one_type && out_dt == HIPNX_S32) HIPNX_SELECT(int64_t, HIPNX_S32);
    else if (one_type && out_dt == HIPNX_S64) HIPNX_SELECT(int64_t, HIPNX_S64);
    else if (narrow) HIPNX_SELECT(float, -1);
    else if (fl) HIPNX_SELECT(double, -1);
    else HIPNX_SELECT(int64_t, -1);
#undef HIPNX_SELECT
  } else {
    dim3 grid(grid_for(n)), block(BLOCK);
    if (fl) hipLaunchKernelGGL((select_nd_kernel<double>), grid, block, 0, ctx->stream, pred->ptr, on_true->ptr, on_false->ptr, out->ptr,
                               pred_dt, true_dt, false_dt, out_dt, n, s);
    else hipLaunchKernelGGL((select_nd_kernel<int64_t>), grid, block, 0, ctx->stream, pred->ptr, on_true->ptr, on_false->ptr, out->ptr,
                            pred_dt, true_dt, false_dt, out_dt, n, s);
  }
  HIPNX_HIP(hipGetLastError());
  return HIPNX_OK;
}

extern "C" int hipnx_clip(hipnx_ctx *ctx, int in_dt, int min_dt, int max_dt, int out_dt, int64_t n,
                          const hipnx_buf *inb, const hipnx_buf *min, const hipnx_buf *max, hipnx_buf *out) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (dtype_size(in_dt) < 0 || dtype_size(min_dt) < 0 || dtype_size(max_dt) < 0 || dtype_size(out_dt) < 0)
    return set_error(HIPNX_EINVAL, "clip: unknown element type");
  if (n < 0) return set_error(HIPNX_EINVAL, "clip: negative size");
  if (!is_float(out_dt) && (is_float(in_dt) || is_float(min_dt) || is_float(max_dt)))
    return set_error(HIPNX_EINVAL, "clip: float operands with an integer output");
  if (int st = check_buf(ctx, inb, (uint64_t)n * dtype_size(in_dt), "clip in")) return st;
  if (int st = check_buf(ctx, min, dtype_size(min_dt), "clip min")) return st;
  if (int st = check_buf(ctx, max, dtype_size(max_dt), "clip max")) return st;
  if (int st = check_buf(ctx, out, (uint64_t)n * dtype_size(out_dt), "clip out")) return st;
  if (n == 0) return HIPNX_OK;
  const dim3 block(BLOCK);
  const bool past_cache = n * (int64_t)dtype_size(out_dt) >= (256ll << 20);
#define HIPNX_CLIP(CT, FIX)                                                                                                        \
  do {                                                                                                                             \
    const dim3 grid(grid_for((n + fixed_elems(FIX) - 1) / fixed_elems(FIX)));                                                       \
    if (FIX >= 0 && past_cache)                                                                                                    \
      hipLaunchKernelGGL((clip_kernel<CT, FIX, (FIX >= 0)>), grid, block, 0, ctx->stream, inb->ptr, min->ptr, max->ptr, out->ptr, in_dt, min_dt, max_dt, out_dt, n); \
    else                                                                                                                           \
      hipLaunchKernelGGL((clip_kernel<CT, FIX>), grid, block, 0, ctx->stream, inb->ptr, min->ptr, max->ptr, out->ptr, in_dt, min_dt, max_dt, out_dt, n); \
  } while (0)
  if (narrow_float(in_dt) && narrow_float(min_dt) && narrow_float(max_dt) && narrow_float(out_dt)) {
    if (in_dt == out_dt && out_dt == HIPNX_F32) HIPNX_CLIP(float, HIPNX_F32);
    else if (in_dt == out_dt && out_dt == HIPNX_BF16) HIPNX_CLIP(float, HIPNX_BF16);
    else if (in_dt == out_dt && out_dt == HIPNX_F16) HIPNX_CLIP(float, HIPNX_F16);
    else HIPNX_CLIP(float, -1);
  } else if (is_float(out_dt)) HIPNX_CLIP(double, -1);
  else if (in_dt == out_dt && out_dt == HIPNX_S32) HIPNX_CLIP(int64_t, HIPNX_S32);
  else HIPNX_CLIP(int64_t, -1);
#undef HIPNX_CLIP
  HIPNX_HIP(hipGetLastError());
  return HIPNX_OK;
}

namespace {
template <typename T>
void launch_copy(const hipnx_ctx *ctx, const void *in, void *out, int64_t n, const Copy &c) {
  hipLaunchKernelGGL((copy_nd_kernel<T>), dim3(grid_for(n)), dim3(BLOCK), 0, ctx->stream, (const T *)in, (T *)out, n, c);
}
}  // namespace

extern "C" int hipnx_strided_copy(hipnx_ctx *ctx, int elem_bytes, int rank, const int64_t *dims,
                                  const int64_t *in_strides, int64_t in_offset, const int64_t *out_strides,
                                  int64_t out_offset, const hipnx_buf *inb, hipnx_buf *out) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8)
    return set_error(HIPNX_EINVAL, "strided_copy: element size %d is not 1, 2, 4 or 8", elem_bytes);
  if (rank < 0 || rank > 64 || (rank > 0 && (!dims || !in_strides || !out_strides))) return set_error(HIPNX_EINVAL, "strided_copy: bad rank");
  if (in_offset < 0 || out_offset < 0) return set_error(HIPNX_EINVAL, "strided_copy: negative offset");
  int64_t n = 1, ie = in_offset + 1, oe = out_offset + 1, ifirst = in_offset;
  for (int a = 0; a < rank; a++) {
    // the input may be walked backwards along an axis (reverse); the output never is
    if (dims[a] < 0 || out_strides[a] < 0) return set_error(HIPNX_EINVAL, "strided_copy: negative dimension or output stride");
    n *= dims[a];
  }
  if (n > 0)
    for (int a = 0; a < rank; a++) {
      if (in_strides[a] >= 0) ie += (dims[a] - 1) * in_strides[a];
      else ifirst += (dims[a] - 1) * in_strides[a];
      oe += (dims[a] - 1) * out_strides[a];
    }
  if (n > 0 && ifirst < 0) return set_error(HIPNX_EINVAL, "strided_copy: the input walk leaves the buffer at its start");
  if (int st = check_buf(ctx, inb, n > 0 ? (uint64_t)ie * elem_bytes : 0, "strided_copy in")) return st;
  if (int st = check_buf(ctx, out, n > 0 ? (uint64_t)oe * elem_bytes : 0, "strided_copy out")) return st;
  if (n == 0) return HIPNX_OK;
  Copy c;
  int m = 0;
  for (int a = 0; a < rank; a++) {
    const int64_t d = dims[a];
    if (d == 1) continue;
    if (m > 0 && c.is[m - 1] == in_strides[a] * d && c.os[m - 1] == out_strides[a] * d) {
      c.dims[m - 1] *= d; c.is[m - 1] = in_strides[a]; c.os[m - 1] = out_strides[a];
    } else {
      if (m == MAXR) return set_error(HIPNX_EUNSUPPORTED, "strided_copy: more than %d non-collapsible axes", MAXR);
      c.dims[m] = d; c.is[m] = in_strides[a]; c.os[m] = out_strides[a]; m++;
    }
  }
  if (m == 0) { c.dims[0] = 1; c.is[0] = c.os[0] = 0; m = 1; }
  c.rank = m;
  // widen: when the innermost axis is dense on both sides and everything else sits on 16-byte
  // boundaries, move 16 bytes per lane instead of one element
  int eb = elem_bytes;
  int64_t io = in_offset, oo = out_offset;
  const int per = 16 / elem_bytes;
  bool wide = c.is[m - 1] == 1 && c.os[m - 1] == 1 && c.dims[m - 1] % per == 0 && io % per == 0 && oo % per == 0 &&
              ((uintptr_t)inb->ptr % 16 == 0) && ((uintptr_t)out->ptr % 16 == 0);
  for (int a = 0; a + 1 < m && wide; a++) wide = c.is[a] % per == 0 && c.os[a] % per == 0;
  if (wide && per > 1) {
    c.dims[m - 1] /= per;
    for (int a = 0; a + 1 < m; a++) { c.is[a] /= per; c.os[a] /= per; }
    io /= per; oo /= per; n /= per; eb = 16;
  }
  const char *src = (const char *)inb->ptr + io * eb;
  char *dst = (char *)out->ptr + oo * eb;
  if (eb < 8 && c.os[m - 1] == 1 && (c.is[m - 1] == 1 || c.is[m - 1] == -1) && c.dims[m - 1] >= 2 * (16 / eb)) {
    const int V = 16 / eb;
    const int64_t row_len = c.dims[m - 1];
    const int reversed = c.is[m - 1] < 0;
    c.dims[m - 1] = (row_len + V - 1) / V;
    const int64_t nvec = n / row_len * c.dims[m - 1];
    dim3 grid(grid_for(nvec)), block(BLOCK);
    switch (eb) {
      case 1: hipLaunchKernelGGL((copy_runs_kernel<uint8_t>), grid, block, 0, ctx->stream, (const uint8_t *)src, (uint8_t *)dst, nvec, c, row_len, reversed); break;
      case 2: hipLaunchKernelGGL((copy_runs_kernel<uint16_t>), grid, block, 0, ctx->stream, (const uint16_t *)src, (uint16_t *)dst, nvec, c, row_len, reversed); break;
      default: hipLaunchKernelGGL((copy_runs_kernel<uint32_t>), grid, block, 0, ctx->stream, (const uint32_t *)src, (uint32_t *)dst, nvec, c, row_len, reversed); break;
    }
    HIPNX_HIP(hipGetLastError());
    return HIPNX_OK;
  }
  switch (eb) {
    case 1: launch_copy<uint8_t>(ctx, src, dst, n, c); break;
    case 2: launch_copy<uint16_t>(ctx, src, dst, n, c); break;
    case 4: launch_copy<uint32_t>(ctx, src, dst, n, c); break;
    case 8: launch_copy<uint64_t>(ctx, src, dst, n, c); break;
    default: launch_copy<uint4>(ctx, src, dst, n, c); break;
  }
  HIPNX_HIP(hipGetLastError());
  return HIPNX_OK;
}

static int iota_like(hipnx_ctx *ctx, int out_dt, int64_t n, int64_t dim, int64_t inner, int mode, hipnx_buf *out, const char *what) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (dtype_size(out_dt) < 0) return set_error(HIPNX_EINVAL, "%s: unknown element type", what);
  if (n < 0 || dim < 1 || inner < 1) return set_error(HIPNX_EINVAL, "%s: bad extents", what);
  if (int st = check_buf(ctx, out, (uint64_t)n * dtype_size(out_dt), what)) return st;
  if (n == 0) return HIPNX_OK;
  dim3 block(BLOCK);
  // an extent beyond the element count never wraps: clamp it so that it fits the counter type
  if (dim > n) dim = n;
  if (inner > n) inner = n;
  const bool small = n < (1ll << 31);
#define HIPNX_IOTA(CT, IT, ODT, EV) hipLaunchKernelGGL((iota_kernel<CT, IT, ODT, EV>), dim3(grid_for((n + EV - 1) / EV)), block, 0, ctx->stream, out->ptr, out_dt, n, dim, inner, mode)
  if (small && out_dt == HIPNX_F32) HIPNX_IOTA(float, int32_t, HIPNX_F32, 8);
  else if (small && out_dt == HIPNX_BF16) HIPNX_IOTA(float, int32_t, HIPNX_BF16, 8);
  else if (small && out_dt == HIPNX_S32) HIPNX_IOTA(int64_t, int32_t, HIPNX_S32, 8);
  else if (small && out_dt == HIPNX_S64) HIPNX_IOTA(int64_t, int32_t, HIPNX_S64, 4);
  else if (small && out_dt == HIPNX_U8) HIPNX_IOTA(int64_t, int32_t, HIPNX_U8, 8);
  else if (small && is_float(out_dt) && out_dt != HIPNX_F64) HIPNX_IOTA(float, int32_t, -1, 8);
  else if (is_float(out_dt)) HIPNX_IOTA(double, int64_t, -1, 8);
  else if (small) HIPNX_IOTA(int64_t, int32_t, -1, 8);
  else HIPNX_IOTA(int64_t, int64_t, -1, 8);
#undef HIPNX_IOTA
  HIPNX_HIP(hipGetLastError());
  return HIPNX_OK;
}

extern "C" int hipnx_iota(hipnx_ctx *ctx, int out_dt, int64_t n, int64_t dim, int64_t inner, hipnx_buf *out) {
  return iota_like(ctx, out_dt, n, dim, inner, 0, out, "iota");
}

extern "C" int hipnx_eye(hipnx_ctx *ctx, int out_dt, int64_t n, int64_t rows, int64_t cols, hipnx_buf *out) {
  return iota_like(ctx, out_dt, n, rows, cols, 1, out, "eye");
}
