// Axis reductions: sum / product / reduce_max / reduce_min and argmax / argmin.
//
// The input is viewed as [outer, red, inner].
//   inner == 1  ("rows"):    the reduced axis is contiguous.  One wavefront (short rows) or one
//                            256-lane block (long rows) per row streams it with 16-byte loads,
//                            folds in registers, then combines across lanes with wave shuffles
//                            and across the block's 4 waves through LDS.  A few very long rows
//                            are split into segments and finished by a second tiny kernel.
//   inner  > 1  ("columns"): lanes run along `inner` (coalesced), each walks `red` serially.
// Accumulators: floats sum in f64 (the reference folds in f64 and rounds once,
// nx/lib/nx/binary_backend.ex:1315-1324, 2342-2360; any f64 summation order rounds to the same
// f32 except in rare half-ulp cases), integers in wrapping 64-bit (exact low bits).
// Max/min keep NaN sticky (binary_backend.ex:1349-1375); arg-reductions carry (value, index)
// pairs whose combine rule is associative and commutative, so the tree order cannot change the
// answer: a NaN beats every number and the larger index wins among NaNs (the reference's
// sequential scan lets every NaN replace the current extreme, binary_backend.ex:1419-1427);
// otherwise the better value wins and equal values resolve to the smaller (tie LOW) or larger
// (tie HIGH) index.
// Algorithmic traffic: bytes(in) + bytes(out).
#pragma once
#include <type_traits>
#include <utility>

#include "internal.h"
#include "reduce_ops.cuh"

namespace hipnx {

// ---- rows: inner == 1 -----------------------------------------------------------------------
// TPR lanes per row (64 or 256); a block of 256 lanes covers 256/TPR rows.  Row `row` segment
// `seg` covers elements [seg*seg_len, min(red, (seg+1)*seg_len)).  With nseg == 1 the result is
// encoded into `out`; otherwise the raw accumulator goes to `partial[row*nseg + seg]`.
// IDT >= 0: the input's element type, known when the kernel is compiled (the type switch inside every
// vector load, and the scalar bookkeeping the compiler builds around it, fold away); -1: read from `idt_`.
// Elements a lane takes per load where the reducer allows any assignment of elements to lanes and the element type is
// known at compile time: 16 bytes (one access per lane, lanes side by side, so that a wave instruction covers whole
// lines), instead of the eight elements whose order of folding a sum's bits depend on.
constexpr int reduce_type_bytes(int dt) {
  return dt < 0 ? 0 : (dt == HIPNX_U8 || dt == HIPNX_S8) ? 1 : (dt == HIPNX_U16 || dt == HIPNX_S16 || dt == HIPNX_F16 || dt == HIPNX_BF16) ? 2
         : (dt == HIPNX_U32 || dt == HIPNX_S32 || dt == HIPNX_F32) ? 4 : 8;
}
template <typename R>
constexpr int reduce_load_elems(int idt) {
  return R::any_order && reduce_type_bytes(idt) >= 4 ? 16 / reduce_type_bytes(idt) : E;
}

// NT: the input is far larger than the last-level cache and is read with the non-temporal hint (a template parameter:
// where a branch chooses between a hinted and a plain load the compiler merges them and drops the hint).
template <typename R, typename CT, int TPR, bool VEC, int IDT = -1, bool NT = false>
__global__ void __launch_bounds__(BLOCK)
reduce_rows_kernel(const void *__restrict__ in, void *__restrict__ out, typename R::acc_t *__restrict__ partial,
                   int idt_, int odt, int64_t rows, int64_t red, int64_t seg_len, int nseg) {
  const int idt = IDT >= 0 ? IDT : idt_;
  constexpr int RPB = BLOCK / TPR;
  const int sub = threadIdx.x / TPR, lane = threadIdx.x % TPR;
  // (the grid is capped: a launch may not hold 2^32 lanes, and rows * nseg has no such bound)
  for (int64_t first = (int64_t)blockIdx.x * RPB; first < rows * nseg; first += (int64_t)gridDim.x * RPB) {
  const int64_t unit = first + sub;  // (row, seg) pair
  // (whole rows, the usual case, without the division, whose 64-bit form is some hundred instructions per wave)
  const int64_t row = nseg == 1 ? unit : unit / nseg;
  const int seg = nseg == 1 ? 0 : (int)(unit - row * nseg);
  typename R::acc_t acc = R::init();
  if (row < rows) {
    const int64_t k0 = (int64_t)seg * seg_len;
    const int64_t k1 = k0 + seg_len < red ? k0 + seg_len : red;
    const int64_t base = row * red;
    if constexpr (VEC) {  // red % E == 0 and seg_len % E == 0: every vector is aligned
      // two (then one) vectors per step: both loads are issued before either is folded.  A vector is eight elements,
      // or 16 bytes where the reducer lets the lanes share a row any way (EL: maxima, arg-reductions, all / any)
      constexpr int EL = reduce_load_elems<R>(IDT);
      int64_t k = k0 + (int64_t)lane * EL;
      if (k < k1) acc = R::seed(acc, k);
      const int64_t step = (int64_t)TPR * EL;
      for (; k + step < k1; k += 2 * step) {
        CT v[EL], w[EL];
        load_vec<CT, EL, true, NT>(in, idt, base + k, v);
        load_vec<CT, EL, true, NT>(in, idt, base + k + step, w);
#pragma unroll
        for (int i = 0; i < EL; i++) acc = R::accumulate(acc, v[i], k + i);
#pragma unroll
        for (int i = 0; i < EL; i++) acc = R::accumulate(acc, w[i], k + step + i);
      }
      for (; k < k1; k += step) {
        CT v[EL];
        load_vec<CT, EL, true, NT>(in, idt, base + k, v);
#pragma unroll
        for (int i = 0; i < EL; i++) acc = R::accumulate(acc, v[i], k + i);
      }
    } else if constexpr (TPR < WAVE) {
      // a short row that is not whole vectors (33 elements): vectors fetched at whatever address they have, the
      // last few elements one per lane; a lane meets its elements in rising order
      const int64_t nv = (k1 - k0) / E, kt = k0 + nv * E;
      if (lane < nv) acc = R::seed(acc, k0 + (int64_t)lane * E);
      else if (kt + lane < k1) acc = R::seed(acc, kt + lane);
      for (int64_t v = lane; v < nv; v += TPR) {
        CT x[E];
        load_vec<CT, E, false>(in, idt, base + k0 + v * E, x);
#pragma unroll
        for (int i = 0; i < E; i++) acc = R::accumulate(acc, x[i], k0 + v * E + i);
      }
      if (kt + lane < k1) acc = R::accumulate(acc, load_one<CT>(in, idt, base + kt + lane), kt + lane);
    } else {
      // a row that is not whole vectors (a vocabulary of 50257 entries): its first elements up to a vector boundary of
      // the BUFFER one per lane, then whole aligned vectors, then the last few elements one per lane.  A lane still
      // meets its elements in rising order, as the index reducers expect.  (One element per lane and step moved
      // 256 bytes per wave instruction: f32 rows of 16381 ran at 2.5 TB/s.)
      const int64_t head0 = (E - (base + k0) % E) % E, head = head0 < k1 - k0 ? head0 : k1 - k0;
      const int64_t kb = k0 + head, nv = (k1 - kb) / E, kt = kb + nv * E;
      if (lane < head) acc = R::seed(acc, k0 + lane);
      else if (lane < nv) acc = R::seed(acc, kb + (int64_t)lane * E);
      else if (kt + lane < k1) acc = R::seed(acc, kt + lane);
      if (lane < head) acc = R::accumulate(acc, load_one<CT>(in, idt, base + k0 + lane), k0 + lane);
      int64_t v = lane;
      for (; v + TPR < nv; v += 2 * TPR) {
        CT x[E], y[E];
        load_vec<CT, E>(in, idt, base + kb + v * E, x);
        load_vec<CT, E>(in, idt, base + kb + (v + TPR) * E, y);
#pragma unroll
        for (int i = 0; i < E; i++) acc = R::accumulate(acc, x[i], kb + v * E + i);
#pragma unroll
        for (int i = 0; i < E; i++) acc = R::accumulate(acc, y[i], kb + (v + TPR) * E + i);
      }
      for (; v < nv; v += TPR) {
        CT x[E];
        load_vec<CT, E>(in, idt, base + kb + v * E, x);
#pragma unroll
        for (int i = 0; i < E; i++) acc = R::accumulate(acc, x[i], kb + v * E + i);
      }
      if (kt + lane < k1) acc = R::accumulate(acc, load_one<CT>(in, idt, base + kt + lane), kt + lane);
    }
  }
  acc = wave_reduce<R, (TPR < WAVE ? TPR : WAVE)>(acc);
  if constexpr (TPR > WAVE) {
    __shared__ typename R::acc_t sm[BLOCK / WAVE];
    if (threadIdx.x % WAVE == 0) sm[threadIdx.x / WAVE] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
      for (int w = 1; w < BLOCK / WAVE; w++) acc = R::combine(acc, sm[w]);
    }
    __syncthreads();  // before the next pass writes sm again
  }
  if (lane == 0 && row < rows) {
    if (nseg == 1) finalize(out, odt, row, acc);
    else partial[row * nseg + seg] = acc;
  }
  }
}

// rows that give every lane of their group at most one vector (red <= TPR * E; whole vectors): what the kernel above
// does for them -- a lane folds its vector in rising order, the group combines -- without its loops over segments,
// rows beyond the grid and vectors beyond the first, whose 64-bit bookkeeping cost a wave more instructions than
// the fold itself (sum of 16384 f32 rows of 512, held by the caches: 5.8 -> 4.4 us).  Same order, same bits.
template <typename R, typename CT, int TPR, int IDT>
__global__ void __launch_bounds__(BLOCK)
reduce_rows_once_kernel(const void *__restrict__ in, void *__restrict__ out, int odt, uint32_t rows, uint32_t red) {
  constexpr int RPB = BLOCK / TPR;
  const uint32_t row = blockIdx.x * RPB + threadIdx.x / TPR, lane = threadIdx.x % TPR, k = lane * E;
  typename R::acc_t acc = R::init();
  if (row < rows && k < red) {
    acc = R::seed(acc, (int64_t)k);
    CT v[E];
    load_vec<CT, E>(in, IDT, (int64_t)row * red + k, v);
#pragma unroll
    for (int i = 0; i < E; i++) acc = R::accumulate(acc, v[i], (int64_t)k + i);
  }
  acc = wave_reduce<R, TPR>(acc);
  if (lane == 0 && row < rows) finalize(out, odt, row, acc);
}

// rows of up to 16 elements: one lane per row, walking it in order.  A group of 8 lanes (the narrowest above) would
// leave most of its lanes without an element (f32 rows of 8: 1.3 TB/s; rows of 2, which are not whole vectors and took
// a wave each: 0.06 TB/s).  Adjacent lanes read adjacent rows, so a wave's loads stay within `red` neighbouring lines.
template <typename R, typename CT, int IDT = -1>
__global__ void __launch_bounds__(BLOCK)
reduce_rows_short_kernel(const void *__restrict__ in, void *__restrict__ out, int idt_, int odt, int64_t rows, int red) {
  const int idt = IDT >= 0 ? IDT : idt_;
  for (int64_t row = (int64_t)blockIdx.x * BLOCK + threadIdx.x; row < rows; row += (int64_t)gridDim.x * BLOCK) {
    typename R::acc_t acc = red > 0 ? R::seed(R::init(), 0) : R::init();
    const int64_t base = row * red;
    int k = 0;
    for (; k + E <= red; k += E) {  // whole vectors at whatever address the row has (rows of 8 ... 16 elements)
      CT v[E];
      load_vec<CT, E, false>(in, idt, base + k, v);
#pragma unroll
      for (int i = 0; i < E; i++) acc = R::accumulate(acc, v[i], k + i);
    }
    for (; k < red; k++) acc = R::accumulate(acc, load_one<CT>(in, idt, base + k), k);
    finalize(out, odt, row, acc);
  }
}

// second pass of a split row reduction: one wave per row folds its nseg partials
template <typename R>
__global__ void __launch_bounds__(BLOCK)
combine_partials_kernel(const typename R::acc_t *__restrict__ partial, void *__restrict__ out, int odt, int64_t rows,
                        int nseg) {
  const int64_t row = (int64_t)blockIdx.x * (BLOCK / WAVE) + threadIdx.x / WAVE;
  const int lane = threadIdx.x % WAVE;
  typename R::acc_t acc = R::init();
  if (row < rows)
    for (int s = lane; s < nseg; s += WAVE) acc = R::combine(acc, partial[row * nseg + s]);
  acc = wave_reduce<R>(acc);
  if (lane == 0 && row < rows) finalize(out, odt, row, acc);
}

// ---- columns: inner > 1 ---------------------------------------------------------------------
// One lane per E adjacent inner positions (VEC) or per position; walks k in its segment.
// With nseg == 1 results are encoded into out[outer, inner]; otherwise raw accumulators go to
// partial[outer, nseg, inner].
// UNAL (with VEC): `inner` is not a multiple of E (a row of 50257 columns), so a row begins at any offset from a
// vector boundary: whole vectors are fetched at whatever address they have, the last lane of a row takes its
// remaining columns one by one (one column per lane moved 256 bytes per wave instruction: 1.6-1.9 TB/s).
template <typename R, typename CT, bool VEC, int IDT = -1, bool UNAL = false, bool NT = false>
__global__ void __launch_bounds__(BLOCK)
reduce_cols_kernel(const void *__restrict__ in, void *__restrict__ out, typename R::acc_t *__restrict__ partial,
                   int idt_, int odt, int64_t outer, int64_t red, int64_t inner, int64_t seg_len, int nseg) {
  const int idt = IDT >= 0 ? IDT : idt_;
  constexpr int W = VEC ? E : 1;
  const int64_t ivecs = UNAL ? (inner + W - 1) / W : inner / W;
  const int64_t total = outer * nseg * ivecs;
  for (int64_t t = (int64_t)blockIdx.x * BLOCK + threadIdx.x; t < total; t += (int64_t)gridDim.x * BLOCK) {
    const int64_t iv = t % ivecs, os = t / ivecs;
    const int64_t o = os / nseg;
    const int seg = (int)(os - o * nseg);
    const int64_t k0 = (int64_t)seg * seg_len, k1 = k0 + seg_len < red ? k0 + seg_len : red;
    typename R::acc_t acc[W];
#pragma unroll
    for (int i = 0; i < W; i++) acc[i] = k0 < k1 ? R::seed(R::init(), k0) : R::init();
    const int64_t base = o * red * inner + iv * W;
    const int valid = UNAL && iv * W + W > inner ? (int)(inner - iv * W) : W;  // columns of this lane inside the row
    if (UNAL && valid < W) {
      for (int i = 0; i < valid; i++) {
        typename R::acc_t a = k0 < k1 ? R::seed(R::init(), k0) : R::init();
        for (int64_t k = k0; k < k1; k++) a = R::accumulate(a, load_one<CT>(in, idt, base + k * inner + i), k);
        if (nseg == 1) finalize(out, odt, o * inner + iv * W + i, a);
        else partial[(o * nseg + seg) * inner + iv * W + i] = a;
      }
      continue;
    }
    int64_t k = k0;
    for (; k + 3 < k1; k += 4) {  // four independent row loads in flight per lane
      CT v0[W], v1[W], v2[W], v3[W];
      load_vec<CT, W, !UNAL, NT>(in, idt, base + k * inner, v0);
      load_vec<CT, W, !UNAL, NT>(in, idt, base + (k + 1) * inner, v1);
      load_vec<CT, W, !UNAL, NT>(in, idt, base + (k + 2) * inner, v2);
      load_vec<CT, W, !UNAL, NT>(in, idt, base + (k + 3) * inner, v3);
#pragma unroll
      for (int i = 0; i < W; i++) {
        acc[i] = R::accumulate(acc[i], v0[i], k);
        acc[i] = R::accumulate(acc[i], v1[i], k + 1);
        acc[i] = R::accumulate(acc[i], v2[i], k + 2);
        acc[i] = R::accumulate(acc[i], v3[i], k + 3);
      }
    }
    for (; k < k1; k++) {
      CT v[W];
      load_vec<CT, W, !UNAL>(in, idt, base + k * inner, v);
#pragma unroll
      for (int i = 0; i < W; i++) acc[i] = R::accumulate(acc[i], v[i], k);
    }
#pragma unroll
    for (int i = 0; i < W; i++) {
      if (nseg == 1) finalize(out, odt, o * inner + iv * W + i, acc[i]);
      else partial[(o * nseg + seg) * inner + iv * W + i] = acc[i];
    }
  }
}

// fold partial[outer, nseg, inner] -> out[outer, inner].  A work-group takes 32 adjacent outputs; its eight rows
// of 32 lanes each fold a slice of the segments (four loads in flight per lane), and the first row folds the eight
// slices in segment order.  (One lane per output walking all segments is a chain of up to 1024 dependent
// round trips to L2: 30-50 us on a 4096 x 4096 input, more than the first pass.)
constexpr int COMBINE_COLS_X = 32, COMBINE_COLS_Y = BLOCK / COMBINE_COLS_X;
template <typename R>
__global__ void __launch_bounds__(BLOCK)
combine_cols_kernel(const typename R::acc_t *__restrict__ partial, void *__restrict__ out, int odt, int64_t outer,
                    int64_t inner, int nseg) {
  typedef typename R::acc_t acc_t;
  __shared__ acc_t sm[COMBINE_COLS_Y][COMBINE_COLS_X];
  const int tx = threadIdx.x % COMBINE_COLS_X, ty = threadIdx.x / COMBINE_COLS_X;
  const int64_t total = outer * inner;
  const int per = (nseg + COMBINE_COLS_Y - 1) / COMBINE_COLS_Y;
  const int s0 = ty * per, s1 = s0 + per < nseg ? s0 + per : nseg;
  for (int64_t t0 = (int64_t)blockIdx.x * COMBINE_COLS_X; t0 < total; t0 += (int64_t)gridDim.x * COMBINE_COLS_X) {
    const int64_t t = t0 + tx;
    acc_t acc = R::init();
    if (t < total) {
      const int64_t o = t / inner, i = t - o * inner;
      const acc_t *p = partial + o * nseg * inner + i;
      int sgm = s0;
      for (; sgm + 3 < s1; sgm += 4) {
        const acc_t a0 = p[(int64_t)sgm * inner], a1 = p[(int64_t)(sgm + 1) * inner], a2 = p[(int64_t)(sgm + 2) * inner], a3 = p[(int64_t)(sgm + 3) * inner];
        acc = R::combine(R::combine(R::combine(R::combine(acc, a0), a1), a2), a3);
      }
      for (; sgm < s1; sgm++) acc = R::combine(acc, p[(int64_t)sgm * inner]);
    }
    sm[ty][tx] = acc;
    __syncthreads();
    if (ty == 0 && t < total) {
#pragma unroll
      for (int y = 1; y < COMBINE_COLS_Y; y++) acc = R::combine(acc, sm[y][tx]);
      finalize(out, odt, t, acc);
    }
    __syncthreads();
  }
}

// ---- host side ------------------------------------------------------------------------------

static int64_t round_up(int64_t a, int64_t b) { return (a + b - 1) / b * b; }

// a launch may hold at most 2^32 - 1 lanes along x: the kernels loop over what a capped grid leaves
constexpr int64_t MAX_BLOCKS = ((1ll << 32) - 1) / BLOCK;

// Partial results of a split reduction live either in a block of the context's pool (handed back
// right after the launches: later work on this stream is ordered behind them) or, for the entry
// point that allocates nothing, in this file's static device array.
static int partials_acquire(hipnx_ctx *ctx, bool static_ws, size_t bytes, void **ws, size_t *ws_cap) {
  if (!static_ws) return pool_alloc(ctx, bytes, ws, ws_cap);
  *ws_cap = 0;
  if (bytes > HIPNX_REDUCE_STATIC_SCRATCH_BYTES)
    return set_error(HIPNX_EUNSUPPORTED, "reduce_static: this shape needs %zu bytes of partial results, the static scratch holds %zu",
                     bytes, (size_t)HIPNX_REDUCE_STATIC_SCRATCH_BYTES);
  if (!ctx->reduce_scratch) return set_error(HIPNX_EHIP, "reduce_static: the static scratch of this device was not resolved");
  *ws = ctx->reduce_scratch;
  return HIPNX_OK;
}
static void partials_release(hipnx_ctx *ctx, bool static_ws, void *ws, size_t ws_cap) {
  if (ws && !static_ws) pool_free(ctx, ws, ws_cap);
}

// A few very long rows are cut into segments, a work-group each, so that the whole device reads them; a second
// small kernel folds the segments' raw accumulators in segment order.  The rule is shared by everything that
// must add in the same order (the reduction fused into an element-wise group follows it).
static inline void plan_row_segments(const hipnx_ctx *ctx, int64_t rows, int64_t red, int *nseg, int64_t *seg_len) {
  const int64_t target_units = (int64_t)ctx->num_cus * 8;  // units of parallel work wanted
  const int64_t min_row = 32768;                           // a row shorter than this stays whole: the second kernel costs more
  const int64_t min_seg = 4096;                            // elements per segment worth a block (sixteen per lane)
  *nseg = 1;
  *seg_len = red;
  if (rows < target_units && red >= min_row) {
    const int64_t want = target_units / (rows > 0 ? rows : 1), maxs = red / min_seg;
    int n = (int)(want < maxs ? want : maxs);
    if (n > 1024) n = 1024;
    if (n < 1) n = 1;
    *seg_len = round_up((red + n - 1) / n, E);
    *nseg = (int)((red + *seg_len - 1) / *seg_len);
  }
}

template <typename R, typename CT, int IDT>
static int run_reduce_t(hipnx_ctx *ctx, bool static_ws, int idt, int odt, int64_t outer, int64_t red, int64_t inner,
                        const void *in, void *out) {
  typedef typename R::acc_t acc_t;
  // an input far larger than the 256 MB last-level cache is read with the non-temporal hint -- where a lane's vector is
  // one access (elements of 1 or 2 bytes: bf16 row sums over 16384^2 88 -> 80 us): the two 16-byte accesses of eight
  // f32 each take half of the same lines, and a line that is let go early is fetched twice (f32: 169 -> 180 us)
  // (reducers that let a lane take 16 bytes at a time read any type that way)
  const int stream = outer * red * inner * (int64_t)dtype_size(idt) >= (256ll << 20) &&
                     (dtype_size(idt) * E <= 16 || (R::any_order && IDT >= 0));
  if (inner == 1) {
    const int64_t rows = outer;
    const bool vec = red % E == 0;
    int tpr = red <= 4096 ? WAVE : BLOCK;
    int nseg = 1;
    int64_t seg_len = red;
    plan_row_segments(ctx, rows, red, &nseg, &seg_len);
    acc_t *partial = nullptr;
    void *ws = nullptr;
    size_t ws_cap = 0;
    if (nseg > 1) {
      if (int st = partials_acquire(ctx, static_ws, sizeof(acc_t) * (size_t)(rows * nseg), &ws, &ws_cap)) return st;
      partial = (acc_t *)ws;
    }
    // A short row leaves most of a wave without an element: when every lane of a narrower group gets at most
    // one vector (red <= TPR * E) the group does exactly what the wave would -- the idle lanes only ever
    // contributed the neutral element, and the group's combine steps are the wave's last ones -- so rows of
    // up to 64 / 128 / 256 elements take 8 / 16 / 32 lanes, eight to two rows per wave, with the same bits.
    // (compiled for the common element types only: IDT >= 0)
    if (IDT >= 0 && vec && nseg == 1 && red <= 32 * E) tpr = red <= 8 * E ? 8 : red <= 16 * E ? 16 : 32;
    // rows that are not whole vectors are read element by element, a lane group per row: 8 / 16 / 32 lanes for up to
    // 64 / 128 / 256 elements instead of a wave (f32 rows of 33: 0.6 TB/s with a wave per row)
    const bool narrow_scalar = !vec && nseg == 1 && red <= 256;
    if (narrow_scalar) tpr = red <= 64 ? 8 : red <= 128 ? 16 : 32;
    const int rpb = BLOCK / tpr;
    const int64_t blocks = (rows * nseg + rpb - 1) / rpb;
    dim3 grid((unsigned)(blocks < MAX_BLOCKS ? blocks : MAX_BLOCKS)), block(BLOCK);
    if (rows * nseg > 0 && red <= 16) {
      const int64_t b1 = (rows + BLOCK - 1) / BLOCK;
      hipLaunchKernelGGL((reduce_rows_short_kernel<R, CT, IDT>), dim3((unsigned)(b1 < MAX_BLOCKS ? b1 : MAX_BLOCKS)), block, 0, ctx->stream, in, out,
                         idt, odt, rows, (int)red);
    } else if (IDT >= 0 && vec && nseg == 1 && rows > 0 && rows < (1ll << 31) && red <= (tpr < WAVE ? tpr : WAVE) * E) {
      if constexpr (IDT >= 0) {
        const dim3 g1((unsigned)((rows + rpb - 1) / rpb));
        const uint32_t rows32 = (uint32_t)rows, red32 = (uint32_t)red;
        if (tpr == 8) hipLaunchKernelGGL((reduce_rows_once_kernel<R, CT, 8, IDT>), g1, block, 0, ctx->stream, in, out, odt, rows32, red32);
        else if (tpr == 16) hipLaunchKernelGGL((reduce_rows_once_kernel<R, CT, 16, IDT>), g1, block, 0, ctx->stream, in, out, odt, rows32, red32);
        else if (tpr == 32) hipLaunchKernelGGL((reduce_rows_once_kernel<R, CT, 32, IDT>), g1, block, 0, ctx->stream, in, out, odt, rows32, red32);
        else hipLaunchKernelGGL((reduce_rows_once_kernel<R, CT, WAVE, IDT>), g1, block, 0, ctx->stream, in, out, odt, rows32, red32);
      }
    } else if (rows * nseg > 0) {
      if (narrow_scalar) {
        if (tpr == 8) hipLaunchKernelGGL((reduce_rows_kernel<R, CT, 8, false, IDT>), grid, block, 0, ctx->stream, in, out, partial, idt, odt, rows, red, seg_len, nseg);
        else if (tpr == 16) hipLaunchKernelGGL((reduce_rows_kernel<R, CT, 16, false, IDT>), grid, block, 0, ctx->stream, in, out, partial, idt, odt, rows, red, seg_len, nseg);
        else hipLaunchKernelGGL((reduce_rows_kernel<R, CT, 32, false, IDT>), grid, block, 0, ctx->stream, in, out, partial, idt, odt, rows, red, seg_len, nseg);
      } else if (tpr < WAVE) {
        if constexpr (IDT >= 0) {
          if (tpr == 8) hipLaunchKernelGGL((reduce_rows_kernel<R, CT, 8, true, IDT>), grid, block, 0, ctx->stream, in, out, partial, idt, odt, rows, red, seg_len, nseg);
          else if (tpr == 16) hipLaunchKernelGGL((reduce_rows_kernel<R, CT, 16, true, IDT>), grid, block, 0, ctx->stream, in, out, partial, idt, odt, rows, red, seg_len, nseg);
          else hipLaunchKernelGGL((reduce_rows_kernel<R, CT, 32, true, IDT>), grid, block, 0, ctx->stream, in, out, partial, idt, odt, rows, red, seg_len, nseg);
        }
      } else if (tpr == WAVE) {
        if (vec && stream && IDT >= 0) hipLaunchKernelGGL((reduce_rows_kernel<R, CT, WAVE, true, IDT, (IDT >= 0)>), grid, block, 0, ctx->stream, in, out, partial, idt, odt, rows, red, seg_len, nseg);
        else if (vec) hipLaunchKernelGGL((reduce_rows_kernel<R, CT, WAVE, true, IDT>), grid, block, 0, ctx->stream, in, out, partial, idt, odt, rows, red, seg_len, nseg);
        else hipLaunchKernelGGL((reduce_rows_kernel<R, CT, WAVE, false, IDT>), grid, block, 0, ctx->stream, in, out, partial, idt, odt, rows, red, seg_len, nseg);
      } else {
        if (vec && stream && IDT >= 0) hipLaunchKernelGGL((reduce_rows_kernel<R, CT, BLOCK, true, IDT, (IDT >= 0)>), grid, block, 0, ctx->stream, in, out, partial, idt, odt, rows, red, seg_len, nseg);
        else if (vec) hipLaunchKernelGGL((reduce_rows_kernel<R, CT, BLOCK, true, IDT>), grid, block, 0, ctx->stream, in, out, partial, idt, odt, rows, red, seg_len, nseg);
        else hipLaunchKernelGGL((reduce_rows_kernel<R, CT, BLOCK, false, IDT>), grid, block, 0, ctx->stream, in, out, partial, idt, odt, rows, red, seg_len, nseg);
      }
      if (nseg > 1) {
        dim3 g2((unsigned)((rows + BLOCK / WAVE - 1) / (BLOCK / WAVE)));  // (rows < 8 * CUs here)
        hipLaunchKernelGGL((combine_partials_kernel<R>), g2, block, 0, ctx->stream, partial, out, odt, rows, nseg);
      }
    }
    partials_release(ctx, static_ws, ws, ws_cap);
  } else {
    const bool vec = inner % E == 0;
    const bool unal = !vec && inner >= 8 * E && IDT >= 0;  // long rows off the vector grid (compiled for the common element types)
    const int64_t lanes = outer * (unal ? (inner + E - 1) / E : inner / (vec ? E : 1));
    int nseg = 1;
    int64_t seg_len = red;
    // Waves wanted per CU: what keeps about 128 bytes per lane-row times 64 lanes in flight -- 4 for f32 (32 bytes
    // per lane and row), 8 for 2-byte types, 16 for bytes (measured on 16384 x 16384: f32 6.3 TB/s with 4 against
    // 6.0 with 8 and 5.0 with 16; bf16 5.3 / 5.7 / 5.0; u8 2.5 / 3.6 / 4.7).  More segments than that only add
    // partial results.
    const int lane_bytes = (vec || unal ? E : 1) * dtype_size(idt);
    const int colw = lane_bytes >= 64 ? 2 : lane_bytes <= 8 ? 16 : 128 / lane_bytes;
    const int64_t want_lanes = (int64_t)ctx->num_cus * colw * WAVE;
    if (lanes < want_lanes && red >= 64) {
      int64_t want = want_lanes / (lanes > 0 ? lanes : 1), maxs = red / 32;
      nseg = (int)(want < maxs ? want : maxs);
      if (nseg > 1024) nseg = 1024;
      if (nseg < 1) nseg = 1;
      seg_len = (red + nseg - 1) / nseg;
      nseg = (int)((red + seg_len - 1) / seg_len);
    }
    acc_t *partial = nullptr;
    void *ws = nullptr;
    size_t ws_cap = 0;
    if (nseg > 1) {
      if (int st = partials_acquire(ctx, static_ws, sizeof(acc_t) * (size_t)(outer * nseg * inner), &ws, &ws_cap)) return st;
      partial = (acc_t *)ws;
    }
    int64_t total = lanes * nseg;
    int64_t blocks = (total + BLOCK - 1) / BLOCK;
    const int64_t cap = MAX_BLOCKS;
    dim3 grid((unsigned)(blocks < 1 ? 1 : (blocks < cap ? blocks : cap))), block(BLOCK);
    if (total > 0) {
      if (vec && stream && IDT >= 0) hipLaunchKernelGGL((reduce_cols_kernel<R, CT, true, IDT, false, (IDT >= 0)>), grid, block, 0, ctx->stream, in, out, partial, idt, odt, outer, red, inner, seg_len, nseg);
      else if (vec) hipLaunchKernelGGL((reduce_cols_kernel<R, CT, true, IDT>), grid, block, 0, ctx->stream, in, out, partial, idt, odt, outer, red, inner, seg_len, nseg);
      else if (unal) hipLaunchKernelGGL((reduce_cols_kernel<R, CT, true, IDT, true>), grid, block, 0, ctx->stream, in, out, partial, idt, odt, outer, red, inner, seg_len, nseg);
      else hipLaunchKernelGGL((reduce_cols_kernel<R, CT, false>), grid, block, 0, ctx->stream, in, out, partial, idt, odt, outer, red, inner, seg_len, nseg);
      if (nseg > 1) {
        int64_t b2 = (outer * inner + COMBINE_COLS_X - 1) / COMBINE_COLS_X;
        dim3 g2((unsigned)(b2 < cap ? b2 : cap));
        hipLaunchKernelGGL((combine_cols_kernel<R>), g2, block, 0, ctx->stream, partial, out, odt, outer, inner, nseg);
      }
    }
    partials_release(ctx, static_ws, ws, ws_cap);
  }
  HIPNX_HIP(hipGetLastError());
  return HIPNX_OK;
}

// the vectorised kernels compiled for the input's element type where it is one of the common ones
template <typename R, typename CT>
static int run_reduce(hipnx_ctx *ctx, bool static_ws, int idt, int odt, int64_t outer, int64_t red, int64_t inner,
                      const void *in, void *out) {
#define HIPNX_RED_AS(T) if (idt == T) return run_reduce_t<R, CT, T>(ctx, static_ws, idt, odt, outer, red, inner, in, out);
  if constexpr (std::is_floating_point<CT>::value) {
    HIPNX_RED_AS(HIPNX_F32) HIPNX_RED_AS(HIPNX_BF16) HIPNX_RED_AS(HIPNX_F16)
    if constexpr (std::is_same<CT, double>::value) { HIPNX_RED_AS(HIPNX_F64) }
  } else {
    HIPNX_RED_AS(HIPNX_S32) HIPNX_RED_AS(HIPNX_U8)
  }
#undef HIPNX_RED_AS
  return run_reduce_t<R, CT, -1>(ctx, static_ws, idt, odt, outer, red, inner, in, out);
}

}  // namespace hipnx
