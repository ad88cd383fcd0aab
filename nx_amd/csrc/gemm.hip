// Nx.dot as a dense batched contraction  out[b, m, n] = sum_k l[b, m, k] * r[b, n, k]:
// argument checks and the choice of kernel.
//
//   bf16 / f16 / f32 operand pairs (f32 accumulation) and s8 pairs (exact s32 accumulation):
//     K a multiple of 128 bytes  -> the pipelined MFMA kernel (gemm_mfma.cuh), which takes both
//       operand layouts directly; only a K-outer operand whose row count is not a multiple of
//       its transpose block (16 s8 / 8 bf16,f16 / 4 f32 rows) is first re-laid by the tiled
//       transpose.
//     K a multiple of 16 bytes   -> gemm_kinner_kernel below: same MFMA fragments, single LDS
//       stage, register-staged loads, zero-filled K tail.
//   everything else (f64, wide integers, mixed operand types, tiny problems): dot_generic_kernel,
//     a plain tiled kernel accumulating in f64 or wrapping 64-bit integers.
//
// Algorithmic work: 2*B*M*N*K flop; minimum traffic bytes(l) + bytes(r) + bytes(out).
#include <type_traits>

#include <algorithm>
#include <cstdlib>

#include "gemm_launch.cuh"

namespace hipnx {

constexpr int GEMM_BLOCK = 256;
constexpr int BM = 128, BN = 128;

// l: [batch, M, Kb bytes], r: [batch, N, Kb bytes]  (Kb = K * element size, multiple of 16)
template <int DT>
__global__ void __launch_bounds__(GEMM_BLOCK)
gemm_kinner_kernel(const unsigned char *__restrict__ l, const unsigned char *__restrict__ r, void *__restrict__ out,
                   int odt, int64_t M, int64_t N, int64_t Kb, int tiles_m, int tiles_n) {
  typedef typename Mma<DT>::acc_t acc_t;
    __shared__ __attribute__((aligned(16))) unsigned char sA[BM * SLAB];
  __shared__ __attribute__((aligned(16))) unsigned char sB[BN * SLAB];

  const int tile = blockIdx.x;
  const int tm = tile / tiles_n, tn = tile % tiles_n;
  const int64_t b = blockIdx.y;
  const unsigned char *lb = l + b * M * Kb;
  const unsigned char *rb = r + b * N * Kb;
  const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;

  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int wm = (wave / 2) * 64, wn = (wave % 2) * 64;

  acc_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int q = 0; q < 16; q++) acc[i][j][q] = 0;

  // global -> LDS assignment: 128 rows x 8 chunks = 1024 chunks per operand, 4 per lane
  const int ld_chunk = tid % CHUNKS;  // 0..7
  const int ld_row = tid / CHUNKS;    // 0..31, +32 per pass

  for (int64_t k0 = 0; k0 < Kb; k0 += SLAB) {
    v4i ra[4], rbv[4];
#pragma unroll
    for (int p = 0; p < 4; p++) {
      const int row = ld_row + 32 * p;
      const int64_t kb = k0 + ld_chunk * 16;
      int64_t gm = m0 + row, gn = n0 + row;
      gm = gm < M ? gm : M - 1;  // rows past the edge are loaded (clamped) and never stored
      gn = gn < N ? gn : N - 1;
      if (kb < Kb) {
        ra[p] = *reinterpret_cast<const v4i *>(lb + gm * Kb + kb);
        rbv[p] = *reinterpret_cast<const v4i *>(rb + gn * Kb + kb);
      } else {
        ra[p] = v4i{0, 0, 0, 0};  // K tail: zero contributes nothing
        rbv[p] = v4i{0, 0, 0, 0};
      }
    }
    __syncthreads();  // previous slab fully consumed
#pragma unroll
    for (int p = 0; p < 4; p++) {
      const int row = ld_row + 32 * p;
      const int sw = (ld_chunk ^ (row & 7)) * 16;
      *reinterpret_cast<v4i *>(sA + row * SLAB + sw) = ra[p];
      *reinterpret_cast<v4i *>(sB + row * SLAB + sw) = rbv[p];
    }
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < SLAB / 32; ks++) {
      v4i fa[2], fb[2];
      const int chunk = 2 * ks + lane / 32;
#pragma unroll
      for (int i = 0; i < 2; i++) {
        const int rowa = wm + 32 * i + lane % 32;
        fa[i] = *reinterpret_cast<const v4i *>(sA + rowa * SLAB + ((chunk ^ (rowa & 7)) * 16));
        const int rowb = wn + 32 * i + lane % 32;
        fb[i] = *reinterpret_cast<const v4i *>(sB + rowb * SLAB + ((chunk ^ (rowb & 7)) * 16));
      }
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) Mma<DT>::step(acc[i][j], fa[i], fb[j]);
    }
  }

  // epilogue: D[i][j] of a 32x32 MFMA tile sits in lane (j + 32*((i/4)%2)), register 4*(i/8)+i%4
  unsigned char *ob = (unsigned char *)out;
  const int64_t obase = b * M * N;
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int q = 0; q < 16; q++) {
        const int64_t gm = m0 + wm + 32 * i + 8 * (q / 4) + 4 * (lane / 32) + (q % 4);
        const int64_t gn = n0 + wn + 32 * j + lane % 32;
        if (gm < M && gn < N) {
          if constexpr (DT == HIPNX_S8) store_one<int64_t>(ob, odt, obase + gm * N + gn, (int64_t)acc[i][j][q]);
          else store_one<float>(ob, odt, obase + gm * N + gn, (float)acc[i][j][q]);
        }
      }
}

// Plain tiled contraction for every other type combination.  16 x 16 outputs per block, K
// walked in slabs of 16 through LDS; operands are decoded to CT (double or wrapping int64).
// lk / rk: 1 when the operand is K-inner ([rows, K]), 0 when K-outer ([K, rows]).
template <typename CT>
__global__ void __launch_bounds__(256)
dot_generic_kernel(const void *__restrict__ l, const void *__restrict__ r, void *__restrict__ out, int ldt, int rdt,
                   int odt, int64_t M, int64_t N, int64_t K, int lk, int rk) {
  constexpr int T = 16;
  __shared__ CT sA[T][T + 1], sB[T][T + 1];
  const int tx = threadIdx.x % T, ty = threadIdx.x / T;
  // (tiles of M along x, which holds 2^31 - 1 groups: [2M, 3] . [3, 3] has 131072 of them; tiles of N along y)
  const int64_t b = blockIdx.z;
  const int64_t m = (int64_t)blockIdx.x * T + ty, n = (int64_t)blockIdx.y * T + tx;
  const int64_t lbase = b * M * K, rbase = b * N * K;
  CT acc = 0;
  for (int64_t k0 = 0; k0 < K; k0 += T) {
    {  // sA[ty][tx] = l[m, k0 + tx]; sB[ty][tx] = r[n0 + ty, k0 + tx]
      const int64_t k = k0 + tx;
      const int64_t mm = (int64_t)blockIdx.x * T + ty, nn = (int64_t)blockIdx.y * T + ty;
      sA[ty][tx] = (mm < M && k < K) ? load_one<CT>(l, ldt, lbase + (lk ? mm * K + k : k * M + mm)) : (CT)0;
      sB[ty][tx] = (nn < N && k < K) ? load_one<CT>(r, rdt, rbase + (rk ? nn * K + k : k * N + nn)) : (CT)0;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < T; kk++) {
      if constexpr (std::is_same<CT, double>::value) acc = sA[ty][kk] * sB[tx][kk] + acc;
      else acc = (int64_t)((uint64_t)sA[ty][kk] * (uint64_t)sB[tx][kk] + (uint64_t)acc);
    }
    __syncthreads();
  }
  if (m < M && n < N) store_one<CT>(out, odt, b * M * N + m * N + n, acc);
}

// Many small matrices (a 3 x 3 transform per point, a 4 x 4 block per item): one lane per output over the whole batch,
// walking k in order -- the tiled kernel above spends a work-group of 256 lanes on each item's nine outputs.
template <typename CT>
__global__ void __launch_bounds__(256)
dot_small_batched_kernel(const void *__restrict__ l, const void *__restrict__ r, void *__restrict__ out, int ldt, int rdt,
                         int odt, int64_t batch, int M, int N, int K, int lk, int rk) {
  const int64_t total = batch * M * N;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t b = i / (M * N);
    const int mn = (int)(i - b * (M * N)), m = mn / N, n = mn - m * N;
    const int64_t lbase = b * M * K, rbase = b * N * K;
    CT acc = 0;
    for (int k = 0; k < K; k++) {
      const CT x = load_one<CT>(l, ldt, lbase + (lk ? m * K + k : k * M + m)), y = load_one<CT>(r, rdt, rbase + (rk ? n * K + k : k * N + n));
      if constexpr (std::is_same<CT, double>::value) acc = x * y + acc;
      else acc = (int64_t)((uint64_t)x * (uint64_t)y + (uint64_t)acc);
    }
    store_one<CT>(out, odt, i, acc);
  }
}

// The same contraction on 64 x 64 tiles with 4 x 4 outputs per lane: eight LDS reads per sixteen multiply-adds
// instead of two per one, each output still accumulated over k in order (the same bits as the kernel above).
// f64 / s32 / mixed-type 4096^3: 8.4 TFLOP/s there.
template <typename CT>
__global__ void __launch_bounds__(256)
dot_blocked_kernel(const void *__restrict__ l, const void *__restrict__ r, void *__restrict__ out, int ldt, int rdt,
                   int odt, int64_t M, int64_t N, int64_t K, int lk, int rk) {
  constexpr int TM = 64, TN = 64, TK = 16;
  __shared__ CT sA[TK][TM + 4], sB[TK][TN + 4];
  const int tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
  const int64_t b = blockIdx.z, m0 = (int64_t)blockIdx.x * TM, n0 = (int64_t)blockIdx.y * TN;
  const int64_t lbase = b * M * K, rbase = b * N * K;
  CT acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = 0;
  for (int64_t k0 = 0; k0 < K; k0 += TK) {
#pragma unroll
    for (int q = 0; q < TM * TK / 256; q++) {
      const int e = tid + q * 256;
      // consecutive lanes along the operand's contiguous axis
      const int am = lk ? e / TK : e % TM, ak = lk ? e % TK : e / TM;
      const int bn = rk ? e / TK : e % TN, bk = rk ? e % TK : e / TN;
      const int64_t mm = m0 + am, nn = n0 + bn, ka = k0 + ak, kb = k0 + bk;
      sA[ak][am] = (mm < M && ka < K) ? load_one<CT>(l, ldt, lbase + (lk ? mm * K + ka : ka * M + mm)) : (CT)0;
      sB[bk][bn] = (nn < N && kb < K) ? load_one<CT>(r, rdt, rbase + (rk ? nn * K + kb : kb * N + nn)) : (CT)0;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < TK; kk++) {
      CT a[4], c[4];
#pragma unroll
      for (int i = 0; i < 4; i++) a[i] = sA[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; j++) c[j] = sB[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
          if constexpr (std::is_same<CT, double>::value) acc[i][j] = a[i] * c[j] + acc[i][j];
          else acc[i][j] = (int64_t)((uint64_t)a[i] * (uint64_t)c[j] + (uint64_t)acc[i][j]);
        }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int64_t m = m0 + ty * 4 + i, n = n0 + tx * 4 + j;
      if (m < M && n < N) store_one<CT>(out, odt, b * M * N + m * N + n, acc[i][j]);
    }
}

// A handful of outputs over a long contraction (the dot of two vectors, a [16, K] . [K, 16] Gram block): a work-group per
// output and segment of K, lanes along k, partial sums in f64 (wrapping 64-bit integers), then one small pass that adds
// an output's segments in order and encodes it.  The tiled kernels give such a problem one tile -- one work-group,
// or below 256 outputs one lane of the kernel above walking all of K (4M-element vectors: 0.26 s).
// l element (m, k) = l[m * l_sm + k * l_sk], r element (n, k) = r[n * r_sn + k * r_sk].
template <typename CT>
__global__ void __launch_bounds__(256)
dot_reduce_kernel(const void *__restrict__ l, const void *__restrict__ r, CT *__restrict__ partial, void *__restrict__ out, int ldt,
                  int rdt, int odt, int64_t M, int64_t N, int64_t K, int64_t l_sm, int64_t l_sk, int64_t r_sn, int64_t r_sk,
                  int64_t seg_len, int nseg, int vec) {
  constexpr int V = 8;
  const int64_t mn = blockIdx.y, b = blockIdx.z, m = mn / N, n = mn - m * N;
  const int seg = blockIdx.x;
  const int64_t k0 = (int64_t)seg * seg_len, k1 = k0 + seg_len < K ? k0 + seg_len : K;
  const int64_t lb = b * M * K + m * l_sm, rb = b * N * K + n * r_sn;
  CT acc = 0;
  auto mac = [&](CT x, CT y) {
    if constexpr (std::is_same<CT, double>::value) acc = x * y + acc;
    else acc = (int64_t)((uint64_t)x * (uint64_t)y + (uint64_t)acc);
  };
  if (vec) {  // both operands contiguous along k, every row and segment on a vector boundary
    for (int64_t k = k0 + (int64_t)threadIdx.x * V; k < k1; k += 256 * V) {
      CT x[V], y[V];
      load_vec<CT, V>(l, ldt, lb + k, x);
      load_vec<CT, V>(r, rdt, rb + k, y);
#pragma unroll
      for (int i = 0; i < V; i++) mac(x[i], y[i]);
    }
  } else {
    for (int64_t k = k0 + threadIdx.x; k < k1; k += 256) mac(load_one<CT>(l, ldt, lb + k * l_sk), load_one<CT>(r, rdt, rb + k * r_sk));
  }
  __shared__ CT sm[256];
  sm[threadIdx.x] = acc;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w) {
      if constexpr (std::is_same<CT, double>::value) sm[threadIdx.x] = sm[threadIdx.x] + sm[threadIdx.x + w];
      else sm[threadIdx.x] = (int64_t)((uint64_t)sm[threadIdx.x] + (uint64_t)sm[threadIdx.x + w]);
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    if (nseg == 1) store_one<CT>(out, odt, b * M * N + mn, sm[0]);
    else partial[(b * M * N + mn) * nseg + seg] = sm[0];
  }
}

template <typename CT>
__global__ void __launch_bounds__(256)
dot_reduce_finish_kernel(const CT *__restrict__ partial, void *__restrict__ out, int odt, int64_t outputs, int nseg) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < outputs; i += (int64_t)gridDim.x * 256) {
    CT acc = partial[i * nseg];
    for (int s = 1; s < nseg; s++) {
      if constexpr (std::is_same<CT, double>::value) acc = acc + partial[i * nseg + s];
      else acc = (int64_t)((uint64_t)acc + (uint64_t)partial[i * nseg + s]);
    }
    store_one<CT>(out, odt, i, acc);
  }
}

template <int DT>
static void launch_mfma(const hipnx_ctx *ctx, const void *l, const void *r, void *out, int odt, int64_t batch,
                        int64_t M, int64_t N, int64_t Kb) {
  int tiles_m = (int)((M + BM - 1) / BM), tiles_n = (int)((N + BN - 1) / BN);
  dim3 grid((unsigned)(tiles_m * tiles_n), (unsigned)batch);
  hipLaunchKernelGGL((gemm_kinner_kernel<DT>), grid, dim3(GEMM_BLOCK), 0, ctx->stream, (const unsigned char *)l,
                     (const unsigned char *)r, out, odt, M, N, Kb, tiles_m, tiles_n);
}

}  // namespace hipnx

using namespace hipnx;

// defined in move.hip
extern "C" int hipnx_transpose(hipnx_ctx *ctx, int elem_bytes, int rank, const int64_t *in_dims, const int *perm,
                               const hipnx_buf *inb, hipnx_buf *out);

// scale_mode != NONE: the scaled form (out_dt is then f32 over an s32 sum)
// Second pass of a contraction whose K was split over S work-groups per tile: out[i] = the S partial
// results of element i added in split order (f32 adds for the float types, wrapping 32-bit adds -- exact --
// for int8), then encoded once.
template <typename AT>
__global__ void __launch_bounds__(256)
splitk_combine_kernel(const AT *__restrict__ part, void *__restrict__ out, int odt, int64_t mn, int splits) {
  typedef typename std::conditional<std::is_same<AT, float>::value, float, int64_t>::type CT;
  const int64_t nvec = mn / 4;
  for (int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * 256) {
    typedef __attribute__((ext_vector_type(4))) AT vec_t;
    vec_t acc = *reinterpret_cast<const vec_t *>(part + v * 4);
    for (int s = 1; s < splits; s++) {
      const vec_t p = *reinterpret_cast<const vec_t *>(part + s * mn + v * 4);
#pragma unroll
      for (int e = 0; e < 4; e++) acc[e] += p[e];
    }
    CT x[4];
#pragma unroll
    for (int e = 0; e < 4; e++) x[e] = (CT)acc[e];
    store_vec<CT, 4>(out, odt, v * 4, x);
  }
}

// k_use > 0: contract only the first k_use of the K elements (a whole number of slabs); the operands keep their shapes
static int dot_impl(hipnx_ctx *ctx, int l_dt, int r_dt, int out_dt, int64_t batch, int64_t M, int64_t N,
                    int64_t K, int l_layout, int r_layout, const hipnx_buf *l, const hipnx_buf *r,
                    hipnx_buf *out, int scale_mode, const hipnx_buf *scale, int64_t k_use = 0);

// A copy of a dot operand ([batch, rows, K] or [batch, K, rows]) with K extended to Kp by zeros.
static int pad_k(hipnx_ctx *ctx, int esz, int64_t batch, int64_t rows, int64_t K, int64_t Kp, int layout,
                 const hipnx_buf *in, hipnx_buf **out) {
  int st = hipnx_buf_alloc(ctx, (size_t)(batch * rows * Kp * esz), out);
  if (st) return st;
  const unsigned char zero = 0;
  st = hipnx_fill(ctx, *out, 1, &zero, batch * rows * Kp * esz);
  if (st) return st;
  if (layout == HIPNX_K_INNER) {
    const int64_t dims[2] = {batch * rows, K}, is[2] = {K, 1}, os[2] = {Kp, 1};
    return hipnx_strided_copy(ctx, esz, 2, dims, is, 0, os, 0, in, *out);
  }
  const int64_t dims[2] = {batch, K * rows}, is[2] = {K * rows, 1}, os[2] = {Kp * rows, 1};
  return hipnx_strided_copy(ctx, esz, 2, dims, is, 0, os, 0, in, *out);
}

static int dot_impl(hipnx_ctx *ctx, int l_dt, int r_dt, int out_dt, int64_t batch, int64_t M, int64_t N,
                    int64_t K, int l_layout, int r_layout, const hipnx_buf *l, const hipnx_buf *r,
                    hipnx_buf *out, int scale_mode, const hipnx_buf *scale, int64_t k_use) {
  // More batch items than a grid's second dimension holds (100000 small matrices): runs of 65535 items, each over
  // borrowed handles on its part of the three buffers.
  if (batch > 65535 && M > 0 && N > 0 && l && r && out && dtype_size(l_dt) > 0 && dtype_size(r_dt) > 0 && out_dtype_size(out_dt) > 0 && K >= 0) {
    {
      Enter in(ctx);
      if (in.status) return in.status;
      if (int st = check_buf(ctx, l, (uint64_t)batch * M * K * dtype_size(l_dt), "dot lhs")) return st;
      if (int st = check_buf(ctx, r, (uint64_t)batch * N * K * dtype_size(r_dt), "dot rhs")) return st;
      if (int st = check_buf(ctx, out, (uint64_t)batch * M * N * out_dtype_size(out_dt), "dot out")) return st;
    }
    const size_t lb = (size_t)(M * K) * dtype_size(l_dt), rb = (size_t)(N * K) * dtype_size(r_dt), ob = (size_t)(M * N) * out_dtype_size(out_dt);
    for (int64_t b0 = 0; b0 < batch; b0 += 65535) {
      const int64_t nb = batch - b0 < 65535 ? batch - b0 : 65535;
      hipnx_buf *lw = nullptr, *rw = nullptr, *ow = nullptr;
      int st = hipnx_buf_wrap(ctx, (char *)l->ptr + b0 * lb, nb * lb > 0 ? nb * lb : 1, &lw);
      if (!st) st = hipnx_buf_wrap(ctx, (char *)r->ptr + b0 * rb, nb * rb > 0 ? nb * rb : 1, &rw);
      if (!st) st = hipnx_buf_wrap(ctx, (char *)out->ptr + b0 * ob, nb * ob, &ow);
      if (!st) st = dot_impl(ctx, l_dt, r_dt, out_dt, nb, M, N, K, l_layout, r_layout, lw, rw, ow, scale_mode, scale, k_use);
      if (lw) hipnx_buf_destroy(lw);
      if (rw) hipnx_buf_destroy(rw);
      if (ow) hipnx_buf_destroy(ow);
      if (st) return st;
    }
    return HIPNX_OK;
  }
  // A contraction length that is not a whole number of 128-byte slabs keeps a large MFMA-typed problem off the
  // tiled kernels (K not a multiple of 16 bytes even sends it to the generic kernel: a few TFLOP/s).  Both
  // operands are then copied with K extended by zeros -- products of two zeros, which add nothing -- and the
  // contraction runs on the copies.
  {
    const int esz = dtype_size(l_dt);
    const bool typed = l_dt == r_dt && esz > 0 && out_dtype_size(out_dt) > 0 &&
                       (((l_dt == HIPNX_BF16 || l_dt == HIPNX_F16 || l_dt == HIPNX_F32) && is_float(out_dt)) ||
                        (l_dt == HIPNX_S8 && !is_float(out_dt) && K <= (1ll << 16)));
    if (!k_use && typed && scale_mode == HIPNX_SCALE_NONE && K > 0 && batch > 0 && M > 0 && N > 0 && (K * esz) % SLAB != 0 && M * N >= 256 &&
        (double)M * (double)N * (double)K * (double)batch >= 16777216.0 && l && r &&
        (l_layout == HIPNX_K_INNER || l_layout == HIPNX_K_OUTER) && (r_layout == HIPNX_K_INNER || r_layout == HIPNX_K_OUTER)) {
      const int64_t per = SLAB / esz, Kp = (K + per - 1) / per * per;
      const int64_t Kmain = K / per * per, Ktail = K - Kmain;
      if (!k_use && batch == 1 && (K * esz) % 16 == 0 && Kmain >= 8 * per && (M * N) % 4 == 0) {
        // Rows that are whole 16-byte blocks need no copy of the operands: the whole slabs of K are contracted in
        // place (the kernels take a row pitch), the last part of K from two small zero-extended copies of one slab
        // per row, and the two f32 (s32) results are added and encoded by the pass that finishes a split K.  (A copy
        // of both operands extended to whole slabs: f32 [60000, 784] . [784, 10] 172 us for a 35 us contraction.)
        const int ws_dt = l_dt == HIPNX_S8 ? HIPNX_S32 : HIPNX_F32;
        const int64_t mn = M * N;
        hipnx_buf *ws = nullptr, *ws2 = nullptr, *lt = nullptr, *rt = nullptr;
        int st = hipnx_buf_alloc(ctx, (size_t)(2 * mn * 4), &ws);
        if (!st) st = hipnx_buf_wrap(ctx, (char *)ws->ptr + mn * 4, (size_t)(mn * 4), &ws2);
        if (!st) st = dot_impl(ctx, l_dt, r_dt, ws_dt, 1, M, N, K, l_layout, r_layout, l, r, ws, scale_mode, scale, Kmain);
        const unsigned char zero = 0;
        if (!st) st = hipnx_buf_alloc(ctx, (size_t)(M * SLAB), &lt);
        if (!st) st = hipnx_buf_alloc(ctx, (size_t)(N * SLAB), &rt);
        if (!st) st = hipnx_fill(ctx, lt, 1, &zero, M * SLAB);
        if (!st) st = hipnx_fill(ctx, rt, 1, &zero, N * SLAB);
        if (!st) {
          const int64_t dims[2] = {M, Ktail}, os[2] = {per, 1};
          const int64_t is_in[2] = {K, 1}, is_out[2] = {1, M};
          st = hipnx_strided_copy(ctx, esz, 2, dims, l_layout == HIPNX_K_INNER ? is_in : is_out,
                                  l_layout == HIPNX_K_INNER ? Kmain : Kmain * M, os, 0, l, lt);
        }
        if (!st) {
          const int64_t dims[2] = {N, Ktail}, os[2] = {per, 1};
          const int64_t is_in[2] = {K, 1}, is_out[2] = {1, N};
          st = hipnx_strided_copy(ctx, esz, 2, dims, r_layout == HIPNX_K_INNER ? is_in : is_out,
                                  r_layout == HIPNX_K_INNER ? Kmain : Kmain * N, os, 0, r, rt);
        }
        if (!st) st = dot_impl(ctx, l_dt, r_dt, ws_dt, 1, M, N, per, HIPNX_K_INNER, HIPNX_K_INNER, lt, rt, ws2, scale_mode, scale);
        if (!st) {
          Enter in(ctx);
          st = in.status;
          if (!st) st = check_buf(ctx, out, (uint64_t)mn * out_dtype_size(out_dt), "dot out");
          if (!st) {
            dim3 grid((unsigned)std::min<int64_t>((mn / 4 + 255) / 256, 1 << 20)), block(256);
            if (ws_dt == HIPNX_S32) hipLaunchKernelGGL((splitk_combine_kernel<int>), grid, block, 0, ctx->stream, (const int *)ws->ptr, out->ptr, out_dt, mn, 2);
            else hipLaunchKernelGGL((splitk_combine_kernel<float>), grid, block, 0, ctx->stream, (const float *)ws->ptr, out->ptr, out_dt, mn, 2);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) st = hip_fail(e, "combine launch");
          }
        }
        if (lt) hipnx_buf_destroy(lt);
        if (rt) hipnx_buf_destroy(rt);
        if (ws2) hipnx_buf_destroy(ws2);
        if (ws) hipnx_buf_destroy(ws);
        return st;
      }
      hipnx_buf *lp = nullptr, *rp = nullptr;
      int st = pad_k(ctx, esz, batch, M, K, Kp, l_layout, l, &lp);
      if (!st) st = pad_k(ctx, esz, batch, N, K, Kp, r_layout, r, &rp);
      if (!st) st = dot_impl(ctx, l_dt, r_dt, out_dt, batch, M, N, Kp, l_layout, r_layout, lp, rp, out, scale_mode, scale);
      if (lp) hipnx_buf_destroy(lp);
      if (rp) hipnx_buf_destroy(rp);
      return st;
    }
  }
  int64_t Kb = 0;
  bool mfma = false;
  {
    Enter in(ctx);
    if (in.status) return in.status;
    if (dtype_size(l_dt) < 0 || dtype_size(r_dt) < 0 || out_dtype_size(out_dt) < 0)
      return set_error(HIPNX_EINVAL, "dot: unknown element type");
    if (batch < 0 || M < 0 || N < 0 || K < 0) return set_error(HIPNX_EINVAL, "dot: negative extent");
    if ((l_layout != HIPNX_K_INNER && l_layout != HIPNX_K_OUTER) || (r_layout != HIPNX_K_INNER && r_layout != HIPNX_K_OUTER))
      return set_error(HIPNX_EINVAL, "dot: unknown operand layout");
    if (int st = check_buf(ctx, l, (uint64_t)batch * M * K * dtype_size(l_dt), "dot lhs")) return st;
    if (int st = check_buf(ctx, r, (uint64_t)batch * N * K * dtype_size(r_dt), "dot rhs")) return st;
    if (int st = check_buf(ctx, out, (uint64_t)batch * M * N * out_dtype_size(out_dt), "dot out")) return st;
    if (batch * M * N == 0) return HIPNX_OK;
    if (batch > 65535) return set_error(HIPNX_EUNSUPPORTED, "dot: more than 65535 batch items");

    Kb = (k_use ? k_use : K) * dtype_size(l_dt);  // what is contracted; the rows keep their pitch of K elements
    const bool float_pair = l_dt == r_dt && (l_dt == HIPNX_BF16 || l_dt == HIPNX_F16 || l_dt == HIPNX_F32 || l_dt == HIPNX_F64) && is_float(out_dt);
    const bool scaled = scale_mode != HIPNX_SCALE_NONE;
    const bool int8_pair = l_dt == HIPNX_S8 && r_dt == HIPNX_S8 && (scaled || !is_float(out_dt)) && K <= (1ll << 16);
    mfma = (float_pair || int8_pair) && K > 0 && Kb % 16 == 0 && M * N >= 256 && (l_dt != HIPNX_F64 || Kb % SLAB == 0);  // (f64: the slab kernels only)
    if (scaled) {
      if (!(int8_pair && mfma && Kb % SLAB == 0)) return set_error(HIPNX_EUNSUPPORTED, "dot_scaled: s8 x s8 with K a multiple of 128 and at most 65536, M * N >= 256");
      if (scale_mode == HIPNX_SCALE_PER_ROW && batch != 1) return set_error(HIPNX_EUNSUPPORTED, "dot_scaled: a scale per row with more than one batch item");
      const int64_t need = scale_mode == HIPNX_SCALE_PER_COLUMN ? N : scale_mode == HIPNX_SCALE_PER_ROW ? M : 1;
      if (int st = check_buf(ctx, scale, (uint64_t)need * 4, "dot_scaled scale")) return st;
    }

    // at most 32 x 32 outputs over a contraction of 4096 elements or more: the reduction kernels
    // (also a matrix against one to four vectors in f32 or wider types, where the matrix is contiguous along k: an MFMA
    // tile would be all but empty, and its f32 work costs more than the bytes -- [1, 8192] . [8192, 8192]^T 105 us)
    const bool few_vectors = dtype_size(l_dt) >= 4 && dtype_size(r_dt) >= 4 && K >= 1024 &&
                             ((M <= 4 && r_layout == HIPNX_K_INNER) || (N <= 4 && l_layout == HIPNX_K_INNER));
    if (!k_use && !scaled && ((M <= 32 && N <= 32 && (K >= 4096 || (M * N <= 4 && K >= 128))) || few_vectors) && M * N <= 65535 && batch * M * N <= 65535 && !(!is_float(l_dt) && !is_float(r_dt) && is_float(out_dt))) {
      const bool any_float = is_float(l_dt) || is_float(r_dt);
      const int lk = l_layout == HIPNX_K_INNER, rk = r_layout == HIPNX_K_INNER;
      const int64_t l_sm = lk ? K : 1, l_sk = lk ? 1 : M, r_sn = rk ? K : 1, r_sk = rk ? 1 : N;
      const int64_t outputs = batch * M * N;
      int64_t nseg = (2 * (int64_t)ctx->num_cus + outputs - 1) / outputs;
      if (nseg > K / 2048) nseg = K / 2048;
      if (nseg > 1024) nseg = 1024;
      if (nseg < 1) nseg = 1;
      int64_t seg_len = ((K + nseg - 1) / nseg + 7) / 8 * 8;
      nseg = (K + seg_len - 1) / seg_len;
      const int vec = l_sk == 1 && r_sk == 1 && K % 8 == 0 && ((uintptr_t)l->ptr % 32 == 0) && ((uintptr_t)r->ptr % 32 == 0);
      void *ws = nullptr;
      size_t ws_cap = 0;
      if (nseg > 1)
        if (int st = pool_alloc(ctx, (size_t)(outputs * nseg) * 8, &ws, &ws_cap)) return st;
      dim3 grid((unsigned)nseg, (unsigned)(M * N), (unsigned)batch), block(256);
      if (any_float) {
        hipLaunchKernelGGL((dot_reduce_kernel<double>), grid, block, 0, ctx->stream, l->ptr, r->ptr, (double *)ws, out->ptr, l_dt, r_dt, out_dt, M, N, K,
                           l_sm, l_sk, r_sn, r_sk, seg_len, (int)nseg, vec);
        if (nseg > 1)
          hipLaunchKernelGGL((dot_reduce_finish_kernel<double>), dim3((unsigned)((outputs + 255) / 256)), block, 0, ctx->stream, (const double *)ws,
                             out->ptr, out_dt, outputs, (int)nseg);
      } else {
        hipLaunchKernelGGL((dot_reduce_kernel<int64_t>), grid, block, 0, ctx->stream, l->ptr, r->ptr, (int64_t *)ws, out->ptr, l_dt, r_dt, out_dt, M, N, K,
                           l_sm, l_sk, r_sn, r_sk, seg_len, (int)nseg, vec);
        if (nseg > 1)
          hipLaunchKernelGGL((dot_reduce_finish_kernel<int64_t>), dim3((unsigned)((outputs + 255) / 256)), block, 0, ctx->stream, (const int64_t *)ws,
                             out->ptr, out_dt, outputs, (int)nseg);
      }
      if (ws) pool_free(ctx, ws, ws_cap);  // later work is ordered on the same stream
      HIPNX_HIP(hipGetLastError());
      return HIPNX_OK;
    }

    // many small matrices (up to 64 outputs, K up to 64): a lane per output over the whole batch (16 x 16 x 16 items are
    // faster on the tiled kernels: 51 us against 175 us for 8192 of them)
    if (!scaled && !k_use && M * N <= 64 && K <= 64 && batch >= 64 && !(!is_float(l_dt) && !is_float(r_dt) && is_float(out_dt))) {
      const bool any_float = is_float(l_dt) || is_float(r_dt);
      const int lk = l_layout == HIPNX_K_INNER, rk = r_layout == HIPNX_K_INNER;
      const int64_t blocks = (batch * M * N + 255) / 256;
      dim3 gs((unsigned)(blocks < (1ll << 24) - 1 ? blocks : (1ll << 24) - 1)), block(256);
      if (any_float)
        hipLaunchKernelGGL((dot_small_batched_kernel<double>), gs, block, 0, ctx->stream, l->ptr, r->ptr, out->ptr, l_dt, r_dt, out_dt, batch, (int)M, (int)N, (int)K, lk, rk);
      else
        hipLaunchKernelGGL((dot_small_batched_kernel<int64_t>), gs, block, 0, ctx->stream, l->ptr, r->ptr, out->ptr, l_dt, r_dt, out_dt, batch, (int)M, (int)N, (int)K, lk, rk);
      HIPNX_HIP(hipGetLastError());
      return HIPNX_OK;
    }

    if (!mfma) {
      const bool any_float = is_float(l_dt) || is_float(r_dt);
      if (!any_float && is_float(out_dt)) return set_error(HIPNX_EUNSUPPORTED, "dot: integer operands with a float output");
      dim3 grid((unsigned)((M + 15) / 16), (unsigned)((N + 15) / 16), (unsigned)batch), block(256);
      if ((N + 15) / 16 > 65535 || (M + 15) / 16 >= (1ll << 31) / 256)
        return set_error(HIPNX_EUNSUPPORTED, "dot: more than a million columns (or 134 million rows) on the plain kernel");
      const int lk = l_layout == HIPNX_K_INNER, rk = r_layout == HIPNX_K_INNER;
      // tiles of 64 x 64, sixteen outputs per lane, where they still give every CU two work-groups (512^3: 64 tiles, 143 us
      // against 53 us on 16 x 16 tiles)
      if (M >= 64 && N >= 64 && (N + 63) / 64 <= 65535 && ((M + 63) / 64) * ((N + 63) / 64) * batch >= 2 * (int64_t)ctx->num_cus) {
        dim3 g64((unsigned)((M + 63) / 64), (unsigned)((N + 63) / 64), (unsigned)batch);
        if (any_float)
          hipLaunchKernelGGL((dot_blocked_kernel<double>), g64, block, 0, ctx->stream, l->ptr, r->ptr, out->ptr, l_dt, r_dt, out_dt, M, N, K, lk, rk);
        else
          hipLaunchKernelGGL((dot_blocked_kernel<int64_t>), g64, block, 0, ctx->stream, l->ptr, r->ptr, out->ptr, l_dt, r_dt, out_dt, M, N, K, lk, rk);
        HIPNX_HIP(hipGetLastError());
        return HIPNX_OK;
      }
      if (any_float)
        hipLaunchKernelGGL((dot_generic_kernel<double>), grid, block, 0, ctx->stream, l->ptr, r->ptr, out->ptr, l_dt, r_dt, out_dt, M, N, K, lk, rk);
      else
        hipLaunchKernelGGL((dot_generic_kernel<int64_t>), grid, block, 0, ctx->stream, l->ptr, r->ptr, out->ptr, l_dt, r_dt, out_dt, M, N, K, lk, rk);
      HIPNX_HIP(hipGetLastError());
      return HIPNX_OK;
    }
  }

  // MFMA path.  Which operands need the tiled transpose to become K-inner first?
  const int esz = dtype_size(l_dt);
  const bool pipelined = Kb % SLAB == 0;
  // the pipelined kernel transposes K-outer operands itself when the rows come in whole blocks
  const int row_block = esz == 1 ? 16 : (esz == 2 ? 8 : esz == 4 ? 4 : 2);
  const bool l_relay = l_layout == HIPNX_K_OUTER && !(pipelined && M % row_block == 0);
  const bool r_relay = r_layout == HIPNX_K_OUTER && !(pipelined && N % row_block == 0);
  hipnx_buf *lt = nullptr, *rt = nullptr;
  int st = HIPNX_OK;
  if (l_relay) {
    st = hipnx_buf_alloc(ctx, (size_t)(batch * M * K * esz), &lt);
    if (!st) {
      int64_t dims[3] = {batch, K, M};
      int perm[3] = {0, 2, 1};
      st = hipnx_transpose(ctx, esz, 3, dims, perm, l, lt);
    }
  }
  if (!st && r_relay) {
    st = hipnx_buf_alloc(ctx, (size_t)(batch * N * K * esz), &rt);
    if (!st) {
      int64_t dims[3] = {batch, K, N};
      int perm[3] = {0, 2, 1};
      st = hipnx_transpose(ctx, esz, 3, dims, perm, r, rt);
    }
  }
  if (!st) {
    Enter in(ctx);
    st = in.status;
    // the lock was dropped for the re-layout above: the operands may have been freed meanwhile
    if (!st) st = check_buf(ctx, l, (uint64_t)batch * M * K * dtype_size(l_dt), "dot lhs");
    if (!st) st = check_buf(ctx, r, (uint64_t)batch * N * K * dtype_size(r_dt), "dot rhs");
    if (!st) st = check_buf(ctx, out, (uint64_t)batch * M * N * out_dtype_size(out_dt), "dot out");
    if (!st && scale_mode != HIPNX_SCALE_NONE) st = check_buf(ctx, scale, 4, "dot_scaled scale");
    if (!st) {
      const void *lp = lt ? lt->ptr : l->ptr, *rp = rt ? rt->ptr : r->ptr;
      if (pipelined) {
        const bool l_kin = l_layout == HIPNX_K_INNER || l_relay, r_kin = r_layout == HIPNX_K_INNER || r_relay;
        GemmArgs a{};
        a.l = (const unsigned char *)lp;
        a.r = (const unsigned char *)rp;
        a.out = out->ptr;
        a.odt = out_dt;
        a.M = M; a.N = N; a.Kb = Kb;
        a.ld_l = l_kin ? K * esz : M * esz;
        a.ld_r = r_kin ? K * esz : N * esz;
        a.bs_l = M * K * esz;
        a.bs_r = N * K * esz;
        a.scale = scale_mode != HIPNX_SCALE_NONE ? (const float *)scale->ptr : nullptr;
        a.scale_mode = scale_mode;
        // tile choice: the largest tile that still gives every CU work; few rows against a long
        // weight matrix stream the weights with many small tiles
        const int64_t t256 = ((M + 255) / 256) * ((N + 255) / 256) * batch;
        const int64_t t128 = ((M + 127) / 128) * ((N + 127) / 128);
        const int64_t tw = ((M + 255) / 256) * ((N + 127) / 128) * batch;
        const bool two_byte = l_dt == HIPNX_BF16 || l_dt == HIPNX_F16;
        const bool big_ok = M >= 192 && N >= 192;
        int cfg;
        // few rows: 64-row tiles (f32: whatever its cost model below picks), except for a 2-byte K-outer operand
        // (x . W with W stored [K, N]), which only the 128-row kernels read by transposing loads
        // (64 x 4096 x 4096 bf16: 72 us on 64 x 32 tiles, 16.5 us there)
        const bool wide = l_dt == HIPNX_F32 || l_dt == HIPNX_F64;  // (an f64 slab costs the matrix pipes what an f32 one does)
        if (M <= 64 && !wide && !(two_byte && !(l_kin && r_kin) && N >= 128)) cfg = GEMM_CFG_64x32;
        else if (t256 * 4 >= (int64_t)ctx->num_cus * 3 && big_ok) cfg = GEMM_CFG_256;
        else if (two_byte && M >= 192 && N >= 128 && t128 * batch > ctx->num_cus)
          // More 128 x 128 tiles than CUs: half-width tiles of the two-group kernel while they fit the CUs in one
          // round, even where they leave some idle (1280 x 4096 x 4096, 160 tiles: 66 us; as 320 tiles of
          // 128 x 128 in two rounds: 76 us); where they would need a second round, full tiles on what is then more
          // than half of the CUs (3072^3: 144 tiles of 256 x 256 72 us, 288 half-width tiles 100 us)
          cfg = tw <= ctx->num_cus || !big_ok ? GEMM_CFG_256x128 : GEMM_CFG_256;
        else if (l_dt == HIPNX_S8 && big_ok && t256 * 2 >= ctx->num_cus)
          cfg = GEMM_CFG_256;  // int8 has no half-width tile: full tiles from half of the CUs on (3072^3: 46 us against 57 us)
        else cfg = GEMM_CFG_128;
        // many rows against at most 32 columns (a layer with a few outputs): a 128-column tile would be three
        // quarters empty or more, and its MFMA work is what bounds f32
        if (N <= 32 && M > 64 && cfg == GEMM_CFG_128) cfg = GEMM_CFG_128x32;
        // A grid of 128 x 128 tiles that leaves three quarters of the CUs idle (a few hundred rows against a long
        // weight matrix: 128 x 4096 x 4096 is 32 tiles walking 64 slabs each) splits K over S work-groups per tile:
        // f32 (s32) partial results in pool workspace, then one pass that adds them in split order.
        int splits = 1;
        const int64_t nslab = Kb / SLAB;
        const bool splittable = (cfg == GEMM_CFG_128 || cfg == GEMM_CFG_128x32) && batch == 1 && scale_mode == HIPNX_SCALE_NONE && (M * N) % 4 == 0 &&
                                (l_dt == HIPNX_S8 ? !is_float(out_dt) : true) && l_dt != HIPNX_F64;  // (partial results are f32 / s32)
        if (wide && cfg == GEMM_CFG_128x32) {
          // (0.6 us per slab of a 128 x 32 tile; the split as below)
          const int64_t cus = ctx->num_cus, tiles = t128 * batch;
          double best = 10.0 + (double)((tiles + cus - 1) / cus) * (double)nslab * 0.6;
          if (splittable)
            for (int cand = 2; cand <= 64; cand *= 2) {
              if (tiles * cand > cus || nslab % cand != 0 || nslab / cand < 2) continue;
              const double t = 10.0 + (double)(nslab / cand) * 0.6 + 5.0 + 2.0 * (double)cand * (double)(M * N) * 4.0 / 8.0e6;
              if (t < best) { best = t; splits = cand; }
            }
        } else if (wide) {
          // An f32 slab is eight times the MFMA work of a 2-byte one (2.6 us per slab of a 128 x 128 tile, 0.55 us
          // for a 64 x 32 tile, the second pass of a split about 8 us), so a grid that leaves CUs idle is cut much
          // earlier: the cheapest, by those figures, of whole 128 x 128 tiles, K split up to 64 ways (2 slabs or
          // more each) and 64 x 32 tiles.  512^3: 41 -> 18 us; 256 x 256 x 16384: 84 -> 40 us.
          if (cfg == GEMM_CFG_128) {
            const int64_t cus = ctx->num_cus;
            auto rounds = [&](int64_t groups) { return (double)((groups + cus - 1) / cus); };
            double best = 10.0 + rounds(t128 * batch) * (double)nslab * 2.6;
            // second launch, then the partial results written and read once (mostly from cache: ~8 MB per us)
            auto split_cost = [&](int cand) { return 5.0 + 2.0 * (double)cand * (double)(M * N) * 4.0 / 8.0e6; };
            if (splittable)
              for (int cand = 2; cand <= 64; cand *= 2) {
                if (t128 * cand > cus || nslab % cand != 0 || nslab / cand < 2) continue;
                const double t = 10.0 + (double)(nslab / cand) * 2.6 + split_cost(cand);
                if (t < best) { best = t; splits = cand; }
              }
            // tiles of 64 x 128, half the MFMA work per slab: up to 64 rows a 128-row tile would be half empty, and a grid
            // of 128 x 128 tiles whose last round leaves most CUs idle ends sooner in halves (3072^3: 576 tiles in three
            // rounds, 1152 in five of half the length)
            {
              const int64_t tn = ((M + 63) / 64) * ((N + 127) / 128) * batch;
              const double whole = 10.0 + rounds(tn) * (double)nslab * 1.3;
              if (whole < best) { best = whole; cfg = GEMM_CFG_64x128; splits = 1; }
              if (splittable)
                for (int cand = 2; cand <= 64; cand *= 2) {
                  if (tn * cand > cus || nslab % cand != 0 || nslab / cand < 2) continue;
                  const double t = 10.0 + (double)(nslab / cand) * 1.3 + split_cost(cand);
                  if (t < best) { best = t; cfg = GEMM_CFG_64x128; splits = cand; }
                }
            }
            const int64_t t64 = ((M + 63) / 64) * ((N + 31) / 32) * batch;
            if (10.0 + rounds(t64) * (double)nslab * 0.55 < best) { cfg = GEMM_CFG_64x32; splits = 1; }
          }
        } else if (splittable && t128 * 2 <= ctx->num_cus && nslab >= (t128 * 4 <= ctx->num_cus ? 32 : 64))
          // (the second pass and the partial results cost about 10 us: worth it from K = 32 slabs on -- 64 where
          // the grid already covers more than a quarter of the CUs -- with at least 8 slabs left per split and no
          // more work-groups than CUs; 1024 x 2048 x 2048, 128 tiles of 32 slabs, is faster whole: 21 us against
          // 22 us in two halves and 27 us in four quarters)
          for (int cand = 16; cand >= 2; cand /= 2)
            if (t128 * cand <= (int64_t)ctx->num_cus && nslab % cand == 0 && nslab / cand >= 8) { splits = cand; break; }
        void *ws = nullptr;
        size_t ws_cap = 0;
        if (splits > 1 && pool_alloc(ctx, (size_t)splits * M * N * 4, &ws, &ws_cap) != HIPNX_OK) splits = 1;
        if (splits > 1) {
          GemmArgs p = a;
          p.Kb = Kb / splits;
          p.bs_l = l_kin ? p.Kb : (p.Kb / esz) * a.ld_l;  // split s begins p.Kb bytes (or that many k-rows) further on
          p.bs_r = r_kin ? p.Kb : (p.Kb / esz) * a.ld_r;
          p.out = ws;
          p.odt = l_dt == HIPNX_S8 ? HIPNX_S32 : HIPNX_F32;
          switch (l_dt) {
            case HIPNX_BF16: st = launch_gemm_bf16(ctx, cfg, l_kin, r_kin, p, splits); break;
            case HIPNX_F16: st = launch_gemm_f16(ctx, cfg, l_kin, r_kin, p, splits); break;
            case HIPNX_F32: st = launch_gemm_f32(ctx, cfg, l_kin, r_kin, p, splits); break;
            case HIPNX_F64: st = launch_gemm_f64(ctx, cfg, l_kin, r_kin, p, splits); break;
            default: st = launch_gemm_s8(ctx, cfg, l_kin, r_kin, p, splits); break;
          }
          if (!st) {
            const int64_t mn = M * N;
            dim3 grid((unsigned)std::min<int64_t>((mn / 4 + 255) / 256, 1 << 20)), block(256);
            if (l_dt == HIPNX_S8) hipLaunchKernelGGL((splitk_combine_kernel<int>), grid, block, 0, ctx->stream, (const int *)ws, out->ptr, out_dt, mn, splits);
            else hipLaunchKernelGGL((splitk_combine_kernel<float>), grid, block, 0, ctx->stream, (const float *)ws, out->ptr, out_dt, mn, splits);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) st = hip_fail(e, "split-K combine launch");
          }
          pool_free(ctx, ws, ws_cap);  // later work is ordered on the same stream
        } else
        switch (l_dt) {
          case HIPNX_BF16: st = launch_gemm_bf16(ctx, cfg, l_kin, r_kin, a, batch); break;
          case HIPNX_F16: st = launch_gemm_f16(ctx, cfg, l_kin, r_kin, a, batch); break;
          case HIPNX_F32: st = launch_gemm_f32(ctx, cfg, l_kin, r_kin, a, batch); break;
          case HIPNX_F64: st = launch_gemm_f64(ctx, cfg, l_kin, r_kin, a, batch); break;
          default: st = launch_gemm_s8(ctx, cfg, l_kin, r_kin, a, batch); break;
        }
      } else {
        switch (l_dt) {
          case HIPNX_BF16: launch_mfma<HIPNX_BF16>(ctx, lp, rp, out->ptr, out_dt, batch, M, N, Kb); break;
          case HIPNX_F16: launch_mfma<HIPNX_F16>(ctx, lp, rp, out->ptr, out_dt, batch, M, N, Kb); break;
          case HIPNX_F32: launch_mfma<HIPNX_F32>(ctx, lp, rp, out->ptr, out_dt, batch, M, N, Kb); break;
          default: launch_mfma<HIPNX_S8>(ctx, lp, rp, out->ptr, out_dt, batch, M, N, Kb); break;
        }
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) st = hip_fail(e, "gemm launch");
      }
    }
  }
  // handing the workspaces back to the pool is safe: later work is ordered on the same stream
  if (lt) hipnx_buf_destroy(lt);
  if (rt) hipnx_buf_destroy(rt);
  return st;
}

extern "C" int hipnx_dot(hipnx_ctx *ctx, int l_dt, int r_dt, int out_dt, int64_t batch, int64_t M, int64_t N,
                         int64_t K, int l_layout, int r_layout, const hipnx_buf *l, const hipnx_buf *r,
                         hipnx_buf *out) {
  return dot_impl(ctx, l_dt, r_dt, out_dt, batch, M, N, K, l_layout, r_layout, l, r, out, HIPNX_SCALE_NONE, nullptr);
}

extern "C" int hipnx_dot_scaled(hipnx_ctx *ctx, int l_dt, int r_dt, int64_t batch, int64_t M, int64_t N, int64_t K,
                                int l_layout, int r_layout, const hipnx_buf *l, const hipnx_buf *r, int scale_mode,
                                const hipnx_buf *scale, hipnx_buf *out) {
  if (scale_mode != HIPNX_SCALE_PER_COLUMN && scale_mode != HIPNX_SCALE_PER_ROW && scale_mode != HIPNX_SCALE_ONE)
    return set_error(HIPNX_EINVAL, "dot_scaled: scale mode %d", scale_mode);
  return dot_impl(ctx, l_dt, r_dt, HIPNX_F32, batch, M, N, K, l_layout, r_layout, l, r, out, scale_mode, scale);
}
