// Data movement: fill (constant), transpose, broadcast, gather / take.  Pure byte copies -- the
// bit patterns of the source survive unchanged (NaN payloads included), as in the reference,
// where these callbacks only slice and concatenate binaries
// (nx/lib/nx/binary_backend.ex:215-319, 1902-1959).
#include <cstring>

#include "dtypes.cuh"
#include "internal.h"

namespace hipnx {

constexpr int BLOCK = 256;
constexpr int MAXR = 8;

template <typename T>
__global__ void __launch_bounds__(BLOCK) fill_kernel(T *__restrict__ out, T value, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < n; i += (int64_t)gridDim.x * BLOCK) out[i] = value;
}

struct Strided {
  int rank;
  int64_t dims[MAXR];     // output extents
  int64_t strides[MAXR];  // input stride (elements) per output axis
};

// out[i] = in[sum c_a * stride_a]; one element per lane per step
template <typename T>
__global__ void __launch_bounds__(BLOCK)
strided_copy_kernel(const T *__restrict__ in, T *__restrict__ out, int64_t n, Strided s) {
  for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < n; i += (int64_t)gridDim.x * BLOCK) {
    int64_t rem = i, off = 0;
    for (int a = s.rank - 1; a >= 0; a--) {
      int64_t q = rem / s.dims[a];
      off += (rem - q * s.dims[a]) * s.strides[a];
      rem = q;
    }
    out[i] = in[off];
  }
}

// batched 2-D transpose through an LDS tile: in [B, R, C] -> out [B, C, R].  The 64x64 tile is
// read with lanes along C and written with lanes along R, so both sides are coalesced; the
// +1 padding keeps the transposed LDS reads off a single bank.
template <typename T>
__global__ void __launch_bounds__(BLOCK)
transpose2d_kernel(const T *__restrict__ in, T *__restrict__ out, int64_t R, int64_t C, int64_t tiles_r,
                   int64_t tiles_c) {
  constexpr int TILE = 64;
  __shared__ T tile[TILE][TILE + 1];
  int64_t t = blockIdx.x;
  const int64_t tc = t % tiles_c;
  t /= tiles_c;
  const int64_t tr = t % tiles_r, b = t / tiles_r;
  const T *src = in + b * R * C;
  T *dst = out + b * R * C;
  const int tx = threadIdx.x % TILE, ty = threadIdx.x / TILE;  // 64 x 4
  for (int j = ty; j < TILE; j += BLOCK / TILE) {
    int64_t r = tr * TILE + j, c = tc * TILE + tx;
    if (r < R && c < C) tile[j][tx] = src[r * C + c];
  }
  __syncthreads();
  for (int j = ty; j < TILE; j += BLOCK / TILE) {
    int64_t c = tc * TILE + j, r = tr * TILE + tx;
    if (r < R && c < C) dst[c * R + r] = tile[tx][j];
  }
}

// The same with 16-byte accesses on both sides, for R and C that are multiples of 16 / sizeof(T) elements
// and 16-byte aligned buffers: a lane loads V = 16 / sizeof(T) elements along C (a tile row is 128 bytes or
// more: whole cache lines), the tile goes to LDS row by row with an odd pitch in words, and a lane then
// collects V elements down a column -- V consecutive elements of an output row -- and stores them as one
// 16-byte vector; lanes run along the output row, so a store instruction writes whole lines too.  The
// one-element-per-lane kernel above moves 128 bytes (2-byte elements) per wave instruction.
template <typename T>
__global__ void __launch_bounds__(BLOCK)
transpose2d_vec_kernel(const T *__restrict__ in, T *__restrict__ out, int64_t R, int64_t C, int64_t tiles_r,
                       int64_t tiles_c, int64_t total) {
  constexpr int S = sizeof(T), V = 16 / S, TILE = S <= 2 ? 128 : 64, CH = TILE / V;  // CH vectors per tile row
  constexpr int PITCH = TILE * S / 4 + (S == 8 ? 2 : 1);                           // words per tile row in LDS
  constexpr int RPP = BLOCK / CH;                                                    // tile rows per pass
  constexpr int NLD = TILE / RPP;                                                    // vectors a lane loads per tile
  extern __shared__ uint32_t lds[];  // TILE * PITCH words
  // Tile order: bands of BAND tile rows walked column by column, so that the work-groups in flight at one time cover
  // a compact block of tiles (runs of several tile widths on the input rows they read and on the output rows they
  // write).  A work-group walks tiles blockIdx.x, blockIdx.x + gridDim.x, ..: the next tile's vectors are requested
  // right after this tile's have gone to LDS, so its loads are in flight while this tile is turned and stored --
  // with one tile per work-group a CU alternated between a phase of loads and a phase of stores and the memory
  // system saw half as many requests in flight as it takes (bf16 16384^2: 4.2 TB/s against 6.1 for a plain copy).
  constexpr int BAND = 8;
  const int64_t per_matrix = tiles_r * tiles_c, per_band = BAND * tiles_c;
  const int q = threadIdx.x % CH, j0 = threadIdx.x / CH;
  auto locate = [&](int64_t t, int64_t &b, int64_t &tr, int64_t &tc) {
    b = t / per_matrix;
    t -= b * per_matrix;
    const int64_t first = (t / per_band) * BAND;
    const int64_t rows = tiles_r - first < BAND ? tiles_r - first : BAND, within = t % per_band;
    tr = first + within % rows;
    tc = within / rows;
  };
  uint4 v[NLD];
  auto fetch = [&](int64_t t) {
    int64_t b, tr, tc;
    locate(t, b, tr, tc);
    const T *src = in + b * R * C;
#pragma unroll
    for (int p = 0; p < NLD; p++) {
      const int64_t r = tr * TILE + j0 + p * RPP, c = tc * TILE + q * V;
      if (r < R && c < C) v[p] = *reinterpret_cast<const uint4 *>(src + r * C + c);
    }
  };
  int64_t t = blockIdx.x;
  if (t < total) fetch(t);
  for (; t < total; t += gridDim.x) {
    int64_t b, tr, tc;
    locate(t, b, tr, tc);
    T *dst = out + b * R * C;
#pragma unroll
    for (int p = 0; p < NLD; p++) {
      uint32_t *w = lds + (j0 + p * RPP) * PITCH + q * 4;
      w[0] = v[p].x; w[1] = v[p].y; w[2] = v[p].z; w[3] = v[p].w;
    }
    __syncthreads();
    if (t + gridDim.x < total) fetch(t + gridDim.x);
    if constexpr (S >= 4) {
      const T *cell = reinterpret_cast<const T *>(lds);
#pragma unroll
      for (int p = 0; p < NLD; p++) {
        const int cc = j0 + p * RPP;  // tile column = output row
        const int64_t c = tc * TILE + cc, r = tr * TILE + q * V;
        if (c < C && r < R) {
          T e[V];
#pragma unroll
          for (int k = 0; k < V; k++) e[k] = cell[(size_t)(q * V + k) * (PITCH * 4 / S) + cc];
          *reinterpret_cast<uint4 *>(dst + c * R + r) = *reinterpret_cast<const uint4 *>(e);
        }
      }
    } else {
      // elements narrower than a word: a lane reads whole words down a group of G = 4 / S adjacent columns
      // (V word reads instead of G * V element reads) and takes them apart into G output vectors
      constexpr int G = 4 / S;
#pragma unroll
      for (int p = 0; p < TILE / (RPP * G); p++) {
        const int cg = j0 + p * RPP;  // group of G tile columns = G output rows
        const int64_t c = tc * TILE + (int64_t)cg * G, r = tr * TILE + q * V;
        if (c < C && r < R) {
          uint32_t w[V];
#pragma unroll
          for (int k = 0; k < V; k++) w[k] = lds[(q * V + k) * PITCH + cg];
#pragma unroll
          for (int g = 0; g < G; g++) {
            uint32_t o[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
              uint32_t x = 0;
#pragma unroll
              for (int e = 0; e < G; e++) x |= ((w[i * G + e] >> (8 * S * g)) & ((1u << (8 * S)) - 1u)) << (8 * S * e);
              o[i] = x;
            }
            if (c + g < C) *reinterpret_cast<uint4 *>(dst + (c + g) * R + r) = *reinterpret_cast<const uint4 *>(o);
          }
        }
      }
    }
    __syncthreads();  // the tile has left LDS before the next one enters
  }
}

// gather: tuple i of `idx` ([n_tuples, depth]) selects a slice of `slice_bytes` bytes.
// LPR lanes (a power of two, at most one wavefront) copy one slice with W-byte accesses (W = 16 where the
// slices are whole 16-byte vectors, else the widest of 8, 4, 2, 1 that divides them: the element of a
// gather of single elements), four independent accesses in flight per lane; a 256-lane block works on 256/LPR
// slices at once so that the index -> address -> data dependency of one slice overlaps with the
// others'.  flag[0] receives the smallest (tuple * depth + axis) whose index is out of range, and the
// pinned host word `host_seen` is set so that the host learns of it without a copy.
// `period` > 0 is take along an axis with axes before it: output slice i is (o, j) = (i / period, i % period), the
// index is idx[j] for every o, and the source moves on by `outer_bytes` per o.
template <int W>
__global__ void __launch_bounds__(BLOCK)
gather_kernel(const unsigned char *__restrict__ t, const void *__restrict__ idx, unsigned char *__restrict__ out,
              int idx_dt, int64_t n_tuples, int depth, Strided tdims /* dims = leading extents, strides = bytes */,
              int64_t slice_bytes, int lpr, int clamp, unsigned long long *__restrict__ flag,
              unsigned int *__restrict__ host_seen, unsigned long long *__restrict__ deferred, int64_t period,
              int64_t outer_bytes) {
  typedef raw_vec<W> vec_t;
  const int64_t chunks = slice_bytes / W;
  const int rpb = BLOCK / lpr;
  const int sub = threadIdx.x / lpr, lane = threadIdx.x % lpr;
  for (int64_t row = (int64_t)blockIdx.x * rpb + sub; row < n_tuples; row += (int64_t)gridDim.x * rpb) {
    int64_t off = 0, irow = row;
    if (period > 0) {
      const int64_t o = row / period;
      irow = row - o * period;
      off = o * outer_bytes;
    }
    bool ok = true;
    for (int a = 0; a < depth; a++) {
      int64_t v = load_one<int64_t>(idx, idx_dt, irow * depth + a);
      const int64_t dim = tdims.dims[a];
      bool oob = v < 0 || v >= dim || (idx_dt == HIPNX_U64 && (uint64_t)v >= (uint64_t)dim);
      if (oob) {
        if (clamp) v = (v < 0 && idx_dt != HIPNX_U64) ? 0 : dim - 1;
        else {
          ok = false;
          if (lane == 0) {
            if (deferred) {  // the policy that reports late: code 6 (HIPNX_RAISE_INDEX) and the offending index
              __hip_atomic_store(deferred, (6ull << 56) | ((unsigned long long)v & 0x00FFFFFFFFFFFFFFull), __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_SYSTEM);
            } else {
              atomicMin(flag, (unsigned long long)(irow * depth + a));
              __hip_atomic_store(host_seen, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);  // pinned host word
            }
          }
          break;
        }
      }
      off += v * tdims.strides[a];
    }
    if (!ok) continue;
    const vec_t *src = reinterpret_cast<const vec_t *>(t + off);
    vec_t *dst = reinterpret_cast<vec_t *>(out + row * slice_bytes);
    int64_t c = lane;
    for (; c + 3 * (int64_t)lpr < chunks; c += 4 * (int64_t)lpr) {
      vec_t v0 = src[c], v1 = src[c + lpr], v2 = src[c + 2 * lpr], v3 = src[c + 3 * lpr];
      dst[c] = v0; dst[c + lpr] = v1; dst[c + 2 * lpr] = v2; dst[c + 3 * lpr] = v3;
    }
    for (; c < chunks; c += lpr) dst[c] = src[c];
  }
}

// gather of slices of SB = 1, 2, 4 or 8 bytes (single elements), launched for take along the innermost axis with
// rows before it (`period` > 0), whose reads stay within a row: one lane per 16-byte vector of the OUTPUT (8
// bytes for SB = 1), i.e. S = 16 / SB slices, so that the row number is taken apart once per S slices, the
// S reads are in flight together and the store is whole.  With one slice per lane, take along the last axis
// of 4096^2 f32 ran at 1.4 TB/s although every read hits a line its neighbours fetched.  The slices of one vector are walked by incrementing (o, j), which also
// covers a vector that crosses into the next `o`.  A vector with a rejected index (or the partial last
// one) is stored slice by slice.
template <int SB>
__global__ void __launch_bounds__(BLOCK)
gather_small_kernel(const unsigned char *__restrict__ t, const void *__restrict__ idx, unsigned char *__restrict__ out,
                    int idx_dt, int64_t n_tuples, int depth, Strided tdims, int clamp,
                    unsigned long long *__restrict__ flag, unsigned int *__restrict__ host_seen,
                    unsigned long long *__restrict__ deferred, int64_t period, int64_t outer_bytes) {
  typedef raw_vec<SB> el_t;
  constexpr int S = SB == 1 ? 8 : 16 / SB, VB = S * SB;  // 8 slices at most: the offsets are 64-bit registers
  const int64_t nvec = (n_tuples + S - 1) / S;
  for (int64_t v = (int64_t)blockIdx.x * BLOCK + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * BLOCK) {
    const int64_t row0 = v * S;
    int64_t o = 0, j = row0;
    if (period > 0) {
      if (row0 < (1ll << 31) && period < (1ll << 31)) o = (uint32_t)row0 / (uint32_t)period;
      else o = row0 / period;
      j = row0 - o * period;
    }
    // all S index tuples first (axis by axis, S loads in flight), then the S reads: the memory counter retires in
    // order, so a read issued between two index loads would be waited for with the second
    int64_t jj[S], off[S];
    unsigned okmask = 0;
#pragma unroll
    for (int s = 0; s < S; s++) {
      jj[s] = j;
      off[s] = o * outer_bytes;
      if (row0 + s < n_tuples) okmask |= 1u << s;
      if (period > 0) {
        if (++j == period) { j = 0; o++; }
      } else j++;
    }
    for (int a = 0; a < depth; a++) {
      const int64_t dim = tdims.dims[a], stride = tdims.strides[a];
      int64_t x[S];
#pragma unroll
      for (int s = 0; s < S; s++) x[s] = (okmask >> s & 1u) ? load_one<int64_t>(idx, idx_dt, jj[s] * depth + a) : 0;
#pragma unroll
      for (int s = 0; s < S; s++) {
        const bool oob = x[s] < 0 || x[s] >= dim || (idx_dt == HIPNX_U64 && (uint64_t)x[s] >= (uint64_t)dim);
        if (oob) {
          if (clamp) x[s] = (x[s] < 0 && idx_dt != HIPNX_U64) ? 0 : dim - 1;
          else {
            okmask &= ~(1u << s);
            if (deferred) {
              __hip_atomic_store(deferred, (6ull << 56) | ((unsigned long long)x[s] & 0x00FFFFFFFFFFFFFFull), __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_SYSTEM);
            } else {
              atomicMin(flag, (unsigned long long)(jj[s] * depth + a));
              __hip_atomic_store(host_seen, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            }
            x[s] = 0;
          }
        }
        off[s] += x[s] * stride;
      }
    }
    alignas(16) el_t e[S];
#pragma unroll
    for (int s = 0; s < S; s++)
      if (okmask >> s & 1u) e[s] = *reinterpret_cast<const el_t *>(t + off[s]);
    if (okmask == (1u << S) - 1u) {
      *reinterpret_cast<raw_vec<VB> *>(out + row0 * SB) = *reinterpret_cast<const raw_vec<VB> *>(e);
    } else {
#pragma unroll
      for (int s = 0; s < S; s++)
        if (okmask >> s & 1u) *reinterpret_cast<el_t *>(out + (row0 + s) * SB) = e[s];
    }
  }
}

// take along the innermost axis with the source row staged in LDS: t [outer, axis_len], out [outer, n_idx],
// elements of SB bytes.  Through the vector memory path a wave's 64 reads of scattered elements of one row
// cost one cache line each (the kernel above stays near 1-2 TB/s on rows of 16 KB and drops with longer
// ones); here a work-group copies the row in with whole-line loads, the scattered reads go to LDS banks,
// and the stores are 16-byte vectors.  Needs row and output row sizes that are multiples of 16 bytes and
// 16-byte aligned buffers; a group walks rows o = blockIdx.x, blockIdx.x + gridDim.x, ...
constexpr int TAKE_ROW_BLOCK = 512;
template <int SB>
__global__ void __launch_bounds__(TAKE_ROW_BLOCK)
take_row_lds_kernel(const unsigned char *__restrict__ t, const void *__restrict__ idx, unsigned char *__restrict__ out,
                    int idx_dt, int64_t outer, int64_t axis_len, int64_t n_idx, int clamp,
                    unsigned long long *__restrict__ flag, unsigned int *__restrict__ host_seen,
                    unsigned long long *__restrict__ deferred) {
  typedef raw_vec<SB> el_t;
  constexpr int S = 16 / SB;
  extern __shared__ uint4 take_row_lds[];
  const el_t *cell = reinterpret_cast<const el_t *>(take_row_lds);
  const int64_t row_vecs = axis_len * SB / 16, out_vecs = n_idx / S;
  for (int64_t o = blockIdx.x; o < outer; o += gridDim.x) {
    const uint4 *src = reinterpret_cast<const uint4 *>(t + o * axis_len * SB);
    __syncthreads();  // the reads of the row before are done
    for (int64_t c = threadIdx.x; c < row_vecs; c += TAKE_ROW_BLOCK) take_row_lds[c] = src[c];
    __syncthreads();
    for (int64_t v = threadIdx.x; v < out_vecs; v += TAKE_ROW_BLOCK) {
      alignas(16) el_t e[S];
      unsigned okmask = 0;
      int64_t x[S];
      if (idx_dt == HIPNX_S32 || idx_dt == HIPNX_U32) {  // S indices as loads of up to 16 bytes
        alignas(16) uint32_t raw[S];
        constexpr int CH = S * 4 < 16 ? S * 4 : 16;  // bytes per load
#pragma unroll
        for (int q = 0; q < S * 4 / CH; q++)
          *reinterpret_cast<raw_vec<CH> *>(raw + q * (CH / 4)) = reinterpret_cast<const raw_vec<CH> *>(idx)[v * (S * 4 / CH) + q];
#pragma unroll
        for (int s = 0; s < S; s++) x[s] = idx_dt == HIPNX_S32 ? (int64_t)(int32_t)raw[s] : (int64_t)raw[s];
      } else {
#pragma unroll
        for (int s = 0; s < S; s++) x[s] = load_one<int64_t>(idx, idx_dt, v * S + s);
      }
#pragma unroll
      for (int s = 0; s < S; s++) {
        int64_t xi = x[s];
        bool ok = true;
        if (xi < 0 || xi >= axis_len || (idx_dt == HIPNX_U64 && (uint64_t)xi >= (uint64_t)axis_len)) {
          if (clamp) xi = (xi < 0 && idx_dt != HIPNX_U64) ? 0 : axis_len - 1;
          else {
            ok = false;
            if (deferred) {
              __hip_atomic_store(deferred, (6ull << 56) | ((unsigned long long)xi & 0x00FFFFFFFFFFFFFFull), __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_SYSTEM);
            } else {
              atomicMin(flag, (unsigned long long)(v * S + s));
              __hip_atomic_store(host_seen, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            }
          }
        }
        if (ok) {
          e[s] = cell[xi];
          okmask |= 1u << s;
        }
      }
      unsigned char *dst = out + (o * n_idx + v * S) * SB;
      if (okmask == (1u << S) - 1u) {
        *reinterpret_cast<raw_vec<16> *>(dst) = *reinterpret_cast<const raw_vec<16> *>(e);
      } else {
#pragma unroll
        for (int s = 0; s < S; s++)
          if (okmask >> s & 1u) *reinterpret_cast<el_t *>(dst + s * SB) = e[s];
      }
    }
  }
}

// The same with one 16-byte vector of the OUTPUT per lane, for an innermost output axis that is a multiple of
// V = 16 / sizeof(T) elements (`s.dims[rank - 1]` counts vectors here): the index is taken apart once per
// vector, the V inputs are one 16-byte load (inner stride 1, aligned), one element repeated (inner stride 0:
// a column or a scalar broadcast along rows) or V loads, and the store is whole.  One element per lane is
// bound by instructions, not bytes: broadcasting to 16384^2 took 335-500 us whatever the element size.
template <typename T>
__global__ void __launch_bounds__(BLOCK)
strided_copy_vec_kernel(const T *__restrict__ in, T *__restrict__ out, int64_t nvec, Strided s, int64_t inner_stride) {
  constexpr int V = 16 / sizeof(T);
  for (int64_t v = (int64_t)blockIdx.x * BLOCK + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * BLOCK) {
    int64_t rem = v, off = 0;
    for (int a = s.rank - 1; a >= 0; a--) {
      int64_t q, c;
      if (rem < (1ll << 31) && s.dims[a] < (1ll << 31)) { q = (uint32_t)rem / (uint32_t)s.dims[a]; c = (uint32_t)rem - (uint32_t)q * (uint32_t)s.dims[a]; }
      else { q = rem / s.dims[a]; c = rem - q * s.dims[a]; }
      off += c * s.strides[a] * (a == s.rank - 1 ? V : 1);
      rem = q;
    }
    T e[V];
    if (inner_stride == 1 && ((reinterpret_cast<uintptr_t>(in + off)) & 15) == 0) {
      *reinterpret_cast<uint4 *>(e) = *reinterpret_cast<const uint4 *>(in + off);
    } else if (inner_stride == 0) {
      const T x = in[off];
#pragma unroll
      for (int k = 0; k < V; k++) e[k] = x;
    } else {
#pragma unroll
      for (int k = 0; k < V; k++) e[k] = in[off + k * inner_stride];
    }
    *reinterpret_cast<uint4 *>(out + v * V) = *reinterpret_cast<const uint4 *>(e);
  }
}

// The same for an innermost output axis that is NOT a multiple of V (broadcasting a column along rows of 50257
// elements): vectors of the flat output, which may run across row ends.  A lane takes its first element's index
// apart, walks along the innermost axis and takes the index apart again only where a row ends.  The last vector
// may be partial.  (One element per lane: 2.0 TB/s on that broadcast.)
template <typename T>
__global__ void __launch_bounds__(BLOCK)
strided_copy_flat_kernel(const T *__restrict__ in, T *__restrict__ out, int64_t n, Strided s) {
  constexpr int V = 16 / sizeof(T);
  const int64_t nvec = (n + V - 1) / V, inner = s.dims[s.rank - 1], istride = s.strides[s.rank - 1];
  for (int64_t v = (int64_t)blockIdx.x * BLOCK + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * BLOCK) {
    const int64_t i0 = v * V;
    int64_t base = 0, c = 0;
    auto locate = [&](int64_t i) {  // base = offset of the outer coordinates of flat index i, c = its innermost one
      int64_t rem = i;
      base = 0;
      for (int a = s.rank - 1; a >= 0; a--) {
        int64_t q, r;
        if (rem < (1ll << 31) && s.dims[a] < (1ll << 31)) { q = (uint32_t)rem / (uint32_t)s.dims[a]; r = (uint32_t)rem - (uint32_t)q * (uint32_t)s.dims[a]; }
        else { q = rem / s.dims[a]; r = rem - q * s.dims[a]; }
        if (a == s.rank - 1) c = r;
        else base += r * s.strides[a];
        rem = q;
      }
    };
    locate(i0);
    T e[V];
    const int nel = i0 + V <= n ? V : (int)(n - i0);
#pragma unroll
    for (int k = 0; k < V; k++) {
      if (k < nel) {
        e[k] = in[base + c * istride];
        if (++c == inner && k + 1 < nel) locate(i0 + k + 1);
      }
    }
    if (nel == V) *reinterpret_cast<uint4 *>(out + i0) = *reinterpret_cast<const uint4 *>(e);
    else
      for (int k = 0; k < nel; k++) out[i0 + k] = e[k];
  }
}

// 16 bytes of the repeated element per lane
__global__ void __launch_bounds__(BLOCK) fill16_kernel(uint4 *__restrict__ out, uint4 pattern, int64_t nvec) {
  for (int64_t i = (int64_t)blockIdx.x * BLOCK + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * BLOCK) out[i] = pattern;
}

static int grid_for(const hipnx_ctx *ctx, int64_t items, int per_block) {
  int64_t blocks = (items + per_block - 1) / per_block;
  (void)ctx;
  int64_t cap = ((1ll << 32) - 1) / BLOCK;  // cover the whole index space (faster here than a resident grid that loops) up to the 2^32 - 1 lanes a launch may hold
  if (blocks < 1) blocks = 1;
  return (int)(blocks < cap ? blocks : cap);
}

template <typename T>
static void launch_strided(const hipnx_ctx *ctx, const void *in, void *out, int64_t n, const Strided &s) {
  constexpr int V = 16 / (int)sizeof(T);
  if (s.rank >= 1 && s.dims[s.rank - 1] % V == 0 && ((uintptr_t)out & 15) == 0) {
    Strided sv = s;
    sv.dims[s.rank - 1] /= V;
    hipLaunchKernelGGL((strided_copy_vec_kernel<T>), dim3(grid_for(ctx, n / V, BLOCK)), dim3(BLOCK), 0, ctx->stream,
                       (const T *)in, (T *)out, n / V, sv, s.strides[s.rank - 1]);
    return;
  }
  if (s.rank >= 1 && n >= 4 * V && ((uintptr_t)out & 15) == 0) {
    hipLaunchKernelGGL((strided_copy_flat_kernel<T>), dim3(grid_for(ctx, (n + V - 1) / V, BLOCK)), dim3(BLOCK), 0, ctx->stream,
                       (const T *)in, (T *)out, n, s);
    return;
  }
  hipLaunchKernelGGL((strided_copy_kernel<T>), dim3(grid_for(ctx, n, BLOCK)), dim3(BLOCK), 0, ctx->stream,
                     (const T *)in, (T *)out, n, s);
}

static int strided_copy(const hipnx_ctx *ctx, int elem_bytes, const void *in, void *out, int64_t n, const Strided &s) {
  switch (elem_bytes) {
    case 1: launch_strided<uint8_t>(ctx, in, out, n, s); break;
    case 2: launch_strided<uint16_t>(ctx, in, out, n, s); break;
    case 4: launch_strided<uint32_t>(ctx, in, out, n, s); break;
    case 8: launch_strided<uint64_t>(ctx, in, out, n, s); break;
    default: return set_error(HIPNX_EINVAL, "element size %d is not 1, 2, 4 or 8", elem_bytes);
  }
  return HIPNX_OK;
}

template <typename T>
static void launch_t2d(const hipnx_ctx *ctx, const void *in, void *out, int64_t B, int64_t R, int64_t C) {
  constexpr int V = 16 / (int)sizeof(T), TILE = sizeof(T) <= 2 ? 128 : 64;
  if (R % V == 0 && C % V == 0 && (((uintptr_t)in | (uintptr_t)out) & 15) == 0) {
    const int64_t vr = (R + TILE - 1) / TILE, vc = (C + TILE - 1) / TILE;
    // as many work-groups as their LDS tiles allow to be resident (33 KiB for 1- and 2-byte elements, 16.5 KiB
    // above), each walking its share of the tiles
    constexpr int lds_bytes = TILE * (TILE * (int)sizeof(T) / 4 + (sizeof(T) == 8 ? 2 : 1)) * 4;
    const int64_t total = B * vr * vc, resident = (int64_t)ctx->num_cus * (160 * 1024 / lds_bytes);
    auto kern = transpose2d_vec_kernel<T>;
    if (lds_bytes > 64 * 1024) {
      hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
      if (e != hipSuccess) return;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)(total < resident ? total : resident)), dim3(BLOCK), lds_bytes, ctx->stream,
                       (const T *)in, (T *)out, R, C, vr, vc, total);
    return;
  }
  int64_t tr = (R + 63) / 64, tc = (C + 63) / 64;
  hipLaunchKernelGGL((transpose2d_kernel<T>), dim3((unsigned)(B * tr * tc)), dim3(BLOCK), 0, ctx->stream,
                     (const T *)in, (T *)out, R, C, tr, tc);
}

}  // namespace hipnx

using namespace hipnx;

extern "C" int hipnx_fill(hipnx_ctx *ctx, hipnx_buf *dst, int elem_bytes, const void *elem, int64_t n) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (!elem || n < 0) return set_error(HIPNX_EINVAL, "fill: null element or negative count");
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8)
    return set_error(HIPNX_EINVAL, "fill: element size %d is not 1, 2, 4 or 8", elem_bytes);
  if (int st = check_buf(ctx, dst, (uint64_t)n * elem_bytes, "fill dst")) return st;
  if (n == 0) return HIPNX_OK;
  // whole 16-byte vectors of the repeated element first, then what is left (fewer than 16 bytes) by element
  const int64_t nvec = ((uintptr_t)dst->ptr & 15) == 0 ? n * elem_bytes / 16 : 0;
  if (nvec > 0) {
    unsigned char pat[16];
    for (int i = 0; i < 16; i += elem_bytes) std::memcpy(pat + i, elem, (size_t)elem_bytes);
    uint4 pattern;
    std::memcpy(&pattern, pat, 16);
    hipLaunchKernelGGL(fill16_kernel, dim3(grid_for(ctx, nvec, BLOCK)), dim3(BLOCK), 0, ctx->stream, (uint4 *)dst->ptr, pattern, nvec);
    const int64_t done = nvec * 16 / elem_bytes;
    if (done == n) { HIPNX_HIP(hipGetLastError()); return HIPNX_OK; }
    // the tail: fewer than 16 / elem_bytes elements
    unsigned char *tail = (unsigned char *)dst->ptr + nvec * 16;
    const int64_t left = n - done;
    dim3 g1(1), block1(BLOCK);
    switch (elem_bytes) {
      case 1: hipLaunchKernelGGL((fill_kernel<uint8_t>), g1, block1, 0, ctx->stream, (uint8_t *)tail, *(const uint8_t *)elem, left); break;
      case 2: { uint16_t v; std::memcpy(&v, elem, 2); hipLaunchKernelGGL((fill_kernel<uint16_t>), g1, block1, 0, ctx->stream, (uint16_t *)tail, v, left); break; }
      case 4: { uint32_t v; std::memcpy(&v, elem, 4); hipLaunchKernelGGL((fill_kernel<uint32_t>), g1, block1, 0, ctx->stream, (uint32_t *)tail, v, left); break; }
      default: { uint64_t v; std::memcpy(&v, elem, 8); hipLaunchKernelGGL((fill_kernel<uint64_t>), g1, block1, 0, ctx->stream, (uint64_t *)tail, v, left); break; }
    }
    HIPNX_HIP(hipGetLastError());
    return HIPNX_OK;
  }
  dim3 grid(grid_for(ctx, n, BLOCK)), block(BLOCK);
  switch (elem_bytes) {
    case 1: hipLaunchKernelGGL((fill_kernel<uint8_t>), grid, block, 0, ctx->stream, (uint8_t *)dst->ptr, *(const uint8_t *)elem, n); break;
    case 2: { uint16_t v; std::memcpy(&v, elem, 2); hipLaunchKernelGGL((fill_kernel<uint16_t>), grid, block, 0, ctx->stream, (uint16_t *)dst->ptr, v, n); break; }
    case 4: { uint32_t v; std::memcpy(&v, elem, 4); hipLaunchKernelGGL((fill_kernel<uint32_t>), grid, block, 0, ctx->stream, (uint32_t *)dst->ptr, v, n); break; }
    default: { uint64_t v; std::memcpy(&v, elem, 8); hipLaunchKernelGGL((fill_kernel<uint64_t>), grid, block, 0, ctx->stream, (uint64_t *)dst->ptr, v, n); break; }
  }
  HIPNX_HIP(hipGetLastError());
  return HIPNX_OK;
}

extern "C" int hipnx_transpose(hipnx_ctx *ctx, int elem_bytes, int rank, const int64_t *in_dims, const int *perm,
                               const hipnx_buf *inb, hipnx_buf *out) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (rank < 0 || rank > 64 || (rank > 0 && (!in_dims || !perm))) return set_error(HIPNX_EINVAL, "transpose: bad rank");
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8)
    return set_error(HIPNX_EINVAL, "transpose: element size %d is not 1, 2, 4 or 8", elem_bytes);
  int64_t n = 1;
  uint64_t seen = 0;
  for (int a = 0; a < rank; a++) {
    if (in_dims[a] < 0) return set_error(HIPNX_EINVAL, "transpose: negative dimension");
    if (perm[a] < 0 || perm[a] >= rank || (seen >> perm[a] & 1)) return set_error(HIPNX_EINVAL, "transpose: not a permutation");
    seen |= 1ull << perm[a];
    n *= in_dims[a];
  }
  if (int st = check_buf(ctx, inb, (uint64_t)n * elem_bytes, "transpose in")) return st;
  if (int st = check_buf(ctx, out, (uint64_t)n * elem_bytes, "transpose out")) return st;
  if (n == 0) return HIPNX_OK;
  // input strides, then walk the output axes: drop unit axes, merge output neighbours that are
  // also neighbours (in order) in the input
  int64_t in_str[64];
  int64_t s = 1;
  for (int a = rank - 1; a >= 0; a--) { in_str[a] = s; s *= in_dims[a]; }
  int64_t dims[64], str[64];
  int m = 0;
  for (int a = 0; a < rank; a++) {
    int64_t d = in_dims[perm[a]], st = in_str[perm[a]];
    if (d == 1) continue;
    if (m > 0 && str[m - 1] == st * d) { dims[m - 1] *= d; str[m - 1] = st; }
    else { dims[m] = d; str[m] = st; m++; }
  }
  if (m <= 1) {  // the permutation moves nothing in memory
    HIPNX_HIP(hipMemcpyAsync(out->ptr, inb->ptr, (size_t)n * elem_bytes, hipMemcpyDeviceToDevice, ctx->stream));
    return HIPNX_OK;
  }
  // [B, R, C] -> [B, C, R] : out axes (B?, C, R) with strides (R*C, 1, C)
  bool two_d = (m == 2 && str[0] == 1 && str[1] == dims[0]) ||
               (m == 3 && str[1] == 1 && str[2] == dims[1] && str[0] == dims[1] * dims[2]);
  if (two_d) {
    int64_t B = m == 3 ? dims[0] : 1, C = dims[m - 2], R = dims[m - 1];
    if (B * ((R + 63) / 64) * ((C + 63) / 64) < (1ll << 31)) {
      switch (elem_bytes) {
        case 1: launch_t2d<uint8_t>(ctx, inb->ptr, out->ptr, B, R, C); break;
        case 2: launch_t2d<uint16_t>(ctx, inb->ptr, out->ptr, B, R, C); break;
        case 4: launch_t2d<uint32_t>(ctx, inb->ptr, out->ptr, B, R, C); break;
        default: launch_t2d<uint64_t>(ctx, inb->ptr, out->ptr, B, R, C); break;
      }
      HIPNX_HIP(hipGetLastError());
      return HIPNX_OK;
    }
  }
  if (m > MAXR) return set_error(HIPNX_EUNSUPPORTED, "transpose: more than %d non-collapsible axes", MAXR);
  Strided sd;
  sd.rank = m;
  for (int q = 0; q < m; q++) { sd.dims[q] = dims[q]; sd.strides[q] = str[q]; }
  if (int st = strided_copy(ctx, elem_bytes, inb->ptr, out->ptr, n, sd)) return st;
  HIPNX_HIP(hipGetLastError());
  return HIPNX_OK;
}

extern "C" int hipnx_broadcast(hipnx_ctx *ctx, int elem_bytes, int rank, const int64_t *out_dims,
                               const int64_t *in_strides, const hipnx_buf *inb, hipnx_buf *out) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (rank < 0 || rank > 64 || (rank > 0 && (!out_dims || !in_strides))) return set_error(HIPNX_EINVAL, "broadcast: bad rank");
  int64_t n = 1, ext = 1;
  for (int a = 0; a < rank; a++) {
    if (out_dims[a] < 0 || in_strides[a] < 0) return set_error(HIPNX_EINVAL, "broadcast: negative dimension or stride");
    n *= out_dims[a];
  }
  if (n > 0)
    for (int a = 0; a < rank; a++) ext += (out_dims[a] - 1) * in_strides[a];
  if (int st = check_buf(ctx, inb, n > 0 ? (uint64_t)ext * elem_bytes : 0, "broadcast in")) return st;
  if (int st = check_buf(ctx, out, (uint64_t)n * elem_bytes, "broadcast out")) return st;
  if (n == 0) return HIPNX_OK;
  int64_t dims[64], str[64];
  int m = 0;
  for (int a = 0; a < rank; a++) {
    int64_t d = out_dims[a], st = in_strides[a];
    if (d == 1) continue;
    if (m > 0 && str[m - 1] == st * d) { dims[m - 1] *= d; str[m - 1] = st; }
    else { dims[m] = d; str[m] = st; m++; }
  }
  if (m == 0) { dims[0] = 1; str[0] = 0; m = 1; }
  if (m > MAXR) return set_error(HIPNX_EUNSUPPORTED, "broadcast: more than %d non-collapsible axes", MAXR);
  Strided sd;
  sd.rank = m;
  for (int q = 0; q < m; q++) { sd.dims[q] = dims[q]; sd.strides[q] = str[q]; }
  if (int st = strided_copy(ctx, elem_bytes, inb->ptr, out->ptr, n, sd)) return st;
  HIPNX_HIP(hipGetLastError());
  return HIPNX_OK;
}

// launch and, under the raising policy, the wait and the reference's message; `n_tuples` output slices, whose
// index tuples are idx[i] (period = 0) or idx[i % period] (take along an axis with `outer` axes before it).
// `msg_dims[rank]` is the shape the message names (the tensor with its indexed axes leading).
static int gather_run(hipnx_ctx *ctx, int idx_dt, int64_t n_tuples, int depth, int oob_policy, const hipnx_buf *t,
                      const hipnx_buf *idx, hipnx_buf *out, const Strided &td, int64_t slice_bytes, int64_t period,
                      int64_t outer_bytes, int rank, const int64_t *t_dims) {
  // bounds report: a device word that stays all-ones until a kernel finds a bad index (it is set
  // when the context is created and re-armed below after a failure), so the common path needs
  // no launch to clear it
  unsigned long long *flag = (unsigned long long *)ctx->flag;
  const int width = slice_bytes % 16 == 0 ? 16 : slice_bytes % 8 == 0 ? 8 : slice_bytes % 4 == 0 ? 4 : slice_bytes % 2 == 0 ? 2 : 1;
  int64_t chunks = slice_bytes / width;
  int lpr = 64;  // lanes per slice: at most one wavefront, fewer for short slices
  while (lpr > 1 && lpr / 2 >= chunks) lpr >>= 1;
  dim3 grid(grid_for(ctx, n_tuples, BLOCK / lpr)), block(BLOCK);
#define HIPNX_GATHER(W) hipLaunchKernelGGL((gather_kernel<W>), grid, block, 0, ctx->stream, (const unsigned char *)t->ptr, idx->ptr, \
                                          (unsigned char *)out->ptr, idx_dt, n_tuples, depth, td, slice_bytes, lpr, (int)(oob_policy == HIPNX_OOB_CLAMP), flag, \
                                          (unsigned int *)ctx->flag_host_dev, oob_policy == HIPNX_OOB_DEFER ? deferred_error_word(ctx) : nullptr, period, outer_bytes)
#define HIPNX_GATHER_SMALL(SB) hipLaunchKernelGGL((gather_small_kernel<SB>), dim3(grid_for(ctx, (n_tuples + (SB == 1 ? 8 : 16 / SB) - 1) / (SB == 1 ? 8 : 16 / SB), BLOCK)), block, 0, \
                                                 ctx->stream, (const unsigned char *)t->ptr, idx->ptr, (unsigned char *)out->ptr, idx_dt, n_tuples, depth, td, \
                                                 (int)(oob_policy == HIPNX_OOB_CLAMP), flag, (unsigned int *)ctx->flag_host_dev, \
                                                 oob_policy == HIPNX_OOB_DEFER ? deferred_error_word(ctx) : nullptr, period, outer_bytes)
  bool launched = false;
  // take along the innermost axis (one index per slice, rows before it) with rows of 2 to 128 KB, at least half
  // as many picks as the row has elements and a row per compute unit or more: the row goes through LDS
  {
    const int64_t row_bytes = td.dims[0] * slice_bytes;
    const bool lds_rows = depth == 1 && period > 0 && slice_bytes <= 8 && slice_bytes == width && outer_bytes == row_bytes &&
                          row_bytes >= 2048 && row_bytes <= 128 * 1024 && row_bytes % 16 == 0 && (period * slice_bytes) % 16 == 0 &&
                          period * 2 >= td.dims[0] && n_tuples / period >= ctx->num_cus &&
                          ((reinterpret_cast<uintptr_t>(out->ptr) | reinterpret_cast<uintptr_t>(t->ptr) | reinterpret_cast<uintptr_t>(idx->ptr)) & 15) == 0;
    if (lds_rows) {
      const int64_t outer = n_tuples / period;
      const int per_cu = row_bytes <= 32 * 1024 ? 4 : row_bytes <= 64 * 1024 ? 2 : 1;
      const unsigned blocks = (unsigned)std::min<int64_t>(outer, (int64_t)ctx->num_cus * per_cu * 2);
#define HIPNX_TAKE_ROW(SB)                                                                                                        \
  do {                                                                                                                            \
    auto kern = take_row_lds_kernel<SB>;                                                                                          \
    HIPNX_ALLOW_DYNAMIC_LDS(ctx, kern, 128 * 1024);                                                                               \
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(TAKE_ROW_BLOCK), (size_t)row_bytes, ctx->stream, (const unsigned char *)t->ptr,   \
                       idx->ptr, (unsigned char *)out->ptr, idx_dt, outer, td.dims[0], period, (int)(oob_policy == HIPNX_OOB_CLAMP), \
                       flag, (unsigned int *)ctx->flag_host_dev, oob_policy == HIPNX_OOB_DEFER ? deferred_error_word(ctx) : nullptr); \
  } while (0)
      switch (width) {
        case 8: HIPNX_TAKE_ROW(8); break;
        case 4: HIPNX_TAKE_ROW(4); break;
        case 2: HIPNX_TAKE_ROW(2); break;
        default: HIPNX_TAKE_ROW(1); break;
      }
#undef HIPNX_TAKE_ROW
      launched = true;
    }
  }
  // single elements picked along an axis with rows before it (reads that stay within a row, which the caches hold);
  // picks scattered over the whole tensor (gather with a full tuple, take from a vector) are bound by the misses in
  // flight and do better with one slice per lane: 8M f32 out of 64 MB took 155 us that way, 187 us this way
  const bool small = period > 0 && slice_bytes <= 8 && slice_bytes == width && (reinterpret_cast<uintptr_t>(out->ptr) & 15) == 0;
  if (launched) {
  } else if (small) {
    switch (width) {
      case 8: HIPNX_GATHER_SMALL(8); break;
      case 4: HIPNX_GATHER_SMALL(4); break;
      case 2: HIPNX_GATHER_SMALL(2); break;
      default: HIPNX_GATHER_SMALL(1); break;
    }
  } else
  switch (width) {
    case 16: HIPNX_GATHER(16); break;
    case 8: HIPNX_GATHER(8); break;
    case 4: HIPNX_GATHER(4); break;
    case 2: HIPNX_GATHER(2); break;
    default: HIPNX_GATHER(1); break;
  }
#undef HIPNX_GATHER
#undef HIPNX_GATHER_SMALL
  HIPNX_HIP(hipGetLastError());
  if (oob_policy == HIPNX_OOB_RAISE) {
    // the reference raises on the first offending index: wait, then report it the same way.
    // The kernel marks a pinned host word when it meets one, so the good path costs the wait only.
    volatile unsigned int *seen = (volatile unsigned int *)ctx->flag_host;
    HIPNX_HIP(hipStreamSynchronize(ctx->stream));
    if (seen[0] == 0) return deferred_error(ctx);  // nothing of this call; something recorded earlier surfaces here
    if (seen[0] != 0) {
      unsigned long long first = ~0ull;
      HIPNX_HIP(hipMemcpy(&first, flag, 8, hipMemcpyDeviceToHost));
      const int64_t pos = (int64_t)first;
      seen[0] = 0;
      HIPNX_HIP(hipMemsetAsync(flag, 0xFF, 8, ctx->stream));  // re-arm
      const int axis = (int)(pos % depth);
      unsigned char raw[8] = {0};
      const int isz = dtype_size(idx_dt);
      HIPNX_HIP(hipMemcpy(raw, (const char *)idx->ptr + pos * isz, isz, hipMemcpyDeviceToHost));
      long long v = 0;
      switch (idx_dt) {
        case HIPNX_U8: v = *(uint8_t *)raw; break;
        case HIPNX_U16: { uint16_t x; std::memcpy(&x, raw, 2); v = x; break; }
        case HIPNX_U32: { uint32_t x; std::memcpy(&x, raw, 4); v = x; break; }
        case HIPNX_S8: v = *(int8_t *)raw; break;
        case HIPNX_S16: { int16_t x; std::memcpy(&x, raw, 2); v = x; break; }
        case HIPNX_S32: { int32_t x; std::memcpy(&x, raw, 4); v = x; break; }
        default: { int64_t x; std::memcpy(&x, raw, 8); v = x; break; }
      }
      char shape[256] = "{";
      for (int q = 0; q < rank; q++) {
        char one[32];
        snprintf(one, sizeof one, q ? ", %lld" : "%lld", (long long)t_dims[q]);
        strncat(shape, one, sizeof shape - strlen(shape) - 2);
      }
      strcat(shape, "}");
      if (idx_dt == HIPNX_U64)
        return set_error(HIPNX_EINDEX, "index %llu is out of bounds for axis %d in shape %s", (unsigned long long)v, axis, shape);
      return set_error(HIPNX_EINDEX, "index %lld is out of bounds for axis %d in shape %s", v, axis, shape);
    }
  }
  return HIPNX_OK;
}

// Indices the library wrote itself as positions along an axis no longer than the one they now address (the result
// of hipnx_argreduce, untouched since, read as the type it was written in) cannot be out of range: the raising
// policy then has nothing to wait for.  The kernel still checks them and records a violation for the next wait
// (the late-raising policy), so a wrong claim would surface instead of passing silently.
static bool indices_known_in_range(const hipnx_buf *idx, int idx_dt, uint64_t idx_bytes, int depth, int64_t axis_len) {
  return depth == 1 && idx->index_bound > 0 && idx->index_dt == idx_dt && idx->index_bytes >= idx_bytes && idx->index_bound <= axis_len;
}

extern "C" int hipnx_gather(hipnx_ctx *ctx, int elem_bytes, int rank, const int64_t *t_dims, int idx_dt,
                            int64_t n_tuples, int depth, int oob_policy, const hipnx_buf *t, const hipnx_buf *idx,
                            hipnx_buf *out) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (rank < 0 || rank > 64 || depth < 0 || depth > rank || depth > MAXR || n_tuples < 0 || (rank > 0 && !t_dims))
    return set_error(HIPNX_EINVAL, "gather: bad rank / depth");
  if (elem_bytes <= 0 || dtype_size(idx_dt) < 0 || is_float(idx_dt))
    return set_error(HIPNX_EINVAL, "gather: indices must be an integer type");
  if (oob_policy != HIPNX_OOB_RAISE && oob_policy != HIPNX_OOB_CLAMP && oob_policy != HIPNX_OOB_DEFER)
    return set_error(HIPNX_EINVAL, "gather: bad policy");
  int64_t total = 1, slice = 1;
  for (int a = 0; a < rank; a++) {
    if (t_dims[a] < 0) return set_error(HIPNX_EINVAL, "gather: negative dimension");
    total *= t_dims[a];
    if (a >= depth) slice *= t_dims[a];
  }
  const int64_t slice_bytes = slice * elem_bytes;
  if (int st = check_buf(ctx, t, (uint64_t)total * elem_bytes, "gather tensor")) return st;
  if (int st = check_buf(ctx, idx, (uint64_t)n_tuples * depth * dtype_size(idx_dt), "gather indices")) return st;
  if (int st = check_buf(ctx, out, (uint64_t)n_tuples * slice_bytes, "gather out")) return st;
  if (oob_policy == HIPNX_OOB_RAISE && rank > 0 &&
      indices_known_in_range(idx, idx_dt, (uint64_t)n_tuples * depth * dtype_size(idx_dt), depth, t_dims[0]))
    oob_policy = HIPNX_OOB_DEFER;
  if (oob_policy == HIPNX_OOB_RAISE) HIPNX_NOT_CAPTURING(ctx, "gather with the raising bounds policy");
  if (n_tuples == 0 || slice_bytes == 0) return HIPNX_OK;
  if (total == 0) {
    if (oob_policy == HIPNX_OOB_CLAMP) return set_error(HIPNX_EINVAL, "gather: cannot clamp into an empty tensor");
    return set_error(HIPNX_EINDEX, "gather: index into an empty tensor");
  }
  Strided td;
  td.rank = depth;
  {
    int64_t s = slice_bytes;
    for (int a = depth - 1; a >= 0; a--) { td.dims[a] = t_dims[a]; td.strides[a] = s; s *= t_dims[a]; }
  }
  return gather_run(ctx, idx_dt, n_tuples, depth, oob_policy, t, idx, out, td, slice_bytes, 0, 0, rank, t_dims);
}

// concatenate: parts [outer, a_i, inner] -> out [outer, sum a_i, inner], up to 64 parts per launch (their pointers
// and where each begins within a row of the output travel as kernel arguments).  One launch per part cost 6 us of
// host time each: 64 parts of 2 MiB 425 us, 256 small ones 1.5 ms.
constexpr int CONCAT_PARTS = 64;
struct ConcatArgs {
  const unsigned char *src[CONCAT_PARTS];
  int64_t begin[CONCAT_PARTS + 1];  // bytes from the start of an output row to the part (last entry: end of the last part)
  int n;
};

template <int W>
__global__ void __launch_bounds__(BLOCK)
concat_kernel(ConcatArgs a, unsigned char *__restrict__ out, int64_t outer, int64_t row_bytes) {
  typedef raw_vec<W> vec_t;
  const int64_t first = a.begin[0], span = a.begin[a.n] - first;  // this launch's share of an output row
  const int64_t per_row = span / W, total = outer * per_row;
  for (int64_t v = (int64_t)blockIdx.x * BLOCK + threadIdx.x; v < total; v += (int64_t)gridDim.x * BLOCK) {
    const int64_t o = v / per_row, within = first + (v - o * per_row) * W;
    int lo = 0, hi = a.n - 1;  // the last part that begins at or before `within`
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (a.begin[mid] <= within) lo = mid;
      else hi = mid - 1;
    }
    const int64_t len = a.begin[lo + 1] - a.begin[lo];
    *reinterpret_cast<vec_t *>(out + o * row_bytes + within) =
        *reinterpret_cast<const vec_t *>(a.src[lo] + o * len + (within - a.begin[lo]));
  }
}

extern "C" int hipnx_concat(hipnx_ctx *ctx, int elem_bytes, int n_parts, const hipnx_buf *const *parts, const int64_t *extents,
                            int64_t outer, int64_t inner, hipnx_buf *out) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (elem_bytes <= 0 || n_parts < 0 || outer < 0 || inner < 0 || (n_parts > 0 && (!parts || !extents)))
    return set_error(HIPNX_EINVAL, "concat: bad argument");
  int64_t sum = 0;
  for (int p = 0; p < n_parts; p++) {
    if (extents[p] < 0) return set_error(HIPNX_EINVAL, "concat: negative extent");
    if (int st = check_buf(ctx, parts[p], (uint64_t)outer * extents[p] * inner * elem_bytes, "concat part")) return st;
    sum += extents[p];
  }
  const int64_t row_bytes = sum * inner * elem_bytes;
  if (int st = check_buf(ctx, out, (uint64_t)outer * row_bytes, "concat out")) return st;
  if (outer * row_bytes == 0) return HIPNX_OK;
  // the widest access that every part's row and address allows
  int width = 16;
  uintptr_t bits = reinterpret_cast<uintptr_t>(out->ptr) | (uintptr_t)row_bytes;
  for (int p = 0; p < n_parts; p++)
    if (extents[p] > 0) bits |= reinterpret_cast<uintptr_t>(parts[p]->ptr) | (uintptr_t)(extents[p] * inner * elem_bytes);
  while (width > 1 && (bits & (uintptr_t)(width - 1))) width >>= 1;
  int64_t begin = 0;
  int p = 0;
  while (p < n_parts) {
    ConcatArgs a;
    a.n = 0;
    while (p < n_parts && a.n < CONCAT_PARTS) {
      if (extents[p] > 0) {
        a.src[a.n] = (const unsigned char *)parts[p]->ptr;
        a.begin[a.n] = begin;
        a.n++;
        begin += extents[p] * inner * elem_bytes;
      }
      p++;
    }
    if (a.n == 0) break;
    a.begin[a.n] = begin;
    const int64_t total = outer * ((a.begin[a.n] - a.begin[0]) / width);
    dim3 grid(grid_for(ctx, total, BLOCK)), block(BLOCK);
    switch (width) {
      case 16: hipLaunchKernelGGL((concat_kernel<16>), grid, block, 0, ctx->stream, a, (unsigned char *)out->ptr, outer, row_bytes); break;
      case 8: hipLaunchKernelGGL((concat_kernel<8>), grid, block, 0, ctx->stream, a, (unsigned char *)out->ptr, outer, row_bytes); break;
      case 4: hipLaunchKernelGGL((concat_kernel<4>), grid, block, 0, ctx->stream, a, (unsigned char *)out->ptr, outer, row_bytes); break;
      case 2: hipLaunchKernelGGL((concat_kernel<2>), grid, block, 0, ctx->stream, a, (unsigned char *)out->ptr, outer, row_bytes); break;
      default: hipLaunchKernelGGL((concat_kernel<1>), grid, block, 0, ctx->stream, a, (unsigned char *)out->ptr, outer, row_bytes); break;
    }
  }
  HIPNX_HIP(hipGetLastError());
  return HIPNX_OK;
}

extern "C" int hipnx_take(hipnx_ctx *ctx, int elem_bytes, int64_t outer, int64_t axis_len, int64_t inner, int idx_dt,
                          int64_t n_idx, int oob_policy, int rank, const int64_t *msg_dims, const hipnx_buf *t,
                          const hipnx_buf *idx, hipnx_buf *out) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (elem_bytes <= 0 || dtype_size(idx_dt) < 0 || is_float(idx_dt)) return set_error(HIPNX_EINVAL, "take: indices must be an integer type");
  if (outer < 0 || axis_len < 0 || inner < 0 || n_idx < 0 || rank < 0 || rank > 64 || (rank > 0 && !msg_dims))
    return set_error(HIPNX_EINVAL, "take: negative extent or bad rank");
  if (oob_policy != HIPNX_OOB_RAISE && oob_policy != HIPNX_OOB_CLAMP && oob_policy != HIPNX_OOB_DEFER)
    return set_error(HIPNX_EINVAL, "take: bad policy");
  const int64_t slice_bytes = inner * elem_bytes;
  if (int st = check_buf(ctx, t, (uint64_t)outer * axis_len * slice_bytes, "take tensor")) return st;
  if (int st = check_buf(ctx, idx, (uint64_t)n_idx * dtype_size(idx_dt), "take indices")) return st;
  if (int st = check_buf(ctx, out, (uint64_t)outer * n_idx * slice_bytes, "take out")) return st;
  if (oob_policy == HIPNX_OOB_RAISE && indices_known_in_range(idx, idx_dt, (uint64_t)n_idx * dtype_size(idx_dt), 1, axis_len))
    oob_policy = HIPNX_OOB_DEFER;
  if (oob_policy == HIPNX_OOB_RAISE) HIPNX_NOT_CAPTURING(ctx, "take with the raising bounds policy");
  if (outer * n_idx == 0 || slice_bytes == 0) return HIPNX_OK;
  if (axis_len == 0) {
    if (oob_policy == HIPNX_OOB_CLAMP) return set_error(HIPNX_EINVAL, "take: cannot clamp into an empty axis");
    return set_error(HIPNX_EINDEX, "take: index into an empty axis");
  }
  Strided td;
  td.rank = 1;
  td.dims[0] = axis_len;
  td.strides[0] = slice_bytes;
  return gather_run(ctx, idx_dt, outer * n_idx, 1, oob_policy, t, idx, out, td, slice_bytes, outer > 1 ? n_idx : 0,
                    axis_len * slice_bytes, rank, msg_dims);
}
