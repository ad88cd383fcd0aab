// Pipelined MFMA contraction kernel  out[b, m, n] = sum_k l[b, m, k] * r[b, n, k]  for gfx950.
//
// Work-group tile BM x BN = (WM*TM*32) x (WN*TN*32): WM x WN wavefronts, each owning
// 2TM x 2TN MFMA tiles of 16 x 16 whose accumulators stay in registers for the whole K walk.
// (Under the power cap the 16x16 MFMA shapes sustain 10-20 % more than the 32x32 ones with the
// same operands, and the f32 16x16x4 form almost 1.5x the 32x32x2 form.)
//
// K is walked in slabs of 128 bytes per row (64 bf16/f16, 128 s8, 32 f32): one full cache line
// per row, the granularity at which a CU ingests L2-resident data fastest (half lines halve it).
// LDS holds NSTAGE stages of one slab each (BM + BN rows x 128 B).
//   K-inner operand ([rows, K], K contiguous): `global_load_lds_dwordx4` -- each lane moves 16 B
//     straight from global memory into LDS, no VGPR round trip.  A wave instruction fills 1 KiB of
//     LDS (8 rows x 8 chunks); the lane picks the *global* chunk that belongs at its LDS slot.
//     LDS layout: row-major, 128 B per row, the 16-byte chunk index XOR-ed with
//     ((row ^ row>>3) & 7): conflict-free for the fragment reads (16 consecutive rows, one chunk)
//     and for the transposed writes below (rows 8 apart, one chunk).
//   K-outer operand ([K, rows], rows contiguous), 2-byte elements, tiles of 128 rows or more: the
//     slab is copied k-major with the same direct-to-LDS loads and the fragment is built by the
//     transposing LDS read `ds_read_b64_tr_b16`.
//   K-outer operand otherwise: each lane loads a small k x rows block with 16-byte row loads,
//     transposes it in registers (byte permutes) and writes K-runs into the K-inner LDS layout.
//   Either way a plain `Nx.dot(a, b)` needs no re-layout pass.
// Fragments: for one 64-byte K-step a lane's MFMA operand is chunk (4*step + lane/16) of row
// (lane%16) -- 8 bf16/f16, 16 s8 or 4 f32 (fed to four 16x16x4 MFMAs; both operands use the same
// k <-> slot map).  The MFMA is issued with the r-fragment as its first operand so that a lane
// ends up with 4 consecutive n per accumulator: the epilogue stores 4 outputs at a time.
#pragma once
#include <type_traits>

#include "dtypes.cuh"

namespace hipnx {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

constexpr int SLAB = 128;          // bytes of K per row per slab
constexpr int CHUNKS = SLAB / 16;  // 16-byte chunks per row

template <int DT> struct Mma;
template <> struct Mma<HIPNX_BF16> {
  typedef v16f acc_t;
  static __device__ __forceinline__ void step(acc_t &c, const v4i &a, const v4i &b) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
  }
};
template <> struct Mma<HIPNX_F16> {
  typedef v16f acc_t;
  static __device__ __forceinline__ void step(acc_t &c, const v4i &a, const v4i &b) {
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
  }
};
template <> struct Mma<HIPNX_S8> {
  typedef v16i acc_t;
  static __device__ __forceinline__ void step(acc_t &c, const v4i &a, const v4i &b) {
    c = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
  }
};
template <> struct Mma<HIPNX_F32> {
  typedef v16f acc_t;
  static __device__ __forceinline__ void step(acc_t &c, const v4i &a, const v4i &b) {
#pragma unroll
    for (int s = 0; s < 4; s++)
      c = __builtin_amdgcn_mfma_f32_32x32x2f32(__int_as_float(a[s]), __int_as_float(b[s]), c, 0, 0, 0);
  }
};

typedef float v4f __attribute__((ext_vector_type(4)));

// 16x16 MFMA forms used by the pipelined kernel (one 16-byte operand chunk per lane and step)
template <int DT> struct Mma16;
template <> struct Mma16<HIPNX_BF16> {
  typedef v4f acc_t;
  static __device__ __forceinline__ void step(acc_t &c, const v4i &a, const v4i &b) {
    c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
  }
};
template <> struct Mma16<HIPNX_F16> {
  typedef v4f acc_t;
  static __device__ __forceinline__ void step(acc_t &c, const v4i &a, const v4i &b) {
    c = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
  }
};
template <> struct Mma16<HIPNX_S8> {
  typedef v4i acc_t;
  static __device__ __forceinline__ void step(acc_t &c, const v4i &a, const v4i &b) {
    c = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
  }
};
template <> struct Mma16<HIPNX_F32> {
  typedef v4f acc_t;
  static __device__ __forceinline__ void step(acc_t &c, const v4i &a, const v4i &b) {
#pragma unroll
    for (int s = 0; s < 4; s++)
      c = __builtin_amdgcn_mfma_f32_16x16x4f32(__int_as_float(a[s]), __int_as_float(b[s]), c, 0, 0, 0);
  }
};

// f64: a lane's 16 bytes are two consecutive k; v_mfma_f64_16x16x4_f64 takes one value per lane (k = lane / 16), so the
// two instructions contract k = {0, 2, 4, 6} and {1, 3, 5, 7} of the 8-k step.  Its result sits differently from the
// other types' (measured on the part): register e of lane l is row 4 e + l / 16 of the first operand, column l % 16.
typedef double v4d __attribute__((ext_vector_type(4)));
typedef double v2d __attribute__((ext_vector_type(2)));
template <> struct Mma16<HIPNX_F64> {
  typedef v4d acc_t;
  static __device__ __forceinline__ void step(acc_t &c, const v4i &a, const v4i &b) {
    const v2d x = __builtin_bit_cast(v2d, a), y = __builtin_bit_cast(v2d, b);
    c = __builtin_amdgcn_mfma_f64_16x16x4f64(x[0], y[0], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f64_16x16x4f64(x[1], y[1], c, 0, 0, 0);
  }
};

// Swizzle of the [row][k] LDS layout: 16-byte chunk index XOR a 3-bit function of the row.  Its
// part in the low four row bits (bit0 = r0^r2, bit1 = r1^r2, bit2 = r2^r3) is one of the maps a
// sweep over all linear maps of those bits measured as conflict-free for the fragment read
// (16 consecutive rows x 4 chunks per ds_read_b128: 4 clocks per instruction instead of 8); row
// bits 4..6 are constant within a fragment and are mixed in for the transposed writes of the
// register-staged operands, whose lanes hold rows 4, 8 or 16 apart.
__device__ __forceinline__ int lds_slot(int row, int chunk) {
  const int low = ((row ^ (row >> 2)) & 1) | ((((row >> 1) ^ (row >> 2)) & 1) << 1) | ((((row >> 2) ^ (row >> 3)) & 1) << 2);
  return chunk ^ low ^ ((row >> 4) & 7);
}

typedef __attribute__((address_space(3))) void *lptr_t;

// One direct-to-LDS load: every lane moves 16 bytes from its global address to
// LDS[lds_base + 16 * lane] (lds_base wave-uniform, carried in M0).  Written as inline assembly
// rather than through the compiler's builtin on purpose: after the builtin the compiler no
// longer trusts the in-order return of LDS reads and turns every partial lgkmcnt(n) wait of the
// fragment pipeline into lgkmcnt(0).  The compiler therefore does not count these loads: the
// kernel waits for them itself (wait_vmcnt) before the barrier that publishes a slab; the
// compiler's own vmcnt waits only become stricter by loads it does not know of.
__device__ __forceinline__ void lds_dma16(const unsigned char *g, unsigned char *lds) {
  const unsigned base = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(lptr_t)lds);
  // (M0 is named as clobbered so that the compiler re-initialises it for its own uses; the
  // diagnostic about reserved registers in a clobber list is expected)
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(base) : "memory", "m0");
#pragma clang diagnostic pop
}

// K-inner slab loader: ROWS x 128 B, direct to LDS.  The per-lane source pointers (row clamp,
// row * stride, swizzled chunk) are computed once; per slab only the K offset moves.
// Rows past `rows_valid` are clamped (loaded from the last valid row; their results are never
// stored).
template <int ROWS, int NWAVES>
struct KInnerLoader {
  static constexpr int INSTR = ROWS / 8;  // wave instructions per slab (1 KiB of LDS each)
  static constexpr int PER = INSTR / NWAVES;
  static_assert(INSTR % NWAVES == 0, "slab rows must split evenly over the waves");
  const unsigned char *src[PER];
  int lds_off[PER];

  __device__ __forceinline__ void init(const unsigned char *__restrict__ g, int64_t ld, int64_t row0, int64_t rows_valid,
                                       int wave, int lane) {
#pragma unroll
    for (int i = 0; i < PER; i++) {
      const int t = wave + NWAVES * i;
      const int r = t * 8 + (lane >> 3);
      const int chunk = lds_slot(r, lane & 7);  // the XOR map is an involution: slot -> chunk
      int64_t gr = row0 + r;
      gr = gr < rows_valid ? gr : rows_valid - 1;
      src[i] = g + gr * ld + chunk * 16;
      lds_off[i] = t * 1024;
    }
  }
  __device__ __forceinline__ void issue(int64_t kbyte0, unsigned char *lds) const {
#pragma unroll
    for (int i = 0; i < PER; i++)
      lds_dma16(src[i] + kbyte0, lds + lds_off[i]);
  }
  // instruction i of the slab goes out at step i * spread / PER + phase (+ skew, which may be a
  // run-time value); with t, spread and phase known after unrolling the tests fold away
  __device__ __forceinline__ void issue_at(int t, int spread, int phase, int skew, int64_t kbyte0, unsigned char *lds) const {
#pragma unroll
    for (int i = 0; i < PER; i++)
      if (t == i * spread / PER + phase + skew) lds_dma16(src[i] + kbyte0, lds + lds_off[i]);
  }
};

// ---- K-outer operands: g is [K, rows] (rows contiguous).  A lane loads a small block of
// 16-byte row runs at consecutive k, transposes it in registers and writes K-runs into the same
// [row][k] LDS layout the K-inner loader produces.  Block shape per element size ES:
//   ES = 2:  8 k x  8 rows -> eight 16-byte K-runs (v_perm_b32 pairs halves)
//   ES = 4:  4 k x  4 rows -> four 16-byte K-runs (pure register renaming)
//   ES = 1:  4 k x 16 rows -> sixteen 4-byte K-runs (4 x 4 byte transposes with v_perm_b32)
// `rows_valid` must be a multiple of the block's row count (the host falls back to a transpose
// pass otherwise); k never runs past K because K*ES is a multiple of the slab.
template <int ES> struct KOuterShape;
template <> struct KOuterShape<2> { static constexpr int KB = 8, RB = 8; };
template <> struct KOuterShape<4> { static constexpr int KB = 4, RB = 4; };
template <> struct KOuterShape<1> { static constexpr int KB = 4, RB = 16; };
template <> struct KOuterShape<8> { static constexpr int KB = 2, RB = 2; };

template <int ES, int ROWS, int NTHREADS>
struct KOuterStage {
  static constexpr int KB = KOuterShape<ES>::KB, RB = KOuterShape<ES>::RB;
  static constexpr int KSLAB = SLAB / ES;                       // k values per slab
  static constexpr int BLOCKS = (ROWS / RB) * (KSLAB / KB);
  static constexpr int PER = (BLOCKS + NTHREADS - 1) / NTHREADS;
  static constexpr int LOADS = PER * KB;                        // vector-memory ops per slab per lane
  v4i v[PER][KB];

  __device__ __forceinline__ void fetch(const unsigned char *__restrict__ g, int64_t ld, int64_t row0, int64_t rows_valid,
                                        int64_t k0, int tid) {
#pragma unroll
    for (int p = 0; p < PER; p++) {
      const int blk = tid + p * NTHREADS;
      if (blk >= BLOCKS) break;
      const int rb = blk % (ROWS / RB), kb = blk / (ROWS / RB);
      int64_t col = row0 + rb * RB;
      col = col + RB <= rows_valid ? col : rows_valid - RB;  // tile rows past the edge: any valid run
#pragma unroll
      for (int j = 0; j < KB; j++)
        v[p][j] = *reinterpret_cast<const v4i *>(g + (k0 + kb * KB + j) * ld + col * ES);
    }
  }

  __device__ __forceinline__ void store(unsigned char *lds, int tid) const {
#pragma unroll
    for (int p = 0; p < PER; p++) {
      const int blk = tid + p * NTHREADS;
      if (blk >= BLOCKS) break;
      const int rb = blk % (ROWS / RB), kb = blk / (ROWS / RB);
      if constexpr (ES == 2) {
#pragma unroll
        for (int i = 0; i < 8; i++) {  // row i: dword j = { k = 2j , k = 2j+1 }
          v4i t;
#pragma unroll
          for (int j = 0; j < 4; j++) {
            const unsigned lo = (unsigned)v[p][2 * j][i >> 1], hi = (unsigned)v[p][2 * j + 1][i >> 1];
            t[j] = (int)__builtin_amdgcn_perm(hi, lo, (i & 1) ? 0x07060302u : 0x05040100u);
          }
          const int r = rb * 8 + i;
          *reinterpret_cast<v4i *>(lds + r * SLAB + lds_slot(r, kb) * 16) = t;
        }
      } else if constexpr (ES == 4) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const v4i t = {v[p][0][i], v[p][1][i], v[p][2][i], v[p][3][i]};
          const int r = rb * 4 + i;
          *reinterpret_cast<v4i *>(lds + r * SLAB + lds_slot(r, kb) * 16) = t;
        }
      } else if constexpr (ES == 8) {
#pragma unroll
        for (int i = 0; i < 2; i++) {  // row i: its two k of this block, 8 bytes each
          const v4i t = {v[p][0][2 * i], v[p][0][2 * i + 1], v[p][1][2 * i], v[p][1][2 * i + 1]};
          const int r = rb * 2 + i;
          *reinterpret_cast<v4i *>(lds + r * SLAB + lds_slot(r, kb) * 16) = t;
        }
      } else {
#pragma unroll
        for (int c = 0; c < 4; c++) {  // dword column c holds rows 4c .. 4c+3 of the four k
          const unsigned w0 = (unsigned)v[p][0][c], w1 = (unsigned)v[p][1][c], w2 = (unsigned)v[p][2][c], w3 = (unsigned)v[p][3][c];
          const unsigned a01 = __builtin_amdgcn_perm(w1, w0, 0x05010400u), b01 = __builtin_amdgcn_perm(w1, w0, 0x07030602u);
          const unsigned a23 = __builtin_amdgcn_perm(w3, w2, 0x05010400u), b23 = __builtin_amdgcn_perm(w3, w2, 0x07030602u);
          const unsigned o[4] = {__builtin_amdgcn_perm(a23, a01, 0x05040100u), __builtin_amdgcn_perm(a23, a01, 0x07060302u),
                                 __builtin_amdgcn_perm(b23, b01, 0x05040100u), __builtin_amdgcn_perm(b23, b01, 0x07060302u)};
#pragma unroll
          for (int i = 0; i < 4; i++) {  // row 4c+i: its four k bytes are dword (kb % 4) of chunk (kb / 4)
            const int r = rb * 16 + 4 * c + i;
            *reinterpret_cast<unsigned *>(lds + r * SLAB + lds_slot(r, kb >> 2) * 16 + (kb & 3) * 4) = o[i];
          }
        }
      }
    }
  }
};

// ---- K-outer 1- and 2-byte operands of the big tiles: no register staging at all.  The slab is
// copied as it lies in memory -- [k][ROWS], ROWS*ES bytes per k -- straight into LDS, and the MFMA
// fragments are fetched with the transposing LDS reads of gfx950 (semantics measured on the part).
// Within each group of 16 lanes every lane supplies the address of an 8-byte run, and
//   ds_read_b64_tr_b16: lane j receives element j%4 of the runs of lanes j/4 + {0, 4, 8, 12};
//     with lane i pointing at (k0 + i/4, n0 + 4*(i%4)) lane j receives [k0..k0+3][n0 + j];
//   ds_read_b64_tr_b8:  lane j receives byte j%8 of the runs of lanes j/8 + {0, 2, .., 14};
//     with lane i pointing at (k0 + i/2, n0 + 8*(i%2)) lane j receives [k0..k0+7][n0 + j]
// -- in both cases half an MFMA operand (8 bytes of consecutive k of one row).
// LDS layout: k-major, the 16-byte chunk index of a k-row XOR-ed with a function of k chosen so
// that the 32 lanes served per clock (lanes 0..31, then 32..63) cover all 64 banks
// (SQ_LDS_BANK_CONFLICT = 0): per clock the 16-bit form touches 8 k-rows x 32 bytes
// (k = 8g + 4h + 0..3 for lane groups g and g+1), the 8-bit form 16 k-rows x 16 bytes
// (k = 16g + 8h + 0..7).  A k-row must span all banks, i.e. at least 256 bytes.
typedef short v4s __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));

template <int ES>
__device__ __forceinline__ int tr_slot(int k, int chunk) {
  if constexpr (ES == 2) return chunk ^ ((k & 3) << 2) ^ (((k >> 3) & 1) << 1);
  else return chunk ^ (k & 7) ^ (((k >> 4) & 1) << 3);
}

// the same for k-rows narrower than the 256 bytes that span all LDS banks (int8 tiles of 64 or 128 columns): the
// chunk index XOR as many low bits of k as the row has chunk bits
template <int ES, int RBYTES>
__device__ __forceinline__ int tr_slot_w(int k, int chunk) {
  if constexpr (RBYTES >= 256) return tr_slot<ES>(k, chunk);
  else {
    static_assert(ES == 1 && (RBYTES == 128 || RBYTES == 64), "narrow k-rows: int8 tiles of 64 or 128 columns");
    return chunk ^ (k & (RBYTES / 16 - 1));
  }
}

template <int ES, int ROWS, int NWAVES>
struct KOuterDmaLoader {
  static constexpr int RBYTES = ROWS * ES;     // bytes per k-row of the slab
  static constexpr int INSTR = ROWS / 8;       // (128 / ES) k-rows * RBYTES / 1 KiB
  static constexpr int PER = INSTR / NWAVES;
  static_assert(RBYTES >= 256 && INSTR % NWAVES == 0, "needs at least 16 chunks per k-row");
  const unsigned char *src[PER];
  int lds_off[PER];

  // g: [K, cols] with `ld` bytes per k; the tile covers columns col0 .. col0+ROWS-1, of which
  // cols_valid (a multiple of 16 bytes' worth) exist: chunks past the edge re-read the last valid one
  __device__ __forceinline__ void init(const unsigned char *__restrict__ g, int64_t ld, int64_t col0, int64_t cols_valid,
                                       int wave, int lane) {
#pragma unroll
    for (int i = 0; i < PER; i++) {
      const int t = wave + NWAVES * i;
      const int o = t * 1024 + lane * 16;
      const int k = o / RBYTES, slot = (o % RBYTES) / 16;
      int64_t byte = col0 * ES + tr_slot<ES>(k, slot) * 16;
      const int64_t last = cols_valid * ES - 16;
      byte = byte <= last ? byte : last;
      src[i] = g + (int64_t)k * ld + byte;
      lds_off[i] = t * 1024;
    }
  }
  __device__ __forceinline__ void issue(int64_t k0, int64_t ld, unsigned char *lds) const {
#pragma unroll
    for (int i = 0; i < PER; i++)
      lds_dma16(src[i] + k0 * ld, lds + lds_off[i]);
  }
  __device__ __forceinline__ void issue_at(int t, int spread, int phase, int skew, int64_t k0, int64_t ld, unsigned char *lds) const {
#pragma unroll
    for (int i = 0; i < PER; i++)
      if (t == i * spread / PER + phase + skew) lds_dma16(src[i] + k0 * ld, lds + lds_off[i]);
  }
};

// MFMA operand fragment (16 bytes of consecutive k per lane) of rows row0 .. row0+15 for K step
// `ks` (64 bytes of k) out of a k-major slab: two transposing reads.
template <int ES, int ROWS>
__device__ __forceinline__ v4i read_fragment_tr(const unsigned char *slab, int row0, int ks, int lane) {
  const int i16 = lane & 15;
  v4i out;
  if constexpr (ES == 2) {
    const int n = row0 + 4 * (i16 & 3);
    const int kbase = 32 * ks + 8 * (lane >> 4) + (i16 >> 2);
#pragma unroll
    for (int h = 0; h < 2; h++) {
      const int k = kbase + 4 * h;
      const unsigned char *p = slab + k * (ROWS * 2) + tr_slot<2>(k, n >> 3) * 16 + (n & 7) * 2;
      const v4s r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s *)p);
      const int2 w = __builtin_bit_cast(int2, r);
      out[2 * h] = w.x;
      out[2 * h + 1] = w.y;
    }
  } else {
    const int n = row0 + 8 * (i16 & 1);
    const int kbase = 64 * ks + 16 * (lane >> 4) + (i16 >> 1);
#pragma unroll
    for (int h = 0; h < 2; h++) {
      const int k = kbase + 8 * h;
      const unsigned char *p = slab + k * ROWS + tr_slot_w<1, ROWS>(k, n >> 4) * 16 + (n & 15);
      const v2i r = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) v2i *)p);
      out[2 * h] = r[0];
      out[2 * h + 1] = r[1];
    }
  }
  return out;
}

struct GemmArgs {
  const unsigned char *l, *r;
  void *out;
  int odt;
  int64_t M, N, Kb;      // Kb = K in bytes (a multiple of 128 for this kernel)
  int64_t ld_l, ld_r;    // bytes between consecutive rows (K-inner) or consecutive k (K-outer)
  int64_t bs_l, bs_r;    // bytes between batch items
  int tiles_m, tiles_n;
  int group_m;  // tile rows per group of the tile order (see gemm_group_m)
  // s8 x s8 with an f32 output: out = (float)(the s32 sum) * scale -- the conversion and the
  // multiplication that follow the contraction of a quantised linear layer, done on the accumulators
  const float *scale;
  int scale_mode;  // HIPNX_SCALE_NONE / PER_COLUMN (scale[n]) / PER_ROW (scale[m]) / ONE (scale[0])
};

// Epilogue of one wave: for 16x16 tile (i, j) a lane holds m = 16*i + lane%16 and
// n = 16*j + 4*(lane/16) + 0..3.  ODT is a compile-time constant here, so the typed stores fold
// to plain vector stores; every accumulator index is a constant (the accumulators must never be
// addressed dynamically, or they leave the register file).
template <int DT, int ODT, int TM, int TN>
__device__ __forceinline__ void gemm_epilogue(typename Mma16<DT>::acc_t (&acc)[TM][TN], void *out, int64_t obase,
                                              int64_t M, int64_t N, int64_t row0, int64_t col0, int lane,
                                              const float *scale = nullptr, int scale_mode = 0,
                                              unsigned char *wave_lds = nullptr) {
  constexpr bool int_acc = DT == HIPNX_S8;
  constexpr bool int_out = ODT < HIPNX_F16;
  if constexpr (DT == HIPNX_F64) {
    // f64 accumulators: register e of a lane is n = 4 e + lane / 16 (Mma16<HIPNX_F64>), one rounding to the output type
    if constexpr (int_out) return;  // the host never pairs them
    else {
#pragma unroll
      for (int i = 0; i < TM; i++) {
        const int64_t gm = row0 + 16 * i + (lane & 15);
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const int64_t gn = col0 + 16 * j + 4 * e + (lane >> 4);
            if (gm < M && gn < N) store_one<double>(out, ODT, obase + gm * N + gn, acc[i][j][e]);
          }
      }
    }
  } else if constexpr (int_acc && ODT == HIPNX_F32) {
    // as_type(s32 -> f32) then multiply, each rounding once, as the two separate kernels would
    if (scale_mode == HIPNX_SCALE_NONE) return;  // the host pairs them only with a scale
    const bool vec_ok = (N % 4) == 0;
    const float one = scale_mode == HIPNX_SCALE_ONE ? scale[0] : 0.0f;
#pragma unroll
    for (int i = 0; i < TM; i++) {
      const int64_t gm = row0 + 16 * i + (lane & 15);
      const float per_row = scale_mode == HIPNX_SCALE_PER_ROW && gm < M ? scale[gm] : one;
#pragma unroll
      for (int j = 0; j < TN; j++) {
        const int64_t gn = col0 + 16 * j + 4 * (lane >> 4);
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const float sc = scale_mode == HIPNX_SCALE_PER_COLUMN ? (gn + e < N ? scale[gn + e] : 0.0f) : per_row;
          v[e] = (float)(int32_t)acc[i][j][e] * sc;
        }
        const int64_t idx = obase + gm * N + gn;
        if (gm < M) {
          if (vec_ok && gn + 4 <= N) store_vec<float, 4>(out, HIPNX_F32, idx, v);
          else {
#pragma unroll
            for (int e = 0; e < 4; e++)
              if (gn + e < N) store_one<float>(out, HIPNX_F32, idx + e, v[e]);
          }
        }
      }
    }
  } else if constexpr (int_acc != int_out) return;  // the host never pairs them
  else if constexpr (!int_acc && (ODT == HIPNX_BF16 || ODT == HIPNX_BF16_RNE || ODT == HIPNX_F16) && TN % 2 == 0) {
    // 2-byte outputs: a lane's 4 outputs of a tile are only 8 bytes, and a store instruction made of
    // 32-byte runs per row is slow (measured on the 4096^3 bf16 case: 11 us of the kernel, twice the
    // time the s32 epilogue takes for twice the bytes).  Two neighbouring column tiles are written
    // together instead: lanes 16 apart hold adjacent groups of 4 columns, so they trade halves --
    // the lane of the even group keeps tile j and receives its neighbour's 4 columns of tile j, the
    // other keeps tile j+1 -- and every lane stores 16 bytes, 64 contiguous bytes per row.
    const bool odd = (lane >> 4) & 1;
    const int64_t gc = col0 + 4 * ((lane >> 4) & 2);  // first of this lane's 8 columns within its tile
    auto pack = [](float lo, float hi) -> uint32_t {
      if constexpr (ODT == HIPNX_BF16) return (uint32_t)f32_to_bf16_bits_trunc(lo) | ((uint32_t)f32_to_bf16_bits_trunc(hi) << 16);
      else if constexpr (ODT == HIPNX_BF16_RNE) return (uint32_t)f32_to_bf16_bits_rne(lo) | ((uint32_t)f32_to_bf16_bits_rne(hi) << 16);
      else return (uint32_t)f32_to_f16_bits(lo) | ((uint32_t)f32_to_f16_bits(hi) << 16);
    };
    // N % 8 == 0: a group of 8 columns lies wholly inside or outside, and row starts keep the 16-byte alignment
    const bool paired = (N % 8) == 0 && ((uintptr_t)out & 15) == 0;
    // A second exchange makes the runs whole cache lines: of two neighbouring PAIRS of tiles the lanes of
    // rows 8..15 hand their first pair's 16 bytes to the lane 8 rows up and take that lane's second pair, so
    // that one store instruction covers rows 0..7 with 128 contiguous bytes each (four tiles wide) and the
    // next one rows 8..15 -- instead of 16 rows of 64 bytes.
    const bool hi = (lane >> 3) & 1;
    auto pair16 = [&](int i, int j) -> v4i {  // this lane's 8 columns of tiles j, j+1 (see above)
      const uint32_t a0 = pack(acc[i][j][0], acc[i][j][1]), a1 = pack(acc[i][j][2], acc[i][j][3]);
      const uint32_t b0 = pack(acc[i][j + 1][0], acc[i][j + 1][1]), b1 = pack(acc[i][j + 1][2], acc[i][j + 1][3]);
      const uint32_t r0 = (uint32_t)__shfl_xor((int)(odd ? a0 : b0), 16, 64);
      const uint32_t r1 = (uint32_t)__shfl_xor((int)(odd ? a1 : b1), 16, 64);
      v4i v;
      v[0] = (int)(odd ? r0 : a0); v[1] = (int)(odd ? r1 : a1); v[2] = (int)(odd ? b0 : r0); v[3] = (int)(odd ? b1 : r1);
      return v;
    };
    auto put16 = [&](int64_t gm, int64_t gn, const v4i &v) {
      if (gm < M && gn < N) *reinterpret_cast<v4i *>((unsigned char *)out + (obase + gm * N + gn) * 2) = v;
    };
    if constexpr (TN % 4 == 0) {
      if (wave_lds != nullptr && paired) {
        // with LDS of its own the wave turns four tiles (16 rows x 128 bytes) around instead, as the 4-byte
        // branch below describes: every cache line leaves as one run of eight neighbouring lanes
        const int wr = lane & 15, wc = lane >> 4, rr = lane >> 3, rp = lane & 7;
        const int w_off = wr * 128 + (wc & 1) * 8, w_swz = (wr >> 1) & 7;
        const int r_off0 = rr * 128 + ((rp ^ ((rr >> 1) & 7)) * 16), r_off1 = (rr + 8) * 128 + ((rp ^ (((rr + 8) >> 1) & 7)) * 16);
#pragma unroll
        for (int i = 0; i < TM; i++) {
#pragma unroll
          for (int j = 0; j < TN; j += 4) {
            unsigned char *half = wave_lds + (((i * TN + j) >> 2) & 1) * 2048;  // two halves in turn
#pragma unroll
            for (int t = 0; t < 4; t++) {
              typedef __attribute__((ext_vector_type(2))) unsigned int v2u;
              v2u pk;
              pk[0] = pack(acc[i][j + t][0], acc[i][j + t][1]);
              pk[1] = pack(acc[i][j + t][2], acc[i][j + t][3]);
              *reinterpret_cast<v2u *>(half + w_off + (((2 * t + (wc >> 1)) ^ w_swz) * 16)) = pk;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            const v4i lo = *reinterpret_cast<const v4i *>(half + r_off0);
            const v4i up = *reinterpret_cast<const v4i *>(half + r_off1);
            const int64_t gm = row0 + 16 * i + rr, gn = col0 + 16 * j + 8 * rp;
            put16(gm, gn, lo);
            put16(gm + 8, gn, up);
          }
        }
        return;
      }
    }
#pragma unroll
    for (int i = 0; i < TM; i++) {
      const int64_t gm = row0 + 16 * i + (lane & 15);
      if constexpr (TN % 4 == 0) {
        if (paired) {
#pragma unroll
          for (int j = 0; j < TN; j += 4) {
            const v4i v = pair16(i, j), w = pair16(i, j + 2);
            v4i got;  // the partner's other pair: rows 0..7 receive the second pair of rows 8..15 and vice versa
#pragma unroll
            for (int e = 0; e < 4; e++) got[e] = __shfl_xor(hi ? v[e] : w[e], 8, 64);
            const int64_t gn0 = gc + 16 * (j + (odd ? 1 : 0)), gn1 = gn0 + 32;
            // rows 0..7 of the 16: own first pair (rows < 8) | the partner's second pair, stored for row - 8
            put16(hi ? gm - 8 : gm, hi ? gn1 : gn0, hi ? got : v);
            // rows 8..15: own second pair stays with rows >= 8 | rows < 8 store the partner's first pair for row + 8
            put16(hi ? gm : gm + 8, hi ? gn1 : gn0, hi ? w : got);
          }
          continue;
        }
      }
#pragma unroll
      for (int j = 0; j < TN; j += 2) {
        if (paired) {
          put16(gm, gc + 16 * (j + (odd ? 1 : 0)), pair16(i, j));
        } else {
#pragma unroll
          for (int jj = j; jj < j + 2; jj++) {
            const int64_t gn = col0 + 16 * jj + 4 * (lane >> 4);
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = acc[i][jj][e];
            const int64_t idx = obase + gm * N + gn;
            if (gm < M) {
              if ((N % 4) == 0 && gn + 4 <= N) store_vec<float, 4>(out, ODT, idx, v);
              else {
#pragma unroll
                for (int e = 0; e < 4; e++)
                  if (gn + e < N) store_one<float>(out, ODT, idx + e, v[e]);
              }
            }
          }
        }
      }
    }
  } else if constexpr ((ODT == HIPNX_S32 || ODT == HIPNX_U32 || ODT == HIPNX_F32) && TN % 2 == 0) {
    // 4-byte outputs: a lane's 4 outputs of a tile are 16 bytes, 64 contiguous bytes per row.  Of two
    // neighbouring column tiles the lanes of rows 8..15 hand their first tile's values to the lane 8 rows up
    // and take that lane's second tile, so that a store instruction writes 8 rows of 128 contiguous bytes
    // (whole cache lines) instead of 16 rows of 64: the 64 MiB s32 result of the int8 kernel is the longest
    // part of its epilogue, and nothing overlaps it when every CU holds one tile.
    auto word = [](typename Mma16<DT>::acc_t const &c, int e) -> int {
      if constexpr (int_acc) return (int)c[e];  // the low 32 bits: the wrap of shared.ex:190-194
      else return (int)f32_canon_bits(c[e]);
    };
    const bool hi = (lane >> 3) & 1;
    const bool lines = (N % 4) == 0 && ((uintptr_t)out & 15) == 0;
    auto put16 = [&](int64_t gm, int64_t gn, const v4i &v) {
      if (gm < M && gn < N) *reinterpret_cast<v4i *>((unsigned char *)out + (obase + gm * N + gn) * 4) = v;
    };
    if (wave_lds != nullptr && lines) {
      // With 4 KiB of LDS of its own a wave turns each pair of tiles (16 rows x 128 bytes) around first:
      // written as the accumulators hold it (lane = row, 16-byte piece c of either tile), read back with
      // eight consecutive lanes along one row, so that every cache line of the result leaves as ONE
      // contiguous 128-byte run of eight neighbouring lanes.  In the exchange-only form below a line is made
      // of eight 16-byte pieces from four different quarters of the wave; when the result is larger than the
      // L2s (the 64 MiB s32 result of a 4096^2 int8 contraction) lines are evicted between their pieces,
      // and the counters show the cost: 94 MiB written and 30 MiB read back for 64 MiB of output.
      // Piece index XOR (row / 2) % 8 keeps both the write and the read free of bank conflicts.
      const int wr = lane & 15, wc = lane >> 4, rr = lane >> 3, rp = lane & 7;
      const int w_off = wr * 128, w_swz = (wr >> 1) & 7;
      const int r_off0 = rr * 128 + ((rp ^ ((rr >> 1) & 7)) * 16), r_off1 = (rr + 8) * 128 + ((rp ^ (((rr + 8) >> 1) & 7)) * 16);
#pragma unroll
      for (int i = 0; i < TM; i++) {
#pragma unroll
        for (int j = 0; j < TN; j += 2) {
          unsigned char *half = wave_lds + (((i * TN + j) >> 1) & 1) * 2048;  // two halves in turn
          v4i v, w;
#pragma unroll
          for (int e = 0; e < 4; e++) { v[e] = word(acc[i][j], e); w[e] = word(acc[i][j + 1], e); }
          *reinterpret_cast<v4i *>(half + w_off + ((wc ^ w_swz) * 16)) = v;
          *reinterpret_cast<v4i *>(half + w_off + (((4 + wc) ^ w_swz) * 16)) = w;
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
          __builtin_amdgcn_wave_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
          const v4i lo = *reinterpret_cast<const v4i *>(half + r_off0);
          const v4i up = *reinterpret_cast<const v4i *>(half + r_off1);
          const int64_t gm = row0 + 16 * i + rr, gn = col0 + 16 * j + 4 * rp;
          put16(gm, gn, lo);
          put16(gm + 8, gn, up);
        }
      }
      return;
    }
#pragma unroll
    for (int i = 0; i < TM; i++) {
      const int64_t gm = row0 + 16 * i + (lane & 15);
#pragma unroll
      for (int j = 0; j < TN; j += 2) {
        const int64_t gn0 = col0 + 16 * j + 4 * (lane >> 4), gn1 = gn0 + 16;
        v4i v, w;
#pragma unroll
        for (int e = 0; e < 4; e++) { v[e] = word(acc[i][j], e); w[e] = word(acc[i][j + 1], e); }
        if (lines) {
          v4i got;
#pragma unroll
          for (int e = 0; e < 4; e++) got[e] = __shfl_xor(hi ? v[e] : w[e], 8, 64);
          put16(hi ? gm - 8 : gm, hi ? gn1 : gn0, hi ? got : v);  // rows 0..7 of the 16, both tiles
          put16(hi ? gm : gm + 8, hi ? gn1 : gn0, hi ? w : got);  // rows 8..15
        } else {
#pragma unroll
          for (int e = 0; e < 4; e++) {
            if (gm < M && gn0 + e < N) *reinterpret_cast<int *>((unsigned char *)out + (obase + gm * N + gn0 + e) * 4) = v[e];
            if (gm < M && gn1 + e < N) *reinterpret_cast<int *>((unsigned char *)out + (obase + gm * N + gn1 + e) * 4) = w[e];
          }
        }
      }
    }
  } else {
    typedef typename std::conditional<int_acc, int64_t, float>::type S;
    const bool vec_ok = (N % 4) == 0;
#pragma unroll
    for (int i = 0; i < TM; i++) {
      const int64_t gm = row0 + 16 * i + (lane & 15);
#pragma unroll
      for (int j = 0; j < TN; j++) {
        const int64_t gn = col0 + 16 * j + 4 * (lane >> 4);
        S v[4];
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = (S)acc[i][j][e];
        const int64_t idx = obase + gm * N + gn;
        if (gm < M) {
          if (vec_ok && gn + 4 <= N) store_vec<S, 4>(out, ODT, idx, v);
          else {
#pragma unroll
            for (int e = 0; e < 4; e++)
              if (gn + e < N) store_one<S>(out, ODT, idx + e, v[e]);
          }
        }
      }
    }
  }
}

// Rows per group of the tile order: the largest power of two not above the square root of the
// number of tiles one XCD works on at a time.
inline int gemm_group_m(int tiles_m, int tiles_n) {
  int per_xcd = (tiles_m * tiles_n + 7) / 8;
  if (per_xcd > 64) per_xcd = 64;
  int g = 1;
  while ((2 * g) * (2 * g) <= per_xcd && 2 * g <= tiles_m) g *= 2;
  return g;
}

// Tile order: consecutive work-group ids go to different XCDs (id % 8), so each XCD takes a run of
// total/8 consecutive positions of the order below; the order walks groups of `group_m` tile rows
// column by column, which makes such a run a compact rectangle of tiles whose operand panels are
// shared through the XCD's own L2.
__device__ __forceinline__ void gemm_tile_position(const GemmArgs &a, int block, int &tm, int &tn) {
  int tile = block;
  const int total = a.tiles_m * a.tiles_n;
  if (total % 8 == 0) tile = (block % 8) * (total / 8) + block / 8;
  const int per_group = a.group_m * a.tiles_n;
  const int first = (tile / per_group) * a.group_m;
  const int rows = min(a.group_m, a.tiles_m - first);
  const int in = tile % per_group;
  tm = first + in % rows;
  tn = in / rows;
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {  // s_waitcnt vmcnt(N), other counters untouched
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

template <int DT, int WM, int WN, int TM, int TN, bool L_KIN, bool R_KIN, int NSTAGE = 2, bool EARLY = false>
// (f64: at least two waves per SIMD, i.e. at most 256 registers and all of them VGPRs.  With the 512 that a work-group
// of four waves may have, the compiler keeps some accumulators in AGPRs and moves them to and fro inside the K loop --
// 128 copies per slab beside 64 MFMAs, each waiting for the MFMA that last wrote its source: 2048^3 404 -> 329 us,
// 4096^3 2.8 -> 2.0 ms.  f64 with both operands K-outer does not fit 256 registers and would spill; the f32 kernels
// lose by the same limit, 2048^3 152 -> 167 us.)
__global__ void __launch_bounds__(WM *WN * 64) __attribute__((amdgpu_waves_per_eu(DT == HIPNX_F64 && (L_KIN || R_KIN) ? 2 : 1)))
gemm_pipelined_kernel(GemmArgs a) {
  typedef typename Mma16<DT>::acc_t acc_t;
  constexpr int NW = WM * WN, NT = NW * 64;
  constexpr int TM16 = 2 * TM, TN16 = 2 * TN;  // 16x16 MFMA tiles per wave
  constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
  constexpr int STAGE = (BM + BN) * SLAB;
  constexpr int KSTEPS = SLAB / 64;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

  int tm, tn;
  gemm_tile_position(a, blockIdx.x, tm, tn);
  const int64_t b = blockIdx.y;
  const unsigned char *lb = a.l + b * a.bs_l;
  const unsigned char *rb = a.r + b * a.bs_r;
  const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = (wave / WN) * (TM * 32), wn = (wave % WN) * (TN * 32);

  acc_t acc[TM16][TN16];
#pragma unroll
  for (int i = 0; i < TM16; i++)
#pragma unroll
    for (int j = 0; j < TN16; j++)
#pragma unroll
      for (int q = 0; q < 4; q++) acc[i][j][q] = 0;

  KInnerLoader<BM, NW> lload;
  KInnerLoader<BN, NW> rload;
  if constexpr (L_KIN) lload.init(lb, a.ld_l, m0, a.M, wave, lane);
  if constexpr (R_KIN) rload.init(rb, a.ld_r, n0, a.N, wave, lane);
  constexpr int ES = (DT == HIPNX_S8) ? 1 : (DT == HIPNX_F32 ? 4 : DT == HIPNX_F64 ? 8 : 2);
  static_assert(DT != HIPNX_F64 || TM16 * TN16 <= 16, "f64 accumulators are two registers an element: wave tiles up to 64 x 64");
  // K-outer 1- and 2-byte operands of tiles whose k-rows span all LDS banks: DMA + transposing reads
  constexpr bool L_TR = !L_KIN && ES <= 2 && BM * ES >= 256 && (BM / 8) % NW == 0;
  constexpr bool R_TR = !R_KIN && ES <= 2 && BN * ES >= 256 && (BN / 8) % NW == 0;
  constexpr int TR_ES = ES <= 2 ? ES : 2;
  KOuterDmaLoader<TR_ES, L_TR ? BM : 256 * NW, NW> ltr;
  KOuterDmaLoader<TR_ES, R_TR ? BN : 256 * NW, NW> rtr;
  if constexpr (L_TR) ltr.init(lb, a.ld_l, m0, a.M, wave, lane);
  if constexpr (R_TR) rtr.init(rb, a.ld_r, n0, a.N, wave, lane);
  KOuterStage<ES, BM, NT> lregs;
  KOuterStage<ES, BN, NT> rregs;

  auto issue = [&](int stage, int64_t kbyte0) {
    unsigned char *sA = smem + stage * STAGE, *sB = sA + BM * SLAB;
    if constexpr (L_KIN) lload.issue(kbyte0, sA);
    else if constexpr (L_TR) ltr.issue(kbyte0 / ES, a.ld_l, sA);
    else lregs.fetch(lb, a.ld_l, m0, a.M, kbyte0 / ES, tid);
    if constexpr (R_KIN) rload.issue(kbyte0, sB);
    else if constexpr (R_TR) rtr.issue(kbyte0 / ES, a.ld_r, sB);
    else rregs.fetch(rb, a.ld_r, n0, a.N, kbyte0 / ES, tid);
  };
  auto commit = [&](int stage) {  // register-staged K-outer operands: transposed LDS writes
    unsigned char *sA = smem + stage * STAGE, *sB = sA + BM * SLAB;
    if constexpr (!L_KIN && !L_TR) lregs.store(sA, tid);
    if constexpr (!R_KIN && !R_TR) rregs.store(sB, tid);
  };

  // ---- the K walk.  NSTAGE LDS stages; slab s lives in stage s % NSTAGE and the requests for
  // slab s+NSTAGE-1 go out while slab s is computed (more than two stages only when every
  // operand arrives by direct-to-LDS loads: these are counted by hand, vmcnt(n) leaves the
  // younger slabs in flight).
  // One step = one column of 16x16 tiles (TM16 MFMAs) of one K step; a slab is STEPS steps.
  // Fragment reads run DIST steps ahead of the MFMAs that use them (r fragments in a ring of
  // four, l fragments of the next K step fetched during the last steps of the current one), and
  // the waits in between are partial (lgkmcnt(n): LDS reads return in order).
  // The one barrier per slab sits after step BAR = STEPS-DIST-1, by which a wave has issued every
  // read of the slab.  Before it the wave drains its reads (so the stage may be overwritten) and
  // its direct-to-LDS loads of the next slab (so that slab may be read); after it the remaining
  // DIST steps of MFMAs run on fragments already in registers while the first fragments of the
  // next slab are fetched -- no wave sits idle behind the barrier waiting for LDS.
  // The next slab's global requests go out one instruction at a time during the steps before
  // BAR (l and r in alternate steps): a wave that issues a slab's loads back to back sits in
  // the issue stage until the address unit has taken them all and feeds no MFMA meanwhile.
  constexpr int STEPS = KSTEPS * TN16;
  constexpr int DIST = STEPS >= 8 ? 3 : 2;
  constexpr int RING = 4;
  constexpr int BAR = STEPS - DIST - 1;
  constexpr int SPREAD = BAR * 3 / 4 > 0 ? BAR * 3 / 4 : 1;
  static_assert(KSTEPS == 2 && TN16 >= TM16 && STEPS % RING == 0 && BAR >= 1 && BAR >= TN16 - 1 && SPREAD <= BAR,
                "wave tile shape does not fit the fragment pipeline");
  auto issue_step = [&](int t, int stage, int64_t kbyte0) {
    unsigned char *sA = smem + stage * STAGE, *sB = sA + BM * SLAB;
    if constexpr (L_KIN) lload.issue_at(t, SPREAD, 0, 0, kbyte0, sA);
    else if constexpr (L_TR) ltr.issue_at(t, SPREAD, 0, 0, kbyte0 / ES, a.ld_l, sA);
    else if (t == 0) lregs.fetch(lb, a.ld_l, m0, a.M, kbyte0 / ES, tid);
    if constexpr (R_KIN) rload.issue_at(t, SPREAD, 1, 0, kbyte0, sB);
    else if constexpr (R_TR) rtr.issue_at(t, SPREAD, 1, 0, kbyte0 / ES, a.ld_r, sB);
    else if (t == 0) rregs.fetch(rb, a.ld_r, n0, a.N, kbyte0 / ES, tid);
  };
  auto read_l = [&](const unsigned char *st, int ks, int i) -> v4i {
    const int row = wm + 16 * i + (lane & 15);
    if constexpr (L_TR) return read_fragment_tr<TR_ES, BM>(st, wm + 16 * i, ks, lane);
    else return *reinterpret_cast<const v4i *>(st + row * SLAB + lds_slot(row, 4 * ks + (lane >> 4)) * 16);
  };
  auto read_r = [&](const unsigned char *st, int t) -> v4i {  // step t = (K step, column tile)
    const int ks = t / TN16, j = t % TN16;
    const int row = wn + 16 * j + (lane & 15);
    const unsigned char *sB = st + BM * SLAB;
    if constexpr (R_TR) return read_fragment_tr<TR_ES, BN>(sB, wn + 16 * j, ks, lane);
    else return *reinterpret_cast<const v4i *>(sB + row * SLAB + lds_slot(row, 4 * ks + (lane >> 4)) * 16);
  };

  constexpr bool ALL_DMA = (L_KIN || L_TR) && (R_KIN || R_TR);
  static_assert(NSTAGE == 2 || ALL_DMA, "register-staged operands need the two-stage walk");
  // EARLY (two stages, every operand by direct-to-LDS loads): the requests of a slab start right
  // behind the barrier that frees its stage -- in the POST steps that follow the barrier of the slab
  // before the previous one's successor -- instead of at the next slab's first step, one
  // instruction per step (l in even, r in odd virtual steps u = 0, 1, ..): the last request then
  // has POST more steps to land before the barrier that publishes the slab.
  constexpr int POST = STEPS - 1 - BAR;
  static_assert(!EARLY || (NSTAGE == 2 && ALL_DMA), "early requests need two stages of direct-to-LDS operands");
  auto issue_early = [&](int u, int stage, int64_t kbyte0) {
    unsigned char *sA = smem + stage * STAGE, *sB = sA + BM * SLAB;
    if constexpr (L_KIN) lload.issue_at(u, 2 * KInnerLoader<BM, NW>::PER, 0, 0, kbyte0, sA);
    else if constexpr (L_TR) ltr.issue_at(u, 2 * KOuterDmaLoader<TR_ES, L_TR ? BM : 256 * NW, NW>::PER, 0, 0, kbyte0 / ES, a.ld_l, sA);
    if constexpr (R_KIN) rload.issue_at(u, 2 * KInnerLoader<BN, NW>::PER, 1, 0, kbyte0, sB);
    else if constexpr (R_TR) rtr.issue_at(u, 2 * KOuterDmaLoader<TR_ES, R_TR ? BN : 256 * NW, NW>::PER, 1, 0, kbyte0 / ES, a.ld_r, sB);
  };
  constexpr int OPS = (L_KIN ? KInnerLoader<BM, NW>::PER : L_TR ? KOuterDmaLoader<TR_ES, L_TR ? BM : 256 * NW, NW>::PER : 0) +
                      (R_KIN ? KInnerLoader<BN, NW>::PER : R_TR ? KOuterDmaLoader<TR_ES, R_TR ? BN : 256 * NW, NW>::PER : 0);
  constexpr int INFLIGHT = OPS * (NSTAGE - 2);  // requests of younger slabs that may stay outstanding
  static_assert(INFLIGHT < 64, "vmcnt is a 6-bit counter");
  const int nslab = (int)(a.Kb / SLAB);
#pragma unroll
  for (int p = 0; p < NSTAGE - 1; p++)
    if (p < nslab) issue(p, (int64_t)p * SLAB);
  commit(0);
  if (nslab >= NSTAGE - 1) wait_vmcnt<INFLIGHT>();
  else wait_vmcnt<0>();
  __syncthreads();
  if constexpr (EARLY) {  // the first requests of slab 1 (what the steps behind a barrier would have issued)
    if (1 < nslab) {
#pragma unroll
      for (int u = 0; u < POST; u++) issue_early(u, 1, SLAB);
    }
  }
  v4i fa[2][TM16], fb[RING];
#pragma unroll
  for (int i = 0; i < TM16; i++) fa[0][i] = read_l(smem, 0, i);
#pragma unroll
  for (int d = 0; d < DIST; d++) fb[d] = read_r(smem, d);

  for (int s = 0; s < nslab; s++) {
    const unsigned char *cur = smem + (s % NSTAGE) * STAGE, *nxt = smem + ((s + 1) % NSTAGE) * STAGE;
    const bool more = s + 1 < nslab;                  // another slab to compute after this one
    const bool request = s + NSTAGE - 1 < nslab;      // another slab to request during this one
    const int req_stage = (s + NSTAGE - 1) % NSTAGE;
    const int64_t req_kbyte = (int64_t)(s + NSTAGE - 1) * SLAB;
#pragma unroll
    for (int t = 0; t < STEPS; t++) {
      const int ks = t / TN16, j = t % TN16;
      // The two waves of a SIMD take turns step by step: a wave holds the higher priority from its
      // fragment reads to the last MFMA of the step and drops it for an instant afterwards, which is
      // when the other wave's step gets in.  Without it their instructions interleave and the MFMA
      // bursts break up (measured on the 4096^3 bf16 case, 100 timed launches after 20: 1.03-1.05 ->
      // 1.07-1.08 PFLOP/s; high priority for the MFMAs alone or for the reads alone: 1.05).
      __builtin_amdgcn_s_setprio(1);
      // r fragment of step t + DIST (of the next slab once past the end of this one)
      if (t + DIST < STEPS) fb[(t + DIST) % RING] = read_r(cur, t + DIST);
      else if (more) fb[(t + DIST) % RING] = read_r(nxt, t + DIST - STEPS);
      // l fragments of the next K step: within the slab during the last TM16 steps of this K
      // step, across the slab boundary spread over the DIST steps behind the barrier
      if (ks + 1 < KSTEPS) {
        if (j >= TN16 - TM16) fa[(ks + 1) & 1][j - (TN16 - TM16)] = read_l(cur, ks + 1, j - (TN16 - TM16));
      } else if (more && t >= STEPS - DIST) {
        const int d = t - (STEPS - DIST);
#pragma unroll
        for (int i = 0; i < TM16; i++)
          if (i >= d * TM16 / DIST && i < (d + 1) * TM16 / DIST) fa[0][i] = read_l(nxt, 0, i);
      }
      if constexpr (EARLY) {
        if (t > BAR) {
          if (s + 2 < nslab) issue_early(t - BAR - 1, s % NSTAGE, (int64_t)(s + 2) * SLAB);
        } else if (request) issue_early(t + POST, req_stage, req_kbyte);
      } else if (request && t <= BAR) issue_step(t, req_stage, req_kbyte);
#pragma unroll
      for (int i = 0; i < TM16; i++) Mma16<DT>::step(acc[i][j], fb[t % RING], fa[ks & 1][i]);
      __builtin_amdgcn_s_setprio(0);
      if (t == BAR && more) {
        commit(req_stage);                   // (two stages: the slab requested is the next one)
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): my reads of this slab have returned
        if (request) wait_vmcnt<INFLIGHT>(); // my loads of the next slab have landed
        else wait_vmcnt<0>();
        __syncthreads();
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // epilogue: the output type is wave-uniform; branch once, then every store is straight-line
  const int64_t obase = b * a.M * a.N;
  // every wave has read its last fragments: the stages are free, and each wave takes 4 KiB of them to turn its
  // result tiles into whole cache lines (a stage is at least (BM + BN) * 128 bytes = 6 KiB per wave)
  __syncthreads();
  switch (a.odt) {
#define HIPNX_EPI(T) case T: gemm_epilogue<DT, T, TM16, TN16>(acc, a.out, obase, a.M, a.N, m0 + wm, n0 + wn, lane, a.scale, a.scale_mode, smem + wave * 4096); break;
    HIPNX_EPI(HIPNX_BF16) HIPNX_EPI(HIPNX_F16) HIPNX_EPI(HIPNX_F32) HIPNX_EPI(HIPNX_F64) HIPNX_EPI(HIPNX_BF16_RNE)
    HIPNX_EPI(HIPNX_S8) HIPNX_EPI(HIPNX_U8) HIPNX_EPI(HIPNX_S16) HIPNX_EPI(HIPNX_U16)
    HIPNX_EPI(HIPNX_S32) HIPNX_EPI(HIPNX_U32) HIPNX_EPI(HIPNX_S64) HIPNX_EPI(HIPNX_U64)
#undef HIPNX_EPI
  }
}

}  // namespace hipnx
