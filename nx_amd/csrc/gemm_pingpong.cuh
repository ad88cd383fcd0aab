// The 256 x 256 tile of the MFMA contraction as a two-group walk: the eight waves of a work-group
// form two groups of four (one wave of each group per SIMD), and in every phase one group only
// issues MFMAs while the other only moves data -- fragment reads out of LDS and the direct-to-LDS
// requests of later slabs -- then they trade places at a work-group barrier.  The matrix pipe of a
// SIMD is fed by one wave at a time from registers that are already loaded, and whatever a memory
// instruction costs in the issue stage (a direct-to-LDS request sits there until the address unit
// has taken it) is paid by a wave that has no MFMA to issue anyway.
//
// Wave tile 64 x 128 as in gemm_pipelined_kernel (4 x 8 MFMA tiles of 16 x 16, accumulators in
// registers); K in slabs of 128 bytes per row, two LDS stages of one slab each.  A phase is one
// K step (64 bytes of K): 12 fragment reads + 4 requests for the memory group, 32 MFMAs for the
// other.  With p the phase number, group 0 (waves 0-3, the upper 128 rows of the tile) reads K step
// q in phase 2q and multiplies in 2q+1; group 1 (waves 4-7, the lower rows) runs one phase behind.
//
// Requests (64 per slab, 16 per phase, 4 per wave and memory phase; s = slab being read):
//   phase 4s   group 0: its share of the right operand of slab s+1
//   phase 4s+1 group 1: its share of the right operand of slab s+1
//   phase 4s+2 group 0: left rows 128..255 of slab s+1      (read by group 1 only: free since 4s)
//   phase 4s+3 group 1: left rows   0..127 of slab s+2      (read by group 0 only: free since 4s+3)
// Every request has two and a half phases to land: the wave that issued it waits for it at the end
// of its next memory phase (vmcnt(4): everything but what it has just issued), the barrier behind
// that wait publishes it, and the first reader comes a phase later or more.
#pragma once
#include "gemm_mfma.cuh"

namespace hipnx {

// Only the stand-alone timeline program (gemm_timeline.hip) defines HIPNX_GEMM_TIMELINE: the 256-row kernel then
// leaves, per work-group, the constant-rate clock at its start, at the first phase of the walk, at the end of the
// walk and after its last store was issued, the shader clocks the walk took, and the XCD it ran on.  The same
// program sets HIPNX_PP_EXP for timing-only builds of the walk (their results are wrong): 1 = no requests after
// the prologue, 32 = no fragment reads after the first slab, 64 = no wait for the requests.  The library is built
// without either.
#ifdef HIPNX_GEMM_TIMELINE
__device__ unsigned long long g_timeline[4096 * 8];
#define HIPNX_TL_STAMP(var) const unsigned long long var = wall_clock64()
#define HIPNX_TL_CLOCK(var) const unsigned long long var = clock64()
#else
#define HIPNX_TL_STAMP(var)
#define HIPNX_TL_CLOCK(var)
#endif
#ifndef HIPNX_PP_EXP
#define HIPNX_PP_EXP 0
#endif

// Swizzle of the [row][k] LDS layout of this kernel: the 16-byte chunk index XOR the part of
// lds_slot() that depends on the low four row bits only (the part that makes a fragment read of 16
// consecutive rows conflict-free).  A fragment's address is then one per-lane base per K step plus
// a compile-time multiple of 16 rows, which the LDS instruction carries as its immediate offset:
// two address registers per operand instead of one per fragment.
__device__ __forceinline__ int lds_slot16(int row, int chunk) {
  return chunk ^ (((row ^ (row >> 2)) & 1) | ((((row >> 1) ^ (row >> 2)) & 1) << 1) | ((((row >> 2) ^ (row >> 3)) & 1) << 2));
}

// a pointer every lane of the wave holds the same value of, moved to scalar registers
__device__ __forceinline__ const unsigned char *wave_uniform(const unsigned char *p) {
  const uint64_t u = (uint64_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)u), hi = __builtin_amdgcn_readfirstlane((uint32_t)(u >> 32));
  return (const unsigned char *)(((uint64_t)hi << 32) | lo);
}

// direct-to-LDS load with a wave-uniform 64-bit base and a 32-bit byte offset per lane
__device__ __forceinline__ void lds_dma16_at(const unsigned char *base, unsigned off, unsigned char *lds) {
  const unsigned dst = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(lptr_t)lds);
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off), "s"(base), "s"(dst) : "memory", "m0");
#pragma clang diagnostic pop
}

// K-inner rows [row0, row0 + ROWS) of an operand, ROWS x 128 B per slab, shared by NWAVES waves:
// PER instructions per wave, each filling 1 KiB of LDS (8 rows x 8 chunks).  Offsets are relative
// to the operand's first tile row (clamped into the matrix), so they fit 32 bits whenever
// 2 * ROWS * ld does (the host checks).
template <int ROWS, int NWAVES>
struct PPKInnerLoader {
  static constexpr int PER = ROWS / 8 / NWAVES;
  const unsigned char *base;
  unsigned off[PER];
  __device__ __forceinline__ void init(const unsigned char *g, int64_t ld, int64_t row0, int64_t rows_valid, int wave, int lane) {
    const int64_t first = row0 < rows_valid ? row0 : rows_valid - 1;
    base = wave_uniform(g + first * ld);
#pragma unroll
    for (int i = 0; i < PER; i++) {
      const int r = (wave + NWAVES * i) * 8 + (lane >> 3);
      int64_t gr = row0 + r;
      gr = gr < rows_valid ? gr : rows_valid - 1;
      off[i] = (unsigned)((gr - first) * ld) + lds_slot16(r, lane & 7) * 16;
    }
  }
  __device__ __forceinline__ void issue(int64_t kbyte0, unsigned char *lds, int wave) const {
    const unsigned char *b = base + kbyte0;
#pragma unroll
    for (int i = 0; i < PER; i++) lds_dma16_at(b, off[i], lds + (wave + NWAVES * i) * 1024);
  }
};

// K-outer columns [col0, col0 + ROWS) of an operand copied k-major ([k][ROWS * ES bytes]) for the
// transposing fragment reads (tr_slot layout of gemm_mfma.cuh), with 32-bit offsets from the tile's
// first column (clamped).
template <int ES, int ROWS, int NWAVES>
struct PPKOuterLoader {
  static constexpr int RBYTES = ROWS * ES;
  static constexpr int PER = ROWS / 8 / NWAVES;
  static_assert(RBYTES >= 256 || ES == 1, "a 2-byte k-row must span all LDS banks");
  const unsigned char *base;
  unsigned off[PER];
  __device__ __forceinline__ void init(const unsigned char *g, int64_t ld, int64_t col0, int64_t cols_valid, int wave, int lane) {
    const int64_t last = cols_valid * ES - 16;
    const int64_t first = col0 * ES <= last ? col0 * ES : last;
    base = wave_uniform(g + first);
#pragma unroll
    for (int i = 0; i < PER; i++) {
      const int o = (wave + NWAVES * i) * 1024 + lane * 16;
      const int k = o / RBYTES, slot = (o % RBYTES) / 16;
      int64_t byte = col0 * ES + tr_slot_w<ES, RBYTES>(k, slot) * 16;
      byte = byte <= last ? byte : last;
      off[i] = (unsigned)((int64_t)k * ld + (byte - first));
    }
  }
  __device__ __forceinline__ void issue(int64_t k0, int64_t ld, unsigned char *lds, int wave) const {
    const unsigned char *b = base + k0 * ld;
#pragma unroll
    for (int i = 0; i < PER; i++) lds_dma16_at(b, off[i], lds + (wave + NWAVES * i) * 1024);
  }
};

// TALL = false: wave tile 64 x 128 (waves 4 x 2); TALL = true: 128 x 64 (waves 2 x 4).  Either way
// waves 0-3 own the upper 128 rows.  A transposing fragment read moves 8 bytes per lane, a plain one
// 16, so the operand that needs the transposing reads should be the one with fewer fragments per
// wave: a K-outer right operand wants TALL, a K-outer left operand the other shape.
// BN = 128 halves the tile along N (wave tiles 64 x 64 or 128 x 32, 16 MFMAs per phase): twice the tiles for
// problems whose 256 x 256 grid leaves CUs idle, at a somewhat lower rate per tile.
template <int DT, bool L_KIN, bool R_KIN, bool TALL = false, bool PRIO = true, int BN_ = 256>
__global__ void __launch_bounds__(512)
gemm_pingpong_kernel(GemmArgs a) {
  typedef typename Mma16<DT>::acc_t acc_t;
  constexpr int NW = 8, BM = 256, BN = BN_, HALF = 128, TM16 = TALL ? 8 : 4, TN16 = TALL ? BN / 64 : BN / 32;
  constexpr int RPER = BN / 8 / NW;  // requests of the right operand per wave and memory phase (the left one's: 4)
  static_assert(BN == 256 || BN == 128, "tile widths of the two-group kernel");
  constexpr int STAGE = (BM + BN) * SLAB;
  constexpr int ES = (DT == HIPNX_S8) ? 1 : 2;
  static_assert(DT == HIPNX_BF16 || DT == HIPNX_F16 || DT == HIPNX_S8, "2-byte and 1-byte MFMA types");
  static_assert(L_KIN || ES == 2, "a K-outer left operand is split into two 128-row halves: 2-byte types only");
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  HIPNX_TL_STAMP(tl_start);

  int tm, tn;
  gemm_tile_position(a, blockIdx.x, tm, tn);
  const int64_t b = blockIdx.y;
  const unsigned char *lb = a.l + b * a.bs_l;
  const unsigned char *rb = a.r + b * a.bs_r;
  const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int grp = wave >> 2;                     // waves w and w + 4 share a SIMD
  const int wm = TALL ? (wave >> 2) * 128 : (wave >> 1) * 64;  // group 0: rows 0..127, group 1: 128..255
  const int wn = TALL ? (wave & 3) * (BN / 4) : (wave & 1) * (BN / 2);

  acc_t acc[TM16][TN16];
#pragma unroll
  for (int i = 0; i < TM16; i++)
#pragma unroll
    for (int j = 0; j < TN16; j++)
#pragma unroll
      for (int q = 0; q < 4; q++) acc[i][j][q] = 0;

  // right operand: the eight waves share its 32 instructions per slab (any split will do)
  PPKInnerLoader<BN, NW> rload;
  PPKOuterLoader<ES, BN, NW> rtr;
  if constexpr (R_KIN) rload.init(rb, a.ld_r, n0, a.N, wave, lane);
  else rtr.init(rb, a.ld_r, n0, a.N, wave, lane);
  // left operand: a group requests the half the OTHER group reads (it is the half that is free in
  // the group's own memory phase): group 0 rows 128..255, group 1 rows 0..127
  const int lhalf = grp ^ 1;
  constexpr int TR_ES = 2;
  PPKInnerLoader<HALF, 4> lload;
  PPKOuterLoader<TR_ES, HALF, 4> ltr;
  if constexpr (L_KIN) lload.init(lb, a.ld_l, m0 + lhalf * HALF, a.M, wave & 3, lane);
  else ltr.init(lb, a.ld_l, m0 + lhalf * HALF, a.M, wave & 3, lane);

  auto issue_r = [&](int stage, int64_t kbyte0) {
    unsigned char *sB = smem + stage * STAGE + BM * SLAB;
    if constexpr (R_KIN) rload.issue(kbyte0, sB, wave);
    else rtr.issue(kbyte0 / ES, a.ld_r, sB, wave);
  };
  auto issue_l = [&](int stage, int64_t kbyte0) {  // a half is HALF rows x 128 bytes in either layout
    unsigned char *sA = smem + stage * STAGE + lhalf * (HALF * SLAB);
    if constexpr (L_KIN) lload.issue(kbyte0, sA, wave & 3);
    else ltr.issue(kbyte0 / ES, a.ld_l, sA, wave & 3);
  };

  // fragment addresses within a stage: one per-lane base per operand and K step; the tile index
  // (16 rows = 2 KiB apart in the [row][k] layout) is a compile-time offset
  int a_rd[2], b_rd[2];
  if constexpr (L_KIN) {
    const int row = wm + (lane & 15);
#pragma unroll
    for (int ks = 0; ks < 2; ks++) a_rd[ks] = row * SLAB + lds_slot16(row, 4 * ks + (lane >> 4)) * 16;
  }
  if constexpr (R_KIN) {
    const int row = wn + (lane & 15);
#pragma unroll
    for (int ks = 0; ks < 2; ks++) b_rd[ks] = BM * SLAB + row * SLAB + lds_slot16(row, 4 * ks + (lane >> 4)) * 16;
  }
  auto read_l = [&](const unsigned char *st, int ks, int i) -> v4i {
    if constexpr (L_KIN) return *reinterpret_cast<const v4i *>(st + a_rd[ks] + i * (16 * SLAB));
    else return read_fragment_tr<TR_ES, HALF>(st + grp * (HALF * SLAB), (wm & (HALF - 1)) + 16 * i, ks, lane);  // two k-major halves
  };
  auto read_r = [&](const unsigned char *st, int ks, int j) -> v4i {
    if constexpr (R_KIN) return *reinterpret_cast<const v4i *>(st + b_rd[ks] + j * (16 * SLAB));
    else return read_fragment_tr<ES, BN>(st + BM * SLAB, wn + 16 * j, ks, lane);
  };

  const int nslab = (int)(a.Kb / SLAB);
  // prologue: slabs 0 and 1 into the two stages; slab 0 must have landed before the first phase
  issue_r(0, 0);
  issue_l(0, 0);
  if (nslab > 1) {
    issue_r(1, SLAB);
    issue_l(1, SLAB);
    wait_vmcnt<RPER + 4>();
  } else {
    wait_vmcnt<0>();
  }
  __builtin_amdgcn_s_barrier();
  if (grp) __builtin_amdgcn_s_barrier();  // group 1 runs one phase behind
  HIPNX_TL_STAMP(tl_walk);
  HIPNX_TL_CLOCK(tl_c0);

  v4i fa[TM16], fb[TN16];
  for (int s = 0; s < nslab; s++) {
    const unsigned char *cur = smem + (s & 1) * STAGE;
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
      // ---- memory phase: fragments of K step ks, then this phase's requests
#if HIPNX_PP_EXP & 32
      if (s == 0) {
#endif
#pragma unroll
      for (int i = 0; i < TM16; i++) fa[i] = read_l(cur, ks, i);
#pragma unroll
      for (int j = 0; j < TN16; j++) fb[j] = read_r(cur, ks, j);
#if HIPNX_PP_EXP & 32
      }
#endif
      bool issued = false, issued_r = false;
#if !(HIPNX_PP_EXP & 1)
      if (ks == 0) {
        if (s >= 1 && s + 1 < nslab) {
          issue_r((s + 1) & 1, (int64_t)(s + 1) * SLAB);
          issued_r = true;
        }
      } else if (grp == 0) {
        if (s >= 1 && s + 1 < nslab) {
          issue_l((s + 1) & 1, (int64_t)(s + 1) * SLAB);
          issued = true;
        }
      } else if (s + 2 < nslab) {
        issue_l(s & 1, (int64_t)(s + 2) * SLAB);
        issued = true;
      }
#endif
      // what I requested a memory phase ago (or in the prologue) has to be in LDS before the barrier
      // that publishes it; in the very first phase nothing is due yet (slab 1 is first read in phase 4)
#if !(HIPNX_PP_EXP & 64)
      if (issued) wait_vmcnt<4>();
      else if (issued_r) wait_vmcnt<RPER>();
      else if (!(s == 0 && ks == 0)) wait_vmcnt<0>();
#endif
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): my fragments are in registers
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      // ---- compute phase: 32 MFMAs from registers
      if constexpr (PRIO) __builtin_amdgcn_s_setprio(1);
      // (down one column of tiles and up the next: the left fragment stays where the column changes, so that every
      // MFMA shares an operand with the one before it -- worth 1 % of the clock the power management grants)
#pragma unroll
      for (int j = 0; j < TN16; j++)
#pragma unroll
        for (int ii = 0; ii < TM16; ii++) {
          const int i = (j & 1) ? TM16 - 1 - ii : ii;
          Mma16<DT>::step(acc[i][j], fb[j], fa[i]);
        }
      if constexpr (PRIO) __builtin_amdgcn_s_setprio(0);
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  if (!grp) __builtin_amdgcn_s_barrier();  // group 0 finishes one phase ahead
  HIPNX_TL_STAMP(tl_done);
  HIPNX_TL_CLOCK(tl_c1);

  const int64_t obase = b * a.M * a.N;
  switch (a.odt) {
#define HIPNX_EPI(T) case T: gemm_epilogue<DT, T, TM16, TN16>(acc, a.out, obase, a.M, a.N, m0 + wm, n0 + wn, lane, a.scale, a.scale_mode, smem + wave * 4096); break;
    HIPNX_EPI(HIPNX_BF16) HIPNX_EPI(HIPNX_F16) HIPNX_EPI(HIPNX_F32) HIPNX_EPI(HIPNX_F64) HIPNX_EPI(HIPNX_BF16_RNE)
    HIPNX_EPI(HIPNX_S8) HIPNX_EPI(HIPNX_U8) HIPNX_EPI(HIPNX_S16) HIPNX_EPI(HIPNX_U16)
    HIPNX_EPI(HIPNX_S32) HIPNX_EPI(HIPNX_U32) HIPNX_EPI(HIPNX_S64) HIPNX_EPI(HIPNX_U64)
#undef HIPNX_EPI
  }
#ifdef HIPNX_GEMM_TIMELINE
  if (threadIdx.x == 0 && blockIdx.x < 4096) {
    unsigned long long *p = g_timeline + (size_t)blockIdx.x * 8;
    p[0] = tl_start; p[1] = tl_walk; p[2] = tl_done; p[3] = wall_clock64(); p[4] = tl_c1 - tl_c0;
    p[5] = __builtin_amdgcn_s_getreg((31 << 11) | 20);  // XCC_ID
  }
#endif
}

// ---- the two-group walk on a 128 x 128 tile ----------------------------------------------------------
//
// Problems with fewer than a few hundred tiles of 256 x 128 take 128 x 128 tiles, one per CU.  The one-group
// kernel (gemm_pipelined_kernel) has a single wave per SIMD there, which reads its fragments and issues its
// MFMAs in turn: 1600-2100 clocks per slab for 512 clocks of MFMA work.  Here two groups of four waves walk
// the same tile, each with the one-group kernel's wave tiles of 64 x 64 (so no more LDS traffic than there),
// and share K: group 0 takes the even slabs, group 1 the odd ones.  In phase p the group p % 2 reads the 16
// fragments of slab p and requests slab p + 3 while the other group issues the 32 MFMAs of slab p - 1; the
// two partial sums meet in LDS at the end, where each group takes over the finished half (32 rows of every
// wave tile) it then scales, converts and stores.
//
// A slab (both operands) is 32 KiB, the NSTAGE LDS stages hold slabs p .. p + NSTAGE - 1.  Slab p + NSTAGE - 1
// lands in the stage of slab p - 1, whose last reader waited for its fragments before the barrier that opened
// phase p.  The waves that requested a slab wait for it at the end of the memory phase before the one that
// reads it (vmcnt: all but their (NSTAGE - 2) / 2 younger slabs), and the barrier behind that wait publishes it.
//
// BM_ = BN_ = 64 is the shape for a few rows against a long K-inner weight matrix: 64 rows of the weights per
// work-group (a slab of them is 8 KiB, as is a slab of the rows, which comes from L2), either eight stages of one
// slab or, with SPP = 2, four stages of two slabs -- a phase then covers 256 bytes of K and there are half as
// many barriers.  The ring's depth hardly matters there (four, six and eight stages measured alike): a
// work-group takes in as many bytes of the rows as of the weights, and a CU's intake is what bounds it.
template <int DT, bool L_KIN, bool R_KIN, int BM_ = 128, int BN_ = 128, int NSTAGE_ = 4, int SPP = 1>
__global__ void __launch_bounds__(512)
gemm_pingpong128_kernel(GemmArgs a) {
  typedef typename Mma16<DT>::acc_t acc_t;
  constexpr int BM = BM_, BN = BN_, TM16 = BM / 32, TN16 = BN / 32, NSTAGE = NSTAGE_, AHEAD = NSTAGE - 1;
  static_assert((BM == 128 || BM == 64) && (BN == 128 || BN == 64) && NSTAGE % 2 == 0 && NSTAGE >= 4, "tile extents of 64 or 128, an even number of stages");
  static_assert((BM == 128 || L_KIN || DT == HIPNX_S8) && (BN == 128 || R_KIN || DT == HIPNX_S8),
                "a 64-row 2-byte operand is K-inner (a k-row of a K-outer one must span all LDS banks)");
  constexpr int LREQ = BM / 32, RREQ = BN / 32, REQ = SPP * (LREQ + RREQ);  // requests per wave and phase
  // a stage holds the SPP slabs of one phase, each as [left rows | right rows]
  constexpr int SLAB1 = (BM + BN) * SLAB, STAGE = SPP * SLAB1, KS = 2 * SPP;
  constexpr int ES = (DT == HIPNX_S8) ? 1 : 2;
  static_assert(DT == HIPNX_BF16 || DT == HIPNX_F16 || DT == HIPNX_S8 || (DT == HIPNX_F32 && L_KIN && R_KIN),
                "2-byte MFMA types and int8; f32 with K-inner operands");
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  HIPNX_TL_STAMP(tl_start);

  int tm, tn;
  gemm_tile_position(a, blockIdx.x, tm, tn);
  const int64_t b = blockIdx.y;
  const unsigned char *lb = a.l + b * a.bs_l;
  const unsigned char *rb = a.r + b * a.bs_r;
  const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int grp = wave >> 2, w4 = wave & 3;  // waves w and w + 4 share a SIMD and a wave tile
  const int wm = (w4 >> 1) * (BM / 2), wn = (w4 & 1) * (BN / 2);

  acc_t acc[TM16][TN16];
#pragma unroll
  for (int i = 0; i < TM16; i++)
#pragma unroll
    for (int j = 0; j < TN16; j++)
#pragma unroll
      for (int q = 0; q < 4; q++) acc[i][j][q] = 0;

  // the four waves of the memory group request a whole slab: LREQ + RREQ instructions per wave
  struct Unused {};  // (only the loader of an operand's own layout is instantiated)
  std::conditional_t<L_KIN, PPKInnerLoader<BM, 4>, Unused> lkin;
  std::conditional_t<R_KIN, PPKInnerLoader<BN, 4>, Unused> rkin;
  std::conditional_t<L_KIN, Unused, PPKOuterLoader<ES, BM, 4>> lkout;
  std::conditional_t<R_KIN, Unused, PPKOuterLoader<ES, BN, 4>> rkout;
  if constexpr (L_KIN) lkin.init(lb, a.ld_l, m0, a.M, w4, lane);
  else lkout.init(lb, a.ld_l, m0, a.M, w4, lane);
  if constexpr (R_KIN) rkin.init(rb, a.ld_r, n0, a.N, w4, lane);
  else rkout.init(rb, a.ld_r, n0, a.N, w4, lane);
  // (below, "slab" stands for the SPP slabs of one phase)
  auto issue = [&](int slab) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < SPP; u++) {
      unsigned char *dst = smem + (slab % NSTAGE) * STAGE + u * SLAB1;
      const int64_t kbyte0 = ((int64_t)slab * SPP + u) * SLAB;
      if constexpr (L_KIN) lkin.issue(kbyte0, dst, w4);
      else lkout.issue(kbyte0 / ES, a.ld_l, dst, w4);
      if constexpr (R_KIN) rkin.issue(kbyte0, dst + BM * SLAB, w4);
      else rkout.issue(kbyte0 / ES, a.ld_r, dst + BM * SLAB, w4);
    }
  };

  int a_rd[2], b_rd[2];
  if constexpr (L_KIN) {
    const int row = wm + (lane & 15);
#pragma unroll
    for (int ks = 0; ks < 2; ks++) a_rd[ks] = row * SLAB + lds_slot16(row, 4 * ks + (lane >> 4)) * 16;
  }
  if constexpr (R_KIN) {
    const int row = wn + (lane & 15);
#pragma unroll
    for (int ks = 0; ks < 2; ks++) b_rd[ks] = BM * SLAB + row * SLAB + lds_slot16(row, 4 * ks + (lane >> 4)) * 16;
  }

  const int nslab = (int)(a.Kb / (SPP * SLAB));  // the host sends whole phases only
  v4i fa[KS][TM16], fb[KS][TN16];
  auto mem_phase = [&](int p) __attribute__((always_inline)) {
    const unsigned char *cur = smem + (p % NSTAGE) * STAGE;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      const unsigned char *sl = cur + (ks >> 1) * SLAB1;
#pragma unroll
      for (int i = 0; i < TM16; i++) {
        if constexpr (L_KIN) fa[ks][i] = *reinterpret_cast<const v4i *>(sl + a_rd[ks & 1] + i * (16 * SLAB));
        else fa[ks][i] = read_fragment_tr<ES, BM>(sl, wm + 16 * i, ks & 1, lane);
      }
#pragma unroll
      for (int j = 0; j < TN16; j++) {
        if constexpr (R_KIN) fb[ks][j] = *reinterpret_cast<const v4i *>(sl + b_rd[ks & 1] + j * (16 * SLAB));
        else fb[ks][j] = read_fragment_tr<ES, BN>(sl + BM * SLAB, wn + 16 * j, ks & 1, lane);
      }
    }
    // this group's requests in flight, oldest first: slabs p + 1, p + 3, .. p + AHEAD; slab p + 1 is read next phase
    if (p + AHEAD < nslab) {
      issue(p + AHEAD);
      wait_vmcnt<(AHEAD - 1) / 2 * REQ>();
    } else {
      wait_vmcnt<0>();
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the fragments are in registers
  };
  auto compute_phase = [&]() __attribute__((always_inline)) {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int ks = 0; ks < KS; ks++)
#pragma unroll
      for (int j = 0; j < TN16; j++)
#pragma unroll
        for (int ii = 0; ii < TM16; ii++) {
          const int i = (j & 1) ? TM16 - 1 - ii : ii;  // down one column of tiles and up the next
          Mma16<DT>::step(acc[i][j], fb[ks][j], fa[ks][i]);
        }
    __builtin_amdgcn_s_setprio(0);
    __builtin_amdgcn_sched_barrier(0);
  };

  // prologue: slabs 0 .. AHEAD - 1, slab q by the group (q + 1) % 2 as in the walk (a group requests what the
  // other one reads); group 1 holds slab 0 and waits for it here, slab 1 is awaited by group 0 in phase 0
#pragma unroll
  for (int q = 0; q < AHEAD; q++)
    if (q < nslab && ((q + 1) & 1) == grp) issue(q);
  if (grp == 1) {
    if (nslab >= AHEAD) wait_vmcnt<(AHEAD - 1) / 2 * REQ>();
    else wait_vmcnt<0>();
  }
  __builtin_amdgcn_s_barrier();
  HIPNX_TL_STAMP(tl_walk);
  HIPNX_TL_CLOCK(tl_c0);

  // phases 0 .. nslab, every wave passes the barrier that ends each of them
  if (grp == 0) {
    for (int p = 0; p <= nslab; p += 2) {
      if (p < nslab) mem_phase(p);
      __builtin_amdgcn_s_barrier();
      if (p + 1 > nslab) break;
      compute_phase();
      __builtin_amdgcn_s_barrier();
    }
  } else {
    for (int p = 0; p <= nslab; p += 2) {
      __builtin_amdgcn_s_barrier();
      if (p + 1 > nslab) break;
      if (p + 1 < nslab) mem_phase(p + 1);
      __builtin_amdgcn_s_barrier();
      if (p + 1 < nslab) compute_phase();
    }
  }

  HIPNX_TL_STAMP(tl_done);
  HIPNX_TL_CLOCK(tl_c1);
  // the two partial sums: every wave hands the half of its tile the other group finishes to that group
  // (TM16 / 2 x TN16 accumulator tiles of 1 KiB) and adds what it is handed
  {
    constexpr int HM = TM16 / 2, XBYTES = HM * TN16 * 1024;
    unsigned char *mine = smem + wave * XBYTES, *theirs = smem + (wave ^ 4) * XBYTES;
    // (a branch per group rather than a selection per tile: the accumulators must keep constant indices)
    if (grp == 0) {
#pragma unroll
      for (int i = 0; i < HM; i++)
#pragma unroll
        for (int j = 0; j < TN16; j++) *reinterpret_cast<acc_t *>(mine + (i * TN16 + j) * 1024 + lane * 16) = acc[i + HM][j];
    } else {
#pragma unroll
      for (int i = 0; i < HM; i++)
#pragma unroll
        for (int j = 0; j < TN16; j++) *reinterpret_cast<acc_t *>(mine + (i * TN16 + j) * 1024 + lane * 16) = acc[i][j];
    }
    __syncthreads();
    acc_t fin[HM][TN16];
#pragma unroll
    for (int i = 0; i < HM; i++)
#pragma unroll
      for (int j = 0; j < TN16; j++) fin[i][j] = *reinterpret_cast<const acc_t *>(theirs + (i * TN16 + j) * 1024 + lane * 16);
    // the even slabs' sum first, as a single walk over K would have it
    if (grp == 0) {
#pragma unroll
      for (int i = 0; i < HM; i++)
#pragma unroll
        for (int j = 0; j < TN16; j++) fin[i][j] = acc[i][j] + fin[i][j];
    } else {
#pragma unroll
      for (int i = 0; i < HM; i++)
#pragma unroll
        for (int j = 0; j < TN16; j++) fin[i][j] = fin[i][j] + acc[i + HM][j];
    }
    const int64_t obase = b * a.M * a.N;
    unsigned char *turn = smem + 8 * XBYTES + wave * 4096;  // past the exchanged halves, which the other group may still be reading
    static_assert(8 * XBYTES + 8 * 4096 <= NSTAGE * STAGE, "the exchange and the epilogue's turn buffers fit the stages");
    switch (a.odt) {
#define HIPNX_EPI(T) case T: gemm_epilogue<DT, T, HM, TN16>(fin, a.out, obase, a.M, a.N, m0 + wm + grp * (16 * HM), n0 + wn, lane, a.scale, a.scale_mode, turn); break;
      HIPNX_EPI(HIPNX_BF16) HIPNX_EPI(HIPNX_F16) HIPNX_EPI(HIPNX_F32) HIPNX_EPI(HIPNX_F64) HIPNX_EPI(HIPNX_BF16_RNE)
      HIPNX_EPI(HIPNX_S8) HIPNX_EPI(HIPNX_U8) HIPNX_EPI(HIPNX_S16) HIPNX_EPI(HIPNX_U16)
      HIPNX_EPI(HIPNX_S32) HIPNX_EPI(HIPNX_U32) HIPNX_EPI(HIPNX_S64) HIPNX_EPI(HIPNX_U64)
#undef HIPNX_EPI
    }
  }
#ifdef HIPNX_GEMM_TIMELINE
  if (threadIdx.x == 0 && blockIdx.x < 4096) {
    unsigned long long *p = g_timeline + (size_t)blockIdx.x * 8;
    p[0] = tl_start; p[1] = tl_walk; p[2] = tl_done; p[3] = wall_clock64(); p[4] = tl_c1 - tl_c0;
    p[5] = __builtin_amdgcn_s_getreg((31 << 11) | 20);  // XCC_ID
  }
#endif
}

}  // namespace hipnx
