// Contraction of a few rows against a long matrix:  out[b, m, n] = sum_k l[b, m, k] * r[b, n, k]
// with M <= 64 and both operands K-inner -- the shape of a linear layer applied to a small batch
// (x {64, K} against weights {N, K}).  Every weight is used once, so the kernel is a stream of r
// from HBM, bound by the bytes in flight: a wave's walk over K is serial, so what it cannot keep
// in flight is paid in latency (measured with 16 KiB in flight per wave: 12 us for 45 MB with
// everything but the loads switched off).
//
// K is walked in runs of 512 bytes per row.  A *group* is what one run needs: its slice of l and
// its slice of r.  Groups are requested DEPTH-1 runs ahead, strictly in the order in which they
// are needed -- vmcnt counts in order, so a request that is needed early must never sit behind
// requests that are needed late.  Everything is plain loads into registers, so the compiler
// counts the waits (vmcnt(n) leaving the younger groups in flight); no hand-counted waits here.
//   * r never passes through LDS.  A wave owns 16 rows of r and loads them straight into MFMA
//     operand registers (lane -> row lane%16, 16 bytes at chunk lane/16 of a 64-byte K step): 8
//     loads per run, back to back.
//   * l (at most 64 rows, L2-resident) is shared by the waves of a work-group through LDS: each
//     lane loads 16-byte pieces of full cache lines (8 per run), keeps them in registers until the
//     run comes up, then writes them into the swizzled [row][k] layout of the pipelined kernel
//     (lds_slot).  Two LDS stages of 32 KiB, one barrier per run.
//   * per run and wave: 32 LDS fragment reads (two K steps ahead of their MFMAs), 32 MFMAs.
// One wave per SIMD (4 waves), so the 512 registers of a lane hold DEPTH groups.
#include "gemm_launch.cuh"

namespace hipnx {

constexpr int RUN = 512;              // bytes of K per row per run
constexpr int RUN_STEPS = RUN / 64;   // K steps (64 bytes) per run
constexpr int RUN_SLABS = RUN / SLAB; // 128-byte slabs of l per run
constexpr int ROWS_DEPTH = 3;         // groups held in registers (DEPTH-1 in flight + 1 in use); four no
                                      // longer fit the 256 plain VGPRs, and a loaded value that is moved to
                                      // another register file must be waited for at once

template <int DT, int NW, int CHUNK>
__global__ void __launch_bounds__(NW * 64) gemm_rows_kernel(GemmArgs a) {
  typedef typename Mma16<DT>::acc_t acc_t;
  constexpr int DEPTH = ROWS_DEPTH;
  constexpr int LSLAB = 64 * SLAB;    // bytes of one slab of l in LDS
  constexpr int STAGE = 64 * RUN;     // one run of l
  constexpr int LPER = 8 / NW;        // 1 KiB pieces (8 rows x 128 B) of a slab per wave
  static_assert(8 % NW == 0, "a slab of l is 8 pieces of 8 rows");
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];  // 2 stages
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t b = blockIdx.y;
  const unsigned char *lb = a.l + b * a.bs_l;
  const unsigned char *rb = a.r + b * a.bs_r;
  const int64_t n0 = (int64_t)blockIdx.x * (NW * 16) + wave * 16;

  // r: this lane's row and chunk (rows past N re-read the last row; never stored)
  int64_t gn = n0 + (lane & 15);
  gn = gn < a.N ? gn : a.N - 1;
  const unsigned char *rp = rb + gn * a.ld_r + (lane >> 4) * 16;
  // l: piece p of a slab is rows 8p .. 8p+7; this lane moves the chunk that belongs at LDS slot
  // lane%8 of row 8p + lane/8 (rows past M re-read the last row; their results are never stored)
  const unsigned char *lp[LPER];
  int lds_off[LPER];
#pragma unroll
  for (int i = 0; i < LPER; i++) {
    const int row = (wave + NW * i) * 8 + (lane >> 3);
    const int64_t gm = row < a.M ? row : a.M - 1;
    lp[i] = lb + gm * a.ld_l + lds_slot(row, lane & 7) * 16;  // the XOR map is an involution
    lds_off[i] = row * SLAB + (lane & 7) * 16;
  }

  acc_t acc[4][1];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int q = 0; q < 4; q++) acc[i][0][q] = 0;

  const int nrun = (int)(a.Kb / RUN);  // a multiple of CHUNK (the host checks)
  v4i w[DEPTH][RUN_STEPS];             // r: one run per slot
  v4i xl[DEPTH][RUN_SLABS * LPER];     // l: this lane's pieces of one run per slot
  auto request = [&](v4i (&wd)[RUN_STEPS], v4i (&xd)[RUN_SLABS * LPER], int run) {
    const int64_t kb = (int64_t)run * RUN;
#pragma unroll
    for (int q = 0; q < RUN_SLABS; q++)
#pragma unroll
      for (int i = 0; i < LPER; i++) xd[q * LPER + i] = *reinterpret_cast<const v4i *>(lp[i] + kb + q * SLAB);
#pragma unroll
    for (int kk = 0; kk < RUN_STEPS; kk++) wd[kk] = *reinterpret_cast<const v4i *>(rp + kb + kk * 64);
  };
  auto compute = [&](const v4i (&wr)[RUN_STEPS], const v4i (&xr)[RUN_SLABS * LPER], int run) {
    unsigned char *st = smem + (run & 1) * STAGE;
    // this run's l goes to LDS; the stage was last read two runs ago, i.e. before the barrier
    // every wave passed at the top of the previous run
#pragma unroll
    for (int q = 0; q < RUN_SLABS; q++)
#pragma unroll
      for (int i = 0; i < LPER; i++) *reinterpret_cast<v4i *>(st + q * LSLAB + lds_off[i]) = xr[q * LPER + i];
    __syncthreads();
    // l fragments run two K steps ahead of their MFMAs (ring of three)
    v4i x[3][4];
    auto read_l = [&](int kk, int i) -> v4i {  // K step kk of the run = K step kk%2 of slab kk/2
      const int row = 16 * i + (lane & 15);
      return *reinterpret_cast<const v4i *>(st + (kk / 2) * LSLAB + row * SLAB + lds_slot(row, 4 * (kk % 2) + (lane >> 4)) * 16);
    };
#pragma unroll
    for (int i = 0; i < 4; i++) x[0][i] = read_l(0, i);
#pragma unroll
    for (int i = 0; i < 4; i++) x[1][i] = read_l(1, i);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int kk = 0; kk < RUN_STEPS; kk++) {
      if (kk + 2 < RUN_STEPS) {
#pragma unroll
        for (int i = 0; i < 4; i++) x[(kk + 2) % 3][i] = read_l(kk + 2, i);
      }
#pragma unroll
      for (int i = 0; i < 4; i++) Mma16<DT>::step(acc[i][0], wr[kk], x[kk % 3][i]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // K is walked in chunks of CHUNK runs written out straight-line: inside a loop over runs the
  // compiler's wait insertion gives up at the loop header and drains every load in flight (it
  // emitted vmcnt(7) at the top of each trip), which is exactly the depth this kernel lives on.
  // A chunk ramps up and drains by itself, so the loop over chunks carries nothing in flight.
  for (int c = 0; c < nrun; c += CHUNK) {
#pragma unroll
    for (int d = 0; d < DEPTH - 1; d++) request(w[d], xl[d], c + d);
#pragma unroll
    for (int j = 0; j < CHUNK; j++) {
      // the group DEPTH-1 runs ahead goes into the slot the previous run has just freed
      if (j + DEPTH - 1 < CHUNK) request(w[(j + DEPTH - 1) % DEPTH], xl[(j + DEPTH - 1) % DEPTH], c + j + DEPTH - 1);
      compute(w[j % DEPTH], xl[j % DEPTH], c + j);
    }
  }

  const int64_t obase = b * a.M * a.N;
  switch (a.odt) {
#define HIPNX_EPI(T) case T: gemm_epilogue<DT, T, 4, 1>(acc, a.out, obase, a.M, a.N, 0, n0, lane, a.scale, a.scale_mode); break;
    HIPNX_EPI(HIPNX_BF16) HIPNX_EPI(HIPNX_F16) HIPNX_EPI(HIPNX_F32) HIPNX_EPI(HIPNX_F64) HIPNX_EPI(HIPNX_BF16_RNE)
    HIPNX_EPI(HIPNX_S8) HIPNX_EPI(HIPNX_U8) HIPNX_EPI(HIPNX_S16) HIPNX_EPI(HIPNX_U16)
    HIPNX_EPI(HIPNX_S32) HIPNX_EPI(HIPNX_U32) HIPNX_EPI(HIPNX_S64) HIPNX_EPI(HIPNX_U64)
#undef HIPNX_EPI
  }
}

template <int DT>
static int launch_rows_dt(const hipnx_ctx *ctx, GemmArgs a, int64_t batch) {
  constexpr int NW = 4, CHUNK = 8;
  constexpr int smem = 2 * 64 * RUN;
  auto kern = gemm_rows_kernel<DT, NW, CHUNK>;
  static bool configured = false;
  if (!configured) {
    HIPNX_HIP(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem));
    configured = true;
  }
  dim3 grid((unsigned)((a.N + NW * 16 - 1) / (NW * 16)), (unsigned)batch), block(NW * 64);
  hipLaunchKernelGGL(kern, grid, block, smem, ctx->stream, a);
  HIPNX_HIP(hipGetLastError());
  return HIPNX_OK;
}

// M <= 64, both operands K-inner, Kb a multiple of RUN * CHUNK = 4096
int launch_gemm_rows(const hipnx_ctx *ctx, int dt, GemmArgs a, int64_t batch) {
  switch (dt) {
    case HIPNX_BF16: return launch_rows_dt<HIPNX_BF16>(ctx, a, batch);
    case HIPNX_F16: return launch_rows_dt<HIPNX_F16>(ctx, a, batch);
    case HIPNX_F32: return launch_rows_dt<HIPNX_F32>(ctx, a, batch);
    default: return launch_rows_dt<HIPNX_S8>(ctx, a, batch);
  }
}

}  // namespace hipnx
