// Launcher shared by the per-type translation units of the pipelined MFMA kernel (one unit per
// operand type keeps the build parallel).
#pragma once
#include "gemm_mfma.cuh"
#include "gemm_pingpong.cuh"
#include "internal.h"

namespace hipnx {

// tile configurations of gemm_pipelined_kernel<DT, WM, WN, TM, TN, ...>
enum {
  GEMM_CFG_256x128 = 3,  // 256 x 128, the two-group kernel with half-width wave tiles: 2-byte types whose 256 x 256 grid is too small
  GEMM_CFG_256 = 0,  // 256 x 256, 8 waves (4 x 2, each 64 x 128): large square-ish problems
  GEMM_CFG_128 = 1,  // 128 x 128: mid-size and batched problems; 4 waves (2 x 2, each 64 x 64), or two such groups sharing K
  GEMM_CFG_64x32 = 2, // 64 x 32, 2 waves: few rows against a long weight matrix (HBM streaming)
  GEMM_CFG_64x128 = 4, // 64 x 128, 4 waves (2 x 2, each 32 x 64): f32 with up to 64 rows
  GEMM_CFG_128x32 = 5  // 128 x 32, 4 waves (4 x 1, each 32 x 32): many rows against up to 32 columns (a layer with a few outputs)
};

int launch_gemm_bf16(const hipnx_ctx *ctx, int cfg, bool l_kin, bool r_kin, GemmArgs a, int64_t batch);
int launch_gemm_f16(const hipnx_ctx *ctx, int cfg, bool l_kin, bool r_kin, GemmArgs a, int64_t batch);
int launch_gemm_f32(const hipnx_ctx *ctx, int cfg, bool l_kin, bool r_kin, GemmArgs a, int64_t batch);
int launch_gemm_s8(const hipnx_ctx *ctx, int cfg, bool l_kin, bool r_kin, GemmArgs a, int64_t batch);
int launch_gemm_f64(const hipnx_ctx *ctx, int cfg, bool l_kin, bool r_kin, GemmArgs a, int64_t batch);  // (tiles of 128 rows or fewer)

template <int DT, int WM, int WN, int TM, int TN, bool LK, bool RK, int NSTAGE = 2>
static int launch_one(const hipnx_ctx *ctx, GemmArgs a, int64_t batch) {
  constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
  constexpr int smem_max = NSTAGE * (BM + BN) * SLAB;
  // a K of one slab only ever touches the first stage: the rest of the LDS stays with other work-groups
  const int smem = a.Kb <= SLAB ? (BM + BN) * SLAB : smem_max;
  auto kern = gemm_pipelined_kernel<DT, WM, WN, TM, TN, LK, RK, NSTAGE>;
  HIPNX_ALLOW_DYNAMIC_LDS(ctx, kern, smem_max);
  a.tiles_m = (int)((a.M + BM - 1) / BM);
  a.tiles_n = (int)((a.N + BN - 1) / BN);
  a.group_m = gemm_group_m(a.tiles_m, a.tiles_n);
  dim3 grid((unsigned)(a.tiles_m * a.tiles_n), (unsigned)batch), block(WM * WN * 64);
  hipLaunchKernelGGL(kern, grid, block, smem, ctx->stream, a);
  HIPNX_HIP(hipGetLastError());
  return HIPNX_OK;
}

// the two-group 256 x 256 kernel (gemm_pingpong.cuh): bf16 / f16 in every layout, s8 with a K-inner
// left operand; its request offsets are 32 bits from the tile's first row or column
template <int DT, bool LK, bool RK, int BN = 256>
static int launch_pingpong(const hipnx_ctx *ctx, GemmArgs a, int64_t batch) {
  constexpr bool TALL = LK && !RK;  // the operand read by transposing loads gets the fewer fragments
  constexpr int smem = 2 * (256 + BN) * SLAB;
  auto kern = gemm_pingpong_kernel<DT, LK, RK, TALL, true, BN>;
  HIPNX_ALLOW_DYNAMIC_LDS(ctx, kern, smem);
  a.tiles_m = (int)((a.M + 255) / 256);
  a.tiles_n = (int)((a.N + BN - 1) / BN);
  a.group_m = gemm_group_m(a.tiles_m, a.tiles_n);
  dim3 grid((unsigned)(a.tiles_m * a.tiles_n), (unsigned)batch), block(512);
  hipLaunchKernelGGL(kern, grid, block, smem, ctx->stream, a);
  HIPNX_HIP(hipGetLastError());
  return HIPNX_OK;
}

// the two-group kernel on 128 x 128 tiles (four LDS stages of 32 KiB) or 64 x 64 tiles (eight of 16 KiB):
// one work-group per CU
template <int DT, bool LK, bool RK, int BM = 128, int BN = 128, int NSTAGE = 4, int SPP = 1>
static int launch_pingpong128(const hipnx_ctx *ctx, GemmArgs a, int64_t batch) {
  constexpr int smem = NSTAGE * SPP * (BM + BN) * SLAB;
  auto kern = gemm_pingpong128_kernel<DT, LK, RK, BM, BN, NSTAGE, SPP>;
  HIPNX_ALLOW_DYNAMIC_LDS(ctx, kern, smem);
  a.tiles_m = (int)((a.M + BM - 1) / BM);
  a.tiles_n = (int)((a.N + BN - 1) / BN);
  a.group_m = gemm_group_m(a.tiles_m, a.tiles_n);
  dim3 grid((unsigned)(a.tiles_m * a.tiles_n), (unsigned)batch), block(512);
  hipLaunchKernelGGL(kern, grid, block, smem, ctx->stream, a);
  HIPNX_HIP(hipGetLastError());
  return HIPNX_OK;
}

template <int DT, bool LK, bool RK>
static int launch_cfg(const hipnx_ctx *ctx, int cfg, const GemmArgs &a, int64_t batch) {
  if constexpr (DT == HIPNX_F64) {
    // f64 accumulators take two registers an element: wave tiles of 64 x 64 at most, on the one-group kernel (an f64
    // slab is 4096 clocks of MFMA work, as an f32 one: the data movement beside it is a few hundred)
    switch (cfg) {
      case GEMM_CFG_128x32:
        if constexpr (LK && RK) return launch_one<DT, 4, 1, 1, 1, LK, RK, 4>(ctx, a, batch);
        else return launch_one<DT, 4, 1, 1, 1, LK, RK>(ctx, a, batch);
      case GEMM_CFG_64x128: return launch_one<DT, 2, 2, 1, 2, LK, RK>(ctx, a, batch);
      case GEMM_CFG_64x32:
        if constexpr (LK && RK) return launch_one<DT, 2, 1, 1, 1, LK, RK, 6>(ctx, a, batch);
        else return launch_one<DT, 2, 1, 1, 1, LK, RK>(ctx, a, batch);
      default: {
        const int64_t groups = ((a.M + 127) / 128) * ((a.N + 127) / 128) * batch;
        if constexpr (LK && RK)
          if (a.Kb >= 4 * SLAB && groups <= ctx->num_cus) return launch_one<DT, 2, 2, 2, 2, LK, RK, 4>(ctx, a, batch);
        return launch_one<DT, 2, 2, 2, 2, LK, RK>(ctx, a, batch);
      }
    }
  } else
  switch (cfg) {
    case GEMM_CFG_256:
      if constexpr (DT == HIPNX_BF16 || DT == HIPNX_F16 || (DT == HIPNX_S8 && LK)) {
        // 256 rows (or 128 k-rows) times the row pitch must fit the 32-bit request offsets
        if (a.ld_l < (1ll << 23) && a.ld_r < (1ll << 23)) return launch_pingpong<DT, LK, RK>(ctx, a, batch);
      }
      return launch_one<DT, 4, 2, 2, 4, LK, RK>(ctx, a, batch);
    case GEMM_CFG_256x128:
      if constexpr (DT == HIPNX_BF16 || DT == HIPNX_F16) {
        if (a.ld_l < (1ll << 23) && a.ld_r < (1ll << 23)) return launch_pingpong<DT, LK, RK, 128>(ctx, a, batch);
      }
      return launch_one<DT, 2, 2, 2, 2, LK, RK>(ctx, a, batch);
    case GEMM_CFG_128: {
      // one wave per SIMD and 0.25 us of MFMA work per slab: two stages cannot cover the latency of the next
      // slab's requests (measured 2100 clocks per slab, 1580 with four stages); four stages where every
      // operand is copied straight into LDS (the condition of the kernel's L_TR / R_TR)
      constexpr int ES = DT == HIPNX_S8 ? 1 : DT == HIPNX_F32 ? 4 : 2;
      constexpr bool tr = ES <= 2 && 128 * ES >= 256;
      // From 8 slabs of K on, the two-group kernel (2-byte types and int8; f32 with both operands K-inner): 730 clocks per
      // slab against the 1600-2100 below.  It holds a CU's LDS alone, so for the 2-byte types only where no
      // second work-group would share the CU; int8 has no wider two-group tile to fall back on and takes it
      // for every grid (2048 x 4096 x 4096, 512 tiles: 52 -> 42 us).
      if constexpr (DT == HIPNX_BF16 || DT == HIPNX_F16 || DT == HIPNX_S8 || (DT == HIPNX_F32 && LK && RK)) {
        const int64_t groups = ((a.M + 127) / 128) * ((a.N + 127) / 128) * batch;
        if (a.Kb >= 8 * SLAB && a.ld_l < (1ll << 23) && a.ld_r < (1ll << 23) && (DT == HIPNX_S8 || DT == HIPNX_F32 || groups <= ctx->num_cus))
          return launch_pingpong128<DT, LK, RK>(ctx, a, batch);
      }
      if constexpr ((LK || tr) && (RK || tr)) {
        // (128 KiB of LDS: one work-group per CU, so only where the grid has no second one to give it)
        const int64_t groups = ((a.M + 127) / 128) * ((a.N + 127) / 128) * batch;
        if (a.Kb >= 4 * SLAB && groups <= ctx->num_cus) return launch_one<DT, 2, 2, 2, 2, LK, RK, 4>(ctx, a, batch);
      }
      return launch_one<DT, 2, 2, 2, 2, LK, RK>(ctx, a, batch);
    }
    case GEMM_CFG_128x32:
      if constexpr (LK && RK) return launch_one<DT, 4, 1, 1, 1, LK, RK, 4>(ctx, a, batch);
      else return launch_one<DT, 4, 1, 1, 1, LK, RK>(ctx, a, batch);
    case GEMM_CFG_64x128:
      if constexpr (DT == HIPNX_F32) return launch_one<DT, 2, 2, 1, 2, LK, RK>(ctx, a, batch);
      return launch_one<DT, 2, 2, 2, 2, LK, RK>(ctx, a, batch);
    default:
      // K-inner 2-byte operands and int8 in either layout: the two-group kernel on 64 x 64 tiles -- 64 rows of the weights per
      // work-group, their slabs requested three phases (six slabs) ahead, two slabs per phase where K allows
      // (int8 64 x 11008 x 4096: kernel 13.0 us; the 64 x 32 tiles below 18.7 us)
      if constexpr ((LK && RK && (DT == HIPNX_BF16 || DT == HIPNX_F16)) || DT == HIPNX_S8) {
        if (a.Kb >= 8 * SLAB && a.ld_l < (1ll << 24) && a.ld_r < (1ll << 24)) {
          if constexpr (DT == HIPNX_S8 && !RK) {
            // int8 weights stored [K, N]: a k-row of a 64-column tile is half a cache line; where 128-column tiles
            // still give 3/8 of the CUs work they stream the weights as fast as the K-inner layout
            // (64 x 32000 x 4096: 50 -> 28 us; with 32 such tiles, 64 x 4096 x 4096, they are slower: 12 -> 18 us)
            if (((a.N + 127) / 128) * batch * 8 >= (int64_t)ctx->num_cus * 3) return launch_pingpong128<DT, LK, RK, 64, 128, 6, 1>(ctx, a, batch);
          }
          if (a.Kb % (2 * SLAB) == 0) return launch_pingpong128<DT, LK, RK, 64, 64, 4, 2>(ctx, a, batch);
          return launch_pingpong128<DT, LK, RK, 64, 64, 8, 1>(ctx, a, batch);
        }
      }
      // streaming a long weight matrix past a few rows is bound by the bytes in flight: six
      // stages (five slabs of 12 KiB requested ahead per work-group) when both operands are copied
      // straight into LDS
      if constexpr (LK && RK) return launch_one<DT, 2, 1, 1, 1, LK, RK, 6>(ctx, a, batch);
      else return launch_one<DT, 2, 1, 1, 1, LK, RK>(ctx, a, batch);
  }
}

template <int DT>
static int launch_layouts(const hipnx_ctx *ctx, int cfg, bool l_kin, bool r_kin, const GemmArgs &a, int64_t batch) {
  if (l_kin && r_kin) return launch_cfg<DT, true, true>(ctx, cfg, a, batch);
  if (l_kin) return launch_cfg<DT, true, false>(ctx, cfg, a, batch);
  if (r_kin) return launch_cfg<DT, false, true>(ctx, cfg, a, batch);
  return launch_cfg<DT, false, false>(ctx, cfg, a, batch);
}

}  // namespace hipnx
