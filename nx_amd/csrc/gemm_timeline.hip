// Where the time of the 256 x 256 two-group contraction kernel goes: a stand-alone program that compiles
// gemm_pingpong.cuh with HIPNX_GEMM_TIMELINE (the same kernel plus five clock reads and one store per
// work-group), launches it back to back until the part's clocks have settled, and prints one JSON line with the
// timeline of the last launch -- start-up, walk, epilogue, drain -- the shader clock during the walk and the share
// of the walk's clocks the MFMA pipe needs for the work.
//
//   hipnx_gemm_timeline <bf16|s8> [n = 4096] [settle ms = 400] [launches = 100]
//
// Environment: HIPNX_TL_ZERO=1 fills the operands with zeros (the same instructions and traffic with the least
// switching in the data paths: what the clock does to the figure); HIPNX_TL_HALF_WIDTH=1 runs 256 x 128 tiles
// (two per compute unit at n = 4096); HIPNX_TL_TILE_128=1 runs the two-group kernel on 128 x 128 tiles (the mid-size
// problems' kernel: one tile per compute unit at n = 2048); HIPNX_TL_GROUP_M sets the tile order's group height.  The Makefile also
// builds hipnx_gemm_timeline_exp1 / _exp32 / _exp64 from this file with -DHIPNX_PP_EXP=1 / 32 / 64: the walk
// without its requests, without its fragment reads, without the wait for its requests (timing only, results
// wrong -- "sampled_outputs_wrong" says so) -- what each of the three costs the walk.
//
// bf16: left operand K-inner, right operand K-outer (the plain Nx.dot(a, b) of the headline), bf16 output;
// s8: the same layouts, s32 output.  Operands are drawn like the benchmark's (normal / 64 cut to bf16; uniform
// integers in [-127, 127]).  The launch duration comes from a HIP event pair around the launches; the per-group
// stamps are the 100 MHz constant clock (wall_clock64) and the shader clock (clock64).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#define HIPNX_GEMM_TIMELINE 1
#include "gemm_pingpong.cuh"

using namespace hipnx;

#define CK(x)                                                                              \
  do {                                                                                     \
    hipError_t e__ = (x);                                                                  \
    if (e__ != hipSuccess) {                                                               \
      fprintf(stderr, "%s: %s (%s:%d)\n", #x, hipGetErrorString(e__), __FILE__, __LINE__); \
      exit(1);                                                                             \
    }                                                                                      \
  } while (0)

// sampled rows of the result recomputed one output per lane (f32 / s32 accumulation in k order)
template <int DT>
__global__ void sample_rows(const unsigned char *l, const unsigned char *r, float *out, int n, const int *rows) {
  const int col = blockIdx.x * blockDim.x + threadIdx.x, row = rows[blockIdx.y];
  if (col >= n) return;
  if constexpr (DT == HIPNX_S8) {
    int acc = 0;
    for (int k = 0; k < n; k++) acc += (int)(signed char)l[(size_t)row * n + k] * (int)(signed char)r[(size_t)k * n + col];
    reinterpret_cast<int *>(out)[(size_t)blockIdx.y * n + col] = acc;  // compared bit for bit with the s32 result
  } else {
    const uint16_t *a = (const uint16_t *)l, *b = (const uint16_t *)r;
    float acc = 0;
    for (int k = 0; k < n; k++)
      acc += __uint_as_float((uint32_t)a[(size_t)row * n + k] << 16) * __uint_as_float((uint32_t)b[(size_t)k * n + col] << 16);
    out[(size_t)blockIdx.y * n + col] = acc;
  }
}

// BM = 256: the 256-row two-group kernel (BN = 256 or 128); BM = 128: the two-group kernel on 128 x 128 tiles
template <int DT, int BN = 256, int BM = 256>
static int run(int n, double settle_ms, int launches) {
  constexpr int ES = DT == HIPNX_S8 ? 1 : 2, OS = DT == HIPNX_S8 ? 4 : 2;
  constexpr int MFMA_K = DT == HIPNX_S8 ? 64 : 32;  // k per 16 x 16 MFMA of 16 clocks
  if (n % 256 != 0 || n <= 0 || (n / BM) * (n / BN) > 4096) {
    fprintf(stderr, "n must be a multiple of 256 with at most 4096 tiles\n");
    return 2;
  }
  std::mt19937_64 rng(2);
  std::vector<unsigned char> hl((size_t)n * n * ES), hr((size_t)n * n * ES);
  if constexpr (DT == HIPNX_S8) {
    std::uniform_int_distribution<int> u(-127, 127);
    for (auto &x : hl) x = (unsigned char)(signed char)u(rng);
    for (auto &x : hr) x = (unsigned char)(signed char)u(rng);
  } else {
    std::normal_distribution<float> g(0.0f, 1.0f / 64);
    auto fill = [&](std::vector<unsigned char> &v) {
      uint16_t *p = (uint16_t *)v.data();
      for (size_t i = 0; i < v.size() / 2; i++) {
        const float f = g(rng);
        uint32_t w;
        std::memcpy(&w, &f, 4);
        p[i] = (uint16_t)(w >> 16);
      }
    };
    fill(hl);
    fill(hr);
  }
  if (getenv("HIPNX_TL_ZERO")) {  // all-zero operands: the same instructions and traffic with the least switching in the data paths
    std::fill(hl.begin(), hl.end(), 0);
    std::fill(hr.begin(), hr.end(), 0);
  }
  unsigned char *dl, *dr, *dout;
  CK(hipMalloc(&dl, hl.size()));
  CK(hipMalloc(&dr, hr.size()));
  CK(hipMalloc(&dout, (size_t)n * n * OS));
  CK(hipMemcpy(dl, hl.data(), hl.size(), hipMemcpyHostToDevice));
  CK(hipMemcpy(dr, hr.data(), hr.size(), hipMemcpyHostToDevice));

  GemmArgs a{};
  a.l = dl;
  a.r = dr;
  a.out = dout;
  a.odt = DT == HIPNX_S8 ? HIPNX_S32 : HIPNX_BF16;
  a.M = a.N = n;
  a.Kb = (int64_t)n * ES;
  a.ld_l = (int64_t)n * ES;  // [M, K], K contiguous
  a.ld_r = (int64_t)n * ES;  // [K, N], N contiguous
  a.tiles_m = n / BM;
  a.tiles_n = n / BN;
  a.group_m = getenv("HIPNX_TL_GROUP_M") ? atoi(getenv("HIPNX_TL_GROUP_M")) : gemm_group_m(a.tiles_m, a.tiles_n);
  // (the instantiations the library launches for these layouts)
  void (*kern)(GemmArgs);
  if constexpr (BM == 256) kern = gemm_pingpong_kernel<DT, true, false, true, true, BN>;
  else kern = gemm_pingpong128_kernel<DT, true, false, 128, 128, 4, 1>;
  const int smem = BM == 256 ? 2 * (256 + BN) * SLAB : 4 * (128 + 128) * SLAB;
  CK(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem));
  const dim3 grid(a.tiles_m * a.tiles_n), block(512);

  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  // settle: untimed launches for `settle_ms` (the power controller's transient)
  float spent = 0;
  while (spent < settle_ms) {
    CK(hipEventRecord(e0));
    for (int i = 0; i < 50; i++) hipLaunchKernelGGL(kern, grid, block, smem, 0, a);
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    float ms;
    CK(hipEventElapsedTime(&ms, e0, e1));
    spent += ms;
  }
  CK(hipEventRecord(e0));
  for (int i = 0; i < launches; i++) hipLaunchKernelGGL(kern, grid, block, smem, 0, a);
  CK(hipEventRecord(e1));
  CK(hipEventSynchronize(e1));
  CK(hipGetLastError());
  float ms;
  CK(hipEventElapsedTime(&ms, e0, e1));
  const double launch_us = ms * 1e3 / launches;

  // the result of the last launch against sampled rows recomputed plainly (s8: exact; bf16: within the rounding of the output)
  int bad = 0;
  {
    const int nrows = 24;
    std::vector<int> rows(nrows);
    for (int i = 0; i < nrows; i++) rows[i] = (int)(((long long)i * 2654435761ll + 77) % n);
    rows[0] = 0, rows[1] = n - 1, rows[2] = 127, rows[3] = 128, rows[4] = 255, rows[5] = 256;
    int *drows;
    float *dref;
    CK(hipMalloc(&drows, nrows * 4));
    CK(hipMalloc(&dref, (size_t)nrows * n * 4));
    CK(hipMemcpy(drows, rows.data(), nrows * 4, hipMemcpyHostToDevice));
    hipLaunchKernelGGL(sample_rows<DT>, dim3((n + 255) / 256, nrows), dim3(256), 0, 0, dl, dr, dref, n, drows);
    std::vector<float> ref((size_t)nrows * n);
    std::vector<unsigned char> got((size_t)n * n * OS);
    CK(hipMemcpy(ref.data(), dref, ref.size() * 4, hipMemcpyDeviceToHost));
    CK(hipMemcpy(got.data(), dout, got.size(), hipMemcpyDeviceToHost));
    for (int i = 0; i < nrows; i++)
      for (int c = 0; c < n; c++) {
        if constexpr (DT == HIPNX_S8) {
          if (((const int *)got.data())[(size_t)rows[i] * n + c] != ((const int *)ref.data())[(size_t)i * n + c]) bad++;
        } else {
          const uint32_t u = (uint32_t)((const uint16_t *)got.data())[(size_t)rows[i] * n + c] << 16;
          float g;
          std::memcpy(&g, &u, 4);
          const float w = ref[(size_t)i * n + c];
          if (!(fabsf(g - w) <= 0.01f * fabsf(w) + 1e-3f)) bad++;
        }
      }
  }

  const int nb = a.tiles_m * a.tiles_n;
  std::vector<unsigned long long> h((size_t)nb * 8);
  CK(hipMemcpyFromSymbol(h.data(), HIP_SYMBOL(hipnx::g_timeline), h.size() * 8));
  unsigned long long t0 = ~0ull, tend = 0;
  for (int b = 0; b < nb; b++) {
    t0 = std::min(t0, h[b * 8]);
    tend = std::max(tend, h[b * 8 + 3]);
  }
  const double tick = 0.01;  // us per tick of the 100 MHz clock
  double start = 0, start_max = 0, walk0 = 0, walk0_max = 0, walk1 = 0, walk1_max = 0, stored = 0, stored_max = 0, clocks = 0, dur = 0,
         dur_min = 1e30, dur_max = 0;
  double xcc_dur[8] = {0}, xcc_clk[8] = {0};
  int xcc_n[8] = {0};
  for (int b = 0; b < nb; b++) {
    const double s = (h[b * 8] - t0) * tick, w0 = (h[b * 8 + 1] - t0) * tick, w1 = (h[b * 8 + 2] - t0) * tick, st = (h[b * 8 + 3] - t0) * tick;
    start += s, walk0 += w0, walk1 += w1, stored += st;
    start_max = std::max(start_max, s), walk0_max = std::max(walk0_max, w0), walk1_max = std::max(walk1_max, w1), stored_max = std::max(stored_max, st);
    clocks += (double)h[b * 8 + 4];
    dur += w1 - w0, dur_min = std::min(dur_min, w1 - w0), dur_max = std::max(dur_max, w1 - w0);
    const int x = (int)(h[b * 8 + 5] & 7);
    xcc_dur[x] += w1 - w0, xcc_clk[x] += (double)h[b * 8 + 4], xcc_n[x]++;
  }
  start /= nb, walk0 /= nb, walk1 /= nb, stored /= nb, clocks /= nb, dur /= nb;
  // MFMA work of a work-group's walk: per SIMD two waves of 32 tiles each, 16 clocks per MFMA, K / MFMA_K steps
  const double mfma_clocks = BM == 256 ? 2.0 * (32 * BN / 256) * 16 * ((double)n / MFMA_K) : 16.0 * 16 * ((double)n / MFMA_K);
  const double ops = 2.0 * n * n * (double)n;
  printf("{\"kernel\": \"%s<%s, K-inner x K-outer, %d x %d>\", \"variant\": \"%s\", \"operands\": \"%s\", \"n\": %d, \"work_groups\": %d, \"launches\": %d, "
         "\"launch_us\": %.2f, \"rate_T\": %.1f, \"sampled_outputs_wrong\": %d, "
         "\"timeline_us_from_first_start\": {\"group_start\": {\"avg\": %.2f, \"max\": %.2f}, \"walk_begins\": {\"avg\": %.2f, \"max\": %.2f}, "
         "\"walk_ends\": {\"avg\": %.2f, \"max\": %.2f}, \"last_store_issued\": {\"avg\": %.2f, \"max\": %.2f}, \"span\": %.2f}, "
         "\"walk_us\": {\"min\": %.2f, \"avg\": %.2f, \"max\": %.2f}, \"epilogue_us_avg\": %.2f, \"after_last_store_us\": %.2f, "
         "\"walk_shader_clocks\": %.0f, \"walk_shader_clock_MHz\": %.0f, \"mfma_clocks_needed\": %.0f, \"mfma_share_of_walk_clocks\": %.4f, "
         "\"walk_us_avg_per_xcc\": [",
         BM == 256 ? "gemm_pingpong_kernel" : "gemm_pingpong128_kernel", DT == HIPNX_S8 ? "s8" : "bf16", BM, BN, HIPNX_PP_EXP == 0 ? "the library's kernel" : HIPNX_PP_EXP == 1 ? "timing only: no requests after the prologue" : HIPNX_PP_EXP == 32 ? "timing only: no fragment reads after the first slab" : HIPNX_PP_EXP == 64 ? "timing only: no wait for the requests" : "timing only", getenv("HIPNX_TL_ZERO") ? "all zero" : "as the benchmark draws them", n, nb, launches, launch_us, ops / launch_us / 1e6, bad, start, start_max, walk0, walk0_max, walk1, walk1_max,
         stored, stored_max, (tend - t0) * tick, dur_min, dur, dur_max, stored - walk1, launch_us - stored_max, clocks, clocks / dur,
         mfma_clocks, mfma_clocks / clocks);
  for (int x = 0; x < 8; x++) printf("%s%.2f", x ? ", " : "", xcc_n[x] ? xcc_dur[x] / xcc_n[x] : 0.0);
  printf("], \"walk_shader_clock_MHz_per_xcc\": [");
  for (int x = 0; x < 8; x++) printf("%s%.0f", x ? ", " : "", xcc_dur[x] > 0 ? xcc_clk[x] / xcc_dur[x] : 0.0);
  printf("]}\n");
  return 0;
}

int main(int argc, char **argv) {
  const std::string type = argc > 1 ? argv[1] : "bf16";
  const int n = argc > 2 ? atoi(argv[2]) : 4096;
  const double settle = argc > 3 ? atof(argv[3]) : 400.0;
  const int launches = argc > 4 ? atoi(argv[4]) : 100;
  const bool half = getenv("HIPNX_TL_HALF_WIDTH") != nullptr;  // 256 x 128 tiles: two per compute unit at n = 4096
  if (getenv("HIPNX_TL_TILE_128")) {  // the two-group kernel on 128 x 128 tiles (what the library launches at n = 2048)
    if (type == "bf16") return run<HIPNX_BF16, 128, 128>(n, settle, launches);
    if (type == "s8") return run<HIPNX_S8, 128, 128>(n, settle, launches);
  }
  if (type == "bf16") return half ? run<HIPNX_BF16, 128>(n, settle, launches) : run<HIPNX_BF16>(n, settle, launches);
  if (type == "s8") return half ? run<HIPNX_S8, 128>(n, settle, launches) : run<HIPNX_S8>(n, settle, launches);
  fprintf(stderr, "usage: hipnx_gemm_timeline <bf16|s8> [n] [settle ms] [launches]\n");
  return 2;
}
