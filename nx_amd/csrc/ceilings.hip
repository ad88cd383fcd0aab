// hipnx_ceilings: what this MI355X sustains on the two rooflines the library is judged against,
// measured the way the library's own kernels are timed (back-to-back launches on one stream, HIP
// events), so that a kernel's fraction of the published peak can be read beside the fraction of what
// the part actually delivers under its power management.
//
//   hipnx_ceilings mfma <bf16|f16|s8|f32|f64> <random|normal|zero> [ms]
//       an MFMA-only loop (the 16x16 forms the contraction kernel uses, 8 waves per CU, 32
//       independent accumulator tiles per wave, operands in registers, no memory traffic) launched
//       back to back for `ms` milliseconds; throughput is reported for the first 2 ms, for each fifth
//       of the run and for the last fifth (the sustained figure: the clock the part settles at
//       under this load depends on the operand bits and takes tens of milliseconds to settle)
//   hipnx_ceilings stream <read|write|copy> [MiB] [ms]
//       16-byte-per-lane streaming kernels over a buffer larger than the 256 MB last-level cache, the best of
//       1, 2, 4 and 8 accesses in flight per lane
//   hipnx_ceilings ingest <l2|llc|hbm> [ms]
//       what a compute unit takes in: 256 work-groups of 8 waves, one per CU, each pulling 4 MiB into LDS with
//       direct-to-LDS loads of 16 bytes per lane (the contraction kernels' way; 4, 8 and 16 KiB in flight per wave,
//       the best reported), from a region its XCD's L2 holds (`l2`: the work-groups of an XCD share 2 MiB), from
//       the last-level cache (`llc`: 512 KiB per work-group, 128 MiB in all) or from HBM (`hbm`: 4 MiB per
//       work-group, 1 GiB in all); bytes per clock of the shader clock measured in the last launch
//   hipnx_ceilings weights <work-groups> <none|interleaved|first> [KiB of rows per work-group]
//       the requests of a few rows against a long weight matrix (64 x 4096 int8 rows, 11008 x 4096 int8 weights: 45 MB
//       streamed once) without the arithmetic: `work-groups` work-groups of 8 waves share the weights evenly and pull
//       them into LDS with direct-to-LDS loads, 8 KiB in flight per wave, from one of ten copies in turn (nothing comes
//       from the last-level cache); beside them no bytes of the rows (`none`), as many bytes of the rows as of the
//       weights, request by request, from 256 KiB that L2 holds (`interleaved`: what a tile of the contraction kernels
//       takes in), or a fixed share of the rows before the first weights (`first`: what a work-group with its share of
//       the rows resident would take in).  Microseconds per launch over 400 launches back to back.
//
// Each run prints one JSON line.  Built by the Makefile into nx_amd/lib/hipnx_ceilings; bench.py runs
// it when present and copies the sustained figures into its `measured_ceiling` fields.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#define CK(x)                                                                          \
  do {                                                                                 \
    hipError_t e__ = (x);                                                              \
    if (e__ != hipSuccess) {                                                           \
      fprintf(stderr, "HIP error %s at line %d\n", hipGetErrorString(e__), __LINE__);  \
      return 1;                                                                        \
    }                                                                                  \
  } while (0)

typedef __attribute__((ext_vector_type(8))) __bf16 v8bf;
typedef __attribute__((ext_vector_type(8))) _Float16 v8h;
typedef __attribute__((ext_vector_type(4))) float v4f;
typedef __attribute__((ext_vector_type(4))) int v4i;

__device__ unsigned long long g_clk[2];

enum { K_BF16 = 0, K_F16 = 1, K_S8 = 2, K_F32 = 3 };

// 4 x 8 accumulator tiles of 16 x 16 per wave (the contraction kernel's wave tile); one trip of the
// loop = 2 K steps x 32 tiles = 64 MFMA instructions (f32: 4 x 64, one per 4 k)
template <int KIND>
__global__ void __launch_bounds__(512) mfma_loop(const v4i *src, float *out, int iters) {
  const int tid = threadIdx.x;
  v4i pa[4], pb[8];
  for (int q = 0; q < 4; q++) pa[q] = src[(blockIdx.x * 512 + tid) * 12 + q];
  for (int q = 0; q < 8; q++) pb[q] = src[(blockIdx.x * 512 + tid) * 12 + 4 + q];
  const unsigned long long c0 = clock64(), w0 = wall_clock64();
  float sum = 0;
  if constexpr (KIND == K_S8) {
    v4i acc[4][8];
    for (int i = 0; i < 4; i++) for (int j = 0; j < 8; j++) for (int q = 0; q < 4; q++) acc[i][j][q] = 0;
    for (int it = 0; it < iters; it++) {
#pragma unroll
      for (int ks = 0; ks < 2; ks++)
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
          for (int j = 0; j < 8; j++)
            acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(pb[(ks + j) & 7], pa[(ks + i) & 3], acc[i][j], 0, 0, 0);
    }
    for (int i = 0; i < 4; i++) for (int j = 0; j < 8; j++) for (int q = 0; q < 4; q++) sum += acc[i][j][q];
  } else {
    v4f acc[4][8];
    for (int i = 0; i < 4; i++) for (int j = 0; j < 8; j++) for (int q = 0; q < 4; q++) acc[i][j][q] = 0;
    for (int it = 0; it < iters; it++) {
#pragma unroll
      for (int ks = 0; ks < (KIND == K_F32 ? 8 : 2); ks++)
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
          for (int j = 0; j < 8; j++) {
            if constexpr (KIND == K_BF16)
              acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, pb[(ks + j) & 7]), __builtin_bit_cast(v8bf, pa[(ks + i) & 3]), acc[i][j], 0, 0, 0);
            else if constexpr (KIND == K_F16)
              acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, pb[(ks + j) & 7]), __builtin_bit_cast(v8h, pa[(ks + i) & 3]), acc[i][j], 0, 0, 0);
            else
              acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(__int_as_float(pb[j][ks & 3]), __int_as_float(pa[i][ks & 3]), acc[i][j], 0, 0, 0);
          }
    }
    for (int i = 0; i < 4; i++) for (int j = 0; j < 8; j++) for (int q = 0; q < 4; q++) sum += acc[i][j][q];
  }
  out[blockIdx.x * 512 + tid] = sum;
  if (blockIdx.x == 8 && tid == 0) {
    g_clk[0] = clock64() - c0;
    g_clk[1] = wall_clock64() - w0;
  }
}

// The f64 form: 4 x 4 accumulator tiles per wave (the f64 contraction kernel's wave tile: f64 accumulators take two
// registers an element), one trip = 8 k x 16 tiles = 128 v_mfma_f64_16x16x4_f64.
typedef __attribute__((ext_vector_type(4))) double v4d;
__global__ void __launch_bounds__(512) mfma_loop_f64(const double *src, double *out, int iters) {
  const int tid = threadIdx.x;
  double pa[8], pb[8];
  for (int q = 0; q < 8; q++) pa[q] = src[(size_t)(blockIdx.x * 512 + tid) * 16 + q], pb[q] = src[(size_t)(blockIdx.x * 512 + tid) * 16 + 8 + q];
  const unsigned long long c0 = clock64(), w0 = wall_clock64();
  v4d acc[4][4];
  for (int i = 0; i < 4; i++) for (int j = 0; j < 4; j++) for (int q = 0; q < 4; q++) acc[i][j][q] = 0;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int ks = 0; ks < 8; ks++)
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(pb[(ks + j) & 7], pa[(ks + i) & 7], acc[i][j], 0, 0, 0);
  }
  double sum = 0;
  for (int i = 0; i < 4; i++) for (int j = 0; j < 4; j++) for (int q = 0; q < 4; q++) sum += acc[i][j][q];
  out[blockIdx.x * 512 + tid] = sum;
  if (blockIdx.x == 8 && tid == 0) {
    g_clk[0] = clock64() - c0;
    g_clk[1] = wall_clock64() - w0;
  }
}

// One direct-to-LDS load as the contraction kernels issue it: every lane moves 16 bytes from its global address to
// LDS[base + 16 * lane], the wave-uniform base carried in M0.
typedef __attribute__((address_space(3))) void *lds_ptr_t;
__device__ __forceinline__ void lds_dma16(const unsigned char *g, unsigned char *lds) {
  const unsigned base = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(lds_ptr_t)lds);
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(base) : "memory", "m0");
#pragma clang diagnostic pop
}

// A work-group pulls `bytes_per_wg` from its region into LDS, DEPTH KiB in flight per wave.  Consecutive work-group
// ids go to different XCDs, so the groups with equal id % 8 share the regions of one XCD.
template <int DEPTH>
__global__ void __launch_bounds__(512) ingest_loop(const unsigned char *src, size_t region_bytes, int regions, size_t bytes_per_wg, unsigned *sink) {
  extern __shared__ unsigned char ingest_lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int xcd = blockIdx.x % 8, within = blockIdx.x / 8, per_xcd = regions / 8;
  const unsigned char *base = src + (size_t)(xcd * per_xcd + within % per_xcd) * region_bytes;
  const unsigned per_step = 8 * 1024, steps = (unsigned)(bytes_per_wg / per_step);  // the 8 waves move 8 KiB per step
  const unsigned mask = (unsigned)region_bytes - 1, mine_at = wave * 1024 + lane * 16;  // (regions are powers of two: a 64-bit
  // remainder per load costs a lane more instructions than the load and halves the rate measured)
  unsigned char *mine = ingest_lds + wave * DEPTH * 1024;
  const unsigned long long c0 = clock64(), w0 = wall_clock64();
  for (unsigned s = 0; s < steps; s += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; d++) lds_dma16(base + (((s + d) * per_step + mine_at) & mask), mine + d * 1024);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  if (((unsigned *)mine)[lane] == 0x12345678u) sink[0] = 1;  // (keeps the loads alive)
  if (blockIdx.x == 8 && threadIdx.x == 0) {
    g_clk[0] = clock64() - c0;
    g_clk[1] = wall_clock64() - w0;
  }
}

// The requests of the few-rows contraction without its arithmetic: a work-group pulls `w_per_wg` bytes of weights,
// 8 KiB in flight per wave; x_mode 1: every request for weights is followed by one for the rows (a 256 KiB region
// that L2 holds); x_mode 2: `xbytes` of the rows first.
__global__ void __launch_bounds__(512) weights_requests(const unsigned char *w, size_t w_per_wg, const unsigned char *x, size_t xbytes, int x_mode, unsigned *sink) {
  extern __shared__ unsigned char ingest_lds[];
  constexpr int DEPTH = 8;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const unsigned char *wb = w + (size_t)blockIdx.x * w_per_wg;
  unsigned char *mine = ingest_lds + wave * DEPTH * 1024;
  const unsigned at = wave * 1024 + lane * 16, per_step = 8 * 1024, xmask = 256 * 1024 - 1;
  const unsigned steps = (unsigned)(w_per_wg / per_step);
  if (x_mode == 2)
    for (unsigned s = 0; s < xbytes / per_step; s += DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; d++) lds_dma16(x + (((s + d) * per_step + at) & xmask), mine + d * 1024);
    }
  for (unsigned s = 0; s < steps; s += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; d++) {
      const unsigned o = s + d < steps ? (s + d) * per_step + at : at;
      lds_dma16(wb + o, mine + d * 1024);
      if (x_mode == 1) lds_dma16(x + (o & xmask), mine + d * 1024);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  if (((unsigned *)mine)[lane] == 0x12345678u) sink[0] = 1;  // (keeps the loads alive)
}

// Streaming kernels with a grid that covers the buffer (no grid-stride loop; on this part a resident grid
// that loops streams slower): a work-group of 256 lanes owns U * 4 KiB of contiguous memory, every lane has
// U independent 16-byte accesses in flight.  Which U streams fastest depends on the direction, so each run
// tries U = 1, 2, 4, 8 and reports the best.
template <int U>
__global__ void __launch_bounds__(256) stream_read(const v4i *__restrict__ in, v4i *__restrict__ out, size_t n) {
  const size_t base = (size_t)blockIdx.x * (256 * U) + threadIdx.x;
  v4i v[U];
#pragma unroll
  for (int u = 0; u < U; u++) v[u] = base + u * 256 < n ? in[base + u * 256] : v4i{0, 0, 0, 0};
  v4i acc = v[0];
#pragma unroll
  for (int u = 1; u < U; u++) acc ^= v[u];
  if (acc[0] == 0x12345678 && acc[1] == 0x0BADF00D) out[0] = acc;  // keeps the loads alive; practically never taken
}
template <int U>
__global__ void __launch_bounds__(256) stream_write(v4i *__restrict__ out, size_t n, int v) {
  const v4i x = {v, v + 1, v + 2, v + 3};
  const size_t base = (size_t)blockIdx.x * (256 * U) + threadIdx.x;
#pragma unroll
  for (int u = 0; u < U; u++)
    if (base + u * 256 < n) out[base + u * 256] = x;
}
template <int U>
__global__ void __launch_bounds__(256) stream_copy(const v4i *__restrict__ in, v4i *__restrict__ out, size_t n) {
  const size_t base = (size_t)blockIdx.x * (256 * U) + threadIdx.x;
  v4i v[U];
#pragma unroll
  for (int u = 0; u < U; u++) v[u] = base + u * 256 < n ? in[base + u * 256] : v4i{0, 0, 0, 0};
#pragma unroll
  for (int u = 0; u < U; u++)
    if (base + u * 256 < n) out[base + u * 256] = v[u];
}
template <int U>
static void launch_stream(int m, const v4i *a, v4i *b, size_t n) {
  const unsigned grid = (unsigned)((n + 256 * U - 1) / (256 * U));
  if (m == 0) hipLaunchKernelGGL(stream_read<U>, dim3(grid), dim3(256), 0, 0, a, b, n);
  else if (m == 1) hipLaunchKernelGGL(stream_write<U>, dim3(grid), dim3(256), 0, 0, b, n, 7);
  else hipLaunchKernelGGL(stream_copy<U>, dim3(grid), dim3(256), 0, 0, a, b, n);
}

static void launch_mfma(int kind, const v4i *d, float *o, int iters) {
  switch (kind) {
    case K_BF16: hipLaunchKernelGGL(mfma_loop<K_BF16>, dim3(256), dim3(512), 0, 0, d, o, iters); break;
    case K_F16: hipLaunchKernelGGL(mfma_loop<K_F16>, dim3(256), dim3(512), 0, 0, d, o, iters); break;
    case K_S8: hipLaunchKernelGGL(mfma_loop<K_S8>, dim3(256), dim3(512), 0, 0, d, o, iters); break;
    default: hipLaunchKernelGGL(mfma_loop<K_F32>, dim3(256), dim3(512), 0, 0, d, o, iters); break;
  }
}

// times `chunks` chunks of back-to-back launches with one event pair each; returns ms per chunk
template <typename F>
static int timed_chunks(F &&launch, int chunks, int per_chunk, std::vector<float> &ms) {
  std::vector<hipEvent_t> ev(chunks + 1);
  for (int i = 0; i <= chunks; i++) {
    hipEvent_t x;
    CK(hipEventCreate(&x));
    ev[i] = x;
  }
  CK(hipEventRecord(ev[0]));
  for (int c = 0; c < chunks; c++) {
    for (int i = 0; i < per_chunk; i++) launch();
    CK(hipEventRecord(ev[c + 1]));
  }
  CK(hipEventSynchronize(ev[chunks]));
  ms.resize(chunks);
  for (int c = 0; c < chunks; c++) CK(hipEventElapsedTime(&ms[c], ev[c], ev[c + 1]));
  CK(hipGetLastError());
  return 0;
}

static int run_mfma_f64(const char *data, double want_ms) {
  const size_t n = (size_t)256 * 512 * 16;
  std::vector<double> h(n);
  srand(1);
  auto uni = [] { return rand() / (double)RAND_MAX; };
  for (size_t i = 0; i < n; i++)
    h[i] = !strcmp(data, "random") ? uni() * 2 - 1 : !strcmp(data, "normal") ? sqrt(-2 * log((rand() + 1.0) / (RAND_MAX + 2.0))) * cos(6.283185307179586 * uni()) / 64 : 0.0;
  double *d, *o;
  CK(hipMalloc(&d, n * 8));
  CK(hipMalloc(&o, 256 * 512 * 8));
  CK(hipMemcpy(d, h.data(), n * 8, hipMemcpyHostToDevice));
  const int iters = 12;  // about 100 us per launch
  const double flop = 256.0 * 8 * iters * 128 * (2.0 * 16 * 16 * 4);
  auto launch = [&] { hipLaunchKernelGGL(mfma_loop_f64, dim3(256), dim3(512), 0, 0, d, o, iters); };
  std::vector<float> probe;
  if (timed_chunks(launch, 1, 5, probe)) return 1;
  const double launch_ms = probe[0] / 5;
  const int per_chunk = std::max(1, (int)(2.0 / launch_ms));
  const int chunks = std::max(5, (int)(want_ms / (per_chunk * launch_ms)));
  CK(hipDeviceSynchronize());
  std::vector<float> ms;
  if (timed_chunks(launch, chunks, per_chunk, ms)) return 1;
  unsigned long long c[2];
  CK(hipMemcpyFromSymbol(c, HIP_SYMBOL(g_clk), sizeof(c)));
  auto rate = [&](int a, int b) { double t = 0; for (int i = a; i < b; i++) t += ms[i]; return flop * per_chunk * (b - a) / t / 1e9; };
  printf("{\"kind\": \"mfma\", \"dtype\": \"f64\", \"operands\": \"%s\", \"unit\": \"TFLOP/s\", \"first_2ms\": %.1f, \"fifths\": [", data, rate(0, 1));
  for (int q = 0; q < 5; q++) printf("%s%.1f", q ? ", " : "", rate(chunks * q / 5, chunks * (q + 1) / 5));
  printf("], \"sustained\": %.1f, \"launch_us\": %.1f, \"clock_mhz_last_launch\": %.0f, \"clocks_per_instruction\": %.2f}\n", rate(chunks * 4 / 5, chunks),
         1000 * ms[chunks - 1] / per_chunk, c[0] / (c[1] / 100.0), (double)c[0] / ((double)iters * 128));
  return 0;
}

static int run_mfma(const char *type, const char *data, double want_ms) {
  if (!strcmp(type, "f64")) return run_mfma_f64(data, want_ms);
  const int kind = !strcmp(type, "bf16") ? K_BF16 : !strcmp(type, "f16") ? K_F16 : !strcmp(type, "s8") ? K_S8 : !strcmp(type, "f32") ? K_F32 : -1;
  if (kind < 0) { fprintf(stderr, "unknown type %s\n", type); return 2; }
  const size_t nwords = (size_t)256 * 512 * 12 * 4;  // v4i per lane x 12
  std::vector<uint32_t> h(nwords);
  srand(1);
  auto uni = [] { return rand() / (float)RAND_MAX; };
  for (size_t w = 0; w < nwords; w++) {
    uint32_t word = 0;
    const int per = kind == K_S8 ? 4 : kind == K_F32 ? 1 : 2;
    for (int e = 0; e < per; e++) {
      float f = 0;
      if (!strcmp(data, "random")) f = uni() * 2 - 1;
      else if (!strcmp(data, "normal")) f = sqrtf(-2 * logf((float)((rand() + 1.0) / (RAND_MAX + 2.0)))) * cosf(6.2831853f * uni()) / 64;  // the benchmark's operands
      uint32_t bits;
      std::memcpy(&bits, &f, 4);
      if (kind == K_S8) word |= (uint32_t)(uint8_t)(int8_t)(strcmp(data, "zero") ? (rand() % 255) - 127 : 0) << (8 * e);
      else if (kind == K_F32) word = bits;
      else if (kind == K_BF16) word |= (bits >> 16) << (16 * e);
      else { _Float16 hf = (_Float16)f; uint16_t hb; std::memcpy(&hb, &hf, 2); word |= (uint32_t)hb << (16 * e); }
    }
    h[w] = word;
  }
  v4i *d;
  float *o;
  CK(hipMalloc(&d, nwords * 4));
  CK(hipMalloc(&o, 256 * 512 * 4));
  CK(hipMemcpy(d, h.data(), nwords * 4, hipMemcpyHostToDevice));
  const int iters = kind == K_F32 ? 24 : 96;  // about 100 us per launch
  // flop per launch: 256 groups x 8 waves x iters x instructions x flop per instruction
  const double per_instr = kind == K_S8 ? 2.0 * 16 * 16 * 64 : kind == K_F32 ? 2.0 * 16 * 16 * 4 : 2.0 * 16 * 16 * 32;
  const double flop = 256.0 * 8 * iters * (kind == K_F32 ? 256 : 64) * per_instr;
  std::vector<float> probe;
  if (timed_chunks([&] { launch_mfma(kind, d, o, iters); }, 1, 5, probe)) return 1;
  const double launch_ms = probe[0] / 5;
  const int per_chunk = std::max(1, (int)(2.0 / launch_ms));               // about 2 ms per chunk
  const int chunks = std::max(5, (int)(want_ms / (per_chunk * launch_ms)));
  CK(hipDeviceSynchronize());
  std::vector<float> ms;
  if (timed_chunks([&] { launch_mfma(kind, d, o, iters); }, chunks, per_chunk, ms)) return 1;
  unsigned long long c[2];
  CK(hipMemcpyFromSymbol(c, HIP_SYMBOL(g_clk), sizeof(c)));
  auto rate = [&](int a, int b) { double t = 0; for (int i = a; i < b; i++) t += ms[i]; return flop * per_chunk * (b - a) / t / 1e9; };
  printf("{\"kind\": \"mfma\", \"dtype\": \"%s\", \"operands\": \"%s\", \"unit\": \"%s\", \"first_2ms\": %.1f, \"fifths\": [", type, data,
         kind == K_S8 ? "TOP/s" : "TFLOP/s", rate(0, 1));
  for (int q = 0; q < 5; q++) printf("%s%.1f", q ? ", " : "", rate(chunks * q / 5, chunks * (q + 1) / 5));
  printf("], \"sustained\": %.1f, \"run_ms\": %.1f, \"launch_us\": %.1f, \"clock_mhz_last_launch\": %.0f, \"clocks_per_instruction\": %.2f}\n",
         rate(chunks * 4 / 5, chunks), [&] { double t = 0; for (float x : ms) t += x; return t; }(), 1000 * ms[chunks - 1] / per_chunk,
         c[0] / (c[1] / 100.0), (double)c[0] / ((double)iters * (kind == K_F32 ? 256 : 64)));
  return 0;
}

static int run_stream(const char *mode, size_t mib, double want_ms) {
  const size_t bytes = mib << 20, n = bytes / 16;
  v4i *a, *b;
  CK(hipMalloc(&a, bytes));
  CK(hipMalloc(&b, bytes));
  CK(hipMemset(a, 1, bytes));
  CK(hipMemset(b, 2, bytes));
  const int m = !strcmp(mode, "read") ? 0 : !strcmp(mode, "write") ? 1 : !strcmp(mode, "copy") ? 2 : -1;
  if (m < 0) { fprintf(stderr, "unknown mode %s\n", mode); return 2; }
  const double moved = (m == 2 ? 2.0 : 1.0) * bytes;
  double best = 0, best_chunk = 0, best_us = 0;
  int best_u = 0;
  for (int u : {1, 2, 4, 8}) {
    auto launch = [&] {
      switch (u) {
        case 1: launch_stream<1>(m, a, b, n); break;
        case 2: launch_stream<2>(m, a, b, n); break;
        case 4: launch_stream<4>(m, a, b, n); break;
        default: launch_stream<8>(m, a, b, n); break;
      }
    };
    std::vector<float> probe;
    if (timed_chunks(launch, 1, 3, probe)) return 1;
    const double launch_ms = probe[0] / 3;
    const int per_chunk = std::max(1, (int)(2.0 / launch_ms));
    const int chunks = std::max(5, (int)(want_ms / 4 / (per_chunk * launch_ms)));
    std::vector<float> ms;
    if (timed_chunks(launch, chunks, per_chunk, ms)) return 1;
    auto rate = [&](int x, int y) { double t = 0; for (int i = x; i < y; i++) t += ms[i]; return moved * per_chunk * (y - x) / t / 1e6; };
    std::vector<float> sorted(ms);
    std::sort(sorted.begin(), sorted.end());
    const double sustained = rate(chunks * 4 / 5, chunks);
    if (sustained > best) {
      best = sustained;
      best_chunk = moved * per_chunk / sorted[0] / 1e6;
      best_us = 1000 * ms[chunks - 1] / per_chunk;
      best_u = u;
    }
  }
  printf("{\"kind\": \"stream\", \"mode\": \"%s\", \"MiB\": %zu, \"unit\": \"GB/s\", \"bytes_counted\": \"%s\", \"sustained\": %.0f, \"best_chunk\": %.0f, \"launch_us\": %.1f, \"accesses_per_lane\": %d}\n",
         mode, mib, m == 2 ? "read + written" : "one direction", best, best_chunk, best_us, best_u);
  return 0;
}

static int run_ingest(const char *from, double want_ms) {
  const int level = !strcmp(from, "l2") ? 0 : !strcmp(from, "llc") ? 1 : !strcmp(from, "hbm") ? 2 : -1;
  if (level < 0) { fprintf(stderr, "unknown source %s\n", from); return 2; }
  const size_t region = level == 0 ? (2u << 20) : level == 1 ? (512u << 10) : (4u << 20), per_wg = 4u << 20;
  const int regions = level == 0 ? 8 : 256;
  unsigned char *src;
  unsigned *sink;
  CK(hipMalloc(&src, region * regions));
  CK(hipMalloc(&sink, 4));
  CK(hipMemset(src, 1, region * regions));
  double best = 0, best_us = 0, best_clk = 0;
  int best_depth = 0;
  for (int depth : {4, 8, 16}) {
    const int lds = 8 * depth * 1024;
    auto launch = [&] {
      if (depth == 4) hipLaunchKernelGGL(ingest_loop<4>, dim3(256), dim3(512), lds, 0, src, region, regions, per_wg, sink);
      else if (depth == 8) hipLaunchKernelGGL(ingest_loop<8>, dim3(256), dim3(512), lds, 0, src, region, regions, per_wg, sink);
      else hipLaunchKernelGGL(ingest_loop<16>, dim3(256), dim3(512), lds, 0, src, region, regions, per_wg, sink);
    };
    if (depth == 16) CK(hipFuncSetAttribute((const void *)ingest_loop<16>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    std::vector<float> probe;
    if (timed_chunks(launch, 1, 3, probe)) return 1;
    const double launch_ms = probe[0] / 3;
    const int per_chunk = std::max(1, (int)(2.0 / launch_ms));
    const int chunks = std::max(5, (int)(want_ms / 3 / (per_chunk * launch_ms)));
    std::vector<float> ms;
    if (timed_chunks(launch, chunks, per_chunk, ms)) return 1;
    unsigned long long c[2];
    CK(hipMemcpyFromSymbol(c, HIP_SYMBOL(g_clk), sizeof(c)));
    double t = 0;
    for (int i = chunks * 4 / 5; i < chunks; i++) t += ms[i];
    const double us = 1000 * t / ((chunks - chunks * 4 / 5) * per_chunk), rate = 256.0 * per_wg / us / 1e3;  // GB/s
    if (rate > best) {
      best = rate;
      best_us = us;
      best_clk = c[0] / (c[1] / 100.0);
      best_depth = depth;
    }
  }
  printf("{\"kind\": \"ingest\", \"from\": \"%s\", \"unit\": \"GB/s\", \"sustained\": %.0f, \"per_cu\": %.1f, \"bytes_per_clock_per_cu\": %.1f, "
         "\"clock_mhz_last_launch\": %.0f, \"launch_us\": %.1f, \"KiB_in_flight_per_wave\": %d}\n",
         from, best, best / 256, best / 256 * 1e3 / best_clk, best_clk, best_us, best_depth);
  return 0;
}

static int run_weights(int groups, const char *rows, size_t x_kib) {
  const int x_mode = !strcmp(rows, "none") ? 0 : !strcmp(rows, "interleaved") ? 1 : !strcmp(rows, "first") ? 2 : -1;
  if (x_mode < 0 || groups < 1 || groups > 4096) { fprintf(stderr, "weights <work-groups> <none|interleaved|first> [KiB]\n"); return 2; }
  const size_t total = 11008ull * 4096, step = 8 * 1024, per = (total / groups + step - 1) / step * step, wbuf = per * groups;
  const int copies = 10, lds = 8 * 8 * 1024, launches = 400;
  unsigned char *w, *x;
  unsigned *sink;
  CK(hipMalloc(&w, wbuf * copies));
  CK(hipMalloc(&x, 256 * 1024));
  CK(hipMalloc(&sink, 4));
  CK(hipMemset(w, 1, wbuf * copies));
  CK(hipMemset(x, 1, 256 * 1024));
  int turn = 0;
  auto launch = [&] {
    hipLaunchKernelGGL(weights_requests, dim3(groups), dim3(512), lds, 0, w + (size_t)(turn++ % copies) * wbuf, per, x, x_kib * 1024, x_mode, sink);
  };
  std::vector<float> ms;
  if (timed_chunks(launch, 1, 50, ms)) return 1;
  if (timed_chunks(launch, 1, launches, ms)) return 1;
  const double us = 1000.0 * ms[0] / launches;
  printf("{\"kind\": \"weights\", \"work_groups\": %d, \"rows\": \"%s\", \"KiB_of_weights_per_work_group\": %zu, \"KiB_of_rows_per_work_group\": %zu, "
         "\"launch_us\": %.2f, \"GBps_of_weights\": %.0f}\n",
         groups, rows, per / 1024, x_mode == 1 ? per / 1024 : x_mode == 2 ? x_kib : (size_t)0, us, (double)wbuf / us / 1e3);
  return 0;
}

int main(int argc, char **argv) {
  if (argc >= 4 && !strcmp(argv[1], "weights")) return run_weights(atoi(argv[2]), argv[3], argc > 4 ? (size_t)atol(argv[4]) : 64);
  if (argc >= 3 && !strcmp(argv[1], "ingest")) return run_ingest(argv[2], argc > 3 ? atof(argv[3]) : 100.0);
  if (argc >= 4 && !strcmp(argv[1], "mfma")) return run_mfma(argv[2], argv[3], argc > 4 ? atof(argv[4]) : 300.0);
  if (argc >= 3 && !strcmp(argv[1], "stream")) return run_stream(argv[2], argc > 3 ? (size_t)atol(argv[3]) : 2048, argc > 4 ? atof(argv[4]) : 100.0);
  fprintf(stderr, "usage: hipnx_ceilings mfma <bf16|f16|s8|f32|f64> <random|normal|zero> [ms]\n       hipnx_ceilings stream <read|write|copy> [MiB] [ms]\n"
                  "       hipnx_ceilings ingest <l2|llc|hbm> [ms]\n       hipnx_ceilings weights <work-groups> <none|interleaved|first> [KiB of rows]\n");
  return 2;
}
