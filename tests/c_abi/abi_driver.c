/* What a NIF would see: the callbacks of benchmark configuration 1 (add, multiply by 0.5, exp, sum over
 * axis 1 at 1024 x 1024 f32) and of `take` (8192 rows of a bf16 {32000, 4096} table) issued through
 * libhipnx.so from plain C -- no Python, no ctypes -- with an output buffer allocated and freed per
 * call as the Elixir backend does.  Prints one JSON line: host microseconds per call (time to enqueue),
 * the chain's time per pass with the device kept busy, and `take` under the three bounds policies.
 * Build: gcc -O2 -I include tests/c_abi/abi_driver.c -L nx_amd/lib -lhipnx -Wl,-rpath,'$ORIGIN' (the
 * library's Makefile does it); run: nx_amd/lib/hipnx_abi_driver [passes]. */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include "hipnx.h"

#define CK(call)                                                        \
  do {                                                                  \
    int st__ = (call);                                                  \
    if (st__ != HIPNX_OK) {                                             \
      char msg[512];                                                    \
      hipnx_last_error(msg, sizeof msg);                                \
      fprintf(stderr, "%s failed (%d): %s\n", #call, st__, msg);        \
      return 1;                                                         \
    }                                                                   \
  } while (0)

static double now_us(void) {
  struct timespec t;
  clock_gettime(CLOCK_MONOTONIC, &t);
  return t.tv_sec * 1e6 + t.tv_nsec * 1e-3;
}

int main(int argc, char **argv) {
  const int passes = argc > 1 ? atoi(argv[1]) : 2000;
  const int64_t n = 1024, N = n * n;
  hipnx_ctx *ctx;
  CK(hipnx_ctx_create(0, &ctx));
  float *host = (float *)malloc(N * 4);
  srand(1);
  for (int64_t i = 0; i < N; i++) host[i] = (float)rand() / RAND_MAX * 2 - 1;
  hipnx_buf *a, *b, *half;
  CK(hipnx_buf_alloc(ctx, N * 4, &a));
  CK(hipnx_buf_alloc(ctx, N * 4, &b));
  CK(hipnx_buf_alloc(ctx, 4, &half));
  CK(hipnx_h2d(ctx, a, 0, host, N * 4));
  CK(hipnx_h2d(ctx, b, 0, host, N * 4));
  const float h = 0.5f;
  CK(hipnx_fill(ctx, half, 4, &h, 1));
  const int64_t dims[2] = {n, n}, dense[2] = {n, 1}, scalar[2] = {0, 0};

  double t_call[4] = {0, 0, 0, 0};
  hipnx_buf *t1, *t2, *t3, *out;
  /* warm the pool and the clocks */
  for (int p = 0; p < 200 + passes; p++) {
    const int timed = p >= 200;
    double t0 = now_us();
    CK(hipnx_buf_alloc(ctx, N * 4, &t1));
    CK(hipnx_binary(ctx, HIPNX_ADD, HIPNX_F32, HIPNX_F32, HIPNX_F32, 2, dims, dense, dense, a, b, t1));
    double t_1 = now_us();
    CK(hipnx_buf_alloc(ctx, N * 4, &t2));
    CK(hipnx_binary(ctx, HIPNX_MULTIPLY, HIPNX_F32, HIPNX_F32, HIPNX_F32, 2, dims, dense, scalar, t1, half, t2));
    CK(hipnx_buf_destroy(t1));
    double t_2 = now_us();
    CK(hipnx_buf_alloc(ctx, N * 4, &t3));
    CK(hipnx_unary(ctx, HIPNX_EXP, HIPNX_F32, HIPNX_F32, N, t2, t3));
    CK(hipnx_buf_destroy(t2));
    double t_3 = now_us();
    CK(hipnx_buf_alloc(ctx, n * 4, &out));
    CK(hipnx_reduce(ctx, HIPNX_RED_SUM, HIPNX_F32, HIPNX_F32, n, n, 1, t3, out));
    CK(hipnx_buf_destroy(t3));
    CK(hipnx_buf_destroy(out));
    double t_4 = now_us();
    if (timed) { t_call[0] += t_1 - t0; t_call[1] += t_2 - t_1; t_call[2] += t_3 - t_2; t_call[3] += t_4 - t_3; }
    if (p == 199) { CK(hipnx_sync(ctx)); CK(hipnx_timer_start(ctx)); }
  }
  float chain_ms = 0;
  CK(hipnx_timer_stop(ctx, &chain_ms));

  /* take: one row-copy kernel per call (hipnx_gather, depth 1) */
  const int64_t rows = 32000, width = 4096, picks = 8192;
  hipnx_buf *table, *idx, *taken;
  CK(hipnx_buf_alloc(ctx, rows * width * 2, &table));
  CK(hipnx_buf_alloc(ctx, picks * 4, &idx));
  unsigned *hidx = (unsigned *)malloc(picks * 4);
  for (int64_t i = 0; i < picks; i++) hidx[i] = (unsigned)(rand() % rows);
  CK(hipnx_h2d(ctx, idx, 0, hidx, picks * 4));
  const int64_t tdims[2] = {rows, width};
  double take_us[3] = {0, 0, 0};
  const int take_passes = passes / 4 > 50 ? passes / 4 : 50;
  for (int policy = 0; policy < 3; policy++) {
    for (int p = 0; p < 20 + take_passes; p++) {
      if (p == 20) { CK(hipnx_sync(ctx)); CK(hipnx_timer_start(ctx)); }
      CK(hipnx_buf_alloc(ctx, picks * width * 2, &taken));
      CK(hipnx_gather(ctx, 2, 2, tdims, HIPNX_U32, picks, 1, policy, table, idx, taken));
      CK(hipnx_buf_destroy(taken));
    }
    float ms = 0;
    CK(hipnx_timer_stop(ctx, &ms));
    take_us[policy] = ms * 1e3 / take_passes;
  }
  printf("{\"passes\": %d, \"host_us_per_call\": {\"add\": %.2f, \"multiply\": %.2f, \"exp\": %.2f, \"sum\": %.2f}, "
         "\"config1_chain_f32_1024_us\": %.2f, \"take_bf16_8192_of_32000x4096_us\": {\"raise\": %.2f, \"clamp\": %.2f, \"defer\": %.2f}, "
         "\"note\": \"plain C over libhipnx.so; every call allocates and frees its output buffer\"}\n",
         passes, t_call[0] / passes, t_call[1] / passes, t_call[2] / passes, t_call[3] / passes, chain_ms * 1e3 / passes,
         take_us[0], take_us[1], take_us[2]);
  CK(hipnx_ctx_destroy(ctx));
  return 0;
}
