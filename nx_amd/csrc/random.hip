// Threefry-2x32 (20 rounds) over a counter range in one kernel: the fused form of the
// reference's threefry2x32/2 (nx/lib/nx/random.ex:214-285), which composes it from about 110
// element-wise callbacks.  Same counters, same key schedule, same output order:
//   half = ceil(n / 2); pair i has counters (i, half + i) -- the second one is the zero pad when
//   n is odd and i is the last pair -- and writes out[i] and out[half + i].
// Integer work bound by the HBM writes (4 bytes per output word, ~10 integer ops per byte).
#include "internal.h"

namespace hipnx {

constexpr int RBLOCK = 256;

__device__ __forceinline__ uint32_t rotl32(uint32_t x, int r) { return (x << r) | (x >> (32 - r)); }

__global__ void __launch_bounds__(RBLOCK)
threefry2x32_kernel(const uint32_t *__restrict__ key, uint32_t *__restrict__ out, int64_t n, int64_t half) {
  const uint32_t key1 = key[0], key2 = key[1];
  for (int64_t i = (int64_t)blockIdx.x * RBLOCK + threadIdx.x; i < half; i += (int64_t)gridDim.x * RBLOCK) {
    const bool second = half + i < n;
    uint32_t x1 = (uint32_t)i + key1, x2 = (second ? (uint32_t)(half + i) : 0u) + key2;
    uint32_t k1 = key2, k2 = key1 ^ key2 ^ 0x1BD11BDAu, k3 = key1;
    constexpr int R[2][4] = {{13, 15, 26, 6}, {17, 29, 16, 24}};
#pragma unroll
    for (int g = 1; g <= 5; g++) {
#pragma unroll
      for (int r = 0; r < 4; r++) {
        x1 += x2;
        x2 = rotl32(x2, R[(g - 1) & 1][r]) ^ x1;
      }
      x1 += k1;
      x2 += k2 + (uint32_t)g;
      const uint32_t t = k1; k1 = k2; k2 = k3; k3 = t;
    }
    out[i] = x1;
    if (second) out[half + i] = x2;
  }
}

}  // namespace hipnx

using namespace hipnx;

extern "C" int hipnx_threefry2x32(hipnx_ctx *ctx, const hipnx_buf *key, int64_t n, hipnx_buf *out) {
  Enter in(ctx);
  if (in.status) return in.status;
  if (n < 0) return set_error(HIPNX_EINVAL, "threefry2x32: negative count");
  if (int st = check_buf(ctx, key, 8, "threefry2x32 key")) return st;
  if (int st = check_buf(ctx, out, (uint64_t)n * 4, "threefry2x32 out")) return st;
  if (n == 0) return HIPNX_OK;
  const int64_t half = (n + 1) / 2;
  int64_t blocks = (half + RBLOCK - 1) / RBLOCK;
  if (blocks > (1ll << 30)) blocks = 1ll << 30;
  hipLaunchKernelGGL(threefry2x32_kernel, dim3((unsigned)blocks), dim3(RBLOCK), 0, ctx->stream,
                     (const uint32_t *)key->ptr, (uint32_t *)out->ptr, n, half);
  HIPNX_HIP(hipGetLastError());
  return HIPNX_OK;
}
