// Threefry-2x32 (20 rounds) over a counter range in one kernel: the fused form of the
// reference's threefry2x32/2 (nx/lib/nx/random.ex:214-285), which composes it from about 110
// element-wise callbacks.  Same counters, same key schedule, same output order:
//   half = ceil(n / 2); pair i has counters (i, half + i) -- the second one is the zero pad when
//   n is odd and i is the last pair -- and writes out[i] and out[half + i].
// Bound by integer work, not by the HBM writes: about 75 vector operations per 8 output bytes.
#include "internal.h"

namespace hipnx {

constexpr int RBLOCK = 256;
constexpr int RPAIRS = 4;  // counter pairs per lane: one 16-byte store into each half of the output

__device__ __forceinline__ uint32_t rotl32(uint32_t x, int r) { return (x << r) | (x >> (32 - r)); }

// 20 rounds on one counter pair, key already split into the three schedule words
__device__ __forceinline__ void threefry_pair(uint32_t &x1, uint32_t &x2, uint32_t key1, uint32_t key2) {
  uint32_t k1 = key2, k2 = key1 ^ key2 ^ 0x1BD11BDAu, k3 = key1;
  x1 += key1;
  x2 += key2;
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
}

// One lane takes RPAIRS consecutive pairs.  `vec` says that half is a multiple of RPAIRS and the output 16-byte aligned, so both
// stores of a lane whose pairs all exist are 16-byte aligned; every other lane stores word by word.
__global__ void __launch_bounds__(RBLOCK)
threefry2x32_kernel(const uint32_t *__restrict__ key, uint32_t *__restrict__ out, int64_t n, int64_t half, int vec) {
  const uint32_t key1 = key[0], key2 = key[1];
  const int64_t groups = (half + RBLOCK * RPAIRS - 1) / (RBLOCK * RPAIRS);
  for (int64_t g = blockIdx.x; g < groups; g += gridDim.x) {
    const int64_t i0 = (g * RBLOCK + threadIdx.x) * RPAIRS;
    if (i0 >= half) break;
    uint32_t a[RPAIRS], b[RPAIRS];
#pragma unroll
    for (int j = 0; j < RPAIRS; j++) {
      a[j] = (uint32_t)(i0 + j);
      b[j] = half + i0 + j < n ? (uint32_t)(half + i0 + j) : 0u;
      threefry_pair(a[j], b[j], key1, key2);
    }
    if (vec && half + i0 + RPAIRS <= n) {
      *reinterpret_cast<uint4 *>(out + i0) = make_uint4(a[0], a[1], a[2], a[3]);
      *reinterpret_cast<uint4 *>(out + half + i0) = make_uint4(b[0], b[1], b[2], b[3]);
      continue;
    }
#pragma unroll
    for (int j = 0; j < RPAIRS; j++) {
      if (i0 + j < half) out[i0 + j] = a[j];
      if (half + i0 + j < n && i0 + j < half) out[half + i0 + j] = b[j];
    }
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
  const int64_t per_block = (int64_t)RBLOCK * RPAIRS;
  int64_t blocks = (half + per_block - 1) / per_block;
  if (blocks > ((1ll << 32) - 1) / RBLOCK) blocks = ((1ll << 32) - 1) / RBLOCK;  // a launch may hold at most 2^32 - 1 lanes
  hipLaunchKernelGGL(threefry2x32_kernel, dim3((unsigned)blocks), dim3(RBLOCK), 0, ctx->stream,
                     (const uint32_t *)key->ptr, (uint32_t *)out->ptr, n, half, (int)(half % RPAIRS == 0 && (uintptr_t)out->ptr % 16 == 0));
  HIPNX_HIP(hipGetLastError());
  return HIPNX_OK;
}
