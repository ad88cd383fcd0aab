// Instantiations of the pipelined MFMA kernel for s8 operands (K-inner operands; K-outer
// operands of this type are re-laid by the tiled transpose first).
#include "gemm_launch.cuh"

namespace hipnx {
int launch_gemm_s8(const hipnx_ctx *ctx, int cfg, GemmArgs a, int64_t batch) {
  return launch_cfg<HIPNX_S8, true, true>(ctx, cfg, a, batch);
}
}  // namespace hipnx
