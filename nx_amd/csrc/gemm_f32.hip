// Instantiations of the pipelined MFMA kernel for f32 operands (K-inner operands; K-outer
// operands of this type are re-laid by the tiled transpose first).
#include "gemm_launch.cuh"

namespace hipnx {
int launch_gemm_f32(const hipnx_ctx *ctx, int cfg, GemmArgs a, int64_t batch) {
  return launch_cfg<HIPNX_F32, true, true>(ctx, cfg, a, batch);
}
}  // namespace hipnx
