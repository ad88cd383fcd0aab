// Instantiations of the pipelined MFMA kernel for s8 operands (all four operand layouts).
#include "gemm_launch.cuh"

namespace hipnx {
int launch_gemm_s8(const hipnx_ctx *ctx, int cfg, bool l_kin, bool r_kin, GemmArgs a, int64_t batch) {
  return launch_layouts<HIPNX_S8>(ctx, cfg, l_kin, r_kin, a, batch);
}
}  // namespace hipnx
