// Instantiations of the pipelined MFMA kernel for f64 operands (all four operand layouts).
#include "gemm_launch.cuh"

namespace hipnx {
int launch_gemm_f64(const hipnx_ctx *ctx, int cfg, bool l_kin, bool r_kin, GemmArgs a, int64_t batch) {
  return launch_layouts<HIPNX_F64>(ctx, cfg, l_kin, r_kin, a, batch);
}
}  // namespace hipnx
