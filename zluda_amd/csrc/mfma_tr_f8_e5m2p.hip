// transposing MFMA kernel, FP8 with operand P in E5M2 and operand Q in E4M3
#include "mfma_tr_launch.hpp"
namespace zluda_amd {
uint32_t launch_tr_f8_e5m2p(const MfmaParams &prm, const zluda_gemm_plan &plan, bool pkc, bool qkc, hipStream_t s) {
  return launch_tr_variant<KIND_F8, 0, 1>(prm, plan, pkc, qkc, s);
}
} // namespace zluda_amd
