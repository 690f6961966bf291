// Mixed E4M3 / E5M2 MFMA GEMM instantiations (format code 1 = E5M2 on one operand).
#include "mfma_launch.hpp"
namespace zluda_amd {
uint32_t launch_mfma_f8_e5m2(const MfmaParams &prm, const zluda_gemm_plan &plan, int fq, int fp, hipStream_t s) {
  if (fq == 0 && fp == 1) return launch_mfma_variant<KIND_F8, 0, 1>(prm, plan, s);
  if (fq == 1 && fp == 0) return launch_mfma_variant<KIND_F8, 1, 0>(prm, plan, s);
  return CUBLAS_STATUS_NOT_SUPPORTED;  // E5M2 x E5M2 is not a cuBLASLt combination
}
} // namespace zluda_amd
