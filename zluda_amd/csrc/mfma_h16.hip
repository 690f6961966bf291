// f16 x f16 and bf16 x bf16 -> fp32 MFMA GEMM instantiations (v_mfma_f32_32x32x16_f16 / _bf16).
#include "mfma_launch.hpp"
namespace zluda_amd {
uint32_t launch_mfma_h16(const MfmaParams &prm, const zluda_gemm_plan &plan, bool bf16, hipStream_t s) {
  return bf16 ? launch_mfma_variant<KIND_BF16, 0, 0>(prm, plan, s) : launch_mfma_variant<KIND_F16, 0, 0>(prm, plan, s);
}
} // namespace zluda_amd
