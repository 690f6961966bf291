// f32 x f32 -> fp32 MFMA GEMM instantiations (v_mfma_f32_32x32x2_f32).
#include "mfma_launch.hpp"
namespace zluda_amd {
uint32_t launch_mfma_f32(const MfmaParams &prm, const zluda_gemm_plan &plan, hipStream_t s) {
  return launch_mfma_variant<KIND_F32, 0, 0>(prm, plan, s);
}
} // namespace zluda_amd
