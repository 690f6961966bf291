// MXFP4 (E2M1 + UE8M0 per 32) MFMA GEMM instantiations (v_mfma_scale_f32_32x32x64_f8f6f4, cbsz=blgp=4).
#include "mfma_launch.hpp"
namespace zluda_amd {
uint32_t launch_mfma_mxf4(const MfmaParams &prm, const zluda_gemm_plan &plan, hipStream_t s) {
  return launch_mfma_variant<KIND_MXF4, 4, 4>(prm, plan, s);
}
} // namespace zluda_amd
