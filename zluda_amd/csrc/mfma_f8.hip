// OCP FP8 (E4M3 x E4M3) MFMA GEMM instantiations (v_mfma_f32_32x32x64_f8f6f4, formats 0/0).
#include "mfma_launch.hpp"
namespace zluda_amd {
uint32_t launch_mfma_f8_e5m2(const MfmaParams &prm, const zluda_gemm_plan &plan, int fq, int fp, hipStream_t s);
uint32_t launch_mfma_f8(const MfmaParams &prm, const zluda_gemm_plan &plan, int fq, int fp, hipStream_t s) {
  if (fq == 0 && fp == 0) return launch_mfma_variant<KIND_F8, 0, 0>(prm, plan, s);
  return launch_mfma_f8_e5m2(prm, plan, fq, fp, s);
}
} // namespace zluda_amd
