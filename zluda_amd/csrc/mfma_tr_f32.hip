// f32 instantiations of the transposing MFMA kernel (v_mfma_f32_32x32x2_f32).
#include "mfma_tr_launch.hpp"
namespace zluda_amd {
uint32_t launch_tr_f32(const MfmaParams &prm, const zluda_gemm_plan &plan, bool pkc, bool qkc, hipStream_t s) {
  return launch_tr_variant<KIND_F32, 0, 0>(prm, plan, pkc, qkc, s);
}
} // namespace zluda_amd
