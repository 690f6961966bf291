// bf16 instantiations of the transposing MFMA kernel (v_mfma_f32_32x32x16_bf16).
#include "mfma_tr_launch.hpp"
namespace zluda_amd {
uint32_t launch_tr_bf16(const MfmaParams &prm, const zluda_gemm_plan &plan, bool pkc, bool qkc, hipStream_t s) {
  return launch_tr_variant<KIND_BF16, 0, 0>(prm, plan, pkc, qkc, s);
}
} // namespace zluda_amd
