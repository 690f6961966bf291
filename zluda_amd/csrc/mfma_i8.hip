// int8 x int8 -> int32 MFMA GEMM instantiations (v_mfma_i32_32x32x32_i8).
#include "mfma_launch.hpp"
namespace zluda_amd {
uint32_t launch_mfma_i8(const MfmaParams &prm, const zluda_gemm_plan &plan, hipStream_t s) {
  return launch_mfma_variant<KIND_I8, 0, 0>(prm, plan, s);
}
} // namespace zluda_amd
