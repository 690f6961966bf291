// The four-wave persistent MFMA kernel for MXFP4 (E2M1 x E2M1 with UE8M0 block scales), bf16 output.
#include "kernels/gemm_mfma_w4.hpp"
#include "mfma_launch.hpp"

namespace zluda_amd {

static_assert(W4_CLASS_BF16 == W4_EPI_BF16 && W4_CLASS_BF16_GELU == W4_EPI_BF16_GELU, "the planner's classes are the kernel's epilogues");

uint32_t launch_mfma_w4_mxf4(const MfmaParams &prm, int epi, uint32_t grid, hipStream_t s) {
  switch (epi) {
  case W4_CLASS_BF16: return launch_kernel(gemm_mfma_w4_kernel<KIND_MXF4, 0, 0, W4_EPI_BF16>, dim3(grid), dim3(256), s, prm);
  case W4_CLASS_BF16_GELU: return launch_kernel(gemm_mfma_w4_kernel<KIND_MXF4, 0, 0, W4_EPI_BF16_GELU>, dim3(grid), dim3(256), s, prm);
  default: return CUBLAS_STATUS_INVALID_VALUE;
  }
}

} // namespace zluda_amd
