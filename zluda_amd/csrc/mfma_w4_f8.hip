// e4m3 x e4m3 -> bf16 / f16 on the four-wave persistent kernel (v_mfma_f32_16x16x128_f8f6f4, accumulators in AGPRs).
#include "kernels/gemm_mfma_w4.hpp"
#include "mfma_launch.hpp"
namespace zluda_amd {
static_assert(W4_CLASS_BF16 == W4_EPI_BF16 && W4_CLASS_BF16_GELU == W4_EPI_BF16_GELU, "epilogue classes of the planner and of the kernel");
uint32_t launch_mfma_w4_f8(const MfmaParams &prm, int epi, uint32_t grid, int fq, int fp, hipStream_t s) {
  if (fq || fp) return launch_mfma_w4_f8_e5m2(prm, epi, grid, fq, fp, s);  // mixed formats: mfma_w4_f8_e5m2.hip
  if (epi == W4_CLASS_BF16_GELU) return launch_kernel(gemm_mfma_w4_kernel<KIND_F8, 0, 0, W4_EPI_BF16_GELU>, dim3(grid), dim3(256), s, prm);
  if (epi == W4_CLASS_BF16) return launch_kernel(gemm_mfma_w4_kernel<KIND_F8, 0, 0, W4_EPI_BF16>, dim3(grid), dim3(256), s, prm);
  return CUBLAS_STATUS_NOT_SUPPORTED;
}
} // namespace zluda_amd
