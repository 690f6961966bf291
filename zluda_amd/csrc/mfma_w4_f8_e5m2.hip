// Mixed E4M3 / E5M2 operands on the four-wave persistent kernel (format code 1 = E5M2 on one operand).
#include "kernels/gemm_mfma_w4.hpp"
#include "mfma_launch.hpp"
namespace zluda_amd {
template <int FQ, int FP>
static uint32_t launch_mix(const MfmaParams &prm, int epi, uint32_t grid, hipStream_t s) {
  if (epi == W4_CLASS_BF16_GELU) return launch_kernel(gemm_mfma_w4_kernel<KIND_F8, FQ, FP, W4_EPI_BF16_GELU>, dim3(grid), dim3(256), s, prm);
  if (epi == W4_CLASS_BF16) return launch_kernel(gemm_mfma_w4_kernel<KIND_F8, FQ, FP, W4_EPI_BF16>, dim3(grid), dim3(256), s, prm);
  return CUBLAS_STATUS_NOT_SUPPORTED;
}
uint32_t launch_mfma_w4_f8_e5m2(const MfmaParams &prm, int epi, uint32_t grid, int fq, int fp, hipStream_t s) {
  if (fq == 0 && fp == 1) return launch_mix<0, 1>(prm, epi, grid, s);
  if (fq == 1 && fp == 0) return launch_mix<1, 0>(prm, epi, grid, s);
  return CUBLAS_STATUS_NOT_SUPPORTED;  // E5M2 x E5M2 is not a cuBLASLt combination
}
} // namespace zluda_amd
