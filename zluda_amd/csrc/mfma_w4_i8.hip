// int8 x int8 -> int32 on the four-wave persistent kernel (v_mfma_i32_16x16x64_i8, accumulators in AGPRs).
#include "kernels/gemm_mfma_w4.hpp"
#include "mfma_launch.hpp"
namespace zluda_amd {
static_assert(W4_CLASS_I32 == W4_EPI_I32, "epilogue classes of the planner and of the kernel");
uint32_t launch_mfma_w4_i8(const MfmaParams &prm, int epi, uint32_t grid, hipStream_t s) {
  if (epi != W4_CLASS_I32) return launch_mfma_w4_i8f(prm, epi, grid, s);  // float epilogues: mfma_w4_i8f.hip
  return launch_kernel(gemm_mfma_w4_kernel<KIND_I8, 0, 0, W4_EPI_I32>, dim3(grid), dim3(256), s, prm);
}
} // namespace zluda_amd
