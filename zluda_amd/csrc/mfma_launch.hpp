// Launchers of the MFMA GEMM instantiations; one translation unit per element kind so that the
// template instantiations compile in parallel.
#pragma once
#include <hip/hip_runtime.h>

#include "kernels/gemm_mfma.hpp"
#include "planner.hpp"

namespace zluda_amd {

// plan.variant: 0..3 = kMfmaVariants[v] with register staging, 4..7 = same tiles with
// direct-to-LDS loads.
template <int KIND, int FQ, int FP>
inline uint32_t launch_mfma_variant(const MfmaParams &prm, const zluda_gemm_plan &plan, hipStream_t s) {
  dim3 grid(plan.grid_x, plan.grid_y, 1);
  switch (plan.variant) {
  case 0: hipLaunchKernelGGL((gemm_mfma_kernel<KIND, FQ, FP, 256, 256, 2, 2, 0>), grid, dim3(256), 0, s, prm); break;
  case 1: hipLaunchKernelGGL((gemm_mfma_kernel<KIND, FQ, FP, 128, 128, 2, 2, 0>), grid, dim3(256), 0, s, prm); break;
  case 2: hipLaunchKernelGGL((gemm_mfma_kernel<KIND, FQ, FP, 256, 128, 2, 2, 0>), grid, dim3(256), 0, s, prm); break;
  case 3: hipLaunchKernelGGL((gemm_mfma_kernel<KIND, FQ, FP, 256, 256, 2, 4, 0>), grid, dim3(512), 0, s, prm); break;
  case 4: hipLaunchKernelGGL((gemm_mfma_kernel<KIND, FQ, FP, 256, 256, 2, 2, 1>), grid, dim3(256), 0, s, prm); break;
  case 5: hipLaunchKernelGGL((gemm_mfma_kernel<KIND, FQ, FP, 128, 128, 2, 2, 1>), grid, dim3(256), 0, s, prm); break;
  case 6: hipLaunchKernelGGL((gemm_mfma_kernel<KIND, FQ, FP, 256, 128, 2, 2, 1>), grid, dim3(256), 0, s, prm); break;
  case 7: hipLaunchKernelGGL((gemm_mfma_kernel<KIND, FQ, FP, 256, 256, 2, 4, 1>), grid, dim3(512), 0, s, prm); break;
  default: return CUBLAS_STATUS_INVALID_VALUE;
  }
  return CUBLAS_STATUS_SUCCESS;
}

uint32_t launch_mfma_i8(const MfmaParams &prm, const zluda_gemm_plan &plan, hipStream_t s);
uint32_t launch_mfma_f8(const MfmaParams &prm, const zluda_gemm_plan &plan, int fq, int fp, hipStream_t s);
uint32_t launch_mfma_mxf4(const MfmaParams &prm, const zluda_gemm_plan &plan, hipStream_t s);

} // namespace zluda_amd
