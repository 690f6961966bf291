// Launchers of the transposing 8-bit MFMA kernel (kernels/gemm_mfma_tr.hpp); one translation unit per
// element kind so that the template instantiations compile in parallel.
#pragma once
#include <hip/hip_runtime.h>

#include "kernels/gemm_mfma_tr.hpp"
#include "planner.hpp"

namespace zluda_amd {

// plan.variant indexes kTrVariants (planner.hpp); pkc / qkc: operand P / Q has unit stride along K
template <int KIND, int FQ, int FP>
inline uint32_t launch_tr_variant(const MfmaParams &prm, const zluda_gemm_plan &plan, bool pkc, bool qkc, hipStream_t s) {
  const dim3 grid(plan.grid_x, plan.grid_y, 1), block(256);
  static_assert(kNumTrVariants == 2 && kTrVariants[0].bp == 128 && kTrVariants[0].bq == 128 &&
                kTrVariants[1].bp == 64 && kTrVariants[1].bq == 64, "variant table mismatch");
#define ZLUDA_TR_CASE(B, PK, QK)                                                                                \
  if (pkc == PK && qkc == QK) {                                                                                 \
    hipLaunchKernelGGL((gemm_mfma_tr_kernel<KIND, FQ, FP, B, B, PK, QK>), grid, block, 0, s, prm);              \
    return CUBLAS_STATUS_SUCCESS;                                                                               \
  }
  if (plan.variant == 0) {
    ZLUDA_TR_CASE(128, false, false) ZLUDA_TR_CASE(128, false, true) ZLUDA_TR_CASE(128, true, false) ZLUDA_TR_CASE(128, true, true)
  } else if (plan.variant == 1) {
    ZLUDA_TR_CASE(64, false, false) ZLUDA_TR_CASE(64, false, true) ZLUDA_TR_CASE(64, true, false) ZLUDA_TR_CASE(64, true, true)
  }
#undef ZLUDA_TR_CASE
  return CUBLAS_STATUS_INVALID_VALUE;
}

uint32_t launch_tr_i8(const MfmaParams &prm, const zluda_gemm_plan &plan, bool pkc, bool qkc, hipStream_t s);
uint32_t launch_tr_f8(const MfmaParams &prm, const zluda_gemm_plan &plan, int fq, int fp, bool pkc, bool qkc, hipStream_t s);

} // namespace zluda_amd
