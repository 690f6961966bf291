// Launchers of the transposing MFMA kernel (kernels/gemm_mfma_tr.hpp); one translation unit per
// element kind so that the template instantiations compile in parallel.
#pragma once
#include <hip/hip_runtime.h>

#include "kernels/gemm_mfma_tr.hpp"
#include "launch_util.hpp"
#include "planner.hpp"

namespace zluda_amd {

// plan.variant indexes kTrVariants (planner.hpp); pkc / qkc: operand P / Q has unit stride along K
template <int KIND, int FQ, int FP>
inline uint32_t launch_tr_variant(const MfmaParams &prm, const zluda_gemm_plan &plan, bool pkc, bool qkc, hipStream_t s) {
  const dim3 grid(plan.grid_x, plan.grid_y, plan.grid_z > 1 ? plan.grid_z : 1);  // z: split-K shares
#define ZLUDA_TR_MODE(BP, BQ, WP, WQ, PK, QK)                                                                   \
  if (pkc == PK && qkc == QK) {                                                                                 \
    return launch_kernel(gemm_mfma_tr_kernel<KIND, FQ, FP, BP, BQ, WP, WQ, PK, QK>, grid, dim3(WP * WQ * 64), s, prm); \
  }
#define ZLUDA_TR_CASE(V, BP, BQ, WP, WQ)                                                                        \
  case V:                                                                                                       \
    static_assert(kTrVariants[V].bp == BP && kTrVariants[V].bq == BQ && kTrVariants[V].wp == WP &&              \
                  kTrVariants[V].wq == WQ && !kTrVariants[V].m16, "variant table mismatch");                                           \
    ZLUDA_TR_MODE(BP, BQ, WP, WQ, false, false) ZLUDA_TR_MODE(BP, BQ, WP, WQ, false, true)                      \
    ZLUDA_TR_MODE(BP, BQ, WP, WQ, true, false) ZLUDA_TR_MODE(BP, BQ, WP, WQ, true, true)                        \
    break;
  switch (plan.variant) {
    ZLUDA_TR_CASE(0, 256, 256, 2, 4)
    ZLUDA_TR_CASE(1, 128, 128, 2, 2)
    ZLUDA_TR_CASE(2, 64, 64, 2, 2)
  case 3:  // variant 0's tile on the 16x16 MFMA shape (int8, f16, bf16)
    static_assert(kTrVariants[3].bp == 256 && kTrVariants[3].bq == 256 && kTrVariants[3].wp == 2 && kTrVariants[3].wq == 4 &&
                  kTrVariants[3].m16, "variant table mismatch");
    if constexpr (KIND == KIND_I8 || kind_is_h16(KIND)) {
#define ZLUDA_TR16_MODE(PK, QK)                                                                                  \
  if (pkc == PK && qkc == QK)                                                                                    \
    return launch_kernel(gemm_mfma_tr_kernel<KIND, FQ, FP, 256, 256, 2, 4, PK, QK, true>, grid, dim3(512), s, prm);
      ZLUDA_TR16_MODE(false, false) ZLUDA_TR16_MODE(false, true) ZLUDA_TR16_MODE(true, false) ZLUDA_TR16_MODE(true, true)
#undef ZLUDA_TR16_MODE
    }
    break;
  default: break;
  }
#undef ZLUDA_TR_CASE
#undef ZLUDA_TR_MODE
  return CUBLAS_STATUS_INVALID_VALUE;
}

uint32_t launch_tr_i8(const MfmaParams &prm, const zluda_gemm_plan &plan, bool pkc, bool qkc, hipStream_t s);
uint32_t launch_tr_f8(const MfmaParams &prm, const zluda_gemm_plan &plan, int fq, int fp, bool pkc, bool qkc, hipStream_t s);
uint32_t launch_tr_f8_e5m2q(const MfmaParams &prm, const zluda_gemm_plan &plan, bool pkc, bool qkc, hipStream_t s);
uint32_t launch_tr_f8_e5m2p(const MfmaParams &prm, const zluda_gemm_plan &plan, bool pkc, bool qkc, hipStream_t s);
uint32_t launch_tr_f16(const MfmaParams &prm, const zluda_gemm_plan &plan, bool pkc, bool qkc, hipStream_t s);
uint32_t launch_tr_bf16(const MfmaParams &prm, const zluda_gemm_plan &plan, bool pkc, bool qkc, hipStream_t s);
uint32_t launch_tr_f32(const MfmaParams &prm, const zluda_gemm_plan &plan, bool pkc, bool qkc, hipStream_t s);

} // namespace zluda_amd
