// Launchers of the MFMA GEMM instantiations; one translation unit per element kind so that the
// template instantiations compile in parallel.
#pragma once
#include <hip/hip_runtime.h>

#include "kernels/gemm_mfma_pipe16.hpp"
#include "launch_util.hpp"
#include "planner.hpp"

namespace zluda_amd {

// plan.variant indexes kMfmaVariants (planner.hpp); the template arguments below restate that table.
template <int KIND, int FQ, int FP>
inline uint32_t launch_mfma_variant(const MfmaParams &prm, const zluda_gemm_plan &plan, hipStream_t s) {
  dim3 grid(plan.grid_x, plan.grid_y, plan.grid_z > 1 ? plan.grid_z : 1);  // z: split-K shares
#define ZLUDA_MFMA_CASE(V, BP, BQ, WP, WQ, BKB, NS)                                                        \
  case V:                                                                                                  \
    static_assert(kMfmaVariants[V].bp == BP && kMfmaVariants[V].bq == BQ && kMfmaVariants[V].wp == WP &&   \
                  kMfmaVariants[V].wq == WQ && kMfmaVariants[V].bkb == BKB && kMfmaVariants[V].stages == NS && \
                  !kMfmaVariants[V].m16, "variant table mismatch");                                        \
    return launch_kernel(gemm_mfma_pipe_kernel<KIND, FQ, FP, BP, BQ, WP, WQ, BKB, NS>, grid,               \
                         dim3(WP * WQ * 64), s, prm);
  switch (plan.variant) {
    ZLUDA_MFMA_CASE(0, 256, 256, 2, 4, 128, 2)
    ZLUDA_MFMA_CASE(1, 256, 256, 2, 2, 128, 2)
    ZLUDA_MFMA_CASE(2, 256, 128, 2, 2, 128, 2)
    ZLUDA_MFMA_CASE(3, 128, 128, 2, 2, 128, 2)
    ZLUDA_MFMA_CASE(4, 128, 128, 2, 2, 64, 4)
    ZLUDA_MFMA_CASE(5, 128, 64, 2, 2, 128, 3)
    ZLUDA_MFMA_CASE(6, 64, 64, 2, 2, 128, 3)
    ZLUDA_MFMA_CASE(7, 192, 256, 2, 4, 128, 2)
#define ZLUDA_MFMA16_CASE(V, BP, BQ, WP, WQ)                                                                \
  case V:  /* the 16x16 MFMA shapes: int8, fp8, f16, bf16 */                                               \
    static_assert(kMfmaVariants[V].bp == BP && kMfmaVariants[V].bq == BQ && kMfmaVariants[V].wp == WP &&   \
                  kMfmaVariants[V].wq == WQ && kMfmaVariants[V].bkb == 128 && kMfmaVariants[V].stages == 2 && \
                  kMfmaVariants[V].m16, "variant table mismatch");                                         \
    if constexpr (KIND != KIND_I8 && KIND != KIND_F8 && !kind_is_h16(KIND)) return CUBLAS_STATUS_INVALID_VALUE;                                   \
    else return launch_kernel(gemm_mfma_pipe16_kernel<KIND, FQ, FP, BP, BQ, WP, WQ>, grid, dim3(WP * WQ * 64), s, prm);
    ZLUDA_MFMA16_CASE(8, 256, 256, 2, 4)
    ZLUDA_MFMA16_CASE(9, 192, 256, 2, 4)
#undef ZLUDA_MFMA16_CASE
  case 10:
    static_assert(kMfmaVariants[10].bp == 64 && kMfmaVariants[10].bq == 64 && kMfmaVariants[10].wp == 2 && kMfmaVariants[10].wq == 2 &&
                  kMfmaVariants[10].bkb == 128 && kMfmaVariants[10].stages == 6 && !kMfmaVariants[10].m16, "variant table mismatch");
    if constexpr (KIND == KIND_MXF4) return CUBLAS_STATUS_INVALID_VALUE;
    else return launch_kernel(gemm_mfma_pipe_kernel<KIND, FQ, FP, 64, 64, 2, 2, 128, 6>, grid, dim3(256), s, prm);
  default: return CUBLAS_STATUS_INVALID_VALUE;
  }
#undef ZLUDA_MFMA_CASE
  return CUBLAS_STATUS_INVALID_VALUE;
}

uint32_t launch_mfma_i8(const MfmaParams &prm, const zluda_gemm_plan &plan, hipStream_t s);
uint32_t launch_mfma_f8(const MfmaParams &prm, const zluda_gemm_plan &plan, int fq, int fp, hipStream_t s);
uint32_t launch_mfma_mxf4(const MfmaParams &prm, const zluda_gemm_plan &plan, hipStream_t s);
uint32_t launch_mfma_h16(const MfmaParams &prm, const zluda_gemm_plan &plan, bool bf16, hipStream_t s);
uint32_t launch_mfma_f32(const MfmaParams &prm, const zluda_gemm_plan &plan, hipStream_t s);
// the four-wave persistent kernel (variant 11; kernels/gemm_mfma_w4.hpp), `epi` = W4_CLASS_* of planner.hpp, `grid` workgroups
uint32_t launch_mfma_w4_i8(const MfmaParams &prm, int epi, uint32_t grid, hipStream_t s);
uint32_t launch_mfma_w4_i8f(const MfmaParams &prm, int epi, uint32_t grid, hipStream_t s);
// (fq, fp: 1 = E5M2 for the operand that is Q / P)
uint32_t launch_mfma_w4_f8(const MfmaParams &prm, int epi, uint32_t grid, int fq, int fp, hipStream_t s);
uint32_t launch_mfma_w4_f8_e5m2(const MfmaParams &prm, int epi, uint32_t grid, int fq, int fp, hipStream_t s);
uint32_t launch_mfma_w4_mxf4(const MfmaParams &prm, int epi, uint32_t grid, hipStream_t s);
uint32_t launch_mfma_w4_bf16(const MfmaParams &prm, int epi, uint32_t grid, hipStream_t s);
uint32_t launch_mfma_w4_f16(const MfmaParams &prm, int epi, uint32_t grid, hipStream_t s);

} // namespace zluda_amd
