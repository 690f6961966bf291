// OCP FP8 instantiations of the transposing MFMA kernel (v_mfma_f32_32x32x64_f8f6f4; format 0 = E4M3,
// 1 = E5M2; E5M2 x E5M2 is not offered, as in the K-contiguous family).  E4M3 x E4M3 here, the mixed
// pairs in translation units of their own.
#include "mfma_tr_launch.hpp"
namespace zluda_amd {
uint32_t launch_tr_f8(const MfmaParams &prm, const zluda_gemm_plan &plan, int fq, int fp, bool pkc, bool qkc, hipStream_t s) {
  if (fq == 0 && fp == 0) return launch_tr_variant<KIND_F8, 0, 0>(prm, plan, pkc, qkc, s);
  if (fq == 1 && fp == 0) return launch_tr_f8_e5m2q(prm, plan, pkc, qkc, s);
  if (fq == 0 && fp == 1) return launch_tr_f8_e5m2p(prm, plan, pkc, qkc, s);
  return CUBLAS_STATUS_NOT_SUPPORTED;
}
} // namespace zluda_amd
