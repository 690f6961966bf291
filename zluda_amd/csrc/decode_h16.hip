// f16 / bf16 instantiations of the slab decode kernel (v_mfma_f32_16x16x32_f16 / _bf16).
#include "decode_launch.hpp"
namespace zluda_amd {
uint32_t launch_decode_slab_h16(const DecodeParams &prm, const zluda_gemm_plan &plan, int nb, bool bf16, hipStream_t s) {
  return bf16 ? launch_decode_slab<KIND_BF16>(prm, plan, nb, s) : launch_decode_slab<KIND_F16>(prm, plan, nb, s);
}
} // namespace zluda_amd
