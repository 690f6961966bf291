// fp8 (e4m3 x e4m3) instantiations of the LDS-streaming decode kernels (v_mfma_f32_16x16x128_f8f6f4).
#include "decode_launch.hpp"
namespace zluda_amd {
uint32_t launch_decode_stream_f8(const DecodeParams &prm, const zluda_gemm_plan &plan, int nb, hipStream_t s) {
  return launch_decode_stream_variant<KIND_F8>(prm, plan, nb, s);
}
uint32_t launch_decode_slab_f8(const DecodeParams &prm, const zluda_gemm_plan &plan, int nb, hipStream_t s) {
  return launch_decode_slab<KIND_F8>(prm, plan, nb, s);
}
} // namespace zluda_amd
