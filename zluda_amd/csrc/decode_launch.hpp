// Launchers of the LDS-streaming decode kernel (kernels/decode_stream.hpp), shared by the int8
// instantiations in launch.hip and the fp8 ones in decode_f8.hip.
#pragma once
#include <hip/hip_runtime.h>

#include "kernels/decode_slab.hpp"
#include "launch_util.hpp"
#include "planner.hpp"

namespace zluda_amd {

template <int N, int I = 0, class F>
inline void static_for_host(F &&f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for_host<N, I + 1>(f);
  }
}

// every output of the problem can leave through the packed 8-byte store of decode_stream_kernel
inline bool decode_packed_output(const GemmArgs &g, bool swapped) {
  const int64_t d_sr = swapped ? g.d_sj : g.d_si, d_st = swapped ? g.d_si : g.d_sj;
  const int rows = swapped ? g.N : g.M;
  return !g.int_scale && (g.d_type == CUDA_R_16BF || g.d_type == CUDA_R_16F) && d_sr == 1 &&
         g.beta_mode == SCALAR_VALUE && g.beta_val.f == 0.0f && ((uintptr_t)g.D & 7) == 0 && (d_st & 3) == 0 &&
         (g.d_sb & 3) == 0 && (rows & 3) == 0;
}

template <int NW, int SPW, int KIND>
inline uint32_t launch_decode_stream(const DecodeParams &prm, const zluda_gemm_plan &plan, int nb, hipStream_t s) {
  dim3 grid(plan.grid_x, plan.grid_y, 1), block(NW * 64);
  const bool fast = decode_packed_output(prm.g, prm.swapped != 0);
  uint32_t st = CUBLAS_STATUS_NOT_SUPPORTED;
  static_for_host<4>([&](auto nb_c) {
    constexpr int NB = decltype(nb_c)::value + 1;
    if constexpr (NB * SPW <= kDecodeStreamMaxFragments) {
      if (nb == NB) {
        const bool tail = prm.g.K < NW * SPW * 64;
        if (tail)
          st = fast ? launch_kernel(decode_stream_kernel<NW, SPW, NB, true, KIND, true>, grid, block, s, prm)
                    : launch_kernel(decode_stream_kernel<NW, SPW, NB, false, KIND, true>, grid, block, s, prm);
        else
          st = fast ? launch_kernel(decode_stream_kernel<NW, SPW, NB, true, KIND>, grid, block, s, prm)
                    : launch_kernel(decode_stream_kernel<NW, SPW, NB, false, KIND>, grid, block, s, prm);
      }
    }
  });
  return st;
}

// plan.variant -> instantiation of the stream kernel for one element kind (the table restates
// kDecodeVariants, planner.hpp)
template <int KIND>
inline uint32_t launch_decode_stream_variant(const DecodeParams &prm, const zluda_gemm_plan &plan, int nb, hipStream_t s) {
  switch (plan.variant) {
#define ZLUDA_STREAM_CASE(V, NW, SPW)                                                         \
  case V:                                                                                     \
    static_assert(kDecodeVariants[V].nw == NW && kDecodeVariants[V].steps == SPW && kDecodeVariants[V].stream == 1, \
                  "variant table mismatch");                                                  \
    return launch_decode_stream<NW, SPW, KIND>(prm, plan, nb, s);
    ZLUDA_STREAM_CASE(4, 8, 8)
    ZLUDA_STREAM_CASE(5, 8, 16)
    ZLUDA_STREAM_CASE(6, 8, 28)
    ZLUDA_STREAM_CASE(7, 4, 8)
    ZLUDA_STREAM_CASE(8, 8, 12)
    ZLUDA_STREAM_CASE(9, 8, 24)
    ZLUDA_STREAM_CASE(10, 4, 4)
    ZLUDA_STREAM_CASE(11, 8, 20)
    ZLUDA_STREAM_CASE(12, 4, 28)
    ZLUDA_STREAM_CASE(13, 4, 12)
    ZLUDA_STREAM_CASE(14, 4, 20)
    ZLUDA_STREAM_CASE(15, 8, 32)
    static_assert(kDecodeVariants[16].stream == 2 && kDecodeVariants[20].stream == 2, "variants 16 .. 20 are the slab kernel, launched by launch_decode_slab");
#undef ZLUDA_STREAM_CASE
  default: return CUBLAS_STATUS_INVALID_VALUE;
  }
}

// the slab form of the stream kernel (kernels/decode_slab.hpp): up to 16 tokens; 4 waves x one 1 KiB unit for
// K <= 4096 (steps == 16), 8 waves x steps / 8 units of 512 bytes for K <= 16384
template <int KIND>
inline uint32_t launch_decode_slab(const DecodeParams &prm, const zluda_gemm_plan &plan, int nb, hipStream_t s) {
  const DecodeVariant &v = kDecodeVariants[plan.variant];
  dim3 grid(plan.grid_x, plan.grid_y, 1), block(v.nw * 64);
  // 0: element-wise epilogue, 1: packed store, 2: packed store behind a GELU
  const int fast = !decode_packed_output(prm.g, prm.swapped != 0) ? 0 : prm.g.act == ACT_GELU ? 2 : 1;
  const bool tail = prm.g.K * (kind_is_h16(KIND) ? 2 : 1) < v.nw * v.steps * 64;  // K bytes against the cover
  uint32_t st = CUBLAS_STATUS_NOT_SUPPORTED;
  static_for_host<3>([&](auto fast_c) {
    constexpr int FAST = decltype(fast_c)::value;
    if (fast != FAST) return;
    if (v.nw == 4 && v.steps == 16 && nb == 1) {
      st = tail ? launch_kernel(decode_slab_kernel<FAST, KIND, true>, grid, block, s, prm)
                : launch_kernel(decode_slab_kernel<FAST, KIND, false>, grid, block, s, prm);
    } else if (v.nw == 8 && nb == 1) {
      static_for_host<3>([&](auto q_c) {
        constexpr int Q = decltype(q_c)::value + 2;
        if (v.steps == Q * 8) st = launch_kernel(decode_slab_kernel<FAST, KIND, true, 8, 512, Q>, grid, block, s, prm);
      });
    } else if (v.nw == 8 && nb == 2) {  // two token blocks: one or two units per slab
      if (v.steps == 8) st = launch_kernel(decode_slab_kernel<FAST, KIND, true, 8, 512, 1, 2>, grid, block, s, prm);
      else if (v.steps == 16) st = launch_kernel(decode_slab_kernel<FAST, KIND, true, 8, 512, 2, 2>, grid, block, s, prm);
    }
  });
  return st;
}

uint32_t launch_decode_slab_i8(const DecodeParams &prm, const zluda_gemm_plan &plan, int nb, hipStream_t s);
uint32_t launch_decode_slab_h16(const DecodeParams &prm, const zluda_gemm_plan &plan, int nb, bool bf16, hipStream_t s);
uint32_t launch_decode_slab_f8(const DecodeParams &prm, const zluda_gemm_plan &plan, int nb, hipStream_t s);
uint32_t launch_decode_stream_i8(const DecodeParams &prm, const zluda_gemm_plan &plan, int nb, hipStream_t s);
uint32_t launch_decode_stream_f8(const DecodeParams &prm, const zluda_gemm_plan &plan, int nb, hipStream_t s);

} // namespace zluda_amd
