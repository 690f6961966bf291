// Device functions for PTX mma.sync on gfx950 (see kernels/ptx_mma.hpp) under the names ZLUDA's PTX
// compiler calls, and the host entry point of include/zluda_ptx_mma.h.
#include "../../include/zluda_ptx_mma.h"
#include "kernels/ptx_mma.hpp"
#include "launch_util.hpp"

using namespace zluda_amd::ptx_mma;

// ptx/lib/zluda_ptx_impl.cpp:109 : kept even when nothing in this module calls them
#define FUNC(NAME) __device__ __attribute__((retain, used)) __zluda_ptx_impl_##NAME

extern "C" {
f32x4 FUNC(mma_sync_aligned_m16n8k16_row_col_f32_f16_f16_f32)(u32x4 a, u32x2 b, f32x4 c) { return mma_sync<F16>(a, b, c); }
f32x4 FUNC(mma_sync_aligned_m16n8k16_row_col_f32_bf16_bf16_f32)(u32x4 a, u32x2 b, f32x4 c) { return mma_sync<BF16>(a, b, c); }
u32x4 FUNC(mma_sync_aligned_m16n8k32_row_col_s32_s8_s8_s32)(u32x4 a, u32x2 b, u32x4 c) {
  return __builtin_bit_cast(u32x4, mma_sync<S8>(a, b, __builtin_bit_cast(i32x4, c)));
}
}

template <int KIND>
__global__ void ptx_mma_run_kernel(const u32x4 *a, const u32x2 *b, const u32x4 *c, u32x4 *d, uint32_t masked_warps) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  const u32x4 av = a[i], cv = c[i];
  const u32x2 bv = b[i];
  u32x4 dv = cv;
  if (!masked_warps || ((threadIdx.x >> 5) & 1) == ((masked_warps - 1) & 1)) {   // 1: the even warps run, 2: the odd ones
    if constexpr (KIND == S8) dv = __zluda_ptx_impl_mma_sync_aligned_m16n8k32_row_col_s32_s8_s8_s32(av, bv, cv);
    else if constexpr (KIND == F16)
      dv = __builtin_bit_cast(u32x4, __zluda_ptx_impl_mma_sync_aligned_m16n8k16_row_col_f32_f16_f16_f32(av, bv, __builtin_bit_cast(f32x4, cv)));
    else
      dv = __builtin_bit_cast(u32x4, __zluda_ptx_impl_mma_sync_aligned_m16n8k16_row_col_f32_bf16_bf16_f32(av, bv, __builtin_bit_cast(f32x4, cv)));
  }
  d[i] = dv;
}

// c <- mma(a, b, c) `iters` times in a dependent chain: the cost of one instruction, for measurement
template <int KIND, bool PER_LANE>
__global__ void ptx_mma_chain_kernel(const u32x4 *a, const u32x2 *b, const u32x4 *c, u32x4 *d, uint32_t iters) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  const u32x4 av = a[i];
  const u32x2 bv = b[i];
  typename Acc<KIND>::type acc = __builtin_bit_cast(typename Acc<KIND>::type, c[i]);
  const int lane = lane_id();
  for (uint32_t it = 0; it < iters; it++) acc = PER_LANE ? mma_per_lane<KIND>(av, bv, acc, lane) : mma_wave64<KIND>(av, bv, acc, lane);
  d[i] = __builtin_bit_cast(u32x4, acc);
}

extern "C" uint32_t zluda_ptx_mma_chain(uint32_t kind, const uint32_t *a, const uint32_t *b, const void *c, void *d,
                                        uint32_t threads, uint32_t block, uint32_t iters, uint32_t per_lane, void *stream) {
  if (!a || !b || !c || !d || kind > ZLUDA_PTX_MMA_BF16) return 7;
  if (block == 0 || block > 1024 || block % 64 || threads == 0 || threads % block) return 7;
  const dim3 grid(threads / block), blk(block);
  hipStream_t s = (hipStream_t)stream;
  const u32x4 *av = (const u32x4 *)a, *cv = (const u32x4 *)c;
  const u32x2 *bv = (const u32x2 *)b;
  u32x4 *dv = (u32x4 *)d;
  uint32_t st;
#define ZLUDA_CHAIN(K)                                                                                \
  st = per_lane ? zluda_amd::launch_kernel(ptx_mma_chain_kernel<K, true>, grid, blk, s, av, bv, cv, dv, iters) \
                : zluda_amd::launch_kernel(ptx_mma_chain_kernel<K, false>, grid, blk, s, av, bv, cv, dv, iters)
  switch (kind) {
  case ZLUDA_PTX_MMA_S8: ZLUDA_CHAIN(S8); break;
  case ZLUDA_PTX_MMA_F16: ZLUDA_CHAIN(F16); break;
  default: ZLUDA_CHAIN(BF16); break;
  }
#undef ZLUDA_CHAIN
  return st;  // 0 or 13 (CUBLAS_STATUS_EXECUTION_FAILED)
}

extern "C" uint32_t zluda_ptx_mma_run(uint32_t kind, const uint32_t *a, const uint32_t *b, const void *c, void *d,
                                      uint32_t threads, uint32_t block, uint32_t masked_warps, void *stream) {
  if (!a || !b || !c || !d || kind > ZLUDA_PTX_MMA_BF16) return 7;
  if (block == 0 || block > 1024 || block % 32 || threads == 0 || threads % block) return 7;
  const dim3 grid(threads / block), blk(block);
  hipStream_t s = (hipStream_t)stream;
  const u32x4 *av = (const u32x4 *)a, *cv = (const u32x4 *)c;
  const u32x2 *bv = (const u32x2 *)b;
  u32x4 *dv = (u32x4 *)d;
  switch (kind) {
  case ZLUDA_PTX_MMA_S8: return zluda_amd::launch_kernel(ptx_mma_run_kernel<S8>, grid, blk, s, av, bv, cv, dv, masked_warps);
  case ZLUDA_PTX_MMA_F16: return zluda_amd::launch_kernel(ptx_mma_run_kernel<F16>, grid, blk, s, av, bv, cv, dv, masked_warps);
  default: return zluda_amd::launch_kernel(ptx_mma_run_kernel<BF16>, grid, blk, s, av, bv, cv, dv, masked_warps);
  }
}
