/*
 * zluda_ptx_mma.h -- PTX `mma.sync.aligned` for gfx950: the device functions ZLUDA's PTX compiler
 * calls for the instruction, and a host entry point that runs them on caller-provided fragments.
 *
 * Device side (code object / bitcode `zluda_ptx_impl_mma`, built from zluda_amd/csrc/ptx_mma.hip).
 * Same names and signatures as the functions the reference's compiler emits calls to
 * (ptx/src/pass/replace_instructions_with_functions.rs:468-486) and defines in
 * ptx/lib/zluda_ptx_impl.cpp:1039, 1052, 1072; vectors are 32-bit x N ext-vectors:
 *
 *   float4 __zluda_ptx_impl_mma_sync_aligned_m16n8k16_row_col_f32_f16_f16_f32  (uint4 a, uint2 b, float4 c)
 *   float4 __zluda_ptx_impl_mma_sync_aligned_m16n8k16_row_col_f32_bf16_bf16_f32(uint4 a, uint2 b, float4 c)
 *   uint4  __zluda_ptx_impl_mma_sync_aligned_m16n8k32_row_col_s32_s8_s8_s32    (uint4 a, uint2 b, uint4 c)
 *
 * Each is called by every lane of a warp with that lane's fragment registers.  A 64-wide wavefront
 * carries two warps (lanes 0-31, 32-63); when both call together one MFMA serves both.
 */
#ifndef ZLUDA_AMD_PTX_MMA_H
#define ZLUDA_AMD_PTX_MMA_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
/* the declarations below are the library's exported symbols (it is built with -fvisibility=hidden) */
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

#define ZLUDA_PTX_MMA_S8 0u   /* m16n8k32.row.col.s32.s8.s8.s32 */
#define ZLUDA_PTX_MMA_F16 1u  /* m16n8k16.row.col.f32.f16.f16.f32 */
#define ZLUDA_PTX_MMA_BF16 2u /* m16n8k16.row.col.f32.bf16.bf16.f32 */

/* Runs one mma.sync per warp the way the reference's test programs do
 * (ptx/src/test/spirv_run/mma_m16n8k32_s32_s8_s8_s32.ptx: one thread = one lane, registers from and to
 * memory): thread i reads a[4i..4i+3], b[2i..2i+1], c[4i..4i+3] and writes d[4i..4i+3], all device
 * pointers to 32-bit words (c and d hold int32 for S8, float otherwise).  `threads` lanes in blocks of
 * `block` threads (a multiple of 32, at most 1024; `threads` a multiple of `block`), enqueued on
 * `stream` (a hipStream_t).  `masked_warps` 1 lets only the even warps of each block execute the
 * instruction, 2 only the odd ones (the others copy c to d), which exercises wavefronts of which only
 * the low or only the high half is there.
 * Returns 0, or 7 (invalid value) / 13 (launch failed) with cublasStatus_t numbering. */
uint32_t zluda_ptx_mma_run(uint32_t kind, const uint32_t *a, const uint32_t *b, const void *c, void *d,
                           uint32_t threads, uint32_t block, uint32_t masked_warps, void *stream);

/* Measurement aid: every thread runs c <- mma(a, b, c) `iters` times in a dependent chain and writes
 * the last c to d.  Whole wavefronts only (`block` a multiple of 64); `per_lane` != 0 forces the form
 * that a half-present wavefront falls back to, so that the two can be timed side by side. */
uint32_t zluda_ptx_mma_chain(uint32_t kind, const uint32_t *a, const uint32_t *b, const void *c, void *d,
                             uint32_t threads, uint32_t block, uint32_t iters, uint32_t per_lane,
                             void *stream);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif
#ifdef __cplusplus
}
#endif
#endif
