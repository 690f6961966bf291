// Host-side lowering of a cuBLASLt-level problem to kernel arguments, and kernel selection.
#pragma once
#include "../../include/cublaslt_abi.h"
#include "../../include/zluda_gemm_launch.h"
#include "gemm_args.hpp"

namespace zluda_amd {

// MFMA tile configurations (index = plan.variant for the MFMA families): workgroup tile bp x bq,
// wp x wq waves, `bkb` bytes of K per LDS stage, `stages` LDS stages
struct MfmaVariant { int bp, bq, wp, wq, bkb, stages, m16, w4; };  // m16: the 16x16 MFMA shapes (gemm_mfma_pipe16.hpp; not MXFP4, not f32)
                                                                // w4: the persistent four-wave kernel (gemm_mfma_w4.hpp; int8, fp8, MXFP4, f16, bf16)
constexpr MfmaVariant kMfmaVariants[] = {
    {256, 256, 2, 4, 128, 2, 0, 0},  // 0: 8 waves, 128x64 per wave
    {256, 256, 2, 2, 128, 2, 0, 0},  // 1: 4 waves, 128x128 per wave
    {256, 128, 2, 2, 128, 2, 0, 0},  // 2: 4 waves, 128x64 per wave
    {128, 128, 2, 2, 128, 2, 0, 0},  // 3: 4 waves, 64x64 per wave, two workgroups per CU
    {128, 128, 2, 2, 64, 4, 0, 0},   // 4: same tile, half-line stages, deeper ring (short K)
    {128, 64, 2, 2, 128, 3, 0, 0},   // 5: 4 waves, 64x32 per wave: skinny problems
    {64, 64, 2, 2, 128, 3, 0, 0},    // 6: 4 waves, 32x32 per wave: problems of a few hundred tiles at most
    {192, 256, 2, 4, 128, 2, 0, 0},  // 7: 8 waves, 96x64 per wave: extents that 256 divides badly (3072, 6144, ...)
    // the same tiles on v_mfma_*_16x16x* (int8, fp8, f16, bf16): less energy per multiply-add, and GEMMs that keep the
    // chip busy are power bound
    {256, 256, 2, 4, 128, 2, 1, 0},  // 8: variant 0's
    {192, 256, 2, 4, 128, 2, 1, 0},  // 9: variant 7's
    // skinny, memory-bound problems of at most one workgroup per CU: variant 6's tile with a ring of 6 stages, i.e. 80 KiB
    // instead of 32 KiB of operand rows in flight per CU (not MXFP4: its scale chunks span 4 stages)
    {64, 64, 2, 2, 128, 6, 0, 0},    // 10
    // variant 8's tile with four waves of 128 x 128, one workgroup per CU walking a list of tiles (int8, fp8, MXFP4, f16 and
    // bf16 operands with the epilogues w4_epilogue_class() admits; no split along K): 5-20 % less time than variant 8 / 0
    {256, 256, 2, 2, 128, 2, 1, 1},  // 11
};
constexpr int kNumMfmaVariants32 = 8;  // the first ones, on the 32x32 shapes: what MXFP4 has
constexpr int kNumMfmaVariantsH16 = 12;  // f16 / bf16: all of them
constexpr int kNumMfmaVariants = sizeof(kMfmaVariants) / sizeof(kMfmaVariants[0]);

// tile configurations of the transposing 8-bit MFMA kernel (index = plan.variant for
// ZLUDA_KERNEL_MFMA_TR8): workgroup tile bp x bq, wp x wq waves, always 64 K bytes per stage
struct TrVariant { int bp, bq, wp, wq, m16; };  // m16: int8 / f16 / bf16 on the 16x16 MFMA shapes (as the variants 8 .. above)
constexpr TrVariant kTrVariants[] = {
    {256, 256, 2, 4, 0},  // 0: 8 waves, 128x64 per wave, one workgroup per CU
    {128, 128, 2, 2, 0},  // 1: 4 waves, 64x64 per wave, two workgroups per CU
    {64, 64, 2, 2, 0},    // 2: 4 waves, 32x32 per wave, four or more per CU: small and skinny problems
    {256, 256, 2, 4, 1},  // 3: variant 0 on the 16x16 MFMA shape, int8 / f16 / bf16: grids that fill the chip
};
constexpr int kNumTrVariants = sizeof(kTrVariants) / sizeof(kTrVariants[0]);

// decode configurations (index = plan.variant for ZLUDA_KERNEL_DECODE_W8A8).
// stream == 0: weights loaded straight into registers, any K (grid-stride over 16-row blocks).
// stream == 1: weights streamed through LDS in whole cache lines; covers K <= nw * steps * 64 (the planner
// gives an instantiation the K values down to three quarters of its cover).
// stream == 2: the slab form of the stream kernel (whole 512-byte or 1 KiB row segments, activations through LDS, one
// reduction per workgroup): at most 4 blocks of 16 rows per workgroup; 4 waves x 1 KiB for K down to half of 4096 and
// up to 16 tokens, 8 waves x (steps / 8) units of 512 bytes each for the K between one cover and the next; the
// 8-wave shapes of one or two units also take a second block of 16 tokens.
struct DecodeVariant { int nw, steps, stream; };
constexpr DecodeVariant kDecodeVariants[] = {
    {8, 8, 0},   // 0: 8 waves x 512 B of K per pass
    {8, 16, 0},  // 1: 8 waves x 1024 B
    {4, 16, 0},  // 2: 4 waves x 1024 B
    {4, 8, 0},   // 3: 4 waves x 512 B
    {8, 8, 1},   // 4: K = 4096
    {8, 16, 1},  // 5: K = 8192
    {8, 28, 1},  // 6: K = 14336
    {4, 8, 1},   // 7: K = 2048
    {8, 12, 1},  // 8: K = 6144
    {8, 24, 1},  // 9: K = 12288
    {4, 4, 1},   // 10: K = 1024
    {8, 20, 1},  // 11: K = 10240
    {4, 28, 1},  // 12: K = 7168
    {4, 12, 1},  // 13: K = 3072
    {4, 20, 1},  // 14: K = 5120
    {8, 32, 1},  // 15: K = 16384 (one block of 16 tokens: 32 fragments)
    {4, 16, 2},  // 16: slab form, 2048 < K <= 4096, up to 16 tokens, up to 64 rows per workgroup
    {8, 16, 2},  // 17: slab form, 4096 < K <= 8192 (8 waves x 2 units of 512 bytes)
    {8, 24, 2},  // 18: slab form, 8192 < K <= 12288
    {8, 32, 2},  // 19: slab form, 12288 < K <= 16384
    {8, 8, 2},   // 20: slab form, 2048 < K <= 4096 for 17 .. 32 tokens (8 waves x 1 unit of 512 bytes, two token blocks)
};
constexpr int kNumDecodeVariants = sizeof(kDecodeVariants) / sizeof(kDecodeVariants[0]);
// Tokens come in blocks of 16; a wave keeps blocks x steps activation fragments (4 VGPRs each) in
// registers for the whole kernel.
constexpr int kDecodeStreamMaxFragments = 32;  // stream kernel: up to 64 tokens at K = 4096
constexpr int kDecodeMaxTokens = 64;      // what the family can run
constexpr int kDecodeAutoMaxTokens = 32;  // what the planner gives it whatever the variant ...
constexpr int kDecodeAutoMaxTokensStream = 48;  // ... and when the LDS-streaming variant applies: 3 token blocks still beat
                                                // 64-wide MFMA tiles (6144x48x4096 fp8: 13 us against 16), 4 blocks do not
                                                // (14336x56x4096: 21 us against 19); three blocks only up to 32 rows per CU
                                                // (planner.cpp: beyond, the 6-stage 64 x 64 tiles are as fast or faster)

// the fast epilogues the four-wave kernel is instantiated with (gemm_mfma_w4.hpp: W4_EPI_*); what else a problem asks for
// runs on variant 8
enum { W4_CLASS_NONE = -1, W4_CLASS_I32 = 0, W4_CLASS_BF16 = 1, W4_CLASS_BF16_GELU = 2 };

struct Lowered {
  GemmArgs g;
  bool has_bias;              // the epilogue adds a bias vector (its pointer may still be NULL when planning)
  bool a_kcontig, b_kcontig;  // unit K stride
  bool aligned16;             // A, B, their row pitches and batch strides are 16-byte aligned
  bool span_ok;               // one batch of A and of B each spans < 2 GiB
};

// Validates `p` and fills `out`.  With dry=true (heuristic time) data pointers and host scalars are
// not dereferenced and NULL data pointers are allowed.
uint32_t lower_problem(const zluda_gemm_problem *p, bool dry, Lowered *out);

// the fast epilogue of the four-wave kernel that serves the problem, or W4_CLASS_NONE; `dry`: planning (beta and the
// pointers are not known yet and are taken to be zero / aligned)
int w4_epilogue_class(const Lowered &l, bool dry);

// which kernel families can run the lowered problem
bool family_supports(uint32_t kernel, const Lowered &l);

// Lowers `p` with its real pointers and enqueues the kernel `plan` names on `stream` (a hipStream_t).
// `ws` / `ws_size`: device scratch for split-K partial tiles, at least plan->workspace bytes.
uint32_t launch_planned(const zluda_gemm_problem *p, const zluda_gemm_plan *plan, void *ws, uint64_t ws_size, void *stream);

} // namespace zluda_amd
