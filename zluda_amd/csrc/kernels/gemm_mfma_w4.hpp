// Persistent MFMA GEMM for K-contiguous operands on gfx950: four waves, one per SIMD, each with a 128 x 128 share of
// a 256 x 256 workgroup tile, on the 16x16 instruction shapes
//   int8 : v_mfma_i32_16x16x64_i8            fp8 (e4m3, e5m2 mixes) : v_mfma_f32_16x16x128_f8f6f4
//   f16 / bf16 : v_mfma_f32_16x16x32_*       MXFP4 : v_mfma_scale_f32_16x16x128_f8f6f4 with block scales
// for problems whose tiles fill the chip at least once.
//
// Against gemm_mfma_pipe16.hpp (eight waves of 128 x 64), same LDS ring, DMA, swizzle and fragment layout:
//   * A 128 x 128 wave tile multiplies every fragment it reads from LDS with eight others instead of four or
//     eight: 32 ds_read_b128 per wave and stage, 128 per workgroup instead of 192.
//   * The 64 accumulator tiles of a wave (256 registers) live in the AGPRs, which leaves the 256 architectural
//     VGPRs to the fragments.  The MFMAs are inline assembly with the accumulator as a tied "+a" operand: given
//     the builtin, the register allocator picks different registers for the result and the addend of most
//     MFMAs at this pressure and fills the loop with v_accvgpr moves and spills.  For the same reason the
//     epilogues fetch the accumulators with explicit v_accvgpr_read (left to itself the allocator parks most of
//     them in scratch memory right behind their last MFMA).
//   * Inline assembly is opaque to the scheduler, so the order of the loop is the order of the source: every
//     sub-step is written out as MFMA, the LDS reads and DMA instructions that follow it, MFMA, ...
//   * A wave that has its SIMD to itself has nobody to issue MFMAs while it waits, so what it waits for matters
//     more than how many instructions it issues.  Measured on MI355X (cycles per 16x16x128 MFMA of a lone wave):
//     MFMAs alone 32; with one vector memory instruction behind every MFMA 64, behind every second one 40 -- the
//     CU's address unit takes one 1 KiB instruction per 16 clocks for all four SIMDs, and a wave that queues them
//     faster stalls at issue.  The 16 DMA instructions of a stage are therefore spread over the two sub-steps
//     that follow the barrier, one behind every second MFMA (all 16 in the first of them: 7 % slower at 8192^3).
//   * One workgroup per CU walks a list of tiles (workgroup w takes tiles w, w + G, w + 2G, ... of the XCD-aware
//     order of the other kernels; G = grid size), and the stream of K stages runs on across tile boundaries:
//     the DMA is two stages ahead whatever tile they belong to.  The epilogue of a tile (straight from the
//     accumulators, no LDS) runs between two stages with the next tile's first two stages in flight, so neither
//     the fill latency of a tile's first stages nor the wait for a new workgroup is paid per tile.
//   * Every wait for the DMA is vmcnt(0) (a stage is requested one stage time before it is read and nothing
//     younger is in flight at that point), so no assumption about the order in which loads retire is made.
//
// Hazards the compiler cannot see through the assembly are covered by hand: s_nop between the accumulator
// initialisation and the first MFMA, and between the last MFMA of a tile and the first read of its results.
#pragma once
#include "gemm_mfma_pipe16.hpp"

namespace zluda_amd {

// Cache policy of the int32 epilogue's stores.  Non-temporal stores keep a D that is far larger than the memory-side
// cache from pushing the operand panels out of it, which every tile row and column reads again: 8192^3 (128 MiB of
// operands, 256 MiB of D) takes 392 us with the hint and 402 without.  Where operands and D fit that cache together the
// hint costs 4 % instead (4096^3: 62.7 us against 60.0; 8192 x 4096 x 4096: 119.7 against 115.0; 8192 x 8192 x 2048, whose
// operands are small: 145.0 against 139.6), so it is used from 128 MiB of operands and 256 MiB of D on.  (The bf16
// epilogues, with half the bytes spread over the GELU arithmetic, measure 0.3 % slower with it at 8192^3 and never use it.)
__device__ __forceinline__ bool w4_stream_d_i32(const GemmArgs &g) {
  const int64_t d_bytes = (int64_t)g.M * g.N * g.batch * 4, ab_bytes = ((int64_t)g.M + g.N) * g.K * g.batch;
  return d_bytes >= (256ll << 20) && ab_bytes >= (128ll << 20);
}

// the fast epilogue an instantiation carries; everything else a problem may ask for (and every tile that is not
// complete along P) takes the element-wise path through LDS
enum { W4_EPI_I32 = 0, W4_EPI_BF16 = 1, W4_EPI_BF16_GELU = 2 };

// one accumulator element, AGPR -> VGPR
typedef unsigned v2u __attribute__((ext_vector_type(2)));

template <class T>
__device__ __forceinline__ int w4_acc_read(const T &elem) {
  int raw = 0;
#if defined(__HIP_DEVICE_COMPILE__)  // (the register constraints mean something else to the host pass)
  asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(raw) : "a"(elem));
#endif
  return raw;
}

// The lane number, computed where it is used.  Nothing an epilogue needs per lane may stay live across the K loop: the
// loop has no register to spare, what is kept is spilled to scratch memory, and a reload from there (like every load from
// memory in an epilogue) first waits for the next tile's stages, which are in flight and older.
__device__ __forceinline__ int w4_lane_here() {
  int l = 0;
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
#endif
  return l;
}

// A value every lane holds alike, moved to a scalar register now (not where the compiler would next need it).  The
// compiler does not look inside the assembly, so the wait states it would add around the instruction are written out:
// one between a VALU write of the source and the read, two between the write of the SGPR and a VALU read of it.
__device__ __forceinline__ float w4_uniform_now(float v) {
  int o = 0;
  (void)v;
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_nop 0\n\tv_readfirstlane_b32 %0, %1\n\ts_nop 1" : "=s"(o) : "v"(f2bits(v)));
#endif
  return bits2f((uint32_t)o);
}

// Hides a scalar register's value from the optimiser at this point: what is computed from it is computed here, per tile,
// instead of once in front of the tile loop into a vector register that then has to be kept across the K loop.
__device__ __forceinline__ void w4_scalar_here(float &v) {
  int b = (int)f2bits(v);
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("" : "+s"(b));
#endif
  v = bits2f((uint32_t)b);
}

// What a wave has staged in LDS for the epilogue of its current tile: up to three vectors along P, WTP = 128 entries each
// (slot 0: the per-P scale vector alpha[] or, for a row-major D, B's; slot 1: A's; slot 2: the bias in its storage type),
// and up to two scale vectors along Q, WTQ = 128 entries each (slot 3: B's outer scales or, for a row-major D, alpha[];
// slot 4: for a row-major D, A's).  A 16-bit bias that starts at an odd element is copied from the dword in front of it:
// bias_skip = 1 element to skip.
struct W4Staged {
  static constexpr int WORDS = 128 + 4;  // per slot: 128 dwords and the one a skipped element pushes out
  static constexpr int SLOTS = 5;
  const int *area;                       // the wave's slots
  bool has[SLOTS];
  int bias_skip;
};

// Float epilogue of the four-wave kernel: D bf16 / f16 = act((scale_p * scale_q) * acc + bias) * scale_d straight from the
// accumulators (layout of gemm_mfma_pipe16.hpp: lane l holds P = 16a + 4 (l / 16) + e, Q = 16b + l % 16) on tiles complete
// along P, for problems in which nothing varies along Q (no per-column scale vector; for a row-major D no per-row vector
// or bias).  A wave that has its SIMD to itself cannot hide branches or dependent chains behind another wave, so everything
// that depends on the problem's modes is decided once, up front, into per-lane factors, and the 64 tiles are straight-line
// code: one FMA per element, then the activation (ACT fixed at compile time) with D's scale folded into it.
// QV: the problem has a scale vector along Q (one more multiplication per element, which problems without one are spared).
template <int KIND, int ACT, bool BF16, bool QV, int WTP, int WTQ, int TP, int TQ, class AccV>
__device__ __forceinline__ void w4_store_f16(const MfmaParams &prm, AccV (&acc)[TP][TQ], int p0, int q0, int NP, int NQ, int bt,
                                             int wp, int wq, const EpilogueScalars &scalars, const W4Staged &st) {
  const GemmArgs &g = prm.g;
  const int lane = w4_lane_here();
  EpilogueScalars here = scalars;
  w4_scalar_here(here.alpha_s); w4_scalar_here(here.sa_s); w4_scalar_here(here.sb_s); w4_scalar_here(here.sd);
  const bool swp = prm.swapped != 0;
  const int d_sq = (int)(swp ? g.d_si : g.d_sj);  // < 2^22 (checked before this path is taken)
  const int pc = p0 + wp * WTP, qc = q0 + wq * WTQ;
  const int64_t corner = (int64_t)qc * d_sq + pc;
  const bool to_f32 = g.d_type == CUDA_R_32F;  // (four bytes per element: a lane's four rows are its 16 bytes, no trade)
  const int dsz = to_f32 ? 4 : 2;
  char *Dw = (char *)g.D + (g.d_sb * bt + corner) * dsz;
  const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)Dw, 0, tile_window_bytes(d_sq, NP, NQ, corner, dsz), 0x00020000);
  // the scalar factor along Q (1 beside a vector) and D's scale: without an activation both fold into the P factors
  const float q_u = swp ? here.alpha_s * here.sa_s : here.sb_s;
  const float fold = ACT == ACT_NONE ? q_u * here.sd : q_u;
  const float inv_sd = 1.0f / here.sd;
  const bool to_bf16 = g.d_type == CUDA_R_16BF;  // (else f16)
  const bool relu = ACT == ACT_NONE && g.act == ACT_RELU;
  const float clip_lo = here.sd >= 0.0f ? 0.0f : -__builtin_inff(), clip_hi = here.sd >= 0.0f ? __builtin_inff() : 0.0f;
  // The factors along P (a lane's four consecutive indices of each of the TP tile rows), every mode decided once.  The
  // vectors come from the wave's staging area in LDS, never from memory: a load from memory here would first wait for
  // the next tile's stages, which are in flight and older.
  float ps[TP][4], pb[TP][4];
  const float uni = (swp ? here.sb_s : here.alpha_s * here.sa_s) * fold;  // (a scalar beside a vector is 1)
  const int l4 = 4 * (lane >> 4);  // the lane's first P index inside a 16 x 16 tile
#pragma unroll
  for (int a = 0; a < TP; a++)
#pragma unroll
    for (int e = 0; e < 4; e++) ps[a][e] = uni;
#pragma unroll
  for (int v = 0; v < 2; v++)
    if (st.has[v]) {
      v4f t[TP];
#pragma unroll
      for (int a = 0; a < TP; a++) t[a] = *(const v4f *)((const float *)st.area + v * W4Staged::WORDS + l4 + a * 16);
#pragma unroll
      for (int a = 0; a < TP; a++)
#pragma unroll
        for (int e = 0; e < 4; e++) ps[a][e] *= t[a][e];
    }
#pragma unroll
  for (int a = 0; a < TP; a++)
#pragma unroll
    for (int e = 0; e < 4; e++) pb[a][e] = 0.0f;
  if (st.has[2]) {
    const float bfold = ACT == ACT_NONE ? here.sd : 1.0f;
    const int *bias_words = st.area + 2 * W4Staged::WORDS;
    if (g.bias_type == CUDA_R_32F) {
      v4f t[TP];
#pragma unroll
      for (int a = 0; a < TP; a++) t[a] = *(const v4f *)((const float *)bias_words + l4 + a * 16);
#pragma unroll
      for (int a = 0; a < TP; a++)
#pragma unroll
        for (int e = 0; e < 4; e++) pb[a][e] = t[a][e] * bfold;
    } else {
      const bool is_bf16 = g.bias_type == CUDA_R_16BF;
      const uint16_t *q = (const uint16_t *)bias_words + st.bias_skip + l4;
      uint32_t h[TP][4];
      if (st.bias_skip == 0) {
        v2i t[TP];
#pragma unroll
        for (int a = 0; a < TP; a++) t[a] = *(const v2i *)(q + a * 16);
#pragma unroll
        for (int a = 0; a < TP; a++) {
          h[a][0] = (uint32_t)t[a][0] & 0xffffu; h[a][1] = (uint32_t)t[a][0] >> 16;
          h[a][2] = (uint32_t)t[a][1] & 0xffffu; h[a][3] = (uint32_t)t[a][1] >> 16;
        }
      } else {
#pragma unroll
        for (int a = 0; a < TP; a++)
#pragma unroll
          for (int e = 0; e < 4; e++) h[a][e] = q[a * 16 + e];
      }
#pragma unroll
      for (int a = 0; a < TP; a++)
#pragma unroll
        for (int e = 0; e < 4; e++) pb[a][e] = (is_bf16 ? dec_bf16((uint16_t)h[a][e]) : dec_f16((uint16_t)h[a][e])) * bfold;
    }
  }
  // the factors along Q: one per tile column, the lane's own column of it
  float qs[TQ];
  if constexpr (QV) {
#pragma unroll
    for (int b = 0; b < TQ; b++) qs[b] = 1.0f;
#pragma unroll
    for (int v = 3; v < 5; v++)
      if (st.has[v]) {
        float t[TQ];
#pragma unroll
        for (int b = 0; b < TQ; b++) t[b] = *((const float *)st.area + v * W4Staged::WORDS + b * 16 + (lane & 15));
#pragma unroll
        for (int b = 0; b < TQ; b++) qs[b] *= t[b];
      }
  }
  __builtin_amdgcn_sched_barrier(0);
  // One column of 16 x 16 tiles (TP tiles, 16 Q indices) at a time.  Lane l = 16 g + c holds rows 4g .. 4g + 3 of column c of
  // each tile: two packed dwords.  Tiles a and a + 1 trade halves between the lane groups g and g ^ 1 (v_permlane16_swap:
  // the odd groups' registers of the first operand against the even groups' of the second), after which a lane of an even
  // group holds rows 4g .. 4g + 7 of tile a and a lane of an odd group rows 4(g-1) .. 4(g-1) + 7 of tile a + 1: 16 bytes per
  // lane, and a store instruction writes 64 contiguous bytes of each of 16 columns instead of 32.
  static_assert(TP % 2 == 0, "tiles along P are stored in pairs");
  const int grp = lane >> 4;
  const int voff16 = ((lane & 15) * d_sq + ((grp & 1) ? 4 * grp + 12 : 4 * grp)) * 2;
#pragma unroll
  for (int b = 0; b < TQ; b++) {
    // The column's accumulators first, by explicit reads (left to itself the register allocator parks most accumulators
    // in scratch memory between their last MFMA and this point instead of leaving them in the AGPRs); then TP * 4
    // independent chains, written stage by stage over the whole column, which is the order the scheduler then keeps:
    // every instruction has TP * 4 - 1 independent ones between itself and its consumer.
    int raw[TP][4];
#pragma unroll
    for (int a = 0; a < TP; a++)
#pragma unroll
      for (int e = 0; e < 4; e++) raw[a][e] = w4_acc_read(acc[a][b][e]);
    float x[TP][4], z[TP][4];
#pragma unroll
    for (int a = 0; a < TP; a++)
#pragma unroll
      for (int e = 0; e < 4; e++) {
        float accf = KIND == KIND_I8 ? (float)raw[a][e] : bits2f((uint32_t)raw[a][e]);
        if constexpr (QV) accf *= qs[b];
        x[a][e] = __builtin_fmaf(accf, ps[a][e], pb[a][e]);
      }
    if constexpr (ACT == ACT_GELU) {
      // x * sigmoid(2u) * sd (gelu_tanh of numeric.hpp) with sd folded into the reciprocal: x / ((1 + e) / sd)
      const float c0 = -2.0f * 0.7978845608028654f * 1.4426950408889634f, c1 = 0.044715f * c0;
#pragma unroll
      for (int a = 0; a < TP; a++)
#pragma unroll
        for (int e = 0; e < 4; e++) z[a][e] = x[a][e] * x[a][e];
#pragma unroll
      for (int a = 0; a < TP; a++)
#pragma unroll
        for (int e = 0; e < 4; e++) z[a][e] = __builtin_fmaf(z[a][e], c1, c0);
#pragma unroll
      for (int a = 0; a < TP; a++)
#pragma unroll
        for (int e = 0; e < 4; e++) z[a][e] = x[a][e] * z[a][e];
#pragma unroll
      for (int a = 0; a < TP; a++)
#pragma unroll
        for (int e = 0; e < 4; e++) z[a][e] = __builtin_amdgcn_exp2f(z[a][e]);
#pragma unroll
      for (int a = 0; a < TP; a++)
#pragma unroll
        for (int e = 0; e < 4; e++) z[a][e] = __builtin_fmaf(z[a][e], inv_sd, inv_sd);
#pragma unroll
      for (int a = 0; a < TP; a++)
#pragma unroll
        for (int e = 0; e < 4; e++) z[a][e] = __builtin_amdgcn_rcpf(z[a][e]);
#pragma unroll
      for (int a = 0; a < TP; a++)
#pragma unroll
        for (int e = 0; e < 4; e++) x[a][e] = x[a][e] * z[a][e];
    } else {
      // ReLU rides on the plain instantiation (one uniform branch per tile column): D's scale is already folded into x,
      // so the clip is at zero from below for a positive scale and from above for a negative one
      if (relu) {
#pragma unroll
        for (int a = 0; a < TP; a++)
#pragma unroll
          for (int e = 0; e < 4; e++) x[a][e] = __builtin_amdgcn_fmed3f(x[a][e], clip_lo, clip_hi);
      }
    }
    // bf16 or f16 output: one uniform branch per tile column
    auto pack_store = [&](auto bf16_c) __attribute__((always_inline)) {
      constexpr bool TO_BF16 = decltype(bf16_c)::value != 0;
#pragma unroll
      for (int a = 0; a < TP; a += 2) {
        uint32_t lo[2], hi[2];  // tile a, tile a + 1
        if constexpr (TO_BF16) {
          lo[0] = pack_bf16x2(x[a][0], x[a][1]); lo[1] = pack_bf16x2(x[a][2], x[a][3]);
          hi[0] = pack_bf16x2(x[a + 1][0], x[a + 1][1]); hi[1] = pack_bf16x2(x[a + 1][2], x[a + 1][3]);
        } else {
          lo[0] = pack_f16x2(x[a][0], x[a][1]); lo[1] = pack_f16x2(x[a][2], x[a][3]);
          hi[0] = pack_f16x2(x[a + 1][0], x[a + 1][1]); hi[1] = pack_f16x2(x[a + 1][2], x[a + 1][3]);
        }
        v4i pk;
#if defined(__HIP_DEVICE_COMPILE__)
        const v2u s0 = __builtin_amdgcn_permlane16_swap(lo[0], hi[0], false, false);
        const v2u s1 = __builtin_amdgcn_permlane16_swap(lo[1], hi[1], false, false);
        pk = v4i{(int)s0[0], (int)s1[0], (int)s0[1], (int)s1[1]};
#else
        pk = v4i{(int)lo[0], (int)lo[1], (int)hi[0], (int)hi[1]};
#endif
        buffer_store_b128_guarded(pk, rs, voff16, (b * 16 * d_sq + a * 16) * 2);
      }
    };
    if (to_f32) {
      const int voff32 = ((lane & 15) * d_sq + 4 * grp) * 4;
#pragma unroll
      for (int a = 0; a < TP; a++) {
        const v4i pk = {(int)f2bits(x[a][0]), (int)f2bits(x[a][1]), (int)f2bits(x[a][2]), (int)f2bits(x[a][3])};
        buffer_store_b128_guarded(pk, rs, voff32, (b * 16 * d_sq + a * 16) * 4);
      }
    } else if (to_bf16) {
      pack_store(std::integral_constant<int, 1>{});
    } else {
      pack_store(std::integral_constant<int, 0>{});
    }
    __builtin_amdgcn_sched_barrier(0);  // one tile column at a time: what the scheduler hoists across them costs registers
  }
}

// Integer epilogue of the four-wave kernel: D int32 = alpha * acc (beta == 0, scalar alpha) on tiles complete along P
// with 16-byte aligned columns: 16 bytes per lane straight from the accumulators.
template <int WTP, int WTQ, int AUX, int TP, int TQ, class AccV>
__device__ __forceinline__ void w4_store_i32(const MfmaParams &prm, AccV (&acc)[TP][TQ], int p0, int q0, int NP, int NQ, int bt,
                                             int wp, int wq, int ialpha) {
  const GemmArgs &g = prm.g;
  const int lane = w4_lane_here();
  const int64_t d_sq = prm.swapped ? g.d_si : g.d_sj;
  const int pc = p0 + wp * WTP, qc = q0 + wq * WTQ;
  const int64_t corner = (int64_t)qc * d_sq + pc;
  int32_t *Dw = (int32_t *)g.D + g.d_sb * bt + corner;
  const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)Dw, 0, tile_window_bytes(d_sq, NP, NQ, corner, 4), 0x00020000);
  const int pitch = (int)d_sq;
  const int voff = ((lane & 15) * pitch + 4 * (lane >> 4)) * 4;
#pragma unroll
  for (int a = 0; a < TP; a++) {
    v4i v[TQ];
#pragma unroll
    for (int b = 0; b < TQ; b++)
#pragma unroll
      for (int e = 0; e < 4; e++) v[b][e] = w4_acc_read(acc[a][b][e]);
#pragma unroll
    for (int b = 0; b < TQ; b++) {
      if (ialpha != 1) v[b] *= ialpha;
      buffer_store_b128_guarded<AUX>(v[b], rs, voff, (b * 16 * pitch + a * 16) * 4);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

// Everything else (tiles that are partial along P, C reads, other output types, vectors along Q, unaligned D): element by
// element through the scalar epilogue, one row of 16 x 16 tiles at a time staged in the wave's share of LDS.  Correct for
// whatever the planner admits; not fast.  The caller guarantees that no wave still needs the LDS tiles.
template <int KIND, int WTP, int WTQ, int TP, int TQ, class AccV>
__device__ __forceinline__ void w4_store_general(const MfmaParams &prm, AccV (&acc)[TP][TQ], int *lds_words, int p0, int q0, int NP,
                                                 int NQ, int bt, int wp, int wq) {
  const GemmArgs &g = prm.g;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  int *stage = lds_words + wave * (WTQ * 16);  // [Q index of the wave tile][16 P indices of the row]
  Epilogue ep(g, bt);
  const bool swp = prm.swapped != 0;
#pragma unroll
  for (int a = 0; a < TP; a++) {
#pragma unroll
    for (int b = 0; b < TQ; b++) {
      v4i v;
#pragma unroll
      for (int e = 0; e < 4; e++) v[e] = w4_acc_read(acc[a][b][e]);
      *(v4i *)&stage[(b * 16 + (lane & 15)) * 16 + 4 * (lane >> 4)] = v;
    }
    // (LDS executes the writes and reads of one wave in program order: no barrier for wave-private rows)
#pragma unroll 1
    for (int e = lane; e < WTQ * 16; e += 64) {
      const int ql = e / 16, pl = e % 16;
      const int pi = p0 + wp * WTP + a * 16 + pl, qi = q0 + wq * WTQ + ql;
      if (pi >= NP || qi >= NQ) continue;
      const int raw = stage[ql * 16 + pl];
      const int i = swp ? qi : pi, j = swp ? pi : qi;
      if (g.int_scale) ep.store_int(i, j, raw);
      else ep.store_f(i, j, KIND == KIND_I8 ? (float)raw : bits2f((uint32_t)raw));
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

// whether the instantiation's fast epilogue serves the problem (on tiles complete along P)
template <int KIND, int EPI>
__device__ __forceinline__ bool w4_fast_epilogue_ok(const MfmaParams &prm) {
  const GemmArgs &g = prm.g;
  const int64_t d_sq = prm.swapped ? g.d_si : g.d_sj;
  const int dbytes = (EPI == W4_EPI_I32 || g.d_type == CUDA_R_32F) ? 4 : 2;
  const bool aligned = (((uintptr_t)g.D) & 15) == 0 && ((d_sq * dbytes) & 15) == 0 && ((g.d_sb * dbytes) & 15) == 0 &&
                       d_sq < (1 << 22);
  if (!aligned) return false;
  if constexpr (EPI == W4_EPI_I32) {
    return KIND == KIND_I8 && g.int_scale && g.d_type == CUDA_R_32I && g.alpha_mode != VECTOR_DEV && g.beta_mode == SCALAR_VALUE &&
           g.beta_val.i == 0;
  } else {
    // a bias that runs along Q (a row-major D's) is not served; scale vectors along Q are
    const bool q_vec = prm.swapped && g.bias != nullptr;
    // (MXFP4 has no room in LDS for staged vectors: no alpha[], no bias)
    const bool p_vec = g.alpha_mode == VECTOR_DEV || g.bias != nullptr;
    // bf16, f16 and f32 outputs; the GELU instantiation for GELU, the plain one without an activation and for ReLU
    const bool act_ok = EPI == W4_EPI_BF16_GELU ? g.act == ACT_GELU : (g.act == ACT_NONE || g.act == ACT_RELU);
    return !g.int_scale && g.beta_mode == SCALAR_VALUE && g.beta_val.f == 0.0f &&
           (g.d_type == CUDA_R_16BF || g.d_type == CUDA_R_16F || g.d_type == CUDA_R_32F) &&
           !q_vec && !(KIND == KIND_MXF4 && p_vec) && act_ok;
  }
}

template <int KIND, int FQ, int FP, int EPI>
__global__ __launch_bounds__(256) void gemm_mfma_w4_kernel(MfmaParams prm) {
  static_assert(KIND == KIND_I8 || KIND == KIND_F8 || KIND == KIND_MXF4 || kind_is_h16(KIND), "int8, fp8, MXFP4, f16 and bf16 operands");
  constexpr bool H16 = kind_is_h16(KIND);  // v_mfma_f32_16x16x32_f16 / _bf16: the byte geometry of int8 (16 bytes of K per lane and K step)
  constexpr bool MX = KIND == KIND_MXF4;
  constexpr int BP = 256, BQ = 256, WP = 2, WQ = 2;
  constexpr int NWV = 4;
  constexpr int BKB = 128, CPR = 8, RPW = 8;
  constexpr int RPP = NWV * RPW;               // rows filled per DMA pass of the workgroup
  constexpr int LP = BP / RPP, LQ = BQ / RPP;  // DMA instructions per thread, stage and operand
  constexpr int NLOAD = LP + LQ;
  constexpr int WTP = BP / WP, WTQ = BQ / WQ, TP = WTP / 16, TQ = WTQ / 16;
  constexpr int HP = TP / 2, HQ = TQ / 2;      // fragments per half of the wave tile
  constexpr int KS = KIND == KIND_F8 ? 1 : 2;  // MFMAs per fragment pair (K halves of the 128-byte stage)
  constexpr int STAGE_V4 = (BP + BQ) * CPR;    // one slot in 16-byte words: P rows, then Q rows
  constexpr int NM = HP * HQ * KS;             // MFMAs per sub-step
  constexpr int NRD = 2 * HP;                  // ds_read_b128 per sub-step (HP == HQ)
  static_assert(HP == HQ, "square wave tile");
  using acc_v = typename std::conditional<KIND == KIND_I8, v4i, v4f>::type;
  using frag_v = typename std::conditional<KIND != KIND_F8, v4i, v8i>::type;
  struct Frag { frag_v k[KS]; };

  // the two slots; behind them each wave's staging area for the vectors its epilogue needs (W4Staged).  (One array: with
  // a second LDS object in the kernel the compiler puts a vmcnt(0) in front of every LDS read that follows a DMA
  // instruction.)
  // MXFP4: behind the slots two chunks of block scales instead -- 32 scale bytes (1024 K elements = 4 stages) of each of
  // the tile's 512 rows per chunk, [row][32 bytes] -- which fills the CU's LDS: no staged vectors, and no fast epilogue
  // for problems that have any.
  constexpr int STG_WAVE = W4Staged::SLOTS * W4Staged::WORDS;
  constexpr int STG_V4 = (EPI == W4_EPI_I32 || MX) ? 0 : NWV * STG_WAVE / 4;
  constexpr int SC_CHUNK_V4 = MX ? (BP + BQ) * 2 : 0;
  constexpr int SC_BASE = 2 * STAGE_V4 + STG_V4;
  static_assert((SC_BASE + 2 * SC_CHUNK_V4) * 16 <= 160 * 1024, "LDS capacity");
  __shared__ v4i lds[SC_BASE + 2 * SC_CHUNK_V4];

  const GemmArgs &g = prm.g;
  const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wp = wave % WP, wq = wave / WP;
  const int r16 = lane & 15, g4 = lane >> 4;

  const int NP = prm.swapped ? g.N : g.M, NQ = prm.swapped ? g.M : g.N;
  const int Kbytes = MX ? g.K / 2 : H16 ? g.K * 2 : g.K;  // (two E2M1 per byte)
  const int KT2 = (Kbytes + 2 * BKB - 1) / (2 * BKB) * 2;  // stages per tile, an even number: a last odd one multiplies zeros
  const int total = prm.tiles_p * prm.tiles_q;
  const int ntiles = total * g.batch;
  const int G = (int)gridDim.x;
  const int my_tiles = (ntiles - (int)blockIdx.x + G - 1) / G;  // >= 1: the grid never exceeds the tile count
  const int ldp = ((int)(prm.swapped ? g.b_sj : g.a_si) << (H16 ? 1 : 0)) >> (MX ? 1 : 0);  // bytes
  const int ldq = ((int)(prm.swapped ? g.a_si : g.b_sj) << (H16 ? 1 : 0)) >> (MX ? 1 : 0);

  // n-th tile of this workgroup -> tile corner and batch (the order of gemm_mfma_pipe_kernel: the 8 XCDs take
  // turns at workgroup ids, so ids are spread over 8 contiguous ranges of the tile order, which walks groups
  // of group_p tiles along P; G is a multiple of 8 whenever total is)
  auto tile_coords = [&](int n, int &p0, int &q0, int &bt) __attribute__((always_inline)) {
    const int idx = (int)blockIdx.x + n * G;
    bt = idx / total;
    int w = idx - bt * total;
    if ((total & 7) == 0) w = (w & 7) * (total >> 3) + (w >> 3);
    const int group = prm.group_p * prm.tiles_q;
    const int gid = w / group, first_p = gid * prm.group_p;
    const int gsz = min(prm.tiles_p - first_p, prm.group_p);
    p0 = (first_p + (w % group) % gsz) * BP;
    q0 = ((w % group) / gsz) * BQ;
  };

  // ---- MXFP4 block scales ---------------------------------------------------------------------------------------
  // A chunk = 32 scale bytes (four stages) of each of the tile's 512 rows, [row][32] in one of two LDS buffers, filled
  // by 16 DMA instructions of 32 rows x 32 bytes (lane l -> row l / 2, half l % 2), four per wave: wave w issues parts
  // w, 4 + w (P rows), 8 + w, 12 + w (Q rows).  The planner admits K % 1024 == 0, so chunks and tiles end together and
  // stream chunk number s (tile ordinal * chunks per tile + chunk) lives in buffer s % 2.  When they are issued
  // (always behind a stage's barrier, with the data that refills the slot):
  //   chunk C >= 1 of a tile: parts 0 and 1 in the tile's stage 4 C - 4, part 2 in stage 4 C - 3, part 3 in stage 4 C - 2.
  //     Chunk C - 2, which the buffer held, was last read (the scales of stage 4 C - 5, fetched at the end of stage
  //     4 C - 6) two barriers earlier, and the chunk has landed by the barrier of stage 4 C - 1, behind which the scales
  //     of stage 4 C are fetched;
  //   chunk 0 of the next tile: all four parts in the last but one stage of the tile, right after the DMA side has moved
  //     on to that tile (landed by the last stage's barrier, behind which the next tile's first scales are fetched);
  //   chunk 0 of the first tile: with the first two stages, before the stream starts.
  // A lane needs two bytes per tile row and stage (its K blocks 2 g4 and 2 g4 + 1 of the stage's eight); op_sel picks
  // the K step's byte.
  const int KB = g.K / 32;                 // scale bytes per row
  int scP[2][MX ? TP : 1], scQ[2][MX ? TQ : 1];  // [stage parity][tile row set]
  int ss = 0;                              // stream stage number of the MFMA side
  int sc_p0 = 0, sc_q0 = 0, sc_first = 0;  // the DMA side's tile: corner, stream number of its chunk 0
  __amdgpu_buffer_rsrc_t rsSP, rsSQ;
  auto scale_tile = [&](int n, int p0, int q0, int bt) __attribute__((always_inline)) {
    if constexpr (MX) {
      sc_p0 = p0; sc_q0 = q0; sc_first = n * (KT2 / 4);
      const uint8_t *Ps = (const uint8_t *)(prm.swapped ? g.b_scale : g.a_scale) + (int64_t)bt * NP * KB;
      const uint8_t *Qs = (const uint8_t *)(prm.swapped ? g.a_scale : g.b_scale) + (int64_t)bt * NQ * KB;
      rsSP = __builtin_amdgcn_make_buffer_rsrc((void *)Ps, 0, NP * KB, 0x00020000);
      rsSQ = __builtin_amdgcn_make_buffer_rsrc((void *)Qs, 0, NQ * KB, 0x00020000);
    }
  };
  // this wave's part j (0 .. 3) of chunk c of the DMA side's tile.  (Never issued "dead": an out-of-range instruction
  // fetches nothing but still writes its zeros into LDS.)
  auto issue_scale_part = [&](int c, int j) __attribute__((always_inline)) {
    if constexpr (MX) {
      const int pt = 4 * j + wave;  // (uniform) parts 0 .. 7: P rows, 8 .. 15: Q rows
      v4i *dst = &lds[SC_BASE + ((sc_first + c) & 1) * SC_CHUNK_V4 + pt * 64];
      const int col = 32 * c + 16 * (lane & 1);
      if (j < 2) lds_dma16(rsSP, dst, min(sc_p0 + 32 * pt + (lane >> 1), NP - 1) * KB + col, 0);
      else lds_dma16(rsSQ, dst, min(sc_q0 + 32 * (pt - 8) + (lane >> 1), NQ - 1) * KB + col, 0);
    }
  };
  // ---- the DMA side: two stages ahead of the MFMAs, across tile boundaries ----------------------------------
  // one wave instruction fills 8 rows x 128 bytes; lane l -> row l / 8, slot l % 8, global chunk slot ^ swizzle(row)
  const int dr = lane / CPR, dslot = lane % CPR;
  const int drow = wave * RPW + dr;  // passes advance by RPP = 32 rows: same swizzle
  const int dcg = dslot ^ swz(drow);
  const int lane_k_left = Kbytes - dcg * 16;  // a stage that starts at or beyond this many K bytes is past the end for this lane
  int d_live = -1;         // 0 once the list is exhausted: the loads that remain read one cache line nobody uses
  int voffP[LP], voffQ[LQ];
  __amdgpu_buffer_rsrc_t rsP, rsQ;
  auto dma_tile = [&](int n) __attribute__((always_inline)) {
    int p0, q0, bt;
    tile_coords(n, p0, q0, bt);
    constexpr int SH = MX ? 1 : 0, SL = H16 ? 1 : 0;  // elements -> bytes
    const uint8_t *Pg = prm.swapped ? (const uint8_t *)g.B + (((g.b_sb * bt) << SL) >> SH) : (const uint8_t *)g.A + (((g.a_sb * bt) << SL) >> SH);
    const uint8_t *Qg = prm.swapped ? (const uint8_t *)g.A + (((g.a_sb * bt) << SL) >> SH) : (const uint8_t *)g.B + (((g.b_sb * bt) << SL) >> SH);
    // 2 GiB raw buffer windows: an offset with bit 31 set is out of range and reads as zero
    rsP = __builtin_amdgcn_make_buffer_rsrc((void *)Pg, 0, 0x80000000, 0x00020000);
    rsQ = __builtin_amdgcn_make_buffer_rsrc((void *)Qg, 0, 0x80000000, 0x00020000);
#pragma unroll
    for (int i = 0; i < LP; i++) voffP[i] = min(p0 + drow + RPP * i, NP - 1) * ldp + dcg * 16;
#pragma unroll
    for (int i = 0; i < LQ; i++) voffQ[i] = min(q0 + drow + RPP * i, NQ - 1) * ldq + dcg * 16;
    scale_tile(n, p0, q0, bt);
  };
  // instructions [I0, I1) of the NLOAD that bring stage dk of the DMA side's tile into the slot at `so`.  Lanes
  // past the end of K (the tail of the last stage, the whole padding stage of an odd stage count) are out of
  // range: zeros, no traffic.
  // PLAIN (whole stages of a live tile: no K tail, no padding stage, the tile list not exhausted): the offsets as they
  // are, no instruction per DMA to mask them.  `wave_rows` = wave * RPW * CPR, which the MXFP4 loop hides from the
  // optimiser once per stage: hoisted out of the loop, the 32 LDS addresses of a stage pair do not fit the scalar
  // registers and come back through v_readlane, each with its wait states.
  auto issue_part = [&](int dk, int so, auto i0_c, auto i1_c, auto plain_c, int wave_rows) __attribute__((always_inline)) {
    constexpr int I0 = decltype(i0_c)::value, I1 = decltype(i1_c)::value;
    constexpr bool PLAIN = decltype(plain_c)::value != 0;
    const int soff = PLAIN ? dk * BKB : (dk * BKB) & d_live;
    const int oob = soff < lane_k_left ? 0 : (int)0x80000000;
    v4i *base = &lds[so];
    static_for<I1 - I0>([&](auto k_c) {
      constexpr int k = I0 + decltype(k_c)::value;
      if constexpr (k < LP) lds_dma16(rsP, base + wave_rows + RPP * k * CPR, PLAIN ? voffP[k] : (voffP[k] | oob) & d_live, soff);
      else lds_dma16(rsQ, base + BP * CPR + wave_rows + RPP * (k - LP) * CPR, PLAIN ? voffQ[k - LP] : (voffQ[k - LP] | oob) & d_live, soff);
    });
  };

  // ---- fragment addressing (as gemm_mfma_pipe16_kernel) -------------------------------------------------------
  int fragP[2][2], fragQ[2][2];  // [tile parity][first / second 16-byte piece of the lane], 16-byte words inside a slot
#pragma unroll
  for (int par = 0; par < 2; par++)
#pragma unroll
    for (int kk = 0; kk < 2; kk++) {
      const int row = par * 16 + r16;
      // fp8: the lane's 32 bytes of its K group; int8: 16 bytes of each K half; MXFP4: 16 bytes (one scale block of 32
      // elements) of each K step from the lane group's own 32-byte range, so that its two scale bytes are neighbours
      const int ch = ((KIND == KIND_I8 || H16) ? 4 * kk + g4 : 2 * g4 + kk) ^ swz(row);
      fragP[par][kk] = (wp * WTP + row) * CPR + ch;
      fragQ[par][kk] = (BP + wq * WTQ + row) * CPR + ch;
    }
  Frag pf[2][HP], qf[2][HQ];  // [half of the wave tile][fragment]
  // ds_read_b128 number r (0 .. NRD-1) of half h of P / of Q from the slot at `so`
  auto read_piece = [&](int so, const int (&fr)[2][2], Frag (&dst)[HP], auto h_c, auto r_c) {
    constexpr int h = decltype(h_c)::value, r = decltype(r_c)::value;
    constexpr int i = r / 2, kk = r % 2, tile = h * HP + i;
    const v4i x = lds[so + (tile >> 1) * 32 * CPR + fr[tile & 1][kk]];
    if constexpr (KIND == KIND_F8) {
#pragma unroll
      for (int e = 0; e < 4; e++) dst[i].k[0][4 * kk + e] = x[e];
    } else {
      dst[i].k[kk] = x;
    }
  };

  // Scale number r (0 .. TP + TQ - 1: P tile rows, then Q's) of a stage into the registers of parity `par`, from the two
  // byte addresses scale_addr() gives for the stage: a tile row set is 16 rows x 32 bytes further on, an immediate.  (The
  // start of the chunks in LDS is hidden from the optimiser: folded into the immediates it would exceed their 16 bits and
  // every read would get an address addition of its own.)
  const int sc_lane_p = (wp * WTP + r16) * 32 + 2 * g4, sc_lane_q = (BP + wq * WTQ + r16) * 32 + 2 * g4;  // bytes in a chunk
  uint32_t sc_lds = 0;
#if defined(__HIP_DEVICE_COMPILE__)
  if constexpr (MX) {
    sc_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)&lds[SC_BASE];
    asm volatile("" : "+s"(sc_lds));
  }
#endif
  uint32_t sc_ap = 0, sc_aq = 0;
  auto scale_addr = [&](int st) __attribute__((always_inline)) {
    if constexpr (MX) {
      const uint32_t chunk = sc_lds + ((st >> 2) & 1) * (SC_CHUNK_V4 * 16) + (st & 3) * 8;  // (uniform)
      sc_ap = chunk + sc_lane_p;
      sc_aq = chunk + sc_lane_q;
    }
  };
  auto read_scale = [&](auto par_c, auto r_c) __attribute__((always_inline)) {
#if defined(__HIP_DEVICE_COMPILE__)
    if constexpr (MX) {
      constexpr int par = decltype(par_c)::value, r = decltype(r_c)::value;
      typedef __attribute__((address_space(3))) const uint16_t *lds_u16;
      if constexpr (r < TP) scP[par][r] = *(lds_u16)(uintptr_t)(sc_ap + r * 512);
      else scQ[par][r - TP] = *(lds_u16)(uintptr_t)(sc_aq + (r - TP) * 512);
    }
#endif
  };

  acc_v acc[TP][TQ];
  auto zero_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int a = 0; a < TP; a++)
#pragma unroll
      for (int b = 0; b < TQ; b++)
#pragma unroll
        for (int v = 0; v < 4; v++) acc[a][b][v] = 0;
    // (the pins keep the zeros in the AGPRs the MFMAs use; the s_nop covers VALU write -> MFMA read of SrcC)
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
    for (int a = 0; a < TP; a++)
#pragma unroll
      for (int b = 0; b < TQ; b++) asm volatile("" : "+a"(acc[a][b]));
    asm volatile("s_nop 4" ::: "memory");
#endif
  };
  // MFMA number x of the sub-step (P half ph, Q half qh): K half x / (HP * HQ), tile pair (i, j) with i the
  // slower index, so that the fragments a sub-step reads first are the ones the next sub-step multiplies first
  // par_c: the stage's parity (which MXFP4 scale registers), + 2 in a tile's first stage: the first K step of every
  // tile pair then takes 0 as its addend instead of the accumulator, which saves zeroing 256 registers per tile
  auto mfma_one = [&](auto ph_c, auto qh_c, auto x_c, auto par_c) __attribute__((always_inline)) {
    constexpr int ph = decltype(ph_c)::value, qh = decltype(qh_c)::value, x = decltype(x_c)::value, par = decltype(par_c)::value & 1;
    constexpr int ks = x / (HP * HQ), i = (x % (HP * HQ)) / HQ, j = x % HQ;
    constexpr bool ZC = (decltype(par_c)::value & 2) != 0 && ks == 0;
    acc_v &c = acc[ph * HP + i][qh * HQ + j];
    const frag_v &pa = pf[ph][i].k[ks], &qb = qf[qh][j].k[ks];  // (named here: asm operands alone do not capture)
    (void)c; (void)pa; (void)qb; (void)par;
#if defined(__HIP_DEVICE_COMPILE__)  // (the register constraints mean something else to the host pass)
#define W4_MFMA(op, tail)                                                                 \
  do {                                                                                    \
    if constexpr (ZC) asm volatile(op " %0, %1, %2, 0" tail : "=a"(c) : "v"(pa), "v"(qb)); \
    else asm volatile(op " %0, %1, %2, %0" tail : "+a"(c) : "v"(pa), "v"(qb));             \
  } while (0)
#define W4_MFMA_SCALED(sel)                                                                                                   \
  do {                                                                                                                        \
    if constexpr (ZC)                                                                                                         \
      asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, 0, %3, %4 op_sel:[" sel ",0] op_sel_hi:[0,0,0] cbsz:4 blgp:4" \
                   : "=a"(c) : "v"(pa), "v"(qb), "v"(sa), "v"(sb));                                                            \
    else                                                                                                                      \
      asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel:[" sel ",0] op_sel_hi:[0,0,0] cbsz:4 blgp:4" \
                   : "+a"(c) : "v"(pa), "v"(qb), "v"(sa), "v"(sb));                                                            \
  } while (0)
    if constexpr (KIND == KIND_I8) {
      W4_MFMA("v_mfma_i32_16x16x64_i8", "");
    } else if constexpr (KIND == KIND_F16) {
      W4_MFMA("v_mfma_f32_16x16x32_f16", "");
    } else if constexpr (KIND == KIND_BF16) {
      W4_MFMA("v_mfma_f32_16x16x32_bf16", "");
    } else if constexpr (MX) {
      const int &sa = scP[par][ph * HP + i], &sb = scQ[par][qh * HQ + j];
      if constexpr (ks == 0) W4_MFMA_SCALED("0,0");
      else W4_MFMA_SCALED("1,1");
    } else if constexpr (FP == 0 && FQ == 0) {
      W4_MFMA("v_mfma_f32_16x16x128_f8f6f4", "");
    } else if constexpr (FP == 1 && FQ == 0) {
      W4_MFMA("v_mfma_f32_16x16x128_f8f6f4", " cbsz:1");
    } else if constexpr (FP == 0 && FQ == 1) {
      W4_MFMA("v_mfma_f32_16x16x128_f8f6f4", " blgp:1");
    } else {
      W4_MFMA("v_mfma_f32_16x16x128_f8f6f4", " cbsz:1 blgp:1");
    }
#undef W4_MFMA
#undef W4_MFMA_SCALED
#endif
  };

  // One sub-step: its NM MFMAs in order; behind each of the first NRD of them one fragment read (`rd(r)`), and the
  // NLOAD DMA instructions spread evenly behind all of them when the sub-step refills a slot.
  auto substep = [&](auto ph_c, auto qh_c, auto par_c, auto &&rd, auto &&extra, auto l0_c, auto l1_c, auto plain_c, int dma_dk, int dma_so,
                     int wave_rows) __attribute__((always_inline)) {
    constexpr int L0 = decltype(l0_c)::value, L1 = decltype(l1_c)::value;  // DMA instructions [L0, L1) of the stage ride along
    static_assert(NM >= NRD && NM >= L1 - L0, "room for the reads and the DMA of a sub-step");
    static_for<NM>([&](auto x_c) {
      constexpr int x = decltype(x_c)::value;
      mfma_one(ph_c, qh_c, x_c, par_c);
      if constexpr (x < NRD) rd(x_c);
      extra(x_c);
      if constexpr (L1 > L0) {
        // spread evenly: a wave that has its SIMD to itself and queues vector memory instructions faster than the CU's
        // address unit takes them (one 1 KiB instruction per 16 clocks, for all four SIMDs) keeps its next MFMA waiting
        constexpr int D0 = L0 + (L1 - L0) * x / NM, D1 = L0 + (L1 - L0) * (x + 1) / NM;
        if constexpr (D1 > D0) issue_part(dma_dk, dma_so, std::integral_constant<int, D0>{}, std::integral_constant<int, D1>{}, plain_c, wave_rows);
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  using P0 = std::integral_constant<int, 0>;
  using P1 = std::integral_constant<int, 1>;
  // One stage of the stream; ODD = parity of its number = its slot (a tile has an even number of stages, so the
  // parity inside a tile is the parity in the stream).  On entry P half 0 and Q half ODD are in registers; it
  // leaves P half 0 and Q half 1 - ODD of the next stage there, and refills its slot with stage dk of the DMA
  // side's tile.
  //   (P0, QA) reads QB | (P0, QB) reads P1 | barrier | (P1, QB) reads P0', refills the slot | (P1, QA) reads QB'
  auto do_stage = [&](auto odd_c, auto last_c, int dk) __attribute__((always_inline)) {
    constexpr int ODD = decltype(odd_c)::value;
    // last_c: 2 = the tile's last two stages (which fetch stages 0 and 1 of the next tile, if there is one); 1 = stages
    // that fetch the tile's last two stages (the K tail and the padding stage of an odd count live there); 0 = stages
    // that fetch whole stages of a live tile: their DMA offsets need no masking; 3 = a tile's first stage (as 1, and its
    // MFMAs start the accumulators instead of adding to them)
    constexpr bool LAST = decltype(last_c)::value == 2;
    using PAR = std::integral_constant<int, ODD + (decltype(last_c)::value == 3 ? 2 : 0)>;
    constexpr int so = ODD * STAGE_V4, so_next = (1 - ODD) * STAGE_V4;
    using QA = std::integral_constant<int, ODD>;
    using QB = std::integral_constant<int, 1 - ODD>;
    using Z = std::integral_constant<int, 0>;
    using LS = std::integral_constant<int, NLOAD / 2>;
    using LN = std::integral_constant<int, NLOAD>;
    auto none = [](auto) {};
    using PL = std::integral_constant<int, decltype(last_c)::value == 0 ? 1 : 0>;
    int wave_rows = wave * RPW * CPR;
#if defined(__HIP_DEVICE_COMPILE__)
    if constexpr (MX) asm volatile("" : "+s"(wave_rows));
#endif
    substep(P0{}, QA{}, PAR{}, [&](auto r_c) { read_piece(so, fragQ, qf[1 - ODD], QB{}, r_c); }, none, Z{}, Z{}, PL{}, 0, 0, 0);
    substep(P0{}, QB{}, PAR{}, [&](auto r_c) { read_piece(so, fragP, pf[1], P1{}, r_c); }, none, Z{}, Z{}, PL{}, 0, 0, 0);
    // every fragment of the stage has been requested: wait for them and for this wave's share of the next stage,
    // meet the other waves; then this slot is free and the other one readable
    wait_vmcnt_barrier<0>();
    // (MXFP4: the wave's scale instruction of this stage rides behind the second MFMA, and the next stage's scales are
    // fetched behind the fragment reads of the last sub-step)
    substep(P1{}, QB{}, PAR{}, [&](auto r_c) { read_piece(so_next, fragP, pf[0], P0{}, r_c); },
            [&](auto x_c) {
              constexpr int x = decltype(x_c)::value;
              if constexpr (MX && LAST) {
                // the next tile's chunk 0, if there is a next tile
                if constexpr (ODD == 0 && (x & 1) == 1 && x < 8) {
                  if (d_live) issue_scale_part(0, x / 2);
                }
              } else if constexpr (MX && (x == 1 || x == 3)) {
                // this is the tile's stage dk - 2: chunk (dk + 2) / 4, by the stage's position in its group of four
                const int c = (dk + 2) >> 2, phase = (dk + 2) & 3;
                if (dk + 2 < KT2) {
                  if constexpr (x == 1) {
                    if (phase != 3) issue_scale_part(c, phase == 0 ? 0 : phase + 1);
                  } else {
                    if (phase == 0) issue_scale_part(c, 1);
                  }
                }
              }
            }, Z{}, LS{}, PL{}, dk, so, wave_rows);
    substep(P1{}, QA{}, PAR{}, [&](auto r_c) { read_piece(so_next, fragQ, qf[1 - ODD], QB{}, r_c); },
            [&](auto x_c) {
              constexpr int x = decltype(x_c)::value;
              if constexpr (MX && x == NRD - 1) scale_addr(ss + 1);
              if constexpr (MX && x >= NRD && x < NRD + TP + TQ)
                read_scale(std::integral_constant<int, 1 - ODD>{}, std::integral_constant<int, x - NRD>{});
            }, LS{}, LN{}, PL{}, dk, so, wave_rows);
    if constexpr (MX) ss++;
  };
  // two stages, which refill their slots with stages dk and dk + 1 of the DMA side's tile
  auto do_pair = [&](int dk, auto last_c) __attribute__((always_inline)) {
    do_stage(std::integral_constant<int, 0>{}, last_c, dk);
    do_stage(std::integral_constant<int, 1>{}, last_c, dk + 1);
  };
  // the fragments a tile's first stage expects in registers (P half 0, Q half 0), from slot 0
  auto first_frags = [&]() __attribute__((always_inline)) {
    static_for<NRD>([&](auto r_c) { read_piece(0, fragP, pf[0], P0{}, r_c); });
    static_for<NRD>([&](auto r_c) { read_piece(0, fragQ, qf[0], P0{}, r_c); });
  };
  // (re)starts the stream at tile n: its first two stages requested and landed, its first fragments in registers
  auto prime = [&](int n) __attribute__((always_inline)) {
    d_live = -1;
    dma_tile(n);
    if constexpr (MX) {
      // (only the stream's very first tile: later ones had their chunk 0 requested in the tile before)
      if (n == 0) {
#pragma unroll
        for (int j = 0; j < 4; j++) issue_scale_part(0, j);
      }
    }
    issue_part(0, 0, std::integral_constant<int, 0>{}, std::integral_constant<int, NLOAD>{}, std::integral_constant<int, 0>{}, wave * RPW * CPR);
    issue_part(1, STAGE_V4, std::integral_constant<int, 0>{}, std::integral_constant<int, NLOAD>{}, std::integral_constant<int, 0>{}, wave * RPW * CPR);
    wait_vmcnt_barrier<0>();
    first_frags();
  };

  const bool fast = w4_fast_epilogue_ok<KIND, EPI>(prm);
  // The scalars behind device pointers, once for all tiles and wave-uniform (SGPRs): fetched in a tile's epilogue each
  // would first wait for the next tile's stages, which are in flight and older.
  EpilogueScalars scalars(g);
  scalars.alpha_s = w4_uniform_now(scalars.alpha_s); scalars.beta_s = w4_uniform_now(scalars.beta_s);
  scalars.sa_s = w4_uniform_now(scalars.sa_s); scalars.sb_s = w4_uniform_now(scalars.sb_s);
  scalars.sc = w4_uniform_now(scalars.sc); scalars.sd = w4_uniform_now(scalars.sd);
  int ialpha = 1;
  const bool stream_d = EPI == W4_EPI_I32 && w4_stream_d_i32(g);  // (uniform: a property of the problem)
  if constexpr (EPI == W4_EPI_I32) {
    int raw = g.alpha_mode == SCALAR_VALUE ? g.alpha_val.i : (g.alpha_mode == SCALAR_DEV ? *(const int32_t *)g.alpha_ptr : 1);
    ialpha = (int)f2bits(w4_uniform_now(bits2f((uint32_t)raw)));
  }
  W4Staged staged{(const int *)&lds[2 * STAGE_V4] + (STG_V4 == 0 ? 0 : wave * STG_WAVE), {false, false, false, false, false}, 0};
  // epilogue of the tile at (p0, q0, bt); returns false when it needed the LDS (the stream must be primed again)
  auto epilogue = [&](int p0, int q0, int bt) __attribute__((always_inline)) -> bool {
    // MFMA write -> read of the accumulators: the wait states the compiler would insert if it could see the MFMAs.
    // Nothing that reads an accumulator may be scheduled in front of them (every MFMA is followed by a scheduling
    // barrier, and so are they).
    asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    if (fast && p0 + BP <= NP) {
      if constexpr (EPI == W4_EPI_I32) {
        if (stream_d) w4_store_i32<WTP, WTQ, 2>(prm, acc, p0, q0, NP, NQ, bt, wp, wq, ialpha);
        else w4_store_i32<WTP, WTQ, 0>(prm, acc, p0, q0, NP, NQ, bt, wp, wq, ialpha);
      }
      else if (staged.has[3] || staged.has[4])
        w4_store_f16<KIND, EPI == W4_EPI_BF16_GELU ? ACT_GELU : ACT_NONE, true, true, WTP, WTQ>(prm, acc, p0, q0, NP, NQ, bt, wp, wq, scalars, staged);
      else
        w4_store_f16<KIND, EPI == W4_EPI_BF16_GELU ? ACT_GELU : ACT_NONE, true, false, WTP, WTQ>(prm, acc, p0, q0, NP, NQ, bt, wp, wq, scalars, staged);
      return true;
    }
    // the element-wise epilogue stages the accumulators in LDS: let the stages in flight land first
    wait_vmcnt_barrier<0>();
    w4_store_general<KIND, WTP, WTQ>(prm, acc, (int *)&lds[0], p0, q0, NP, NQ, bt, wp, wq);
    __syncthreads();
    return false;
  };

  // The vectors along P that the epilogue of the tile at (p0, bt) needs, this wave's WTP entries of each, into the wave's
  // staging area: requested at the top of the tile, landed by the vmcnt(0) waits of the tile's last two stages (there
  // always are two).  Only the wave itself reads them, after those waits and before it requests the next tile's.
  auto stage_vectors = [&](int p0, int q0, int bt) __attribute__((always_inline)) {
    if constexpr (EPI != W4_EPI_I32 && !MX) {
      staged.has[0] = staged.has[1] = staged.has[2] = staged.has[3] = staged.has[4] = false;
      staged.bias_skip = 0;
      if (fast && p0 + BP <= NP) {
        const int ln4 = w4_lane_here() * 4;
        const int pc = p0 + wp * WTP;
        int *const area = (int *)&lds[2 * STAGE_V4] + wave * STG_WAVE;
        // 128 dwords of a slot (and the one behind them); what lies past `bytes` is out of range and lands as zero
        auto copy = [&](const void *src, int bytes, int slot) __attribute__((always_inline)) {
          const __amdgpu_buffer_rsrc_t rsv = __builtin_amdgcn_make_buffer_rsrc((void *)src, 0, bytes, 0x00020000);
          lds_dma4(rsv, area + slot * W4Staged::WORDS, ln4, 0);
          lds_dma4(rsv, area + slot * W4Staged::WORDS + 64, ln4 + 256, 0);
        };
        const bool swp = prm.swapped != 0;
        const float *v1 = swp ? (g.b_scale_mode == SCALE_OUTER_VEC ? (const float *)g.b_scale : nullptr)
                              : (g.alpha_mode == VECTOR_DEV ? (const float *)g.alpha_ptr + g.alpha_sb * bt : nullptr);
        const float *v2 = !swp && g.a_scale_mode == SCALE_OUTER_VEC ? (const float *)g.a_scale : nullptr;
        if (v1 != nullptr) { copy(v1 + pc, WTP * 4, 0); staged.has[0] = true; }
        if (v2 != nullptr) { copy(v2 + pc, WTP * 4, 1); staged.has[1] = true; }
        if (!swp && g.bias != nullptr) {
          const int es = g.bias_type == CUDA_R_32F ? 4 : 2;
          const char *src = (const char *)g.bias + (g.bias_sb * bt + pc) * es;
          const int skip = (int)(((uintptr_t)src) & 3) >> 1;  // (dword loads)
          // (whole dwords are range-checked: the last one of a skipped start ends two bytes past the vector, inside
          // the aligned dword that holds the vector's last element)
          copy(src - 2 * skip, WTP * es + 4 * skip, 2);
          staged.has[2] = true;
          staged.bias_skip = skip;
        }
        // scale vectors along Q: what the tile has of this wave's WTQ entries (a ragged last tile: the rest reads as zero
        // and belongs to columns whose stores fall outside D's window)
        const int qc = q0 + wq * WTQ, qn = min(WTQ, NQ - qc);
        const float *q1 = swp ? (g.alpha_mode == VECTOR_DEV ? (const float *)g.alpha_ptr + g.alpha_sb * bt : nullptr)
                              : (g.b_scale_mode == SCALE_OUTER_VEC ? (const float *)g.b_scale : nullptr);
        const float *q2 = swp && g.a_scale_mode == SCALE_OUTER_VEC ? (const float *)g.a_scale : nullptr;
        if (q1 != nullptr && qn > 0) { copy(q1 + qc, qn * 4, 3); staged.has[3] = true; }
        if (q2 != nullptr && qn > 0) { copy(q2 + qc, qn * 4, 4); staged.has[4] = true; }
      }
    }
  };

  // ---- the stream -------------------------------------------------------------------------------------------------
  static_assert(!MX || NM >= NRD + TP + TQ, "room for the scale reads in a sub-step");
  prime(0);
  if constexpr (MX) {
    scale_addr(0);
    static_for<TP + TQ>([&](auto r_c) { read_scale(std::integral_constant<int, 0>{}, r_c); });
  }
  for (int n = 0; n < my_tiles; n++) {
    int p0, q0, bt;
    tile_coords(n, p0, q0, bt);
    stage_vectors(p0, q0, bt);
    if (KT2 > 2) {
      // the tile's first stage starts the accumulators
      do_stage(std::integral_constant<int, 0>{}, std::integral_constant<int, 3>{}, 2);
      do_stage(std::integral_constant<int, 1>{}, std::integral_constant<int, 1>{}, 3);
      for (int kt = 4; kt + 2 < KT2; kt += 2) do_pair(kt, std::integral_constant<int, 0>{});
      // (MXFP4: K is a whole number of stage pairs)
      if (KT2 > 4) do_pair(KT2 - 2, std::integral_constant<int, MX ? 0 : 1>{});
    } else {
      zero_acc();  // (a tile of two stages: they are the last two)
    }
    // the last two stages of the tile fetch the first two of the next one
    if (n + 1 < my_tiles) dma_tile(n + 1);
    else d_live = 0;
    do_pair(0, std::integral_constant<int, 2>{});
    const bool kept = epilogue(p0, q0, bt);
    // The first fragments of the next tile are fetched again behind the epilogue (its first stage landed before the
    // last barrier): holding them across it would take 64 of the registers the epilogue needs.
    if (n + 1 < my_tiles) {
      if (kept) first_frags();
      else prime(n + 1);
    }
  }
  __builtin_amdgcn_s_waitcnt(0);  // the loads past the end of the list have landed before the wave ends
}

} // namespace zluda_amd
