// MFMA GEMM for K-contiguous int8 / fp8 operands on gfx950 built on the 16x16 instruction shapes
//   int8 : v_mfma_i32_16x16x64_i8            fp8 : v_mfma_f32_16x16x128_f8f6f4
// inside the K loop of gemm_mfma_pipe.hpp (LDS ring filled by buffer_load ... lds in whole 128-byte row
// segments, XOR-swizzled 16-byte chunks, XCD-aware workgroup -> tile order, one barrier per stage, split-K
// through the workspace).
//
// Why a second MFMA shape: the part is power limited under matrix load, so a large GEMM takes as long as
// its energy allows, and the 16x16 shapes need less of it.  Measured on MI355X at its 1400 W cap (8192^3,
// kernels running back to back for seconds, board power read from hwmon): with nothing changed but the
// instruction, the 256 x 256 tile kernel takes 5 % less time for fp8 and 7 % less for int8.  The 16x16
// shapes reduce over a deeper K per instruction and touch the accumulators half as often per multiply-add.
//
// What differs from gemm_mfma_pipe.hpp:
//   * P is the MFMA operand "A": the 16x16 result layout then gives every lane FOUR CONSECUTIVE elements
//     along D's unit-stride dimension (rows 4*(lane/16) .. +3 of a 16-row tile, column lane%16), so the
//     epilogue stores 16 bytes (int32 / f32) or 8 bytes (bf16 / f16) per lane straight from the
//     accumulators: no LDS staging, no lane exchange.
//   * A fragment is 16 rows x 128 K bytes: lane l holds row l%16 and the K bytes of lane group l/16 --
//     fp8: chunks 2*(l/16) and 2*(l/16)+1 of the 128-byte row (one instruction per stage and tile pair);
//     int8: chunks l/16 and 4 + l/16 (two instructions, K halves).  Both operands use the same assignment,
//     which is all a dot product needs.
//   * A stage is walked in four sub-steps over (P half, Q half) of the wave tile in snake order, so that
//     consecutive sub-steps share one half and only the other is fetched:
//         even stages: (P0,Q0) (P0,Q1) | (P1,Q1) (P1,Q0)        odd stages: (P0,Q1) (P0,Q0) | (P1,Q0) (P1,Q1)
//     Every fragment of the stage has been requested when its second sub-step ends; the barrier sits
//     there ("|"), and behind it the slot is refilled with stage kt+2 while the last two sub-steps fetch
//     the first fragments of stage kt+1 from the other slot into the registers that have just become free.
//     The fragment registers (both P halves, both Q halves) are as many as in gemm_mfma_pipe.hpp.
#pragma once
#include "gemm_mfma_pipe.hpp"
#include "mfma_wait_counts.hpp"

namespace zluda_amd {

// ---- epilogues for the 16x16 accumulator layout ------------------------------------------------------
// acc[a][b] is the 16 x 16 tile at (P tile a, Q tile b) of the wave tile; lane l holds elements
// P = 16a + 4*(l/16) + v (v = 0..3), Q = 16b + l%16.

// raw accumulators (int32 or fp32 bits) of a whole wave tile into a matrix of `pitch` dwords per Q column
// through the window `rs` that starts at the wave tile's corner
template <int TP, int TQ, class AccV>
__device__ __forceinline__ void mfma16_store_raw(__amdgpu_buffer_rsrc_t rs, int pitch, AccV (&acc)[TP][TQ], int mul) {
  const int lane = threadIdx.x & 63;
  const int voff = ((lane & 15) * pitch + 4 * (lane >> 4)) * 4;
#pragma unroll
  for (int b = 0; b < TQ; b++)
#pragma unroll
    for (int a = 0; a < TP; a++) {
      v4i v;
#pragma unroll
      for (int e = 0; e < 4; e++) v[e] = to_bits(acc[a][b][e]);
      if (mul != 1) v *= mul;
      buffer_store_b128_guarded(v, rs, voff, (b * 16 * pitch + a * 16) * 4);
    }
}

// float epilogue without a C read on tiles complete along P: D bf16 / f16 (8-byte stores) or f32 (WIDE:
// 16-byte stores).  The activation and the 16-bit format are workgroup-uniform branches per 16 x 16 tile
// (one instantiation serves them all: the 64 tiles of a wave are unrolled, so every further template
// argument multiplies a large body).
// FENCE: the scheduler may not move instructions from one row of 16 x 16 tiles to the next (a wave that holds more
// than the accumulators across the epilogue has no registers for what the scheduler would otherwise hoist).
// ACT_T / BF16_T >= 0 fix the activation / the 16-bit format at compile time (no branch per tile: a wave that has its
// SIMD to itself cannot hide them behind another wave's work).
template <int KIND, int WP, int WQ, int TP, int TQ, bool WIDE, bool FENCE = false, int ACT_T = -1, int BF16_T = -1, class AccV>
__device__ __forceinline__ void mfma16_store_f(const MfmaParams &prm, AccV (&acc)[TP][TQ], int p0, int q0, int NP, int NQ, int bt) {
  constexpr int WTP = TP * 16, WTQ = TQ * 16;
  constexpr int ESZ = WIDE ? 4 : 2;
  const GemmArgs &g = prm.g;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wp = wave % WP, wq = wave / WP;
  Epilogue ep(g, bt);
  const bool swp = prm.swapped != 0;
  const int act = ACT_T >= 0 ? ACT_T : g.act;
  const bool to_bf16 = BF16_T >= 0 ? BF16_T != 0 : g.d_type == CUDA_R_16BF;
  const int d_sq = (int)(swp ? g.d_si : g.d_sj);  // < 2^22 (checked by the dispatcher)
  const int pc = p0 + wp * WTP, qc = q0 + wq * WTQ;
  const int64_t corner = (int64_t)qc * d_sq + pc;
  char *Dw = (char *)g.D + (g.d_sb * bt + corner) * ESZ;
  const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)Dw, 0, tile_window_bytes(d_sq, NP, NQ, corner, ESZ), 0x00020000);
  const int voff = ((lane & 15) * d_sq + 4 * (lane >> 4)) * ESZ;
  // per-Q factors (one Q index per lane and tile column); columns past the end are dropped by the window
  float qs[TQ], qb[TQ];
#pragma unroll
  for (int b = 0; b < TQ; b++) {
    const int qi = min(qc + b * 16 + (lane & 15), NQ - 1);
    qs[b] = swp ? ep.row_scale(qi) : ep.col_scale(qi);
    qb[b] = swp ? ep.bias_at(qi) : 0.0f;
  }
  // per-P bias: the four consecutive rows of a lane are fetched with one load where the vector's type and
  // alignment allow (raw bits now, all tiles of the wave in one burst; values when they are used)
  const int bsz = g.bias_type == CUDA_R_32F ? 4 : 2;
  const bool pbias = !swp && g.bias != nullptr;
  const char *bias_b = (const char *)g.bias + g.bias_sb * bt * bsz;
  const bool wide_bias = pbias && (((uintptr_t)bias_b) & (4 * bsz - 1)) == 0;  // rows start at multiples of 4
  v4i braw[TP];
#pragma unroll
  for (int a = 0; a < TP; a++) {
    const int pi = pc + a * 16 + 4 * (lane >> 4);  // + 3 < NP: the tile is complete along P
    braw[a] = v4i{0, 0, 0, 0};
    if (wide_bias) {
      if (bsz == 4) braw[a] = *(const v4i *)(bias_b + (int64_t)pi * 4);
      else {
        const v2i h = *(const v2i *)(bias_b + (int64_t)pi * 2);
        braw[a] = v4i{h[0] & 0xffff, (int)((uint32_t)h[0] >> 16), h[1] & 0xffff, (int)((uint32_t)h[1] >> 16)};
      }
    } else if (pbias) {
#pragma unroll
      for (int e = 0; e < 4; e++) braw[a][e] = (int)ep.bias_raw(pi + e);
    }
  }
#pragma unroll
  for (int a = 0; a < TP; a++) {
    float ps[4], pb[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const int pi = pc + a * 16 + 4 * (lane >> 4) + e;
      ps[e] = swp ? ep.col_scale(pi) : ep.row_scale(pi);
      pb[e] = pbias ? ep.bias_from_raw((uint32_t)braw[a][e]) : 0.0f;
    }
#pragma unroll
    for (int b = 0; b < TQ; b++) {
      float x[4];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const float accf = KIND == KIND_I8 ? (float)to_bits(acc[a][b][e]) : bits2f((uint32_t)to_bits(acc[a][b][e]));
        x[e] = (swp ? qs[b] * ps[e] : ps[e] * qs[b]) * accf + (swp ? qb[b] : pb[e]);
      }
      if (act == ACT_GELU) {
#pragma unroll
        for (int e = 0; e < 4; e++) x[e] = gelu_tanh(x[e]);
      } else if (act == ACT_RELU) {
#pragma unroll
        for (int e = 0; e < 4; e++) x[e] = x[e] > 0.0f ? x[e] : 0.0f;
      }
#pragma unroll
      for (int e = 0; e < 4; e++) x[e] *= ep.sd;
      const int soff = (b * 16 * d_sq + a * 16) * ESZ;  // uniform
      if constexpr (WIDE) {
        const v4i pk = {(int)f2bits(x[0]), (int)f2bits(x[1]), (int)f2bits(x[2]), (int)f2bits(x[3])};
        buffer_store_b128_guarded(pk, rs, voff, soff);
      } else {
        v2i pk;
        if (to_bf16) { pk[0] = (int)pack_bf16x2(x[0], x[1]); pk[1] = (int)pack_bf16x2(x[2], x[3]); }
        else { pk[0] = (int)pack_f16x2(x[0], x[1]); pk[1] = (int)pack_f16x2(x[2], x[3]); }
        buffer_store_b64_guarded(pk, rs, voff, soff);
      }
    }
    if constexpr (FENCE) __builtin_amdgcn_sched_barrier(0);
  }
}

// the largest divisor of `tq` that does not exceed `fit`
constexpr int staging_columns(int fit, int tq) {
  int c = fit < tq ? fit : tq;
  while (c > 1 && tq % c != 0) c--;
  return c;
}

// everything else (partial tiles along P, C reads, 8-bit outputs, unaligned D, integer alpha vectors):
// element by element through the scalar epilogue.  Correct for whatever the planner admits; not fast.
// The accumulators are staged in the wave's share of the (now free) LDS, as many tile columns per pass as
// fit, so that the scalar epilogue is a rolled loop (a function call would do as well, but a call anywhere
// in the kernel makes the compiler keep the kernel arguments in private memory).
// The caller guarantees that every wave of the workgroup is done with the LDS tiles (a barrier behind the
// K loop); `lds_words` / `lds_bytes`: the workgroup's LDS.
template <int KIND, int WP, int WQ, int TP, int TQ, int LDS_BYTES, class AccV>
__device__ __forceinline__ void mfma16_store_general(const MfmaParams &prm, AccV (&acc)[TP][TQ], int *lds_words, int p0, int q0,
                                                     int NP, int NQ, int bt) {
  constexpr int WTP = TP * 16, WTQ = TQ * 16;
  constexpr int PER_WAVE = LDS_BYTES / (WP * WQ);            // bytes of staging per wave
  constexpr int COLS = staging_columns(PER_WAVE / (16 * WTP * 4), TQ);  // tile columns per pass
  static_assert(COLS >= 1 && TQ % COLS == 0, "staging passes");
  const GemmArgs &g = prm.g;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wp = wave % WP, wq = wave / WP;
  int *stage = lds_words + wave * (PER_WAVE / 4);
  Epilogue ep(g, bt);
  const bool swp = prm.swapped != 0;
#pragma unroll
  for (int pass = 0; pass < TQ / COLS; pass++) {
#pragma unroll
    for (int bb = 0; bb < COLS; bb++)
#pragma unroll
      for (int a = 0; a < TP; a++) {
        v4i v;
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = to_bits(acc[a][pass * COLS + bb][e]);
        *(v4i *)&stage[(bb * 16 + (lane & 15)) * WTP + a * 16 + 4 * (lane >> 4)] = v;
      }
    // (LDS executes the writes and reads of one wave in program order: no barrier for wave-private rows)
#pragma unroll 1
    for (int e = lane; e < COLS * 16 * WTP; e += 64) {
      const int ql = e / WTP, pl = e % WTP;
      const int pi = p0 + wp * WTP + pl, qi = q0 + wq * WTQ + pass * COLS * 16 + ql;
      if (pi >= NP || qi >= NQ) continue;
      const int raw = stage[ql * WTP + pl];
      const int i = swp ? qi : pi, j = swp ? pi : qi;
      if (g.int_scale) ep.store_int(i, j, raw);
      else ep.store_f(i, j, KIND == KIND_I8 ? (float)raw : bits2f((uint32_t)raw));
    }
  }
}

template <int KIND, int WP, int WQ, int TP, int TQ, int LDS_BYTES, class AccV>
__device__ __forceinline__ void mfma16_store_tile(const MfmaParams &prm, AccV (&acc)[TP][TQ], int *lds_words, int p0, int q0, int NP,
                                                  int NQ, int bt) {
  constexpr int WTP = TP * 16, WTQ = TQ * 16;
  const GemmArgs &g = prm.g;
  const bool swp = prm.swapped != 0;
  const int64_t d_sq = swp ? g.d_si : g.d_sj;
  const bool full = p0 + WP * WTP <= NP;  // along Q the store window cuts the tile
  const int dbytes = (g.d_type == CUDA_R_32F || g.d_type == CUDA_R_32I) ? 4 : (g.d_type == CUDA_R_8I ? 1 : 2);
  const bool aligned = (((uintptr_t)g.D) & 15) == 0 && ((d_sq * dbytes) & 15) == 0 && ((g.d_sb * dbytes) & 15) == 0 &&
                       d_sq < (1 << 22);
  if constexpr (KIND == KIND_I8) {
    if (g.int_scale && full && aligned && g.alpha_mode != VECTOR_DEV && g.beta_mode == SCALAR_VALUE && g.beta_val.i == 0) {
      const int ialpha = g.alpha_mode == SCALAR_VALUE ? g.alpha_val.i : *(const int32_t *)g.alpha_ptr;
      const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
      const int pc = p0 + (wave % WP) * WTP, qc = q0 + (wave / WP) * WTQ;
      const int64_t corner = (int64_t)qc * d_sq + pc;
      int32_t *Dw = (int32_t *)g.D + g.d_sb * bt + corner;
      const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)Dw, 0, tile_window_bytes(d_sq, NP, NQ, corner, 4), 0x00020000);
      mfma16_store_raw<TP, TQ>(rs, (int)d_sq, acc, ialpha);
      return;
    }
  }
  if (!g.int_scale && full && aligned && g.beta_mode == SCALAR_VALUE && g.beta_val.f == 0.0f &&
      (g.d_type == CUDA_R_16BF || g.d_type == CUDA_R_16F || g.d_type == CUDA_R_32F)) {
    if (g.d_type == CUDA_R_32F) mfma16_store_f<KIND, WP, WQ, TP, TQ, true>(prm, acc, p0, q0, NP, NQ, bt);
    else mfma16_store_f<KIND, WP, WQ, TP, TQ, false>(prm, acc, p0, q0, NP, NQ, bt);
    return;
  }
  __syncthreads();  // (workgroup-uniform branch) the LDS tiles become staging
  mfma16_store_general<KIND, WP, WQ, TP, TQ, LDS_BYTES>(prm, acc, lds_words, p0, q0, NP, NQ, bt);
}

// ---- the kernel ----------------------------------------------------------------------------------------
template <int KIND, int FQ, int FP, int BP, int BQ, int WP, int WQ>
__global__ __launch_bounds__(WP *WQ * 64) void gemm_mfma_pipe16_kernel(MfmaParams prm) {
  static_assert(KIND == KIND_I8 || KIND == KIND_F8 || kind_is_h16(KIND), "int8, fp8, f16 and bf16 operands");
  constexpr int ESZ = kind_esz(KIND);          // f16 / bf16: the byte geometry of int8 (v_mfma_f32_16x16x32_*: 16 bytes of K per lane)
  constexpr int NT = WP * WQ * 64, NWV = NT / 64;
  constexpr int BKB = 128, CPR = 8, RPW = 8;
  constexpr Pipe16Counts PC = pipe16_counts(BP, BQ, WP, WQ);  // (shared with the host program that checks the waits)
  constexpr int RPP = PC.rpp;                  // rows filled per DMA pass of the workgroup
  constexpr int LP = PC.lp, LQ = PC.lq;        // DMA instructions per thread, stage and operand
  constexpr int NLOAD = PC.nload;
  static_assert(RPP == NWV * RPW, "eight rows per DMA instruction");
  constexpr int WTP = BP / WP, WTQ = BQ / WQ, TP = WTP / 16, TQ = WTQ / 16;
  constexpr int HP = TP / 2, HQ = TQ / 2;      // fragments per half of the wave tile
  constexpr int KS = KIND == KIND_F8 ? 1 : 2;  // MFMAs per fragment pair (K halves of the 128-byte stage)
  constexpr int NSTAGE = 2;
  constexpr int STAGE_V4 = (BP + BQ) * CPR;    // one slot in 16-byte words: P rows, then Q rows
  static_assert(BP % RPP == 0 && BQ % RPP == 0, "tile / copy-pass mismatch");
  static_assert(WTP % 32 == 0 && WTQ % 32 == 0, "wave tiles start on multiples of 32 rows (fragment swizzle)");
  static_assert(NSTAGE * STAGE_V4 * 16 <= 160 * 1024, "LDS capacity");
  using acc_v = typename std::conditional<KIND == KIND_I8, v4i, v4f>::type;
  using frag_v = typename std::conditional<KIND != KIND_F8, v4i, v8i>::type;
  struct Frag { frag_v k[KS]; };

  __shared__ v4i lds[NSTAGE * STAGE_V4];

  const GemmArgs &g = prm.g;
  const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wp = wave % WP, wq = wave / WP;
  const int r16 = lane & 15, g4 = lane >> 4;
  const int bt = blockIdx.y;

  // ---- workgroup -> tile (as in gemm_mfma_pipe_kernel) ----------------------------------------------------
  const int total = prm.tiles_p * prm.tiles_q;
  int w = blockIdx.x;
  if ((total & 7) == 0) w = (w & 7) * (total >> 3) + (w >> 3);
  const int group = prm.group_p * prm.tiles_q;
  const int gid = w / group, first_p = gid * prm.group_p;
  const int gsz = min(prm.tiles_p - first_p, prm.group_p);
  const int tile_p = first_p + (w % group) % gsz, tile_q = (w % group) / gsz;
  const int p0 = tile_p * BP, q0 = tile_q * BQ;

  const int NP = prm.swapped ? g.N : g.M, NQ = prm.swapped ? g.M : g.N;
  const int Kbytes = g.K * ESZ;
  const uint8_t *Pg, *Qg;
  int ldp, ldq;
  if (!prm.swapped) {
    Pg = (const uint8_t *)g.A + g.a_sb * bt * ESZ; ldp = (int)g.a_si * ESZ;
    Qg = (const uint8_t *)g.B + g.b_sb * bt * ESZ; ldq = (int)g.b_sj * ESZ;
  } else {
    Pg = (const uint8_t *)g.B + g.b_sb * bt * ESZ; ldp = (int)g.b_sj * ESZ;
    Qg = (const uint8_t *)g.A + g.a_sb * bt * ESZ; ldq = (int)g.a_si * ESZ;
  }
  // split-K: this workgroup's share of the stages starts k0 bytes into every row
  int Kbytes_local = Kbytes, k0 = 0;
  if (prm.splits > 1) {
    k0 = (int)blockIdx.z * prm.split_stages * BKB;
    Kbytes_local = max(0, min(Kbytes - k0, prm.split_stages * BKB));
  }
  const int KT = (Kbytes_local + BKB - 1) / BKB;  // real stages

  // 2 GiB raw buffer windows: an offset with bit 31 set is out of range and reads as zero (the lanes of a
  // K tail)
  const __amdgpu_buffer_rsrc_t rsP = __builtin_amdgcn_make_buffer_rsrc((void *)Pg, 0, 0x80000000, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsQ = __builtin_amdgcn_make_buffer_rsrc((void *)Qg, 0, 0x80000000, 0x00020000);

  // DMA: one wave instruction fills 8 rows x 128 bytes; lane l -> row l / 8, slot l % 8, global chunk
  // slot ^ swizzle(row)
  const int dr = lane / CPR, dslot = lane % CPR;
  const int drow = wave * RPW + dr;  // passes advance by RPP, a multiple of 32: same swizzle
  const int dcg = dslot ^ swz(drow);
  int voffP[LP], voffQ[LQ];
#pragma unroll
  for (int i = 0; i < LP; i++) voffP[i] = min(p0 + drow + RPP * i, NP - 1) * ldp + dcg * 16;
#pragma unroll
  for (int i = 0; i < LQ; i++) voffQ[i] = min(q0 + drow + RPP * i, NQ - 1) * ldq + dcg * 16;
  const int tail_bytes = Kbytes_local - (KT - 1) * BKB;
  const int oob_last = dcg * 16 < tail_bytes ? 0 : (int)0x80000000;

  // stage kt -> LDS slot at 16-byte offset `so`.  Stages kt >= KT are never multiplied; they are issued
  // only so that every stage has the same vector memory operations in flight, as real loads of one cache
  // line (an instruction whose lanes are all out of range completes without a memory round trip and can
  // retire ahead of older loads).
  auto issue_stage = [&](int kt, int so) {
    const int live = kt < KT ? -1 : 0;  // uniform
    const int oob = kt == KT - 1 ? oob_last : 0;
    const int soff = (k0 + kt * BKB) & live;
    v4i *base = &lds[so];
#pragma unroll
    for (int i = 0; i < LP; i++)
      lds_dma16(rsP, base + (wave * RPW + RPP * i) * CPR, (voffP[i] | oob) & live, soff);
#pragma unroll
    for (int i = 0; i < LQ; i++)
      lds_dma16(rsQ, base + (BP + wave * RPW + RPP * i) * CPR, (voffQ[i] | oob) & live, soff);
  };

  // ---- fragment addressing --------------------------------------------------------------------------------
  // Tiles start on multiples of 16 rows; the swizzle depends on the row mod 32, so even and odd tiles
  // differ.  [tile parity][first / second 16-byte piece of the lane] in 16-byte words inside a slot
  int fragP[2][2], fragQ[2][2];
#pragma unroll
  for (int par = 0; par < 2; par++)
#pragma unroll
    for (int kk = 0; kk < 2; kk++) {
      const int row = par * 16 + r16;
      const int ch = (KIND == KIND_F8 ? 2 * g4 + kk : 4 * kk + g4) ^ swz(row);
      fragP[par][kk] = (wp * WTP + row) * CPR + ch;
      fragQ[par][kk] = (BP + wq * WTQ + row) * CPR + ch;
    }
  // 16-row tile `tile` of the wave tile, from the stage in the slot at `so`
  auto load_frag = [&](int so, const int (&fr)[2][2], auto tile_c, Frag &f) {
    constexpr int tile = decltype(tile_c)::value;
    const v4i *base = &lds[so + (tile >> 1) * 32 * CPR];
    const v4i lo = base[fr[tile & 1][0]], hi = base[fr[tile & 1][1]];
    if constexpr (KIND == KIND_F8) {
      f.k[0] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    } else {
      f.k[0] = lo;
      f.k[1] = hi;
    }
  };

  acc_v acc[TP][TQ];
#pragma unroll
  for (int a = 0; a < TP; a++)
#pragma unroll
    for (int b = 0; b < TQ; b++)
#pragma unroll
      for (int v = 0; v < 4; v++) acc[a][b][v] = 0;

  Frag pf[2][HP], qf[2][HQ];  // [half of the wave tile][fragment]
  // fragments [I0, I1) of P half h
  auto load_p_part = [&](int so, auto h_c, auto i0_c, auto i1_c) {
    constexpr int h = decltype(h_c)::value, I0 = decltype(i0_c)::value, I1 = decltype(i1_c)::value;
    static_for<I1 - I0>([&](auto i_c) {
      constexpr int i = I0 + decltype(i_c)::value;
      load_frag(so, fragP, std::integral_constant<int, h * HP + i>{}, pf[h][i]);
    });
  };
  auto load_p_half = [&](int so, auto h_c) {
    load_p_part(so, h_c, std::integral_constant<int, 0>{}, std::integral_constant<int, HP>{});
  };
  auto load_q_half = [&](int so, auto h_c) {
    constexpr int h = decltype(h_c)::value;
    static_for<HQ>([&](auto i_c) {
      constexpr int i = decltype(i_c)::value;
      load_frag(so, fragQ, std::integral_constant<int, h * HQ + i>{}, qf[h][i]);
    });
  };
  // the MFMAs of P half ph against Q half qh; K half by K half, so that the two instructions of a tile
  // (int8) are a whole sub-step's worth of independent instructions apart
  auto mfma_halves = [&](auto ph_c, auto qh_c) {
    constexpr int ph = decltype(ph_c)::value, qh = decltype(qh_c)::value;
#pragma unroll
    for (int ks = 0; ks < KS; ks++)
#pragma unroll
      for (int x = 0; x < HP * HQ; x++) {
          const int i = x / HQ, j = x % HQ;
          acc_v &c = acc[ph * HP + i][qh * HQ + j];
          if constexpr (KIND == KIND_I8) c = __builtin_amdgcn_mfma_i32_16x16x64_i8(pf[ph][i].k[ks], qf[qh][j].k[ks], c, 0, 0, 0);
          else if constexpr (KIND == KIND_F16)
            c = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, pf[ph][i].k[ks]), __builtin_bit_cast(v8h, qf[qh][j].k[ks]), c, 0, 0, 0);
          else if constexpr (KIND == KIND_BF16)
            c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8b, pf[ph][i].k[ks]), __builtin_bit_cast(v8b, qf[qh][j].k[ks]), c, 0, 0, 0);
          else c = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(pf[ph][i].k[ks], qf[qh][j].k[ks], c, FP, FQ, 0, 0, 0, 0);
        }
  };
  // issue order of a sub-step: its NM MFMAs back to back, with the NDS fragment reads slotted PER_DS at a
  // time behind the first ones (what they fetch is needed one sub-step later, or by the barrier) and the
  // NVM DMA instructions behind the MFMAs that follow
  auto pattern = [&](auto nds_c, auto nvm_c) {
    constexpr int NM = HP * HQ * KS, NDS = decltype(nds_c)::value, NVM = decltype(nvm_c)::value;
    constexpr int PER_DS = 2;  // (1 and 4 per MFMA both measured slower)
    constexpr int MD = (NDS + PER_DS - 1) / PER_DS < NM ? (NDS + PER_DS - 1) / PER_DS : NM;  // MFMAs with reads behind them
    constexpr int MV = NM - MD > 0 ? NM - MD : 1;
    static_for<NM>([&](auto i_c) {
      constexpr int i = decltype(i_c)::value;
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
      if constexpr (i < MD) {
        constexpr int n = NDS * (i + 1) / MD - NDS * i / MD;
        if constexpr (n > 0) __builtin_amdgcn_sched_group_barrier(0x100, n, 0);  // DS reads
      }
      if constexpr (i >= NM - MV && NVM > 0) {
        constexpr int j = i - (NM - MV), n = NVM * (j + 1) / MV - NVM * j / MV;
        if constexpr (n > 0) __builtin_amdgcn_sched_group_barrier(0x010, n, 0);  // VMEM (LDS DMA)
      }
    });
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- prologue: stages 0 and 1 in flight, stage 0 landed, its first fragments in registers -----------------
  issue_stage(0, 0);
  issue_stage(1, STAGE_V4);
  wait_vmcnt_barrier<PC.wait_prologue>();
  load_p_half(0, std::integral_constant<int, 0>{});
  load_q_half(0, std::integral_constant<int, 0>{});

  // ---- one stage ----------------------------------------------------------------------------------------------
  // ODD = 0: on entry P half 0 and Q half 0 of the stage are in registers; the next stage will find P half 0
  // and Q half 1 of its own.  ODD = 1: the same with the Q halves exchanged.
  auto do_stage = [&](int kt, int so, int so_next, auto odd_c) {
    constexpr int QA = decltype(odd_c)::value, QB_ = 1 - QA;  // the Q half that is resident / that is fetched
    using P0 = std::integral_constant<int, 0>;
    using P1 = std::integral_constant<int, 1>;
    using QAc = std::integral_constant<int, QA>;
    using QBc = std::integral_constant<int, QB_>;
    constexpr int DSP = 2 * HP, DSQ = 2 * HQ;  // ds_read_b128 per half
    // The fragment reads are spread over the four sub-steps (the LDS is the busiest unit of the loop: 24 KiB
    // per wave and stage): EARLY fragments of P half 1 come with QB, LATE fragments of the next stage's P
    // half 0 with its first Q half.
    constexpr int EARLY = 1, LATE = 1;  // (0 / 0: 1.5 % slower at 8192^3 int8; 2 / 1: no better; whole halves early: far slower)
    using I0 = std::integral_constant<int, 0>;
    using IE = std::integral_constant<int, EARLY>;
    using IL = std::integral_constant<int, HP - LATE>;
    using IH = std::integral_constant<int, HP>;
    // (P0, QA) while QB arrives
    load_q_half(so, QBc{});
    load_p_part(so, P1{}, I0{}, IE{});
    mfma_halves(P0{}, QAc{});
    pattern(std::integral_constant<int, DSQ + 2 * EARLY>{}, std::integral_constant<int, 0>{});
    // (P0, QB) while P1 arrives
    load_p_part(so, P1{}, IE{}, IH{});
    mfma_halves(P0{}, QBc{});
    pattern(std::integral_constant<int, DSP - 2 * EARLY>{}, std::integral_constant<int, 0>{});
    // every fragment of the stage has been requested: wait for them and for this wave's share of stage
    // kt+1, meet the other waves; then the slot is free and the other one readable
    wait_vmcnt_barrier<PC.wait_stage>();
    // (P1, QB): refill this slot with stage kt+2, P half 0 of stage kt+1 arrives
    load_p_part(so_next, P0{}, I0{}, IL{});
    issue_stage(kt + NSTAGE, so);
    mfma_halves(P1{}, QBc{});
    pattern(std::integral_constant<int, DSP - 2 * LATE>{}, std::integral_constant<int, NLOAD>{});
    // (P1, QA): Q half QB of stage kt+1 arrives (that stage starts with it)
    load_p_part(so_next, P0{}, IL{}, IH{});
    load_q_half(so_next, QBc{});
    mfma_halves(P1{}, QAc{});
    pattern(std::integral_constant<int, DSQ + 2 * LATE>{}, std::integral_constant<int, 0>{});
  };

  int kt = 0;
  for (; kt + 2 <= KT; kt += 2) {
    do_stage(kt, 0, STAGE_V4, std::integral_constant<int, 0>{});
    do_stage(kt + 1, STAGE_V4, 0, std::integral_constant<int, 1>{});
  }
  if (kt < KT) do_stage(kt, 0, STAGE_V4, std::integral_constant<int, 0>{});

  __builtin_amdgcn_s_waitcnt(0);  // every DMA of the padding stages has landed before the LDS is reused or the wave ends
  if (prm.splits > 1) {
    const int ws_np = prm.tiles_p * BP, ws_nq = prm.tiles_q * BQ;
    int32_t *ws_tile = (int32_t *)prm.ws + ((int64_t)blockIdx.z * g.batch + bt) * ws_np * ws_nq + (int64_t)(q0 + wq * WTQ) * ws_np + p0 + wp * WTP;
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)ws_tile, 0, 0xFFFFFFFF, 0x00020000);
    mfma16_store_raw<TP, TQ>(rs, ws_np, acc, 1);
    return;
  }
  mfma16_store_tile<KIND, WP, WQ, TP, TQ, (int)sizeof(lds)>(prm, acc, (int *)&lds[0], p0, q0, NP, NQ, bt);
}

} // namespace zluda_amd
