// Software-pipelined MFMA GEMM for K-contiguous operands on gfx950: the production kernel of the
// int8 / fp8 / MXFP4 families.
//
// Same tiling, operand naming (P / Q) and epilogue as gemm_mfma.hpp; what differs is the K loop:
//
//   * LDS holds NSTAGE = 4 stages of 64 K-bytes per tile row.  Global memory is copied straight into
//     LDS (buffer_load_dwordx4 ... lds) three stages ahead of the one being multiplied, so every
//     workgroup keeps ~3 x 32 KiB of loads in flight and the L2 / Infinity-Fabric latency is covered
//     by three stage periods instead of one.
//   * The LDS -> register fragment loads run one MFMA sub-step ahead of the MFMAs that consume them
//     (double-buffered fragment registers), so a wave never waits on the ds_read it just issued.
//   * One s_barrier per stage, with a counted s_waitcnt vmcnt(n) in front of it that only waits for
//     the stage about to be read; younger stages stay in flight across the barrier.
//
// LDS rows are 64 B = four 16-byte chunks; chunk c of row r sits at slot c ^ ((r >> 2) & 3), which
// makes both the 1 KiB-per-instruction LDS DMA writes and the ds_read_b128 fragment reads (32 rows,
// same chunk) bank-conflict free.
#pragma once
#include "gemm_mfma.hpp"

namespace zluda_amd {

constexpr int PIPE_BKB = 64;    // K bytes per stage
constexpr int PIPE_NSTAGE = 4;  // LDS ring depth

__device__ __forceinline__ int swz4(int r) { return (r >> 2) & 3; }

// s_waitcnt with only the vector-memory counter constrained (gfx9 encoding: vmcnt = [3:0] | [15:14])
// Wait until at most N vector-memory operations of this wave are outstanding, then join the
// workgroup barrier.  Written as inline assembly with a memory clobber: the compiler must neither
// move LDS accesses across the barrier nor add the vmcnt(0) a fence would bring (younger stages have
// to stay in flight).
template <int N>
__device__ __forceinline__ void wait_vmcnt_barrier() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(N) : "memory");
}

// 4 bytes per lane from a buffer straight into LDS (buffer_load_dword ... lds): lane l lands at byte
// l*4 of the 256-byte block starting at the wave-uniform `lds_dst`.
__device__ __forceinline__ void lds_dma4(__amdgpu_buffer_rsrc_t rs, void *lds_dst, int voff, int soff) {
#if defined(__HIP_DEVICE_COMPILE__)
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void *)lds_dst, 4, voff,
                                           soff, 0, 0);
#endif
}

template <int KIND, int FQ, int FP, int BP, int BQ, int WP, int WQ>
__global__ __launch_bounds__(WP *WQ * 64) void gemm_mfma_pipe_kernel(MfmaParams prm) {
  constexpr int NT = WP * WQ * 64;
  constexpr int RPP = NT / 4;                  // rows filled per DMA pass (16 per wave)
  constexpr int LP = BP / RPP, LQ = BQ / RPP;  // DMA instructions per thread, stage and operand
  constexpr int LS = KIND == KIND_MXF4 ? (BP + BQ) / NT : 0;  // scale DMA instructions per thread and stage
  constexpr int NLOAD = LP + LQ + LS;          // vmcnt units per stage
  constexpr int WTP = BP / WP, WTQ = BQ / WQ;
  constexpr int TP = WTP / 32, TQ = WTQ / 32;
  constexpr int KS = KIND == KIND_F8 ? 1 : 2;  // MFMA sub-steps per stage
  // one stage in 16-byte units: P rows, Q rows, then (MXFP4) one scale dword per P row and Q row
  constexpr int STAGE_V4 = (BP + BQ) * 4 + (KIND == KIND_MXF4 ? (BP + BQ) / 4 : 0);
  static_assert(BP % RPP == 0 && BQ % RPP == 0 && RPP % 16 == 0, "tile / copy-pass mismatch");
  static_assert((BP + BQ) % NT == 0 && BP % 64 == 0, "scale rows are copied 64 per wave instruction");
  using acc_v = typename std::conditional<KIND == KIND_I8, v16i, v16f>::type;
  using frag_v = typename std::conditional<KIND == KIND_I8, v4i, v8i>::type;
  struct Frags {
    frag_v p[TP], q[TQ];
    int sp[KIND == KIND_MXF4 ? TP : 1], sq[KIND == KIND_MXF4 ? TQ : 1];
  };

  __shared__ v4i lds[PIPE_NSTAGE * STAGE_V4];

  const GemmArgs &g = prm.g;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wp = wave % WP, wq = wave / WP;
  const int lr = lane & 31, gsel = lane >> 5;
  const int bt = blockIdx.y;

  // ---- workgroup -> tile (see gemm_mfma.hpp) ---------------------------------------------------
  const int total = prm.tiles_p * prm.tiles_q;
  int w = blockIdx.x;
  if ((total & 7) == 0) w = (w & 7) * (total >> 3) + (w >> 3);
  const int group = prm.group_p * prm.tiles_q;
  const int gid = w / group, first_p = gid * prm.group_p;
  const int gsz = min(prm.tiles_p - first_p, prm.group_p);
  const int tile_p = first_p + (w % group) % gsz, tile_q = (w % group) / gsz;
  const int p0 = tile_p * BP, q0 = tile_q * BQ;

  const int NP = prm.swapped ? g.N : g.M, NQ = prm.swapped ? g.M : g.N;
  constexpr int ebits = KIND == KIND_MXF4 ? 4 : 8;
  const int Kbytes = (int)((int64_t)g.K * ebits / 8);
  const uint8_t *Pg, *Qg;
  int ldp, ldq;
  if (!prm.swapped) {
    Pg = (const uint8_t *)g.A + g.a_sb * bt * ebits / 8; ldp = (int)(g.a_si * ebits / 8);
    Qg = (const uint8_t *)g.B + g.b_sb * bt * ebits / 8; ldq = (int)(g.b_sj * ebits / 8);
  } else {
    Pg = (const uint8_t *)g.B + g.b_sb * bt * ebits / 8; ldp = (int)(g.b_sj * ebits / 8);
    Qg = (const uint8_t *)g.A + g.a_sb * bt * ebits / 8; ldq = (int)(g.a_si * ebits / 8);
  }
  const int KT = (Kbytes + PIPE_BKB - 1) / PIPE_BKB;  // real stages
  const int KT2 = (KT + 1) & ~1;                      // stages run: the loop body handles two

  // 2 GiB raw buffer windows: an offset with bit 31 set is out of range and reads as zero
  const __amdgpu_buffer_rsrc_t rsP = __builtin_amdgcn_make_buffer_rsrc((void *)Pg, 0, 0x80000000, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsQ = __builtin_amdgcn_make_buffer_rsrc((void *)Qg, 0, 0x80000000, 0x00020000);

  // DMA: one wave instruction fills 16 rows x 64 B; lane l -> row l/4, slot l%4, global chunk
  // slot ^ swz4(row)
  const int drow = wave * 16 + (lane >> 2), dslot = lane & 3, dcg = dslot ^ swz4(lane >> 2);
  int voffP[LP], voffQ[LQ];
#pragma unroll
  for (int i = 0; i < LP; i++) voffP[i] = min(p0 + drow + RPP * i, NP - 1) * ldp + dcg * 16;
#pragma unroll
  for (int i = 0; i < LQ; i++) voffQ[i] = min(q0 + drow + RPP * i, NQ - 1) * ldq + dcg * 16;
  const int tail_bytes = Kbytes - (KT - 1) * PIPE_BKB;
  const int oob_last = dcg * 16 < tail_bytes ? 0 : (int)0x80000000;

  // MX block scales: stage kt covers K blocks 4kt..4kt+3 of a row = one aligned dword of the
  // [row][K/32] scale tensor.  Row r of the tile (P rows first, then Q rows) is copied by the thread
  // with t + NT*i == r; bytes gsel*2 + ks of the dword belong to lane group gsel.
  __amdgpu_buffer_rsrc_t rsS[LS > 0 ? LS : 1];
  int voffS[LS > 0 ? LS : 1];
  if constexpr (KIND == KIND_MXF4) {
    const int KB = g.K / 32;
    const uint8_t *Ps = (const uint8_t *)(prm.swapped ? g.b_scale : g.a_scale) + (int64_t)bt * NP * KB;
    const uint8_t *Qs = (const uint8_t *)(prm.swapped ? g.a_scale : g.b_scale) + (int64_t)bt * NQ * KB;
#pragma unroll
    for (int i = 0; i < LS; i++) {
      const int r = t + NT * i;  // BP is a multiple of 64, so a wave never straddles P and Q
      const bool isq = r >= BP;
      rsS[i] = __builtin_amdgcn_make_buffer_rsrc((void *)(isq ? Qs : Ps), 0, 0x80000000, 0x00020000);
      voffS[i] = isq ? min(q0 + r - BP, NQ - 1) * KB : min(p0 + r, NP - 1) * KB;
    }
  }

  // stage kt -> LDS slot (16-byte units `so`); kt >= KT is a padding stage that is zero-filled
  auto issue_stage = [&](int kt, int so) {
    const int oob = kt >= KT ? (int)0x80000000 : (kt == KT - 1 ? oob_last : 0);
    v4i *base = &lds[so];
#pragma unroll
    for (int i = 0; i < LP; i++)
      lds_dma16(rsP, base + (wave * 16 + RPP * i) * 4, voffP[i] | oob, kt * PIPE_BKB);
#pragma unroll
    for (int i = 0; i < LQ; i++)
      lds_dma16(rsQ, base + (BP + wave * 16 + RPP * i) * 4, voffQ[i] | oob, kt * PIPE_BKB);
    if constexpr (KIND == KIND_MXF4) {
      int *sbase = (int *)(base + (BP + BQ) * 4);
#pragma unroll
      for (int i = 0; i < LS; i++)
        lds_dma4(rsS[i], sbase + wave * 64 + NT * i, voffS[i], min(kt, KT - 1) * 4);
    }
  };

  // fragment (and MX scale) loads of sub-step ks of the stage in LDS slot `so`
  const int fsw = swz4(lr);  // wave-tile bases are multiples of 32: swz4(row) == swz4(lr)
  auto load_frags = [&](int so, int ks, Frags &f) {
    const v4i *Pl = &lds[so + (wp * WTP + lr) * 4];
    const v4i *Ql = &lds[so + (BP + wq * WTQ + lr) * 4];
    if constexpr (KIND == KIND_F8) {
      const int c0 = (gsel * 2) ^ fsw, c1 = (gsel * 2 + 1) ^ fsw;
#pragma unroll
      for (int i = 0; i < TP; i++) {
        const v4i lo = Pl[i * 32 * 4 + c0], hi = Pl[i * 32 * 4 + c1];
        f.p[i] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
#pragma unroll
      for (int i = 0; i < TQ; i++) {
        const v4i lo = Ql[i * 32 * 4 + c0], hi = Ql[i * 32 * 4 + c1];
        f.q[i] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
    } else {
      // int8: chunk ks*2+gsel (natural K order); fp4: chunk gsel*2+ks, so that the two sub-steps of
      // a lane group use consecutive scale bytes
      const int ch = (KIND == KIND_I8 ? ks * 2 + gsel : gsel * 2 + ks) ^ fsw;
#pragma unroll
      for (int i = 0; i < TP; i++) {
        const v4i lo = Pl[i * 32 * 4 + ch];
        if constexpr (KIND == KIND_I8) f.p[i] = lo;
        else f.p[i] = v8i{lo[0], lo[1], lo[2], lo[3], 0, 0, 0, 0};
      }
#pragma unroll
      for (int i = 0; i < TQ; i++) {
        const v4i lo = Ql[i * 32 * 4 + ch];
        if constexpr (KIND == KIND_I8) f.q[i] = lo;
        else f.q[i] = v8i{lo[0], lo[1], lo[2], lo[3], 0, 0, 0, 0};
      }
      if constexpr (KIND == KIND_MXF4) {
        const int *Sl = (const int *)&lds[so + (BP + BQ) * 4];
#pragma unroll
        for (int i = 0; i < TP; i++) f.sp[i] = Sl[wp * WTP + i * 32 + lr] >> (gsel * 16);
#pragma unroll
        for (int i = 0; i < TQ; i++) f.sq[i] = Sl[BP + wq * WTQ + i * 32 + lr] >> (gsel * 16);
      }
    }
  };

  acc_v acc[TQ][TP];
#pragma unroll
  for (int a = 0; a < TQ; a++)
#pragma unroll
    for (int b = 0; b < TP; b++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[a][b][v] = 0;

  auto mfma_all = [&](const Frags &f, auto ks_c) {
    constexpr int ks = decltype(ks_c)::value;
#pragma unroll
    for (int a = 0; a < TQ; a++)
#pragma unroll
      for (int b = 0; b < TP; b++) {
        if constexpr (KIND == KIND_I8)
          acc[a][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.q[a], f.p[b], acc[a][b], 0, 0, 0);
        else if constexpr (KIND == KIND_F8)
          acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(f.q[a], f.p[b], acc[a][b], FQ, FP, 0, 0, 0, 0);
        else
          acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(f.q[a], f.p[b], acc[a][b], 4, 4, ks, f.sq[a],
                                                                       ks, f.sp[b]);
      }
  };
  using c0_t = std::integral_constant<int, 0>;
  using c1_t = std::integral_constant<int, 1>;

  // ---- prologue: stages 0 .. 2 in flight, stage 0 landed ------------------------------------------
  issue_stage(0, 0);
  issue_stage(1, STAGE_V4);
  issue_stage(2, 2 * STAGE_V4);
  wait_vmcnt_barrier<2 * NLOAD>();

  Frags fa, fb;
  load_frags(0, 0, fa);

  // One stage.  On entry the fragments of its first sub-step are in `cur`; on exit the fragments
  // of the next stage's first sub-step are in `cur` (KS == 2) or in `oth` (KS == 1).  Before the
  // last sub-step: wait for stage kt+1 (younger stages stay in flight), barrier (every wave is now
  // also done reading stage kt-1), refill that slot with stage kt+3, fetch the next fragments.
  auto do_stage = [&](int kt, int so, Frags &cur, Frags &oth) {
    const int so_next = so == 3 * STAGE_V4 ? 0 : so + STAGE_V4;
    const int so_issue = so == 0 ? 3 * STAGE_V4 : so - STAGE_V4;
    // sched_barrier(0) pins the order "fetch the next fragments, then the whole MFMA cluster": left
    // alone, the scheduler sinks each ds_read to just before its first use and the wave stalls on it.
    if constexpr (KS == 2) {
      load_frags(so, 1, oth);
      __builtin_amdgcn_sched_barrier(0);
      mfma_all(cur, c0_t{});
      __builtin_amdgcn_sched_barrier(0);
      wait_vmcnt_barrier<NLOAD>();
      issue_stage(kt + 3, so_issue);
      load_frags(so_next, 0, cur);
      __builtin_amdgcn_sched_barrier(0);
      mfma_all(oth, c1_t{});
      __builtin_amdgcn_sched_barrier(0);
    } else {
      wait_vmcnt_barrier<NLOAD>();
      issue_stage(kt + 3, so_issue);
      load_frags(so_next, 0, oth);
      __builtin_amdgcn_sched_barrier(0);
      mfma_all(cur, c0_t{});
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // K loop, two stages per trip, no other control flow.  Padding stages (kt >= KT) multiply zeros.
  int so = 0;
  for (int kt = 0; kt < KT2; kt += 2) {
    do_stage(kt, so, fa, fb);
    if constexpr (KS == 2) do_stage(kt + 1, so + STAGE_V4, fa, fb);
    else do_stage(kt + 1, so + STAGE_V4, fb, fa);
    so = so == 0 ? 2 * STAGE_V4 : 0;
  }

  // every wave is done with the LDS tiles (and every DMA has landed) before they become staging
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  mfma_store_tile<KIND, WP, WQ, WTP, WTQ>(prm, acc, (int *)&lds[0], sizeof(lds), p0, q0, NP, NQ, bt);
}

} // namespace zluda_amd
