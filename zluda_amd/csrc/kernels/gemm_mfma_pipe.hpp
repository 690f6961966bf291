// Software-pipelined MFMA GEMM for K-contiguous operands on gfx950: the production kernel of the
// int8 / fp8 / MXFP4 / f16 / bf16 / f32 families.
//
// Same tiling, operand naming (P / Q) and epilogue as gemm_mfma.hpp; what differs is the K loop:
//
//   * LDS is a ring of NSTAGE stages of BKB K-bytes per tile row, filled straight from global memory
//     (buffer_load_dwordx4 ... lds).  BKB = 128 makes every row segment a whole 128-byte cache line:
//     measured on MI355X, L2-resident panels stream into LDS at ~126 GB/s per CU with 128-byte
//     segments and at half that with 64-byte segments.
//   * A slot is refilled as soon as its last fragments are in registers (one MFMA sub-step before
//     its stage ends), NSTAGE stages ahead of the stage it will hold.
//   * The LDS -> register fragment loads run one MFMA sub-step ahead of the MFMAs that consume them
//     (double-buffered fragment registers, order pinned with sched_barrier), so a wave never waits
//     on a ds_read it has just issued.
//   * One s_barrier per stage with a counted s_waitcnt vmcnt(n) in front of it that only waits for
//     the stage about to be read; younger stages stay in flight across the barrier.
//
// LDS rows are BKB bytes = BKB/16 chunks of 16 bytes, XOR-swizzled with the row number so that the
// 1 KiB-per-instruction DMA writes and the ds_read_b128 fragment reads are bank-conflict free.
#pragma once
#include "gemm_mfma.hpp"
#include "mfma_wait_counts.hpp"

namespace zluda_amd {

// chunk swizzles: 8 chunks per 128-byte row (swz, gemm_mfma.hpp) or 4 chunks per 64-byte row
__device__ __forceinline__ int swz4(int r) { return (r >> 2) & 3; }

// Wait until at most N vector-memory operations of this wave are outstanding and every LDS read it
// issued has returned, then join the workgroup barrier.  Inline assembly with a memory clobber: the
// compiler must neither move LDS accesses across the barrier nor add the vmcnt(0) a fence would
// bring (younger stages have to stay in flight).
template <int N>
__device__ __forceinline__ void wait_vmcnt_barrier() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory");
}

template <int KIND, int FQ, int FP, int BP, int BQ, int WP, int WQ, int BKB_, int NSTAGE>
__global__ __launch_bounds__(WP *WQ * 64) void gemm_mfma_pipe_kernel(MfmaParams prm) {
  constexpr int NT = WP * WQ * 64;
  // The DMA side's instruction counts and the counted waits come from mfma_wait_counts.hpp, where the rule they rest on
  // is written down and from where a host program replays them.  In short: one wave instruction fills RPW rows x BKB
  // bytes; MX block scales travel in chunks of 32 scale bytes per tile row (1024 K elements = CH stages), double
  // buffered behind the data stages, one DMA instruction per 32 rows x 32 bytes, LS of them per wave and stage (the
  // instructions a chunk does not need read a single cache line, so that the bookkeeping is the same in every stage).
  // The counted waits only count the DATA instructions of the younger stages: the scale instructions of a stage are
  // issued in front of its data, so a wait that also covers them costs nothing, and it does not depend on when the
  // surplus ones are counted as done -- seen on MI355X: with the scale instructions counted, workgroups that follow
  // another one on their CU multiplied 1 KiB blocks of the last operand rows of a stage before they had landed.
  constexpr bool MX = KIND == KIND_MXF4;
  constexpr PipeCounts PC = pipe_counts(MX, BP, BQ, WP, WQ, BKB_, NSTAGE);
  constexpr int CPR = PC.cpr, RPW = PC.rpw, RPP = PC.rpp, LP = PC.lp, LQ = PC.lq;
  constexpr int CH = PC.ch, SPARTS = PC.sparts, NWV = PC.nwv, LS = PC.ls, PRO_S = PC.pro_s;
  constexpr int CHUNK_V4 = MX ? (BP + BQ) * 2 : 0;
  constexpr int NLOAD = PC.nload, NDATA = PC.ndata;
  constexpr int WTP = BP / WP, WTQ = BQ / WQ;
  constexpr int TP = WTP / 32, TQ = WTQ / 32;
  constexpr int KS = BKB_ / (KIND == KIND_F8 ? 64 : 32);  // MFMA sub-steps per stage
  constexpr int SPT = (KS & 1) ? 2 : 1;        // stages per loop trip (fragment roles must realign)
  constexpr int STAGE_V4 = (BP + BQ) * CPR;    // one stage in 16-byte units: P rows, then Q rows
  static_assert(BKB_ == 64 || BKB_ == 128, "row segments are half or whole cache lines");
  static_assert(BP % RPP == 0 && BQ % RPP == 0 && RPP % 32 == 0, "tile / copy-pass mismatch");
  static_assert(!MX || (BP % 32 == 0 && BQ % 32 == 0 && CH > NSTAGE), "scale chunks: 32 rows per instruction, fetched NSTAGE stages early");
  static_assert((NSTAGE - 1) * NLOAD < 64, "vmcnt range");
  static_assert((NSTAGE * STAGE_V4 + 2 * CHUNK_V4) * 16 <= 160 * 1024, "LDS capacity");
  using acc_v = typename std::conditional<KIND == KIND_I8, v16i, v16f>::type;
  constexpr bool B16 = KIND == KIND_I8 || kind_is_h16(KIND) || KIND == KIND_F32;  // 16 bytes of K per lane and sub-step (else 32)
  constexpr int MPS = KIND == KIND_F32 ? 4 : 1;  // MFMAs per fragment pair and sub-step
  using frag_v = typename std::conditional<B16, v4i, v8i>::type;
  struct Frags { frag_v p[TP], q[TQ]; };
  struct Scales { int p[TP], q[TQ]; };  // MX scale dwords of one stage (one per MFMA tile row set)

  __shared__ v4i lds[NSTAGE * STAGE_V4 + 2 * CHUNK_V4];

  const GemmArgs &g = prm.g;
  // the wave index is uniform by construction; readfirstlane tells the compiler (LDS DMA bases and
  // buffer descriptors derived from it then live in SGPRs)
  const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
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
  constexpr int ebits = KIND == KIND_MXF4 ? 4 : 8 * kind_esz(KIND);
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
  // split-K: this workgroup's share of the stages starts k0 bytes into every row; the rest of the
  // kernel sees a shorter K
  int Kbytes_local = Kbytes;
  int k0 = 0;
  int sk0 = 0;  // MX: first scale byte of this workgroup's K range in a row of scales (the host keeps
                // split_stages a multiple of the CH stages of a scale chunk)
  if (prm.splits > 1) {
    k0 = (int)blockIdx.z * prm.split_stages * BKB_;
    Kbytes_local = max(0, min(Kbytes - k0, prm.split_stages * BKB_));
    sk0 = k0 / 16;
  }
  const int KT = (Kbytes_local + BKB_ - 1) / BKB_;  // real stages

  // 2 GiB raw buffer windows: an offset with bit 31 set is out of range and reads as zero (the lanes
  // of a K tail)
  const __amdgpu_buffer_rsrc_t rsP = __builtin_amdgcn_make_buffer_rsrc((void *)Pg, 0, 0x80000000, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsQ = __builtin_amdgcn_make_buffer_rsrc((void *)Qg, 0, 0x80000000, 0x00020000);

  // DMA: one wave instruction fills RPW rows x BKB bytes; lane l -> row l / CPR, slot l % CPR,
  // global chunk slot ^ swizzle(row)
  const int dr = lane / CPR, dslot = lane % CPR;
  const int drow = wave * RPW + dr;  // passes advance by RPP, a multiple of 32: same swizzle
  const int dcg = dslot ^ (CPR == 8 ? swz(drow) : swz4(drow));
  int voffP[LP], voffQ[LQ];
#pragma unroll
  for (int i = 0; i < LP; i++) voffP[i] = min(p0 + drow + RPP * i, NP - 1) * ldp + dcg * 16;
#pragma unroll
  for (int i = 0; i < LQ; i++) voffQ[i] = min(q0 + drow + RPP * i, NQ - 1) * ldq + dcg * 16;
  const int tail_bytes = Kbytes_local - (KT - 1) * BKB_;
  const int oob_last = dcg * 16 < tail_bytes ? 0 : (int)0x80000000;

  // MX block scales: the [row][K/32] byte tensors of both operands, through buffer windows of
  // their exact size (a chunk that runs past the end of a row reads the next row, past the end of
  // the tensor zeros; neither is ever used).  Chunk c, instruction `part`: lane l -> tile row
  // 32*part + l/2, 16-byte half l%2 of that row's bytes [32c, 32c+32).
  const int KB = g.K / 32;
  __amdgpu_buffer_rsrc_t rsSP = rsP, rsSQ = rsQ;
  int srowP = 0, srowQ = 0;
  if constexpr (MX) {
    const uint8_t *Ps = (const uint8_t *)(prm.swapped ? g.b_scale : g.a_scale) + (int64_t)bt * NP * KB;
    const uint8_t *Qs = (const uint8_t *)(prm.swapped ? g.a_scale : g.b_scale) + (int64_t)bt * NQ * KB;
    rsSP = __builtin_amdgcn_make_buffer_rsrc((void *)Ps, 0, NP * KB, 0x00020000);
    rsSQ = __builtin_amdgcn_make_buffer_rsrc((void *)Qs, 0, NQ * KB, 0x00020000);
    srowP = p0 + (lane >> 1);
    srowQ = q0 - BP + (lane >> 1);
  }
  // Every wave issues the same number of scale instructions per stage (the vmcnt bookkeeping needs
  // that), which is more than a chunk has parts.  The surplus ones (part >= SPARTS) are real loads
  // of one cache line (every lane reads the first 16 bytes of the tensor) into the 1 KiB of data slot
  // `so` that this same wave fills with its very next data instruction: loads of one wave return in
  // order, so the bytes never survive.  (Not out-of-range instructions: those complete without a
  // memory round trip and can retire ahead of older loads, see issue_stage.)
  auto issue_scale_part = [&](int c, int part, int so) {
    if constexpr (MX) {
      const bool surplus = part >= SPARTS;
      const bool isq = part >= BP / 32;  // wave-uniform: a part never straddles P and Q
      const int row = isq ? min(srowQ + 32 * part, NQ - 1) : min(srowP + 32 * part, NP - 1);
      // a chunk past the end of K is never used either: it re-reads the start of the tensor
      const int live = (!surplus && c * 32 + sk0 < KB) ? -1 : 0;
      v4i *dst = surplus ? &lds[so + wave * RPW * CPR] : &lds[NSTAGE * STAGE_V4 + (c & 1) * CHUNK_V4 + part * 64];
      lds_dma16(isq ? rsSQ : rsSP, dst, (row * KB + sk0 + c * 32 + (lane & 1) * 16) & live, 0);
    }
  };
  // the LS scale instructions a wave issues in front of the data that refills slot `so` during
  // (consumer) stage kt: its share of chunk kt/CH + 1
  auto issue_scales_for = [&](int kt, int so) {
#pragma unroll
    for (int i = 0; i < LS; i++) issue_scale_part(kt / CH + 1, ((kt % CH) * LS + i) * NWV + wave, so);
  };

  // stage kt -> LDS slot at 16-byte offset `so`.  Stages kt >= KT are never multiplied; they are
  // issued only so that every trip of the loop has the same number of vector memory operations in
  // flight, which the counted waits rely on.  They must be real loads, though (every lane re-reads
  // the first 16 bytes of the operand: one cache line per instruction): an instruction whose lanes
  // are all out of range completes without a memory round trip and was seen to retire ahead of
  // older loads, so a counted wait for the last real stage passed while its data was still on its
  // way.  (A partly out-of-range instruction, as in the K tail below, goes to memory like any other.)
  auto issue_stage = [&](int kt, int so) {
    const int live = kt < KT ? -1 : 0;  // uniform
    const int oob = kt == KT - 1 ? oob_last : 0;
    const int soff = (k0 + kt * BKB_) & live;
    v4i *base = &lds[so];
#pragma unroll
    for (int i = 0; i < LP; i++)
      lds_dma16(rsP, base + (wave * RPW + RPP * i) * CPR, (voffP[i] | oob) & live, soff);
#pragma unroll
    for (int i = 0; i < LQ; i++)
      lds_dma16(rsQ, base + (BP + wave * RPW + RPP * i) * CPR, (voffQ[i] | oob) & live, soff);
  };

  // fragment (and MX scale) loads of sub-step ks of the stage in the LDS slot at offset `so`
  const int fsw = CPR == 8 ? swz(lr) : swz4(lr);  // wave-tile bases are multiples of 32
  auto load_frags = [&](int so, auto ks_c, Frags &f) {
    constexpr int ks = decltype(ks_c)::value;
    const v4i *Pl = &lds[so + (wp * WTP + lr) * CPR];
    const v4i *Ql = &lds[so + (BP + wq * WTQ + lr) * CPR];
    if constexpr (KIND == KIND_F8) {
      const int c0 = (ks * 4 + gsel * 2) ^ fsw, c1 = (ks * 4 + gsel * 2 + 1) ^ fsw;
#pragma unroll
      for (int i = 0; i < TP; i++) {
        const v4i lo = Pl[i * 32 * CPR + c0], hi = Pl[i * 32 * CPR + c1];
        f.p[i] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
#pragma unroll
      for (int i = 0; i < TQ; i++) {
        const v4i lo = Ql[i * 32 * CPR + c0], hi = Ql[i * 32 * CPR + c1];
        f.q[i] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
    } else {
      // int8, f16, bf16: chunk ks*2+gsel (natural K order).  fp4: lane group gsel owns chunks gsel*KS .. +KS-1,
      // so that its sub-steps use consecutive scale bytes
      const int ch = (B16 ? ks * 2 + gsel : gsel * KS + ks) ^ fsw;
#pragma unroll
      for (int i = 0; i < TP; i++) {
        const v4i lo = Pl[i * 32 * CPR + ch];
        if constexpr (B16) f.p[i] = lo;
        else f.p[i] = v8i{lo[0], lo[1], lo[2], lo[3], 0, 0, 0, 0};
      }
#pragma unroll
      for (int i = 0; i < TQ; i++) {
        const v4i lo = Ql[i * 32 * CPR + ch];
        if constexpr (B16) f.q[i] = lo;
        else f.q[i] = v8i{lo[0], lo[1], lo[2], lo[3], 0, 0, 0, 0};
      }
    }
  };
  // MX scales of stage kt.  The K blocks of lane group gsel are gsel*KS .. gsel*KS+KS-1 of the
  // stage:  KS == 2: bytes gsel*2 + ks of the stage's one dword;  KS == 4: dword gsel, byte ks.
  // After the shift, op_sel = ks selects the byte in both cases.
  auto load_scales = [&](int kt, Scales &sc) {
    if constexpr (MX) {
      const int j = kt % CH;
      const int *Sl = (const int *)&lds[NSTAGE * STAGE_V4 + ((kt / CH) & 1) * CHUNK_V4] + (KS == 4 ? 2 * j + gsel : j);
      const int sh = KS == 2 ? gsel * 16 : 0;
#pragma unroll
      for (int i = 0; i < TP; i++) sc.p[i] = Sl[(wp * WTP + i * 32 + lr) * 8] >> sh;
#pragma unroll
      for (int i = 0; i < TQ; i++) sc.q[i] = Sl[(BP + wq * WTQ + i * 32 + lr) * 8] >> sh;
    }
  };

  acc_v acc[TQ][TP];
#pragma unroll
  for (int a = 0; a < TQ; a++)
#pragma unroll
    for (int b = 0; b < TP; b++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[a][b][v] = 0;

  // `sc` carries the MX scale dwords of the stage; op_sel picks byte ks of them
  auto mfma_all = [&](const Frags &f, const Scales &sc, auto ks_c) {
    constexpr int ks = decltype(ks_c)::value;
    (void)sc;
    if constexpr (KIND == KIND_F32) {
      // element by element: TP * TQ independent MFMAs between two that feed the same accumulator
#pragma unroll
      for (int e = 0; e < 4; e++)
#pragma unroll
        for (int a = 0; a < TQ; a++)
#pragma unroll
          for (int b = 0; b < TP; b++)
            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(bits2f((uint32_t)f.q[a][e]), bits2f((uint32_t)f.p[b][e]), acc[a][b], 0, 0, 0);
    } else {
#pragma unroll
    for (int a = 0; a < TQ; a++)
#pragma unroll
      for (int b = 0; b < TP; b++) {
        if constexpr (KIND == KIND_I8)
          acc[a][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f.q[a], f.p[b], acc[a][b], 0, 0, 0);
        else if constexpr (KIND == KIND_F8)
          acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(f.q[a], f.p[b], acc[a][b], FQ, FP, 0, 0, 0, 0);
        else if constexpr (KIND == KIND_F16)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, f.q[a]), __builtin_bit_cast(v8h, f.p[b]),
                                                             acc[a][b], 0, 0, 0);
        else if constexpr (KIND == KIND_BF16)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8b, f.q[a]), __builtin_bit_cast(v8b, f.p[b]),
                                                              acc[a][b], 0, 0, 0);
        else
          acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(f.q[a], f.p[b], acc[a][b], 4, 4, ks, sc.q[a],
                                                                       ks, sc.p[b]);
      }
    }
  };

  // ---- prologue: stages 0 .. NSTAGE-1 in flight, stage 0 landed -----------------------------------
  // (the first scale chunk goes first: the counted wait for stage 0 then covers it; every data stage
  // is preceded by its LS scale instructions, here as in the loop, so that the counts are uniform)
#pragma unroll
  for (int i = 0; i < PRO_S; i++) issue_scale_part(0, i * NWV + wave, 0);
#pragma unroll
  for (int s = 0; s < NSTAGE; s++) {
#pragma unroll
    for (int i = 0; i < LS; i++) issue_scale_part(0, SPARTS, s * STAGE_V4);  // surplus: one line, overwritten by the data
    issue_stage(s, s * STAGE_V4);
  }
  wait_vmcnt_barrier<PC.wait_prologue>();

  Frags fa, fb;
  Scales sc_cur, sc_nxt;
  load_frags(0, std::integral_constant<int, 0>{}, fa);
  load_scales(0, sc_nxt);

  // One stage.  On entry the fragments of its sub-step 0 are in `cur` and its MX scales in sc_nxt.
  // Sub-step s multiplies the fragments fetched during sub-step s-1 while fetching those of
  // sub-step s+1.  Before the last sub-step every fragment of the stage is in registers: wait for
  // stage kt+1 (younger stages stay in flight), barrier, refill this very slot with stage
  // kt+NSTAGE, and fetch the first fragments (and scales) of stage kt+1.
  auto do_stage = [&](int kt, int so, Frags &cur, Frags &oth) {
    const int so_next = so == (NSTAGE - 1) * STAGE_V4 ? 0 : so + STAGE_V4;
    if constexpr (KIND == KIND_MXF4) sc_cur = sc_nxt;
    static_for<KS>([&](auto s_c) {
      constexpr int s = decltype(s_c)::value;
      Frags &use = (s & 1) ? oth : cur;
      Frags &nxt = (s & 1) ? cur : oth;
      constexpr bool last = s + 1 == KS;
      if constexpr (!last) {
        load_frags(so, std::integral_constant<int, (s + 1 < KS ? s + 1 : 1)>{}, nxt);
        // MX: the next stage's scales, early (their chunk landed at least one barrier ago: the last parts
        // of a chunk are issued CH - NSTAGE stages into the chunk before it), so that the last sub-step is
        // left with the fragment reads and the refill
        if constexpr (s == 0) load_scales(kt + 1, sc_nxt);
      } else {
        wait_vmcnt_barrier<PC.wait_stage>();
        // reads first: the compiler cannot prove that the DMA (an LDS write) and these reads hit
        // different slots, so whatever comes second in the source stays second in the schedule
        load_frags(so_next, std::integral_constant<int, 0>{}, nxt);
        if constexpr (KS == 1) load_scales(kt + 1, sc_nxt);
        issue_scales_for(kt, so);
        issue_stage(kt + NSTAGE, so);
      }
      mfma_all(use, sc_cur, s_c);
      // Scheduling pattern of the sub-step: the MFMAs (which only need registers filled one sub-step
      // ago) are issued back to back, with the fragment reads of the next sub-step slotted behind the
      // first half of them and the LDS DMA of the refill behind the second half.  Without the
      // pattern the scheduler either sinks every ds_read to its first use (the wave then stalls on
      // it) or keeps the loads in one block in front of the MFMAs (the matrix pipe idles meanwhile).
      constexpr int NM = TP * TQ * MPS, NDS = (TP + TQ) * (KIND == KIND_F8 ? 2 : 1) + (KIND == KIND_MXF4 && (KS == 1 ? last : s == 0) ? TP + TQ : 0);
      constexpr int NVM = last ? NLOAD : 0, H1 = NM / 2 > 0 ? NM / 2 : 1, H2 = NM - H1 > 0 ? NM - H1 : 1;
      static_for<NM>([&](auto i_c) {
        constexpr int i = decltype(i_c)::value;
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
        if constexpr (i < H1) {
          constexpr int n = NDS * (i + 1) / H1 - NDS * i / H1;
          if constexpr (n > 0) __builtin_amdgcn_sched_group_barrier(0x100, n, 0);  // DS reads
        } else {
          constexpr int j = i - H1, n = NVM * (j + 1) / H2 - NVM * j / H2;
          if constexpr (n > 0) __builtin_amdgcn_sched_group_barrier(0x010, n, 0);  // VMEM (LDS DMA)
        }
      });
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  // K loop: SPT stages per trip, no other control flow; with two stages per trip (the fragment
  // roles realign every other stage) an odd last stage follows on its own
  int so = 0;
  int kt = 0;
  for (; kt + SPT <= KT; kt += SPT) {
    do_stage(kt, so, fa, fb);
    so = so == (NSTAGE - 1) * STAGE_V4 ? 0 : so + STAGE_V4;
    if constexpr (SPT == 2) {
      do_stage(kt + 1, so, fb, fa);
      so = so == (NSTAGE - 1) * STAGE_V4 ? 0 : so + STAGE_V4;
    }
  }
  if constexpr (SPT == 2) {
    if (kt < KT) do_stage(kt, so, fa, fb);
  }

  // every wave is done with the LDS tiles (and every DMA has landed) before they become staging
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (prm.splits > 1) {
    const int ws_np = prm.tiles_p * BP, ws_nq = prm.tiles_q * BQ;
    int32_t *ws_tile = (int32_t *)prm.ws + ((int64_t)blockIdx.z * g.batch + bt) * ws_np * ws_nq + (int64_t)q0 * ws_np + p0;
    mfma_store_tile_raw<WP, WQ, WTP, WTQ>(ws_tile, ws_np, acc);
    return;
  }
  mfma_store_tile<KIND, WP, WQ, WTP, WTQ>(prm, acc, (int *)&lds[0], sizeof(lds), p0, q0, NP, NQ, bt);
}

} // namespace zluda_amd
