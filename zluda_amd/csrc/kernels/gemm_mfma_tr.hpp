// MFMA GEMM for 8-bit operands (int8, OCP fp8), 16-bit operands (f16, bf16) and f32 operands of which at least one is
// NOT K-contiguous: a column-major A without transpose (unit stride along M), a B with transpose (unit
// stride along N), and their row-major counterparts.  v_mfma_i32_32x32x32_i8 / v_mfma_f32_32x32x16_f16 /
// _bf16 / v_mfma_f32_32x32x64_f8f6f4 want 16 / 16 / 32 consecutive K bytes of one matrix row per lane, so
// such an operand is transposed on its way into LDS; from there on the kernel is the K-contiguous one
// (same fragment layout, same epilogues: gemm_mfma.hpp).
//
//   * WP x WQ waves (2 x 2, or 2 x 4 for the 256 x 256 tile), workgroup tile BP x BQ, 64 K bytes per
//     stage, two LDS stages, one barrier per stage.  Every thread serves both operands, in groups of
//     256 threads: with eight waves the second group takes the upper 128 rows of P and of Q (no
//     control flow depends on the wave, so the loop body stays one block the scheduler can mix).
//     The data cannot go straight to LDS because it has to be transposed, so it is prefetched
//     into registers (two register sets per operand): while the first half of stage kt is
//     multiplied, the registers of stage kt+1 are transposed into the other LDS stage; the barrier
//     sits in the middle of the stage, so that the second half of the MFMAs covers the fragment reads
//     of stage kt+1 and the issue of the loads of stage kt+3.
//   * Operand with unit stride along its row index ("MC"): a lane loads a block of 4 K rows x IW row
//     indices (IW = rows/16 bytes: dword, dwordx2, dwordx4), lanes of a wave run along the row index
//     first so that an instruction reads whole 64..256-byte pieces of 4 K rows; 8 v_perm_b32 per 4 x 4 bytes
//     turn the block into one dword of 4 consecutive K bytes per row, written with ds_write_b32.
//     16-bit elements: 2 K rows x IW row indices per lane (2 IW bytes per K row: dwordx2, dwordx4 or two
//     dwordx4), 2 v_perm_b32 per 2 x 2 elements, one dword of 2 consecutive K elements per row.
//     f32: 1 K row x IW row indices per lane; every loaded dword is already one LDS dword (no permute).
//   * Operand with unit stride along K ("KC"): 16 bytes per lane, ds_write_b128.
//   * LDS rows have a pitch of 80 bytes and are stored in permuted order, rho(i) = 16 r + ((g + s r) mod 16)
//     for i = IW g + r, s = 16 / IW.  With that every ds_write_b32 instruction of the transposing path
//     hits 64 distinct banks (row pitch 20 dwords: 20 x 16 consecutive rows are 16 distinct multiples
//     of 4 mod 64) and every ds_read_b128 of 16 consecutive matrix rows hits 16 distinct 16-byte
//     groups (pitch 5 groups, 5 coprime to 16, rho of 16 consecutive rows distinct mod 16).
#pragma once
#include "gemm_mfma_pipe16.hpp"

namespace zluda_amd {

// LDS row of matrix row i (0 <= i < ROWS) of a tile operand
template <int ROWS>
__device__ __forceinline__ constexpr int tr_rho(int g, int r) {
  constexpr int IW = ROWS / 16, STEP = 16 / IW;
  (void)IW;
  return 16 * r + ((g + STEP * r) & 15);
}
template <int ROWS>
__device__ __forceinline__ int tr_rho_of(int i) {
  constexpr int IW = ROWS / 16;
  return tr_rho<ROWS>(i / IW, i % IW);
}

// 4 x 4 byte transpose: x[j] holds bytes (row 0..3) of K index j; out[r] = K bytes 0..3 of row r
__device__ __forceinline__ void transpose4x4(int x0, int x1, int x2, int x3, int (&out)[4]) {
  // v_perm_b32(s0, s1, sel): result byte n = byte sel[n] of the 8 bytes {s0 (4..7), s1 (0..3)}
  const int t01l = __builtin_amdgcn_perm(x1, x0, 0x05010400);  // x0.b0 x1.b0 x0.b1 x1.b1
  const int t01h = __builtin_amdgcn_perm(x1, x0, 0x07030602);  // x0.b2 x1.b2 x0.b3 x1.b3
  const int t23l = __builtin_amdgcn_perm(x3, x2, 0x05010400);
  const int t23h = __builtin_amdgcn_perm(x3, x2, 0x07030602);
  out[0] = __builtin_amdgcn_perm(t23l, t01l, 0x05040100);
  out[1] = __builtin_amdgcn_perm(t23l, t01l, 0x07060302);
  out[2] = __builtin_amdgcn_perm(t23h, t01h, 0x05040100);
  out[3] = __builtin_amdgcn_perm(t23h, t01h, 0x07060302);
}

// 2 x 2 transpose of 16-bit elements: x[j] holds (row 0, row 1) of K index j; lo = K elements 0..1 of
// row 0, hi = of row 1
__device__ __forceinline__ void transpose2x2(int x0, int x1, int &lo, int &hi) {
  lo = __builtin_amdgcn_perm(x1, x0, 0x05040100);  // x0.h0 x1.h0
  hi = __builtin_amdgcn_perm(x1, x0, 0x07060302);  // x0.h1 x1.h1
}

// Global -> register -> LDS path of ROWS rows of a tile operand, served by 256 threads; KC: unit
// stride along K; ESZ: bytes per element.
template <int ROWS, bool KC, int ESZ = 1>
struct TrOperand {
  static constexpr int IW = ROWS / 16;        // MC: row indices per lane
  static constexpr int KR = 4 / ESZ;          // MC: K rows per lane (one dword of K per LDS row)
  static constexpr int NW = IW * ESZ / 4;     // MC: dwords per K row and lane
  static constexpr int NCH = ROWS / 64;       // KC: 16-byte chunks per lane and stage
  static constexpr int NREG = KC ? NCH * 4 : NW * KR;
  static constexpr int NLOADS = KC ? NCH : KR * (NW > 4 ? NW / 4 : 1);  // vector memory instructions per stage
  static constexpr int NPERM = KC ? 0 : (ESZ == 1 ? NREG * 2 : ESZ == 2 ? NREG : 0);   // v_perm_b32 per stage
  static_assert(ESZ == 1 || ESZ == 2 || ESZ == 4, "8-, 16- or 32-bit elements");
  static_assert(ROWS == 64 || ROWS == 128 || ROWS == 256, "64, 128 or 256 rows per group of 256 threads");

  __amdgpu_buffer_rsrc_t rs;
  int voff[KC ? NCH : 1];
  int kstep;     // byte offset of one stage
  int kbytes;    // bytes of K per row
  int ld;        // MC: stride of one K row
  int tc;        // KC: byte offset of this lane's chunk in a stage

  // base: first byte of the operand (this batch); row0: first tile row; nrows: rows of the whole
  // operand; ld_row / ld_k: byte strides (one of them is ESZ); K: elements along K
  // t: index of the thread among the 256 that load this operand
  __device__ __forceinline__ void init(int t, const uint8_t *base, int row0, int nrows, int ld_row, int ld_k, int K) {
    kbytes = K * ESZ;
    tc = (t & 3) * 16;
    if constexpr (KC) {
      rs = __builtin_amdgcn_make_buffer_rsrc((void *)base, 0, 0x80000000, 0x00020000);
#pragma unroll
      for (int n = 0; n < NCH; n++) voff[n] = min(row0 + (t >> 2) + 64 * n, nrows - 1) * ld_row + (t & 3) * 16;
      kstep = 64;
      ld = 0;
    } else {
      // the operand's extent, up to the end of its last dword (the range check is per dword; base
      // and ld_k are multiples of 4, so that dword lies in the same allocation granule): K rows past
      // the end read as zero
      rs = __builtin_amdgcn_make_buffer_rsrc((void *)base, 0, K > 0 ? (((K - 1) * ld_k + nrows * ESZ + 3) & ~3) : 0, 0x00020000);
      voff[0] = ((t >> 4) * KR) * ld_k + (row0 + (t & 15) * IW) * ESZ;
      kstep = (64 / ESZ) * ld_k;
      ld = ld_k;
    }
  }

  __device__ __forceinline__ void load(int kt, int (&regs)[NREG]) const {
    if constexpr (KC) {
#pragma unroll
      for (int n = 0; n < NCH; n++) {
        const int oob = kt * 64 + tc < kbytes ? 0 : (int)0x80000000;
        const v4i v = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rs, voff[n] | oob, kt * kstep, 0));
        regs[n * 4 + 0] = v[0]; regs[n * 4 + 1] = v[1]; regs[n * 4 + 2] = v[2]; regs[n * 4 + 3] = v[3];
      }
    } else {
#pragma unroll
      for (int j = 0; j < KR; j++) {
        if constexpr (NW == 1) {
          regs[j] = __builtin_amdgcn_raw_buffer_load_b32(rs, voff[0] + j * ld, kt * kstep, 0);
        } else if constexpr (NW == 2) {
          const v2i v = __builtin_bit_cast(v2i, __builtin_amdgcn_raw_buffer_load_b64(rs, voff[0] + j * ld, kt * kstep, 0));
          regs[j * 2] = v[0]; regs[j * 2 + 1] = v[1];
        } else {
#pragma unroll
          for (int h = 0; h < NW / 4; h++) {
            const v4i v = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rs, voff[0] + j * ld + h * 16, kt * kstep, 0));
            regs[j * NW + h * 4] = v[0]; regs[j * NW + h * 4 + 1] = v[1]; regs[j * NW + h * 4 + 2] = v[2]; regs[j * NW + h * 4 + 3] = v[3];
          }
        }
      }
    }
  }

  // `dst`: the operand's rows of one LDS stage (80-byte pitch = 5 v4i)
  __device__ __forceinline__ void store(int t, v4i *dst, const int (&regs)[NREG]) const {
    if constexpr (KC) {
#pragma unroll
      for (int n = 0; n < NCH; n++)
        dst[tr_rho_of<ROWS>((t >> 2) + 64 * n) * 5 + (t & 3)] = v4i{regs[n * 4], regs[n * 4 + 1], regs[n * 4 + 2], regs[n * 4 + 3]};
    } else {
      int *d32 = (int *)dst;
      const int g = t & 15, kb = t >> 4;
#pragma unroll
      for (int c = 0; c < NW; c++) {
        if constexpr (ESZ == 1) {
          int out[4];
          transpose4x4(regs[0 * NW + c], regs[1 * NW + c], regs[2 * NW + c], regs[3 * NW + c], out);
#pragma unroll
          for (int r = 0; r < 4; r++) d32[tr_rho<ROWS>(g, 4 * c + r) * 20 + kb] = out[r];
        } else if constexpr (ESZ == 2) {
          int lo, hi;
          transpose2x2(regs[c], regs[NW + c], lo, hi);
          d32[tr_rho<ROWS>(g, 2 * c) * 20 + kb] = lo;
          d32[tr_rho<ROWS>(g, 2 * c + 1) * 20 + kb] = hi;
        } else {
          d32[tr_rho<ROWS>(g, c) * 20 + kb] = regs[c];
        }
      }
    }
  }
};

// M16 (int8, f16, bf16): the MFMAs are v_mfma_i32_16x16x64_i8 / v_mfma_f32_16x16x32_f16 / _bf16 with P as operand "A" and the epilogues of
// gemm_mfma_pipe16.hpp -- the shape that needs less energy per multiply-add, for problems that keep the whole
// chip busy (see there).  A fragment is then 16 rows x the 64 K bytes of a stage (lane l: row l%16, 16-byte
// chunk l/16), one MFMA per pair of fragments and stage.
template <int KIND, int FQ, int FP, int BP, int BQ, int WP, int WQ, bool PKC, bool QKC, bool M16 = false>
__global__ __launch_bounds__(WP *WQ * 64) void gemm_mfma_tr_kernel(MfmaParams prm) {
  static_assert(KIND == KIND_I8 || KIND == KIND_F8 || kind_is_h16(KIND) || KIND == KIND_F32, "8-, 16- or 32-bit operands");
  constexpr int ESZ = kind_esz(KIND);
  constexpr int MPS = KIND == KIND_F32 ? 4 : 1;  // MFMAs per fragment pair and sub-step
  constexpr bool B16 = KIND != KIND_F8;  // 16 bytes of K per lane and MFMA (fp8: 32)
  static_assert(!M16 || KIND == KIND_I8 || kind_is_h16(KIND), "the 16x16 form is instantiated for int8, f16 and bf16");
  using acc16_v = typename std::conditional<KIND == KIND_I8, v4i, v4f>::type;
  constexpr int NT = WP * WQ * 64;
  static_assert(NT == 256 || NT == 512, "operand rows are dealt to groups of 256 threads");
  constexpr int LP = BP * 256 / NT, LQ = BQ * 256 / NT;  // rows of P / Q one group loads
  constexpr int WTP = BP / WP, WTQ = BQ / WQ, TP = WTP / 32, TQ = WTQ / 32;
  constexpr int KS = KIND == KIND_F8 ? 1 : 2;  // MFMA sub-steps per 64-byte stage
  constexpr int STAGE_V4 = (BP + BQ) * 5;
  using acc_v = typename std::conditional<KIND == KIND_I8, v16i, v16f>::type;
  using frag_v = typename std::conditional<B16, v4i, v8i>::type;

  __shared__ v4i lds[2 * STAGE_V4];

  const GemmArgs &g = prm.g;
  const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wp = wave % WP, wq = wave / WP;
  const int lr = lane & 31, gsel = lane >> 5;
  const int bt = blockIdx.y;

  // workgroup -> tile: as in gemm_mfma_pipe_kernel
  const int total = prm.tiles_p * prm.tiles_q;
  int w = blockIdx.x;
  if ((total & 7) == 0) w = (w & 7) * (total >> 3) + (w >> 3);
  const int group = prm.group_p * prm.tiles_q;
  const int gid = w / group, first_p = gid * prm.group_p;
  const int gsz = min(prm.tiles_p - first_p, prm.group_p);
  const int tile_p = first_p + (w % group) % gsz, tile_q = (w % group) / gsz;
  const int p0 = tile_p * BP, q0 = tile_q * BQ;
  const int NP = prm.swapped ? g.N : g.M, NQ = prm.swapped ? g.M : g.N;

  TrOperand<LP, PKC, ESZ> P;
  TrOperand<LQ, QKC, ESZ> Q;
  const int tl = t & 255, grp = wave >> 2;
  const int lds_p = grp * LP * 5, lds_q = (BP + grp * LQ) * 5;  // this group's rows inside a stage
  // split-K (as in gemm_mfma_pipe_kernel): workgroup z of gridDim.z takes stages [z * split_stages, ...)
  // of K; the operands start k0 further along K and the rest of the kernel sees a shorter K
  // (k0, Kl in elements; a stage is 64 bytes of K)
  int k0 = 0, Kl = g.K;
  if (prm.splits > 1) {
    k0 = (int)blockIdx.z * prm.split_stages * (64 / ESZ);
    Kl = max(0, min(g.K - k0, prm.split_stages * (64 / ESZ)));
  }
  {
    const uint8_t *a = (const uint8_t *)g.A + (g.a_sb * bt + (int64_t)k0 * g.a_sk) * ESZ;
    const uint8_t *b = (const uint8_t *)g.B + (g.b_sb * bt + (int64_t)k0 * g.b_sk) * ESZ;
    if (!prm.swapped) {
      P.init(tl, a, p0 + grp * LP, NP, (int)g.a_si * ESZ, (int)g.a_sk * ESZ, Kl);
      Q.init(tl, b, q0 + grp * LQ, NQ, (int)g.b_sj * ESZ, (int)g.b_sk * ESZ, Kl);
    } else {
      P.init(tl, b, p0 + grp * LP, NP, (int)g.b_sj * ESZ, (int)g.b_sk * ESZ, Kl);
      Q.init(tl, a, q0 + grp * LQ, NQ, (int)g.a_si * ESZ, (int)g.a_sk * ESZ, Kl);
    }
  }
  const int KT = (Kl * ESZ + 63) / 64;
  const int KL = max(KT - 1, 0);  // last stage that holds data
  // K % 64 != 0: in the last stage a load instruction of an operand without unit K stride covers K rows
  // 16 * wave + j + 4 * {0..3}; when even the first of them is past the end every lane of the instruction
  // is out of range.  Such an instruction completes without a memory round trip and may be counted as done
  // ahead of older loads, so a wait that leaves "the younger stage" in flight (what the compiler emits in
  // front of the LDS stores, which consume the older stage's registers) could pass too early.  From the
  // first trip whose younger stage is that last stage (stage kt + 2 >= KL) the stores are therefore preceded
  // by a wait for everything.  With K % 64 == 0 no such instruction exists and nothing is added.
  const int tail_from = tr_tail_from(Kl * ESZ);  // (mfma_wait_counts.hpp, where a host program checks it)

  // LDS rows (in v4i units) of this lane's fragment rows
  int prow[TP], qrow[TQ];
#pragma unroll
  for (int b = 0; b < TP; b++) {
    const int i = wp * WTP + b * 32 + lr;
    prow[b] = (i / LP * LP + tr_rho_of<LP>(i % LP)) * 5;
  }
#pragma unroll
  for (int a = 0; a < TQ; a++) {
    const int i = wq * WTQ + a * 32 + lr;
    qrow[a] = (BP + i / LQ * LQ + tr_rho_of<LQ>(i % LQ)) * 5;
  }

  acc_v acc[M16 ? 1 : TQ][M16 ? 1 : TP];
  if constexpr (!M16) {
#pragma unroll
    for (int a = 0; a < TQ; a++)
#pragma unroll
      for (int b = 0; b < TP; b++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[a][b][v] = 0;
  }
  // ---- the 16x16 form ------------------------------------------------------------------------------
  constexpr int TP16 = WTP / 16, TQ16 = WTQ / 16, HP16 = TP16 / 2;
  acc16_v acc16[M16 ? TP16 : 1][M16 ? TQ16 : 1];
  int prow16[M16 ? TP16 : 1], qrow16[M16 ? TQ16 : 1];  // this lane's 16-byte piece of each fragment (v4i units)
  if constexpr (M16) {
    const int r16 = lane & 15, g4 = lane >> 4;
#pragma unroll
    for (int b = 0; b < TP16; b++) {
      const int i = wp * WTP + b * 16 + r16;
      prow16[b] = (i / LP * LP + tr_rho_of<LP>(i % LP)) * 5 + g4;
    }
#pragma unroll
    for (int a = 0; a < TQ16; a++) {
      const int i = wq * WTQ + a * 16 + r16;
      qrow16[a] = (BP + i / LQ * LQ + tr_rho_of<LQ>(i % LQ)) * 5 + g4;
    }
#pragma unroll
    for (int b = 0; b < TP16; b++)
#pragma unroll
      for (int a = 0; a < TQ16; a++) acc16[b][a] = acc16_v{0, 0, 0, 0};
  }
  // fragment registers: both halves of P (the second is read while the first is multiplied) and the Q
  // fragments of two stages (the next stage's arrive while this stage's are still in use)
  v4i fp16[2][M16 ? HP16 : 1], fq16[2][M16 ? TQ16 : 1];
  auto read_p16 = [&](const v4i *buf, auto h_c) {
    constexpr int h = decltype(h_c)::value;
#pragma unroll
    for (int i = 0; i < HP16; i++) fp16[h][i] = buf[prow16[h * HP16 + i]];
  };
  auto read_q16 = [&](const v4i *buf, auto s_c) {
    constexpr int sidx = decltype(s_c)::value;
#pragma unroll
    for (int a = 0; a < TQ16; a++) fq16[sidx][a] = buf[qrow16[a]];
  };
  auto mfma16 = [&](auto h_c, auto s_c) {
    constexpr int h = decltype(h_c)::value, sidx = decltype(s_c)::value;
#pragma unroll
    for (int i = 0; i < HP16; i++)
#pragma unroll
      for (int a = 0; a < TQ16; a++)
      {
        acc16_v &c = acc16[h * HP16 + i][a];
        if constexpr (KIND == KIND_F16)
          c = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, fp16[h][i]), __builtin_bit_cast(v8h, fq16[sidx][a]), c, 0, 0, 0);
        else if constexpr (KIND == KIND_BF16)
          c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8b, fp16[h][i]), __builtin_bit_cast(v8b, fq16[sidx][a]), c, 0, 0, 0);
        else if constexpr (KIND == KIND_I8)
          c = __builtin_amdgcn_mfma_i32_16x16x64_i8(fp16[h][i], fq16[sidx][a], c, 0, 0, 0);
      }
  };

  // fragments of sub-step ks of the stage in `buf`
  struct Frags { frag_v p[TP], q[TQ]; };
  auto read_frags = [&](const v4i *buf, int ks, Frags &f) {
    if constexpr (B16) {
      const int ch = ks * 2 + gsel;
#pragma unroll
      for (int b = 0; b < TP; b++) f.p[b] = buf[prow[b] + ch];
#pragma unroll
      for (int a = 0; a < TQ; a++) f.q[a] = buf[qrow[a] + ch];
    } else {
      const int c0 = gsel * 2;
#pragma unroll
      for (int b = 0; b < TP; b++) {
        const v4i lo = buf[prow[b] + c0], hi = buf[prow[b] + c0 + 1];
        f.p[b] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
#pragma unroll
      for (int a = 0; a < TQ; a++) {
        const v4i lo = buf[qrow[a] + c0], hi = buf[qrow[a] + c0 + 1];
        f.q[a] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      }
    }
  };
  auto mfma_all = [&](const Frags &f) {
    if constexpr (KIND == KIND_F32) {
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
        else if constexpr (KIND == KIND_F16)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, f.q[a]), __builtin_bit_cast(v8h, f.p[b]),
                                                             acc[a][b], 0, 0, 0);
        else if constexpr (KIND == KIND_BF16)
          acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8b, f.q[a]), __builtin_bit_cast(v8b, f.p[b]),
                                                              acc[a][b], 0, 0, 0);
        else
          acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(f.q[a], f.p[b], acc[a][b], FQ, FP, 0, 0, 0, 0);
      }
    }
  };

  // One stage (kt), entered with: stage kt complete in `cur`, its sub-step-0 fragments in `f0`, stage
  // kt+1 in the register sets `sp` / `sq` (loads issued a trip and a half ago), the loads of stage
  // kt+2 in flight into the other sets.
  //   first half : MFMAs of sub-step 0, and between them the transposition of stage kt+1 into `nxt`
  //                (plus the fragment reads of sub-step 1);
  //   barrier    : `nxt` is complete and nobody reads `cur` any more;
  //   second half: loads of stage kt+3 into the sets just emptied, fragment reads of stage kt+1's
  //                sub-step 0, and the MFMAs of sub-step 1 that cover both.
  // (fp8 stages have a single sub-step: its MFMAs all run in the first half.)
  auto stage_trip = [&](int kt, const v4i *cur, v4i *nxt, int (&sp)[P.NREG], int (&sq)[Q.NREG], Frags &f0) {
    Frags f1;
    // K tail: see tail_from above.  (The branch sits right behind the sched_barrier that ends the previous
    // trip, so it does not cut a scheduling region.)
    if (kt >= tail_from) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if constexpr (KS == 2) read_frags(cur, 1, f1);
    P.store(tl, nxt + lds_p, sp);
    Q.store(tl, nxt + lds_q, sq);
    mfma_all(f0);
    {
      // the fragment reads of sub-step 1 go out with the first MFMAs, the byte permutes follow (an LDS
      // write needs the eight permutes of its 4 x 4 block), the LDS writes come behind the later MFMAs
      constexpr int NM = TP * TQ * MPS, H = NM / 2 > 0 ? NM / 2 : 1;
      constexpr int NDR = KS == 2 ? (TP + TQ) : 0;
      constexpr int NPERM = P.NPERM + Q.NPERM;
      constexpr int NDW = (PKC ? P.NCH : P.NREG) + (QKC ? Q.NCH : Q.NREG);
      static_for<NM>([&](auto i_c) {
        constexpr int i = decltype(i_c)::value;
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if constexpr (i < H) {
          constexpr int nr = NDR * (i + 1) / H - NDR * i / H;
          if constexpr (nr > 0) __builtin_amdgcn_sched_group_barrier(0x100, nr, 0);
          constexpr int nv = NPERM * (i + 1) / H - NPERM * i / H;
          if constexpr (nv > 0) __builtin_amdgcn_sched_group_barrier(0x002, nv, 0);
        } else {
          constexpr int nw = NDW * (i - H + 1) / (NM - H) - NDW * (i - H) / (NM - H);
          if constexpr (nw > 0) __builtin_amdgcn_sched_group_barrier(0x200, nw, 0);
        }
      });
    }
    // (register-only instructions may otherwise drift across the barrier: keep both halves whole)
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    // Past the end the last stage is fetched once more (nothing multiplies it).  Not an out-of-range
    // stage: instructions whose lanes are all out of range complete without a memory round trip and
    // can retire ahead of older loads, while the compiler's vmcnt waits count on in-order return.
    P.load(min(kt + 3, KL), sp);
    Q.load(min(kt + 3, KL), sq);
    read_frags(nxt, 0, f0);
    if constexpr (KS == 2) {
      mfma_all(f1);
      constexpr int NM = TP * TQ * MPS, NDR = TP + TQ;
      constexpr int NVM = P.NLOADS + Q.NLOADS;
      static_for<NM>([&](auto i_c) {
        constexpr int i = decltype(i_c)::value;
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        constexpr int nr = NDR * (i + 1) / NM - NDR * i / NM;
        if constexpr (nr > 0) __builtin_amdgcn_sched_group_barrier(0x100, nr, 0);
        constexpr int nv = NVM * (i + 1) / NM - NVM * i / NM;
        if constexpr (nv > 0) __builtin_amdgcn_sched_group_barrier(0x020, nv, 0);
      });
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  // The same trip on the 16x16 form.  PAR = kt & 1 selects the Q register set.  Entered with P half 0 and the
  // Q fragments of stage kt in registers.
  //   first half : MFMAs of P half 0; P half 1 is read and stage kt+1 transposed into `nxt` between them;
  //   barrier;
  //   second half: MFMAs of P half 1 cover the loads of stage kt+3 and the reads of stage kt+1's P half 0 and Q.
  auto stage_trip16 = [&](int kt, const v4i *cur, v4i *nxt, int (&sp)[P.NREG], int (&sq)[Q.NREG], auto par_c) {
    constexpr int PAR = decltype(par_c)::value;
    using H0 = std::integral_constant<int, 0>;
    using H1 = std::integral_constant<int, 1>;
    using SC = std::integral_constant<int, PAR>;
    using SN = std::integral_constant<int, 1 - PAR>;
    if (kt >= tail_from) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    read_p16(cur, H1{});
    P.store(tl, nxt + lds_p, sp);
    Q.store(tl, nxt + lds_q, sq);
    mfma16(H0{}, SC{});
    {
      constexpr int NM = HP16 * TQ16, H = NM / 2 > 0 ? NM / 2 : 1;
      constexpr int NDR = HP16;
      constexpr int NPERM = P.NPERM + Q.NPERM;
      constexpr int NDW = (PKC ? P.NCH : P.NREG) + (QKC ? Q.NCH : Q.NREG);
      static_for<NM>([&](auto i_c) {
        constexpr int i = decltype(i_c)::value;
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if constexpr (i < H) {
          constexpr int nr = NDR * (i + 1) / H - NDR * i / H;
          if constexpr (nr > 0) __builtin_amdgcn_sched_group_barrier(0x100, nr, 0);
          constexpr int nv = NPERM * (i + 1) / H - NPERM * i / H;
          if constexpr (nv > 0) __builtin_amdgcn_sched_group_barrier(0x002, nv, 0);
        } else {
          constexpr int nw = NDW * (i - H + 1) / (NM - H) - NDW * (i - H) / (NM - H);
          if constexpr (nw > 0) __builtin_amdgcn_sched_group_barrier(0x200, nw, 0);
        }
      });
    }
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    P.load(min(kt + 3, KL), sp);
    Q.load(min(kt + 3, KL), sq);
    read_p16(nxt, H0{});
    read_q16(nxt, SN{});
    mfma16(H1{}, SC{});
    {
      constexpr int NM = HP16 * TQ16, NDR = HP16 + TQ16;
      constexpr int NVM = P.NLOADS + Q.NLOADS;
      static_for<NM>([&](auto i_c) {
        constexpr int i = decltype(i_c)::value;
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        constexpr int nr = NDR * (i + 1) / NM - NDR * i / NM;
        if constexpr (nr > 0) __builtin_amdgcn_sched_group_barrier(0x100, nr, 0);
        constexpr int nv = NVM * (i + 1) / NM - NVM * i / NM;
        if constexpr (nv > 0) __builtin_amdgcn_sched_group_barrier(0x020, nv, 0);
      });
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  // two register sets per operand: stage s travels through set s & 1
  int rp0[P.NREG], rp1[P.NREG], rq0[Q.NREG], rq1[Q.NREG];
  v4i *buf0 = &lds[0], *buf1 = &lds[STAGE_V4];
  Frags f0;
  P.load(0, rp0); Q.load(0, rq0);
  P.load(min(1, KL), rp1); Q.load(min(1, KL), rq1);
  if (tail_from < 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // stage 1 is already the K tail
  P.store(tl, buf0 + lds_p, rp0);
  Q.store(tl, buf0 + lds_q, rq0);
  __syncthreads();
  P.load(min(2, KL), rp0); Q.load(min(2, KL), rq0);
  if constexpr (M16) {
    read_p16(buf0, std::integral_constant<int, 0>{});
    read_q16(buf0, std::integral_constant<int, 0>{});
    for (int kt = 0; kt < KT; kt += 2) {
      stage_trip16(kt, buf0, buf1, rp1, rq1, std::integral_constant<int, 0>{});
      if (kt + 1 < KT) stage_trip16(kt + 1, buf1, buf0, rp0, rq0, std::integral_constant<int, 1>{});
    }
  } else {
    read_frags(buf0, 0, f0);
    for (int kt = 0; kt < KT; kt += 2) {
      stage_trip(kt, buf0, buf1, rp1, rq1, f0);
      if (kt + 1 < KT) stage_trip(kt + 1, buf1, buf0, rp0, rq0, f0);
    }
  }

  // every wave is done with the LDS stages before they become epilogue staging
  __syncthreads();
  if constexpr (M16) {
    if (prm.splits > 1) {
      const int ws_np = prm.tiles_p * BP, ws_nq = prm.tiles_q * BQ;
      int32_t *ws_tile = (int32_t *)prm.ws + ((int64_t)blockIdx.z * g.batch + bt) * ws_np * ws_nq + (int64_t)(q0 + wq * WTQ) * ws_np + p0 + wp * WTP;
      const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)ws_tile, 0, 0xFFFFFFFF, 0x00020000);
      mfma16_store_raw<TP16, TQ16>(rs, ws_np, acc16, 1);
      return;
    }
    mfma16_store_tile<KIND, WP, WQ, TP16, TQ16, (int)sizeof(lds)>(prm, acc16, (int *)&lds[0], p0, q0, NP, NQ, bt);
  } else {
  if (prm.splits > 1) {
    const int ws_np = prm.tiles_p * BP, ws_nq = prm.tiles_q * BQ;
    int32_t *ws_tile = (int32_t *)prm.ws + ((int64_t)blockIdx.z * g.batch + bt) * ws_np * ws_nq + (int64_t)q0 * ws_np + p0;
    mfma_store_tile_raw<WP, WQ, WTP, WTQ>(ws_tile, ws_np, acc);
    return;
  }
  mfma_store_tile<KIND, WP, WQ, WTP, WTQ>(prm, acc, (int *)&lds[0], sizeof(lds), p0, q0, NP, NQ, bt);
  }
}

} // namespace zluda_amd
