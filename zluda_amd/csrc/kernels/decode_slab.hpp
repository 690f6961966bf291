// Skinny (<= 16 tokens) W8A8 decode GEMM, slab form of the LDS-streaming kernel (decode_stream.hpp) for
// 2048 < K <= 16384: the same math and epilogue, a different road for the bytes.
//
//   W : R rows x K int8 (or fp8 e4m3), K-contiguous (read exactly once)     X : T <= 16 rows x K, same type
//   out(r, t) = sum_k W[r][k] * X[t][k]     int32 (fp32), then the fused float / integer epilogue
// The same kernel streams f16 / bf16 weights (KIND_F16 / KIND_BF16: v_mfma_f32_16x16x32_f16 / _bf16 take 16 bytes
// of K per lane at the byte positions of the int8 instruction, so only the MFMA and the accumulator type
// differ; every K below is then a count of BYTES, twice the element count).
//
// What differs from decode_stream_kernel, and what each point bought on a 14336 x 4096 int8 matrix with 16
// tokens (MI355X, 58.7 MB, a flat read of the same bytes takes 9.95 us; decode_stream_kernel 14.8 us):
//   * One DMA instruction fetches ONE row x 1 KiB (64 lanes x 16 contiguous bytes) instead of 4 rows x 256
//     bytes, a 16-row block of a wave's K slab is 16 instructions into a 16 KiB slot, two slots per wave.
//     A workgroup is 4 waves, wave v owning K bytes [v*kw, (v+1)*kw) with kw <= 1024.  (Beyond K = 4096: 8 waves,
//     two rows x 512 bytes per instruction, a slab of up to four such units per block; see the template.)
//   * The activations take the same road once (one token x 1 KiB per instruction into the second slot, whole
//     cache lines) and are copied to registers before that slot joins the weight ring; loading them in the
//     MFMA layout straight from global memory asks for 64-byte pieces and costs ~1 us more.
//   * A workgroup runs at most 4 blocks, keeps their accumulators in registers and meets the other waves
//     ONCE, at the end: one barrier and one LDS round trip per workgroup instead of one per block.
//   * Blocks are dealt out round-robin (block b of workgroup w = rows 16 * (b*G + w)), so that at any moment
//     the grid reads one contiguous stripe of W; the rows left over after the last full round of G blocks are
//     split evenly in quads of 4.  ~0.4 us against contiguous row ranges per workgroup.
//   * The epilogue factors are fetched without a branch (a null vector reads a dummy address and is replaced
//     by its scalar afterwards; a bias is read once as 16 and once as 32 bits).  With the usual
//     "pointer ? load : scalar" and per-type bias loads the same kernel measures ~0.55 us slower, wherever
//     in the kernel those loads are issued.
// Together: 12.2-12.5 us.
//
// LDS slot layout: row rho (0..15) x 64 chunks of 16 bytes; chunk c of row rho sits at position
// (c & 48) | ((c ^ rho) & 15) of the row's KiB: the DMA of a row lands linearly (lane l fetches the chunk whose
// position is l) and the 16-rows-same-chunk fragment reads hit 16 different bank groups.
#pragma once
#include "decode_slab_addr.hpp"
#include "decode_stream.hpp"

namespace zluda_amd {

constexpr int kSlabMaxBlocks = 4;   // 16-row blocks a workgroup can run

// FAST != 0 as in decode_stream_kernel: every output leaves through the packed 8-byte store (1: no activation or
// ReLU, 2: GELU; whatever code sits between the last weights and the store is exposed in full, so the path of
// the plain epilogue is kept free of branches).  TAIL: K is shorter than the NW * Q * UB bytes the instantiation
// covers (lanes past a wave's slab or past K fetch nothing and read as zero).
//
// Two shapes of the same kernel:
//   NW = 4, UB = 1024, Q = 1   K <= 4096: a wave's slab of a block is one unit of 16 rows x 1 KiB (one row per
//                              DMA instruction); the activations pass through the second slot while the first
//                              block is already on its way.
//   NW = 8, UB = 512, Q = 2..4 K <= 16384: a slab is Q units of 16 rows x 512 bytes (two rows per instruction,
//                              still four whole cache lines per row); the activations pass through both slots,
//                              two units at a time, BEFORE the weights start: loading them in the MFMA layout
//                              from global memory instead asks for 64-byte pieces of 16 * K bytes per workgroup,
//                              which at K = 13824 and 20 rows per workgroup is 44 % of all it reads.
//   NW = 8, UB = 512, Q = 1..2, NB = 2   17..32 tokens, K <= 8192: a second block of 16 tokens doubles the
//                              activation fragments and the accumulators; the 8 (block, token block) tiles of
//                              the final reduction go one to each wave.
constexpr int kSlabFactorLoads = 21;  // vector memory loads of the packed epilogue's factors, per lane
template <int FAST, int KIND, bool TAIL, int NW = 4, int UB = 1024, int Q = 1, int NB = 1>
__global__ __launch_bounds__(NW * 64) void decode_slab_kernel(DecodeParams prm) {
  static_assert(KIND == KIND_I8 || KIND == KIND_F8 || kind_is_h16(KIND), "int8, fp8 (e4m3 x e4m3), f16 or bf16 operands");
  constexpr int ESZ = kind_is_h16(KIND) ? 2 : 1;           // bytes per element
  constexpr bool B16 = KIND != KIND_F8;                    // 16 bytes of K per lane and MFMA (fp8: 32)
  static_assert((UB == 1024 || UB == 512) && Q >= 1 && Q * NB <= 4 && (Q * NB == 1 || TAIL), "see above; the shapes beyond the first come with the K checks");
  using acc_t = typename std::conditional<KIND == KIND_I8, v4i, v4f>::type;
  constexpr int MAXB = kSlabMaxBlocks;
  constexpr int NDMA = 16 * UB / 1024;  // DMA instructions per unit
  constexpr int RPI = 1024 / UB;        // rows per instruction
  constexpr int CPR = UB / 16;          // 16-byte chunks per row of a unit
  constexpr int NFRAG = UB / 64;        // 16-byte fragments per lane and unit
  constexpr int UNIT_V4 = 16 * CPR;
  static_assert(MAXB * NB <= NW, "one wave per (block, token block) runs the epilogue");
  static_assert(MAXB * NB * 64 <= 2 * UNIT_V4, "a wave's partial tiles fit into its own ring");
  __shared__ v4i ring[NW][2][UNIT_V4];

  const GemmArgs &g = prm.g;
  const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int l16 = lane & 15, g4 = lane >> 4;
  const int bt = blockIdx.y;

  const int R = prm.swapped ? g.N : g.M, T = prm.swapped ? g.M : g.N;
  const uint8_t *Wg = (const uint8_t *)(prm.swapped ? g.B : g.A) + (prm.swapped ? g.b_sb : g.a_sb) * bt * ESZ;
  const uint8_t *Xg = (const uint8_t *)(prm.swapped ? g.A : g.B) + (prm.swapped ? g.a_sb : g.b_sb) * bt * ESZ;
  const int ldw = (int)(prm.swapped ? g.b_sj : g.a_si) * ESZ;  // row pitches and K in bytes
  const int ldx = (int)(prm.swapped ? g.a_si : g.b_sj) * ESZ;
  const int K = g.K * ESZ;

  // Blocks of this workgroup: full_rounds round-robin blocks, then its share [rr0, rr1) (at most 16 rows, a
  // whole number of quads except at the very end of W) of the rows behind the last full round.  The split is
  // done on the host.
  const int G = (int)gridDim.x, wg = (int)blockIdx.x, F = prm.full_rounds;
  const int rr0 = 16 * F * G + 4 * (wg * prm.rows_base + min(wg, prm.rows_rem));
  const int rr1 = min(R, rr0 + 4 * (prm.rows_base + (wg < prm.rows_rem ? 1 : 0)));
  const int nblk = F + (rr1 > rr0 ? 1 : 0);  // <= MAXB (host)
  if (nblk == 0) return;                      // (the whole workgroup)
  auto row_base = [&](int b) { return b < F ? 16 * (b * G + wg) : rr0; };
  auto row_end = [&](int b) { return b < F ? 16 * (b * G + wg) + 16 : rr1; };

  // 2 GiB raw buffer windows; bit 31 of an offset puts a lane out of range: it fetches nothing and its 16
  // bytes of LDS read as zero
  const __amdgpu_buffer_rsrc_t rsW = __builtin_amdgcn_make_buffer_rsrc((void *)Wg, 0, 0x80000000, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsX = __builtin_amdgcn_make_buffer_rsrc((void *)Xg, 0, 0x80000000, 0x00020000);
  const int kw = prm.spw * 64;          // bytes of K per wave (a multiple of 128, at most Q * UB)
  const int kwave = wave * kw;
  // DMA instruction i of a unit fills rows RPI * i .. of the slot linearly: the lane at position p of row rho
  // fetches the chunk whose position is p, i.e. chunk (p & ~15) | ((p ^ rho) & 15) of the row's UB bytes.
  // (UB = 512: the upper half of the wave takes the odd row; its row pitch goes into the vector offset.)
  const int half = RPI == 2 ? lane >> 5 : 0;
  int dma_off[NDMA];
#pragma unroll
  for (int i = 0; i < NDMA; i++) dma_off[i] = slab_dma_offset(UB, lane, i);
  // vector offset of instruction i in unit q of the wave's slab, `pitch` = what the odd row adds.  A unit that holds
  // no byte of K (decode_slab_addr.hpp) is fetched as real loads and its MFMAs are skipped: no instruction the kernel
  // issues has all of its lanes out of range, which the counted waits below depend on.
  auto unit_voff = [&](int i, int q, int pitch) { return slab_unit_voff(TAIL, UB, lane, dma_off[i], q, kw, kwave, K, pitch); };
  auto unit_empty = [&](int q) { return slab_unit_empty(TAIL, UB, q, kw, kwave, K); };  // (wave-uniform)
  auto issue_w = [&](int b, int q, int slot) {
    const int rb = row_base(b), re = row_end(b);
    v4i *dst = &ring[wave][slot][0];
#pragma unroll
    for (int i = 0; i < NDMA; i++) {
      // (rows past the end of a short block repeat its last row: in range, a cache hit, never used; the row
      // goes into the scalar offset, which leaves one scalar multiply per instruction and no vector work)
      const int row = min(rb + RPI * i, re - 1);
      lds_dma16<kWeightStreamAux>(rsW, dst + i * 64, unit_voff(i, q, RPI == 2 && half && row + 1 < re ? ldw : 0), row * ldw);
    }
  };
  // (token 16 * nbk + rho, rho = row of the unit; tokens past T repeat the last one and are never stored)
  auto issue_x = [&](int nbk, int q, int slot) {
    v4i *dst = &ring[wave][slot][0];
#pragma unroll
    for (int i = 0; i < NDMA; i++) {
      const int tok = min(16 * nbk + RPI * i, T - 1);
      lds_dma16(rsX, dst + i * 64, unit_voff(i, q, RPI == 2 && half && tok + 1 < T ? ldx : 0), tok * ldx);
    }
  };
  // fragment f of this lane in a unit: int8, f16, bf16: K step f, 16 bytes at f*64 + g4*16; fp8: half (f & 1) of
  // the 32 bytes at (f/2)*128 + g4*32 of K step f/2
  const uint32_t ring_base = lds_addr(&ring[wave][0][l16 * CPR]);
  auto frag_addr = [&](int slot, int f) {
    const int c = B16 ? 4 * f + g4 : 8 * (f >> 1) + 2 * g4 + (f & 1);
    return ring_base + slot * (UNIT_V4 * 16) + (((c & ~15) | ((c ^ l16) & 15)) << 4);
  };
  // unit n of this wave = (block n / Q, unit n % Q of the slab), in slot n % 2; the wave runs nblk * Q of them
  auto issue_unit = [&](int n, int slot) { issue_w(n / Q, n % Q, slot); };

  v4i xf[NB * Q][NFRAG];  // [token block * Q + unit]
  if constexpr (NB * Q == 1) {
    // Activations into slot 1, the first weights behind them, and as soon as the activations are in registers
    // the second block: nothing that needs more of the kernel arguments than pointers and sizes stands in
    // front of the stream.
    issue_x(0, 0, 1);
    issue_unit(0, 0);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NDMA) : "memory");  // all but the youngest unit: the activations
#pragma unroll
    for (int f = 0; f < NFRAG; f++) xf[0][f] = lds_read16_unordered(frag_addr(1, f));
    lds_values_ready(xf[0]);
  } else {
    // the activations of the whole slab (of every token block), two units at a time through the two slots, then
    // the first weights
#pragma unroll
    for (int c = 0; c < NB * Q; c += 2) {
      issue_x(c / Q, c % Q, 0);
      if (c + 1 < NB * Q) issue_x((c + 1) / Q, (c + 1) % Q, 1);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
      for (int f = 0; f < NFRAG; f++) xf[c][f] = lds_read16_unordered(frag_addr(0, f));
      if (c + 1 < NB * Q) {
#pragma unroll
        for (int f = 0; f < NFRAG; f++) xf[c + 1][f] = lds_read16_unordered(frag_addr(1, f));
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
#pragma unroll
    for (int c = 0; c < NB * Q; c++) lds_values_ready(xf[c]);
    issue_unit(0, 0);
  }
  // Activation fragments of a unit that holds no byte of K: zero, so that the 16 stray bytes per instruction that the
  // unit's weight loads bring multiply to nothing without a branch around the MFMAs.
  // int8: exact.  e4m3 has no infinity, and a NaN among the stray weights is one the row's own product holds too.
  if constexpr (TAIL && !kind_is_h16(KIND)) {
#pragma unroll
    for (int c = 0; c < NB * Q; c++) {
      if (unit_empty(c % Q)) {
#pragma unroll
        for (int f = 0; f < NFRAG; f++) xf[c][f] = v4i{0, 0, 0, 0};
      }
    }
  }
  // (the second unit is issued even when there is none -- then it fetches the first one again, never used -- so
  // that the number of operations in flight is the same on every path)
  issue_unit(nblk * Q > 1 ? 1 : 0, 1);

  // Who runs the epilogue: wave w takes block w % MAXB of token block w / MAXB, lane l the 4 rows (l/16)*4.. of
  // token l%16 of that block, i.e. exactly the accumulator registers lane l holds.
  const int pblk = wave % MAXB, pnb = wave / MAXB;
  const bool has_pair = pblk < nblk && pnb < NB;
  const int ptok = 16 * pnb + l16;
  const int prow0 = row_base(has_pair ? pblk : 0) + g4 * 4, pend = row_end(has_pair ? pblk : 0);
  // Factor loads of the packed epilogue: every factor that lives in device memory -- alpha (scalar or vector),
  // the operand scales (scalar or per row / token), the bias (16 or 32 bits), the scale of D -- is read per
  // lane here, behind the second unit, and nothing waits for it before the last unit does.  Exactly
  // kSlabFactorLoads loads per lane, whatever the problem: a factor that is an immediate or absent reads a
  // dummy address instead, and the index passes through an empty asm so that equal addresses are not merged.
  // The wait for the first unit counts them.
  float f_al[4], f_sa[4], f_sb[4], f_sd = 1.0f;
  uint32_t f_b16[4], f_b32[4];
  const bool al_mem = g.alpha_mode != SCALAR_VALUE, al_vec = g.alpha_mode == VECTOR_DEV;
  const bool sa_mem = g.a_scale_mode == SCALE_SCALAR || g.a_scale_mode == SCALE_OUTER_VEC, sa_vec = g.a_scale_mode == SCALE_OUTER_VEC;
  const bool sb_mem = g.b_scale_mode == SCALE_SCALAR || g.b_scale_mode == SCALE_OUTER_VEC, sb_vec = g.b_scale_mode == SCALE_OUTER_VEC;
  const bool bias16 = g.bias && g.bias_type != CUDA_R_32F, bias32 = g.bias && g.bias_type == CUDA_R_32F;
  const bool counted = FAST && has_pair;
  if (counted) {
    const float *dummy = (const float *)Wg;  // (16-byte aligned, at least 64 rows long)
    const float *al_p = al_mem ? (const float *)g.alpha_ptr + (al_vec ? g.alpha_sb * bt : 0) : dummy;
    const float *sa_p = sa_mem ? (const float *)g.a_scale : dummy, *sb_p = sb_mem ? (const float *)g.b_scale : dummy;
    const uint16_t *b16_p = bias16 ? (const uint16_t *)g.bias + g.bias_sb * bt : (const uint16_t *)dummy;
    const uint32_t *b32_p = bias32 ? (const uint32_t *)g.bias + g.bias_sb * bt : (const uint32_t *)dummy;
#pragma unroll
    for (int v = 0; v < 4; v++) {
      const int row = min(prow0 + v, pend - 1), tok = min(ptok, T - 1);
      int i = prm.swapped ? tok : row, j = prm.swapped ? row : tok;
      asm volatile("" : "+v"(i), "+v"(j));
      f_al[v] = al_p[al_vec ? i : 0];
      f_sa[v] = sa_p[sa_vec ? i : 0];
      f_sb[v] = sb_p[sb_vec ? j : 0];
      f_b16[v] = b16_p[bias16 ? i : 0];
      f_b32[v] = b32_p[bias32 ? i : 0];
    }
    f_sd = *(g.d_scale ? (const float *)g.d_scale : dummy);
    static_assert(kSlabFactorLoads == 4 * 5 + 1, "five loads per output row and the scale of D");
  }
  asm volatile("" ::: "memory");
  // (what the packed store needs of the kernel arguments, read here rather than behind the last weights)
  const bool relu = g.act == ACT_RELU, out_bf16 = g.d_type == CUDA_R_16BF;
  uint16_t *const Dq = (uint16_t *)g.D + g.d_sb * bt + (int64_t)ptok * (prm.swapped ? g.d_si : g.d_sj) + prow0;

  acc_t acc[MAXB][NB];
#pragma unroll
  for (int b = 0; b < MAXB; b++)
#pragma unroll
    for (int nbk = 0; nbk < NB; nbk++) acc[b][nbk] = acc_t{0, 0, 0, 0};
#pragma unroll
  for (int b = 0; b < MAXB; b++) {
    if (b < nblk) {
#pragma unroll
      for (int q = 0; q < Q; q++) {
        const int n = b * Q + q;  // (a compile-time number: both loops are unrolled)
        // Unit n has landed when at most the next one is in flight -- and, for the first unit, the factor loads
        // issued behind the second.  The last unit waits for everything, those loads included (they are as old
        // as the second unit): they are folded into one scale and one bias per row here, where the compiler's
        // own wait for them (vmcnt(0), all it can prove) costs nothing.
        if (q == Q - 1 && b + 1 == nblk) {
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
          if (counted) {
#pragma unroll
            for (int v = 0; v < 4; v++) {
              const float al = al_mem ? f_al[v] : g.alpha_val.f, sa = sa_mem ? f_sa[v] : 1.0f, sb = sb_mem ? f_sb[v] : 1.0f;
              const float b16 = g.bias_type == CUDA_R_16F ? dec_f16((uint16_t)f_b16[v]) : dec_bf16((uint16_t)f_b16[v]);
              f_al[v] = (al * sa) * sb;
              f_sa[v] = bias32 ? bits2f(f_b32[v]) : bias16 ? b16 : 0.0f;
            }
            f_sd = g.d_scale ? f_sd : 1.0f;
          }
        } else if (n == 0 && counted) {
          asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NDMA + kSlabFactorLoads) : "memory");
        } else {
          asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NDMA) : "memory");
        }
        v4i w[NFRAG];
#pragma unroll
        for (int f = 0; f < NFRAG; f++) w[f] = lds_read16_unordered(frag_addr(n & 1, f));
        lds_values_ready(w);  // in registers before the slot is refilled
        if ((n + 2) / Q < nblk) issue_unit(n + 2, n & 1);
        // (a unit that holds no byte of K was fetched for the count only: for 8-bit operands its activation fragments
        // are zero -- see above --, 16-bit ones, whose stray weights may be infinite, skip its MFMAs)
        if constexpr (kind_is_h16(KIND)) {
          if (unit_empty(q)) continue;
        }
#pragma unroll
        for (int nbk = 0; nbk < NB; nbk++) {
          if constexpr (KIND == KIND_I8) {
#pragma unroll
            for (int f = 0; f < NFRAG; f++)
              acc[b][nbk] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[f], xf[nbk * Q + q][f], acc[b][nbk], 0, 0, 0);
          } else if constexpr (KIND == KIND_F16) {
#pragma unroll
            for (int f = 0; f < NFRAG; f++)
              acc[b][nbk] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, w[f]), __builtin_bit_cast(v8h, xf[nbk * Q + q][f]),
                                                                   acc[b][nbk], 0, 0, 0);
          } else if constexpr (KIND == KIND_BF16) {
#pragma unroll
            for (int f = 0; f < NFRAG; f++)
              acc[b][nbk] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8b, w[f]), __builtin_bit_cast(v8b, xf[nbk * Q + q][f]),
                                                                    acc[b][nbk], 0, 0, 0);
          } else {
#pragma unroll
            for (int f = 0; f < NFRAG; f += 2) {
              const v4i x0 = xf[nbk * Q + q][f], x1 = xf[nbk * Q + q][f + 1];
              const v8i wa = {w[f][0], w[f][1], w[f][2], w[f][3], w[f + 1][0], w[f + 1][1], w[f + 1][2], w[f + 1][3]};
              const v8i xb = {x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
              acc[b][nbk] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wa, xb, acc[b][nbk], 0, 0, 0, 0, 0, 0);
            }
          }
        }
      }
    }
  }

  // The one meeting of the workgroup's waves: wave w sums the NW partial tiles of its (block, token block).  A
  // wave parks its tiles at the start of its own ring (everything it fetched has been consumed), tile
  // (b, nbk) at index nbk * MAXB + b, i.e. at the index of the wave that finishes it.
#pragma unroll
  for (int b = 0; b < MAXB; b++)
#pragma unroll
    for (int nbk = 0; nbk < NB; nbk++) ring[wave][0][(nbk * MAXB + b) * 64 + lane] = __builtin_bit_cast(v4i, acc[b][nbk]);
  lds_barrier();
  if (!has_pair) return;
  v4i part[NW];
  const uint32_t red_base = lds_addr(&ring[0][0][wave * 64 + lane]);
#pragma unroll
  for (int w2 = 0; w2 < NW; w2++) part[w2] = lds_read16_unordered(red_base + w2 * (2 * UNIT_V4 * 16));
  lds_values_ready(part);
  acc_t s = __builtin_bit_cast(acc_t, part[0]);
#pragma unroll
  for (int w2 = 1; w2 < NW; w2++) s += __builtin_bit_cast(acc_t, part[w2]);

  if constexpr (FAST != 0) {
    if (ptok < T && prow0 < pend) {  // the row count is a multiple of 4: a quad is inside or outside
      float y[4];
#pragma unroll
      for (int v = 0; v < 4; v++) {
        float x = f_al[v] * (float)s[v] + f_sa[v];  // (scale and bias of the row, folded above)
        if constexpr (FAST == 2) x = gelu_tanh(x);
        else x = relu ? (x > 0.0f ? x : 0.0f) : x;
        y[v] = x * f_sd;
      }
      uint2 pk;
      if (out_bf16) {
        pk.x = pack_bf16x2(y[0], y[1]);
        pk.y = pack_bf16x2(y[2], y[3]);
      } else {
        pk.x = pack_f16x2(y[0], y[1]);
        pk.y = pack_f16x2(y[2], y[3]);
      }
      *(uint2 *)Dq = pk;
    }
  } else {
    const Epilogue ep(g, bt);  // (reads its device scalars on the spot: nothing is in flight any more)
#pragma unroll
    for (int v = 0; v < 4; v++) {
      const int row = prow0 + v;
      if (row < pend && ptok < T) {
        const int i = prm.swapped ? ptok : row, j = prm.swapped ? row : ptok;
        if (KIND == KIND_I8 && g.int_scale) ep.store_int(i, j, (int)s[v]);
        else ep.store_f(i, j, (float)s[v]);
      }
    }
  }
}

} // namespace zluda_amd
