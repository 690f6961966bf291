// Skinny (<= 64 tokens) W8A8 decode GEMM, streaming form: the weights go from HBM straight into LDS
// in whole cache lines and are re-read from LDS in the MFMA operand layout.
//
//   W : R rows x K int8 (or fp8 e4m3), K-contiguous (read exactly once)     X : T <= 64 rows x K, same type
//   out(r, t) = sum_k W[r][k] * X[t][k]     int32 (fp32), then the fused float / integer epilogue
//
// KIND_I8 uses v_mfma_i32_16x16x64_i8 (lane l: row l%16, 16 K-bytes at (l/16)*16 of a 64-byte step),
// KIND_F8 v_mfma_f32_16x16x128_f8f6f4 (lane l: row l%16, 32 K-bytes at (l/16)*32 of a 128-byte step):
// the same four 16-byte LDS reads per lane and 256-byte unit, at different chunk positions.
//
// Why LDS: v_mfma_i32_16x16x64_i8 wants lane l to hold 16 K-bytes of row l%16, so a 128-bit global
// load in that layout touches 16 rows x 64 bytes: half a cache line per row.  Measured on MI355X,
// reading the 58.7 MB of a 14336 x 4096 weight matrix with that pattern takes 15 us against 10 us
// for a flat read.  Here one buffer_load_dwordx4 ... lds instruction copies 4 rows x 256 contiguous
// bytes, occupies no VGPRs while in flight, and the ds_read_b128 that follows is free to use any
// layout.
//
// K: an instantiation covers NW * SPW * 64 bytes of K; any shorter K (a multiple of 16) runs on it with the
// lanes past the end reading zero, so the host takes the smallest instantiation that covers K.
//
// Work split: workgroup w owns the contiguous rows [w*R/G, (w+1)*R/G) (balanced to one row across
// the grid, whatever R is) and walks them in blocks of 16.  K is split across the NW waves of the
// workgroup: wave v streams bytes [v*SPW*64, (v+1)*SPW*64) of every row and keeps the matching
// activation fragments in registers for the whole kernel.  A wave's data path is private: it fills
// its own LDS ring (2 slots of 16 rows x 256 bytes) and only it reads them back, so the only
// workgroup barrier is the one in front of the cross-wave reduction of a finished 16-row block.
// A block has 64 x NB (token, quad of rows) pairs; whoever owns a pair sums its NW partial values,
// applies the epilogue and writes the quad with one store: one rotating wave for up to 32 tokens,
// all waves (one pair per lane) beyond that.
// A slot is refilled as soon as its fragments are in registers, so every wave always has 4-8 KiB in
// flight (64-128 KiB per CU with 16 resident waves).
//
// LDS slot layout: row rho (0..15) x 16 chunks of 16 bytes; logical chunk c of row rho sits at
// position c ^ rho, which makes both the linear 1 KiB LDS fill of one DMA instruction and the
// 16-rows-same-chunk fragment reads bank-conflict free.
#pragma once
#include "decode_w8a8.hpp"

namespace zluda_amd {

// Workgroup barrier that orders LDS traffic only: __syncthreads() would also wait for every vector
// memory operation of the wave, i.e. drain the weight stream at each block.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// 32-bit LDS address of a __shared__ object (the address-space cast only exists in the device pass)
// Cache policy of the weight loads: the weights of a decode GEMM are read exactly once, and marked non-temporal (the nt
// bit) they stream 6 % faster -- 14336 x 4096 int8 in 11.65 us instead of 12.4; a flat read of the same bytes gains 5 %
// from the same hint.  (The activations, which every workgroup reads again, keep the default policy; on the L2-resident
// panels of the large GEMMs the hint is far slower.)
constexpr int kWeightStreamAux = 2;

__device__ __forceinline__ uint32_t lds_addr(const void *p) {
#if defined(__HIP_DEVICE_COMPILE__)
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)p;
#else
  (void)p;
  return 0;
#endif
}

// ds_read_b128 issued behind the compiler's back.  A C++ read of LDS that the compiler cannot prove
// disjoint from an LDS DMA still in flight gets an s_waitcnt vmcnt(0) in front of it; in a loop that
// is every read, which would serialise the weight stream.  The caller orders these reads itself
// (frags_ready below).
__device__ __forceinline__ v4i lds_read16_unordered(uint32_t addr) {
  v4i r;
  asm volatile("ds_read_b128 %0, %1" : "=v"(r) : "v"(addr));
  return r;
}
// Waits for the unordered reads and ties the four fragments to the wait, so that nothing that uses
// them can be scheduled in front of it.  The memory clobber keeps the refill of the slot behind it.
__device__ __forceinline__ void frags_ready(v4i &a, v4i &b, v4i &c, v4i &d) {
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d)::"memory");
}

// frags_ready for an array of values read with lds_read16_unordered
template <int N>
__device__ __forceinline__ void lds_values_ready(v4i (&x)[N]) {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
  for (int i = 0; i < N; i++) asm volatile("" : "+v"(x[i]));
}

// FAST: the host has checked that every output leaves through the packed 8-byte store below (float
// epilogue without C, 16-bit D contiguous along the weight rows, 8-byte aligned, row count a multiple
// of 4); the element-wise epilogue with all its type dispatch is then not even compiled in, which
// keeps the code the reducing wave runs between two blocks short.
// TAIL: K is shorter than the NW * SPW * 64 bytes the instantiation covers (the checks cost ~3 % on an exact K,
// so that case has its own instantiation without them).
template <int NW, int SPW, int NB, bool FAST, int KIND = KIND_I8, bool TAIL = false>
__global__ __launch_bounds__(NW * 64) void decode_stream_kernel(DecodeParams prm) {
  static_assert(KIND == KIND_I8 || KIND == KIND_F8, "int8 or fp8 (e4m3 x e4m3) operands");
  using acc_t = typename std::conditional<KIND == KIND_I8, v4i, v4f>::type;
  constexpr int SEG = 256;             // bytes of one row per unit
  constexpr int Q = SPW * 64 / SEG;    // units per 16-row block (and wave)
  constexpr int NSLOT = 2;
  constexpr int UNIT_V4 = 16 * SEG / 16;
  constexpr int NDMA = 16 * SEG / 1024;  // DMA instructions per unit
  static_assert(SPW % 4 == 0, "a wave's K slice is a whole number of 256-byte units");
  __shared__ v4i ring[NW][NSLOT][UNIT_V4];
  __shared__ v4i red[2][NW][NB][64];

  const GemmArgs &g = prm.g;
  const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int l16 = lane & 15, g4 = lane >> 4;
  const int bt = blockIdx.y;

  const int R = prm.swapped ? g.N : g.M, T = prm.swapped ? g.M : g.N;
  const uint8_t *Wg = (const uint8_t *)(prm.swapped ? g.B : g.A) + (prm.swapped ? g.b_sb : g.a_sb) * bt;
  const uint8_t *Xg = (const uint8_t *)(prm.swapped ? g.A : g.B) + (prm.swapped ? g.a_sb : g.b_sb) * bt;
  const int ldw = (int)(prm.swapped ? g.b_sj : g.a_si);
  const int64_t ldx = prm.swapped ? g.a_si : g.b_sj;

  // rows of this workgroup, in quads of 4 rows so that every lane's 4 outputs start on a multiple
  // of 4: ceil(R / 4) = rows_base * grid + rows_rem quads, the first rows_rem workgroups take one
  // more (the split is done on the host: a 64-bit division here would sit in front of the first
  // load of every wave)
  const int wg = blockIdx.x;
  const int r0 = 4 * (wg * prm.rows_base + min(wg, prm.rows_rem));
  const int r1 = min(R, r0 + 4 * (prm.rows_base + (wg < prm.rows_rem ? 1 : 0)));
  const int nblk = (r1 - r0 + 15) >> 4;
  const int kwave = wave * (SPW * 64);

  // 2 GiB raw buffer window over W.  Rows past r1 of the last block, and the units issued past the
  // last block, are never used; their lanes all read the first 16 bytes of W (one cache line per
  // instruction) instead of going out of range: an instruction whose lanes are all out of range
  // completes without a memory round trip and can retire ahead of older loads, which the counted
  // waits below must not see.
  const __amdgpu_buffer_rsrc_t rsW = __builtin_amdgcn_make_buffer_rsrc((void *)Wg, 0, 0x80000000, 0x00020000);
  // DMA instruction i of a unit: lane -> row rho = 4*i + lane/16 at position lane%16, i.e. logical
  // chunk (lane%16) ^ rho
  int dma_off[NDMA];
#pragma unroll
  for (int i = 0; i < NDMA; i++) {
    const int rho = 4 * i + g4;
    dma_off[i] = ((l16 ^ rho) << 4) + kwave;
  }
  // K may be shorter than the NW * SPW * 64 bytes the instantiation covers: the lanes of a unit that lie past
  // the end of K go out of range (bit 31) and read as zero; a unit that lies past it entirely (a uniform
  // condition: its first byte is kwave + q * SEG) is fetched like the rows past r1 and never multiplied.
  const int K = g.K;
  auto issue_unit = [&](int blk, int q, int slot) {
    const int rb = r0 + blk * 16;
    v4i *dst = &ring[wave][slot][0];
    const bool inside = !TAIL || kwave + q * SEG < K;  // uniform
#pragma unroll
    for (int i = 0; i < NDMA; i++) {
      const int row = rb + 4 * i + g4;
      const int koff = q * SEG + dma_off[i];
      lds_dma16<kWeightStreamAux>(rsW, dst + i * 64, (inside && row < r1) ? ((!TAIL || koff < K) ? row * ldw + koff : (int)0x80000000) : 0, 0);
    }
  };

  // activation fragments of this wave's K slice: lane -> token l16 (+16 per block); int8: 16 bytes
  // at K = kwave + s*64 + g4*16; fp8: the halves (s & 1) of 32 bytes at kwave + (s/2)*128 + g4*32.
  // Issued BEFORE the first weight units: the wait for them below then leaves those units in flight
  // (memory operations are counted in issue order).  The other way round the wave would sit out the
  // arrival of everything it has issued and restart the weight stream from empty: 1.3 us of 14.3 on a
  // 14336 x 4096 matrix.
  v4i xf[NB][SPW];
#pragma unroll
  for (int nb = 0; nb < NB; nb++) {
    const uint8_t *xr = Xg + (int64_t)min(nb * 16 + l16, T - 1) * ldx + kwave + g4 * (KIND == KIND_I8 ? 16 : 32);
#pragma unroll
    for (int s = 0; s < SPW; s++) {
      const int ko = KIND == KIND_I8 ? s * 64 : (s >> 1) * 128 + (s & 1) * 16;
      // (past the end of K: zero, and no load: the bytes behind a row are the next token's, or nobody's)
      xf[nb][s] = (!TAIL || kwave + g4 * (KIND == KIND_I8 ? 16 : 32) + ko < K) ? *(const v4i *)(xr + ko) : v4i{0, 0, 0, 0};
    }
  }

  // prologue: the first NSLOT units
  {
    int blk = 0, q = 0;
#pragma unroll
    for (int u = 0; u < NSLOT; u++) {
      issue_unit(blk, q, u);
      if (++q == Q) { q = 0; blk++; }
    }
  }

  // Pin the wait for the activation loads here, in straight-line code, where the compiler can count the
  // NSLOT * NDMA younger operations.  Left to its own devices it waits at their first use inside the loop,
  // where all it can prove is vmcnt(0): that drains the stream per block.
#pragma unroll
  for (int nb = 0; nb < NB; nb++)
#pragma unroll
    for (int s = 0; s < SPW; s++) asm volatile("" : "+v"(xf[nb][s]));

  Epilogue ep(g, bt);
  // Packed output: a lane's 4 outputs are 4 consecutive weight rows of one token.  When D is 16-bit,
  // contiguous along the weight rows and suitably aligned, and no C is read, they leave as one
  // 8-byte store instead of four scattered 2-byte ones.
  const int64_t d_sr = prm.swapped ? g.d_sj : g.d_si, d_st = prm.swapped ? g.d_si : g.d_sj;
  const bool packed = FAST || (!g.int_scale && (g.d_type == CUDA_R_16BF || g.d_type == CUDA_R_16F) && d_sr == 1 &&
                               g.beta_mode == SCALAR_VALUE && g.beta_val.f == 0.0f && ((uintptr_t)g.D & 7) == 0 &&
                               (d_st & 3) == 0 && (g.d_sb & 3) == 0);
  uint16_t *const Dp = (uint16_t *)g.D + g.d_sb * bt;
  const uint32_t red_base0 = lds_addr(&red[0][0][0][0]);
  const uint32_t ring_base = lds_addr(&ring[wave][0][l16 * 16]);  // this lane's row in slot 0
  int slot = 0;
  // (block, unit) that the next refill fetches: NSLOT units ahead of the one being consumed
  int fblk = NSLOT / Q, fq = NSLOT % Q;

  for (int blk = 0; blk < nblk; blk++) {
    // Who runs the epilogue of the block's 64 * NB (token, quad of rows) pairs.
    //   NB <= 2: one wave (rotating) takes them all, NB per lane.  Its epilogue costs ~1 us per block,
    //            but the other waves are left alone, which measures faster for few tokens.
    //   NB >= 3: every wave takes 64 * NB / NW pairs, one per lane; one wave alone would hold up the
    //            others for several microseconds per block and need 20 * NB registers for the factors.
    // Pair p lives in accumulator lane p % 64 of token block p / 64 of every wave.
    constexpr bool SHARED = NB >= 3;
    constexpr int PPL = SHARED ? 1 : NB;  // pairs per participating lane
    static_assert(!SHARED || (64 * NB % NW == 0 && 64 * NB / NW <= 64), "pairs are dealt out evenly, at most one per lane");
    constexpr int PAIRS_W = 64 * NB / NW;
    const bool has_pair = SHARED ? lane < PAIRS_W : wave == blk % NW;
    int my_nb[PPL], src_lane[PPL], my_tok[PPL], my_row0[PPL];
#pragma unroll
    for (int pp = 0; pp < PPL; pp++) {
      const int pair = SHARED ? wave * PAIRS_W + (lane < PAIRS_W ? lane : 0) : pp * 64 + lane;
      my_nb[pp] = pair >> 6; src_lane[pp] = pair & 63;
      my_tok[pp] = my_nb[pp] * 16 + (src_lane[pp] & 15);
      my_row0[pp] = r0 + blk * 16 + (src_lane[pp] >> 4) * 4;
    }
    // The epilogue factors of those pairs are fetched while the block streams: by the time the
    // weights have gone through the MFMAs they have long arrived, and the epilogue is left without
    // a memory round trip of its own.  Raw loads only: converting or combining them here would make
    // the compiler wait for each load on the spot.
    float f_al[PPL][4], f_sa[PPL][4], f_sb[PPL][4], f_be[PPL][4];
    uint32_t f_bias[PPL][4];
    auto prefetch_factors = [&]() {
      if (has_pair && (FAST || !g.int_scale)) {
#pragma unroll
        for (int pp = 0; pp < PPL; pp++)
#pragma unroll
          for (int v = 0; v < 4; v++) {
            const int row = min(my_row0[pp] + v, r1 - 1), tok = min(my_tok[pp], T - 1);
            const int i = prm.swapped ? tok : row, j = prm.swapped ? row : tok;
            f_al[pp][v] = ep.alpha_v ? ep.alpha_v[i] : ep.alpha_s;
            f_sa[pp][v] = ep.sa_v ? ep.sa_v[i] : ep.sa_s;
            f_sb[pp][v] = ep.sb_v ? ep.sb_v[j] : ep.sb_s;
            if constexpr (!FAST) f_be[pp][v] = ep.beta_v ? ep.beta_v[i] : ep.beta_s;
            f_bias[pp][v] = ep.bias_raw(i);
          }
      }
    };
    acc_t acc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) acc[nb] = acc_t{0, 0, 0, 0};
#pragma unroll
    for (int q = 0; q < Q; q++) {
      // the oldest unit in flight has landed (the younger NSLOT-1 may still be on their way)
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NSLOT - 1) * NDMA) : "memory");
      const uint32_t src = ring_base + slot * (UNIT_V4 * 16);
      v4i w[4];
#pragma unroll
      for (int s = 0; s < 4; s++) {
        const int chunk = KIND == KIND_I8 ? s * 4 + g4 : (s >> 1) * 8 + g4 * 2 + (s & 1);
        w[s] = lds_read16_unordered(src + ((chunk ^ l16) << 4));
      }
      // the fragments are in registers before the slot is overwritten
      frags_ready(w[0], w[1], w[2], w[3]);
      // Issued between the wait for this unit and the refill: the counted wait of the next unit
      // (everything but the NDMA youngest operations) then covers these loads without waiting for
      // anything younger than the unit it needs.
      if (q == 0) prefetch_factors();
      // One unit later the counted wait above has covered those loads as well.  Telling the compiler
      // here (where it can count: the loads are older than one refill) keeps it from waiting for
      // them in the epilogue, where its only safe choice is vmcnt(0), i.e. the units in flight.
      if (Q > 1 && q == Q - 1 && has_pair && (FAST || !g.int_scale)) {
#pragma unroll
        for (int pp = 0; pp < PPL; pp++)
#pragma unroll
          for (int v = 0; v < 4; v++) {
            asm volatile("" : "+v"(f_al[pp][v]), "+v"(f_sa[pp][v]), "+v"(f_sb[pp][v]), "+v"(f_bias[pp][v]));
            if constexpr (!FAST) asm volatile("" : "+v"(f_be[pp][v]));
          }
      }
      issue_unit(fblk, fq, slot);
      if (++fq == Q) { fq = 0; fblk++; }
      slot ^= 1;
      if (TAIL && kwave + q * SEG >= K) continue;  // (uniform) a unit past the end of K holds no data
      if constexpr (KIND == KIND_I8) {
#pragma unroll
        for (int s = 0; s < 4; s++)
#pragma unroll
          for (int nb = 0; nb < NB; nb++)
            acc[nb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[s], xf[nb][q * 4 + s], acc[nb], 0, 0, 0);
      } else {
#pragma unroll
        for (int s = 0; s < 2; s++) {
          const v8i wa = {w[2 * s][0], w[2 * s][1], w[2 * s][2], w[2 * s][3], w[2 * s + 1][0], w[2 * s + 1][1], w[2 * s + 1][2], w[2 * s + 1][3]};
#pragma unroll
          for (int nb = 0; nb < NB; nb++) {
            const v4i x0 = xf[nb][q * 4 + 2 * s], x1 = xf[nb][q * 4 + 2 * s + 1];
            const v8i xb = {x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
            acc[nb] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wa, xb, acc[nb], 0, 0, 0, 0, 0, 0);
          }
        }
      }
    }

    // cross-wave reduction of the finished block (double-buffered: a wave writes its partial sums
    // of block b + 2 only after the barrier of block b + 1, which every wave reaches after its reads
    // of block b)
    const int buf = blk & 1;
#pragma unroll
    for (int nb = 0; nb < NB; nb++) red[buf][wave][nb][lane] = __builtin_bit_cast(v4i, acc[nb]);
    lds_barrier();
    if (has_pair) {
#pragma unroll
      for (int pp = 0; pp < PPL; pp++) {
        // unordered reads again: a C++ read of LDS would wait for this wave's units in flight
        v4i part[NW];
#pragma unroll
        for (int w2 = 0; w2 < NW; w2++)
          part[w2] = lds_read16_unordered(red_base0 + (((buf * NW + w2) * NB + my_nb[pp]) * 64 + src_lane[pp]) * 16);
        lds_values_ready(part);
        acc_t s = __builtin_bit_cast(acc_t, part[0]);
#pragma unroll
        for (int w2 = 1; w2 < NW; w2++) s += __builtin_bit_cast(acc_t, part[w2]);
        const int tok = my_tok[pp], row0 = my_row0[pp];
        if (FAST || (packed && row0 + 3 < r1)) {
          if (tok < T && row0 < r1) {  // FAST: r1 is a multiple of 4, a quad is inside or outside
            float y[4];
#pragma unroll
            for (int v = 0; v < 4; v++)
              y[v] = ep.finish(((f_al[pp][v] * f_sa[pp][v]) * f_sb[pp][v]) * (float)s[v] + ep.bias_from_raw(f_bias[pp][v]));
            uint2 pk;
            if (g.d_type == CUDA_R_16BF) {
              pk.x = pack_bf16x2(y[0], y[1]);
              pk.y = pack_bf16x2(y[2], y[3]);
            } else {
              pk.x = pack_f16x2(y[0], y[1]);
              pk.y = pack_f16x2(y[2], y[3]);
            }
            *(uint2 *)(Dp + (int64_t)tok * d_st + row0) = pk;
          }
        } else if constexpr (!FAST) {
#pragma unroll
          for (int v = 0; v < 4; v++) {
            const int row = row0 + v;
            if (row < r1 && tok < T) {
              const int i = prm.swapped ? tok : row, j = prm.swapped ? row : tok;
              if (KIND == KIND_I8 && g.int_scale) ep.store_int(i, j, (int)s[v]);
              else ep.store_f(i, j, (float)s[v], f_al[pp][v] * f_sa[pp][v], f_sb[pp][v], f_be[pp][v], ep.bias_from_raw(f_bias[pp][v]));
            }
          }
        }
      }
    }
  }
  // the units issued past the last block still target this workgroup's LDS
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

} // namespace zluda_amd
