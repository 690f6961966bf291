// LDS-double-buffered MFMA GEMM for K-contiguous operands on gfx950 (CDNA4).
//
//   KIND_I8   : int8 x int8 -> int32         v_mfma_i32_32x32x32_i8
//   KIND_F8   : e4m3/e5m2 -> fp32            v_mfma_f32_32x32x64_f8f6f4 (formats FP/FQ)
//   KIND_MXF4 : e2m1 + UE8M0 per 32 -> fp32  v_mfma_scale_f32_32x32x64_f8f6f4 (cbsz=blgp=4)
//
// Naming inside the kernel: P is the operand whose row index runs along the unit-stride
// dimension of D (it is fed as MFMA operand "B", so its index lands on lane%32 of the
// accumulator and stores coalesce); Q is the other one (MFMA operand "A", index on the
// accumulator VGPRs).  For a column-major D, P = op(A) rows (i) and Q = op(B) columns (j); for a
// row-major D the planner sets `swapped` and P/Q trade places.
//
// One stage holds BKB = 128 bytes of K for every row of the P and Q tiles.  LDS rows are 128 B,
// split in eight 16-byte chunks whose position is XOR-swizzled with the row number so that both
// the ds_write_b128 of the staging copy and the ds_read_b128 of the fragment loads are
// conflict-free (16 consecutive rows reading the same logical chunk hit 16 distinct 16-byte
// bank groups).
#pragma once
#include "numeric.hpp"

namespace zluda_amd {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

enum { KIND_I8 = 0, KIND_F8 = 1, KIND_MXF4 = 2 };
constexpr int BKB = 128;  // bytes of K per LDS stage

// depends on r mod 32 only, so rows 32 apart (the MFMA tiles of one wave) share a swizzle
__device__ __forceinline__ int swz(int r) { return (r ^ ((r >> 3) & 3)) & 7; }

// Accumulator element -> 32 raw bits.  Takes the element BY VALUE: __builtin_bit_cast applied
// directly to a vector-element expression reads element 0 whatever the index.
__device__ __forceinline__ int to_bits(int x) { return x; }
__device__ __forceinline__ int to_bits(float x) { return (int)f2bits(x); }

template <int N, int I = 0, class F>
__device__ __forceinline__ void static_for(F &f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<N, I + 1>(f);
  }
}

// 16 bytes per lane from a buffer straight into LDS (buffer_load_dwordx4 ... lds).  `lds_dst` is the
// wave-uniform start of the 1 KiB block the instruction fills; lane l lands at byte l*16.
// The address-space cast only exists in the device pass.
__device__ __forceinline__ void lds_dma16(__amdgpu_buffer_rsrc_t rs, void *lds_dst, int voff, int soff) {
#if defined(__HIP_DEVICE_COMPILE__)
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void *)lds_dst, 16, voff,
                                           soff, 0, 0);
#endif
}

struct MfmaParams {
  GemmArgs g;
  int32_t swapped;           // P = op(B)^T rows, Q = op(A) rows
  int32_t tiles_p, tiles_q;  // tile counts along P and Q
  int32_t group_p;           // raster group height (tiles along P)
};

// Fused epilogue shared by the MFMA kernels.  The caller guarantees that every wave of the workgroup
// has finished reading the LDS tiles (a barrier after the K loop); `lds_words` is the start of the
// workgroup's LDS, reused here as per-wave staging.
template <int KIND, int WP, int WQ, int WTP, int WTQ, class AccV>
__device__ __forceinline__ void mfma_store_tile(const MfmaParams &prm, AccV (&acc)[WTQ / 32][WTP / 32],
                                                int *lds_words, size_t lds_bytes, int p0, int q0, int NP,
                                                int NQ, int bt) {
  constexpr int TP = WTP / 32, TQ = WTQ / 32;
  const GemmArgs &g = prm.g;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wp = wave % WP, wq = wave / WP;
  const int lr = lane & 31, gsel = lane >> 5;
  (void)lds_bytes;
  // ---- epilogue --------------------------------------------------------------------------
  // The accumulators go through LDS (free after the main loop) so that every lane ends up with
  // four consecutive elements along the unit-stride dimension of D: stores are 8 B (bf16) or
  // 16 B (int32/fp32) per lane and contiguous across the 16/32 lanes that share a D column.
  // Each wave stages 16 Q-rows x WTP P-columns per pass in its own LDS region.
  constexpr int SROW = WTP + 8;              // dwords; +8 keeps the two lane halves on distinct banks
  constexpr int LPR = WTP / 4;               // lanes per staged row
  constexpr int RPI = 64 / LPR;              // staged rows read per instruction
  constexpr int ITER = 16 / RPI;
  int *stage = lds_words + wave * (16 * SROW);

  Epilogue ep(g, bt);
  const bool swp = prm.swapped != 0;
  const int pl = (lane % LPR) * 4, qsub = lane / LPR;
  const int pi0 = p0 + wp * WTP + pl;
  // quantities that depend on the P index only: fixed per lane for the whole epilogue
  float p_scale[4], p_bias[4], p_beta[4];
#pragma unroll
  for (int e = 0; e < 4; e++) {
    const int pi = min(pi0 + e, NP - 1);
    p_scale[e] = g.int_scale ? 1.0f : (swp ? ep.col_scale(pi) : ep.row_scale(pi));
    p_bias[e] = (g.int_scale || swp) ? 0.0f : ep.bias_at(pi);
    p_beta[e] = (g.int_scale || swp) ? 0.0f : ep.beta_at(pi);
  }
  const int64_t d_sp = swp ? g.d_sj : g.d_si, d_sq = swp ? g.d_si : g.d_sj;  // d_sp == 1
  const int64_t c_sp = swp ? g.c_sj : g.c_si, c_sq = swp ? g.c_si : g.c_sj;
  const uint32_t dbits = g.d_type == CUDA_R_32F || g.d_type == CUDA_R_32I ? 32 : g.d_type == CUDA_R_8I ? 8 : 16;
  const bool int_fast = g.int_scale && g.alpha_mode != VECTOR_DEV && g.beta_mode != VECTOR_DEV;
  int32_t ialpha = 1, ibeta = 0;
  if (int_fast) {
    ialpha = g.alpha_mode == SCALAR_VALUE ? g.alpha_val.i : *(const int32_t *)g.alpha_ptr;
    ibeta = g.beta_mode == SCALAR_VALUE ? g.beta_val.i : *(const int32_t *)g.beta_ptr;
  }

  // `pass` must be a compile-time constant: a rolled loop here would index the accumulator
  // registers dynamically and push them to scratch for the whole kernel.
  auto do_pass = [&](auto pass_c) {
    constexpr int pass = decltype(pass_c)::value;
    constexpr int a = pass >> 1, h = pass & 1;
#pragma unroll
    for (int b = 0; b < TP; b++)
#pragma unroll
      for (int vv = 0; vv < 8; vv++) {
        const int ql = 8 * (vv >> 2) + 4 * gsel + (vv & 3);
        stage[ql * SROW + b * 32 + lr] = to_bits(acc[a][b][h * 8 + vv]);
      }
    __syncthreads();
#pragma unroll 1
    for (int it = 0; it < ITER; it++) {
      const int ql = it * RPI + qsub;
      const int qi = q0 + wq * WTQ + a * 32 + h * 16 + ql;
      const v4i raw = *(const v4i *)&stage[ql * SROW + pl];
      if (qi >= NQ || pi0 >= NP) continue;
      const int64_t dbase = g.d_sb * bt + (int64_t)pi0 * d_sp + (int64_t)qi * d_sq;
      const int64_t cbase = g.c_sb * bt + (int64_t)pi0 * c_sp + (int64_t)qi * c_sq;
      const bool full4 = pi0 + 3 < NP && ((dbase * dbits / 8) & (dbits / 2 - 1)) == 0 &&
                         (((uintptr_t)g.D) & 15) == 0;
      if (g.int_scale) {
        if (int_fast) {
          v4i r;
#pragma unroll
          for (int e = 0; e < 4; e++) {
            uint32_t x = (uint32_t)ialpha * (uint32_t)raw[e];
            if (ibeta != 0 && pi0 + e < NP) x += (uint32_t)ibeta * (uint32_t)((const int32_t *)g.C)[cbase + e * c_sp];
            r[e] = (int)x;
          }
          if (full4) *(v4i *)((int32_t *)g.D + dbase) = r;
          else
#pragma unroll
            for (int e = 0; e < 4; e++) if (pi0 + e < NP) ((int32_t *)g.D)[dbase + e] = r[e];
        } else {
#pragma unroll
          for (int e = 0; e < 4; e++)
            if (pi0 + e < NP) ep.store_int(swp ? qi : pi0 + e, swp ? pi0 + e : qi, raw[e]);
        }
        continue;
      }
      const float q_scale = swp ? ep.row_scale(qi) : ep.col_scale(qi);
      const float q_bias = swp ? ep.bias_at(qi) : 0.0f;
      const float q_beta = swp ? ep.beta_at(qi) : 0.0f;
      float x[4];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const int rawe = raw[e];
        const float accf = KIND == KIND_I8 ? (float)rawe : bits2f((uint32_t)rawe);
        float y = (swp ? q_scale * p_scale[e] : p_scale[e] * q_scale) * accf;
        const float be = swp ? q_beta : p_beta[e];
        if (be != 0.0f && pi0 + e < NP) y += be * ep.sc * load_elem(g.C, g.c_type, cbase + e * c_sp);
        y += swp ? q_bias : p_bias[e];
        x[e] = ep.finish(y);
      }
      if (full4 && dbits == 32 && g.d_type == CUDA_R_32F) {
        *(float4 *)((float *)g.D + dbase) = make_float4(x[0], x[1], x[2], x[3]);
      } else if (full4 && g.d_type == CUDA_R_16BF) {
        uint2 pk;
        pk.x = (uint32_t)enc_bf16(x[0]) | ((uint32_t)enc_bf16(x[1]) << 16);
        pk.y = (uint32_t)enc_bf16(x[2]) | ((uint32_t)enc_bf16(x[3]) << 16);
        *(uint2 *)((uint16_t *)g.D + dbase) = pk;
      } else if (full4 && g.d_type == CUDA_R_16F) {
        uint2 pk;
        pk.x = (uint32_t)enc_f16(x[0]) | ((uint32_t)enc_f16(x[1]) << 16);
        pk.y = (uint32_t)enc_f16(x[2]) | ((uint32_t)enc_f16(x[3]) << 16);
        *(uint2 *)((uint16_t *)g.D + dbase) = pk;
      } else {
#pragma unroll
        for (int e = 0; e < 4; e++)
          if (pi0 + e < NP) store_elem(g.D, g.d_type, dbase + e, x[e]);
      }
    }
    __syncthreads();
  };
  static_for<TQ * 2>(do_pass);
}

// LOADMODE 0: global -> VGPR -> ds_write_b128 (one stage ahead in registers)
// LOADMODE 1: buffer_load ... lds  (global -> LDS directly, no staging registers)
template <int KIND, int FQ, int FP, int BP, int BQ, int WP, int WQ, int LOADMODE>
__global__ __launch_bounds__(WP *WQ * 64) void gemm_mfma_kernel(MfmaParams prm) {
  constexpr int NT = WP * WQ * 64;
  constexpr int RP = NT / 8;          // rows copied per pass of the staging loop
  constexpr int LP = BP / RP, LQ = BQ / RP;
  constexpr int WTP = BP / WP, WTQ = BQ / WQ;  // wave tile
  constexpr int TP = WTP / 32, TQ = WTQ / 32;  // MFMA tiles per wave
  static_assert(BP % RP == 0 && BQ % RP == 0, "tile must be a multiple of the copy pass");
  static_assert(RP % 32 == 0, "the swizzle of a thread's rows must not change between passes");
  using acc_v = typename std::conditional<KIND == KIND_I8, v16i, v16f>::type;

  __shared__ v4i lds[2][(BP + BQ) * 8];

  const GemmArgs &g = prm.g;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int wp = wave % WP, wq = wave / WP;
  const int bt = blockIdx.y;

  // ---- workgroup -> tile: XCD-aware remap, then grouped raster --------------------------
  // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous run of tiles so
  // that the tiles sharing P/Q panels also share an L2.
  const int total = prm.tiles_p * prm.tiles_q;
  int w = blockIdx.x;
  if ((total & 7) == 0) w = (w & 7) * (total >> 3) + (w >> 3);
  const int group = prm.group_p * prm.tiles_q;
  const int gid = w / group, first_p = gid * prm.group_p;
  const int gsz = min(prm.tiles_p - first_p, prm.group_p);
  const int tile_p = first_p + (w % group) % gsz, tile_q = (w % group) / gsz;
  const int p0 = tile_p * BP, q0 = tile_q * BQ;

  // ---- operand views (bytes) --------------------------------------------------------------
  const int NP = prm.swapped ? g.N : g.M, NQ = prm.swapped ? g.M : g.N;
  constexpr int ebits = KIND == KIND_MXF4 ? 4 : 8;
  const int Kbytes = (int)((int64_t)g.K * ebits / 8);
  const uint8_t *Pg, *Qg;
  int ldp, ldq;  // bytes between consecutive rows (the planner keeps whole operands < 2 GiB)
  if (!prm.swapped) {
    Pg = (const uint8_t *)g.A + g.a_sb * bt * ebits / 8; ldp = (int)(g.a_si * ebits / 8);
    Qg = (const uint8_t *)g.B + g.b_sb * bt * ebits / 8; ldq = (int)(g.b_sj * ebits / 8);
  } else {
    Pg = (const uint8_t *)g.B + g.b_sb * bt * ebits / 8; ldp = (int)(g.b_sj * ebits / 8);
    Qg = (const uint8_t *)g.A + g.a_sb * bt * ebits / 8; ldq = (int)(g.a_si * ebits / 8);
  }
  const int KT = (Kbytes + BKB - 1) / BKB;

  // Raw buffer descriptors with a 2 GiB window: an offset with bit 31 set is out of range and
  // reads as zero, which is how the K tail of the last stage is zero-filled without branches.
  const __amdgpu_buffer_rsrc_t rsP = __builtin_amdgcn_make_buffer_rsrc((void *)Pg, 0, 0x80000000, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsQ = __builtin_amdgcn_make_buffer_rsrc((void *)Qg, 0, 0x80000000, 0x00020000);

  // staging copy: thread -> row r0 + RP*i, LDS slot (t & 7), global chunk (t & 7) ^ swz(row)
  const int r0 = t >> 3, slot = t & 7, cg = slot ^ swz(r0);
  int voffP[LP], voffQ[LQ];
#pragma unroll
  for (int i = 0; i < LP; i++) voffP[i] = min(p0 + r0 + RP * i, NP - 1) * ldp + cg * 16;
#pragma unroll
  for (int i = 0; i < LQ; i++) voffQ[i] = min(q0 + r0 + RP * i, NQ - 1) * ldq + cg * 16;
  const int tail_bytes = Kbytes - (KT - 1) * BKB;  // valid bytes of the last stage (1..128)
  const int oob_last = cg * 16 < tail_bytes ? 0 : (int)0x80000000;

  v4i preg[LOADMODE == 0 ? LP : 1], qreg[LOADMODE == 0 ? LQ : 1];
  auto gload = [&](int kt, int buf) {
    const int oob = kt == KT - 1 ? oob_last : 0;
    if constexpr (LOADMODE == 0) {
#pragma unroll
      for (int i = 0; i < LP; i++) preg[i] = __builtin_amdgcn_raw_buffer_load_b128(rsP, voffP[i] | oob, kt * BKB, 0);
#pragma unroll
      for (int i = 0; i < LQ; i++) qreg[i] = __builtin_amdgcn_raw_buffer_load_b128(rsQ, voffQ[i] | oob, kt * BKB, 0);
    } else {
      // each wave instruction fills 1 KiB of LDS: 8 rows x 128 B, lane l -> byte l*16
#pragma unroll
      for (int i = 0; i < LP; i++)
        lds_dma16(rsP, &lds[buf][(wave * 8 + RP * i) * 8], voffP[i] | oob, kt * BKB);
#pragma unroll
      for (int i = 0; i < LQ; i++)
        lds_dma16(rsQ, &lds[buf][(BP + wave * 8 + RP * i) * 8], voffQ[i] | oob, kt * BKB);
    }
  };
  auto lstore = [&](int buf) {
    if constexpr (LOADMODE == 0) {
#pragma unroll
      for (int i = 0; i < LP; i++) lds[buf][(r0 + RP * i) * 8 + slot] = preg[i];
#pragma unroll
      for (int i = 0; i < LQ; i++) lds[buf][(BP + r0 + RP * i) * 8 + slot] = qreg[i];
    }
  };
  auto stage_fence = [&]() {
    if constexpr (LOADMODE == 1) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): LDS DMA landed
    __syncthreads();
  };

  // ---- MX block scales: one dword (4 consecutive K blocks) per lane, row and stage ----------
  // lane group gsel (= lane/32) owns chunks gsel*4 .. gsel*4+3 of the stage, i.e. K blocks
  // kt*8 + gsel*4 + ks, whose scale bytes are one aligned dword of the [row][K/32] scale tensor.
  const int lr = lane & 31, gsel = lane >> 5;
  const uint8_t *sp_row[TP], *sq_row[TQ];
  int sp_cur[TP], sq_cur[TQ], sp_nxt[TP], sq_nxt[TQ];
  if constexpr (KIND == KIND_MXF4) {
    const int KB = g.K / 32;
    const uint8_t *Ps = (const uint8_t *)(prm.swapped ? g.b_scale : g.a_scale) + (int64_t)bt * NP * KB;
    const uint8_t *Qs = (const uint8_t *)(prm.swapped ? g.a_scale : g.b_scale) + (int64_t)bt * NQ * KB;
#pragma unroll
    for (int i = 0; i < TP; i++)
      sp_row[i] = Ps + (int64_t)min(p0 + wp * WTP + i * 32 + lr, NP - 1) * KB + gsel * 4;
#pragma unroll
    for (int i = 0; i < TQ; i++)
      sq_row[i] = Qs + (int64_t)min(q0 + wq * WTQ + i * 32 + lr, NQ - 1) * KB + gsel * 4;
  }
  auto sload = [&](int kt) {
    if constexpr (KIND == KIND_MXF4) {
#pragma unroll
      for (int i = 0; i < TP; i++) sp_nxt[i] = *(const int *)(sp_row[i] + kt * 8);
#pragma unroll
      for (int i = 0; i < TQ; i++) sq_nxt[i] = *(const int *)(sq_row[i] + kt * 8);
    }
  };

  acc_v acc[TQ][TP];
#pragma unroll
  for (int a = 0; a < TQ; a++)
#pragma unroll
    for (int b = 0; b < TP; b++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[a][b][v] = 0;

  gload(0, 0);
  sload(0);
  lstore(0);
  stage_fence();

  int kt = 0;
  do {  // K >= 1, so at least one stage
    const int buf = kt & 1;
    if constexpr (KIND == KIND_MXF4) {
#pragma unroll
      for (int i = 0; i < TP; i++) sp_cur[i] = sp_nxt[i];
#pragma unroll
      for (int i = 0; i < TQ; i++) sq_cur[i] = sq_nxt[i];
    }
    if (kt + 1 < KT) { gload(kt + 1, buf ^ 1); sload(kt + 1); }

    const v4i *Pl = &lds[buf][(wp * WTP + lr) * 8];
    const v4i *Ql = &lds[buf][(BP + wq * WTQ + lr) * 8];
    const int sw = swz(lr);  // wave-tile bases are multiples of 32: swz(row) == swz(lr)

    if constexpr (KIND == KIND_I8) {
#pragma unroll
      for (int ks = 0; ks < 4; ks++) {
        const int ch = (ks * 2 + gsel) ^ sw;
        v4i pf[TP], qf[TQ];
#pragma unroll
        for (int i = 0; i < TP; i++) pf[i] = Pl[i * 32 * 8 + ch];
#pragma unroll
        for (int i = 0; i < TQ; i++) qf[i] = Ql[i * 32 * 8 + ch];
#pragma unroll
        for (int a = 0; a < TQ; a++)
#pragma unroll
          for (int b = 0; b < TP; b++)
            acc[a][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(qf[a], pf[b], acc[a][b], 0, 0, 0);
      }
    } else if constexpr (KIND == KIND_F8) {
#pragma unroll
      for (int ks = 0; ks < 2; ks++) {
        const int c0 = (ks * 4 + gsel * 2) ^ sw, c1 = (ks * 4 + gsel * 2 + 1) ^ sw;
        v8i pf[TP], qf[TQ];
#pragma unroll
        for (int i = 0; i < TP; i++) {
          v4i lo = Pl[i * 32 * 8 + c0], hi = Pl[i * 32 * 8 + c1];
          pf[i] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
#pragma unroll
        for (int i = 0; i < TQ; i++) {
          v4i lo = Ql[i * 32 * 8 + c0], hi = Ql[i * 32 * 8 + c1];
          qf[i] = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
#pragma unroll
        for (int a = 0; a < TQ; a++)
#pragma unroll
          for (int b = 0; b < TP; b++)
            acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(qf[a], pf[b], acc[a][b], FQ, FP,
                                                                         0, 0, 0, 0);
      }
    } else {
#pragma unroll
      for (int ks = 0; ks < 4; ks++) {
        const int ch = (gsel * 4 + ks) ^ sw;
        v8i pf[TP], qf[TQ];
#pragma unroll
        for (int i = 0; i < TP; i++) {
          v4i lo = Pl[i * 32 * 8 + ch];
          pf[i] = v8i{lo[0], lo[1], lo[2], lo[3], 0, 0, 0, 0};
        }
#pragma unroll
        for (int i = 0; i < TQ; i++) {
          v4i lo = Ql[i * 32 * 8 + ch];
          qf[i] = v8i{lo[0], lo[1], lo[2], lo[3], 0, 0, 0, 0};
        }
#pragma unroll
        for (int a = 0; a < TQ; a++)
#pragma unroll
          for (int b = 0; b < TP; b++) {
            // op_sel picks byte ks of each scale dword; the builtin wants it as a constant
            switch (ks) {
            case 0: acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(qf[a], pf[b], acc[a][b], 4, 4, 0, sq_cur[a], 0, sp_cur[b]); break;
            case 1: acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(qf[a], pf[b], acc[a][b], 4, 4, 1, sq_cur[a], 1, sp_cur[b]); break;
            case 2: acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(qf[a], pf[b], acc[a][b], 4, 4, 2, sq_cur[a], 2, sp_cur[b]); break;
            default: acc[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(qf[a], pf[b], acc[a][b], 4, 4, 3, sq_cur[a], 3, sp_cur[b]); break;
            }
          }
      }
    }

    if (kt + 1 < KT) lstore(buf ^ 1);
    stage_fence();
  } while (++kt < KT);

  mfma_store_tile<KIND, WP, WQ, WTP, WTQ>(prm, acc, (int *)&lds[0][0], sizeof(lds), p0, q0, NP, NQ, bt);
}

} // namespace zluda_amd
