// Shared pieces of the MFMA GEMM kernels for K-contiguous operands on gfx950 (CDNA4): vector types,
// LDS swizzle, direct global -> LDS copies, and the fused epilogues.  The K loop is in
// gemm_mfma_pipe.hpp.
//
//   KIND_I8   : int8 x int8 -> int32         v_mfma_i32_32x32x32_i8
//   KIND_F8   : e4m3/e5m2 -> fp32            v_mfma_f32_32x32x64_f8f6f4 (formats FP/FQ)
//   KIND_MXF4 : e2m1 + UE8M0 per 32 -> fp32  v_mfma_scale_f32_32x32x64_f8f6f4 (cbsz=blgp=4)
//   KIND_F16  : f16 x f16 -> fp32            v_mfma_f32_32x32x16_f16
//   KIND_BF16 : bf16 x bf16 -> fp32          v_mfma_f32_32x32x16_bf16
//   KIND_F32  : f32 x f32 -> fp32            v_mfma_f32_32x32x2_f32 (four per 16 bytes of K and lane)
//
// Naming inside the kernel: P is the operand whose row index runs along the unit-stride
// dimension of D (it is fed as MFMA operand "B", so its index lands on lane%32 of the
// accumulator and stores coalesce); Q is the other one (MFMA operand "A", index on the
// accumulator VGPRs).  For a column-major D, P = op(A) rows (i) and Q = op(B) columns (j); for a
// row-major D the planner sets `swapped` and P/Q trade places.
//
// LDS rows of 128 B are split in eight 16-byte chunks whose position is XOR-swizzled with the row
// number so that both the 1 KiB-per-instruction LDS fills and the ds_read_b128 fragment loads are
// conflict-free (16 consecutive rows reading the same logical chunk hit 16 distinct 16-byte bank
// groups).
#pragma once
#include "numeric.hpp"

namespace zluda_amd {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8b __attribute__((ext_vector_type(8)));

enum { KIND_I8 = 0, KIND_F8 = 1, KIND_MXF4 = 2, KIND_F16 = 3, KIND_BF16 = 4, KIND_F32 = 5 };
// 16-bit elements: 16 bytes (8 elements) of K per lane and MFMA, i.e. the byte geometry of int8
constexpr bool kind_is_h16(int kind) { return kind == KIND_F16 || kind == KIND_BF16; }
// bytes per element of the kinds whose elements are whole bytes
constexpr int kind_esz(int kind) { return kind_is_h16(kind) ? 2 : (kind == KIND_F32 ? 4 : 1); }
// f32: a lane's 16 bytes are four K elements, one v_mfma_f32_32x32x2_f32 each; element e of lane group g of the
// 32-byte step s is K index 8 s + 4 g + e for both operands, which is all the instruction asks of a K order

// depends on r mod 32 only, so rows 32 apart (the MFMA tiles of one wave) share a swizzle
__device__ __forceinline__ int swz(int r) { return (r ^ ((r >> 3) & 3)) & 7; }

// Accumulator element -> 32 raw bits.  Takes the element BY VALUE: __builtin_bit_cast applied
// directly to a vector-element expression reads element 0 whatever the index.
__device__ __forceinline__ int to_bits(int x) { return x; }
__device__ __forceinline__ int to_bits(float x) { return (int)f2bits(x); }

template <int N, int I = 0, class F>
__device__ __forceinline__ void static_for(F &&f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<N, I + 1>(f);
  }
}

// 16 bytes per lane from a buffer straight into LDS (buffer_load_dwordx4 ... lds).  `lds_dst` is the
// wave-uniform start of the 1 KiB block the instruction fills; lane l lands at byte l*16.
// The address-space cast only exists in the device pass.
// AUX: the cache policy bits of the instruction (0: default; 2: nt, for bytes that are read once).
template <int AUX = 0>
__device__ __forceinline__ void lds_dma16(__amdgpu_buffer_rsrc_t rs, void *lds_dst, int voff, int soff) {
#if defined(__HIP_DEVICE_COMPILE__)
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void *)lds_dst, 16, voff,
                                           soff, 0, AUX);
#endif
}

// 4 bytes per lane from a buffer straight into LDS (buffer_load_dword ... lds): lane l lands at byte l*4 of the 256-byte
// block that starts at the wave-uniform `lds_dst`.
__device__ __forceinline__ void lds_dma4(__amdgpu_buffer_rsrc_t rs, void *lds_dst, int voff, int soff) {
#if defined(__HIP_DEVICE_COMPILE__)
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void *)lds_dst, 4, voff, soff, 0, 0);
#endif
}

// 128-bit buffer store whose data registers stay untouched for the wait states that follow it.  Observed on
// MI355X: when the instruction right behind a buffer_store_dwordx4 (offen, scalar offset in an SGPR) is a
// VALU write to the first data register, the store now and then writes the new value instead (element 0 of
// the four, in a few hundred of 131072 outputs); the compiler's hazard table does not list this case, so it
// puts no wait state there.  The asm keeps the data registers live across an s_nop that follows the store.
// AUX: cache policy bits (2 = nt: results that nobody reads back soon; measured on the four-wave kernel's 256 MiB of
// int32 at 8192^3: 392 us instead of 402).
template <int AUX = 0>
__device__ __forceinline__ void buffer_store_b128_guarded(v4i data, __amdgpu_buffer_rsrc_t rs, int voff, int soff) {
  __builtin_amdgcn_raw_buffer_store_b128(data, rs, voff, soff, AUX);
  asm volatile("s_nop 1" : "+v"(data)::"memory");
}

// The same guard for a 64-bit store.  The corruption was only ever seen with the 128-bit form, but nothing known about
// it says the narrower store reads its data registers any earlier, and a wait state per store is not measurable in the
// epilogues that use it.
__device__ __forceinline__ void buffer_store_b64_guarded(v2i data, __amdgpu_buffer_rsrc_t rs, int voff, int soff) {
  __builtin_amdgcn_raw_buffer_store_b64(data, rs, voff, soff, 0);
  asm volatile("s_nop 1" : "+v"(data)::"memory");
}

struct MfmaParams {
  GemmArgs g;
  int32_t swapped;           // P = op(B)^T rows, Q = op(A) rows
  int32_t tiles_p, tiles_q;  // tile counts along P and Q
  int32_t group_p;           // raster group height (tiles along P)
  // split-K (splits > 1): workgroup z of gridDim.z handles stages [z * split_stages, ...) of K and
  // writes its raw partial tile to ws[(z * batch + bt)][tiles_q * BQ][tiles_p * BP] (int32 / fp32)
  int32_t splits, split_stages;
  void *ws;
};

// General fused epilogue of the MFMA kernels: any D type, C read, vectors along either dimension,
// partial tiles.  Correct for everything the planner admits, but it spends ~150 instructions per
// four outputs; the fast paths in mfma_store_tile below take the common cases.
// The caller guarantees that every wave of the workgroup has finished reading the LDS tiles (a
// barrier after the K loop); `lds_words` is the start of the workgroup's LDS, reused as staging.
template <int KIND, int WP, int WQ, int WTP, int WTQ, class AccV>
__device__ __forceinline__ void mfma_store_tile_general(const MfmaParams &prm, AccV (&acc)[WTQ / 32][WTP / 32],
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
  constexpr int RPI = 64 / LPR;              // staged rows read per instruction (96-wide wave tiles: 2, lanes 48-63 idle)
  constexpr int ITER = 16 / RPI;
  static_assert(16 % RPI == 0, "whole passes");
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
      if (qi >= NQ || pi0 >= NP || qsub >= RPI) continue;
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

// Size of the buffer window of a wave tile whose corner is `base_elems` elements into this batch's D:
// what is left of the matrix (NQ columns of pitch d_sq, the last one NP long).  Stores of a tile that
// hangs over the last column fall outside the window and are dropped by the hardware, which is what
// lets the fast paths below take tiles that are complete along P only.
__device__ __forceinline__ uint32_t tile_window_bytes(int64_t d_sq, int NP, int NQ, int64_t base_elems, int esz) {
  const int64_t left = ((int64_t)(NQ - 1) * d_sq + NP - base_elems) * esz;
  return left <= 0 ? 0u : (left > 0xFFFFFFFFll ? 0xFFFFFFFFu : (uint32_t)left);
}

// Fast path 1: pure integer epilogue with alpha, beta scalars and beta == 0 on a full tile with
// 16-byte aligned columns: D = alpha * acc straight from the accumulator registers.  Lanes 0..31 of
// a store hold 32 consecutive int32 of one D column (one 128-byte line), so no LDS staging is
// needed; two instructions per output element.
template <int WP, int WQ, int WTP, int WTQ>
__device__ __forceinline__ void mfma_store_tile_i32(const MfmaParams &prm, v16i (&acc)[WTQ / 32][WTP / 32],
                                                    int p0, int q0, int NP, int NQ, int bt, int ialpha) {
  constexpr int TP = WTP / 32, TQ = WTQ / 32;
  const GemmArgs &g = prm.g;
  // the wave index is uniform by construction; say so, or the buffer descriptor built from it is
  // treated as divergent and every store is wrapped in a readfirstlane loop
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wp = wave % WP, wq = wave / WP;
  const int lr = lane & 31, gsel = lane >> 5;
  const int d_sq = (int)(prm.swapped ? g.d_si : g.d_sj);  // < 2^22 (checked by the dispatcher)
  // Buffer stores: wave-uniform descriptor at the wave tile, per-lane byte offset of (row 4*gsel,
  // column lr) in a VGPR, everything else in the scalar offset.
  const int64_t corner = (int64_t)(q0 + wq * WTQ) * d_sq + (p0 + wp * WTP);
  int32_t *Dw = (int32_t *)g.D + g.d_sb * bt + corner;
  const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)Dw, 0, tile_window_bytes(d_sq, NP, NQ, corner, 4), 0x00020000);
  const int voff = (4 * gsel * d_sq + lr) * 4;
  // alpha == 1 (the usual case) stores the accumulator registers as they are
  if (ialpha == 1) {
#pragma unroll
    for (int a = 0; a < TQ; a++)
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const int soff = (a * 32 + 8 * (v >> 2) + (v & 3)) * d_sq * 4;  // uniform
#pragma unroll
        for (int b = 0; b < TP; b++) __builtin_amdgcn_raw_buffer_store_b32(acc[a][b][v], rs, voff, soff + b * 128, 0);
      }
  } else {
#pragma unroll
    for (int a = 0; a < TQ; a++)
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const int soff = (a * 32 + 8 * (v >> 2) + (v & 3)) * d_sq * 4;
#pragma unroll
        for (int b = 0; b < TP; b++)
          __builtin_amdgcn_raw_buffer_store_b32(acc[a][b][v] * ialpha, rs, voff, soff + b * 128, 0);
      }
  }
}

// Split-K partial tile: the raw accumulators (int32, or fp32 bit patterns) of a whole tile into the
// padded workspace matrix of pitch `ws_pitch` dwords; same store pattern as mfma_store_tile_i32.
template <int WP, int WQ, int WTP, int WTQ, class AccV>
__device__ __forceinline__ void mfma_store_tile_raw(int32_t *ws_tile, int ws_pitch, AccV (&acc)[WTQ / 32][WTP / 32]) {
  constexpr int TP = WTP / 32, TQ = WTQ / 32;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wp = wave % WP, wq = wave / WP;
  const int lr = lane & 31, gsel = lane >> 5;
  int32_t *Dw = ws_tile + (int64_t)(wq * WTQ) * ws_pitch + wp * WTP;
  const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)Dw, 0, 0xFFFFFFFF, 0x00020000);
  const int voff = (4 * gsel * ws_pitch + lr) * 4;
#pragma unroll
  for (int a = 0; a < TQ; a++)
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int soff = (a * 32 + 8 * (v >> 2) + (v & 3)) * ws_pitch * 4;  // uniform
#pragma unroll
      for (int b = 0; b < TP; b++) __builtin_amdgcn_raw_buffer_store_b32(to_bits(acc[a][b][v]), rs, voff, soff + b * 128, 0);
    }
}

// Fast path 2: float epilogue without a C read (beta == 0) on a full tile, D of type bf16, f16 or
// f32 with aligned columns.  The accumulators are staged through LDS so that a lane owns four
// consecutive elements of a D column (8- or 16-byte stores, 256/512 contiguous bytes per column and
// instruction).  Everything that does not change inside the inner loop is hoisted; the loop body is
// one ds_read_b128, the arithmetic and one store.
template <int KIND, int WP, int WQ, int WTP, int WTQ, int ACT, int DT, class AccV>
__device__ __forceinline__ void mfma_store_tile_f(const MfmaParams &prm, AccV (&acc)[WTQ / 32][WTP / 32],
                                                  int *lds_words, int p0, int q0, int NP, int NQ, int bt) {
  constexpr int TP = WTP / 32, TQ = WTQ / 32;
  constexpr int SROW = WTP + 8, LPR = WTP / 4, RPI = 64 / LPR, ITER = 16 / RPI;
  static_assert(16 % RPI == 0, "whole passes");
  constexpr int ESZ = DT == 2 ? 4 : 2;
  const GemmArgs &g = prm.g;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wp = wave % WP, wq = wave / WP;
  const int lr = lane & 31, gsel = lane >> 5;
  int *stage = lds_words + wave * (16 * SROW);
  Epilogue ep(g, bt);
  const bool swp = prm.swapped != 0;
  const int pl = (lane % LPR) * 4, qsub = lane / LPR;
  const int pi0 = p0 + wp * WTP + pl;
  float p_scale[4], p_bias[4];
#pragma unroll
  for (int e = 0; e < 4; e++) {
    p_scale[e] = swp ? ep.col_scale(pi0 + e) : ep.row_scale(pi0 + e);
    p_bias[e] = swp ? 0.0f : ep.bias_at(pi0 + e);
  }
  // vectors that run along Q (per-column scale, or per-row quantities of a row-major D)
  const bool q_vec = swp ? (ep.alpha_v || ep.sa_v || g.bias) : (ep.sb_v != nullptr);
  const float q_scale_u = swp ? ep.row_scale(0) : ep.col_scale(0);  // used when !q_vec
  const int d_sq = (int)(swp ? g.d_si : g.d_sj);  // < 2^22 (checked by the dispatcher)
  // buffer stores: uniform descriptor at the wave tile, per-lane byte offset (row qsub, column pl)
  const int64_t corner = (int64_t)(q0 + wq * WTQ) * d_sq + (p0 + wp * WTP);
  char *Dw = (char *)g.D + (g.d_sb * bt + corner) * ESZ;
  const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)Dw, 0, tile_window_bytes(d_sq, NP, NQ, corner, ESZ), 0x00020000);
  const int voff = (qsub * d_sq + pl) * ESZ;
  const int read_off = qsub * SROW + pl;

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
    // no workgroup barrier: the staging rows belong to this wave alone, and LDS executes the
    // writes and reads of one wave in program order
#pragma unroll 2
    for (int it = 0; it < ITER; it++) {
      if (64 % LPR != 0 && qsub >= RPI) continue;  // 96-wide wave tiles: lanes beyond the last whole staged row
      const v4i raw = *(const v4i *)&stage[it * RPI * SROW + read_off];
      float qs = q_scale_u, qb = 0.0f;
      if (q_vec) {
        const int qi = min(q0 + wq * WTQ + a * 32 + h * 16 + it * RPI + qsub, NQ - 1);  // columns past the end: dropped stores
        qs = swp ? ep.row_scale(qi) : ep.col_scale(qi);
        qb = swp ? ep.bias_at(qi) : 0.0f;
      }
      float x[4];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const int rawe = raw[e];
        const float accf = KIND == KIND_I8 ? (float)rawe : bits2f((uint32_t)rawe);
        float y = (swp ? qs * p_scale[e] : p_scale[e] * qs) * accf + (swp ? qb : p_bias[e]);
        if (ACT == ACT_RELU) y = y > 0.0f ? y : 0.0f;
        else if (ACT == ACT_GELU) y = gelu_tanh(y);
        x[e] = y * ep.sd;
      }
      const int soff = (a * 32 + h * 16 + it * RPI) * d_sq * ESZ;  // uniform
      if constexpr (DT == 2) {
        const v4i pk = {(int)f2bits(x[0]), (int)f2bits(x[1]), (int)f2bits(x[2]), (int)f2bits(x[3])};
        buffer_store_b128_guarded(pk, rs, voff, soff);
      } else {
        v2i pk;
        if constexpr (DT == 0) {
          pk[0] = (int)pack_bf16x2(x[0], x[1]);
          pk[1] = (int)pack_bf16x2(x[2], x[3]);
        } else {
          pk[0] = (int)pack_f16x2(x[0], x[1]);
          pk[1] = (int)pack_f16x2(x[2], x[3]);
        }
        buffer_store_b64_guarded(pk, rs, voff, soff);
      }
    }
  };
  static_for<TQ * 2>(do_pass);
}

// Fast path 3: the same float epilogue when nothing varies along Q (no per-column scale vector for a
// column-major D, no per-row vectors for a row-major one), D bf16 or f16: straight from the
// accumulator registers, no LDS.  Lane (lr, gsel) holds element (column lr, row 8*(v/4)+4*gsel+v%4)
// of each 32x32 tile; rows 2k and 2k+1 are paired: after one DPP swap with the neighbouring lane the
// even lane owns columns (lr, lr+1) of row 2k and the odd lane columns (lr-1, lr) of row 2k+1, so
// every lane stores one dword of two 16-bit results and a store instruction writes four 64-byte row
// segments.
template <int KIND, int WP, int WQ, int WTP, int WTQ, int ACT, int DT, class AccV>
__device__ __forceinline__ void mfma_store_tile_f16_direct(const MfmaParams &prm, AccV (&acc)[WTQ / 32][WTP / 32],
                                                           int p0, int q0, int NP, int NQ, int bt) {
  static_assert(DT == 0 || DT == 1, "16-bit outputs");
  constexpr int TP = WTP / 32, TQ = WTQ / 32;
  const GemmArgs &g = prm.g;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wp = wave % WP, wq = wave / WP;
  const int lr = lane & 31, gsel = lane >> 5, odd = lane & 1;
  Epilogue ep(g, bt);
  const bool swp = prm.swapped != 0;
  const float q_scale = swp ? ep.row_scale(0) : ep.col_scale(0);
  float p_scale[TP], p_bias[TP];
#pragma unroll
  for (int b = 0; b < TP; b++) {
    const int pi = p0 + wp * WTP + b * 32 + lr;
    p_scale[b] = swp ? ep.col_scale(pi) : ep.row_scale(pi);
    p_bias[b] = swp ? 0.0f : ep.bias_at(pi);
  }
  const int d_sq = (int)(swp ? g.d_si : g.d_sj);  // < 2^22 (checked by the dispatcher)
  const int64_t corner = (int64_t)(q0 + wq * WTQ) * d_sq + (p0 + wp * WTP);
  char *Dw = (char *)g.D + (g.d_sb * bt + corner) * 2;
  const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)Dw, 0, tile_window_bytes(d_sq, NP, NQ, corner, 2), 0x00020000);
  const int voff = ((4 * gsel + odd) * d_sq + (lr & ~1)) * 2;
  auto value = [&](float accf, int b) {
    float y = (swp ? q_scale * p_scale[b] : p_scale[b] * q_scale) * accf + p_bias[b];
    if (ACT == ACT_RELU) y = y > 0.0f ? y : 0.0f;
    else if (ACT == ACT_GELU) y = gelu_tanh(y);
    return y * ep.sd;
  };
#pragma unroll
  for (int a = 0; a < TQ; a++)
#pragma unroll
    for (int k = 0; k < 8; k++) {
      const int soff = (a * 32 + 8 * (k >> 1) + 2 * (k & 1)) * d_sq * 2;  // uniform: row 2k of tile a
#pragma unroll
      for (int b = 0; b < TP; b++) {
        const float fa = KIND == KIND_I8 ? (float)to_bits(acc[a][b][2 * k]) : bits2f((uint32_t)to_bits(acc[a][b][2 * k]));
        const float fb = KIND == KIND_I8 ? (float)to_bits(acc[a][b][2 * k + 1]) : bits2f((uint32_t)to_bits(acc[a][b][2 * k + 1]));
        const float ya = value(fa, b), yb = value(fb, b);
        // even lanes keep row 2k and need the neighbour's row-2k value; odd lanes the other way round
        const float mine = odd ? yb : ya, give = odd ? ya : yb;
        const float got = bits2f((uint32_t)__builtin_amdgcn_mov_dpp((int)f2bits(give), 0xB1 /* quad_perm [1,0,3,2] */, 0xF, 0xF, true));
        const float lo = odd ? got : mine, hi = odd ? mine : got;
        const uint32_t pk = DT == 0 ? pack_bf16x2(lo, hi) : pack_f16x2(lo, hi);
        __builtin_amdgcn_raw_buffer_store_b32((int)pk, rs, voff, soff + b * 64, 0);
      }
    }
}

// Epilogue dispatch: the fast paths for the common configurations on tiles that are complete along
// P (columns past the end of D are dropped by the store window, so a ragged token count keeps the
// fast path), the general path for the rest.  All conditions are workgroup-uniform.
template <int KIND, int WP, int WQ, int WTP, int WTQ, class AccV>
__device__ __forceinline__ void mfma_store_tile(const MfmaParams &prm, AccV (&acc)[WTQ / 32][WTP / 32],
                                                int *lds_words, size_t lds_bytes, int p0, int q0, int NP,
                                                int NQ, int bt) {
  const GemmArgs &g = prm.g;
  const bool swp = prm.swapped != 0;
  const int64_t d_sq = swp ? g.d_si : g.d_sj;
  const bool full = p0 + WP * WTP <= NP;  // along Q the store window cuts the tile
  const int dbytes = (g.d_type == CUDA_R_32F || g.d_type == CUDA_R_32I) ? 4 : (g.d_type == CUDA_R_8I ? 1 : 2);
  // columns of the tile start 16-byte aligned and the lane offsets fit 32 bits
  const bool aligned = (((uintptr_t)g.D) & 15) == 0 && ((d_sq * dbytes) & 15) == 0 &&
                       ((g.d_sb * dbytes) & 15) == 0 && d_sq < (1 << 22);
  if constexpr (KIND == KIND_I8) {
    if (g.int_scale && full && aligned && g.alpha_mode != VECTOR_DEV && g.beta_mode == SCALAR_VALUE &&
        g.beta_val.i == 0) {
      const int ialpha = g.alpha_mode == SCALAR_VALUE ? g.alpha_val.i : *(const int32_t *)g.alpha_ptr;
      mfma_store_tile_i32<WP, WQ, WTP, WTQ>(prm, acc, p0, q0, NP, NQ, bt, ialpha);
      return;
    }
  }
  if (!g.int_scale && full && aligned && g.beta_mode == SCALAR_VALUE && g.beta_val.f == 0.0f &&
      (g.d_type == CUDA_R_16BF || g.d_type == CUDA_R_16F || g.d_type == CUDA_R_32F)) {
    const int dt = g.d_type == CUDA_R_16BF ? 0 : (g.d_type == CUDA_R_16F ? 1 : 2);
    // vectors that run along Q need the LDS-staged form
    const bool q_vec = swp ? (g.alpha_mode == VECTOR_DEV || g.a_scale_mode == SCALE_OUTER_VEC || g.bias != nullptr)
                           : (g.b_scale_mode == SCALE_OUTER_VEC);
    if (!q_vec && dt != 2) {
#define ZLUDA_EPI_D(ACT_, DT_) mfma_store_tile_f16_direct<KIND, WP, WQ, WTP, WTQ, ACT_, DT_>(prm, acc, p0, q0, NP, NQ, bt)
      if (dt == 0) {
        if (g.act == ACT_GELU) ZLUDA_EPI_D(ACT_GELU, 0);
        else if (g.act == ACT_RELU) ZLUDA_EPI_D(ACT_RELU, 0);
        else ZLUDA_EPI_D(ACT_NONE, 0);
      } else {
        if (g.act == ACT_GELU) ZLUDA_EPI_D(ACT_GELU, 1);
        else if (g.act == ACT_RELU) ZLUDA_EPI_D(ACT_RELU, 1);
        else ZLUDA_EPI_D(ACT_NONE, 1);
      }
#undef ZLUDA_EPI_D
      return;
    }
#define ZLUDA_EPI(ACT_, DT_) mfma_store_tile_f<KIND, WP, WQ, WTP, WTQ, ACT_, DT_>(prm, acc, lds_words, p0, q0, NP, NQ, bt)
    if (dt == 0) {
      if (g.act == ACT_GELU) ZLUDA_EPI(ACT_GELU, 0);
      else if (g.act == ACT_RELU) ZLUDA_EPI(ACT_RELU, 0);
      else ZLUDA_EPI(ACT_NONE, 0);
    } else if (dt == 1) {
      if (g.act == ACT_GELU) ZLUDA_EPI(ACT_GELU, 1);
      else if (g.act == ACT_RELU) ZLUDA_EPI(ACT_RELU, 1);
      else ZLUDA_EPI(ACT_NONE, 1);
    } else {
      if (g.act == ACT_GELU) ZLUDA_EPI(ACT_GELU, 2);
      else if (g.act == ACT_RELU) ZLUDA_EPI(ACT_RELU, 2);
      else ZLUDA_EPI(ACT_NONE, 2);
    }
#undef ZLUDA_EPI
    return;
  }
  mfma_store_tile_general<KIND, WP, WQ, WTP, WTQ>(prm, acc, lds_words, lds_bytes, p0, q0, NP, NQ, bt);
}

} // namespace zluda_amd
