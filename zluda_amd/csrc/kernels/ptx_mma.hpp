// PTX `mma.sync.aligned` m16n8k32 (s8) and m16n8k16 (f16, bf16) on gfx950 matrix cores.
//
// The reference lowers these instructions to per-lane device functions that gather a row and two
// columns with ds_bpermute and run 4 x 8 dot products per lane, written for 32-wide waves
// (ptx/lib/zluda_ptx_impl.cpp:979-1079; names built in
// ptx/src/pass/replace_instructions_with_functions.rs:468-486).  gfx950 only has 64-wide waves and has
// MFMA, so here a wavefront carries two warps (lanes 0-31 and 32-63) and ONE MFMA computes both warps'
// products:
//
//   v_mfma_i32_16x16x64_i8 / v_mfma_f32_16x16x32_{f16,bf16}: src0 lane l = row l%16, src1 lane l =
//   column l%16, both with the 16 bytes of K-group l/16 (4 groups); D lane l = column l%16, rows
//   4*(l/16) .. +3.
//
//   K' = [ K of warp 0 | K of warp 1 ]          (groups 0,1 | 2,3)
//   src0 row  n' = 8*w + n :  column n of warp w's B in warp w's half of K', zeros in the other half
//   src1 col  m            :  row m of warp 0's A | row m of warp 1's A
//   D'[8*w + n][m] = (A_w * B_w)[m][n]
//
// A dot product does not care about the order of K as long as both operands agree, so a K-group is
// made of what two neighbouring lanes of a quad already hold: group (w, h) = lanes t = 2h, 2h+1 of
// each quad of warp w, each giving its two registers of the row (column).  PTX fragment layout, E
// elements per register (4 x s8, 2 x f16), lane = 4*g + t:
//   A register r: row g + 8*(r&1), columns t*E .. +E-1 (+ 4E if r >= 2)
//   B register r: rows t*E .. +E-1 (+ 4E if r == 1), column g
//   C/D register r: row g + 8*(r>>1), column 2*t + (r&1)
//
// Data movement per wavefront (two mma instructions' worth): 4 ds_permute for A, 2 ds_permute (and two
// DPP rotates) for B, 4 ds_permute for D -- each ds_permute is a permutation of the 64 lanes in which the SENDER picks
// which of its registers goes out, which halves the count against pulling (a lane holds two rows of
// A but an MFMA lane wants one) -- plus one MFMA, against 16 ds_bpermute and 32 dot instructions per
// warp in the per-lane form.
//
// Both warps of the wavefront must arrive together for that (EXEC all ones).  When they do not -- a
// 32-thread block, or the two warps on different sides of a branch -- the per-lane form below runs
// instead; it only talks to lanes of its own warp, which `.aligned` guarantees to be there.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace zluda_amd {
namespace ptx_mma {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

enum { S8 = 0, F16 = 1, BF16 = 2 };

__device__ __forceinline__ int lane_id() { return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); }
__device__ __forceinline__ uint32_t pull(int src_lane, uint32_t v) { return (uint32_t)__builtin_amdgcn_ds_bpermute(src_lane << 2, (int)v); }
__device__ __forceinline__ uint32_t push(int dst_lane, uint32_t v) { return (uint32_t)__builtin_amdgcn_ds_permute(dst_lane << 2, (int)v); }

template <int KIND> struct Acc { typedef f32x4 type; };
template <> struct Acc<S8> { typedef i32x4 type; };

__device__ __forceinline__ float elem_f16(uint32_t reg, int e) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(reg >> (16 * e))); }
__device__ __forceinline__ float elem_bf16(uint32_t reg, int e) { return __builtin_bit_cast(float, (reg >> (16 * e)) << 16); }

// c + dot(x, y) over the E elements of one register pair
template <int KIND, typename T>
__device__ __forceinline__ T dot1(uint32_t x, uint32_t y, T c) {
  if constexpr (KIND == S8) {
#pragma unroll
    for (int e = 0; e < 4; e++) c += (T)(int8_t)(x >> (8 * e)) * (T)(int8_t)(y >> (8 * e));
  } else if constexpr (KIND == F16) {
#pragma unroll
    for (int e = 0; e < 2; e++) c = __builtin_fmaf(elem_f16(x, e), elem_f16(y, e), c);
  } else {
#pragma unroll
    for (int e = 0; e < 2; e++) c = __builtin_fmaf(elem_bf16(x, e), elem_bf16(y, e), c);
  }
  return c;
}

// One warp on its own: lane (g, t) computes D[g][2t], D[g][2t+1], D[g+8][2t], D[g+8][2t+1] from rows
// g, g+8 of A (held by the 4 lanes of its own quad) and columns 2t, 2t+1 of B (quads 2t, 2t+1).
template <int KIND>
__device__ __forceinline__ typename Acc<KIND>::type mma_per_lane(u32x4 a, u32x2 b, typename Acc<KIND>::type c, int lane) {
  const int base = lane & 32, g = (lane >> 2) & 7, t = lane & 3;
  auto d0 = c[0], d1 = c[1], d2 = c[2], d3 = c[3];
#pragma unroll
  for (int hh = 0; hh < 2; hh++)
#pragma unroll
    for (int tt = 0; tt < 4; tt++) {
      const uint32_t row_lo = pull(base + 4 * g + tt, a[2 * hh]), row_hi = pull(base + 4 * g + tt, a[2 * hh + 1]);
      const uint32_t col_0 = pull(base + 8 * t + tt, b[hh]), col_1 = pull(base + 8 * t + 4 + tt, b[hh]);
      d0 = dot1<KIND>(row_lo, col_0, d0);
      d1 = dot1<KIND>(row_lo, col_1, d1);
      d2 = dot1<KIND>(row_hi, col_0, d2);
      d3 = dot1<KIND>(row_hi, col_1, d3);
    }
  return {d0, d1, d2, d3};
}

// Two warps at once through one MFMA (every lane of the wavefront active).
template <int KIND>
__device__ __forceinline__ typename Acc<KIND>::type mma_wave64(u32x4 a, u32x2 b, typename Acc<KIND>::type c, int lane) {
  typedef typename Acc<KIND>::type acc_t;
  // this lane as a PTX lane ...
  const int w = lane >> 5, g = (lane >> 2) & 7, t = lane & 3, t_odd = t & 1;
  // ... and as an MFMA lane: row/column index, K-group, upper half of the 16 rows
  const int idx = lane & 15, kq = lane >> 4, hi = idx >> 3;

  // A -> src1.  Send p: a lane with even t sends register (p&1) + 2*(p>>1), one with odd t the other
  // row's, to MFMA lane (column g + 8*(which row), K-group 2w + t/2): the two lanes that share a
  // K-group never aim at the same column.  What arrives in send p belongs at 32-bit position
  // 2*(hi ^ (p&1)) + (p>>1) of the receiver's 16 bytes.
  uint32_t ta[4];
#pragma unroll
  for (int p = 0; p < 4; p++) {
    const uint32_t val = t_odd ? a[(1 - (p & 1)) + 2 * (p >> 1)] : a[(p & 1) + 2 * (p >> 1)];
    ta[p] = push(g + 8 * (t_odd ^ (p & 1)) + 16 * (2 * w + (t >> 1)), val);
  }
  const i32x4 cols = {(int)(hi ? ta[1] : ta[0]), (int)(hi ? ta[3] : ta[2]), (int)(hi ? ta[0] : ta[1]), (int)(hi ? ta[2] : ta[3])};

  // B -> src0.  MFMA row 8*w + n takes column n of warp w, and only in that warp's K-groups; the other
  // half of the MFMA lanes (row of the other warp) holds zeros.  Lanes with even t send their two
  // registers to the MFMA lane that uses them (row 8w + g, K-group 2w + t/2), lanes with odd t to
  // its idle neighbour 8 lanes further in the same row of 16, from where a DPP rotate brings them
  // over: 2 permutations instead of 4.
  const int dst_b = ((8 * w + g) ^ (t_odd << 3)) + 16 * (2 * w + (t >> 1));
  const uint32_t e0 = push(dst_b, b[0]), e1 = push(dst_b, b[1]);
  const uint32_t o0 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)e0, 0x128, 0xf, 0xf, false);  // row_ror:8
  const uint32_t o1 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)e1, 0x128, 0xf, 0xf, false);
  const bool mine = (idx >> 3) == (kq >> 1);
  const i32x4 rows = {mine ? (int)e0 : 0, mine ? (int)e1 : 0, mine ? (int)o0 : 0, mine ? (int)o1 : 0};

  acc_t acc;
  if constexpr (KIND == S8) acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(rows, cols, i32x4{0, 0, 0, 0}, 0, 0, 0);
  else if constexpr (KIND == F16)
    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, rows), __builtin_bit_cast(f16x8, cols), f32x4{0, 0, 0, 0}, 0, 0, 0);
  else
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, rows), __builtin_bit_cast(bf16x8, cols), f32x4{0, 0, 0, 0}, 0, 0, 0);

  // D' -> D.  MFMA lane (m = idx, rq = kq) holds D_w[m][4*(rq&1) + v], w = rq/2, v = 0..3.  Send p: value
  // v = 2*(hi ^ (p&1)) + (p>>1) goes to PTX lane (w, g = m%8, t = 2*(rq&1) + v/2), where it is
  // register 2*((t&1) ^ (p&1)) + (p>>1).
  uint32_t td[4];
#pragma unroll
  for (int p = 0; p < 4; p++) {
    const auto val = hi ? acc[2 * (1 - (p & 1)) + (p >> 1)] : acc[2 * (p & 1) + (p >> 1)];
    td[p] = push(32 * (kq >> 1) + 4 * (idx & 7) + 2 * (kq & 1) + (hi ^ (p & 1)), __builtin_bit_cast(uint32_t, val));
  }
  typedef decltype(acc[0] + acc[0]) elem_t;
  acc_t d;
  d[0] = __builtin_bit_cast(elem_t, t_odd ? td[1] : td[0]);
  d[1] = __builtin_bit_cast(elem_t, t_odd ? td[3] : td[2]);
  d[2] = __builtin_bit_cast(elem_t, t_odd ? td[0] : td[1]);
  d[3] = __builtin_bit_cast(elem_t, t_odd ? td[2] : td[3]);
  if constexpr (KIND == S8) return __builtin_bit_cast(i32x4, __builtin_bit_cast(u32x4, d) + __builtin_bit_cast(u32x4, c));  // wraps
  else return d + c;
}

template <int KIND>
__device__ __forceinline__ typename Acc<KIND>::type mma_sync(u32x4 a, u32x2 b, typename Acc<KIND>::type c) {
  const int lane = lane_id();
  // wave-uniform: every lane of the wavefront is here
  if (__builtin_amdgcn_read_exec() == ~0ull) return mma_wave64<KIND>(a, b, c, lane);
  return mma_per_lane<KIND>(a, b, c, lane);
}

} // namespace ptx_mma
} // namespace zluda_amd
