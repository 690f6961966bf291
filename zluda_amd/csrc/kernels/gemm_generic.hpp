// Generic LDS-tiled GEMM: any order / transpose / supported element type.  This is the
// correctness net under the MFMA kernels (odd alignments, M- or N-contiguous operands, fp32/fp16/
// bf16 inputs); it is not tuned.  64x64 output tile per 256-thread workgroup, 4x4 per thread.
#pragma once
#include "numeric.hpp"

namespace zluda_amd {

constexpr int GEN_T = 64;  // tile edge
constexpr int GEN_K = 16;  // K per step

template <bool INT_ACC>
__global__ __launch_bounds__(256) void gemm_generic_kernel(GemmArgs g) {
  using acc_t = typename std::conditional<INT_ACC, int32_t, float>::type;
  __shared__ acc_t As[GEN_K][GEN_T + 1];
  __shared__ acc_t Bs[GEN_K][GEN_T + 1];

  const int t = threadIdx.x;
  const int bt = blockIdx.z;
  const int i0 = blockIdx.x * GEN_T, j0 = blockIdx.y * GEN_T;
  const int64_t aoff = g.a_sb * bt, boff = g.b_sb * bt;
  const int KB = g.K / 32;
  const uint8_t *sa_blk = g.a_scale_mode == SCALE_BLOCK32_UE8M0
                              ? (const uint8_t *)g.a_scale + (int64_t)bt * g.M * KB : nullptr;
  const uint8_t *sb_blk = g.b_scale_mode == SCALE_BLOCK32_UE8M0
                              ? (const uint8_t *)g.b_scale + (int64_t)bt * g.N * KB : nullptr;

  // thread -> (row, k) of the staging copy; k fastest when the operand is K-contiguous
  const bool a_kfast = g.a_sk == 1, b_kfast = g.b_sk == 1;

  acc_t acc[4][4];
#pragma unroll
  for (int a = 0; a < 4; a++)
#pragma unroll
    for (int b = 0; b < 4; b++) acc[a][b] = 0;

  const int ti = (t & 15) * 4, tj = (t >> 4) * 4;

  for (int k0 = 0; k0 < g.K; k0 += GEN_K) {
#pragma unroll
    for (int r = 0; r < 4; r++) {
      int e = t + 256 * r;  // 0..1023
      int kk = a_kfast ? (e & 15) : (e >> 6);
      int ii = a_kfast ? (e >> 4) : (e & 63);
      int i = i0 + ii, k = k0 + kk;
      acc_t v = 0;
      if (i < g.M && k < g.K) {
        int64_t idx = aoff + (int64_t)i * g.a_si + (int64_t)k * g.a_sk;
        if (INT_ACC) v = (acc_t)((const int8_t *)g.A)[idx];
        else {
          float f = load_elem(g.A, g.a_type, idx);
          if (sa_blk) f *= dec_ue8m0(sa_blk[(int64_t)i * KB + (k >> 5)]);
          v = (acc_t)f;
        }
      }
      As[kk][ii] = v;
      kk = b_kfast ? (e & 15) : (e >> 6);
      int jj = b_kfast ? (e >> 4) : (e & 63);
      int j = j0 + jj;
      k = k0 + kk;
      v = 0;
      if (j < g.N && k < g.K) {
        int64_t idx = boff + (int64_t)k * g.b_sk + (int64_t)j * g.b_sj;
        if (INT_ACC) v = (acc_t)((const int8_t *)g.B)[idx];
        else {
          float f = load_elem(g.B, g.b_type, idx);
          if (sb_blk) f *= dec_ue8m0(sb_blk[(int64_t)j * KB + (k >> 5)]);
          v = (acc_t)f;
        }
      }
      Bs[kk][jj] = v;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GEN_K; kk++) {
      acc_t av[4], bv[4];
#pragma unroll
      for (int a = 0; a < 4; a++) av[a] = As[kk][ti + a];
#pragma unroll
      for (int b = 0; b < 4; b++) bv[b] = Bs[kk][tj + b];
#pragma unroll
      for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < 4; b++) acc[a][b] += av[a] * bv[b];
    }
    __syncthreads();
  }

  Epilogue ep(g, bt);
#pragma unroll
  for (int b = 0; b < 4; b++)
#pragma unroll
    for (int a = 0; a < 4; a++) {
      int i = i0 + ti + a, j = j0 + tj + b;
      if (i < g.M && j < g.N) {
        if (g.int_scale) ep.store_int(i, j, (int32_t)acc[a][b]);
        else ep.store_f(i, j, (float)acc[a][b]);
      }
    }
}

} // namespace zluda_amd
