// Skinny (<= 32 tokens) W8A8 decode GEMM: an HBM-bound streaming kernel.
//
//   W : R rows x K int8, K-contiguous (the weight matrix, 10s of MB, read exactly once)
//   X : T <= 32 rows x K int8, K-contiguous (the activations, a few 10s of KB, L2 resident)
//   out(r, t) = sum_k W[r][k] * X[t][k]           int32, then the fused float epilogue
//
// A workgroup of NW waves owns one block of 16 weight rows at a time (grid-stride over the row
// blocks).  K is split across the NW waves of the workgroup (split-K inside the workgroup): wave w
// streams K bytes [w*SPW*64, (w+1)*SPW*64) of its 16 rows with 128-bit loads laid out exactly as
// v_mfma_i32_16x16x64_i8 wants its A operand (lane l: row l%16, 16 K-bytes at (l/16)*16), so
// nothing is shuffled between the load and the MFMA.  The activation fragments of the wave's K
// slice live in registers for the whole kernel.  The NW partial 16x16 int32 tiles meet in LDS,
// one wave sums them and applies alpha/scale/bias -> bf16.  The next row block's weights are
// already in flight while the current one is reduced.
#pragma once
#include "gemm_mfma.hpp"

namespace zluda_amd {

struct DecodeParams {
  GemmArgs g;
  int32_t swapped;  // 0: W = op(A) (rows i of D), X = op(B) (tokens j);  1: W = op(B)^T, X = op(A)
  int32_t spw;      // MFMA K-steps (64 bytes of K each) per wave
  int32_t nchunks;  // ceil(spw / STEPS)
  int32_t rows_base, rows_rem;  // stream kernel: rows per workgroup and how many workgroups take one more
  int32_t full_rounds;          // slab kernel: round-robin rounds of one 16-row block per workgroup in front of those rows
};

template <int NW, int STEPS, int NB, bool FULL>
__global__ __launch_bounds__(NW * 64) void decode_w8a8_kernel(DecodeParams prm) {
  __shared__ v4i red[2][NW][NB][64];

  const GemmArgs &g = prm.g;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int l16 = lane & 15, g4 = lane >> 4;
  const int bt = blockIdx.y;

  const int R = prm.swapped ? g.N : g.M, T = prm.swapped ? g.M : g.N;
  const int K = g.K;
  const uint8_t *Wg = (const uint8_t *)(prm.swapped ? g.B : g.A) + (prm.swapped ? g.b_sb : g.a_sb) * bt;
  const uint8_t *Xg = (const uint8_t *)(prm.swapped ? g.A : g.B) + (prm.swapped ? g.a_sb : g.b_sb) * bt;
  const int64_t ldw = prm.swapped ? g.b_sj : g.a_si, ldx = prm.swapped ? g.a_si : g.b_sj;

  const int nrb = (R + 15) >> 4;
  const int kw0 = wave * prm.spw * 64 + g4 * 16;  // this lane's first K byte

  // activation fragments of this wave's K slice (single-chunk case: loaded once)
  v4i xf[NB][STEPS];
  auto xload = [&](int chunk) {
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
      const uint8_t *xr = Xg + (int64_t)min(nb * 16 + l16, T - 1) * ldx;
#pragma unroll
      for (int s = 0; s < STEPS; s++) {
        const int k = kw0 + (chunk * STEPS + s) * 64;
        const bool ok = FULL || (chunk * STEPS + s < prm.spw && k < K);
        xf[nb][s] = ok ? *(const v4i *)(xr + k) : v4i{0, 0, 0, 0};
      }
    }
  };

  v4i w0[STEPS], w1[STEPS];
  auto wload = [&](v4i(&wr)[STEPS], int rb, int chunk) {
    const uint8_t *wrow = Wg + (int64_t)min(rb * 16 + l16, R - 1) * ldw;
#pragma unroll
    for (int s = 0; s < STEPS; s++) {
      const int k = kw0 + (chunk * STEPS + s) * 64;
      const bool ok = FULL || (chunk * STEPS + s < prm.spw && k < K);
      wr[s] = ok ? __builtin_nontemporal_load((const v4i *)(wrow + k)) : v4i{0, 0, 0, 0};
    }
  };

  Epilogue ep(g, bt);
  int it = 0;
  auto reduce_store = [&](int rb, v4i(&acc)[NB]) {
    const int buf = it & 1;
#pragma unroll
    for (int nb = 0; nb < NB; nb++) red[buf][wave][nb][lane] = acc[nb];
    __syncthreads();
    if (wave == (it % NW)) {
#pragma unroll
      for (int nb = 0; nb < NB; nb++) {
        v4i s = red[buf][0][nb][lane];
#pragma unroll
        for (int w = 1; w < NW; w++) s += red[buf][w][nb][lane];
        const int tok = nb * 16 + l16;
#pragma unroll
        for (int v = 0; v < 4; v++) {
          const int row = rb * 16 + g4 * 4 + v;
          if (row < R && tok < T) {
            const int i = prm.swapped ? tok : row, j = prm.swapped ? row : tok;
            if (g.int_scale) ep.store_int(i, j, s[v]);
            else ep.store_f(i, j, (float)s[v]);
          }
        }
      }
    }
    it++;
  };

  auto compute = [&](v4i(&wr)[STEPS], v4i(&acc)[NB]) {
#pragma unroll
    for (int s = 0; s < STEPS; s++)
#pragma unroll
      for (int nb = 0; nb < NB; nb++)
        acc[nb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wr[s], xf[nb][s], acc[nb], 0, 0, 0);
  };

  const int stride = gridDim.x;
  int rb = blockIdx.x;

  if (prm.nchunks == 1) {
    xload(0);
    if (rb < nrb) wload(w0, rb, 0);
    while (rb < nrb) {
      int nxt = rb + stride;
      if (nxt < nrb) wload(w1, nxt, 0);
      {
        v4i acc[NB];
#pragma unroll
        for (int nb = 0; nb < NB; nb++) acc[nb] = v4i{0, 0, 0, 0};
        compute(w0, acc);
        reduce_store(rb, acc);
      }
      rb = nxt;
      if (rb >= nrb) break;
      nxt = rb + stride;
      if (nxt < nrb) wload(w0, nxt, 0);
      {
        v4i acc[NB];
#pragma unroll
        for (int nb = 0; nb < NB; nb++) acc[nb] = v4i{0, 0, 0, 0};
        compute(w1, acc);
        reduce_store(rb, acc);
      }
      rb = nxt;
    }
  } else {
    // long K: the activation fragments no longer fit in registers; reload them per chunk
    for (; rb < nrb; rb += stride) {
      v4i acc[NB];
#pragma unroll
      for (int nb = 0; nb < NB; nb++) acc[nb] = v4i{0, 0, 0, 0};
      for (int ch = 0; ch < prm.nchunks; ch++) {
        wload(w0, rb, ch);
        xload(ch);
        compute(w0, acc);
      }
      reduce_store(rb, acc);
    }
  }
}

} // namespace zluda_amd
