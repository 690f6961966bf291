// The second kernel of a split-K matmul (see MfmaParams::splits in gemm_mfma.hpp).
#pragma once
#include "gemm_mfma.hpp"

namespace zluda_amd {

// Sums the partial tiles and applies the full epilogue (any D type,
// C read, vectors).  One thread per 4 consecutive elements along P; grid (ceil(NP / 1024), NQ, batch).
struct SplitKReduceParams {
  GemmArgs g;
  int32_t swapped, splits, acc_is_int;
  int32_t ws_np, ws_nq;  // padded extents of one partial matrix
  const int32_t *ws;
};
__global__ __launch_bounds__(256) void splitk_reduce_kernel(SplitKReduceParams prm) {
  const GemmArgs &g = prm.g;
  const int NP = prm.swapped ? g.N : g.M;
  const int p = (blockIdx.x * 256 + threadIdx.x) * 4, q = blockIdx.y, bt = blockIdx.z;
  if (p >= NP) return;
  const int64_t plane = (int64_t)prm.ws_np * prm.ws_nq;
  const int32_t *src = prm.ws + (int64_t)bt * plane + (int64_t)q * prm.ws_np + p;
  v4i si = *(const v4i *)src;
  float sf[4] = {bits2f((uint32_t)si[0]), bits2f((uint32_t)si[1]), bits2f((uint32_t)si[2]), bits2f((uint32_t)si[3])};
  for (int z = 1; z < prm.splits; z++) {
    const v4i t = *(const v4i *)(src + (int64_t)z * g.batch * plane);
    si += t;
#pragma unroll
    for (int e = 0; e < 4; e++) sf[e] += bits2f((uint32_t)t[e]);
  }
  Epilogue ep(g, bt);
#pragma unroll
  for (int e = 0; e < 4; e++) {
    if (p + e >= NP) break;
    const int i = prm.swapped ? q : p + e, j = prm.swapped ? p + e : q;
    if (g.int_scale) ep.store_int(i, j, si[e]);
    else ep.store_f(i, j, prm.acc_is_int ? (float)si[e] : sf[e]);
  }
}

} // namespace zluda_amd
