// Second, element-wise pass of the epilogues that keep or use the GELU input
// (cuda_types/src/cublaslt.rs:4601-4660; the aux attributes :4182-4236):
//   GELU_AUX[_BIAS]  the GEMM kernel has written x = alpha * op(A) op(B) + beta * C (+ bias) into the aux matrix;
//                    this pass writes D = gelu(x) * d_scale
//   DGELU[_BGRAD]    the GEMM kernel has written y = alpha * op(A) op(B) + beta * C into D; this pass turns it into
//                    D = y * gelu'(aux) and, for _BGRAD, puts the sums of D's rows into the bias buffer
// aux is a matrix of D's type, shape and order.  Both passes see the value the first pass rounded to that type
// (a 16- or 32-bit float type; the planner admits no other here), so D can differ from a single-pass result by
// one more rounding of that type.
#pragma once
#include "numeric.hpp"

namespace zluda_amd {

// d/dx of the tanh form of GELU
__device__ __forceinline__ float dgelu_tanh(float x) {
  const float k0 = 0.7978845608028654f, k1 = 0.044715f;
  const float u = k0 * (x + k1 * x * x * x);
  // tanh(u) = 1 - 2 / (1 + exp(2u)); exp(2u) = inf gives 1, 0 gives -1
  const float t = 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(2.0f * 1.4426950408889634f * u));
  return 0.5f * (1.0f + t) + 0.5f * x * (1.0f - t * t) * k0 * (1.0f + 3.0f * k1 * x * x);
}

// grid (ceil(M * N / 256), batch): one element per thread, consecutive threads along D's contiguous index
__global__ __launch_bounds__(256) void aux_gelu_kernel(GemmArgs g) {
  const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x, bt = blockIdx.y;
  if (e >= (int64_t)g.M * g.N) return;
  const bool col = g.d_si == 1;
  const int64_t i = col ? e % g.M : e / g.N, j = col ? e / g.M : e % g.N;
  const float sd = g.d_scale ? *(const float *)g.d_scale : 1.0f;
  const float x = load_elem(g.aux, g.d_type, g.aux_sb * bt + i * g.aux_si + j * g.aux_sj);
  store_elem(g.D, g.d_type, g.d_sb * bt + i * g.d_si + j * g.d_sj, gelu_tanh(x) * sd);
}

// grid (ceil(M / RB), batch), 256 threads: a workgroup owns RB rows of D and walks all N columns; the lanes
// run along D's contiguous index (64 rows x 4 column phases for a column-major D, 4 rows x 64 column phases for
// a row-major one), so that the row sums of _BGRAD end in one small LDS reduction.
__global__ __launch_bounds__(256) void aux_dgelu_kernel(GemmArgs g) {
  __shared__ float part[256];
  const int t = threadIdx.x;
  const int64_t bt = blockIdx.y;
  const bool col = g.d_si == 1;
  const int rb = col ? 64 : 4, cb = col ? 4 : 64;            // rows per workgroup, column phases
  const int r = col ? t & 63 : t >> 6, c = col ? t >> 6 : t & 63;
  const int64_t i = (int64_t)blockIdx.x * rb + r;
  float sum = 0.0f;
  if (i < g.M) {
    for (int64_t j = c; j < g.N; j += cb) {
      const int64_t didx = g.d_sb * bt + i * g.d_si + j * g.d_sj;
      const float y = load_elem(g.D, g.d_type, didx) * dgelu_tanh(load_elem(g.aux, g.d_type, g.aux_sb * bt + i * g.aux_si + j * g.aux_sj));
      store_elem(g.D, g.d_type, didx, y);
      sum += y;
    }
  }
  if (!g.aux_bgrad) return;
  part[r * cb + c] = sum;
  __syncthreads();
  if (c == 0 && i < g.M) {
    float s = 0.0f;
    for (int k = 0; k < cb; k++) s += part[r * cb + k];
    store_elem(g.bgrad, g.bias_type, i + g.bias_sb * bt, s);
  }
}

} // namespace zluda_amd
