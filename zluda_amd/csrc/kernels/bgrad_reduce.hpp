// Bias-gradient epilogues (CUBLASLT_EPILOGUE_BGRADA / BGRADB): the sum over the GEMM's K dimension of
// each row of op(A) (length M) or each column of op(B) (length N), written to the bias buffer in the
// bias data type.  A second, small kernel behind the matmul on the same stream: it reads the operand
// once more (HBM bound), D is computed by the matmul kernel as with the DEFAULT epilogue.
#pragma once
#include "numeric.hpp"

namespace zluda_amd {

struct BgradParams {
  const void *src;        // A or B
  uint32_t type;          // its cudaDataType
  int32_t rows, K, batch; // `rows` sums of K elements per batch
  int64_t s_row, s_k, s_b; // element strides: row index, K, batch
  void *out;
  uint32_t out_type;
  int64_t out_sb;
};

// K has the smaller stride: one workgroup per row, lanes run along K; grid (rows, batch)
__global__ __launch_bounds__(256) void bgrad_rows_kernel(BgradParams prm) {
  __shared__ float part_f[4];
  __shared__ int32_t part_i[4];
  const int r = blockIdx.x, bt = blockIdx.y;
  const int64_t base = (int64_t)bt * prm.s_b + (int64_t)r * prm.s_row;
  float s = 0.0f;
  int32_t si = 0;
  const bool ints = prm.type == CUDA_R_8I;  // summed exactly in int32, converted once
  for (int k = threadIdx.x; k < prm.K; k += 256) {
    if (ints) si += ((const int8_t *)prm.src)[base + (int64_t)k * prm.s_k];
    else s += load_elem(prm.src, prm.type, base + (int64_t)k * prm.s_k);
  }
#pragma unroll
  for (int off = 32; off; off >>= 1) {
    si += __shfl_xor(si, off, 64);
    s += __shfl_xor(s, off, 64);
  }
  if ((threadIdx.x & 63) == 0) {
    part_f[threadIdx.x >> 6] = s;
    part_i[threadIdx.x >> 6] = si;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    const float total = ints ? (float)(part_i[0] + part_i[1] + part_i[2] + part_i[3]) : (part_f[0] + part_f[1]) + (part_f[2] + part_f[3]);
    store_elem(prm.out, prm.out_type, (int64_t)bt * prm.out_sb + r, total);
  }
}

// the row index has the smaller stride: one thread per row, every step of the K walk reads
// consecutive rows; grid (ceil(rows / 256), batch)
__global__ __launch_bounds__(256) void bgrad_cols_kernel(BgradParams prm) {
  const int r = blockIdx.x * 256 + threadIdx.x, bt = blockIdx.y;
  if (r >= prm.rows) return;
  const int64_t base = (int64_t)bt * prm.s_b + (int64_t)r * prm.s_row;
  float s = 0.0f;
  int32_t si = 0;
  const bool ints = prm.type == CUDA_R_8I;
  for (int k = 0; k < prm.K; k++) {
    if (ints) si += ((const int8_t *)prm.src)[base + (int64_t)k * prm.s_k];
    else s += load_elem(prm.src, prm.type, base + (int64_t)k * prm.s_k);
  }
  store_elem(prm.out, prm.out_type, (int64_t)bt * prm.out_sb + r, ints ? (float)si : s);
}

} // namespace zluda_amd
