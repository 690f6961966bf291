// Kernel-level description of one matmul, shared by the host planner and the device kernels.
//
// The planner (planner.cpp) lowers the cuBLASLt-level problem (orders, transposes, leading
// dimensions) to plain element strides, so that every kernel addresses
//     op(A)(i,k) = A[i*a_si + k*a_sk],  op(B)(k,j) = B[k*b_sk + j*b_sj],
//     C(i,j)     = C[i*c_si + j*c_sj],  D(i,j)     = D[i*d_si + j*d_sj]
// (strides in elements; FP4 elements are half bytes).  Row-major versus column-major and N versus T
// therefore never reach the device code.
#pragma once
#include <stdint.h>

namespace zluda_amd {

enum ScalarMode : int32_t { SCALAR_VALUE = 0, SCALAR_DEV = 1, VECTOR_DEV = 2 };
enum ScaleMode : int32_t { SCALE_NONE = 0, SCALE_SCALAR = 1, SCALE_OUTER_VEC = 2, SCALE_BLOCK32_UE8M0 = 3 };
enum Activation : int32_t { ACT_NONE = 0, ACT_RELU = 1, ACT_GELU = 2 };

struct GemmArgs {
  const void *A, *B, *C;
  void *D;
  int32_t M, N, K, batch;
  int64_t a_si, a_sk, a_sb;
  int64_t b_sk, b_sj, b_sb;
  int64_t c_si, c_sj, c_sb;
  int64_t d_si, d_sj, d_sb;
  uint32_t a_type, b_type, c_type, d_type; // cudaDataType numbers
  int32_t int_scale;                       // 1: alpha/beta/C/D are int32, pure integer epilogue
  int32_t alpha_mode, beta_mode;           // ScalarMode
  union { float f; int32_t i; } alpha_val, beta_val;
  const void *alpha_ptr, *beta_ptr;        // device, when mode != SCALAR_VALUE
  int64_t alpha_sb;                        // batch stride of the alpha vector
  const void *a_scale, *b_scale, *c_scale, *d_scale;
  int32_t a_scale_mode, b_scale_mode;      // ScaleMode (c/d: scalar when the pointer is set)
  const void *bias;                        // device, indexed by the row i of D
  uint32_t bias_type;
  int64_t bias_sb;
  int32_t act;                             // Activation
  // bias-gradient epilogues: the K sums of op(A)'s rows (bgrad_src 1, M values) or of op(B)'s columns
  // (2, N values) go to `bgrad` in bias_type, batches bias_sb apart; `bias` is NULL then
  void *bgrad;
  int32_t bgrad_src;
  // GELU with its input kept (aux_mode 1: aux = x, D = gelu(x)) and its gradient (aux_mode 2: D = D * gelu'(aux),
  // aux_bgrad: the row sums of that D go to `bgrad`).  Run as a second, element-wise pass behind the GEMM
  // kernel; aux is a matrix of D's type and order, strides in elements.
  void *aux;
  int64_t aux_si, aux_sj, aux_sb;
  int32_t aux_mode, aux_bgrad;
};

} // namespace zluda_amd
