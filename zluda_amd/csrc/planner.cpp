// Problem validation, lowering to strides, and kernel selection.  Host code only.
//
// The accepted surface follows the reference's (zluda_blaslt/src/impl.rs:257-305 for the
// attributes, zluda_common/src/lib.rs:575-630 for the type maps) extended by what the quantized
// path needs: scale pointers/modes, pointer modes, FP4/UE8M0 types.
#include "planner.hpp"

#include <algorithm>
#include <cstdlib>
#include <cstring>

namespace zluda_amd {

static int type_bits(uint32_t t) {
  switch (t) {
  case CUDA_R_32F: case CUDA_R_32I: return 32;
  case CUDA_R_16F: case CUDA_R_16BF: return 16;
  case CUDA_R_8I: case CUDA_R_8F_E4M3: case CUDA_R_8F_E5M2: return 8;
  case CUDA_R_4F_E2M1: return 4;
  default: return 0;
  }
}

static bool is_float_in(uint32_t t) {
  return t == CUDA_R_32F || t == CUDA_R_16F || t == CUDA_R_16BF || t == CUDA_R_8F_E4M3 ||
         t == CUDA_R_8F_E5M2 || t == CUDA_R_4F_E2M1;
}

static uint32_t layout_ok(const zluda_matrix_layout &l) {
  if (l.order != CUBLASLT_ORDER_COL && l.order != CUBLASLT_ORDER_ROW) return CUBLAS_STATUS_NOT_SUPPORTED;
  if (!type_bits(l.type)) return CUBLAS_STATUS_NOT_SUPPORTED;
  if (l.rows == 0 || l.cols == 0) return CUBLAS_STATUS_INVALID_VALUE;
  if (l.rows > 0x7fffffffull || l.cols > 0x7fffffffull) return CUBLAS_STATUS_NOT_SUPPORTED;
  const int64_t lead = l.order == CUBLASLT_ORDER_COL ? (int64_t)l.rows : (int64_t)l.cols;
  if (l.ld < lead) return CUBLAS_STATUS_INVALID_VALUE;
  if (l.batch_count < 1) return CUBLAS_STATUS_INVALID_VALUE;
  return CUBLAS_STATUS_SUCCESS;
}

static int convert_scale_mode(int32_t cuda_mode, const void *ptr, bool dry, int32_t *out) {
  switch (cuda_mode) {
  case CUBLASLT_MATMUL_MATRIX_SCALE_SCALAR_32F: *out = ptr ? SCALE_SCALAR : SCALE_NONE; return 0;
  case CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F: *out = SCALE_OUTER_VEC; return (ptr || dry) ? 0 : 1;
  case CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0: *out = SCALE_BLOCK32_UE8M0; return (ptr || dry) ? 0 : 1;
  default: return 2;
  }
}

uint32_t lower_problem(const zluda_gemm_problem *p, bool dry, Lowered *out) {
  if (!p || !out) return CUBLAS_STATUS_INVALID_VALUE;
  const zluda_matmul_desc &op = p->op;
  const zluda_matrix_layout &a = p->a, &b = p->b, &d = p->d;
  const zluda_matrix_layout &c = p->c;
  uint32_t st;
  if ((st = layout_ok(a)) || (st = layout_ok(b)) || (st = layout_ok(c)) || (st = layout_ok(d))) return st;
  if (op.transa > CUBLAS_OP_C || op.transb > CUBLAS_OP_C) return CUBLAS_STATUS_INVALID_VALUE;
  const bool ta = op.transa != CUBLAS_OP_N, tb = op.transb != CUBLAS_OP_N;

  GemmArgs g;
  memset(&g, 0, sizeof(g));
  const uint64_t M = d.rows, N = d.cols, K = ta ? a.rows : a.cols;
  if ((ta ? a.cols : a.rows) != M) return CUBLAS_STATUS_INVALID_VALUE;
  if ((tb ? b.cols : b.rows) != K) return CUBLAS_STATUS_INVALID_VALUE;
  if ((tb ? b.rows : b.cols) != N) return CUBLAS_STATUS_INVALID_VALUE;
  if (c.rows != M || c.cols != N) return CUBLAS_STATUS_INVALID_VALUE;
  g.M = (int32_t)M; g.N = (int32_t)N; g.K = (int32_t)K;

  const bool a_col = a.order == CUBLASLT_ORDER_COL, b_col = b.order == CUBLASLT_ORDER_COL;
  // op(A)(i,k): stored (r,c) = ta ? (k,i) : (i,k)
  if (!ta) { g.a_si = a_col ? 1 : a.ld; g.a_sk = a_col ? a.ld : 1; }
  else     { g.a_sk = a_col ? 1 : a.ld; g.a_si = a_col ? a.ld : 1; }
  // op(B)(k,j): stored (r,c) = tb ? (j,k) : (k,j)
  if (!tb) { g.b_sk = b_col ? 1 : b.ld; g.b_sj = b_col ? b.ld : 1; }
  else     { g.b_sj = b_col ? 1 : b.ld; g.b_sk = b_col ? b.ld : 1; }
  g.c_si = c.order == CUBLASLT_ORDER_COL ? 1 : c.ld; g.c_sj = c.order == CUBLASLT_ORDER_COL ? c.ld : 1;
  g.d_si = d.order == CUBLASLT_ORDER_COL ? 1 : d.ld; g.d_sj = d.order == CUBLASLT_ORDER_COL ? d.ld : 1;

  g.batch = d.batch_count;
  if (a.batch_count != g.batch || b.batch_count != g.batch || c.batch_count != g.batch)
    return CUBLAS_STATUS_INVALID_VALUE;
  g.a_sb = a.batch_stride; g.b_sb = b.batch_stride; g.c_sb = c.batch_stride; g.d_sb = d.batch_stride;
  if (g.batch > 65535) return CUBLAS_STATUS_NOT_SUPPORTED;

  g.a_type = a.type; g.b_type = b.type; g.c_type = c.type; g.d_type = d.type;

  // ---- compute / scale type ------------------------------------------------------------------
  const uint32_t ct = op.compute_type;
  const bool int_path = ct == CUBLAS_COMPUTE_32I || ct == CUBLAS_COMPUTE_32I_PEDANTIC;
  const bool f32_path = ct == CUBLAS_COMPUTE_32F || ct == CUBLAS_COMPUTE_32F_PEDANTIC ||
                        ct == CUBLAS_COMPUTE_32F_FAST_16F || ct == CUBLAS_COMPUTE_32F_FAST_16BF ||
                        ct == CUBLAS_COMPUTE_32F_FAST_TF32;
  if (!int_path && !f32_path) return CUBLAS_STATUS_NOT_SUPPORTED;
  if (int_path) {
    if (a.type != CUDA_R_8I || b.type != CUDA_R_8I) return CUBLAS_STATUS_NOT_SUPPORTED;
    if (op.scale_type == CUDA_R_32I) {
      if (d.type != CUDA_R_32I || c.type != CUDA_R_32I) return CUBLAS_STATUS_NOT_SUPPORTED;
      if (op.epilogue != CUBLASLT_EPILOGUE_DEFAULT) return CUBLAS_STATUS_NOT_SUPPORTED;
      g.int_scale = 1;
    } else if (op.scale_type == CUDA_R_32F) {
      if (!(d.type == CUDA_R_8I || d.type == CUDA_R_32I || d.type == CUDA_R_16BF ||
            d.type == CUDA_R_16F || d.type == CUDA_R_32F))
        return CUBLAS_STATUS_NOT_SUPPORTED;
    } else return CUBLAS_STATUS_NOT_SUPPORTED;
  } else {
    if (!is_float_in(a.type) || !is_float_in(b.type)) return CUBLAS_STATUS_NOT_SUPPORTED;
    if (op.scale_type != CUDA_R_32F) return CUBLAS_STATUS_NOT_SUPPORTED;
    if (!(d.type == CUDA_R_32F || d.type == CUDA_R_16F || d.type == CUDA_R_16BF ||
          d.type == CUDA_R_8F_E4M3 || d.type == CUDA_R_8F_E5M2))
      return CUBLAS_STATUS_NOT_SUPPORTED;
    // 16/32-bit inputs: both operands of one type (as in cuBLASLt); 8/4-bit floats may mix
    if (type_bits(a.type) >= 16 && a.type != b.type) return CUBLAS_STATUS_NOT_SUPPORTED;
    if (type_bits(a.type) != type_bits(b.type)) return CUBLAS_STATUS_NOT_SUPPORTED;
  }
  if (!g.int_scale && (c.type == CUDA_R_4F_E2M1 || d.type == CUDA_R_4F_E2M1)) return CUBLAS_STATUS_NOT_SUPPORTED;

  // FP4 is packed two per byte along K
  if (a.type == CUDA_R_4F_E2M1 && (g.a_sk != 1 || (a.ld & 1) || (a.batch_stride & 1))) return CUBLAS_STATUS_NOT_SUPPORTED;
  if (b.type == CUDA_R_4F_E2M1 && (g.b_sk != 1 || (b.ld & 1) || (b.batch_stride & 1))) return CUBLAS_STATUS_NOT_SUPPORTED;
  if ((a.type == CUDA_R_4F_E2M1 || b.type == CUDA_R_4F_E2M1) && (K & 1)) return CUBLAS_STATUS_INVALID_VALUE;

  // ---- alpha / beta ------------------------------------------------------------------------
  switch (op.pointer_mode) {
  case CUBLASLT_POINTER_MODE_HOST: g.alpha_mode = SCALAR_VALUE; g.beta_mode = SCALAR_VALUE; break;
  case CUBLASLT_POINTER_MODE_DEVICE: g.alpha_mode = SCALAR_DEV; g.beta_mode = SCALAR_DEV; break;
  case CUBLASLT_POINTER_MODE_DEVICE_VECTOR: g.alpha_mode = VECTOR_DEV; g.beta_mode = VECTOR_DEV; break;
  case CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO: g.alpha_mode = VECTOR_DEV; g.beta_mode = SCALAR_VALUE; break;
  case CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_HOST: g.alpha_mode = VECTOR_DEV; g.beta_mode = SCALAR_VALUE; break;
  default: return CUBLAS_STATUS_INVALID_VALUE;
  }
  g.alpha_sb = op.alpha_vector_batch_stride;
  if (op.pointer_mode == CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO && g.alpha_sb != 0)
    return CUBLAS_STATUS_INVALID_VALUE;  // cuda_types/src/cublaslt.rs:4240-4247
  bool beta_maybe_nonzero = true;
  if (!dry) {
    if (!p->alpha) return CUBLAS_STATUS_INVALID_VALUE;
    if (g.alpha_mode == SCALAR_VALUE) memcpy(&g.alpha_val, p->alpha, 4);
    else g.alpha_ptr = p->alpha;
    if (op.pointer_mode == CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO) {
      g.beta_val.i = 0;
    } else {
      if (!p->beta) return CUBLAS_STATUS_INVALID_VALUE;
      if (g.beta_mode == SCALAR_VALUE) memcpy(&g.beta_val, p->beta, 4);
      else g.beta_ptr = p->beta;
    }
    if (g.beta_mode == SCALAR_VALUE) beta_maybe_nonzero = g.int_scale ? g.beta_val.i != 0 : g.beta_val.f != 0.0f;
    if (beta_maybe_nonzero && !p->C) return CUBLAS_STATUS_INVALID_VALUE;
    if (!p->A || !p->B || !p->D) return CUBLAS_STATUS_INVALID_VALUE;
  }
  g.A = p->A; g.B = p->B; g.C = p->C; g.D = p->D;

  // ---- scales --------------------------------------------------------------------------------
  int r;
  if ((r = convert_scale_mode(op.a_scale_mode, op.a_scale, dry, &g.a_scale_mode)))
    return r == 1 ? CUBLAS_STATUS_INVALID_VALUE : CUBLAS_STATUS_NOT_SUPPORTED;
  if ((r = convert_scale_mode(op.b_scale_mode, op.b_scale, dry, &g.b_scale_mode)))
    return r == 1 ? CUBLAS_STATUS_INVALID_VALUE : CUBLAS_STATUS_NOT_SUPPORTED;
  if (op.c_scale_mode != CUBLASLT_MATMUL_MATRIX_SCALE_SCALAR_32F ||
      op.d_scale_mode != CUBLASLT_MATMUL_MATRIX_SCALE_SCALAR_32F)
    return CUBLAS_STATUS_NOT_SUPPORTED;
  g.a_scale = op.a_scale; g.b_scale = op.b_scale; g.c_scale = op.c_scale; g.d_scale = op.d_scale;
  if (g.int_scale && (g.a_scale_mode || g.b_scale_mode || g.c_scale || g.d_scale))
    return CUBLAS_STATUS_INVALID_VALUE;  // cuda_types/src/cublaslt.rs:4266-4267
  if (g.a_scale_mode == SCALE_BLOCK32_UE8M0 && (int_path || g.a_sk != 1 || (K % 32))) return CUBLAS_STATUS_NOT_SUPPORTED;
  if (g.b_scale_mode == SCALE_BLOCK32_UE8M0 && (int_path || g.b_sk != 1 || (K % 32))) return CUBLAS_STATUS_NOT_SUPPORTED;

  // ---- epilogue ------------------------------------------------------------------------------
  bool has_bias = false;
  switch (op.epilogue) {
  case CUBLASLT_EPILOGUE_DEFAULT: g.act = ACT_NONE; break;
  case CUBLASLT_EPILOGUE_RELU: g.act = ACT_RELU; break;
  case CUBLASLT_EPILOGUE_GELU: g.act = ACT_GELU; break;
  case CUBLASLT_EPILOGUE_BIAS: g.act = ACT_NONE; has_bias = true; break;
  case CUBLASLT_EPILOGUE_RELU_BIAS: g.act = ACT_RELU; has_bias = true; break;
  case CUBLASLT_EPILOGUE_GELU_BIAS: g.act = ACT_GELU; has_bias = true; break;
  // the bias buffer is an output here: sums over K of op(A)'s rows / op(B)'s columns, D as with DEFAULT
  case CUBLASLT_EPILOGUE_BGRADA: g.act = ACT_NONE; g.bgrad_src = 1; break;
  case CUBLASLT_EPILOGUE_BGRADB: g.act = ACT_NONE; g.bgrad_src = 2; break;
  // GELU with its input kept, and GELU's gradient: the GEMM kernel runs without the activation, a second
  // element-wise pass (kernels/aux_epilogue.hpp) finishes D
  case CUBLASLT_EPILOGUE_GELU_AUX: g.act = ACT_NONE; g.aux_mode = 1; break;
  case CUBLASLT_EPILOGUE_GELU_AUX_BIAS: g.act = ACT_NONE; g.aux_mode = 1; has_bias = true; break;
  case CUBLASLT_EPILOGUE_DGELU: g.act = ACT_NONE; g.aux_mode = 2; break;
  case CUBLASLT_EPILOGUE_DGELU_BGRAD: g.act = ACT_NONE; g.aux_mode = 2; g.aux_bgrad = 1; break;
  default: return CUBLAS_STATUS_NOT_SUPPORTED;
  }
  if (g.aux_mode) {
    // the aux matrix has D's type, shape and order (cuda_types/src/cublaslt.rs:4207-4236: its leading dimension
    // is no less than D's rows); both passes go through D's type, which has to be a float type of 16 or 32 bits
    if (g.int_scale || !(d.type == CUDA_R_32F || d.type == CUDA_R_16F || d.type == CUDA_R_16BF)) return CUBLAS_STATUS_NOT_SUPPORTED;
    if (op.epilogue_aux_type != -1 && (uint32_t)op.epilogue_aux_type != d.type) return CUBLAS_STATUS_NOT_SUPPORTED;
    const int64_t lead = d.order == CUBLASLT_ORDER_COL ? M : N, other = d.order == CUBLASLT_ORDER_COL ? N : M;
    if (op.epilogue_aux_ld < lead) return CUBLAS_STATUS_INVALID_VALUE;
    if (g.batch > 1 && op.epilogue_aux_batch_stride < op.epilogue_aux_ld * other && op.epilogue_aux_batch_stride != 0)
      return CUBLAS_STATUS_INVALID_VALUE;
    if (g.batch > 1 && op.epilogue_aux_batch_stride == 0 && g.aux_mode == 1) return CUBLAS_STATUS_NOT_SUPPORTED;  // aliased outputs
    if (g.aux_mode == 2 && g.d_scale) return CUBLAS_STATUS_NOT_SUPPORTED;  // (the scale would have to follow the gradient)
    if (!dry && !op.epilogue_aux) return CUBLAS_STATUS_INVALID_VALUE;
    g.aux = op.epilogue_aux;
    g.aux_si = d.order == CUBLASLT_ORDER_COL ? 1 : op.epilogue_aux_ld;
    g.aux_sj = d.order == CUBLASLT_ORDER_COL ? op.epilogue_aux_ld : 1;
    g.aux_sb = op.epilogue_aux_batch_stride;
    if (g.aux_bgrad) {
      if (g.batch > 1 && op.bias_batch_stride == 0) return CUBLAS_STATUS_NOT_SUPPORTED;
      if (!dry && !op.bias) return CUBLAS_STATUS_INVALID_VALUE;
      g.bgrad = const_cast<void *>(op.bias);
    }
  }
  if (g.bgrad_src) {
    // sums of the stored elements: defined here for unscaled operands only
    if (a.type == CUDA_R_4F_E2M1 || b.type == CUDA_R_4F_E2M1 || g.a_scale_mode || g.b_scale_mode)
      return CUBLAS_STATUS_NOT_SUPPORTED;
    // batches with no stride between their gradient vectors would all write the same one
    if (g.batch > 1 && op.bias_batch_stride == 0) return CUBLAS_STATUS_NOT_SUPPORTED;
    if (!dry && !op.bias) return CUBLAS_STATUS_INVALID_VALUE;
    g.bgrad = const_cast<void *>(op.bias);
  }
  if (has_bias || g.bgrad_src || g.aux_bgrad) {
    if (has_bias && !dry && !op.bias) return CUBLAS_STATUS_INVALID_VALUE;
    if (has_bias) g.bias = op.bias;
    g.bias_sb = op.bias_batch_stride;
    if (op.bias_type >= 0) g.bias_type = (uint32_t)op.bias_type;
    else  // cuda_types/src/cublaslt.rs:4395-4403
      g.bias_type = (d.type == CUDA_R_8I || d.type == CUDA_R_32I || d.type == CUDA_R_8F_E4M3 ||
                     d.type == CUDA_R_8F_E5M2) ? CUDA_R_32F : d.type;
    if (!(g.bias_type == CUDA_R_32F || g.bias_type == CUDA_R_16F || g.bias_type == CUDA_R_16BF))
      return CUBLAS_STATUS_NOT_SUPPORTED;
  }

  out->g = g;
  out->has_bias = has_bias;
  out->a_kcontig = g.a_sk == 1;
  out->b_kcontig = g.b_sk == 1;
  auto al16 = [](const void *ptr, int64_t pitch_elems, int64_t bstride, int bits, bool batched) {
    return (((uintptr_t)ptr) & 15) == 0 && ((pitch_elems * bits / 8) & 15) == 0 &&
           (!batched || ((bstride * bits / 8) & 15) == 0);
  };
  out->aligned16 = al16(g.A, g.a_si, g.a_sb, type_bits(a.type), g.batch > 1) &&
                   al16(g.B, g.b_sj, g.b_sb, type_bits(b.type), g.batch > 1) &&
                   (((int64_t)K * type_bits(a.type) / 8) & 15) == 0;
  // the MFMA kernels address each operand through a 2 GiB buffer window
  const int64_t span_a = ((int64_t)(M - 1) * g.a_si + (int64_t)K) * type_bits(a.type) / 8;
  const int64_t span_b = ((int64_t)(N - 1) * g.b_sj + (int64_t)K) * type_bits(b.type) / 8;
  out->span_ok = span_a < 0x7fffffffll && span_b < 0x7fffffffll;
  return CUBLAS_STATUS_SUCCESS;
}

static bool is_f8(uint32_t t) { return t == CUDA_R_8F_E4M3 || t == CUDA_R_8F_E5M2; }

static bool decode_variant_ok(const Lowered &l, int variant) {
  const GemmArgs &g = l.g;
  const DecodeVariant &v = kDecodeVariants[variant];
  const int T = std::min(g.M, g.N), nb = (T + 15) / 16;
  const bool h16 = g.a_type == CUDA_R_16F || g.a_type == CUDA_R_16BF;
  if (h16 && v.stream != 2) return false;  // 16-bit weights: the slab form only
  // the register-streaming kernel is int8 only; token blocks multiply its fragment registers
  if (!v.stream) return g.a_type == CUDA_R_8I && (nb == 1 || (nb == 2 && v.steps <= 8));
  const bool swapped = g.M < g.N;
  const int64_t rows = swapped ? g.N : g.M, ldw = swapped ? g.b_sj : g.a_si;
  if (v.stream == 2) {
    const int64_t ldx = swapped ? g.a_si : g.b_sj;
    // (the 4-wave shape serves K down to half of its 4096; an 8-wave shape the K above the next smaller cover)
    const int cover = v.nw * v.steps * 64, below = cover == 4096 ? cover / 2 : cover - 4096;
    // one block of tokens; two in the 8-wave shapes of one or two units (the one-unit shape exists for them alone)
    const bool tokens_ok = v.nw == 4 ? nb == 1 : v.steps == 8 ? nb == 2 : v.steps == 16 ? nb <= 2 : nb == 1;
    const int64_t esz = h16 ? 2 : 1, kb = (int64_t)g.K * esz;  // covers are bytes of K
    return tokens_ok && kb <= cover && kb > below && (kb & 15) == 0 && rows * ldw * esz < 0x7fffffffll &&
           ((int64_t)(T - 1) * ldx + g.K) * esz < 0x7fffffffll;
  }
  // a stream instantiation covers nw * steps * 64 bytes of K and takes any K up to that (lanes past the end read
  // zero); more than a quarter of idle lanes is left to the smaller instantiations or to the MFMA tiles
  const int cover = v.nw * v.steps * 64;
  return g.K <= cover && g.K * 4 > cover * 3 && (g.K & 15) == 0 && rows * ldw < 0x7fffffffll &&
         nb * v.steps <= kDecodeStreamMaxFragments;
}

static bool any_decode_variant_ok(const Lowered &l) {
  for (int v = 0; v < kNumDecodeVariants; v++)
    if (decode_variant_ok(l, v)) return true;
  return false;
}

bool family_supports(uint32_t kernel, const Lowered &l) {
  const GemmArgs &g = l.g;
  const bool fast_layout = l.a_kcontig && l.b_kcontig && l.aligned16;
  const bool d_fast = g.d_type == CUDA_R_32I || g.d_type == CUDA_R_32F || g.d_type == CUDA_R_16BF ||
                      g.d_type == CUDA_R_16F || g.d_type == CUDA_R_8I;
  switch (kernel) {
  case ZLUDA_KERNEL_GENERIC: return true;
  case ZLUDA_KERNEL_MFMA_I8:
    return fast_layout && l.span_ok && g.a_type == CUDA_R_8I && g.b_type == CUDA_R_8I && d_fast;
  case ZLUDA_KERNEL_MFMA_F8:
    return fast_layout && l.span_ok && is_f8(g.a_type) && is_f8(g.b_type) &&
           !(g.a_type == CUDA_R_8F_E5M2 && g.b_type == CUDA_R_8F_E5M2) &&
           g.a_scale_mode != SCALE_BLOCK32_UE8M0 && g.b_scale_mode != SCALE_BLOCK32_UE8M0 && d_fast;
  case ZLUDA_KERNEL_MFMA_MXF4:
    return fast_layout && l.span_ok && g.a_type == CUDA_R_4F_E2M1 && g.b_type == CUDA_R_4F_E2M1 &&
           g.a_scale_mode == SCALE_BLOCK32_UE8M0 && g.b_scale_mode == SCALE_BLOCK32_UE8M0 &&
           (g.K % 256) == 0 && ((((uintptr_t)g.a_scale) | ((uintptr_t)g.b_scale)) & 3) == 0 && d_fast;
  case ZLUDA_KERNEL_MFMA_H16:
    // f16 x f16 or bf16 x bf16 (lower_problem admits 16-bit operands of one type only)
    return fast_layout && l.span_ok && (g.a_type == CUDA_R_16F || g.a_type == CUDA_R_16BF) && g.b_type == g.a_type &&
           g.a_scale_mode != SCALE_BLOCK32_UE8M0 && g.b_scale_mode != SCALE_BLOCK32_UE8M0 && d_fast;
  case ZLUDA_KERNEL_MFMA_F32:
    return fast_layout && l.span_ok && g.a_type == CUDA_R_32F && g.b_type == CUDA_R_32F && d_fast;
  case ZLUDA_KERNEL_MFMA_TR8: case ZLUDA_KERNEL_MFMA_TR16: case ZLUDA_KERNEL_MFMA_TR32: {
    // 8-bit (TR8), 16-bit (TR16) or f32 (TR32) operands, each with unit stride along K or along its row index; dword-aligned loads
    const bool h16 = g.a_type == CUDA_R_16F || g.a_type == CUDA_R_16BF, f32 = g.a_type == CUDA_R_32F;
    const bool types = kernel == ZLUDA_KERNEL_MFMA_TR32 ? (f32 && g.b_type == CUDA_R_32F)
                       : kernel == ZLUDA_KERNEL_MFMA_TR16
                           ? (h16 && g.b_type == g.a_type)
                           : ((g.a_type == CUDA_R_8I && g.b_type == CUDA_R_8I) ||
                              (is_f8(g.a_type) && is_f8(g.b_type) && !(g.a_type == CUDA_R_8F_E5M2 && g.b_type == CUDA_R_8F_E5M2)));
    const int64_t esz = f32 ? 4 : h16 ? 2 : 1;
    // (strides in bytes from here on)
    auto operand_ok = [&](const void *ptr, int64_t s_row, int64_t s_k, int64_t s_b, int rows) {
      s_row *= esz; s_k *= esz; s_b *= esz;
      if ((((uintptr_t)ptr) & 3) || (g.batch > 1 && (s_b & 3))) return false;
      const int64_t span = (int64_t)(rows - 1) * s_row + (int64_t)(g.K - 1) * s_k + esz;
      if (span >= 0x7fffffffll) return false;
      if (s_k == esz) return (s_row & 3) == 0 && ((g.K * esz) & 15) == 0;  // 16-byte pieces along K
      // (offsets of K rows up to three stages past the end must stay below 2^32, where they are out
      // of range instead of wrapping into it)
      return s_row == esz && (s_k & 3) == 0 && (int64_t)(g.K + 256) * s_k < 0xffffffffll;
    };
    return types && d_fast && g.a_scale_mode != SCALE_BLOCK32_UE8M0 && g.b_scale_mode != SCALE_BLOCK32_UE8M0 &&
           operand_ok(g.A, g.a_si, g.a_sk, g.a_sb, g.M) && operand_ok(g.B, g.b_sj, g.b_sk, g.b_sb, g.N);
  }
  case ZLUDA_KERNEL_DECODE_W8A8:
    // int8, or e4m3 x e4m3 without block scales (the LDS-streaming variants only), or f16 / bf16 (the slab form only)
    return fast_layout && ((g.a_type == CUDA_R_8I && g.b_type == CUDA_R_8I) ||
                           ((g.a_type == CUDA_R_16F || g.a_type == CUDA_R_16BF) && g.b_type == g.a_type) ||
                           (g.a_type == CUDA_R_8F_E4M3 && g.b_type == CUDA_R_8F_E4M3 &&
                            g.a_scale_mode != SCALE_BLOCK32_UE8M0 && g.b_scale_mode != SCALE_BLOCK32_UE8M0)) &&
           std::min(g.M, g.N) <= kDecodeMaxTokens && std::max(g.M, g.N) >= 64 && any_decode_variant_ok(l);
  default: return false;
  }
}

static uint32_t ceil_div(uint32_t a, uint32_t b) { return (a + b - 1) / b; }

int w4_epilogue_class(const Lowered &l, bool dry) {
  const GemmArgs &g = l.g;
  // (the epilogues with an aux matrix are plain problems to the GEMM kernel: launch_planned points D at the aux matrix or
  // runs the gradient pass behind it)
  if (g.beta_mode != SCALAR_VALUE) return W4_CLASS_NONE;
  const bool swapped = g.d_si != 1;
  const int64_t d_sq = swapped ? g.d_si : g.d_sj;
  const int dbytes = (g.d_type == CUDA_R_32I || g.d_type == CUDA_R_32F) ? 4 : 2;
  if (((d_sq * dbytes) & 15) || (g.batch > 1 && ((g.d_sb * dbytes) & 15)) || d_sq >= (1 << 22) || (((uintptr_t)g.D) & 15))
    return W4_CLASS_NONE;
  const bool i8 = g.a_type == CUDA_R_8I && g.b_type == CUDA_R_8I;
  if (i8 && g.int_scale) {
    if (g.d_type != CUDA_R_32I || g.alpha_mode == VECTOR_DEV || (!dry && g.beta_val.i != 0)) return W4_CLASS_NONE;
    return W4_CLASS_I32;
  }
  // float epilogues: int8 with float scaling (W8A8: alpha[] or outer scales per row and per token), fp8, f16 and bf16
  const bool h16 = (g.a_type == CUDA_R_16F || g.a_type == CUDA_R_16BF) && g.b_type == g.a_type;
  const bool f8a = g.a_type == CUDA_R_8F_E4M3 || g.a_type == CUDA_R_8F_E5M2, f8b = g.b_type == CUDA_R_8F_E4M3 || g.b_type == CUDA_R_8F_E5M2;
  const bool f8 = f8a && f8b && !(g.a_type == CUDA_R_8F_E5M2 && g.b_type == CUDA_R_8F_E5M2);  // (E5M2 x E5M2 is not a cuBLASLt combination)
  if ((i8 || h16 || f8) && g.a_scale_mode != SCALE_BLOCK32_UE8M0 &&
      g.b_scale_mode != SCALE_BLOCK32_UE8M0) {
    if ((g.d_type != CUDA_R_16BF && g.d_type != CUDA_R_16F && g.d_type != CUDA_R_32F) || (!dry && g.beta_val.f != 0.0f))
      return W4_CLASS_NONE;  // (ReLU and the output type are run-time choices of the two classes)
    // scale vectors may run either way; a bias only along D's unit stride
    if (swapped && l.has_bias) return W4_CLASS_NONE;
    return g.act == ACT_GELU ? W4_CLASS_BF16_GELU : W4_CLASS_BF16;
  }
  if (g.a_type == CUDA_R_4F_E2M1 && g.b_type == CUDA_R_4F_E2M1 && g.a_scale_mode == SCALE_BLOCK32_UE8M0 &&
      g.b_scale_mode == SCALE_BLOCK32_UE8M0) {
    // MXFP4: whole scale chunks (1024 elements of K) per tile, and no vector along D's unit stride either (the scale
    // chunks take the LDS the other kinds stage such vectors in)
    if ((g.d_type != CUDA_R_16BF && g.d_type != CUDA_R_16F && g.d_type != CUDA_R_32F) || (!dry && g.beta_val.f != 0.0f))
      return W4_CLASS_NONE;  // (ReLU and the output type are run-time choices of the two classes)
    if ((g.K & 1023) || g.alpha_mode == VECTOR_DEV || l.has_bias) return W4_CLASS_NONE;
    return g.act == ACT_GELU ? W4_CLASS_BF16_GELU : W4_CLASS_BF16;
  }
  return W4_CLASS_NONE;
}

static void fill_mfma_plan(const Lowered &l, int variant, uint32_t cus, uint64_t workspace_size,
                           zluda_gemm_plan *plan) {
  const GemmArgs &g = l.g;
  const MfmaVariant &v = kMfmaVariants[variant];
  const bool swapped = g.d_si != 1;  // row-major D: compute D^T
  const uint32_t np = swapped ? g.N : g.M, nq = swapped ? g.M : g.N;
  const uint32_t tp = ceil_div(np, v.bp), tq = ceil_div(nq, v.bq);
  plan->variant = variant;
  plan->swapped = swapped;
  plan->grid_x = tp * tq; plan->grid_y = g.batch; plan->grid_z = 1;
  plan->block = v.wp * v.wq * 64;
  if (v.w4) {
    // one workgroup per CU (a multiple of 8 of them, so that a workgroup's tiles stay on one XCD's share of the tile
    // order) walks the tiles of all batches; never split along K
    const uint64_t all = (uint64_t)tp * tq * g.batch;
    const uint32_t slots = cus >= 8 ? cus / 8 * 8 : cus;
    plan->grid_x = (uint32_t)std::min<uint64_t>(all, slots);
    plan->grid_y = 1;
    plan->waves = (float)all / (float)cus;
    plan->workspace = 0;
    return;
  }
  // data stages, plus two chunks of 32 scale bytes per tile row for MXFP4
  const uint32_t lds = (uint32_t)v.stages * (v.bp + v.bq) * v.bkb + (l.g.a_type == CUDA_R_4F_E2M1 ? 64u * (v.bp + v.bq) : 0u);
  const uint32_t per_cu = std::max(1u, std::min(160u * 1024u / lds, 2048u / plan->block));
  plan->waves = (float)plan->grid_x * plan->grid_y / (float)(cus * per_cu);
  plan->workspace = 0;
  // Split-K: when even the chosen tiles leave half of the CUs idle and K is long, grid_z workgroups
  // share a tile's K range, write their fp32 / int32 partial tiles to the workspace and a second
  // kernel sums them and applies the epilogue.  Only if the caller's workspace holds the partial
  // tiles (padded to whole tiles).  (MXFP4 shares are whole scale chunks: the launcher rounds.)
  const uint64_t tiles = (uint64_t)plan->grid_x * plan->grid_y;
  const uint32_t kt = ceil_div((uint32_t)((int64_t)g.K * type_bits(g.a_type) / 8), v.bkb);
  // (below ~6 KiB of K per row the second kernel and the workspace traffic cost more than the idle CUs)
  const uint32_t kbytes = kt * v.bkb;
  // Skinny problems (<= 64 rows or columns) are memory bound: they split from 2 KiB of K per row on
  // and down to 1 KiB per share, up to two workgroups per CU (fp8 4096x48x4096: 18 -> 13 us; but
  // 14336x64x4096, 224 tiles, must stay whole: 16.5 us against 23.7 split in three).
  const bool skinny = std::min(g.M, g.N) <= 64;
  const bool mx = g.a_type == CUDA_R_4F_E2M1;  // (a byte of FP4 is worth two K steps: 4096x16x4096 loses when split)
  if (tiles * 2 <= cus && kbytes >= (skinny ? (mx ? 4096u : 2048u) : 6144u) &&
      (uint64_t)tp * v.bp <= (1u << 20)) {
    uint32_t s = (uint32_t)std::min<uint64_t>({8, (skinny ? 2 * cus : cus) / tiles, kbytes / (skinny ? 1024 : 2048)});
    const uint64_t per_split = (uint64_t)g.batch * tp * v.bp * tq * v.bq * 4;
    while (s > 1 && s * per_split > workspace_size) s--;
    if (s > 1) {
      plan->grid_z = s;
      plan->workspace = s * per_split;
      plan->waves = (float)tiles * s / (float)(cus * per_cu);
    }
  }
}

// Relative throughput of one CU running tiles of each variant (measured on MI355X, int8 and fp8, K >= 1024;
// variant 0 = 1).  Smaller tiles read more LDS and L2 bytes per MFMA.
// The variants on the 16x16 MFMA shapes (8, 9) need less energy per multiply-add, which is what bounds a GEMM
// that keeps the whole chip busy (the board sits at its power cap): at 4096^3 and 8192^3 they take 8-10 % less
// time than their 32x32 counterparts for int8 and 1-3 % less for fp8.  On a chip that is partly idle the clock
// is the bound instead and they lose (their epilogue is ~3 us per tile slower: 2048^3 int8 30.5 us against
// 27.5), so they are only chosen for grids that fill the chip; the same tiles at 256x128 and 128x128 measured
// no better than the 32x32 ones anywhere and are not instantiated.
static const float kMfmaVariantEfficiency[kNumMfmaVariants] = {1.00f, 0.95f, 0.80f, 0.70f, 0.72f, 0.55f, 0.40f, 0.85f,
                                                               1.05f, 0.89f, 0.40f, 1.10f};

static int pick_mfma_variant(const Lowered &l, uint32_t cus) {
  const GemmArgs &g = l.g;
  const bool swapped = g.d_si != 1;
  const uint32_t np = swapped ? g.N : g.M, nq = swapped ? g.M : g.N;
  // cost = rounds of workgroups over the CUs x time of one tile; the tile shapes trade efficiency
  // per CU against how evenly the problem fills the chip
  int best = 0;
  double best_cost = 0;
  for (int v = 0; v < kNumMfmaVariants; v++) {
    const MfmaVariant &t = kMfmaVariants[v];
    const uint64_t tiles = (uint64_t)ceil_div(np, t.bp) * ceil_div(nq, t.bq) * g.batch;
    if (t.stages > 4) continue;  // the deep ring: see below
    if (t.w4) {
      // The four-wave kernel, for the problems its epilogues serve: level with the best other variant from one round of
      // tiles on, 4-7 % ahead from four (8192^3: int8 410 us against 429, fp8 360 against 389; 8192 x 4096 x 4096 fp8
      // 103 against 109; 4096^3 int8 59.4 against 59.5), but not on a short K, where the per-tile work around the loop
      // shows (16384 x 8192 x 1024 fp8: 167 us against 153 for variant 0)
      if (w4_epilogue_class(l, true) == W4_CLASS_NONE || g.K < 2048) continue;
      if (tiles < (g.a_type == CUDA_R_8I ? ((uint64_t)cus * 3 + 3) / 4 : (uint64_t)cus)) continue;
    } else if (t.m16) {
      const bool h16 = g.a_type == CUDA_R_16F || g.a_type == CUDA_R_16BF;
      if (type_bits(g.a_type) != 8 && !h16) continue;  // the 16x16 shapes serve int8, fp8, f16 and bf16
      // power bound or not: int8 gains from three quarters of the CUs busy on.  fp8 gains little and only on
      // long runs: the 192x256 tile from two full rounds on (6144^3: 190 us against 198), the 256x256 tile
      // from four (8192^3: 405 against 408; at two rounds, 8192x4096x4096, it loses 3 %)
      // (f16 / bf16 as int8: bf16 8192^3 776 us against 840, 4096^3 102 against 108, 6144^3 336 against 360)
      const uint64_t need = (g.a_type == CUDA_R_8I || h16) ? ((uint64_t)cus * 3 + 3) / 4 : (uint64_t)cus * (t.bp == 256 ? 4 : 2);
      if (tiles < need) continue;
    }
    const uint64_t rounds = (tiles + cus - 1) / cus;
    const double cost = (double)rounds * t.bp * t.bq / kMfmaVariantEfficiency[v];
    if (v == 0 || cost < best_cost) { best = v; best_cost = cost; }
  }
  return best;
}

static void fill_tr_plan(const Lowered &l, int variant, uint32_t cus, uint64_t workspace_size, zluda_gemm_plan *plan) {
  const GemmArgs &g = l.g;
  const TrVariant &v = kTrVariants[variant];
  const bool swapped = g.d_si != 1;
  const uint32_t np = swapped ? g.N : g.M, nq = swapped ? g.M : g.N;
  plan->variant = variant;
  plan->swapped = swapped;
  plan->grid_x = ceil_div(np, v.bp) * ceil_div(nq, v.bq); plan->grid_y = g.batch; plan->grid_z = 1;
  plan->block = v.wp * v.wq * 64;
  const uint32_t per_cu = 160u * 1024u / (2u * (v.bp + v.bq) * 80u);  // LDS: two stages of 80-byte rows
  plan->waves = (float)plan->grid_x * plan->grid_y / (float)(cus * std::min(per_cu, 4u));
  plan->workspace = 0;
  // Split-K as for the K-contiguous kernels: grid_z workgroups share a tile's K range through the
  // caller's workspace when K has at least 16 stages and the tiles leave half of the chip idle --
  // half of the CUs, or, for skinny problems (<= 64 rows or columns: memory bound, a workgroup keeps
  // only ~16 KiB in flight), half of the workgroup slots.  N-contiguous weights, 16 tokens, us:
  // 4096x14336 89 -> 25, 4096x4096 31 -> 14, 14336x4096 31 -> 24; 14336x128x4096 would lose (37 -> 42).
  const uint64_t tiles = (uint64_t)plan->grid_x * plan->grid_y;
  const uint64_t slots = (uint64_t)cus * std::min(per_cu, 4u);
  const bool skinny = std::min(g.M, g.N) <= 64;
  const uint64_t kbytes = (uint64_t)g.K * type_bits(g.a_type) / 8;
  if (tiles * 2 <= (skinny ? slots : (uint64_t)cus) && kbytes >= 1024 && (uint64_t)ceil_div(np, v.bp) * v.bp <= (1u << 20)) {
    uint32_t s = (uint32_t)std::min<uint64_t>({8, slots / tiles, kbytes / 512});
    const uint64_t per_split = (uint64_t)g.batch * ceil_div(np, v.bp) * v.bp * ceil_div(nq, v.bq) * v.bq * 4;
    while (s > 1 && s * per_split > workspace_size) s--;
    if (s > 1) {
      plan->grid_z = s;
      plan->workspace = s * per_split;
      plan->waves = (float)tiles * s / (float)slots;
    }
  }
}

// Tile choice of the transposing kernel.  A CU runs up to `per_cu` workgroups of a variant side by
// side; the time it needs for n of them (same K) was measured on MI355X (int8, K = 4096, us):
// 256x256: 71;  128x128: 37 alone, 48 for two;  64x64: 22 alone, 40 for four  ->  base + slope * n.
// Cost of a variant = full rounds x time(per_cu) + time(what is left per CU).
struct TrCost { uint32_t per_cu; float base, slope; };
static const TrCost kTrCost[kNumTrVariants] = {{1, 0.0f, 71.0f}, {2, 26.0f, 11.0f}, {4, 16.0f, 6.0f}, {1, 0.0f, 67.0f}};

static int pick_tr_variant(const Lowered &l, uint32_t cus) {
  const GemmArgs &g = l.g;
  const bool swapped = g.d_si != 1;
  const uint32_t np = swapped ? g.N : g.M, nq = swapped ? g.M : g.N;
  int best = 0;
  double best_cost = 0;
  for (int v = 0; v < kNumTrVariants; v++) {
    const TrVariant &t = kTrVariants[v];
    const TrCost &c = kTrCost[v];
    const uint64_t tiles = (uint64_t)ceil_div(np, t.bp) * ceil_div(nq, t.bq) * g.batch;
    // the 16x16 shape: int8, f16 and bf16, and only where the chip is full enough to sit at its power cap
    const bool m16_type = g.a_type == CUDA_R_8I || g.a_type == CUDA_R_16F || g.a_type == CUDA_R_16BF;
    if (t.m16 && (!m16_type || tiles * 4 < (uint64_t)cus * 3)) continue;
    const uint64_t slots = (uint64_t)cus * c.per_cu;
    const uint64_t full = tiles / slots, rem = tiles % slots;
    double cost = (double)full * (c.base + c.slope * c.per_cu);
    if (rem) cost += c.base + c.slope * (double)((rem + cus - 1) / cus);
    if (v == 0 || cost < best_cost) { best = v; best_cost = cost; }
  }
  return best;
}

static void fill_decode_plan(const Lowered &l, int variant, uint32_t cus, zluda_gemm_plan *plan) {
  const GemmArgs &g = l.g;
  const DecodeVariant &v = kDecodeVariants[variant];
  const bool swapped = g.M < g.N;  // weights are the long operand
  const uint32_t rows = swapped ? g.N : g.M;
  const uint32_t nrb = ceil_div(rows, 16);
  // Stream kernel: 8 waves x 2 slots x 4 KiB = 64 KiB in flight per CU is the measured optimum on
  // MI355X (14.8 us for 58.7 MB; 128 KiB in flight: 15.8-16.8 us, 32 KiB: 15.9 us), so one 8-wave
  // workgroup per CU, two 4-wave ones.
  const uint32_t resident = v.stream == 2 ? cus : v.stream ? cus * (v.nw == 8 ? 1 : 2) : cus * (v.nw == 8 ? 2 : 4);
  uint32_t grid;
  // slab kernel: at most one workgroup per CU (its LDS ring fills the CU), more only when the rows would not fit
  // into 4 blocks per workgroup otherwise
  // (a short block costs its workgroup as many DMA instructions as a full one: the fewest rounds of blocks that
  // fit the CUs, shared out evenly -- 896 blocks on 256 CUs: 224 workgroups x 4)
  if (v.stream == 2) grid = std::max(ceil_div(nrb, ceil_div(nrb, cus)), ceil_div(rows, 64));
  else if (v.stream) grid = std::min(nrb, resident);  // contiguous, balanced row ranges
  else grid = nrb <= resident ? nrb : ceil_div(nrb, ceil_div(nrb, resident));
  plan->variant = variant;
  plan->swapped = swapped;
  plan->grid_x = grid; plan->grid_y = g.batch; plan->grid_z = 1;
  plan->block = v.nw * 64;
  plan->waves = (float)grid * g.batch / (float)resident;
  plan->workspace = 0;
}

static int pick_decode_variant(const Lowered &l, uint32_t cus) {
  const int K = l.g.K;
  // the slab form where it applies and one workgroup per CU holds the rows (14336 x 16 x 4096 int8: 12.4 us
  // against 14.8 for the stream kernel proper)
  // (two token blocks on one unit per slab, variant 20, only up to two blocks of rows per CU: 4096 x 32 x 4096
  // 8.9 us against 10.0, but 14336 x 32 x 4096 18.1 against 16.7; with two units, variant 17, it wins
  // throughout: 8192 x 32 x 8192 15.4 against 22.0)
  // (16-bit weights, which have no other streaming form, also beyond 64 rows per CU when K is long: bf16
  // 28672 x 16 x 8192 in 1.75 rounds of workgroups 80 us against 99 on 128 x 64 MFMA tiles; at K = 4096 the two are level)
  const uint32_t rows = (uint32_t)std::max(l.g.M, l.g.N);
  const bool h16_long = (l.g.a_type == CUDA_R_16F || l.g.a_type == CUDA_R_16BF) && K * 2 > 8192;
  for (int v = 0; v < kNumDecodeVariants; v++)
    if (kDecodeVariants[v].stream == 2 && decode_variant_ok(l, v) && (rows <= 64 * cus || h16_long) &&
        !(kDecodeVariants[v].steps == 8 && rows > 32 * cus))
      return v;
  // the stream instantiation with the least cover that takes K
  int best = -1;
  for (int v = 0; v < kNumDecodeVariants; v++)
    if (kDecodeVariants[v].stream == 1 && decode_variant_ok(l, v) &&
        (best < 0 || kDecodeVariants[v].nw * kDecodeVariants[v].steps < kDecodeVariants[best].nw * kDecodeVariants[best].steps))
      best = v;
  if (best >= 0) return best;
  for (int v = 0; v < kNumDecodeVariants; v++)
    if (!kDecodeVariants[v].stream && K == kDecodeVariants[v].nw * kDecodeVariants[v].steps * 64 && decode_variant_ok(l, v))
      return v;
  return 0;
}

} // namespace zluda_amd

using namespace zluda_amd;

extern "C" uint32_t zluda_gemm_variant_count(uint32_t kernel) {
  switch (kernel) {
  case ZLUDA_KERNEL_GENERIC: return 1;
  case ZLUDA_KERNEL_MFMA_I8: case ZLUDA_KERNEL_MFMA_F8: return kNumMfmaVariants;
  case ZLUDA_KERNEL_MFMA_H16: return kNumMfmaVariantsH16;
  case ZLUDA_KERNEL_MFMA_F32: return kNumMfmaVariants32;  // the 16x16-shape ones serve int8, fp8, f16 and bf16
  case ZLUDA_KERNEL_MFMA_MXF4: return kNumMfmaVariants;   // (the eight 32x32-shape ones and the four-wave kernel; those between are refused)
  case ZLUDA_KERNEL_DECODE_W8A8: return kNumDecodeVariants;
  case ZLUDA_KERNEL_MFMA_TR8: case ZLUDA_KERNEL_MFMA_TR16: return kNumTrVariants;
  case ZLUDA_KERNEL_MFMA_TR32: return kNumTrVariants - 1;  // the 16x16-shape one is not instantiated for f32
  default: return 0;
  }
}

extern "C" uint32_t zluda_gemm_plan_problem(const zluda_gemm_problem *p, uint32_t forced_kernel,
                                            int32_t forced_variant, uint32_t cu_count,
                                            zluda_gemm_plan *plan) {
  if (!plan) return CUBLAS_STATUS_INVALID_VALUE;
  Lowered l;
  // planning never dereferences data: NULL pointers mean "aligned as the preferences promise"
  uint32_t st = lower_problem(p, true, &l);
  if (st) return st;
  if (cu_count == 0) cu_count = 256;
  memset(plan, 0, sizeof(*plan));
  uint32_t kernel = forced_kernel;
  if (kernel == ZLUDA_KERNEL_AUTO) {
    static const uint32_t order[] = {ZLUDA_KERNEL_DECODE_W8A8, ZLUDA_KERNEL_MFMA_I8, ZLUDA_KERNEL_MFMA_F8,
                                     ZLUDA_KERNEL_MFMA_MXF4, ZLUDA_KERNEL_MFMA_H16, ZLUDA_KERNEL_MFMA_TR8,
                                     ZLUDA_KERNEL_MFMA_TR16, ZLUDA_KERNEL_MFMA_F32, ZLUDA_KERNEL_MFMA_TR32, ZLUDA_KERNEL_GENERIC};
    for (uint32_t k : order) {
      if (!family_supports(k, l)) continue;
      if (k == ZLUDA_KERNEL_DECODE_W8A8) {
        // (some variant takes the problem, but not necessarily the one the rules below pick for this chip: 16-bit
        // weights have the slab form only, which is given at most 64 rows per CU)
        if (!decode_variant_ok(l, pick_decode_variant(l, cu_count))) continue;
        const int tokens = std::min(l.g.M, l.g.N);
        const bool stream = kDecodeVariants[pick_decode_variant(l, cu_count)].stream;
        if (tokens > (stream ? kDecodeAutoMaxTokensStream : kDecodeAutoMaxTokens)) continue;
        // three token blocks only up to 32 rows per CU: beyond, 64-wide tiles read the weights as fast
        // (14336 x 48 x 4096 int8: 17.0 us against 20.7; 8192 x 33 x 4096: 14.0 against 13.9)
        if (tokens > 32 && (uint32_t)std::max(l.g.M, l.g.N) > 32 * cu_count) continue;
      }
      if (k == ZLUDA_KERNEL_DECODE_W8A8 && !kDecodeVariants[pick_decode_variant(l, cu_count)].stream &&
          family_supports(ZLUDA_KERNEL_MFMA_I8, l)) {  // (int8 only: fp8 has no such variant)
        // K outside the stream kernel's table: the register-streaming variant measures slower than
        // 64x64 MFMA tiles (split along K when the workspace allows) as soon as those give at
        // least half of the CUs a workgroup (5120x16x13824: 37 us against 23; 18944x32x3584: 46
        // against 25; but 2048x16x2560, 32 tiles: 8 against 12)
        zluda_gemm_plan mfma;
        memset(&mfma, 0, sizeof(mfma));
        fill_mfma_plan(l, pick_mfma_variant(l, cu_count), cu_count, p->workspace_size, &mfma);
        if ((uint64_t)mfma.grid_x * mfma.grid_y * mfma.grid_z * 2 >= cu_count) continue;
      }
      kernel = k;
      break;
    }
  } else if (!family_supports(kernel, l)) {
    return CUBLAS_STATUS_NOT_SUPPORTED;
  }
  plan->kernel = kernel;
  switch (kernel) {
  case ZLUDA_KERNEL_GENERIC:
    plan->variant = 0; plan->swapped = 0;
    plan->grid_x = ceil_div(l.g.M, 64); plan->grid_y = ceil_div(l.g.N, 64); plan->grid_z = l.g.batch;
    plan->block = 256;
    plan->waves = (float)plan->grid_x * plan->grid_y * plan->grid_z / (float)(cu_count * 8);
    if (plan->grid_y > 65535) return CUBLAS_STATUS_NOT_SUPPORTED;
    break;
  case ZLUDA_KERNEL_MFMA_I8: case ZLUDA_KERNEL_MFMA_F8: case ZLUDA_KERNEL_MFMA_MXF4: case ZLUDA_KERNEL_MFMA_H16:
  case ZLUDA_KERNEL_MFMA_F32: {
    int v = forced_variant >= 0 ? forced_variant : pick_mfma_variant(l, cu_count);
    const bool w4 = v < kNumMfmaVariants && kMfmaVariants[v].w4;
    if (v >= kNumMfmaVariants || (v >= kNumMfmaVariants32 && !w4 && kernel != ZLUDA_KERNEL_MFMA_I8 && kernel != ZLUDA_KERNEL_MFMA_F8 &&
                                  kernel != ZLUDA_KERNEL_MFMA_H16) || (v >= kNumMfmaVariantsH16 && kernel == ZLUDA_KERNEL_MFMA_H16) ||
        (w4 && kernel == ZLUDA_KERNEL_MFMA_F32))
      return CUBLAS_STATUS_INVALID_VALUE;
    // the four-wave kernel exists for int8, for fp8 without block scales, for MXFP4, for f16 and for bf16
    if (w4 && !(l.g.a_type == CUDA_R_8I || kernel == ZLUDA_KERNEL_MFMA_F8 ||
                (l.g.a_type == CUDA_R_4F_E2M1 && l.g.b_type == CUDA_R_4F_E2M1) ||
                ((l.g.a_type == CUDA_R_16F || l.g.a_type == CUDA_R_16BF) && l.g.b_type == l.g.a_type)))
      return CUBLAS_STATUS_NOT_SUPPORTED;
    fill_mfma_plan(l, v, cu_count, p->workspace_size, plan);
    // Skinny problems that end up with at most one 64 x 64 workgroup per CU and are not split along K are bound
    // by what a CU keeps in flight: the 6-stage ring of variant 10 (80 KiB instead of 32) takes 8-17 % less time
    // (bf16 14336x64x4096 29.2 us against 32.0, 4096x64x14336 71 against 87; int8 8192x64x8192 24.4 against 29.0).
    if (forced_variant < 0 && v == 6 && kernel != ZLUDA_KERNEL_MFMA_MXF4 && kernel != ZLUDA_KERNEL_MFMA_F32 && plan->grid_z == 1 &&
        (uint64_t)plan->grid_x * plan->grid_y <= cu_count && (int64_t)l.g.K * type_bits(l.g.a_type) / 8 >= 1536)
      fill_mfma_plan(l, 10, cu_count, 0, plan);
    break;
  }
  case ZLUDA_KERNEL_MFMA_TR8: case ZLUDA_KERNEL_MFMA_TR16: case ZLUDA_KERNEL_MFMA_TR32: {
    int v = forced_variant >= 0 ? forced_variant : pick_tr_variant(l, cu_count);
    if (v >= kNumTrVariants || (kTrVariants[v].m16 && l.g.a_type != CUDA_R_8I && l.g.a_type != CUDA_R_16F && l.g.a_type != CUDA_R_16BF))
      return CUBLAS_STATUS_INVALID_VALUE;
    fill_tr_plan(l, v, cu_count, p->workspace_size, plan);
    break;
  }
  case ZLUDA_KERNEL_DECODE_W8A8: {
    int v = forced_variant >= 0 ? forced_variant : pick_decode_variant(l, cu_count);
    if (v >= kNumDecodeVariants) return CUBLAS_STATUS_INVALID_VALUE;
    if (!decode_variant_ok(l, v)) return CUBLAS_STATUS_NOT_SUPPORTED;
    fill_decode_plan(l, v, cu_count, plan);
    break;
  }
  default: return CUBLAS_STATUS_NOT_SUPPORTED;
  }
  return CUBLAS_STATUS_SUCCESS;
}
