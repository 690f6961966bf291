/*
 * ref_gemm.c -- CPU restatement of the cublasLtMatmul contract.  TEST INFRASTRUCTURE ONLY.
 *
 * Nothing in the shipped library links, loads or calls this file; it is the checker that the
 * parity tests, the smoke test and the benchmark's cpu_baseline leg run next to the GPU path.
 *
 * What it restates.  The reference (ZLUDA, zluda_blaslt/src/impl.rs:157-196) contains no
 * arithmetic: it forwards cublasLtMatmul to hipBLASLt (a ROCm system library, version 1.2.1 in
 * this image, not vendored and not part of the reference tree).  The published contract of that
 * call is therefore the algorithm:
 *     D = epilogue(alpha * op(A) * op(B) + beta * C)          ext/hipblaslt-sys/src/lib.rs:1166-1177
 * with the attribute semantics documented beside the CUDA-side enums the reference carries:
 *     bias: length = rows of D, broadcast over columns, added before the activation
 *                                                              cuda_types/src/cublaslt.rs:4563-4566
 *     GELU_BIAS = bias, then GELU                              cuda_types/src/cublaslt.rs:4609-4610
 *     alpha device vector: one entry per row of D              cuda_types/src/cublaslt.rs:4100-4103, 3871-3883
 *     A/B scale pointer: multiplies the operand, NULL = 1      cuda_types/src/cublaslt.rs:4261-4288
 *     VEC32_UE8M0: one UE8M0 byte per 32 elements of the innermost (K) dimension
 *                                                              cuda_types/src/cublaslt.rs:3813-3818
 *     OUTER_VEC_32F: A scale has M entries, B scale N entries  cuda_types/src/cublaslt.rs:3820-3826
 *     layout attributes (order, ld, batch count/stride)        cuda_types/src/cublaslt.rs:3981-4058
 *     GELU_AUX[_BIAS]: as GELU[_BIAS]; the GELU input also goes to the aux matrix
 *                                                              cuda_types/src/cublaslt.rs:4601-4619, 4182-4236
 *     DGELU[_BGRAD]: D = gelu'(aux) * (alpha AB + beta C); _BGRAD: the bias buffer receives the gradient
 *                                                              cuda_types/src/cublaslt.rs:4621-4660, 4151-4166
 * Number formats follow the OCP definitions (E4M3 finite-only, E5M2 IEEE-like, E2M1, UE8M0);
 * the E4M3/E5M2 encoders additionally follow ptx/lib/zluda_ptx_impl.cpp:659-672
 * (round-to-nearest-even, saturate to the largest finite value, |x| < 2^-10 resp. 2^-17 -> +-0).
 *
 * How each piece is pinned (tests/test_oracle_*.py):
 *   - e4m3/e5m2 encode, e4m3/e5m2 decode, bf16 RNE: the reference's own known-answer vectors
 *     ptx/src/test/spirv_run/mod.rs:321-329 (tests/golden/ptx_cvt_kat.json)
 *   - signed int8 dot products with int32 accumulate: the reference's dp4a vector
 *     (mod.rs:480-484) and its 256-entry mma.m16n8k32.s8 result (mod.rs:890-918)
 *   - integer GEMM incl. transposes/orders/ld/batch: brute force and numpy int64 matmul
 *   - e2m1 / ue8m0 decode: exhaustive against the closed-form OCP definition
 *   - float GEMMs: exact rational arithmetic on tiny shapes, numpy float64 otherwise
 *   - epilogue (alpha vector, outer scales, bias, relu/gelu): scalar formulas in numpy
 *   - gelu': central differences of the GELU in float64, its values at 0 (1/2) and far out (0 and 1);
 *     GELU_AUX: gelu(aux) reproduces D; DGELU_BGRAD: numpy row sums of D
 * PARITY UNPINNED (no fixture in the reference, no hipBLASLt run possible without a GPU):
 *   - which GELU hipBLASLt applies: the tanh form is restated here.  No CPU-side fixture pins it;
 *     on a GPU box tests/test_gpu_vs_hipblaslt.py tells the tanh and erf forms apart against
 *     hipBLASLt itself (it applies the tanh form)
 *   - DGELU_BGRAD: that the gradient is the sum over D's columns, one value per row of D (the orientation of the
 *     bias it is the gradient of), and that the aux matrix has D's order: the text cited above gives the lengths and
 *     the leading dimension only.  No CPU-side fixture pins it; on a GPU box tests/test_gpu_aux_epilogues.py
 *     compares D, the aux matrix and the gradient with hipBLASLt itself for f16 operands (it offers these
 *     epilogues for no other input type)
 *   - the batch stride of the UE8M0 scale tensors for batch counts above 1 (restated as batches back to
 *     back, rows * K/32 bytes each): hipBLASLt takes MXFP4 at batch 1 only.  The layout inside a batch,
 *     plain [row][K/32] bytes for both operands, is pinned on a GPU box against hipBLASLt itself by the
 *     impulse responses of tests/test_gpu_vs_hipblaslt.py
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "../include/cublaslt_abi.h"
#include "../include/zluda_gemm_launch.h"

/* ------------------------------------------------------------------ number formats ------- */

static float bits_to_float(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static uint32_t float_to_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}

/* OCP E4M3 (finite-only: S.1111.111 is NaN, no infinities), bias 7. */
float oracle_decode_e4m3(uint8_t v) {
  int s = v >> 7, e = (v >> 3) & 15, m = v & 7;
  float r;
  if (e == 15 && m == 7)
    return NAN;
  if (e == 0)
    r = ldexpf((float)m, -9); /* subnormal: m/8 * 2^-6 */
  else
    r = ldexpf(1.0f + (float)m / 8.0f, e - 7);
  return s ? -r : r;
}

/* OCP E5M2 (IEEE-like), bias 15. */
float oracle_decode_e5m2(uint8_t v) {
  int s = v >> 7, e = (v >> 2) & 31, m = v & 3;
  float r;
  if (e == 31)
    r = m ? NAN : INFINITY;
  else if (e == 0)
    r = ldexpf((float)m, -16);
  else
    r = ldexpf(1.0f + (float)m / 4.0f, e - 15);
  return s ? -r : r;
}

/* OCP E2M1: magnitudes 0, .5, 1, 1.5, 2, 3, 4, 6. */
float oracle_decode_e2m1(uint8_t nibble) {
  static const float mag[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
  float r = mag[nibble & 7];
  return (nibble & 8) ? -r : r;
}

/* OCP UE8M0: 2^(v-127), 0xFF is NaN. */
float oracle_decode_ue8m0(uint8_t v) {
  if (v == 0xFF)
    return NAN;
  return ldexpf(1.0f, (int)v - 127);
}

/* Generic round-to-nearest-even, saturating-to-finite encoder for a small float format with
 * `ebits` exponent bits, `mbits` mantissa bits, bias `bias` and largest finite value `maxv`.
 * `flush_below` reproduces ptx/lib/zluda_ptx_impl.cpp:659-672 (inputs with |x| below it give
 * signed zero); pass 0 for no flush. */
static uint8_t encode_small(float f, int ebits, int mbits, int bias, float maxv, uint8_t max_code,
                            uint8_t nan_code, float flush_below) {
  uint32_t bits = float_to_bits(f);
  uint8_t sign = (bits >> 31) ? (uint8_t)(1u << (ebits + mbits)) : 0;
  float a = fabsf(f);
  if (isnan(f))
    return sign | nan_code;
  if (a < flush_below || a == 0.0f)
    return sign;
  if (a >= maxv)
    return sign | max_code; /* satfinite (also +-inf) */
  /* scale so that one unit = the spacing of the target at this magnitude */
  int e;
  frexpf(a, &e);            /* a = m * 2^e, m in [0.5,1) -> unbiased exponent e-1 */
  int ue = e - 1;
  int emin = 1 - bias;      /* smallest normal exponent */
  if (ue < emin)
    ue = emin;              /* subnormal range shares the spacing of emin */
  float q = ldexpf(a, mbits - ue); /* in units of ulp; exact (power-of-two scaling) */
  float r = nearbyintf(q);         /* RNE in the default rounding mode */
  /* r in [0, 2^(mbits+1)]; renormalise if it rounded up to the next binade */
  int mant = (int)r;
  int biased = ue + bias;
  if (ue == emin && mant < (1 << mbits)) {
    biased = 0; /* subnormal (or zero) */
  } else {
    if (mant >= (2 << mbits)) {
      mant >>= 1;
      biased += 1;
    }
    mant -= (1 << mbits);
  }
  uint8_t code = (uint8_t)((biased << mbits) | mant);
  if (code > max_code)
    code = max_code;
  return sign | code;
}

uint8_t oracle_encode_e4m3(float f) {
  /* min = 0x3A800000 = 2^-10 : zluda_ptx_impl.cpp:665 */
  return encode_small(f, 4, 3, 7, 448.0f, 0x7E, 0x7F, bits_to_float(0x3A800000u));
}
uint8_t oracle_encode_e5m2(float f) {
  /* min = 0x37000000 = 2^-17 : zluda_ptx_impl.cpp:665 */
  return encode_small(f, 5, 2, 15, 57344.0f, 0x7B, 0x7F, bits_to_float(0x37000000u));
}
uint8_t oracle_encode_e2m1(float f) { return encode_small(f, 2, 1, 1, 6.0f, 0x7, 0x7, 0.0f); }

uint16_t oracle_encode_bf16(float f) {
  uint32_t u = float_to_bits(f);
  if (isnan(f))
    return (uint16_t)((u >> 16) | 0x40);
  u += 0x7FFFu + ((u >> 16) & 1u); /* round to nearest even */
  return (uint16_t)(u >> 16);
}
float oracle_decode_bf16(uint16_t v) { return bits_to_float((uint32_t)v << 16); }

float oracle_decode_f16(uint16_t v) {
  int s = v >> 15, e = (v >> 10) & 31, m = v & 1023;
  float r;
  if (e == 31)
    r = m ? NAN : INFINITY;
  else if (e == 0)
    r = ldexpf((float)m, -24);
  else
    r = ldexpf(1.0f + (float)m / 1024.0f, e - 15);
  return s ? -r : r;
}
uint16_t oracle_encode_f16(float f) {
  uint32_t bits = float_to_bits(f);
  uint16_t sign = (uint16_t)((bits >> 16) & 0x8000);
  float a = fabsf(f);
  if (isnan(f))
    return sign | 0x7E00;
  if (a >= 65520.0f)
    return sign | 0x7C00; /* rounds to infinity */
  if (a == 0.0f)
    return sign;
  int e;
  frexpf(a, &e);
  int ue = e - 1;
  if (ue < -14)
    ue = -14;
  float r = nearbyintf(ldexpf(a, 10 - ue));
  int mant = (int)r, biased = ue + 15;
  if (ue == -14 && mant < 1024) {
    biased = 0;
  } else {
    if (mant >= 2048) {
      mant >>= 1;
      biased += 1;
    }
    mant -= 1024;
  }
  return sign | (uint16_t)((biased << 10) | mant);
}

/* array forms, for the input generators of tests and bench */
void oracle_encode_e4m3_array(const float *x, uint8_t *y, size_t n) {
  for (size_t i = 0; i < n; i++)
    y[i] = oracle_encode_e4m3(x[i]);
}
void oracle_encode_e5m2_array(const float *x, uint8_t *y, size_t n) {
  for (size_t i = 0; i < n; i++)
    y[i] = oracle_encode_e5m2(x[i]);
}
void oracle_encode_bf16_array(const float *x, uint16_t *y, size_t n) {
  for (size_t i = 0; i < n; i++)
    y[i] = oracle_encode_bf16(x[i]);
}
void oracle_decode_bf16_array(const uint16_t *x, float *y, size_t n) {
  for (size_t i = 0; i < n; i++)
    y[i] = oracle_decode_bf16(x[i]);
}
void oracle_encode_f16_array(const float *x, uint16_t *y, size_t n) {
  for (size_t i = 0; i < n; i++)
    y[i] = oracle_encode_f16(x[i]);
}
/* x: [rows][k] floats (k % 32 == 0).  Writes packed E2M1 (two per byte, low nibble = even k)
 * into q[rows][k/2] and one UE8M0 byte per 32-block into s[rows][k/32]; the block exponent is
 * floor(log2(max|x|)) - 2 (E2M1's largest exponent), clamped to the UE8M0 range. */
void oracle_quantize_mxfp4(const float *x, uint8_t *q, uint8_t *s, size_t rows, size_t k) {
  for (size_t r = 0; r < rows; r++)
    for (size_t kb = 0; kb < k / 32; kb++) {
      const float *blk = x + r * k + kb * 32;
      float mx = 0.0f;
      for (int t = 0; t < 32; t++)
        mx = fmaxf(mx, fabsf(blk[t]));
      int e = -127;
      if (mx > 0.0f) {
        int fe;
        frexpf(mx, &fe);
        e = (fe - 1) - 2;
        if (e < -127) e = -127;
        if (e > 127) e = 127;
      }
      s[r * (k / 32) + kb] = (uint8_t)(e + 127);
      for (int t = 0; t < 32; t += 2) {
        uint8_t lo = oracle_encode_e2m1(ldexpf(blk[t], -e));
        uint8_t hi = oracle_encode_e2m1(ldexpf(blk[t + 1], -e));
        q[r * (k / 2) + kb * 16 + t / 2] = (uint8_t)(lo | (hi << 4));
      }
    }
}

/* tanh-form GELU (see the header: which form hipBLASLt applies is checked on the GPU box). */
float oracle_gelu(float x) {
  const float k0 = 0.7978845608028654f, k1 = 0.044715f;
  return 0.5f * x * (1.0f + tanhf(k0 * (x + k1 * x * x * x)));
}

/* its derivative: 0.5 (1 + tanh u) + 0.5 x (1 - tanh^2 u) u'(x),  u = k0 (x + k1 x^3) */
float oracle_dgelu(float x) {
  const double k0 = 0.7978845608028654, k1 = 0.044715, xd = x;
  const double t = tanh(k0 * (xd + k1 * xd * xd * xd));
  return (float)(0.5 * (1.0 + t) + 0.5 * xd * (1.0 - t * t) * k0 * (1.0 + 3.0 * k1 * xd * xd));
}

/* ------------------------------------------------------------------ element access ------- */

static size_t type_bits(uint32_t t) {
  switch (t) {
  case CUDA_R_32F: case CUDA_R_32I: return 32;
  case CUDA_R_16F: case CUDA_R_16BF: return 16;
  case CUDA_R_8I: case CUDA_R_8F_E4M3: case CUDA_R_8F_E5M2: case CUDA_R_8F_UE8M0: return 8;
  case CUDA_R_4F_E2M1: return 4;
  default: return 0;
  }
}


/* linear element index of stored element (r, c) */
static int64_t elem_index(const zluda_matrix_layout *l, int64_t r, int64_t c) {
  return l->order == CUBLASLT_ORDER_ROW ? r * l->ld + c : r + c * l->ld;
}

static float load_as_float(const void *base, uint32_t type, int64_t idx) {
  switch (type) {
  case CUDA_R_32F: return ((const float *)base)[idx];
  case CUDA_R_32I: return (float)((const int32_t *)base)[idx];
  case CUDA_R_16F: return oracle_decode_f16(((const uint16_t *)base)[idx]);
  case CUDA_R_16BF: return oracle_decode_bf16(((const uint16_t *)base)[idx]);
  case CUDA_R_8I: return (float)((const int8_t *)base)[idx];
  case CUDA_R_8F_E4M3: return oracle_decode_e4m3(((const uint8_t *)base)[idx]);
  case CUDA_R_8F_E5M2: return oracle_decode_e5m2(((const uint8_t *)base)[idx]);
  case CUDA_R_4F_E2M1: {
    uint8_t byte = ((const uint8_t *)base)[idx >> 1];
    return oracle_decode_e2m1((idx & 1) ? (byte >> 4) : (byte & 15));
  }
  default: return NAN;
  }
}

static int32_t sat_i32(float x) {
  if (isnan(x)) return 0;
  float r = nearbyintf(x);
  if (r >= 2147483648.0f) return INT32_MAX;
  if (r <= -2147483648.0f) return INT32_MIN;
  return (int32_t)r;
}

static void store_from_float(void *base, uint32_t type, int64_t idx, float x) {
  switch (type) {
  case CUDA_R_32F: ((float *)base)[idx] = x; break;
  case CUDA_R_32I: ((int32_t *)base)[idx] = sat_i32(x); break;
  case CUDA_R_16F: ((uint16_t *)base)[idx] = oracle_encode_f16(x); break;
  case CUDA_R_16BF: ((uint16_t *)base)[idx] = oracle_encode_bf16(x); break;
  case CUDA_R_8I: {
    float r = isnan(x) ? 0.0f : nearbyintf(x);
    r = r > 127.0f ? 127.0f : (r < -128.0f ? -128.0f : r);
    ((int8_t *)base)[idx] = (int8_t)r;
    break;
  }
  case CUDA_R_8F_E4M3: ((uint8_t *)base)[idx] = oracle_encode_e4m3(x); break;
  case CUDA_R_8F_E5M2: ((uint8_t *)base)[idx] = oracle_encode_e5m2(x); break;
  default: break;
  }
}

/* ------------------------------------------------------------------ the GEMM -------------- */

/* All pointers in `p` are HOST pointers here, whatever op.pointer_mode says about the device.
 * Returns a cublasStatus_t. */
uint32_t oracle_gemm(const zluda_gemm_problem *p) {
  const zluda_matmul_desc *op = &p->op;
  const int ta = op->transa != CUBLAS_OP_N, tb = op->transb != CUBLAS_OP_N;
  const int64_t M = (int64_t)p->d.rows, N = (int64_t)p->d.cols;
  const int64_t K = (int64_t)(ta ? p->a.rows : p->a.cols);
  if ((int64_t)(ta ? p->a.cols : p->a.rows) != M) return CUBLAS_STATUS_INVALID_VALUE;
  if ((int64_t)(tb ? p->b.cols : p->b.rows) != K) return CUBLAS_STATUS_INVALID_VALUE;
  if ((int64_t)(tb ? p->b.rows : p->b.cols) != N) return CUBLAS_STATUS_INVALID_VALUE;
  if (!type_bits(p->a.type) || !type_bits(p->b.type) || !type_bits(p->d.type))
    return CUBLAS_STATUS_NOT_SUPPORTED;
  const int int_path = op->compute_type == CUBLAS_COMPUTE_32I ||
                       op->compute_type == CUBLAS_COMPUTE_32I_PEDANTIC;
  if (int_path && !(p->a.type == CUDA_R_8I && p->b.type == CUDA_R_8I))
    return CUBLAS_STATUS_NOT_SUPPORTED;
  const int int_scale = op->scale_type == CUDA_R_32I;
  if (int_scale && !(int_path && p->d.type == CUDA_R_32I && op->epilogue == CUBLASLT_EPILOGUE_DEFAULT))
    return CUBLAS_STATUS_NOT_SUPPORTED;
  if (!int_scale && op->scale_type != CUDA_R_32F) return CUBLAS_STATUS_NOT_SUPPORTED;

  const int a_blk = op->a_scale_mode == CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0;
  const int b_blk = op->b_scale_mode == CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0;
  if ((a_blk || b_blk) && (K % 32)) return CUBLAS_STATUS_INVALID_VALUE;
  const int64_t KB = K / 32;

  const int pm = op->pointer_mode;
  const int alpha_vec = pm == CUBLASLT_POINTER_MODE_DEVICE_VECTOR ||
                        pm == CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO ||
                        pm == CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_HOST;
  const int beta_vec = pm == CUBLASLT_POINTER_MODE_DEVICE_VECTOR;
  const int beta_zero = pm == CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO;

  const uint32_t epi = op->epilogue;
  /* GELU_AUX[_BIAS] (cuda_types/src/cublaslt.rs:4601-4619): as GELU[_BIAS], and the GELU input also goes to the aux
   * matrix; DGELU[_BGRAD] (:4621-4660): D = gelu'(aux) * (alpha AB + beta C), _BGRAD: the sums of D's rows go to
   * the bias buffer.  The aux matrix has D's type and order, leading dimension and batch stride from the
   * descriptor (:4182-4236). */
  const int gelu_aux = epi == CUBLASLT_EPILOGUE_GELU_AUX || epi == CUBLASLT_EPILOGUE_GELU_AUX_BIAS;
  const int dgelu = epi == CUBLASLT_EPILOGUE_DGELU || epi == CUBLASLT_EPILOGUE_DGELU_BGRAD;
  const int dgelu_bgrad = epi == CUBLASLT_EPILOGUE_DGELU_BGRAD;
  const int has_bias = epi == CUBLASLT_EPILOGUE_BIAS || epi == CUBLASLT_EPILOGUE_RELU_BIAS ||
                       epi == CUBLASLT_EPILOGUE_GELU_BIAS || epi == CUBLASLT_EPILOGUE_GELU_AUX_BIAS;
  const int relu = epi == CUBLASLT_EPILOGUE_RELU || epi == CUBLASLT_EPILOGUE_RELU_BIAS;
  const int gelu = epi == CUBLASLT_EPILOGUE_GELU || epi == CUBLASLT_EPILOGUE_GELU_BIAS || gelu_aux;
  /* BGRADA / BGRADB (cuda_types/src/cublaslt.rs:4636-4654): D as with DEFAULT; the bias buffer receives the
   * sums over K of op(A)'s rows (M values) / of op(B)'s columns (N values), in the bias data type */
  const int bgrad = epi == CUBLASLT_EPILOGUE_BGRADA ? 1 : epi == CUBLASLT_EPILOGUE_BGRADB ? 2 : 0;
  if (!(epi == CUBLASLT_EPILOGUE_DEFAULT || has_bias || relu || gelu || bgrad || dgelu))
    return CUBLAS_STATUS_NOT_SUPPORTED;
  if (gelu_aux || dgelu) {
    const int64_t lead = p->d.order == CUBLASLT_ORDER_ROW ? N : M;
    if (int_scale || !(p->d.type == CUDA_R_32F || p->d.type == CUDA_R_16F || p->d.type == CUDA_R_16BF))
      return CUBLAS_STATUS_NOT_SUPPORTED;
    if (!op->epilogue_aux || op->epilogue_aux_ld < lead) return CUBLAS_STATUS_INVALID_VALUE;
    if (dgelu && op->d_scale) return CUBLAS_STATUS_NOT_SUPPORTED;
    if (dgelu_bgrad && !op->bias) return CUBLAS_STATUS_INVALID_VALUE;
  }
  if (bgrad && (a_blk || b_blk || op->a_scale || op->b_scale || !op->bias)) return CUBLAS_STATUS_NOT_SUPPORTED;
  uint32_t bias_type = op->bias_type >= 0 ? (uint32_t)op->bias_type
                       : (p->d.type == CUDA_R_8I || p->d.type == CUDA_R_32I ||
                          p->d.type == CUDA_R_8F_E4M3 || p->d.type == CUDA_R_8F_E5M2)
                           ? CUDA_R_32F
                           : p->d.type;

  const int batch = p->d.batch_count > 0 ? p->d.batch_count : 1;
  if ((bgrad || dgelu_bgrad) && batch > 1 && op->bias_batch_stride == 0) return CUBLAS_STATUS_NOT_SUPPORTED; /* aliased outputs */
  if (gelu_aux && batch > 1 && op->epilogue_aux_batch_stride == 0) return CUBLAS_STATUS_NOT_SUPPORTED;
  zluda_matrix_layout auxl = p->d;   /* D's type and order with the aux matrix's own pitch */
  auxl.ld = op->epilogue_aux_ld;
  double *rowsum = dgelu_bgrad ? (double *)calloc((size_t)M, sizeof(double)) : NULL;
  const zluda_matrix_layout *cl = p->C ? &p->c : &p->d;

  /* dense K-contiguous copies of op(A) [M][K] and op(B) [N][K] for one batch */
  float *fa = NULL, *fb = NULL;
  int8_t *ia = NULL, *ib = NULL;
  if (int_path) {
    ia = (int8_t *)malloc((size_t)(M * K) + 1);
    ib = (int8_t *)malloc((size_t)(N * K) + 1);
  } else {
    fa = (float *)malloc(sizeof(float) * (size_t)(M * K) + 4);
    fb = (float *)malloc(sizeof(float) * (size_t)(N * K) + 4);
  }

  for (int bt = 0; bt < batch; bt++) {
    const int64_t aoff = p->a.batch_stride * bt, boff = p->b.batch_stride * bt;
    const int64_t coff = cl->batch_stride * bt, doff = p->d.batch_stride * bt;
    const uint8_t *sa_blk = a_blk ? (const uint8_t *)op->a_scale + (size_t)bt * M * KB : NULL;
    const uint8_t *sb_blk = b_blk ? (const uint8_t *)op->b_scale + (size_t)bt * N * KB : NULL;

#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < M; i++)
      for (int64_t k = 0; k < K; k++) {
        int64_t idx = aoff + (ta ? elem_index(&p->a, k, i) : elem_index(&p->a, i, k));
        if (int_path)
          ia[i * K + k] = ((const int8_t *)p->A)[idx];
        else {
          float v = load_as_float(p->A, p->a.type, idx);
          if (a_blk) v *= oracle_decode_ue8m0(sa_blk[i * KB + k / 32]);
          fa[i * K + k] = v;
        }
      }
#pragma omp parallel for schedule(static)
    for (int64_t j = 0; j < N; j++)
      for (int64_t k = 0; k < K; k++) {
        int64_t idx = boff + (tb ? elem_index(&p->b, j, k) : elem_index(&p->b, k, j));
        if (int_path)
          ib[j * K + k] = ((const int8_t *)p->B)[idx];
        else {
          float v = load_as_float(p->B, p->b.type, idx);
          if (b_blk) v *= oracle_decode_ue8m0(sb_blk[j * KB + k / 32]);
          fb[j * K + k] = v;
        }
      }

    if (bgrad) {
      const int64_t R = bgrad == 1 ? M : N;
      for (int64_t r = 0; r < R; r++) {
        double s = 0.0;
        for (int64_t k = 0; k < K; k++)
          s += int_path ? (double)(bgrad == 1 ? ia : ib)[r * K + k] : (double)(bgrad == 1 ? fa : fb)[r * K + k];
        store_from_float((void *)op->bias, bias_type, r + op->bias_batch_stride * bt, (float)s);
      }
    }

    if (rowsum) memset(rowsum, 0, sizeof(double) * (size_t)M);
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t j = 0; j < N; j++) {
      for (int64_t i = 0; i < M; i++) {
        int32_t iacc = 0;
        double dacc = 0.0;
        if (int_path) {
          const int8_t *ra = ia + i * K, *rb = ib + j * K;
          int32_t s = 0;
          for (int64_t k = 0; k < K; k++)
            s += (int32_t)ra[k] * (int32_t)rb[k];
          iacc = s;
        } else {
          const float *ra = fa + i * K, *rb = fb + j * K;
          double s = 0.0;
          for (int64_t k = 0; k < K; k++)
            s += (double)ra[k] * (double)rb[k];
          dacc = s;
        }
        const int64_t didx = doff + elem_index(&p->d, i, j);
        const int64_t cidx = coff + elem_index(cl, i, j);
        if (int_scale) {
          /* alpha, beta int32; wrap-around arithmetic like the hardware's */
          int32_t al = alpha_vec ? ((const int32_t *)p->alpha)[i + op->alpha_vector_batch_stride * bt]
                                 : *(const int32_t *)p->alpha;
          int32_t be = beta_zero ? 0 : beta_vec ? ((const int32_t *)p->beta)[i] : *(const int32_t *)p->beta;
          uint32_t r = (uint32_t)al * (uint32_t)iacc;
          if (be != 0 && p->C)
            r += (uint32_t)be * (uint32_t)((const int32_t *)p->C)[cidx];
          else if (be != 0)
            r += (uint32_t)be * (uint32_t)((const int32_t *)p->D)[cidx];
          ((int32_t *)p->D)[didx] = (int32_t)r;
          continue;
        }
        float acc = int_path ? (float)iacc : (float)dacc;
        float al = alpha_vec ? ((const float *)p->alpha)[i + op->alpha_vector_batch_stride * bt]
                             : *(const float *)p->alpha;
        float be = beta_zero ? 0.0f : beta_vec ? ((const float *)p->beta)[i] : *(const float *)p->beta;
        float sa = 1.0f, sb = 1.0f, sc = 1.0f, sd = 1.0f;
        if (op->a_scale && !a_blk)
          sa = op->a_scale_mode == CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F
                   ? ((const float *)op->a_scale)[i] : *(const float *)op->a_scale;
        if (op->b_scale && !b_blk)
          sb = op->b_scale_mode == CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F
                   ? ((const float *)op->b_scale)[j] : *(const float *)op->b_scale;
        if (op->c_scale) sc = *(const float *)op->c_scale;
        if (op->d_scale) sd = *(const float *)op->d_scale;
        float x = (al * sa * sb) * acc;
        if (be != 0.0f) {
          const void *cbase = p->C ? p->C : (const void *)p->D;
          x += be * sc * load_as_float(cbase, cl->type, cidx);
        }
        if (has_bias)
          x += load_as_float(op->bias, bias_type, i + op->bias_batch_stride * bt);
        if (relu) x = x > 0.0f ? x : 0.0f;
        const int64_t auxidx = op->epilogue_aux_batch_stride * bt + elem_index(&auxl, i, j);
        if (gelu_aux) store_from_float(op->epilogue_aux, p->d.type, auxidx, x);
        if (gelu) x = oracle_gelu(x);
        if (dgelu) {
          x *= oracle_dgelu(load_as_float(op->epilogue_aux, p->d.type, auxidx));
          if (rowsum) {
#pragma omp atomic
            rowsum[i] += (double)x;
          }
        }
        x *= sd;
        store_from_float(p->D, p->d.type, didx, x);
      }
    }
    if (rowsum)
      for (int64_t i = 0; i < M; i++)
        store_from_float((void *)op->bias, bias_type, i + op->bias_batch_stride * bt, (float)rowsum[i]);
  }
  free(rowsum);
  free(fa); free(fb); free(ia); free(ib);
  return CUBLAS_STATUS_SUCCESS;
}
