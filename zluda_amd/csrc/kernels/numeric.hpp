// Device-side number-format helpers (OCP FP8/FP4/UE8M0, bf16, fp16) and the fused epilogue
//     D(i,j) = cvt( act( alpha_i * sA_i * sB_j * acc + beta_i * sC * C(i,j) + bias_i ) * sD )
// used by every kernel.  cuBLASLt semantics: cuda_types/src/cublaslt.rs:4563-4566 (bias),
// :4609-4610 (GELU_BIAS), :3871-3883 (alpha vector), :3820-3826 (outer-vector scales).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../../include/cublaslt_abi.h"
#include "../gemm_args.hpp"

namespace zluda_amd {

__device__ __forceinline__ float bits2f(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f2bits(float f) { return __builtin_bit_cast(uint32_t, f); }

__device__ __forceinline__ float dec_bf16(uint16_t v) { return bits2f((uint32_t)v << 16); }
// fp32 -> bf16, round to nearest even: gfx950 has the conversion in hardware (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint16_t enc_bf16(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }
// two at once: `lo` in bits 0..15
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  const f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi) {
  return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)lo) | ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)hi) << 16);
}
__device__ __forceinline__ float dec_f16(uint16_t v) {
  return (float)__builtin_bit_cast(_Float16, v);
}
__device__ __forceinline__ uint16_t enc_f16(float f) {
  return __builtin_bit_cast(uint16_t, (_Float16)f);
}

// OCP E4M3 (finite only), E5M2 (IEEE-like), E2M1, UE8M0
__device__ __forceinline__ float dec_e4m3(uint8_t v) {
  uint32_t s = (uint32_t)(v & 0x80) << 24, e = (v >> 3) & 15, m = v & 7;
  float r;
  if (e == 15 && m == 7) return bits2f(s | 0x7FC00000u);
  if (e == 0) r = (float)m * 0.001953125f;              // m * 2^-9
  else r = bits2f(((e + 120u) << 23) | (m << 20));       // 1.m * 2^(e-7)
  return bits2f(f2bits(r) | s);
}
__device__ __forceinline__ float dec_e5m2(uint8_t v) {
  // E5M2 is the top byte of an IEEE half
  return dec_f16((uint16_t)v << 8);
}
__device__ __forceinline__ float dec_e2m1(uint32_t nib) {
  uint32_t e = (nib >> 1) & 3, m = nib & 1;
  float r = e == 0 ? 0.5f * (float)m : bits2f(((e + 126u) << 23) | (m << 22));
  return (nib & 8) ? -r : r;
}
__device__ __forceinline__ float dec_ue8m0(uint8_t v) {
  if (v == 0xFF) return bits2f(0x7FC00000u);
  return v == 0 ? bits2f(0x00400000u) /* 2^-127 */ : bits2f((uint32_t)v << 23);
}

// round-to-nearest-even, saturate-to-finite encoder for E4M3 / E5M2
template <int EBITS, int MBITS, int BIAS>
__device__ __forceinline__ uint8_t enc_small(float f, float maxv, uint8_t max_code, uint8_t nan_code) {
  uint32_t bits = f2bits(f);
  uint8_t sign = (bits >> 31) ? (uint8_t)(1u << (EBITS + MBITS)) : 0;
  float a = __builtin_fabsf(f);
  if (f != f) return sign | nan_code;
  if (a >= maxv) return sign | max_code;
  int ue = (int)((f2bits(a) >> 23) & 0xFF) - 127;
  const int emin = 1 - BIAS;
  if (ue < emin) ue = emin;
  float q = a * bits2f((uint32_t)(127 + MBITS - ue) << 23);
  int mant = (int)__builtin_rintf(q);
  int biased = ue + BIAS;
  if (ue == emin && mant < (1 << MBITS)) {
    biased = 0;
  } else {
    if (mant >= (2 << MBITS)) { mant >>= 1; biased += 1; }
    mant -= (1 << MBITS);
  }
  uint32_t code = (uint32_t)((biased << MBITS) | mant);
  if (code > max_code) code = max_code;
  return sign | (uint8_t)code;
}
__device__ __forceinline__ uint8_t enc_e4m3(float f) { return enc_small<4, 3, 7>(f, 448.0f, 0x7E, 0x7F); }
__device__ __forceinline__ uint8_t enc_e5m2(float f) { return enc_small<5, 2, 15>(f, 57344.0f, 0x7B, 0x7F); }

__device__ __forceinline__ float gelu_tanh(float x) {
  // 0.5 x (1 + tanh(u)) == x * sigmoid(2u) ; u = sqrt(2/pi) (x + 0.044715 x^3)
  // exp(-2u) = exp2(x * (c0 + c1 x^2)) with c0 = -2 sqrt(2/pi) log2(e), c1 = 0.044715 c0: two FMAs, one
  // v_exp_f32, one v_rcp_f32 (1 ulp each, far inside the 16-bit outputs this feeds).  x -> -inf gives
  // exp2 = +inf, rcp = 0, result -0; x -> +inf gives exp2 = 0, result x.
  const float c0 = -2.0f * 0.7978845608028654f * 1.4426950408889634f, c1 = 0.044715f * c0;
  const float z = x * __builtin_fmaf(x * x, c1, c0);
  return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(z));
}

// element loads for C / bias / generic operands
__device__ __forceinline__ float load_elem(const void *base, uint32_t type, int64_t idx) {
  switch (type) {
  case CUDA_R_32F: return ((const float *)base)[idx];
  case CUDA_R_32I: return (float)((const int32_t *)base)[idx];
  case CUDA_R_16F: return dec_f16(((const uint16_t *)base)[idx]);
  case CUDA_R_16BF: return dec_bf16(((const uint16_t *)base)[idx]);
  case CUDA_R_8I: return (float)((const int8_t *)base)[idx];
  case CUDA_R_8F_E4M3: return dec_e4m3(((const uint8_t *)base)[idx]);
  case CUDA_R_8F_E5M2: return dec_e5m2(((const uint8_t *)base)[idx]);
  case CUDA_R_4F_E2M1: {
    uint32_t byte = ((const uint8_t *)base)[idx >> 1];
    return dec_e2m1((idx & 1) ? (byte >> 4) : (byte & 15));
  }
  default: return 0.0f;
  }
}

__device__ __forceinline__ void store_elem(void *base, uint32_t type, int64_t idx, float x) {
  switch (type) {
  case CUDA_R_32F: ((float *)base)[idx] = x; break;
  case CUDA_R_16BF: ((uint16_t *)base)[idx] = enc_bf16(x); break;
  case CUDA_R_16F: ((uint16_t *)base)[idx] = enc_f16(x); break;
  case CUDA_R_32I: {
    float r = __builtin_rintf(x);
    int32_t v = (x != x) ? 0 : r >= 2147483648.0f ? INT32_MAX : r <= -2147483648.0f ? INT32_MIN : (int32_t)r;
    ((int32_t *)base)[idx] = v;
    break;
  }
  case CUDA_R_8I: {
    float r = (x != x) ? 0.0f : __builtin_rintf(x);
    r = r > 127.0f ? 127.0f : (r < -128.0f ? -128.0f : r);
    ((int8_t *)base)[idx] = (int8_t)r;
    break;
  }
  case CUDA_R_8F_E4M3: ((uint8_t *)base)[idx] = enc_e4m3(x); break;
  case CUDA_R_8F_E5M2: ((uint8_t *)base)[idx] = enc_e5m2(x); break;
  default: break;
  }
}

// The scalar factors of a float epilogue, those behind device pointers fetched (a scalar beside a vector is 1).
struct EpilogueScalars {
  float alpha_s, beta_s, sa_s, sb_s, sc, sd;
  __device__ __forceinline__ explicit EpilogueScalars(const GemmArgs &g) {
    alpha_s = beta_s = sa_s = sb_s = sc = sd = 1.0f;
    if (!g.int_scale) {
      if (g.alpha_mode == SCALAR_VALUE) alpha_s = g.alpha_val.f;
      else if (g.alpha_mode == SCALAR_DEV) alpha_s = *(const float *)g.alpha_ptr;
      if (g.beta_mode == SCALAR_VALUE) beta_s = g.beta_val.f;
      else if (g.beta_mode == SCALAR_DEV) beta_s = *(const float *)g.beta_ptr;
      if (g.a_scale_mode == SCALE_SCALAR) sa_s = *(const float *)g.a_scale;
      if (g.b_scale_mode == SCALE_SCALAR) sb_s = *(const float *)g.b_scale;
      if (g.c_scale) sc = *(const float *)g.c_scale;
      if (g.d_scale) sd = *(const float *)g.d_scale;
    }
  }
};

// Per-thread epilogue context: everything that does not depend on (i, j) is read once.
struct Epilogue {
  const GemmArgs &g;
  int64_t bt;
  float alpha_s, beta_s, sa_s, sb_s, sc, sd;
  const float *alpha_v, *beta_v, *sa_v, *sb_v;
  const char *Cb;
  char *Db;

  __device__ __forceinline__ Epilogue(const GemmArgs &g_, int batch) : Epilogue(g_, batch, EpilogueScalars(g_)) {}

  // with the scalars fetched by the caller (a persistent kernel fetches them once, not once per tile)
  __device__ __forceinline__ Epilogue(const GemmArgs &g_, int batch, const EpilogueScalars &s) : g(g_), bt(batch) {
    alpha_v = beta_v = sa_v = sb_v = nullptr;
    alpha_s = s.alpha_s; beta_s = s.beta_s; sa_s = s.sa_s; sb_s = s.sb_s; sc = s.sc; sd = s.sd;
    if (!g.int_scale) {
      if (g.alpha_mode != SCALAR_VALUE && g.alpha_mode != SCALAR_DEV) alpha_v = (const float *)g.alpha_ptr + g.alpha_sb * bt;
      if (g.beta_mode != SCALAR_VALUE && g.beta_mode != SCALAR_DEV) beta_v = (const float *)g.beta_ptr;
      if (g.a_scale_mode == SCALE_OUTER_VEC) sa_v = (const float *)g.a_scale;
      if (g.b_scale_mode == SCALE_OUTER_VEC) sb_v = (const float *)g.b_scale;
    }
  }

  // integer epilogue: D = alpha*acc + beta*C in wrap-around int32
  __device__ __forceinline__ void store_int(int i, int j, int32_t acc) const {
    int32_t al = g.alpha_mode == SCALAR_VALUE ? g.alpha_val.i
                 : g.alpha_mode == SCALAR_DEV ? *(const int32_t *)g.alpha_ptr
                                              : ((const int32_t *)g.alpha_ptr)[i + g.alpha_sb * bt];
    int32_t be = g.beta_mode == SCALAR_VALUE ? g.beta_val.i
                 : g.beta_mode == SCALAR_DEV ? *(const int32_t *)g.beta_ptr
                                             : ((const int32_t *)g.beta_ptr)[i];
    uint32_t r = (uint32_t)al * (uint32_t)acc;
    if (be != 0)
      r += (uint32_t)be * (uint32_t)((const int32_t *)g.C)[g.c_sb * bt + i * g.c_si + j * g.c_sj];
    ((int32_t *)g.D)[g.d_sb * bt + i * g.d_si + j * g.d_sj] = (int32_t)r;
  }

  // row-of-D quantities (alpha_i * sA_i, beta_i, bias_i) and column quantity sB_j
  __device__ __forceinline__ float row_scale(int i) const {
    return (alpha_v ? alpha_v[i] : alpha_s) * (sa_v ? sa_v[i] : sa_s);
  }
  __device__ __forceinline__ float col_scale(int j) const { return sb_v ? sb_v[j] : sb_s; }
  __device__ __forceinline__ float beta_at(int i) const { return beta_v ? beta_v[i] : beta_s; }
  __device__ __forceinline__ float bias_at(int i) const {
    return g.bias ? load_elem(g.bias, g.bias_type, i + g.bias_sb * bt) : 0.0f;
  }

  // The same bias in two steps, for callers that fetch early and convert late (the planner admits
  // fp32, fp16 and bf16 bias vectors): the raw storage bits, then their value.
  __device__ __forceinline__ uint32_t bias_raw(int i) const {
    if (!g.bias) return 0;
    const int64_t idx = i + g.bias_sb * bt;
    return g.bias_type == CUDA_R_32F ? ((const uint32_t *)g.bias)[idx] : (uint32_t)((const uint16_t *)g.bias)[idx];
  }
  __device__ __forceinline__ float bias_from_raw(uint32_t raw) const {
    if (!g.bias) return 0.0f;
    return g.bias_type == CUDA_R_32F ? bits2f(raw) : g.bias_type == CUDA_R_16F ? dec_f16((uint16_t)raw) : dec_bf16((uint16_t)raw);
  }

  __device__ __forceinline__ float finish(float x) const {
    if (g.act == ACT_RELU) x = x > 0.0f ? x : 0.0f;
    else if (g.act == ACT_GELU) x = gelu_tanh(x);
    return x * sd;
  }

  // float epilogue with the per-row / per-column factors supplied by the caller
  __device__ __forceinline__ void store_f(int i, int j, float acc, float rs, float cs, float be,
                                          float bias) const {
    float x = (rs * cs) * acc;
    if (be != 0.0f)
      x += be * sc * load_elem(g.C, g.c_type, g.c_sb * bt + i * g.c_si + j * g.c_sj);
    x += bias;
    store_elem(g.D, g.d_type, g.d_sb * bt + i * g.d_si + j * g.d_sj, finish(x));
  }
  __device__ __forceinline__ void store_f(int i, int j, float acc) const {
    store_f(i, j, acc, row_scale(i), col_scale(j), beta_at(i), bias_at(i));
  }
};

} // namespace zluda_amd
