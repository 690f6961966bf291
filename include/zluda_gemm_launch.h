/*
 * zluda_gemm_launch.h -- the thin extern "C" launch layer under cublasLtMatmul.
 *
 * This is the inner boundary: plain pointers, sizes and enum numbers in, a cublasStatus_t out.
 * It replaces the single call site `hipblasLtMatmul(...)` of the reference
 * (zluda_blaslt/src/impl.rs:176-193) and needs nothing but the HIP runtime
 * (ext/hip_runtime-sys: hipLaunchKernel, hipMemsetAsync-free).  A Rust body binds these with a
 * `extern "C"` block; the C++ host layer in this repository calls them the same way.
 *
 * All enum-typed fields carry the CUDA-side numeric values of cublaslt_abi.h.
 */
#ifndef ZLUDA_AMD_GEMM_LAUNCH_H
#define ZLUDA_AMD_GEMM_LAUNCH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
/* the declarations below are the library's exported symbols (it is built with -fvisibility=hidden) */
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

/* One matrix operand as cublasLtMatrixLayout_t describes it
 * (cuda_types/src/cublaslt.rs:3981-4058; created by zluda_blaslt/src/impl.rs:360-386). */
typedef struct zluda_matrix_layout {
  uint32_t type;        /* cudaDataType */
  int32_t order;        /* CUBLASLT_ORDER_COL / ROW */
  uint64_t rows, cols;  /* of the stored matrix, before op() */
  int64_t ld;           /* leading dimension in elements */
  int32_t batch_count;  /* >= 1 */
  int64_t batch_stride; /* elements between consecutive matrices */
} zluda_matrix_layout;

/* The operation as cublasLtMatmulDesc_t describes it
 * (cuda_types/src/cublaslt.rs:4080-4470; set by zluda_blaslt/src/impl.rs:257-328). */
typedef struct zluda_matmul_desc {
  uint32_t compute_type; /* cublasComputeType_t */
  uint32_t scale_type;   /* cudaDataType of alpha/beta */
  int32_t pointer_mode;  /* cublasLtPointerMode_t */
  uint32_t transa, transb;
  uint32_t epilogue;     /* cublasLtEpilogue_t */
  const void *bias;      /* device, length = rows of D; with the BGRADA / BGRADB epilogues it is written instead:
                          * the sums over K of op(A)'s rows (rows of D values) / of op(B)'s columns (columns of D) */
  int32_t bias_type;     /* cudaDataType or -1 (= default for the D type) */
  int64_t bias_batch_stride;
  int64_t alpha_vector_batch_stride;
  const void *a_scale, *b_scale, *c_scale, *d_scale; /* device pointers or NULL (= 1) */
  int32_t a_scale_mode, b_scale_mode, c_scale_mode, d_scale_mode;
  int8_t fast_accum;
  /* GELU_AUX / GELU_AUX_BIAS: the GELU input (the value in front of the activation) is also written here;
   * DGELU / DGELU_BGRAD: it is read from here (cuda_types/src/cublaslt.rs:4182-4236).  A matrix of D's
   * type, shape and order with its own leading dimension and batch stride (elements). */
  void *epilogue_aux;
  int64_t epilogue_aux_ld;
  int64_t epilogue_aux_batch_stride;
  int32_t epilogue_aux_type; /* cudaDataType or -1 (= D's type, the only one served: anything else is NOT_SUPPORTED) */
} zluda_matmul_desc;

/* A fully specified matmul: what cublasLtMatmul receives (cuda_macros/src/cublaslt.rs:58-75). */
typedef struct zluda_gemm_problem {
  zluda_matmul_desc op;
  zluda_matrix_layout a, b, c, d;
  const void *alpha, *beta; /* host or device according to op.pointer_mode */
  const void *A, *B, *C;
  void *D;
  void *workspace;
  size_t workspace_size;
} zluda_gemm_problem;

/* Kernel families the planner can choose. */
enum {
  ZLUDA_KERNEL_AUTO = 0,
  ZLUDA_KERNEL_GENERIC = 1,   /* any layout / type: LDS-tiled scalar kernel (correctness net) */
  ZLUDA_KERNEL_MFMA_I8 = 2,   /* v_mfma_i32_32x32x32_i8, K-contiguous A and B */
  ZLUDA_KERNEL_MFMA_F8 = 3,   /* v_mfma_f32_32x32x64_f8f6f4 (e4m3/e5m2) */
  ZLUDA_KERNEL_MFMA_MXF4 = 4, /* v_mfma_scale_f32_32x32x64_f8f6f4, E2M1 + UE8M0/32 */
  ZLUDA_KERNEL_DECODE_W8A8 = 5, /* skinny (<= 64 tokens) int8 / fp8 e4m3 streaming kernel, K split inside the workgroup
                                   (its slab form also streams f16 / bf16 weights) */
  ZLUDA_KERNEL_MFMA_TR8 = 6,  /* int8 / fp8 MFMA with transposing loads: A or B not K-contiguous */
  ZLUDA_KERNEL_MFMA_H16 = 7,  /* v_mfma_f32_32x32x16_f16 / _bf16, K-contiguous A and B of one 16-bit type */
  ZLUDA_KERNEL_MFMA_TR16 = 8, /* f16 / bf16 MFMA with transposing loads: A or B not K-contiguous */
  ZLUDA_KERNEL_MFMA_F32 = 9,  /* v_mfma_f32_32x32x2_f32, K-contiguous f32 A and B */
  ZLUDA_KERNEL_MFMA_TR32 = 10 /* f32 MFMA with transposing loads: A or B not K-contiguous */
};

/* The 64-byte algo blob the application round-trips between the heuristic and cublasLtMatmul
 * (the reference packs hipblasLtMatmulAlgo_t into data[0..2]: zluda_blaslt/src/impl.rs:148-155).
 * Ours: data[0] = magic<<32 | kernel, data[1] = variant, data[2] = workspace bytes. */
#define ZLUDA_ALGO_MAGIC 0x5a4c4441u /* "ZLDA" */
typedef struct zluda_gemm_plan {
  uint32_t kernel;        /* ZLUDA_KERNEL_* */
  uint32_t variant;       /* tile configuration index inside the family */
  uint64_t workspace;     /* bytes of workspace the plan needs */
  uint32_t swapped;       /* 1 if the planner computes D^T = op(B)^T op(A)^T */
  uint32_t grid_x, grid_y, grid_z, block;
  float waves;            /* workgroups / (CUs * resident workgroups per CU) */
} zluda_gemm_plan;

/* Validate `p` and choose a kernel (host only, no GPU needed).  `forced_kernel`/`forced_variant`
 * restrict the choice (ZLUDA_KERNEL_AUTO / -1 = free).  Returns CUBLAS_STATUS_NOT_SUPPORTED when
 * no kernel implements the combination, CUBLAS_STATUS_INVALID_VALUE for inconsistent shapes.
 * Pointers inside `p` are only inspected for NULL-ness and alignment. */
uint32_t zluda_gemm_plan_problem(const zluda_gemm_problem *p, uint32_t forced_kernel,
                                 int32_t forced_variant, uint32_t cu_count,
                                 zluda_gemm_plan *plan);

/* Enqueue the matmul on `stream` (a hipStream_t).  Asynchronous; no allocation; the workspace in
 * `p` must be at least plan->workspace bytes. */
uint32_t zluda_gemm_launch(const zluda_gemm_problem *p, const zluda_gemm_plan *plan,
                           void *stream);

/* zluda_gemm_launch for callers that cannot hand over device scratch and cannot allocate any (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference.  Same arguments and results as zluda_gemm_launch, but split-K partial tiles go to an array of
 * ZLUDA_GEMM_STATIC_SCRATCH_BYTES of device memory that is part of the library image (every device the
 * library runs on holds its own copy until the process ends); `p->workspace` is ignored.  Plan with
 * p->workspace_size = ZLUDA_GEMM_STATIC_SCRATCH_BYTES so that zluda_gemm_plan_problem sizes the split for it;
 * a plan that needs more returns CUBLAS_STATUS_ALLOC_FAILED (3) and launches nothing.  The call allocates and
 * frees nothing.  The first call on a device looks up the array's address, which it will not do while `stream` is
 * being captured (CUBLAS_STATUS_NOT_SUPPORTED): make one call on the device outside the capture first; from then on
 * calls may be captured.  All calls on one device -- replays of a captured graph included -- share that
 * device's array: calls that may overlap on one device (two streams, two threads) race on it and must be
 * serialised by the caller; nothing in it needs clearing between calls. */
#define ZLUDA_GEMM_STATIC_SCRATCH_BYTES (32u << 20)
uint32_t zluda_gemm_launch_noalloc(const zluda_gemm_problem *p, const zluda_gemm_plan *plan,
                                   void *stream);

/* cublasGemmEx / cublasGemmStridedBatchedEx on the same kernels: column-major operands, C is read
 * (when beta != 0) and overwritten, alpha and beta are host scalars of the type the compute type
 * implies (int32 for CUBLAS_COMPUTE_32I*, float for CUBLAS_COMPUTE_32F*).  This is what
 * zluda_blas::gemm_ex / gemm_strided_batched_ex (zluda_blas/src/impl.rs:242-289, 376-432) would call
 * for the integer and 8-bit float cases their rocBLAS mapping rejects today
 * (zluda_common/src/lib.rs:553-564).  batch_count == 1 ignores the strides. */
uint32_t zluda_gemm_strided_batched_ex(uint32_t transa, uint32_t transb, int32_t m, int32_t n, int32_t k,
                                       const void *alpha, const void *A, uint32_t a_type, int64_t lda,
                                       int64_t stride_a, const void *B, uint32_t b_type, int64_t ldb,
                                       int64_t stride_b, const void *beta, void *C, uint32_t c_type,
                                       int64_t ldc, int64_t stride_c, int32_t batch_count,
                                       uint32_t compute_type, void *stream);
uint32_t zluda_gemm_ex(uint32_t transa, uint32_t transb, int32_t m, int32_t n, int32_t k, const void *alpha,
                       const void *A, uint32_t a_type, int64_t lda, const void *B, uint32_t b_type,
                       int64_t ldb, const void *beta, void *C, uint32_t c_type, int64_t ldc,
                       uint32_t compute_type, void *stream);

/* Number of tile configurations (plan.variant values) of a kernel family; 1 for the generic kernel,
 * 0 for an unknown family. */
uint32_t zluda_gemm_variant_count(uint32_t kernel);

/* Number of compute units of the current HIP device (0 when no device is usable). */
uint32_t zluda_gemm_device_cu_count(void);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif
#ifdef __cplusplus
}
#endif
#endif
