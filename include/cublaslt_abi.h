/*
 * cublaslt_abi.h -- the C ABI of libcublasLt.so as ZLUDA's zluda_blaslt crate exports it.
 *
 * This header restates, without any CUDA header, the constants, structs and the 45 exported
 * functions a CUDA application (or ZLUDA's own zluda_blas / zluda_trace_blaslt) binds when it
 * loads libcublasLt.so.  Every value is cited to the file:line of the reference tree that
 * defines it (paths relative to the ZLUDA source root).
 *
 * Status of each export in this library:
 *   [live]   implemented (the 13 the reference forwards + the 5 "unmapped" helpers)
 *   [ext]    implemented here although the reference returns NOT_SUPPORTED (Get-attribute,
 *            AlgoCheck ... the calls that surround cublasLtMatmul in real applications)
 *   [n/s]    returns CUBLAS_STATUS_NOT_SUPPORTED exactly like the reference's release build
 *            (zluda_blaslt/src/impl.rs:78-86)
 */
#ifndef ZLUDA_AMD_CUBLASLT_ABI_H
#define ZLUDA_AMD_CUBLASLT_ABI_H

#include <stddef.h>
#include <stdint.h>
#include <stdio.h>

#ifdef __cplusplus
extern "C" {
#endif
/* the declarations below are the library's exported symbols (it is built with -fvisibility=hidden) */
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

/* ---- cublasStatus_t : cuda_types/src/cublas.rs:322-350 ---------------------------------- */
typedef uint32_t cublasStatus_t;
#define CUBLAS_STATUS_SUCCESS 0u
#define CUBLAS_STATUS_NOT_INITIALIZED 1u
#define CUBLAS_STATUS_ALLOC_FAILED 3u
#define CUBLAS_STATUS_INVALID_VALUE 7u
#define CUBLAS_STATUS_ARCH_MISMATCH 8u
#define CUBLAS_STATUS_MAPPING_ERROR 11u
#define CUBLAS_STATUS_EXECUTION_FAILED 13u
#define CUBLAS_STATUS_INTERNAL_ERROR 14u
#define CUBLAS_STATUS_NOT_SUPPORTED 15u
#define CUBLAS_STATUS_LICENSE_ERROR 16u

/* CUBLAS_VERSION : cuda_types/src/cublas.rs:15-19 */
#define ZLUDA_CUBLAS_VERSION 130002u

/* ---- cublasOperation_t : cuda_types/src/cublas.rs:50-67 --------------------------------- */
typedef uint32_t cublasOperation_t;
#define CUBLAS_OP_N 0u
#define CUBLAS_OP_T 1u
#define CUBLAS_OP_C 2u

/* ---- cublasComputeType_t : cuda_types/src/cublas.rs:248-292 ------------------------------ */
typedef uint32_t cublasComputeType_t;
#define CUBLAS_COMPUTE_16F 64u
#define CUBLAS_COMPUTE_16F_PEDANTIC 65u
#define CUBLAS_COMPUTE_32F 68u
#define CUBLAS_COMPUTE_32F_PEDANTIC 69u
#define CUBLAS_COMPUTE_64F 70u
#define CUBLAS_COMPUTE_64F_PEDANTIC 71u
#define CUBLAS_COMPUTE_32I 72u
#define CUBLAS_COMPUTE_32I_PEDANTIC 73u
#define CUBLAS_COMPUTE_32F_FAST_16F 74u
#define CUBLAS_COMPUTE_32F_FAST_16BF 75u
#define CUBLAS_COMPUTE_32F_FAST_TF32 77u

/* ---- cudaDataType : cuda_types/src/cuda.rs:8690-8806 ------------------------------------- */
typedef uint32_t cudaDataType_t;
#define CUDA_R_32F 0u
#define CUDA_R_64F 1u
#define CUDA_R_16F 2u
#define CUDA_R_8I 3u
#define CUDA_R_8U 8u
#define CUDA_R_32I 10u
#define CUDA_R_16BF 14u
#define CUDA_R_8F_E4M3 28u
#define CUDA_R_8F_E5M2 29u
#define CUDA_R_8F_UE8M0 30u
#define CUDA_R_6F_E2M3 31u
#define CUDA_R_6F_E3M2 32u
#define CUDA_R_4F_E2M1 33u

/* ---- cublasLtMatrixLayoutAttribute_t : cuda_types/src/cublaslt.rs:3981-4075 -------------- */
typedef uint32_t cublasLtMatrixLayoutAttribute_t;
#define CUBLASLT_MATRIX_LAYOUT_TYPE 0u                 /* uint32_t */
#define CUBLASLT_MATRIX_LAYOUT_ORDER 1u                /* int32_t  */
#define CUBLASLT_MATRIX_LAYOUT_ROWS 2u                 /* uint64_t */
#define CUBLASLT_MATRIX_LAYOUT_COLS 3u                 /* uint64_t */
#define CUBLASLT_MATRIX_LAYOUT_LD 4u                   /* int64_t  */
#define CUBLASLT_MATRIX_LAYOUT_BATCH_COUNT 5u          /* int32_t  */
#define CUBLASLT_MATRIX_LAYOUT_STRIDED_BATCH_OFFSET 6u /* int64_t, in elements */
#define CUBLASLT_MATRIX_LAYOUT_PLANE_OFFSET 7u
#define CUBLASLT_MATRIX_LAYOUT_BATCH_MODE 8u

/* ---- cublasLtOrder_t : cuda_types/src/cublaslt.rs:3923-3961 ------------------------------ */
#define CUBLASLT_ORDER_COL 0
#define CUBLASLT_ORDER_ROW 1
#define CUBLASLT_ORDER_COL32 2
#define CUBLASLT_ORDER_COL4_4R2_8C 3
#define CUBLASLT_ORDER_COL32_2R_4R4 4

/* ---- cublasLtMatmulDescAttributes_t : cuda_types/src/cublaslt.rs:4080-4470 --------------- */
typedef uint32_t cublasLtMatmulDescAttributes_t;
#define CUBLASLT_MATMUL_DESC_COMPUTE_TYPE 0u  /* int32_t */
#define CUBLASLT_MATMUL_DESC_SCALE_TYPE 1u    /* int32_t */
#define CUBLASLT_MATMUL_DESC_POINTER_MODE 2u  /* int32_t */
#define CUBLASLT_MATMUL_DESC_TRANSA 3u        /* int32_t */
#define CUBLASLT_MATMUL_DESC_TRANSB 4u        /* int32_t */
#define CUBLASLT_MATMUL_DESC_TRANSC 5u        /* int32_t */
#define CUBLASLT_MATMUL_DESC_FILL_MODE 6u
#define CUBLASLT_MATMUL_DESC_EPILOGUE 7u      /* uint32_t */
#define CUBLASLT_MATMUL_DESC_BIAS_POINTER 8u  /* void*    */
#define CUBLASLT_MATMUL_DESC_BIAS_BATCH_STRIDE 10u /* int64_t */
#define CUBLASLT_MATMUL_DESC_EPILOGUE_AUX_POINTER 11u
#define CUBLASLT_MATMUL_DESC_EPILOGUE_AUX_LD 12u
#define CUBLASLT_MATMUL_DESC_EPILOGUE_AUX_BATCH_STRIDE 13u
#define CUBLASLT_MATMUL_DESC_ALPHA_VECTOR_BATCH_STRIDE 14u /* int64_t */
#define CUBLASLT_MATMUL_DESC_SM_COUNT_TARGET 15u /* int32_t */
#define CUBLASLT_MATMUL_DESC_A_SCALE_POINTER 17u /* void* */
#define CUBLASLT_MATMUL_DESC_B_SCALE_POINTER 18u
#define CUBLASLT_MATMUL_DESC_C_SCALE_POINTER 19u
#define CUBLASLT_MATMUL_DESC_D_SCALE_POINTER 20u
#define CUBLASLT_MATMUL_DESC_AMAX_D_POINTER 21u
#define CUBLASLT_MATMUL_DESC_EPILOGUE_AUX_DATA_TYPE 22u
#define CUBLASLT_MATMUL_DESC_EPILOGUE_AUX_SCALE_POINTER 23u
#define CUBLASLT_MATMUL_DESC_EPILOGUE_AUX_AMAX_POINTER 24u
#define CUBLASLT_MATMUL_DESC_FAST_ACCUM 25u       /* int8_t  */
#define CUBLASLT_MATMUL_DESC_BIAS_DATA_TYPE 26u   /* int32_t, default -1 = type of D */
#define CUBLASLT_MATMUL_DESC_A_SCALE_MODE 31u     /* int32_t */
#define CUBLASLT_MATMUL_DESC_B_SCALE_MODE 32u
#define CUBLASLT_MATMUL_DESC_C_SCALE_MODE 33u
#define CUBLASLT_MATMUL_DESC_D_SCALE_MODE 34u
#define CUBLASLT_MATMUL_DESC_EPILOGUE_AUX_SCALE_MODE 35u
#define CUBLASLT_MATMUL_DESC_D_OUT_SCALE_POINTER 36u
#define CUBLASLT_MATMUL_DESC_D_OUT_SCALE_MODE 37u

/* ---- cublasLtPointerMode_t : cuda_types/src/cublaslt.rs:3853-3887 ------------------------ */
#define CUBLASLT_POINTER_MODE_HOST 0
#define CUBLASLT_POINTER_MODE_DEVICE 1
#define CUBLASLT_POINTER_MODE_DEVICE_VECTOR 2
#define CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO 3
#define CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_HOST 4

/* ---- cublasLtMatmulMatrixScale_t : cuda_types/src/cublaslt.rs:3800-3852 ------------------ */
#define CUBLASLT_MATMUL_MATRIX_SCALE_SCALAR_32F 0
#define CUBLASLT_MATMUL_MATRIX_SCALE_VEC16_UE4M3 1
#define CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0 2
#define CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F 3
#define CUBLASLT_MATMUL_MATRIX_SCALE_VEC128_32F 4
#define CUBLASLT_MATMUL_MATRIX_SCALE_BLK128x128_32F 5

/* ---- cublasLtEpilogue_t : cuda_types/src/cublaslt.rs:4547-4660 --------------------------- */
typedef uint32_t cublasLtEpilogue_t;
#define CUBLASLT_EPILOGUE_DEFAULT 1u
#define CUBLASLT_EPILOGUE_RELU 2u
#define CUBLASLT_EPILOGUE_BIAS 4u
#define CUBLASLT_EPILOGUE_RELU_BIAS 6u
#define CUBLASLT_EPILOGUE_GELU 32u
#define CUBLASLT_EPILOGUE_GELU_BIAS 36u
#define CUBLASLT_EPILOGUE_RELU_AUX 130u
#define CUBLASLT_EPILOGUE_RELU_AUX_BIAS 134u
#define CUBLASLT_EPILOGUE_DRELU 136u
#define CUBLASLT_EPILOGUE_DRELU_BGRAD 152u
#define CUBLASLT_EPILOGUE_GELU_AUX 160u
#define CUBLASLT_EPILOGUE_GELU_AUX_BIAS 164u
#define CUBLASLT_EPILOGUE_DGELU 192u
#define CUBLASLT_EPILOGUE_DGELU_BGRAD 208u
#define CUBLASLT_EPILOGUE_BGRADA 256u
#define CUBLASLT_EPILOGUE_BGRADB 512u

/* ---- cublasLtMatmulPreferenceAttributes_t : cuda_types/src/cublaslt.rs:4725-4820 --------- */
typedef uint32_t cublasLtMatmulPreferenceAttributes_t;
#define CUBLASLT_MATMUL_PREF_SEARCH_MODE 0u          /* uint32_t */
#define CUBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES 1u  /* uint64_t */
#define CUBLASLT_MATMUL_PREF_REDUCTION_SCHEME_MASK 3u
#define CUBLASLT_MATMUL_PREF_MIN_ALIGNMENT_A_BYTES 5u /* uint32_t */
#define CUBLASLT_MATMUL_PREF_MIN_ALIGNMENT_B_BYTES 6u
#define CUBLASLT_MATMUL_PREF_MIN_ALIGNMENT_C_BYTES 7u
#define CUBLASLT_MATMUL_PREF_MIN_ALIGNMENT_D_BYTES 8u
#define CUBLASLT_MATMUL_PREF_MAX_WAVES_COUNT 9u      /* float */
#define CUBLASLT_MATMUL_PREF_IMPL_MASK 12u           /* uint64_t */

/* ---- opaque handles: cuda_types/src/cublaslt.rs:38-83 ------------------------------------ */
typedef struct cublasLtContext *cublasLtHandle_t;
typedef struct cublasLtMatmulDescOpaque_st *cublasLtMatmulDesc_t;
typedef struct cublasLtMatrixLayoutOpaque_st *cublasLtMatrixLayout_t;
typedef struct cublasLtMatmulPreferenceOpaque_st *cublasLtMatmulPreference_t;
typedef struct cublasLtMatrixTransformDescOpaque_st *cublasLtMatrixTransformDesc_t;
typedef void *cudaStream_t; /* a raw hipStream_t: zluda_common/src/lib.rs:264 */
typedef uint32_t libraryPropertyType;
typedef uint32_t cublasLtMatrixTransformDescAttributes_t;
typedef uint32_t cublasLtMatmulAlgoCapAttributes_t;
typedef uint32_t cublasLtMatmulAlgoConfigAttributes_t;
typedef void (*cublasLtLoggerCallback_t)(int logLevel, const char *functionName, const char *message);

/* cuda_types/src/cublaslt.rs:55-59 : 64 opaque bytes passed by pointer */
typedef struct cublasLtMatmulAlgo_st {
  uint64_t data[8];
} cublasLtMatmulAlgo_t;

/* cuda_types/src/cublaslt.rs:4825-4841 : 96 bytes */
typedef struct cublasLtMatmulHeuristicResult_st {
  cublasLtMatmulAlgo_t algo;
  size_t workspaceSize;
  cublasStatus_t state;
  float wavesCount;
  int reserved[4];
} cublasLtMatmulHeuristicResult_t;

/* Handle boxing (zluda_common/src/lib.rs:1036-1041): a handle is the address of
 * { size_t cookie; payload }.  zluda_blaslt/src/impl.rs:24-26 and zluda_common/src/constants.rs:6 */
#define ZLUDA_BLASLT_HANDLE_COOKIE 0xd1d9cb43416c9620ull
#define ZLUDA_BLAS_HANDLE_COOKIE 0x57c3fdb0fd72b08eull

/* ------------------------------------------------------------------------------------------
 * The 45 exports: cuda_macros/src/cublaslt.rs:4-583 (signatures), zluda_blaslt/src/lib.rs:44-70
 * (which are live).
 * ------------------------------------------------------------------------------------------ */

/* [live] zluda_blaslt/src/impl.rs:124-132 */
cublasStatus_t cublasLtCreate(cublasLtHandle_t *lightHandle);
/* [live] zluda_blaslt/src/impl.rs:134-146 ; also accepts a ZLUDA cublasHandle_t */
cublasStatus_t cublasLtDestroy(cublasLtHandle_t lightHandle);
/* [live] zluda_blaslt/src/impl.rs:89-110 */
const char *cublasLtGetStatusName(cublasStatus_t status);
const char *cublasLtGetStatusString(cublasStatus_t status);
/* [live] reference bodies are todo!() (impl.rs:112-122); here: CUBLAS_VERSION / 13000 / no-op */
size_t cublasLtGetVersion(void);
size_t cublasLtGetCudartVersion(void);
unsigned cublasLtDisableCpuInstructionsSetMask(unsigned mask);
/* [ext] */
cublasStatus_t cublasLtGetProperty(libraryPropertyType type, int *value);
/* [n/s] */
cublasStatus_t cublasLtHeuristicsCacheGetCapacity(size_t *capacity);
cublasStatus_t cublasLtHeuristicsCacheSetCapacity(size_t capacity);

/* [live] the hot entry point: zluda_blaslt/src/impl.rs:157-196 (cuda_macros/src/cublaslt.rs:58-75).
 * D = epilogue(alpha * op(A) * op(B) + beta * C), enqueued on `stream`, no implicit sync.
 * algo == NULL is accepted (the library picks its first heuristic choice). */
cublasStatus_t cublasLtMatmul(cublasLtHandle_t lightHandle, cublasLtMatmulDesc_t computeDesc,
                              const void *alpha, const void *A, cublasLtMatrixLayout_t Adesc,
                              const void *B, cublasLtMatrixLayout_t Bdesc, const void *beta,
                              const void *C, cublasLtMatrixLayout_t Cdesc, void *D,
                              cublasLtMatrixLayout_t Ddesc, const cublasLtMatmulAlgo_t *algo,
                              void *workspace, size_t workspaceSizeInBytes, cudaStream_t stream);

/* [n/s] */
cublasStatus_t cublasLtMatrixTransform(cublasLtHandle_t lightHandle,
                                       cublasLtMatrixTransformDesc_t transformDesc,
                                       const void *alpha, const void *A,
                                       cublasLtMatrixLayout_t Adesc, const void *beta,
                                       const void *B, cublasLtMatrixLayout_t Bdesc, void *C,
                                       cublasLtMatrixLayout_t Cdesc, cudaStream_t stream);

/* [ext] initialises caller-provided storage (256 bytes for a matmul descriptor, 64 for a layout or a
 * preference: cuda_types/src/cublaslt.rs:43-83) the way the matching Create call does; such an object
 * is never passed to Destroy.  Unimplemented in the reference (zluda_blaslt/src/lib.rs:44-70). */
cublasStatus_t cublasLtMatrixLayoutInit_internal(cublasLtMatrixLayout_t matLayout, size_t size,
                                                 cudaDataType_t type, uint64_t rows,
                                                 uint64_t cols, int64_t ld);
/* [live] zluda_blaslt/src/impl.rs:360-386 */
cublasStatus_t cublasLtMatrixLayoutCreate(cublasLtMatrixLayout_t *matLayout, cudaDataType_t type,
                                          uint64_t rows, uint64_t cols, int64_t ld);
cublasStatus_t cublasLtMatrixLayoutDestroy(cublasLtMatrixLayout_t matLayout);
cublasStatus_t cublasLtMatrixLayoutSetAttribute(cublasLtMatrixLayout_t matLayout,
                                                cublasLtMatrixLayoutAttribute_t attr,
                                                const void *buf, size_t sizeInBytes);
/* [ext] */
cublasStatus_t cublasLtMatrixLayoutGetAttribute(cublasLtMatrixLayout_t matLayout,
                                                cublasLtMatrixLayoutAttribute_t attr, void *buf,
                                                size_t sizeInBytes, size_t *sizeWritten);

/* [ext] as cublasLtMatrixLayoutInit_internal */
cublasStatus_t cublasLtMatmulDescInit_internal(cublasLtMatmulDesc_t matmulDesc, size_t size,
                                               cublasComputeType_t computeType,
                                               cudaDataType_t scaleType);
/* [live] zluda_blaslt/src/impl.rs:243-328 */
cublasStatus_t cublasLtMatmulDescCreate(cublasLtMatmulDesc_t *matmulDesc,
                                        cublasComputeType_t computeType,
                                        cudaDataType_t scaleType);
cublasStatus_t cublasLtMatmulDescDestroy(cublasLtMatmulDesc_t matmulDesc);
cublasStatus_t cublasLtMatmulDescSetAttribute(cublasLtMatmulDesc_t matmulDesc,
                                              cublasLtMatmulDescAttributes_t attr,
                                              const void *buf, size_t sizeInBytes);
/* [ext] */
cublasStatus_t cublasLtMatmulDescGetAttribute(cublasLtMatmulDesc_t matmulDesc,
                                              cublasLtMatmulDescAttributes_t attr, void *buf,
                                              size_t sizeInBytes, size_t *sizeWritten);

/* [n/s] matrix-transform family */
cublasStatus_t cublasLtMatrixTransformDescInit_internal(cublasLtMatrixTransformDesc_t transformDesc,
                                                        size_t size, cudaDataType_t scaleType);
cublasStatus_t cublasLtMatrixTransformDescCreate(cublasLtMatrixTransformDesc_t *transformDesc,
                                                 cudaDataType_t scaleType);
cublasStatus_t cublasLtMatrixTransformDescDestroy(cublasLtMatrixTransformDesc_t transformDesc);
cublasStatus_t cublasLtMatrixTransformDescSetAttribute(
    cublasLtMatrixTransformDesc_t transformDesc, cublasLtMatrixTransformDescAttributes_t attr,
    const void *buf, size_t sizeInBytes);
cublasStatus_t cublasLtMatrixTransformDescGetAttribute(
    cublasLtMatrixTransformDesc_t transformDesc, cublasLtMatrixTransformDescAttributes_t attr,
    void *buf, size_t sizeInBytes, size_t *sizeWritten);

/* [ext] as cublasLtMatrixLayoutInit_internal */
cublasStatus_t cublasLtMatmulPreferenceInit_internal(cublasLtMatmulPreference_t pref, size_t size);
/* [live] zluda_blaslt/src/impl.rs:330-358 */
cublasStatus_t cublasLtMatmulPreferenceCreate(cublasLtMatmulPreference_t *pref);
cublasStatus_t cublasLtMatmulPreferenceDestroy(cublasLtMatmulPreference_t pref);
cublasStatus_t cublasLtMatmulPreferenceSetAttribute(cublasLtMatmulPreference_t pref,
                                                    cublasLtMatmulPreferenceAttributes_t attr,
                                                    const void *buf, size_t sizeInBytes);
/* [ext] */
cublasStatus_t cublasLtMatmulPreferenceGetAttribute(cublasLtMatmulPreference_t pref,
                                                    cublasLtMatmulPreferenceAttributes_t attr,
                                                    void *buf, size_t sizeInBytes,
                                                    size_t *sizeWritten);

/* [live] zluda_blaslt/src/impl.rs:198-241 (cuda_macros/src/cublaslt.rs:375-386) */
cublasStatus_t cublasLtMatmulAlgoGetHeuristic(
    cublasLtHandle_t lightHandle, cublasLtMatmulDesc_t operationDesc, cublasLtMatrixLayout_t Adesc,
    cublasLtMatrixLayout_t Bdesc, cublasLtMatrixLayout_t Cdesc, cublasLtMatrixLayout_t Ddesc,
    cublasLtMatmulPreference_t preference, int requestedAlgoCount,
    cublasLtMatmulHeuristicResult_t *heuristicResultsArray, int *returnAlgoCount);

/* [ext] algorithm enumeration (cuda_macros/src/cublaslt.rs:397-421): an algorithm id is one of the
 * kernel families of zluda_gemm_launch.h that can run the type combination */
cublasStatus_t cublasLtMatmulAlgoGetIds(cublasLtHandle_t lightHandle,
                                        cublasComputeType_t computeType, cudaDataType_t scaleType,
                                        cudaDataType_t Atype, cudaDataType_t Btype,
                                        cudaDataType_t Ctype, cudaDataType_t Dtype,
                                        int requestedAlgoCount, int *algoIdsArray,
                                        int *returnAlgoCount);
cublasStatus_t cublasLtMatmulAlgoInit(cublasLtHandle_t lightHandle,
                                      cublasComputeType_t computeType, cudaDataType_t scaleType,
                                      cudaDataType_t Atype, cudaDataType_t Btype,
                                      cudaDataType_t Ctype, cudaDataType_t Dtype, int algoId,
                                      cublasLtMatmulAlgo_t *algo);
/* [ext] validates an algo token against the descriptors and reports its workspace */
cublasStatus_t cublasLtMatmulAlgoCheck(cublasLtHandle_t lightHandle,
                                       cublasLtMatmulDesc_t operationDesc,
                                       cublasLtMatrixLayout_t Adesc, cublasLtMatrixLayout_t Bdesc,
                                       cublasLtMatrixLayout_t Cdesc, cublasLtMatrixLayout_t Ddesc,
                                       const cublasLtMatmulAlgo_t *algo,
                                       cublasLtMatmulHeuristicResult_t *result);
/* [ext] capabilities and configuration of an algo token (cuda_macros/src/cublaslt.rs:470-518).  The
 * tile variant is CUBLASLT_ALGO_CONFIG_CUSTOM_OPTION: 0 = planner's choice, v + 1 = variant v. */
cublasStatus_t cublasLtMatmulAlgoCapGetAttribute(const cublasLtMatmulAlgo_t *algo,
                                                 cublasLtMatmulAlgoCapAttributes_t attr, void *buf,
                                                 size_t sizeInBytes, size_t *sizeWritten);
cublasStatus_t cublasLtMatmulAlgoConfigSetAttribute(cublasLtMatmulAlgo_t *algo,
                                                    cublasLtMatmulAlgoConfigAttributes_t attr,
                                                    const void *buf, size_t sizeInBytes);
cublasStatus_t cublasLtMatmulAlgoConfigGetAttribute(const cublasLtMatmulAlgo_t *algo,
                                                    cublasLtMatmulAlgoConfigAttributes_t attr,
                                                    void *buf, size_t sizeInBytes,
                                                    size_t *sizeWritten);
cublasStatus_t cublasLtLoggerSetCallback(cublasLtLoggerCallback_t callback);
cublasStatus_t cublasLtLoggerSetFile(FILE *file);
cublasStatus_t cublasLtLoggerOpenFile(const char *logFile);
cublasStatus_t cublasLtLoggerSetLevel(int level);
cublasStatus_t cublasLtLoggerSetMask(int mask);
cublasStatus_t cublasLtLoggerForceDisable(void);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif
#ifdef __cplusplus
}
#endif
#endif /* ZLUDA_AMD_CUBLASLT_ABI_H */
