"""Numeric constants and ctypes structs of the libcublasLt.so C ABI.

Mirrors include/cublaslt_abi.h and include/zluda_gemm_launch.h (which cite the reference's
cuda_types/src/cublaslt.rs, cublas.rs and cuda.rs line by line).
"""
import ctypes as C

# cublasStatus_t -- cuda_types/src/cublas.rs:322-350
CUBLAS_STATUS_SUCCESS = 0
CUBLAS_STATUS_NOT_INITIALIZED = 1
CUBLAS_STATUS_ALLOC_FAILED = 3
CUBLAS_STATUS_INVALID_VALUE = 7
CUBLAS_STATUS_ARCH_MISMATCH = 8
CUBLAS_STATUS_MAPPING_ERROR = 11
CUBLAS_STATUS_EXECUTION_FAILED = 13
CUBLAS_STATUS_INTERNAL_ERROR = 14
CUBLAS_STATUS_NOT_SUPPORTED = 15
CUBLAS_STATUS_LICENSE_ERROR = 16

# cublasOperation_t -- cuda_types/src/cublas.rs:50-67
CUBLAS_OP_N, CUBLAS_OP_T, CUBLAS_OP_C = 0, 1, 2

# cublasComputeType_t -- cuda_types/src/cublas.rs:248-292
CUBLAS_COMPUTE_16F = 64
CUBLAS_COMPUTE_32F = 68
CUBLAS_COMPUTE_64F = 70
CUBLAS_COMPUTE_32I = 72
CUBLAS_COMPUTE_32I_PEDANTIC = 73
CUBLAS_COMPUTE_32F_FAST_16F = 74
CUBLAS_COMPUTE_32F_FAST_16BF = 75
CUBLAS_COMPUTE_32F_FAST_TF32 = 77

# cudaDataType -- cuda_types/src/cuda.rs:8690-8806
CUDA_R_32F = 0
CUDA_R_64F = 1
CUDA_R_16F = 2
CUDA_R_8I = 3
CUDA_R_32I = 10
CUDA_R_16BF = 14
CUDA_R_8F_E4M3 = 28
CUDA_R_8F_E5M2 = 29
CUDA_R_8F_UE8M0 = 30
CUDA_R_4F_E2M1 = 33

# cublasLtMatrixLayoutAttribute_t -- cuda_types/src/cublaslt.rs:3981-4075
CUBLASLT_MATRIX_LAYOUT_TYPE = 0
CUBLASLT_MATRIX_LAYOUT_ORDER = 1
CUBLASLT_MATRIX_LAYOUT_ROWS = 2
CUBLASLT_MATRIX_LAYOUT_COLS = 3
CUBLASLT_MATRIX_LAYOUT_LD = 4
CUBLASLT_MATRIX_LAYOUT_BATCH_COUNT = 5
CUBLASLT_MATRIX_LAYOUT_STRIDED_BATCH_OFFSET = 6
CUBLASLT_MATRIX_LAYOUT_PLANE_OFFSET = 7

# cublasLtOrder_t -- cuda_types/src/cublaslt.rs:3923-3961
CUBLASLT_ORDER_COL, CUBLASLT_ORDER_ROW, CUBLASLT_ORDER_COL32 = 0, 1, 2

# cublasLtMatmulDescAttributes_t -- cuda_types/src/cublaslt.rs:4080-4470
CUBLASLT_MATMUL_DESC_COMPUTE_TYPE = 0
CUBLASLT_MATMUL_DESC_SCALE_TYPE = 1
CUBLASLT_MATMUL_DESC_POINTER_MODE = 2
CUBLASLT_MATMUL_DESC_TRANSA = 3
CUBLASLT_MATMUL_DESC_TRANSB = 4
CUBLASLT_MATMUL_DESC_TRANSC = 5
CUBLASLT_MATMUL_DESC_FILL_MODE = 6
CUBLASLT_MATMUL_DESC_EPILOGUE = 7
CUBLASLT_MATMUL_DESC_BIAS_POINTER = 8
CUBLASLT_MATMUL_DESC_BIAS_BATCH_STRIDE = 10
CUBLASLT_MATMUL_DESC_EPILOGUE_AUX_POINTER = 11
CUBLASLT_MATMUL_DESC_EPILOGUE_AUX_LD = 12
CUBLASLT_MATMUL_DESC_EPILOGUE_AUX_BATCH_STRIDE = 13
CUBLASLT_MATMUL_DESC_ALPHA_VECTOR_BATCH_STRIDE = 14
CUBLASLT_MATMUL_DESC_SM_COUNT_TARGET = 15
CUBLASLT_MATMUL_DESC_A_SCALE_POINTER = 17
CUBLASLT_MATMUL_DESC_B_SCALE_POINTER = 18
CUBLASLT_MATMUL_DESC_C_SCALE_POINTER = 19
CUBLASLT_MATMUL_DESC_D_SCALE_POINTER = 20
CUBLASLT_MATMUL_DESC_AMAX_D_POINTER = 21
CUBLASLT_MATMUL_DESC_FAST_ACCUM = 25
CUBLASLT_MATMUL_DESC_BIAS_DATA_TYPE = 26
CUBLASLT_MATMUL_DESC_A_SCALE_MODE = 31
CUBLASLT_MATMUL_DESC_B_SCALE_MODE = 32
CUBLASLT_MATMUL_DESC_C_SCALE_MODE = 33
CUBLASLT_MATMUL_DESC_D_SCALE_MODE = 34

# cublasLtPointerMode_t -- cuda_types/src/cublaslt.rs:3853-3887
CUBLASLT_POINTER_MODE_HOST = 0
CUBLASLT_POINTER_MODE_DEVICE = 1
CUBLASLT_POINTER_MODE_DEVICE_VECTOR = 2
CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO = 3
CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_HOST = 4

# cublasLtMatmulMatrixScale_t -- cuda_types/src/cublaslt.rs:3800-3852
CUBLASLT_MATMUL_MATRIX_SCALE_SCALAR_32F = 0
CUBLASLT_MATMUL_MATRIX_SCALE_VEC16_UE4M3 = 1
CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0 = 2
CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F = 3
CUBLASLT_MATMUL_MATRIX_SCALE_VEC128_32F = 4
CUBLASLT_MATMUL_MATRIX_SCALE_BLK128x128_32F = 5

# cublasLtEpilogue_t -- cuda_types/src/cublaslt.rs:4547-4660
CUBLASLT_EPILOGUE_DEFAULT = 1
CUBLASLT_EPILOGUE_RELU = 2
CUBLASLT_EPILOGUE_BIAS = 4
CUBLASLT_EPILOGUE_RELU_BIAS = 6
CUBLASLT_EPILOGUE_GELU = 32
CUBLASLT_EPILOGUE_GELU_BIAS = 36
CUBLASLT_EPILOGUE_RELU_AUX = 130
CUBLASLT_EPILOGUE_GELU_AUX = 160
CUBLASLT_EPILOGUE_GELU_AUX_BIAS = 164
CUBLASLT_EPILOGUE_DGELU = 192
CUBLASLT_EPILOGUE_DGELU_BGRAD = 208
CUBLASLT_EPILOGUE_BGRADA = 256
CUBLASLT_EPILOGUE_BGRADB = 512

# cublasLtMatmulPreferenceAttributes_t -- cuda_types/src/cublaslt.rs:4725-4820
CUBLASLT_MATMUL_PREF_SEARCH_MODE = 0
CUBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES = 1
CUBLASLT_MATMUL_PREF_REDUCTION_SCHEME_MASK = 3
CUBLASLT_MATMUL_PREF_MIN_ALIGNMENT_A_BYTES = 5
CUBLASLT_MATMUL_PREF_MIN_ALIGNMENT_B_BYTES = 6
CUBLASLT_MATMUL_PREF_MIN_ALIGNMENT_C_BYTES = 7
CUBLASLT_MATMUL_PREF_MIN_ALIGNMENT_D_BYTES = 8
CUBLASLT_MATMUL_PREF_MAX_WAVES_COUNT = 9
CUBLASLT_MATMUL_PREF_IMPL_MASK = 12

# handle cookies -- zluda_blaslt/src/impl.rs:24-26, zluda_common/src/constants.rs:6
ZLUDA_BLASLT_HANDLE_COOKIE = 0xD1D9CB43416C9620
ZLUDA_BLAS_HANDLE_COOKIE = 0x57C3FDB0FD72B08E

# kernel families of the launch layer (include/zluda_gemm_launch.h)
ZLUDA_KERNEL_AUTO = 0
ZLUDA_KERNEL_GENERIC = 1
ZLUDA_KERNEL_MFMA_I8 = 2
ZLUDA_KERNEL_MFMA_F8 = 3
ZLUDA_KERNEL_MFMA_MXF4 = 4
ZLUDA_KERNEL_DECODE_W8A8 = 5
ZLUDA_KERNEL_MFMA_TR8 = 6
ZLUDA_KERNEL_MFMA_H16 = 7
ZLUDA_KERNEL_MFMA_TR16 = 8
ZLUDA_KERNEL_MFMA_F32 = 9
ZLUDA_KERNEL_MFMA_TR32 = 10
ZLUDA_ALGO_MAGIC = 0x5A4C4441

TYPE_BITS = {CUDA_R_32F: 32, CUDA_R_32I: 32, CUDA_R_16F: 16, CUDA_R_16BF: 16, CUDA_R_8I: 8,
             CUDA_R_8F_E4M3: 8, CUDA_R_8F_E5M2: 8, CUDA_R_8F_UE8M0: 8, CUDA_R_4F_E2M1: 4}


class cublasLtMatmulAlgo_t(C.Structure):  # cuda_types/src/cublaslt.rs:55-59
    _fields_ = [("data", C.c_uint64 * 8)]


class cublasLtMatmulHeuristicResult_t(C.Structure):  # cuda_types/src/cublaslt.rs:4825-4841
    _fields_ = [("algo", cublasLtMatmulAlgo_t), ("workspaceSize", C.c_size_t),
                ("state", C.c_uint32), ("wavesCount", C.c_float), ("reserved", C.c_int * 4)]


class zluda_matrix_layout(C.Structure):
    _fields_ = [("type", C.c_uint32), ("order", C.c_int32), ("rows", C.c_uint64),
                ("cols", C.c_uint64), ("ld", C.c_int64), ("batch_count", C.c_int32),
                ("batch_stride", C.c_int64)]


class zluda_matmul_desc(C.Structure):
    _fields_ = [("compute_type", C.c_uint32), ("scale_type", C.c_uint32),
                ("pointer_mode", C.c_int32), ("transa", C.c_uint32), ("transb", C.c_uint32),
                ("epilogue", C.c_uint32), ("bias", C.c_void_p), ("bias_type", C.c_int32),
                ("bias_batch_stride", C.c_int64), ("alpha_vector_batch_stride", C.c_int64),
                ("a_scale", C.c_void_p), ("b_scale", C.c_void_p), ("c_scale", C.c_void_p),
                ("d_scale", C.c_void_p), ("a_scale_mode", C.c_int32), ("b_scale_mode", C.c_int32),
                ("c_scale_mode", C.c_int32), ("d_scale_mode", C.c_int32), ("fast_accum", C.c_int8),
                ("epilogue_aux", C.c_void_p), ("epilogue_aux_ld", C.c_int64), ("epilogue_aux_batch_stride", C.c_int64),
                ("epilogue_aux_type", C.c_int32)]


class zluda_gemm_problem(C.Structure):
    _fields_ = [("op", zluda_matmul_desc), ("a", zluda_matrix_layout), ("b", zluda_matrix_layout),
                ("c", zluda_matrix_layout), ("d", zluda_matrix_layout), ("alpha", C.c_void_p),
                ("beta", C.c_void_p), ("A", C.c_void_p), ("B", C.c_void_p), ("C", C.c_void_p),
                ("D", C.c_void_p), ("workspace", C.c_void_p), ("workspace_size", C.c_size_t)]


class zluda_gemm_plan(C.Structure):
    _fields_ = [("kernel", C.c_uint32), ("variant", C.c_uint32), ("workspace", C.c_uint64),
                ("swapped", C.c_uint32), ("grid_x", C.c_uint32), ("grid_y", C.c_uint32),
                ("grid_z", C.c_uint32), ("block", C.c_uint32), ("waves", C.c_float)]
