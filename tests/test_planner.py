"""Kernel selection and problem validation of the launch layer (host only)."""
import ctypes as C

import pytest

from oracle.cases import Case
from zluda_amd import abi

K = abi
I8 = dict(a_type=K.CUDA_R_8I, b_type=K.CUDA_R_8I, d_type=K.CUDA_R_32I, compute_type=K.CUBLAS_COMPUTE_32I,
          scale_type=K.CUDA_R_32I)
F8 = dict(a_type=K.CUDA_R_8F_E4M3, b_type=K.CUDA_R_8F_E4M3, d_type=K.CUDA_R_16BF, compute_type=K.CUBLAS_COMPUTE_32F,
          scale_type=K.CUDA_R_32F)
MX = dict(a_type=K.CUDA_R_4F_E2M1, b_type=K.CUDA_R_4F_E2M1, d_type=K.CUDA_R_16BF, compute_type=K.CUBLAS_COMPUTE_32F,
          scale_type=K.CUDA_R_32F, a_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0,
          b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0)


def plan(api, spec, forced=0, variant=-1, cus=256, a_ptr=0, b_ptr=0, workspace=0):
    case = Case.__new__(Case)
    case.spec = dict(spec)
    case.spec.setdefault("c_type", spec["d_type"])
    case.batch = spec.get("batch", 1)
    p = case.problem({"A": a_ptr, "B": b_ptr, "D": 0, "alpha": 0, "beta": 0})
    p.workspace_size = workspace
    out = abi.zluda_gemm_plan()
    st = api.zluda_gemm_plan_problem(C.byref(p), forced, variant, cus, C.byref(out))
    return st, out


def test_baseline_configs_pick_the_intended_kernels(api):
    st, p = plan(api, dict(I8, m=256, n=256, k=256, transa=0, transb=1))            # config 1: A:N B:T
    assert st == 0 and p.kernel == K.ZLUDA_KERNEL_MFMA_TR8 and p.variant == 2 and p.grid_x == 16 and p.block == 256
    st, p = plan(api, dict(I8, m=4096, n=4096, k=4096, transa=1))                   # config 2
    assert st == 0 and p.kernel == K.ZLUDA_KERNEL_MFMA_I8 and p.variant == 11 and p.grid_x == 256 and p.block == 256   # 256x256, four waves, one workgroup per CU
    st, p = plan(api, dict(I8, m=14336, n=16, k=4096, transa=1, d_type=K.CUDA_R_16BF, scale_type=K.CUDA_R_32F,
                           pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO,
                           b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F,
                           epilogue=K.CUBLASLT_EPILOGUE_BIAS, bias_type=K.CUDA_R_32F))       # config 3
    assert st == 0 and p.kernel == K.ZLUDA_KERNEL_DECODE_W8A8 and p.swapped == 0 and p.block == 256
    assert p.variant == 16 and p.grid_x == 224     # streamed through LDS in slabs: 896 blocks of 16 rows, 4 per workgroup
    st, p = plan(api, dict(F8, m=8192, n=8192, k=8192, transa=1, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS))  # config 4
    assert st == 0 and p.kernel == K.ZLUDA_KERNEL_MFMA_F8 and p.variant == 11 and p.grid_x == 256 and p.grid_y == 1   # 1024 tiles, 4 per workgroup
    st, p = plan(api, dict(MX, m=8192, n=8192, k=8192, transa=1, batch=4))          # config 5
    assert st == 0 and p.kernel == K.ZLUDA_KERNEL_MFMA_MXF4 and p.variant == 11 and p.grid_x == 256 and p.grid_y == 1   # 4096 tiles, 16 per workgroup
    assert p.workspace == 0


def test_16_bit_operands_take_the_mfma_family_when_k_contiguous(api):
    for t in (K.CUDA_R_16BF, K.CUDA_R_16F):
        H = dict(a_type=t, b_type=t, d_type=t, compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F)
        st, p = plan(api, dict(H, m=8192, n=8192, k=8192, transa=1))
        assert st == 0 and p.kernel == K.ZLUDA_KERNEL_MFMA_H16 and p.variant == 11 and p.grid_x == 256 and p.block == 256   # the four-wave kernel
        assert plan(api, dict(H, m=8192, n=8192, k=8192, transa=1, d_type=K.CUDA_R_32F))[1].variant == 11                     # (f32 output too)
        st, p = plan(api, dict(H, m=2048, n=2048, k=2048, transa=1))
        assert st == 0 and p.kernel == K.ZLUDA_KERNEL_MFMA_H16 and p.variant in (3, 4) and p.grid_x == 256
        assert plan(api, dict(H, m=6144, n=6144, k=6144, transa=1))[1].variant == 9
        assert api.zluda_gemm_variant_count(K.ZLUDA_KERNEL_MFMA_H16) == 12
        # K in bytes decides the split: 4096 elements of 16 bits are 8 KiB per row
        st, p = plan(api, dict(H, m=512, n=256, k=4096, transa=1), workspace=64 << 20)
        assert st == 0 and p.kernel == K.ZLUDA_KERNEL_MFMA_H16 and p.grid_z > 1
        # pitches that are not multiples of 16 bytes leave the DMA kernel for the transposing one (4-byte alignment) ...
        st, p = plan(api, dict(H, m=512, n=256, k=4096, transa=1, lda=4100))
        assert st == 0 and p.kernel == K.ZLUDA_KERNEL_MFMA_TR16
        # ... which is also what runs operands with unit stride along M or N
        for ta, tb in ((0, 0), (0, 1), (1, 1)):
            st, p = plan(api, dict(H, m=4096, n=4096, k=4096, transa=ta, transb=tb))
            assert st == 0 and p.kernel == K.ZLUDA_KERNEL_MFMA_TR16 and p.variant == 3 and p.grid_x == 256   # 256 x 256 on the 16x16 MFMA shape
        # odd pitches (2-byte alignment) are left to the generic kernel
        st, p = plan(api, dict(H, m=512, n=256, k=4096, transa=0, lda=513))
        assert st == 0 and p.kernel == K.ZLUDA_KERNEL_GENERIC
        assert api.zluda_gemm_variant_count(K.ZLUDA_KERNEL_MFMA_TR16) == 4
        assert plan(api, dict(H, m=2048, n=1024, k=4096, transa=0))[1].variant != 3     # a grid that leaves the chip half idle
        assert plan(api, dict(H, m=4096, n=4096, k=4096), forced=K.ZLUDA_KERNEL_MFMA_TR8)[0] == K.CUBLAS_STATUS_NOT_SUPPORTED
        assert plan(api, dict(I8, m=4096, n=4096, k=4096), forced=K.ZLUDA_KERNEL_MFMA_TR16)[0] == K.CUBLAS_STATUS_NOT_SUPPORTED
        # other operand types never reach it
        assert plan(api, dict(I8, m=512, n=256, k=4096, transa=1), forced=K.ZLUDA_KERNEL_MFMA_H16)[0] == K.CUBLAS_STATUS_NOT_SUPPORTED


def test_f32_operands_take_their_mfma_families(api):
    F = dict(a_type=K.CUDA_R_32F, b_type=K.CUDA_R_32F, d_type=K.CUDA_R_32F, compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F)
    st, p = plan(api, dict(F, m=8192, n=8192, k=8192, transa=1))
    assert st == 0 and (p.kernel, p.variant, p.grid_x, p.block) == (K.ZLUDA_KERNEL_MFMA_F32, 0, 1024, 512)
    for ta, tb in ((0, 0), (0, 1), (1, 1)):
        st, p = plan(api, dict(F, m=4096, n=4096, k=4096, transa=ta, transb=tb))
        assert st == 0 and (p.kernel, p.variant) == (K.ZLUDA_KERNEL_MFMA_TR32, 0)
    # K-contiguous rows of 4-byte alignment only: the transposing kernel, if they are whole 16-byte pieces long
    assert plan(api, dict(F, m=512, n=256, k=4096, transa=1, lda=4097))[1].kernel == K.ZLUDA_KERNEL_MFMA_TR32
    assert plan(api, dict(F, m=512, n=256, k=4097, transa=1))[1].kernel == K.ZLUDA_KERNEL_GENERIC
    # any K when neither operand is K-contiguous
    assert plan(api, dict(F, m=512, n=256, k=4097, transa=0, transb=1))[1].kernel == K.ZLUDA_KERNEL_MFMA_TR32
    assert api.zluda_gemm_variant_count(K.ZLUDA_KERNEL_MFMA_F32) == 8 and api.zluda_gemm_variant_count(K.ZLUDA_KERNEL_MFMA_TR32) == 3
    # a skinny f32 problem is not a decode problem
    assert plan(api, dict(F, m=14336, n=16, k=2048, transa=1))[1].kernel == K.ZLUDA_KERNEL_MFMA_F32
    assert plan(api, dict(F, m=4096, n=4096, k=4096, transa=1), forced=K.ZLUDA_KERNEL_MFMA_H16)[0] == K.CUBLAS_STATUS_NOT_SUPPORTED


def test_16_bit_weights_with_few_tokens_take_the_slab_decode(api):
    """the slab form counts K in bytes: 2048 elements of 16 bits are the 4096 bytes of its first shape"""
    for t in (K.CUDA_R_16BF, K.CUDA_R_16F):
        H = dict(a_type=t, b_type=t, d_type=t, compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F, transa=1)
        for k, variant in ((2048, 16), (1536, 16), (4096, 17), (6144, 18), (8192, 19)):
            st, p = plan(api, dict(H, m=14336, n=16, k=k))
            assert st == 0 and (p.kernel, p.variant) == (K.ZLUDA_KERNEL_DECODE_W8A8, variant), (k, p.kernel, p.variant)
        st, p = plan(api, dict(H, m=4096, n=29, k=2048))
        assert st == 0 and (p.kernel, p.variant) == (K.ZLUDA_KERNEL_DECODE_W8A8, 20)       # two token blocks
        # K beyond 16 KiB per row, too many tokens, or no unit K stride: the MFMA tile kernels
        assert plan(api, dict(H, m=4096, n=16, k=14336))[1].kernel == K.ZLUDA_KERNEL_MFMA_H16
        assert plan(api, dict(H, m=14336, n=48, k=4096))[1].kernel == K.ZLUDA_KERNEL_MFMA_H16
        assert plan(api, dict(H, m=14336, n=16, k=4096, transa=0))[1].kernel == K.ZLUDA_KERNEL_MFMA_TR16
        # more than 64 rows per CU: tiles, unless K is long
        assert plan(api, dict(H, m=28672, n=16, k=4096))[1].kernel == K.ZLUDA_KERNEL_MFMA_H16
        st, p = plan(api, dict(H, m=28672, n=16, k=8192))
        assert st == 0 and (p.kernel, p.variant, p.grid_x) == (K.ZLUDA_KERNEL_DECODE_W8A8, 19, 448)
        # the other decode forms are 8-bit instantiations
        for v in (0, 4, 5):
            assert plan(api, dict(H, m=14336, n=16, k=2048), forced=K.ZLUDA_KERNEL_DECODE_W8A8, variant=v)[0] == K.CUBLAS_STATUS_NOT_SUPPORTED


def test_skinny_problems_of_one_workgroup_per_cu_get_the_deep_ring(api):
    st, p = plan(api, dict(I8, m=14336, n=64, k=4096, transa=1))
    assert st == 0 and (p.kernel, p.variant, p.grid_x, p.grid_z) == (K.ZLUDA_KERNEL_MFMA_I8, 10, 224, 1)
    st, p = plan(api, dict(I8, m=14336, n=64, k=4096, transa=1), cus=128)            # two workgroups per CU: the 3-stage ring, several per CU
    assert st == 0 and p.variant != 10
    st, p = plan(api, dict(I8, m=4096, n=64, k=4096, transa=1), workspace=64 << 20)  # split along K instead
    assert st == 0 and p.variant == 6 and p.grid_z > 1
    st, p = plan(api, dict(I8, m=4096, n=64, k=1024, transa=1))                      # a short K never fills the ring
    assert st == 0 and p.variant == 6
    st, p = plan(api, dict(MX, m=14336, n=64, k=8192, transa=1))                     # MXFP4 scale chunks span 4 stages
    assert st == 0 and p.variant != 10


def test_small_problems_get_smaller_tiles(api):
    st, p = plan(api, dict(I8, m=1024, n=1024, k=1024, transa=1))
    assert st == 0 and p.kernel == K.ZLUDA_KERNEL_MFMA_I8 and p.variant == 6 and p.grid_x == 256
    st, p = plan(api, dict(I8, m=4096, n=2048, k=1024, transa=1))
    assert st == 0 and p.variant == 2 and p.grid_x == 16 * 16


def test_extents_that_256_divides_badly_get_the_192_row_tile(api):
    # (variants 9 and 8 are 7's and 0's tiles on the 16x16 MFMA shapes: taken when the grid fills the chip)
    st, p = plan(api, dict(F8, m=6144, n=4096, k=4096, transa=1))
    assert st == 0 and p.variant == 9 and p.grid_x == 32 * 16          # two full rounds instead of 1.5 -> 2 of 256x256
    st, p = plan(api, dict(I8, m=3072, n=3072, k=3072, transa=1))
    assert st == 0 and p.variant == 9 and p.grid_x == 16 * 12
    st, p = plan(api, dict(F8, m=3072, n=3072, k=3072, transa=1))       # fp8 gains little: only from two rounds on
    assert st == 0 and p.variant == 7
    st, p = plan(api, dict(I8, m=2048, n=2048, k=2048, transa=1, batch=2))   # 128 tiles of 256x256: half of the chip idles
    assert st == 0 and not (p.variant in (8, 9))
    st, p = plan(api, dict(I8, m=8192, n=8192, k=8192, transa=1))
    assert st == 0 and p.variant == 11
    st, p = plan(api, dict(F8, m=14336, n=4096, k=4096, transa=1))   # 5 rounds of 192x256 lose to 4 of 256x256
    assert st == 0 and p.variant == 11
    st, p = plan(api, dict(F8, m=8192, n=8192, k=8192, transa=1))
    assert st == 0 and p.variant == 11
    st, p = plan(api, dict(F8, m=8192, n=4096, k=4096, transa=1))
    assert st == 0 and p.variant == 11
    st, p = plan(api, dict(MX, m=8192, n=8192, k=8192, transa=1))      # MXFP4 has no eight-wave 16x16-shape variant, but the four-wave kernel
    assert st == 0 and p.variant == 11
    for v in (8, 9, 10):
        assert plan(api, dict(MX, m=8192, n=8192, k=8192, transa=1), forced=K.ZLUDA_KERNEL_MFMA_MXF4, variant=v)[0] == K.CUBLAS_STATUS_INVALID_VALUE
    assert api.zluda_gemm_variant_count(K.ZLUDA_KERNEL_MFMA_I8) == 12 and api.zluda_gemm_variant_count(K.ZLUDA_KERNEL_MFMA_MXF4) == 12


def test_the_four_wave_kernel_is_chosen_for_what_its_epilogues_serve(api):
    """variant 11: one workgroup per CU walks the 256 x 256 tiles of all batches; int8 -> int32, and int8 with float scaling,
    fp8, f16, bf16 and MXFP4 -> bf16 / f16 with beta = 0, any of the three activations, scale vectors either way and a bias
    along D's unit stride, from one round of tiles and 2048 elements of K"""
    big = dict(m=8192, n=8192, k=8192, transa=1)
    assert plan(api, dict(F8, **big))[1].variant == 11
    assert plan(api, dict(F8, **big, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS))[1].variant == 11
    assert plan(api, dict(F8, **big, epilogue=K.CUBLASLT_EPILOGUE_BIAS, pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO))[1].variant == 11
    # what it has no epilogue for stays on the eight-wave kernel with the same tile
    assert plan(api, dict(F8, **big, epilogue=K.CUBLASLT_EPILOGUE_RELU))[1].variant == 11      # (ReLU and f16 ride on the bf16 epilogues)
    assert plan(api, dict(F8, **big, d_type=K.CUDA_R_16F))[1].variant == 11
    assert plan(api, dict(F8, **big, d_type=K.CUDA_R_32F))[1].variant == 11
    assert plan(api, dict(F8, **big, d_type=K.CUDA_R_8F_E4M3))[1].variant != 11     # (8-bit outputs: an eight-wave kernel)
    assert plan(api, dict(F8, **big, b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F))[1].variant == 11   # scale vectors may run either way
    assert plan(api, dict(F8, **big, order_c=1, order_d=1, epilogue=K.CUBLASLT_EPILOGUE_BIAS))[1].variant == 8     # a bias only along D's unit stride
    assert plan(api, dict(F8, **big, order_c=1, order_d=1))[1].variant == 11
    assert plan(api, dict(F8, **big, a_type=K.CUDA_R_8F_E5M2))[1].variant == 11     # (either operand may be E5M2)
    assert plan(api, dict(F8, **big, pointer_mode=K.CUBLASLT_POINTER_MODE_DEVICE))[1].variant == 8                 # beta unknown until it runs
    assert plan(api, dict(F8, **big, ldd=8196))[1].variant == 8                                                    # columns of D not 16-byte aligned
    # int8 with float scaling (W8A8: alpha[], per-row and per-token scales, bias, GELU) -> bf16
    w8a8 = dict(I8, **big, d_type=K.CUDA_R_16BF, scale_type=K.CUDA_R_32F)
    assert plan(api, w8a8)[1].variant == 11
    assert plan(api, dict(w8a8, pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS,
                          b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F))[1].variant == 11
    assert plan(api, dict(w8a8, d_type=K.CUDA_R_16F))[1].variant == 11
    assert plan(api, dict(w8a8, epilogue=K.CUBLASLT_EPILOGUE_RELU_BIAS))[1].variant == 11
    assert plan(api, dict(w8a8, d_type=K.CUDA_R_32F))[1].variant == 11
    assert plan(api, dict(w8a8, d_type=K.CUDA_R_8I))[1].variant == 8
    # grids: one workgroup per CU at most, all batches in one list
    st, p = plan(api, dict(F8, m=4096, n=4096, k=4096, transa=1, batch=3))
    assert st == 0 and p.variant == 11 and p.grid_x == 256 and p.grid_y == 1 and p.grid_z == 1 and p.workspace == 0 and p.waves == 3.0
    st, p = plan(api, dict(F8, **big), cus=304)
    assert st == 0 and p.variant == 11 and p.grid_x == 304
    st, p = plan(api, dict(F8, **big), cus=300)     # a multiple of 8, so that a workgroup's tiles stay with one XCD
    assert st == 0 and p.grid_x == 296
    st, p = plan(api, dict(I8, m=4096, n=3072, k=4096, transa=1), forced=K.ZLUDA_KERNEL_MFMA_I8, variant=11)
    assert st == 0 and p.grid_x == 192
    # too few tiles or a short K: other variants
    assert plan(api, dict(F8, m=4096, n=2048, k=4096, transa=1))[1].variant != 11
    assert plan(api, dict(F8, m=16384, n=8192, k=1024, transa=1))[1].variant != 11
    # never with a workspace split, never for other operand types
    assert plan(api, dict(I8, m=1024, n=256, k=8192, transa=1), forced=K.ZLUDA_KERNEL_MFMA_I8, variant=11, workspace=64 << 20)[1].grid_z == 1
    assert plan(api, dict(F8, **big, a_type=K.CUDA_R_8F_E5M2), forced=K.ZLUDA_KERNEL_MFMA_F8, variant=11)[0] == 0
    bf = dict(a_type=K.CUDA_R_16BF, b_type=K.CUDA_R_16BF, d_type=K.CUDA_R_16BF, compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F)
    st, p = plan(api, dict(bf, **big), forced=K.ZLUDA_KERNEL_MFMA_H16, variant=11)     # f16 / bf16 operands have it too
    assert st == 0 and p.grid_x == 256
    # MXFP4: bf16 output, whole scale chunks (K a multiple of 1024), and no vector along D's unit stride at all (its
    # scale chunks take the LDS that holds such vectors for the other kinds)
    assert plan(api, dict(MX, **big))[1].variant == 11
    assert plan(api, dict(MX, **big, epilogue=K.CUBLASLT_EPILOGUE_GELU))[1].variant == 11
    assert plan(api, dict(MX, **big, epilogue=K.CUBLASLT_EPILOGUE_BIAS))[1].variant == 0
    assert plan(api, dict(MX, **big, pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO))[1].variant == 0
    assert plan(api, dict(MX, m=8192, n=8192, k=8192 + 512, transa=1))[1].variant == 0
    assert plan(api, dict(MX, **big, d_type=K.CUDA_R_32F))[1].variant == 11
    f32 = dict(a_type=K.CUDA_R_32F, b_type=K.CUDA_R_32F, d_type=K.CUDA_R_32F, compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F)
    assert plan(api, dict(f32, **big), forced=K.ZLUDA_KERNEL_MFMA_F32, variant=11)[0] == K.CUBLAS_STATUS_INVALID_VALUE


def test_row_major_output_swaps_operands(api):
    st, p = plan(api, dict(I8, m=512, n=1024, k=512, order_a=1, order_b=1, transb=1, order_c=1, order_d=1))
    assert st == 0 and p.kernel == K.ZLUDA_KERNEL_MFMA_I8 and p.swapped == 1
    # tokens along M (row-major activations x weights^T): decode with the weights as operand B
    st, p = plan(api, dict(I8, m=16, n=4096, k=4096, order_a=1, order_b=1, transb=1, order_c=1, order_d=1,
                           d_type=K.CUDA_R_16BF, scale_type=K.CUDA_R_32F))
    assert st == 0 and p.kernel == K.ZLUDA_KERNEL_DECODE_W8A8 and p.swapped == 1


def test_misaligned_or_strided_operands_leave_the_dma_kernels(api):
    spec = dict(I8, m=512, n=512, k=512, transa=1)
    TR8, GEN = K.ZLUDA_KERNEL_MFMA_TR8, K.ZLUDA_KERNEL_GENERIC
    # 4-byte alignment is enough for the register-staged kernel, 16 for the LDS DMA ones
    assert plan(api, spec, a_ptr=0x1004)[1].kernel == TR8
    assert plan(api, spec, a_ptr=0x1002)[1].kernel == GEN
    assert plan(api, dict(spec, lda=520))[1].kernel == TR8                             # pitch not a multiple of 16
    assert plan(api, dict(spec, lda=514))[1].kernel == GEN                             # ... nor of 4
    assert plan(api, dict(spec, k=520, lda=528, ldb=528))[1].kernel == GEN             # K-contiguous, K % 16 != 0
    assert plan(api, dict(spec, k=528, lda=528, ldb=528))[1].kernel == K.ZLUDA_KERNEL_MFMA_I8   # K tail of 16 bytes
    st, _ = plan(api, spec, forced=K.ZLUDA_KERNEL_MFMA_I8, a_ptr=0x1004)
    assert st == K.CUBLAS_STATUS_NOT_SUPPORTED
    # operands that are not K-contiguous: any K
    assert plan(api, dict(spec, transa=0, transb=1, k=100))[1].kernel == TR8
    assert plan(api, dict(spec, transa=0, transb=0, k=100, ldb=100))[1].kernel == GEN  # B K-contiguous: K % 16
    assert plan(api, dict(spec, transa=0, transb=0, k=112, ldb=112))[1].kernel == TR8
    assert plan(api, dict(spec, transa=0, lda=518))[1].kernel == GEN                   # stride of a K row % 4
    # tile choice: 256x256 once every CU gets one, 64x64 for what would leave CUs idle
    # (variant 3 is variant 0's tile on the 16x16 MFMA shape: int8 grids that fill the chip)
    st, p = plan(api, dict(spec, transa=0, transb=1, m=4096, n=4096))
    assert st == 0 and p.kernel == TR8 and p.variant == 3 and p.grid_x == 256 and p.block == 512
    st, p = plan(api, dict(spec, transa=0, transb=1, m=4096, n=1024, k=4096))
    assert st == 0 and p.variant == 1 and p.grid_x == 256 and p.block == 256
    st, p = plan(api, dict(spec, transa=0, transb=1, m=1024, n=1024, k=1024))
    assert st == 0 and p.variant == 2 and p.grid_x == 256 and p.block == 256
    st, p = plan(api, dict(spec, transa=0, transb=1, m=8192, n=4096, k=1024))
    assert st == 0 and p.variant == 3 and p.grid_x == 512
    st, p = plan(api, dict(spec, transa=0, transb=1, m=8192, n=4096, k=1024, a_type=K.CUDA_R_8F_E4M3, b_type=K.CUDA_R_8F_E4M3,
                           d_type=K.CUDA_R_16BF, compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F))
    assert st == 0 and p.kernel == TR8 and p.variant == 0                      # fp8 stays on the 32x32 shape
    assert api.zluda_gemm_variant_count(TR8) == 4
    assert plan(api, dict(spec, transa=0, transb=1), forced=TR8, variant=4)[0] == K.CUBLAS_STATUS_INVALID_VALUE
    assert plan(api, dict(MX, m=256, n=256, k=512, transa=1), forced=TR8)[0] == K.CUBLAS_STATUS_NOT_SUPPORTED
    # MXFP4 needs whole 256-element K stages for the MFMA kernel
    assert plan(api, dict(MX, m=256, n=256, k=384, transa=1))[1].kernel == GEN
    assert plan(api, dict(MX, m=256, n=256, k=512, transa=1))[1].kernel == K.ZLUDA_KERNEL_MFMA_MXF4


@pytest.mark.parametrize("bad,status", [
    (dict(compute_type=K.CUBLAS_COMPUTE_64F), K.CUBLAS_STATUS_NOT_SUPPORTED),
    (dict(a_type=K.CUDA_R_16F), K.CUBLAS_STATUS_NOT_SUPPORTED),                      # int compute wants int8 inputs
    (dict(d_type=K.CUDA_R_16BF), K.CUBLAS_STATUS_NOT_SUPPORTED),                     # int32 scaling wants int32 D
    (dict(epilogue=K.CUBLASLT_EPILOGUE_BIAS), K.CUBLAS_STATUS_NOT_SUPPORTED),        # no bias in pure integer mode
    (dict(lda=100), K.CUBLAS_STATUS_INVALID_VALUE),                                  # ld < rows
    (dict(order_a=K.CUBLASLT_ORDER_COL32), K.CUBLAS_STATUS_NOT_SUPPORTED),
    (dict(pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO, alpha_vector_batch_stride=8),
     K.CUBLAS_STATUS_INVALID_VALUE),
])
def test_rejected_combinations(api, bad, status):
    st, _ = plan(api, dict(dict(I8, m=128, n=128, k=128, transa=1), **bad))
    assert st == status


def test_fp4_must_be_k_contiguous(api):
    st, _ = plan(api, dict(MX, m=256, n=256, k=512, transa=0))
    assert st == K.CUBLAS_STATUS_NOT_SUPPORTED
    st, _ = plan(api, dict(F8, m=256, n=256, k=512, transa=0))          # FP8 may be M-contiguous: generic kernel
    assert st == 0


def test_forced_variants(api):
    spec = dict(I8, m=4096, n=4096, k=4096, transa=1)
    for v, (grid, block) in enumerate([(256, 512), (256, 256), (512, 256), (1024, 256), (1024, 256), (2048, 256), (4096, 256),
                                       (352, 512), (256, 512), (352, 512), (4096, 256), (256, 256)]):
        st, p = plan(api, spec, forced=K.ZLUDA_KERNEL_MFMA_I8, variant=v)
        assert st == 0 and p.variant == v and p.grid_x == grid and p.block == block
    assert plan(api, spec, forced=K.ZLUDA_KERNEL_MFMA_I8, variant=12)[0] == K.CUBLAS_STATUS_INVALID_VALUE
    assert plan(api, dict(MX, m=4096, n=4096, k=4096, transa=1), forced=K.ZLUDA_KERNEL_MFMA_MXF4, variant=10)[0] == K.CUBLAS_STATUS_INVALID_VALUE
    assert plan(api, spec, forced=K.ZLUDA_KERNEL_MFMA_F8)[0] == K.CUBLAS_STATUS_NOT_SUPPORTED


def test_split_k_needs_workspace_and_few_tiles(api):
    """few tiles and a long K: grid_z workgroups share a tile's K range when the workspace holds the
    padded partial tiles (4 bytes x splits x batch x padded M x padded N); never otherwise"""
    spec = dict(I8, m=1024, n=256, k=8192, transa=1)

    def plan_ws(spec, ws):
        return plan(api, spec, workspace=ws)
    st, p = plan_ws(spec, 0)
    assert st == 0 and p.kernel == K.ZLUDA_KERNEL_MFMA_I8 and p.grid_z == 1 and p.workspace == 0
    st, p = plan_ws(spec, 64 << 20)
    assert st == 0 and p.grid_z > 1 and p.grid_x * p.grid_z <= 256
    assert p.workspace == p.grid_z * 1024 * 256 * 4 <= 64 << 20
    # a workspace that holds only 3 partial matrices limits the split
    st, p3 = plan_ws(spec, 3 * 1024 * 256 * 4)
    assert st == 0 and p3.grid_z == 3 and p3.workspace == 3 * 1024 * 256 * 4
    # enough tiles already or short K: no split (MXFP4 counts its K in bytes: 8192 elements are 4 KiB)
    assert plan_ws(dict(I8, m=4096, n=4096, k=8192, transa=1), 1 << 30)[1].grid_z == 1
    assert plan_ws(dict(I8, m=1024, n=256, k=256, transa=1), 1 << 30)[1].grid_z == 1
    assert plan_ws(dict(MX, m=1024, n=256, k=8192, transa=1), 1 << 30)[1].grid_z == 1


def test_decode_k_between_the_stream_instantiations(api):
    """an instantiation of the LDS-streaming decode kernel covers nw * steps * 64 bytes of K and takes any K (a
    multiple of 16) down to three quarters of that; K outside every cover goes to MFMA tiles (split along K through
    the workspace) when they occupy at least half of the CUs, and to the register-streaming decode variant otherwise"""
    dec = dict(I8, transa=1, d_type=K.CUDA_R_16BF, scale_type=K.CUDA_R_32F,
               pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO,
               b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F,
               epilogue=K.CUBLASLT_EPILOGUE_BIAS, bias_type=K.CUDA_R_32F)
    st, p = plan(api, dict(dec, m=14336, n=17, k=4096))                       # exactly one instantiation's cover
    assert st == 0 and p.kernel == K.ZLUDA_KERNEL_DECODE_W8A8 and p.variant == 4
    for ws in (0, 64 << 20):
        st, p = plan(api, dict(dec, m=5120, n=16, k=13824), workspace=ws)     # one block of tokens: the slab form
        assert st == 0 and p.kernel == K.ZLUDA_KERNEL_DECODE_W8A8 and p.variant == 19 and p.workspace == 0
        assert plan(api, dict(dec, m=5120, n=16, k=13824), workspace=ws, forced=K.ZLUDA_KERNEL_DECODE_W8A8, variant=6)[0] == 0   # under the 14336 cover
    st, p = plan(api, dict(dec, m=18944, n=32, k=3584))                       # under the 4096 cover, two token blocks
    assert st == 0 and p.kernel == K.ZLUDA_KERNEL_DECODE_W8A8 and p.variant == 4
    st, p = plan(api, dict(dec, m=2048, n=16, k=2560), workspace=64 << 20, forced=K.ZLUDA_KERNEL_DECODE_W8A8, variant=13)   # under the 3072 cover
    assert st == 0 and p.variant == 13
    assert plan(api, dict(dec, m=2048, n=16, k=2560), forced=K.ZLUDA_KERNEL_DECODE_W8A8, variant=7)[0] == K.CUBLAS_STATUS_NOT_SUPPORTED   # 2048 does not cover it
    st, p = plan(api, dict(dec, m=4096, n=16, k=11008))                       # the slab form again
    assert st == 0 and p.kernel == K.ZLUDA_KERNEL_DECODE_W8A8 and p.variant == 18
    assert plan(api, dict(dec, m=4096, n=16, k=11008), forced=K.ZLUDA_KERNEL_DECODE_W8A8, variant=9)[0] == 0   # under the 12288 cover
    # no cover: K = 1536 lies between 1024 and three quarters of 2048, K = 20480 beyond the largest
    st, p = plan(api, dict(dec, m=8192, n=16, k=20480), workspace=64 << 20)
    assert st == 0 and p.kernel == K.ZLUDA_KERNEL_MFMA_I8 and p.grid_z > 1 and p.grid_x * p.grid_z >= 128
    st, p = plan(api, dict(dec, m=4096, n=16, k=20480))                       # 64 tiles only, no workspace
    assert st == 0 and p.kernel == K.ZLUDA_KERNEL_DECODE_W8A8 and p.variant == 0
    st, p = plan(api, dict(dec, m=16384, n=16, k=1536))                       # 256 tiles without any split
    assert st == 0 and p.kernel == K.ZLUDA_KERNEL_MFMA_I8 and p.grid_z == 1


def test_decode_slab_form_takes_one_token_block(api):
    """the slab form of the stream kernel: up to 16 tokens, 2048 < K <= 16384, int8 or e4m3, as long as 4 blocks of 16 rows
    per CU hold the matrix; its grid is the fewest rounds of blocks shared out evenly"""
    dec = dict(I8, transa=1, d_type=K.CUDA_R_16BF, scale_type=K.CUDA_R_32F,
               pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO,
               b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F,
               epilogue=K.CUBLASLT_EPILOGUE_BIAS, bias_type=K.CUDA_R_32F)
    DEC = K.ZLUDA_KERNEL_DECODE_W8A8
    for spec, grid in ((dict(dec, m=14336, n=16, k=4096), 224), (dict(dec, m=14336, n=1, k=3584), 224),
                       (dict(dec, m=2048, n=16, k=2560), 128), (dict(dec, m=16384, n=9, k=4096), 256),
                       (dict(F8, transa=1, m=14336, n=16, k=4096), 224), (dict(dec, m=4100, n=16, k=2064), 129)):
        st, p = plan(api, spec)
        assert st == 0 and p.kernel == DEC and p.variant == 16 and p.grid_x == grid and p.block == 256 and p.workspace == 0, (spec, p.variant, p.grid_x)
    # beyond 4096: 8 waves x 2, 3, 4 units of 512 bytes, each shape from the next smaller cover up
    for spec, variant, grid in ((dict(dec, m=5120, n=16, k=13824), 19, 160), (dict(dec, m=8192, n=16, k=8192), 17, 256),
                                (dict(dec, m=4096, n=3, k=11008), 18, 256), (dict(dec, m=5120, n=16, k=5120), 17, 160),
                                (dict(dec, m=2048, n=16, k=4112), 17, 128), (dict(F8, transa=1, m=4096, n=16, k=16384), 19, 256),
                                (dict(dec, m=4096, n=16, k=12304), 19, 256)):
        st, p = plan(api, spec)
        assert st == 0 and p.kernel == DEC and p.variant == variant and p.grid_x == grid and p.block == 512, (spec, p.variant, p.grid_x)
    # 17 .. 32 tokens: the 8-wave shapes of one unit (up to two blocks of rows per CU) and of two units
    for spec, variant, grid in ((dict(dec, m=4096, n=32, k=4096), 20, 256), (dict(dec, m=8192, n=17, k=3072), 20, 256),
                                (dict(dec, m=8192, n=32, k=8192), 17, 256), (dict(F8, transa=1, m=5120, n=24, k=5120), 17, 160)):
        st, p = plan(api, spec)
        assert st == 0 and p.kernel == DEC and p.variant == variant and p.grid_x == grid and p.block == 512, (spec, p.variant, p.grid_x)
    assert plan(api, dict(dec, m=8192, n=33, k=8192))[1].variant < 16 and plan(api, dict(dec, m=4096, n=17, k=12288))[1].variant < 16
    # tokens along M: the weights are operand B
    st, p = plan(api, dict(dec, transa=0, transb=1, order_a=1, order_b=1, order_c=1, order_d=1, m=16, n=4096, k=4096))
    assert st == 0 and p.kernel == DEC and p.variant == 16 and p.swapped == 1
    # outside its range: a second token block, K of at most half the cover or beyond it, more rows than 64 per CU
    for spec, variant in ((dict(dec, m=14336, n=17, k=4096), 4), (dict(dec, m=4096, n=16, k=2048), 7),
                          (dict(dec, m=16400, n=16, k=4096), 4)):
        st, p = plan(api, spec)
        assert st == 0 and p.kernel == DEC and p.variant == variant, (spec, p.variant)
        assert plan(api, spec, forced=DEC, variant=16)[0] == (0 if spec["m"] == 16400 else K.CUBLAS_STATUS_NOT_SUPPORTED)
    st, p = plan(api, dict(dec, m=4096, n=16, k=16400))                           # K beyond the largest cover
    assert st == 0 and not (p.kernel == DEC and p.variant >= 16)
    st, p = plan(api, dict(dec, m=16400, n=16, k=4096), forced=DEC, variant=16)   # forced: more workgroups than CUs
    assert st == 0 and p.grid_x == 257
    st, p = plan(api, dict(dec, m=14336, n=16, k=4096), cus=64)                   # a smaller device: too many rows
    assert st == 0 and p.kernel == DEC and p.variant == 4


def test_fp8_decode_takes_the_streaming_kernel_under_a_cover_only(api):
    f8 = dict(F8, transa=1)
    st, p = plan(api, dict(f8, m=14336, n=17, k=4096))
    assert st == 0 and p.kernel == K.ZLUDA_KERNEL_DECODE_W8A8 and p.variant == 4 and p.grid_x == 256
    st, p = plan(api, dict(f8, m=8192, n=48, k=4096))                       # up to 48 tokens while the variant applies ...
    assert st == 0 and p.kernel == K.ZLUDA_KERNEL_DECODE_W8A8
    st, p = plan(api, dict(f8, m=14336, n=48, k=4096))                      # ... and the rows are at most 32 per CU
    assert st == 0 and (p.kernel, p.variant, p.grid_x) == (K.ZLUDA_KERNEL_MFMA_F8, 10, 224)   # 64x64 tiles on the 6-stage ring
    st, p = plan(api, dict(f8, m=14336, n=49, k=4096))                      # beyond: MFMA tiles
    assert st == 0 and p.kernel == K.ZLUDA_KERNEL_MFMA_F8
    st, p = plan(api, dict(f8, m=14336, n=33, k=8192))                      # 3 token blocks x 16 steps: too many fragments
    assert st == 0 and p.kernel == K.ZLUDA_KERNEL_MFMA_F8
    st, p = plan(api, dict(f8, m=4096, n=16, k=11008))                      # one block of tokens: the slab form
    assert st == 0 and p.kernel == K.ZLUDA_KERNEL_DECODE_W8A8 and p.variant == 18
    assert plan(api, dict(f8, m=4096, n=16, k=11008), forced=K.ZLUDA_KERNEL_DECODE_W8A8, variant=9)[0] == 0   # under the 12288 cover
    st, p = plan(api, dict(f8, m=4096, n=16, k=20480))                      # no cover: no fp8 fallback variant
    assert st == 0 and p.kernel == K.ZLUDA_KERNEL_MFMA_F8
    st, p = plan(api, dict(f8, m=4096, n=16, k=4096, b_type=K.CUDA_R_8F_E5M2))
    assert st == 0 and p.kernel == K.ZLUDA_KERNEL_MFMA_F8
    assert plan(api, dict(f8, m=4096, n=16, k=20480), forced=K.ZLUDA_KERNEL_DECODE_W8A8)[0] == K.CUBLAS_STATUS_NOT_SUPPORTED
    assert plan(api, dict(f8, m=4096, n=16, k=4096), forced=K.ZLUDA_KERNEL_DECODE_W8A8, variant=0)[0] == K.CUBLAS_STATUS_NOT_SUPPORTED


def test_transposing_kernel_splits_k_when_tiles_are_few(api):
    spec = dict(I8, transa=0, transb=0, m=4096, n=16, k=14336, ldb=14336)     # N-contiguous weights, decode shape
    st, p = plan(api, spec)
    assert st == 0 and p.kernel == K.ZLUDA_KERNEL_MFMA_TR8 and p.variant == 2 and p.grid_z == 1 and p.workspace == 0
    st, p = plan(api, spec, workspace=64 << 20)
    assert st == 0 and p.grid_x == 64 and p.grid_z == 8 and p.workspace == 8 * 4096 * 64 * 4
    st, p = plan(api, spec, workspace=3 * 4096 * 64 * 4)
    assert st == 0 and p.grid_z == 3
    st, p = plan(api, dict(I8, transa=0, transb=1, m=4096, n=4096, k=4096), workspace=1 << 30)
    assert st == 0 and p.grid_z == 1                                           # enough tiles already
    st, p = plan(api, dict(I8, transa=0, transb=1, m=256, n=256, k=256), workspace=1 << 30)
    assert st == 0 and p.grid_z == 1                                           # short K


def test_bias_gradient_epilogues_are_planned_like_the_plain_problem(api):
    """BGRADA / BGRADB leave the matmul itself as with DEFAULT (the reduction is a second kernel behind it), so
    the plan is the plain problem's; block-scaled and per-tensor-scaled operands are refused (a sum of stored
    codes is not the gradient of anything then)."""
    bf = dict(a_type=K.CUDA_R_16BF, b_type=K.CUDA_R_16BF, d_type=K.CUDA_R_16BF, compute_type=K.CUBLAS_COMPUTE_32F,
              scale_type=K.CUDA_R_32F, m=512, n=384, k=1024, transa=1)
    for spec in (bf, dict(F8, m=4096, n=4096, k=4096, transa=1), dict(I8, m=4096, n=4096, k=4096, transa=1, scale_type=K.CUDA_R_32F)):
        st0, p0 = plan(api, spec)
        for epi in (K.CUBLASLT_EPILOGUE_BGRADA, K.CUBLASLT_EPILOGUE_BGRADB):
            st, p = plan(api, dict(spec, epilogue=epi))
            assert st == 0 and st0 == 0
            assert (p.kernel, p.variant, p.grid_x, p.grid_y, p.grid_z) == (p0.kernel, p0.variant, p0.grid_x, p0.grid_y, p0.grid_z)
    st, _ = plan(api, dict(MX, m=512, n=512, k=512, transa=1, epilogue=K.CUBLASLT_EPILOGUE_BGRADA))
    assert st == K.CUBLAS_STATUS_NOT_SUPPORTED
    st, _ = plan(api, dict(I8, m=512, n=512, k=512, transa=1, epilogue=K.CUBLASLT_EPILOGUE_BGRADB))   # int32 scale type: DEFAULT only
    assert st == K.CUBLAS_STATUS_NOT_SUPPORTED
    st, _ = plan(api, dict(bf, batch=2, epilogue=K.CUBLASLT_EPILOGUE_BGRADA))   # batches would share one output vector
    assert st == K.CUBLAS_STATUS_NOT_SUPPORTED
    st, _ = plan(api, dict(bf, batch=2, bias_batch_stride=512, epilogue=K.CUBLASLT_EPILOGUE_BGRADA))
    assert st == 0
    # GELU with its input kept, GELU's gradient: the plain problem's kernel (a second pass finishes D); the aux matrix needs
    # a leading dimension that holds D's rows, D a float type of 16 or 32 bits
    f8 = dict(F8, m=512, n=512, k=512, transa=1)
    st0, p0 = plan(api, f8)
    for epi in (K.CUBLASLT_EPILOGUE_GELU_AUX, K.CUBLASLT_EPILOGUE_GELU_AUX_BIAS, K.CUBLASLT_EPILOGUE_DGELU, K.CUBLASLT_EPILOGUE_DGELU_BGRAD):
        st, p = plan(api, dict(f8, epilogue=epi, aux_ld=512))
        assert st == 0 and (p.kernel, p.variant, p.grid_x, p.grid_y) == (p0.kernel, p0.variant, p0.grid_x, p0.grid_y)
        assert plan(api, dict(f8, epilogue=epi))[0] == K.CUBLAS_STATUS_INVALID_VALUE
        assert plan(api, dict(f8, epilogue=epi, aux_ld=504))[0] == K.CUBLAS_STATUS_INVALID_VALUE
        assert plan(api, dict(f8, epilogue=epi, aux_ld=512, d_type=K.CUDA_R_8F_E4M3))[0] == K.CUBLAS_STATUS_NOT_SUPPORTED
        # the aux matrix has D's type: naming that type is the same as leaving the default, any other type is not served
        assert plan(api, dict(f8, epilogue=epi, aux_ld=512, aux_type=K.CUDA_R_16BF))[0] == 0
        assert plan(api, dict(f8, epilogue=epi, aux_ld=512, aux_type=K.CUDA_R_16F))[0] == K.CUBLAS_STATUS_NOT_SUPPORTED
        assert plan(api, dict(f8, epilogue=epi, aux_ld=512, aux_type=K.CUDA_R_8F_E4M3))[0] == K.CUBLAS_STATUS_NOT_SUPPORTED
    st, _ = plan(api, dict(I8, m=512, n=512, k=512, transa=1, epilogue=K.CUBLASLT_EPILOGUE_GELU_AUX, aux_ld=512))   # int32 scale type
    assert st == K.CUBLAS_STATUS_NOT_SUPPORTED
