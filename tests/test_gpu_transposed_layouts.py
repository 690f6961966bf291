"""GPU parity of the transposing 8-bit MFMA family (ZLUDA_KERNEL_MFMA_TR8): int8 and fp8 problems in
which A, B or both are not K-contiguous -- benchmark configuration 1's `A:N, B:T`, the N/N and T/T
combinations and their row-major counterparts -- through the exported C ABI, against the CPU oracle
on the same seeded inputs.  int8 -> int32 bit-exact over the whole D storage; float outputs within
1e-2 (floor documented in oracle/cases.py)."""
import itertools

import pytest

from oracle.cases import Case
from zluda_amd import abi

pytestmark = pytest.mark.gpu
K = abi
TR8 = K.ZLUDA_KERNEL_MFMA_TR8

I8 = dict(a_type=K.CUDA_R_8I, b_type=K.CUDA_R_8I, d_type=K.CUDA_R_32I, compute_type=K.CUBLAS_COMPUTE_32I,
          scale_type=K.CUDA_R_32I)
I8F = dict(I8, d_type=K.CUDA_R_16BF, scale_type=K.CUDA_R_32F)
F8 = dict(a_type=K.CUDA_R_8F_E4M3, b_type=K.CUDA_R_8F_E4M3, d_type=K.CUDA_R_16BF, compute_type=K.CUBLAS_COMPUTE_32F,
          scale_type=K.CUDA_R_32F)


def check(gpu_api, spec, seed, kernel=None, variant=-1, expect_kernel=None, tol=None, **case_kw):
    print("case", spec, "seed", seed, "kernel", kernel, "variant", variant, flush=True)
    case = Case(spec, seed, **case_kw)
    ref = case.run_oracle()
    st, got, k, v = case.run_gpu(gpu_api, forced_kernel=kernel, forced_variant=variant)
    assert st == 0, "cublasLtMatmul status %d" % st
    if expect_kernel is not None:
        assert k == expect_kernel, "planner chose kernel %d" % k
    return case.compare(got, ref, tol)


def test_baseline_config_1_runs_on_the_transposing_kernel(gpu_api):
    """256^3 int8, A:N B:T, alpha = 1, beta = 0: the planner's own choice"""
    check(gpu_api, dict(I8, m=256, n=256, k=256, transa=0, transb=1, alpha=1), 0, expect_kernel=TR8)


@pytest.mark.parametrize("variant", range(4))
@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 1), (1, 0)])
def test_int8_every_transpose_combination(gpu_api, variant, ta, tb):
    # full tiles, ragged edges (rows not a multiple of 4 or 8, K not a multiple of 64), padded lds
    check(gpu_api, dict(I8, m=256, n=384, k=192, transa=ta, transb=tb), 200 + variant, TR8, variant)
    ld = dict(lda=(304 if ta == 0 else 272), ldb=(272 if tb == 0 else 216))
    check(gpu_api, dict(I8, m=300, n=212, k=272, transa=ta, transb=tb, **ld), 210 + variant, TR8, variant)
    check(gpu_api, dict(I8, m=77, n=130, k=80, transa=ta, transb=tb, with_c=True, alpha=3, beta=-2,
                        lda=(80 if ta == 0 else 80), ldb=(80 if tb == 0 else 132)), 220 + variant, TR8, variant)


@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 1)])
def test_int8_k_tail_of_the_transposed_operand(gpu_api, ta, tb):
    """K needs no alignment for an operand that is transposed on the way in (K % 16 == 0 only where an
    operand is K-contiguous): 100 and 36 leave partial 4-row blocks and a partial stage"""
    ks = [100, 36] if (ta, tb) == (0, 1) else [112, 48]
    for k in ks:
        check(gpu_api, dict(I8, m=128, n=64, k=k, transa=ta, transb=tb, lda=(128 if ta == 0 else k + (-k) % 4),
                            ldb=(k + (-k) % 4 if tb == 0 else 64)), 230 + k, TR8, 2)
        check(gpu_api, dict(I8, m=128, n=64, k=k, transa=ta, transb=tb, lda=(128 if ta == 0 else k + (-k) % 4),
                            ldb=(k + (-k) % 4 if tb == 0 else 64)), 230 + k, TR8, 0)


@pytest.mark.parametrize("variant", range(4))
def test_int8_row_major_operands_and_output(gpu_api, variant):
    # row-major A (m x k, K-contiguous) with row-major B (k x n, N-contiguous) -> row-major D: the
    # everyday "activations x weights" layout of row-major frameworks
    spec = dict(I8, order_a=1, order_b=1, order_c=1, order_d=1, m=192, n=320, k=256, with_c=True, alpha=2, beta=1)
    check(gpu_api, spec, 240, TR8, variant)
    check(gpu_api, dict(spec, transa=1, transb=1), 241, TR8, variant)
    check(gpu_api, dict(spec, transa=1, order_c=0, order_d=0), 242, TR8, variant)


@pytest.mark.parametrize("variant", range(4))
def test_int8_batched_float_epilogue(gpu_api, variant):
    spec = dict(I8F, transa=0, transb=1, m=260, n=140, k=320, batch=3, epilogue=K.CUBLASLT_EPILOGUE_RELU_BIAS,
                bias_type=K.CUDA_R_32F, pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_HOST,
                with_c=True, a_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F,
                b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F,
                alpha_range=(0.001, 0.002), scale_range=(0.5, 1.5))
    check(gpu_api, spec, 250, TR8, variant)
    check(gpu_api, dict(spec, order_c=1, order_d=1), 251, TR8, variant)
    for dt in (K.CUDA_R_32F, K.CUDA_R_16F):
        check(gpu_api, dict(spec, d_type=dt, c_type=dt, m=256, n=128), 252, TR8, variant)


@pytest.mark.parametrize("variant", range(3))
@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 1), (1, 0)])
def test_fp8_every_transpose_combination(gpu_api, variant, ta, tb):
    check(gpu_api, dict(F8, m=256, n=256, k=256, transa=ta, transb=tb), 300 + variant, TR8, variant)
    check(gpu_api, dict(F8, m=200, n=136, k=400, transa=ta, transb=tb, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS,
                        with_scalar_scales=True, lda=(208 if ta == 0 else 400), ldb=(416 if tb == 0 else 136)),
          310 + variant, TR8, variant)


@pytest.mark.parametrize("at,bt", [(K.CUDA_R_8F_E5M2, K.CUDA_R_8F_E4M3), (K.CUDA_R_8F_E4M3, K.CUDA_R_8F_E5M2)])
def test_fp8_mixed_formats(gpu_api, at, bt):
    for ta, tb, od in itertools.product((0, 1), (0, 1), (0, 1)):
        if (ta, tb) == (1, 0) and od == 0:
            continue
        check(gpu_api, dict(F8, a_type=at, b_type=bt, m=128, n=192, k=256, transa=ta, transb=tb, d_type=K.CUDA_R_32F,
                            order_c=od, order_d=od), 320, TR8, 2 if od else 0)


def test_split_k_through_the_workspace(gpu_api):
    """few tiles and a long K: with a workspace the K range of a tile is shared by several workgroups
    (raw partial tiles + the reduce kernel with the full epilogue); K shares that are empty or partial"""
    ws = 64 << 20
    dec = dict(I8F, transa=0, transb=0, epilogue=K.CUBLASLT_EPILOGUE_BIAS, bias_type=K.CUDA_R_32F,
               pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO,
               b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F, alpha_range=(0.001, 0.002), scale_range=(0.5, 1.5))
    for spec, seed in ((dict(I8, m=1024, n=16, k=4096, transa=0, transb=0), 340),          # N-contiguous weights, decode shape
                       (dict(I8, m=300, n=200, k=1104, transa=0, transb=1, with_c=True, batch=2, lda=304, ldb=200,
                             alpha=2, beta=-1), 341),                                      # 17.25 stages over 8 shares
                       (dict(dec, m=640, n=16, k=2048), 342),
                       (dict(F8, m=512, n=64, k=4096, transa=0, transb=1, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS,
                             with_scalar_scales=True, scale_range=(0.02, 0.03)), 343)):
        print("TR8 split-K case", spec, flush=True)
        case = Case(spec, seed)
        ref = case.run_oracle()
        st, got, kern, variant = case.run_gpu(gpu_api, workspace_bytes=ws)
        assert st == 0 and kern == TR8
        assert case.last_workspace_needed and case.last_workspace_needed <= ws, "the planner did not split K"
        case.compare(got, ref)
        st, got, kern, variant = case.run_gpu(gpu_api)       # and without a workspace: unsplit
        assert st == 0 and kern == TR8 and case.last_workspace_needed == 0
        case.compare(got, ref)


def test_planner_prefers_the_k_contiguous_kernels_when_they_apply(gpu_api):
    check(gpu_api, dict(I8, m=512, n=256, k=512, transa=1, transb=0), 330, expect_kernel=K.ZLUDA_KERNEL_MFMA_I8)
    # K-contiguous but only 4-byte aligned pitches: the LDS DMA kernels need 16
    check(gpu_api, dict(I8, m=512, n=256, k=512, transa=1, transb=0, lda=516, ldb=520), 331, expect_kernel=TR8)
    check(gpu_api, dict(I8, m=2048, n=2048, k=512, transa=0, transb=0), 332, expect_kernel=TR8)
