"""GELU with its input kept (GELU_AUX, GELU_AUX_BIAS) and GELU's gradient (DGELU, DGELU_BGRAD) against the oracle:
the GEMM kernel of every family followed by the element-wise second pass.  cuda_types/src/cublaslt.rs:4601-4660."""
import pytest

from oracle.cases import Case
from zluda_amd import abi as K

pytestmark = pytest.mark.gpu

I8F = dict(a_type=K.CUDA_R_8I, b_type=K.CUDA_R_8I, d_type=K.CUDA_R_16BF, compute_type=K.CUBLAS_COMPUTE_32I, scale_type=K.CUDA_R_32F,
           transa=1, alpha_range=(0.001, 0.002))
F8 = dict(a_type=K.CUDA_R_8F_E4M3, b_type=K.CUDA_R_8F_E4M3, d_type=K.CUDA_R_16BF, compute_type=K.CUBLAS_COMPUTE_32F,
          scale_type=K.CUDA_R_32F, transa=1, with_scalar_scales=True, scale_range=(0.05, 0.06))
MX = dict(a_type=K.CUDA_R_4F_E2M1, b_type=K.CUDA_R_4F_E2M1, d_type=K.CUDA_R_16BF, compute_type=K.CUBLAS_COMPUTE_32F,
          scale_type=K.CUDA_R_32F, transa=1, a_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0,
          b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0)
BF = dict(a_type=K.CUDA_R_16BF, b_type=K.CUDA_R_16BF, d_type=K.CUDA_R_16BF, compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F,
          transb=1, alpha=0.05)
FWD, BWD = (K.CUBLASLT_EPILOGUE_GELU_AUX, K.CUBLASLT_EPILOGUE_GELU_AUX_BIAS), (K.CUBLASLT_EPILOGUE_DGELU, K.CUBLASLT_EPILOGUE_DGELU_BGRAD)


def run(gpu_api, spec, seed, expect_kernel=None, **case_kw):
    print("case", spec, "seed", seed, flush=True)
    case = Case(spec, seed, **case_kw)
    ref = case.run_oracle()
    st, got, kernel, _ = case.run_gpu(gpu_api)
    assert st == 0, "cublasLtMatmul status %d" % st
    if expect_kernel is not None:
        assert kernel == expect_kernel, kernel
    # D goes through one more rounding of its type than a single-pass result: 2 half-ulps of bf16
    case.compare(got, ref, tol=1e-2 if spec["d_type"] != K.CUDA_R_16BF else 1.6e-2)
    if case.aux_mode == 1:
        case.compare_aux(case.aux_got, case.aux_ref)
    if case.bgrad:
        case.compare_bgrad(case.bgrad_got, case.bgrad_ref, floor_frac=1.0)
    return case


@pytest.mark.parametrize("epi", FWD + BWD)
@pytest.mark.parametrize("family", ["i8", "f8", "mx", "bf16", "bf16_kc", "f32", "f32_tr", "generic", "decode", "tr"])
def test_aux_epilogues_through_every_kernel_family(gpu_api, epi, family):
    spec, kernel = {
        "i8": (dict(I8F, m=384, n=264, k=512), K.ZLUDA_KERNEL_MFMA_I8),
        "f8": (dict(F8, m=300, n=200, k=384, d_type=K.CUDA_R_16F), K.ZLUDA_KERNEL_MFMA_F8),
        "mx": (dict(MX, m=256, n=128, k=512), K.ZLUDA_KERNEL_MFMA_MXF4),
        "bf16": (dict(BF, m=150, n=90, k=77, d_type=K.CUDA_R_32F), K.ZLUDA_KERNEL_MFMA_TR16),
        "bf16_kc": (dict(BF, m=150, n=90, k=200, transa=1, transb=0, d_type=K.CUDA_R_32F), K.ZLUDA_KERNEL_MFMA_H16),
        "f32": (dict(BF, a_type=K.CUDA_R_32F, b_type=K.CUDA_R_32F, m=150, n=90, k=200, transa=1, transb=0, d_type=K.CUDA_R_32F), K.ZLUDA_KERNEL_MFMA_F32),
        "f32_tr": (dict(BF, a_type=K.CUDA_R_32F, b_type=K.CUDA_R_32F, m=150, n=90, k=77, d_type=K.CUDA_R_32F), K.ZLUDA_KERNEL_MFMA_TR32),
        # (K-contiguous f32 rows whose length is not a multiple of 16 bytes: nothing but the generic kernel takes them)
        "generic": (dict(BF, a_type=K.CUDA_R_32F, b_type=K.CUDA_R_32F, m=150, n=90, k=77, transa=1, transb=0, d_type=K.CUDA_R_32F), K.ZLUDA_KERNEL_GENERIC),
        "decode": (dict(I8F, m=1024, n=16, k=4096, alpha_range=(0.0002, 0.0004)), K.ZLUDA_KERNEL_DECODE_W8A8),
        "tr": (dict(I8F, transa=0, transb=1, m=256, n=320, k=256), K.ZLUDA_KERNEL_MFMA_TR8),
    }[family]
    spec = dict(spec, epilogue=epi)
    if epi in BWD:
        spec["with_c"] = family in ("i8", "bf16", "f32", "generic")
    run(gpu_api, spec, 600 + epi, expect_kernel=kernel, int_dist="normal" if family == "decode" else "uniform")


@pytest.mark.parametrize("epi", FWD + BWD)
def test_aux_epilogues_on_the_four_wave_kernel(gpu_api, epi):
    """to the GEMM kernel these epilogues are plain problems (D pointed at the aux matrix, or the gradient pass behind
    it), so variant 11 serves them like any other: forced here on problems of a few tiles, all four operand kinds"""
    for i, (base, kernel) in enumerate([(dict(F8, m=512, n=512, k=640), K.ZLUDA_KERNEL_MFMA_F8), (dict(I8F, m=768, n=256, k=512), K.ZLUDA_KERNEL_MFMA_I8),
                                        (dict(MX, m=512, n=256, k=1024), K.ZLUDA_KERNEL_MFMA_MXF4),
                                        (dict(BF, m=512, n=512, k=256, transa=1, transb=0, d_type=K.CUDA_R_16F), K.ZLUDA_KERNEL_MFMA_H16)]):
        if kernel == K.ZLUDA_KERNEL_MFMA_MXF4 and epi in (K.CUBLASLT_EPILOGUE_GELU_AUX_BIAS,):
            continue   # (a bias takes MXFP4 off this variant)
        spec = dict(base, epilogue=epi)
        print("case", spec, flush=True)
        case = Case(spec, 640 + i)
        ref = case.run_oracle()
        st, got, k, v = case.run_gpu(gpu_api, forced_kernel=kernel, forced_variant=11)
        assert st == 0 and k == kernel and v == 11
        case.compare(got, ref, tol=1e-2 if spec["d_type"] != K.CUDA_R_16BF else 1.6e-2)
        if case.aux_mode == 1:
            case.compare_aux(case.aux_got, case.aux_ref)
        if case.bgrad:
            case.compare_bgrad(case.bgrad_got, case.bgrad_ref, floor_frac=1.0)


def test_aux_epilogues_padding_batches_row_major(gpu_api):
    """aux leading dimension and batch stride of its own, row-major D (and aux), batches, the bias gradient at a batch
    stride, a bias of another type than D"""
    base = dict(I8F, m=200, n=136, k=272, batch=3, ldd=208, aux_ld=216, aux_batch_stride=216 * 136 + 40)
    run(gpu_api, dict(base, epilogue=K.CUBLASLT_EPILOGUE_GELU_AUX_BIAS, bias_type=K.CUDA_R_32F, bias_batch_stride=256), 610)
    run(gpu_api, dict(base, epilogue=K.CUBLASLT_EPILOGUE_DGELU_BGRAD, bias_batch_stride=208, with_c=True), 611)
    row = dict(F8, m=120, n=333, k=256, order_c=1, order_d=1, aux_ld=336, batch=2, d_type=K.CUDA_R_32F, c_type=K.CUDA_R_32F)
    run(gpu_api, dict(row, epilogue=K.CUBLASLT_EPILOGUE_GELU_AUX), 612)
    run(gpu_api, dict(row, epilogue=K.CUBLASLT_EPILOGUE_DGELU_BGRAD, bias_batch_stride=128, bias_type=K.CUDA_R_32F), 613)


def test_aux_epilogues_refusals(gpu_api):
    """integer or 8-bit D, an aux leading dimension below D's rows, a missing aux pointer"""
    for spec in (dict(I8F, d_type=K.CUDA_R_8I), dict(I8F, d_type=K.CUDA_R_32I, scale_type=K.CUDA_R_32I, alpha=1),
                 dict(F8, d_type=K.CUDA_R_8F_E4M3)):
        case = Case(dict(spec, m=64, n=64, k=64, epilogue=K.CUBLASLT_EPILOGUE_DEFAULT), 620)
        case.spec.update(epilogue=K.CUBLASLT_EPILOGUE_GELU_AUX, aux_ld=64)
        st, _, _ = case.run_gpu_plan(gpu_api, K.ZLUDA_KERNEL_AUTO)
        assert st == K.CUBLAS_STATUS_NOT_SUPPORTED, st
    case = Case(dict(I8F, m=64, n=64, k=64, epilogue=K.CUBLASLT_EPILOGUE_GELU_AUX, aux_ld=64), 621)
    case.spec["aux_ld"] = 56
    assert case.run_gpu_plan(gpu_api, K.ZLUDA_KERNEL_AUTO)[0] == K.CUBLAS_STATUS_INVALID_VALUE
    case.spec["aux_ld"] = 64
    case.aux = None
    assert case.run_gpu_plan(gpu_api, K.ZLUDA_KERNEL_AUTO)[0] == K.CUBLAS_STATUS_INVALID_VALUE


@pytest.mark.parametrize("epi", FWD + BWD)
@pytest.mark.parametrize("ta,tb", [(1, 0), (0, 1)])
def test_aux_epilogues_against_hipblaslt(gpu_api, epi, ta, tb, typ=K.CUDA_R_16F):
    """the reference's backend on the same buffers (f16 operands: what the installed hipBLASLt offers these epilogues for;
    it has no algorithm for bf16): the same D, the same aux matrix, the same bias gradient -- which pins the orientation of
    the aux matrix and of the sums"""
    spec = dict(BF, a_type=typ, b_type=typ, c_type=typ, d_type=typ, m=256, n=128, k=512, transa=ta, transb=tb, epilogue=epi,
                aux_ld=264)
    case = Case(spec, 960 + epi)
    st, ours, _, _ = case.run_gpu(gpu_api)
    assert st == 0
    theirs, why = case.run_hipblaslt()
    if theirs is None:
        pytest.skip("hipBLASLt offers no algorithm here: " + why)
    case.compare(ours, theirs, tol=1.6e-2, floor_frac=1e-2)
    if case.aux_mode == 1:
        case.compare_aux(case.aux_got, case.aux_theirs)
    if case.bgrad:
        case.compare_bgrad(case.bgrad_got, case.bgrad_theirs, floor_frac=1.0)
