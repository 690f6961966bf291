"""CUBLASLT_EPILOGUE_BGRADA / BGRADB on the GPU (cuda_types/src/cublaslt.rs:4636-4654; the reference converts
them for hipBLASLt in zluda_common/src/lib.rs:795-800): D as with the DEFAULT epilogue, and the bias buffer
receives the sums over K of op(A)'s rows / op(B)'s columns.  Against the CPU oracle for every kernel family that
can carry the problem and both reduction kernels (K-contiguous operand: one workgroup per row; operand with
unit stride along its row index: one thread per row), and against hipBLASLt itself where it offers an
algorithm."""
import numpy as np
import pytest

from oracle.cases import Case
from zluda_amd import abi

pytestmark = pytest.mark.gpu
K = abi

BF = dict(a_type=K.CUDA_R_16BF, b_type=K.CUDA_R_16BF, c_type=K.CUDA_R_16BF, d_type=K.CUDA_R_16BF,
          compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F, alpha=1.0)
I8F = dict(a_type=K.CUDA_R_8I, b_type=K.CUDA_R_8I, c_type=K.CUDA_R_16BF, d_type=K.CUDA_R_16BF,
           compute_type=K.CUBLAS_COMPUTE_32I, scale_type=K.CUDA_R_32F, alpha=0.01)
F8 = dict(a_type=K.CUDA_R_8F_E4M3, b_type=K.CUDA_R_8F_E4M3, c_type=K.CUDA_R_16BF, d_type=K.CUDA_R_16BF,
          compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F, alpha=1.0)

CASES = [
    # (spec, kernel family expected, integer operands)
    (dict(BF, m=96, n=80, k=200, transa=1), K.ZLUDA_KERNEL_MFMA_H16, False),
    (dict(BF, m=96, n=80, k=200, transa=0, transb=1, bias_type=K.CUDA_R_32F), K.ZLUDA_KERNEL_MFMA_TR16, False),
    (dict(BF, m=96, n=80, k=200, transa=1, lda=201), K.ZLUDA_KERNEL_GENERIC, False),     # an odd pitch: 2-byte alignment only
    (dict(BF, a_type=K.CUDA_R_32F, b_type=K.CUDA_R_32F, m=96, n=80, k=200, transa=0, transb=1, bias_type=K.CUDA_R_32F),
     K.ZLUDA_KERNEL_MFMA_TR32, False),
    (dict(BF, a_type=K.CUDA_R_32F, b_type=K.CUDA_R_32F, m=96, n=80, k=200, transa=1, bias_type=K.CUDA_R_32F), K.ZLUDA_KERNEL_MFMA_F32, False),
    (dict(BF, a_type=K.CUDA_R_32F, b_type=K.CUDA_R_32F, m=96, n=80, k=201, transa=1, bias_type=K.CUDA_R_32F), K.ZLUDA_KERNEL_GENERIC, False),
    (dict(I8F, m=512, n=384, k=1024, transa=1, bias_type=K.CUDA_R_32F), K.ZLUDA_KERNEL_MFMA_I8, True),
    (dict(I8F, m=320, n=256, k=768, transa=0, transb=1, bias_type=K.CUDA_R_32F), K.ZLUDA_KERNEL_MFMA_TR8, True),
    (dict(F8, m=1024, n=256, k=2048, transa=1), K.ZLUDA_KERNEL_MFMA_F8, False),
    (dict(F8, m=256, n=192, k=512, transa=1, batch=3, bias_batch_stride=300, bias_type=K.CUDA_R_32F), K.ZLUDA_KERNEL_MFMA_F8, False),
]


@pytest.mark.parametrize("epi", [K.CUBLASLT_EPILOGUE_BGRADA, K.CUBLASLT_EPILOGUE_BGRADB])
@pytest.mark.parametrize("idx", range(len(CASES)))
def test_bias_gradient_against_the_oracle(gpu_api, idx, epi):
    spec, family, ints = CASES[idx]
    spec = dict(spec, epilogue=epi)
    print("bias gradient:", spec, flush=True)
    case = Case(spec, 900 + idx)
    ref = case.run_oracle()
    st, got, kern, _ = case.run_gpu(gpu_api)
    assert st == 0 and kern == family
    case.compare(got, ref)
    # int8 sums are exact in int32; a 32-bit float output then holds them exactly as well
    case.compare_bgrad(case.bgrad_got, case.bgrad_ref, exact=ints and case.bgrad_type == K.CUDA_R_32F)
    if spec.get("batch", 1) > 1:   # the gaps between the batches' vectors keep the canary
        rows = spec["m"] if epi == K.CUBLASLT_EPILOGUE_BGRADA else spec["n"]
        gap = case.bgrad_got[rows:spec["bias_batch_stride"]]
        assert (gap.view(np.uint8) == 0xCD).all()


# (transa, transb, operand type, bias type, epilogue): the combinations for which the installed hipBLASLt
# (1.2.1, gfx950) returns an algorithm, out of {TN, NN, NT} x {bf16/f32 bias, bf16/bf16, f16/f16, f32/f32} x {A, B}
A_, B_ = K.CUBLASLT_EPILOGUE_BGRADA, K.CUBLASLT_EPILOGUE_BGRADB
HIPBLASLT_OFFERS = [(1, 0, K.CUDA_R_16F, K.CUDA_R_16F, A_), (1, 0, K.CUDA_R_16F, K.CUDA_R_16F, B_), (1, 0, K.CUDA_R_32F, K.CUDA_R_32F, B_),
                    (0, 0, K.CUDA_R_16F, K.CUDA_R_16F, A_), (0, 0, K.CUDA_R_16F, K.CUDA_R_16F, B_), (0, 0, K.CUDA_R_32F, K.CUDA_R_32F, B_),
                    (0, 1, K.CUDA_R_16BF, K.CUDA_R_32F, B_), (0, 1, K.CUDA_R_16BF, K.CUDA_R_16BF, B_),
                    (0, 1, K.CUDA_R_16F, K.CUDA_R_16F, A_), (0, 1, K.CUDA_R_16F, K.CUDA_R_16F, B_), (0, 1, K.CUDA_R_32F, K.CUDA_R_32F, B_)]


@pytest.mark.parametrize("ta,tb,typ,bias_type,epi", HIPBLASLT_OFFERS)
def test_bias_gradient_against_hipblaslt(gpu_api, epi, typ, bias_type, ta, tb):
    """the reference's backend on the same buffers: same D, same gradient vector (16- and 32-bit float operands,
    the types these training epilogues exist for)"""
    spec = dict(BF, a_type=typ, b_type=typ, c_type=typ, d_type=typ, m=256, n=128, k=512, transa=ta, transb=tb,
                epilogue=epi, bias_type=bias_type)
    case = Case(spec, 950)
    st, ours, _, _ = case.run_gpu(gpu_api)
    assert st == 0
    theirs, why = case.run_hipblaslt()
    if theirs is None:
        pytest.skip("hipBLASLt offers no algorithm here: " + why)
    case.compare(ours, theirs, tol=1e-2, floor_frac=1e-2)
    case.compare_bgrad(case.bgrad_got, case.bgrad_theirs)
