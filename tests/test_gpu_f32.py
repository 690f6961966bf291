"""f32 x f32 problems on the MFMA kernels (v_mfma_f32_32x32x2_f32: K-contiguous operands on the pipelined kernel, every
other layout on the transposing one) against the float64 oracle and against hipBLASLt called the way the reference
calls it (zluda_blaslt/src/impl.rs:157-196).  Gate 1e-3 of max(|ref|, 1e-2 rms): fp32 sums of a few thousand terms."""
import pytest

from oracle.cases import Case
from zluda_amd import abi as K

pytestmark = pytest.mark.gpu
T = K.CUDA_R_32F
BASE = dict(compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F, alpha=0.05, a_type=T, b_type=T, c_type=T, d_type=T)
F32, TR32 = K.ZLUDA_KERNEL_MFMA_F32, K.ZLUDA_KERNEL_MFMA_TR32

SHAPES = [
    (dict(m=300, n=200, k=384, transa=1, transb=0), F32),
    (dict(m=256, n=256, k=36, transa=1, transb=0), F32),                                       # a K tail inside the first stage
    (dict(m=513, n=130, k=1000, transa=1, transb=0, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS), F32),
    (dict(m=128, n=64, k=2048, transa=1, transb=0, with_c=True, ws=16 << 20), F32),            # split-K through the workspace
    (dict(m=200, n=136, k=264, transa=1, transb=0, batch=3), F32),
    (dict(m=320, n=200, k=256, transa=1, transb=0, order_d=1, order_c=1, epilogue=K.CUBLASLT_EPILOGUE_BIAS), F32),
    (dict(m=300, n=200, k=384, transa=0, transb=0), TR32),
    (dict(m=256, n=256, k=77, transa=0, transb=1), TR32),                                      # odd K, neither operand K-contiguous
    (dict(m=150, n=90, k=2050, transa=0, transb=1, with_c=True), TR32),
    (dict(m=320, n=200, k=256, transa=0, transb=0, order_d=1, order_c=1, epilogue=K.CUBLASLT_EPILOGUE_BIAS), TR32),
    (dict(m=300, n=200, k=392, transa=1, transb=0, lda=395, ldb=399), TR32),                   # K-contiguous, 4-byte aligned pitches
    (dict(m=128, n=512, k=2048, transa=0, transb=0, ws=32 << 20), TR32),
    (dict(m=513, n=131, k=1001, transa=1, transb=1, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS), K.ZLUDA_KERNEL_GENERIC),  # K-contiguous A of 4004-byte rows
]


@pytest.mark.parametrize("shape", range(len(SHAPES)))
def test_f32_operands(gpu_api, shape):
    extra, family = SHAPES[shape]
    extra = dict(extra)
    ws = extra.pop("ws", 0)
    spec = dict(BASE, **extra)
    print("case", spec, flush=True)
    case = Case(spec, 8100 + shape)
    ref = case.run_oracle()
    st, got, kernel, variant = case.run_gpu(gpu_api, workspace_bytes=ws)
    assert st == 0 and kernel == family, (st, kernel)
    assert (case.last_workspace_needed > 0) == (ws > 0)
    case.compare(got, ref, tol=1e-3)
    if family != K.ZLUDA_KERNEL_GENERIC:
        for v in range(gpu_api.zluda_gemm_variant_count(family)):
            st, got_v, k2, v2 = case.run_gpu(gpu_api, forced_kernel=family, forced_variant=v, workspace_bytes=ws)
            assert st == 0 and (k2, v2) == (family, v)
            case.compare(got_v, ref, tol=1e-3)
    if "order_d" in spec:
        return  # (the installed hipBLASLt writes only part of a row-major D with a bias vector)
    theirs, why = case.run_hipblaslt()
    if theirs is None:
        pytest.skip("hipBLASLt offers no algorithm here: " + why)
    case.compare(got, theirs, tol=1e-3, floor_frac=1e-2)
