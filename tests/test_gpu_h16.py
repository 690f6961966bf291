"""f16 x f16 and bf16 x bf16 problems (the 16-bit operand types cublasLtMatmul is mostly called with outside of quantized
inference; the reference forwards them to hipBLASLt like everything else, zluda_blaslt/src/impl.rs:157-196) on the MFMA
kernels (K-contiguous operands on the pipelined kernel, every other layout on the transposing one): against the float64 oracle, and against hipBLASLt called the way the reference calls it."""
import pytest

from oracle.cases import Case
from zluda_amd import abi as K

pytestmark = pytest.mark.gpu

TYPES = {"bf16": K.CUDA_R_16BF, "f16": K.CUDA_R_16F}


def base(typ, **kw):
    t = TYPES[typ]
    return dict(dict(a_type=t, b_type=t, c_type=t, d_type=t, compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F,
                     transa=1, transb=0, alpha=0.05), **kw)


SHAPES = [
    dict(m=300, n=200, k=384),
    dict(m=256, n=256, k=72),                                                   # a K tail inside the first stage
    dict(m=513, n=130, k=1000, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS),
    dict(m=128, n=64, k=4096, with_c=True),
    dict(m=200, n=136, k=264, batch=3, d_type=K.CUDA_R_32F, c_type=K.CUDA_R_32F),
    dict(m=1024, n=1024, k=1024, epilogue=K.CUBLASLT_EPILOGUE_RELU_BIAS),
    dict(m=320, n=200, k=256, order_d=1, order_c=1, epilogue=K.CUBLASLT_EPILOGUE_BIAS),  # row-major D: computed as D^T
]


@pytest.mark.parametrize("typ", ["bf16", "f16"])
@pytest.mark.parametrize("shape", range(len(SHAPES)))
def test_k_contiguous_operands_run_on_the_16_bit_mfma_family(gpu_api, typ, shape):
    spec = base(typ, **SHAPES[shape])
    print("case", spec, flush=True)
    case = Case(spec, 7700 + shape)
    ref = case.run_oracle()
    st, got, kernel, variant = case.run_gpu(gpu_api)
    assert st == 0 and kernel == K.ZLUDA_KERNEL_MFMA_H16, (st, kernel)
    case.compare(got, ref, tol=1e-2)
    # every tile shape of the family gives the same sums (fp32 accumulation in K order inside a tile)
    for v in range(gpu_api.zluda_gemm_variant_count(K.ZLUDA_KERNEL_MFMA_H16)):
        st, got_v, kernel, variant = case.run_gpu(gpu_api, forced_kernel=K.ZLUDA_KERNEL_MFMA_H16, forced_variant=v)
        assert st == 0 and (kernel, variant) == (K.ZLUDA_KERNEL_MFMA_H16, v)
        case.compare(got_v, ref, tol=1e-2)
    if "order_d" in spec:
        return  # (the installed hipBLASLt writes only part of a row-major D with a bias vector)
    theirs, why = case.run_hipblaslt()
    if theirs is None:
        pytest.skip("hipBLASLt offers no algorithm here: " + why)
    case.compare(got, theirs, tol=1e-2, floor_frac=1e-2)


TR_SHAPES = [
    dict(m=300, n=200, k=384, transa=0, transb=0),
    dict(m=256, n=256, k=77, transa=0, transb=1),                                # odd K: neither operand has K pieces of 16 bytes
    dict(m=513, n=130, k=1000, transa=1, transb=1, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS),
    dict(m=150, n=90, k=4100, transa=0, transb=1, with_c=True),
    dict(m=200, n=136, k=264, transa=0, transb=0, batch=3, d_type=K.CUDA_R_32F, c_type=K.CUDA_R_32F),
    dict(m=320, n=200, k=256, transa=0, transb=0, order_d=1, order_c=1, epilogue=K.CUBLASLT_EPILOGUE_BIAS),
    dict(m=300, n=200, k=392, transa=1, transb=0, lda=394, ldb=398),             # K-contiguous, pitches of 4-byte alignment only
    dict(m=128, n=512, k=4096, transa=0, transb=0, ws=32 << 20),                 # few tiles, long K: split through the workspace
]


@pytest.mark.parametrize("typ", ["bf16", "f16"])
@pytest.mark.parametrize("shape", range(len(TR_SHAPES)))
def test_other_layouts_run_on_the_transposing_kernel(gpu_api, typ, shape):
    """A:N, B:T, A:T B:T, row-major D and K-contiguous operands whose pitches are not multiples of 16 bytes"""
    extra = dict(TR_SHAPES[shape])
    ws = extra.pop("ws", 0)
    spec = base(typ, **extra)
    print("case", spec, flush=True)
    case = Case(spec, 7900 + shape)
    ref = case.run_oracle()
    st, got, kernel, variant = case.run_gpu(gpu_api, workspace_bytes=ws)
    assert st == 0 and kernel == K.ZLUDA_KERNEL_MFMA_TR16, (st, kernel)
    assert (case.last_workspace_needed > 0) == (ws > 0)
    case.compare(got, ref, tol=1e-2)
    for v in range(gpu_api.zluda_gemm_variant_count(K.ZLUDA_KERNEL_MFMA_TR16)):
        st, got_v, kernel, variant = case.run_gpu(gpu_api, forced_kernel=K.ZLUDA_KERNEL_MFMA_TR16, forced_variant=v, workspace_bytes=ws)
        assert st == 0 and (kernel, variant) == (K.ZLUDA_KERNEL_MFMA_TR16, v)
        case.compare(got_v, ref, tol=1e-2)
    if "order_d" in spec:
        return  # (the installed hipBLASLt writes only part of a row-major D with a bias vector)
    theirs, why = case.run_hipblaslt()
    if theirs is None:
        pytest.skip("hipBLASLt offers no algorithm here: " + why)
    case.compare(got, theirs, tol=1e-2, floor_frac=1e-2)


DECODE_SHAPES = [
    (dict(m=1024, n=16, k=2048), 16),
    (dict(m=1000, n=5, k=1536, lda=1600), 16),                                    # a K tail, ragged rows, padded pitch
    (dict(m=2048, n=16, k=4096, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS), 17),
    (dict(m=332, n=29, k=2048), 20),                                              # two token blocks
    (dict(m=512, n=32, k=4096), 17),
    (dict(m=1028, n=7, k=6144, epilogue=K.CUBLASLT_EPILOGUE_RELU_BIAS), 18),
    (dict(m=640, n=12, k=7000, d_type=K.CUDA_R_32F, c_type=K.CUDA_R_32F), 19),    # element-wise epilogue
    (dict(m=16, n=2048, k=4096), 17),                                             # tokens along M: the weights are B
    (dict(m=900, n=16, k=4096, with_c=True), 17),
    (dict(m=768, n=16, k=1280, batch=2), 16),
]


@pytest.mark.parametrize("typ", ["bf16", "f16"])
@pytest.mark.parametrize("shape", range(len(DECODE_SHAPES)))
def test_16_bit_weights_stream_through_the_slab_decode(gpu_api, typ, shape):
    """few tokens, K-contiguous 16-bit weights of up to 16 KiB per row: the slab decode kernel with K counted in bytes"""
    extra, variant = DECODE_SHAPES[shape]
    spec = base(typ, **extra)
    print("case", spec, flush=True)
    case = Case(spec, 8000 + shape)
    ref = case.run_oracle()
    st, got, kernel, v = case.run_gpu(gpu_api)
    assert st == 0 and (kernel, v) == (K.ZLUDA_KERNEL_DECODE_W8A8, variant), (st, kernel, v)
    case.compare(got, ref, tol=1e-2)
    theirs, why = case.run_hipblaslt()
    if theirs is None:
        pytest.skip("hipBLASLt offers no algorithm here: " + why)
    case.compare(got, theirs, tol=1e-2, floor_frac=1e-2)


def test_16_bit_slab_decode_on_more_workgroups_than_cus(gpu_api):
    """long K keeps the slab form beyond 64 rows per CU: 320 workgroups, the later ones following another on their CU"""
    case = Case(base("bf16", m=20480, n=16, k=8192), 8050)
    ref = case.run_oracle()
    for rep in range(2):
        st, got, kernel, v = case.run_gpu(gpu_api)
        assert st == 0 and (kernel, v) == (K.ZLUDA_KERNEL_DECODE_W8A8, 19)
        case.compare(got, ref, tol=1e-2)


@pytest.mark.parametrize("typ", ["bf16", "f16"])
def test_16_bit_split_k_through_the_workspace(gpu_api, typ):
    spec = base(typ, m=512, n=256, k=8192, epilogue=K.CUBLASLT_EPILOGUE_BIAS)
    case = Case(spec, 7800)
    ref = case.run_oracle()
    st, got, kernel, _ = case.run_gpu(gpu_api, workspace_bytes=32 << 20)
    assert st == 0 and kernel == K.ZLUDA_KERNEL_MFMA_H16
    assert case.last_workspace_needed > 0, "few tiles and a long K: the plan shares K between workgroups"
    case.compare(got, ref, tol=1e-2)


def test_16_bit_operands_of_two_types_are_refused(gpu_api):
    spec = base("bf16", m=128, n=128, k=128, b_type=K.CUDA_R_16F)
    case = Case.__new__(Case)
    case.spec, case.batch = spec, 1
    import ctypes as C
    p = case.problem({"A": 0, "B": 0, "D": 0, "alpha": 0, "beta": 0})
    out = K.zluda_gemm_plan()
    assert gpu_api.zluda_gemm_plan_problem(C.byref(p), 0, -1, 256, C.byref(out)) == K.CUBLAS_STATUS_NOT_SUPPORTED
