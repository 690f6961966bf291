"""Parity with the reference's own path: the same seeded problem is run through our cublasLtMatmul and
through hipBLASLt called exactly the way ZLUDA forwards it (oracle/hipblaslt_replay.py restates
zluda_blaslt/src/impl.rs:157-241).  int8 -> int32 must be bit-identical; fp8 must agree within the
1e-2 bound of the float configurations.  Where the installed hipBLASLt has no solution for a
configuration the test says so and the CPU oracle alone pins it (tests/test_gpu_parity.py).

The GELU check at the end settles which GELU hipBLASLt's epilogue applies (the tanh form and the erf
form differ by up to ~5e-4 absolute, far more than the bf16 step for |x| < 1, when looked at in fp32)."""
import numpy as np
import pytest

from oracle.cases import Case, decode_storage
from zluda_amd import abi

pytestmark = pytest.mark.gpu
K = abi

I8 = dict(a_type=K.CUDA_R_8I, b_type=K.CUDA_R_8I, c_type=K.CUDA_R_32I, d_type=K.CUDA_R_32I,
          compute_type=K.CUBLAS_COMPUTE_32I, scale_type=K.CUDA_R_32I, transa=1, alpha=1)
F8 = dict(a_type=K.CUDA_R_8F_E4M3, b_type=K.CUDA_R_8F_E4M3, c_type=K.CUDA_R_16BF, d_type=K.CUDA_R_16BF,
          compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F, transa=1, alpha=1.0)


def both(gpu_api, spec, seed, **kw):
    print("hipBLASLt comparison", spec, flush=True)
    case = Case(spec, seed, **kw)
    st, ours, kern, _ = case.run_gpu(gpu_api)
    assert st == 0
    theirs, why = case.run_hipblaslt()
    return case, ours, theirs, why, kern


@pytest.mark.parametrize("n", [1024, 4096])
def test_int8_bit_exact_with_hipblaslt(gpu_api, n):
    """benchmark configuration 2 (and a quarter-size version): every int32 of D identical"""
    case, ours, theirs, why, kern = both(gpu_api, dict(I8, m=n, n=n, k=n), 1)
    assert kern == K.ZLUDA_KERNEL_MFMA_I8
    if theirs is None:
        pytest.skip("hipBLASLt offers no algorithm here: " + why)
    assert np.array_equal(ours, theirs)


@pytest.mark.parametrize("n,ta,tb", [(256, 0, 1), (1024, 0, 0), (1024, 0, 1), (1024, 1, 1), (4096, 0, 1)])
def test_int8_transposed_layouts_bit_exact_with_hipblaslt(gpu_api, n, ta, tb):
    """benchmark configuration 1 (256^3, A:N B:T) and the other layouts in which an operand is not K-contiguous:
    the transposing MFMA kernel against hipBLASLt called the way the reference forwards it"""
    spec = dict(I8, m=n, n=n, k=n, transa=ta, transb=tb)
    case, ours, theirs, why, kern = both(gpu_api, spec, 11)
    assert kern == K.ZLUDA_KERNEL_MFMA_TR8
    if theirs is None:
        pytest.skip("hipBLASLt offers no algorithm here: " + why)
    assert np.array_equal(ours, theirs)


def test_fp8_transposed_layout_within_tolerance_of_hipblaslt(gpu_api):
    spec = dict(F8, m=1024, n=768, k=512, transa=0, transb=1, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS,
                bias_type=K.CUDA_R_16BF, with_scalar_scales=True, scale_range=(0.05, 0.06), bias_std=0.5)
    case, ours, theirs, why, kern = both(gpu_api, spec, 12)
    assert kern == K.ZLUDA_KERNEL_MFMA_TR8
    if theirs is None:
        pytest.skip("hipBLASLt offers no algorithm here: " + why)
    err = case.compare(ours, theirs, tol=1e-2)
    print("max relative difference to hipBLASLt %.3e" % err)


def test_fp8_decode_shape_within_tolerance_of_hipblaslt(gpu_api):
    """a decode-shaped fp8 problem (16 tokens) runs on the streaming kernel; hipBLASLt has algorithms for it"""
    spec = dict(F8, m=6144, n=16, k=4096, epilogue=K.CUBLASLT_EPILOGUE_BIAS, bias_type=K.CUDA_R_16BF,
                with_scalar_scales=True, scale_range=(0.05, 0.06), bias_std=0.5)
    case, ours, theirs, why, kern = both(gpu_api, spec, 13)
    assert kern == K.ZLUDA_KERNEL_DECODE_W8A8
    if theirs is None:
        pytest.skip("hipBLASLt offers no algorithm here: " + why)
    err = case.compare(ours, theirs, tol=1e-2)
    print("max relative difference to hipBLASLt %.3e" % err)


def test_fp8_scaled_bias_gelu_within_tolerance_of_hipblaslt(gpu_api):
    """benchmark configuration 4 at 1024^3: per-tensor scales, bf16 bias, GELU, bf16 output"""
    spec = dict(F8, m=1024, n=1024, k=1024, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS, bias_type=K.CUDA_R_16BF,
                with_scalar_scales=True, scale_range=(0.05, 0.06), bias_std=0.5)
    case, ours, theirs, why, kern = both(gpu_api, spec, 3)
    assert kern == K.ZLUDA_KERNEL_MFMA_F8
    if theirs is None:
        pytest.skip("hipBLASLt offers no algorithm here: " + why)
    err = case.compare(ours, theirs, tol=1e-2)
    print("max relative difference to hipBLASLt %.3e" % err)


def test_decode_config3_decomposed_through_hipblaslt(gpu_api):
    """benchmark configuration 3 at full size.  hipBLASLt has no int8 -> bf16 algorithm with an alpha vector, so
    the reference's backend pins the integer part: its int8 -> int32 GEMM of the same operands, followed on
    the host by the documented epilogue D[i,j] = bf16(alpha[i] * sB[j] * acc[i,j] + bias[i]) in float64,
    against our fused decode kernel (float bar: 1e-2, bf16 rounding included)."""
    from oracle.cases import _encode
    m, n, k = 14336, 16, 4096
    base = {key: v for key, v in I8.items() if key != "alpha"}      # the decode case draws its alpha vector
    dec = Case(dict(base, c_type=K.CUDA_R_16BF, d_type=K.CUDA_R_16BF, scale_type=K.CUDA_R_32F, m=m, n=n, k=k,
                    pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO,
                    b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F, epilogue=K.CUBLASLT_EPILOGUE_BIAS,
                    bias_type=K.CUDA_R_32F, alpha_range=(0.001, 0.01), scale_range=(0.005, 0.02), bias_std=0.02),
               2, int_dist="normal")
    print("hipBLASLt decomposition of config 3", flush=True)
    st, ours, kern, _ = dec.run_gpu(gpu_api)
    assert st == 0 and kern == K.ZLUDA_KERNEL_DECODE_W8A8
    plain = Case(dict(I8, m=m, n=n, k=k), 2, int_dist="normal")
    assert np.array_equal(plain.A, dec.A) and np.array_equal(plain.B, dec.B)
    acc, why = plain.run_hipblaslt()
    if acc is None:
        pytest.skip("hipBLASLt offers no int8 -> int32 algorithm for 14336 x 16 x 4096: " + why)
    acc = acc.astype(np.float64).reshape(n, m)            # column-major D, ld = m
    want = dec.alpha.astype(np.float64)[None, :] * dec.b_scale.astype(np.float64)[:, None] * acc + \
        decode_storage(dec.bias, K.CUDA_R_32F).astype(np.float64)[None, :]
    err = dec.compare(ours, _encode(want.astype(np.float32).ravel(), K.CUDA_R_16BF), tol=1e-2)
    print("max relative difference to hipBLASLt int32 GEMM + host epilogue %.3e" % err)


def test_gelu_form_of_hipblaslt_is_the_tanh_form(gpu_api):
    """fp32 output, K = 16 with one non-zero product per output: D = GELU(x) for a sweep of x.
    The tanh form 0.5x(1+tanh(sqrt(2/pi)(x+0.044715x^3))) and the erf form 0.5x(1+erf(x/sqrt2)) are
    told apart at fp32 resolution."""
    import math
    spec = dict(F8, c_type=K.CUDA_R_32F, d_type=K.CUDA_R_32F, m=256, n=256, k=64,
                epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS, bias_type=K.CUDA_R_32F, bias_std=1.5)
    case, ours, theirs, why, kern = both(gpu_api, spec, 9)
    if theirs is None:
        pytest.skip("hipBLASLt offers no algorithm here: " + why)
    # recover the pre-activation values from the CPU oracle run without an activation
    lin = Case(dict(spec, epilogue=K.CUBLASLT_EPILOGUE_BIAS), 9)
    x = decode_storage(lin.run_oracle(), K.CUDA_R_32F).astype(np.float64)
    t = decode_storage(theirs, K.CUDA_R_32F).astype(np.float64)
    tanh_form = 0.5 * x * (1 + np.tanh(math.sqrt(2 / math.pi) * (x + 0.044715 * x ** 3)))
    erf_form = 0.5 * x * (1 + np.vectorize(math.erf)(x / math.sqrt(2)))
    # judge where the two forms are furthest apart (|x| around 2..3), by the typical deviation there:
    # the library's own approximation error (fast exp / tanh) is common to both comparisons
    apart = np.abs(tanh_form - erf_form) > 2e-4
    assert apart.sum() > 100
    d_tanh, d_erf = np.median(np.abs(t - tanh_form)[apart]), np.median(np.abs(t - erf_form)[apart])
    print("hipBLASLt GELU over %d outputs where the forms differ by > 2e-4: median |diff| to the tanh form %.3e, "
          "to the erf form %.3e; max |diff| overall %.3e / %.3e" % (apart.sum(), d_tanh, d_erf,
                                                                   np.abs(t - tanh_form).max(), np.abs(t - erf_form).max()))
    assert d_tanh < d_erf, "hipBLASLt applies the erf form: the oracle's GELU must follow"
    case.compare(ours, theirs, tol=1e-2)
