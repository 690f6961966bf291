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
    err = case.compare(ours, theirs, tol=1e-2, floor_frac=1e-2)   # both sides use the fp8 MFMA: strict floor
    print("max relative difference to hipBLASLt %.3e" % err)


def test_fp8_decode_shape_within_tolerance_of_hipblaslt(gpu_api):
    """a decode-shaped fp8 problem (16 tokens) runs on the streaming kernel; hipBLASLt has algorithms for it"""
    spec = dict(F8, m=6144, n=16, k=4096, epilogue=K.CUBLASLT_EPILOGUE_BIAS, bias_type=K.CUDA_R_16BF,
                with_scalar_scales=True, scale_range=(0.05, 0.06), bias_std=0.5)
    case, ours, theirs, why, kern = both(gpu_api, spec, 13)
    assert kern == K.ZLUDA_KERNEL_DECODE_W8A8
    if theirs is None:
        pytest.skip("hipBLASLt offers no algorithm here: " + why)
    err = case.compare(ours, theirs, tol=1e-2, floor_frac=1e-2)   # both sides use the fp8 MFMA: strict floor
    print("max relative difference to hipBLASLt %.3e" % err)


def test_fp8_scaled_bias_gelu_within_tolerance_of_hipblaslt(gpu_api):
    """benchmark configuration 4 at 1024^3: per-tensor scales, bf16 bias, GELU, bf16 output"""
    spec = dict(F8, m=1024, n=1024, k=1024, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS, bias_type=K.CUDA_R_16BF,
                with_scalar_scales=True, scale_range=(0.05, 0.06), bias_std=0.5)
    case, ours, theirs, why, kern = both(gpu_api, spec, 3)
    assert kern == K.ZLUDA_KERNEL_MFMA_F8
    if theirs is None:
        pytest.skip("hipBLASLt offers no algorithm here: " + why)
    err = case.compare(ours, theirs, tol=1e-2, floor_frac=1e-2)   # both sides use the fp8 MFMA: strict floor
    print("max relative difference to hipBLASLt %.3e" % err)


def test_config4_fp8_8192_within_tolerance_of_hipblaslt(gpu_api):
    """benchmark configuration 4 at its own size and with its own recipe (x ~ N(0,1), q = e4m3(x * 448 / max|x|), per-tensor
    scales max|x| / 448, bf16 bias ~ N(0, 0.02), GELU, bf16 D), element by element against hipBLASLt called the way the
    reference forwards it.  Both sides use the fp8 MFMA, so the strict floor applies."""
    spec = dict(F8, m=8192, n=8192, k=8192, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS, bias_type=K.CUDA_R_16BF,
                f8_amax_quant=True, bias_std=0.02)
    case, ours, theirs, why, kern = both(gpu_api, spec, 3)
    assert kern == K.ZLUDA_KERNEL_MFMA_F8
    if theirs is None:
        pytest.skip("hipBLASLt offers no algorithm here: " + why)
    err = case.compare(ours, theirs, tol=1e-2, floor_frac=1e-2)
    print("max relative difference to hipBLASLt at 8192^3 %.3e" % err)


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
    case.compare(ours, theirs, tol=1e-2, floor_frac=1e-2)


def test_hipblaslt_fp8_deviates_from_the_fp64_oracle_like_we_do(gpu_api):
    """Why the comparison with the float64 oracle uses floor = 1e-1 * rms for fp8 inputs: the reference's own
    backend, on the same inputs, misses the strict bound (floor 1e-2 * rms) against the exact sum by the same
    order as our kernel does, while the two GPU results agree with each other under the strict floor.  The
    figures of all three comparisons are printed."""
    spec = dict(F8, m=1024, n=1024, k=4096, with_scalar_scales=True, scale_range=(0.05, 0.06))
    case, ours, theirs, why, kern = both(gpu_api, spec, 21)
    assert kern == K.ZLUDA_KERNEL_MFMA_F8
    if theirs is None:
        pytest.skip("hipBLASLt offers no algorithm here: " + why)
    ref = case.run_oracle()
    case.compare(ours, ref)
    e_ours = dict(case.last_errors)
    case.compare(theirs, ref)
    e_theirs = dict(case.last_errors)
    case.compare(ours, theirs, tol=1e-2, floor_frac=1e-2)
    e_both = dict(case.last_errors)
    print("vs float64 oracle: ours %s, hipBLASLt %s; ours vs hipBLASLt %s" % (e_ours, e_theirs, e_both))
    # same order of magnitude: neither implementation is more than 4x further from the exact sum than the other
    hi, lo = max(e_ours["max_abs_over_rms"], e_theirs["max_abs_over_rms"]), min(e_ours["max_abs_over_rms"], e_theirs["max_abs_over_rms"])
    assert hi <= 4 * lo, "one implementation is much further from the exact result than the other"


MX = dict(a_type=K.CUDA_R_4F_E2M1, b_type=K.CUDA_R_4F_E2M1, compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F,
          transa=1, alpha=1.0, a_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0,
          b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0)


def test_mxfp4_scale_tensor_layout_of_hipblaslt(gpu_api):
    """Which byte of the scale tensors does the reference's backend read for (row i, K block kb)?  Answered
    by impulse responses at 256^3, batch 1, fp32 D: every FP4 element of the probed operand is 0 except K
    block kb (all 1.0), the other operand is all 1.0 under unit scales, and byte p of the probed scale tensor
    holds a code that encodes p (two runs: 64 + p % 128 and 64 + p // 128).  D(i, 0) = 32 * 2^(code - 127)
    then names the byte used for (i, kb).  The tensor is four times larger than [256][8] so that a padded or
    tiled layout would show.  Expected: p = i * (K/32) + kb for both operands -- one UE8M0 byte per 32
    elements along K, rows of K/32 bytes, no swizzle (cuda_types/src/cublaslt.rs:3813-3818 read literally)."""
    import ctypes as C
    import torch
    from oracle.hipblaslt_replay import Replay
    n = 256
    kb_count = n // 32
    spec = dict(MX, m=n, n=n, k=n, d_type=K.CUDA_R_32F, c_type=K.CUDA_R_32F)
    print("hipBLASLt MXFP4 scale layout probe", spec, flush=True)
    rp = Replay(spec)
    if rp.why:
        pytest.skip("hipBLASLt cannot describe the problem: " + rp.why)
    dev = torch.device("cuda:0")
    total = 4 * n * kb_count
    d_t = torch.zeros(n * n, dtype=torch.float32, device=dev)
    ones = torch.full((n * n // 2,), 0x22, dtype=torch.uint8, device=dev)       # E2M1 code 2 = 1.0, twice per byte
    flat = torch.full((total,), 127, dtype=torch.uint8, device=dev)              # 2^0
    p = np.arange(total)
    codes = [torch.from_numpy((64 + p % 128).astype(np.uint8)).to(dev), torch.from_numpy((64 + (p // 128) % 128).astype(np.uint8)).to(dev)]
    have_algo = False
    stream = torch.cuda.current_stream().cuda_stream
    try:
        for which in ("A", "B"):
            used = np.zeros((n, kb_count), np.int64)
            for kb in (0, 1, 5, 7):
                data = torch.zeros(n, n // 2, dtype=torch.uint8, device=dev)
                data[:, kb * 16:(kb + 1) * 16] = 0x22
                digits = []
                for enc in range(2):
                    a_s, b_s = (codes[enc], flat) if which == "A" else (flat, codes[enc])
                    assert rp.set_pointers(a_scale=a_s.data_ptr(), b_scale=b_s.data_ptr()), rp.why
                    if not have_algo:
                        if not rp.find_algo():
                            pytest.skip("hipBLASLt offers no MXFP4 algorithm at batch 1: " + rp.why)
                        have_algo = True
                    a_d, b_d = (data, ones) if which == "A" else (ones, data)
                    st = rp.run(C.c_float(1.0), a_d.data_ptr(), b_d.data_ptr(), C.c_float(0.0), None, d_t.data_ptr(), stream)
                    torch.cuda.synchronize()
                    assert st == 0, "hipblasLtMatmul status %d" % st
                    d = d_t.cpu().numpy().astype(np.float64).reshape(n, n)    # [j][i]
                    v = d[0, :] if which == "A" else d[:, 0]
                    assert (v > 0).all()
                    digits.append(np.rint(np.log2(v / 32.0)).astype(np.int64) + 127 - 64)
                used[:, kb] = digits[0] + 128 * digits[1]
                want = np.arange(n) * kb_count + kb
                assert np.array_equal(used[:, kb], want), "operand %s, K block %d: hipBLASLt reads scale bytes %s..., the plain " \
                    "[row][K/32] layout says %s..." % (which, kb, used[:6, kb], want[:6])
    finally:
        rp.close()


@pytest.mark.parametrize("n,dt", [(256, K.CUDA_R_32F), (1024, K.CUDA_R_16BF), (8192, K.CUDA_R_16BF)])
def test_mxfp4_batch1_within_tolerance_of_hipblaslt(gpu_api, n, dt):
    """benchmark configuration 5's problem at batch 1 (the installed hipBLASLt takes block-scaled FP4 for one
    batch only), A:T B:N: random E2M1 codes under scale bytes drawn independently per row and per K block
    (a transposed, tiled or swizzled scale tensor could not agree by accident), ours against hipBLASLt
    called the way the reference forwards it, element by element at the float bar of 1e-2."""
    spec = dict(MX, m=n, n=n, k=n, d_type=dt, c_type=dt, mx_scale_range=(122, 133))
    case, ours, theirs, why, kern = both(gpu_api, spec, 40 + n)
    assert kern == K.ZLUDA_KERNEL_MFMA_MXF4
    if theirs is None:
        pytest.skip("hipBLASLt offers no algorithm here: " + why)
    err = case.compare(ours, theirs, tol=1e-2)
    print("max relative difference to hipBLASLt %.3e" % err)
    if n <= 1024:   # and both against the float64 oracle
        case.compare(theirs, case.run_oracle(), tol=1e-2)
