"""Pins the GEMM half of the CPU oracle without a GPU: the reference's int8 mma.sync and dp4a result
vectors, numpy int64 / float64 matmuls written from the layout definitions (not from the oracle's
code), exact small cases, and the epilogue formulas."""
import ctypes as C
import json
import os
from fractions import Fraction

import numpy as np
import pytest

import oracle
from oracle.cases import Case, decode_storage
from zluda_amd import abi

GOLD = os.path.join(os.path.dirname(__file__), "golden")

I8 = dict(a_type=abi.CUDA_R_8I, b_type=abi.CUDA_R_8I, d_type=abi.CUDA_R_32I,
          compute_type=abi.CUBLAS_COMPUTE_32I, scale_type=abi.CUDA_R_32I)


def logical(case, store, tag, rows, cols, b=0):
    """stored matrix `tag` of batch b as a [rows, cols] array, straight from the layout definition"""
    s = case.spec
    order = s.get("order_" + tag, 0)
    ld = s.get("ld" + tag, rows if order == 0 else cols)
    stride = s.get("stride_" + tag, ld * (cols if order == 0 else rows))
    r = np.arange(rows)[:, None]
    c = np.arange(cols)[None, :]
    idx = (r + c * ld) if order == 0 else (r * ld + c)
    return store[idx + b * stride]


def op_matrices(case, b=0):
    s = case.spec
    m, n, k = s["m"], s["n"], s["k"]
    ta, tb = s.get("transa", 0) != 0, s.get("transb", 0) != 0
    A = logical(case, case.A, "a", k if ta else m, m if ta else k, b)
    B = logical(case, case.B, "b", n if tb else k, k if tb else n, b)
    return (A.T if ta else A), (B.T if tb else B)


def test_reference_mma_m16n8k32_vector():
    f = json.load(open(os.path.join(GOLD, "mma_m16n8k32_s8.json")))
    for w in f["warps"]:
        spec = dict(I8, m=16, n=8, k=32, order_a=1, order_b=0, order_c=1, order_d=1, with_c=True, alpha=1)
        case = Case(spec, 0)
        case.A = np.array(w["A"], dtype=np.int8).ravel()            # row-major 16x32
        case.B = np.array(w["B"], dtype=np.int8).T.copy().ravel()   # col-major 32x8
        case.Cm = np.array(w["C"], dtype=np.int32).ravel()
        case.alpha[:] = 1
        case.beta[:] = 1
        d = case.run_oracle()
        assert np.array_equal(d.reshape(16, 8), np.array(w["D"], dtype=np.int32))


def test_reference_dp4a_vector():
    k = json.load(open(os.path.join(GOLD, "ptx_cvt_kat.json")))["dp4a_s32"]
    a = np.array([k["a"]], dtype=np.uint32).view(np.int8)
    b = np.array([k["b"]], dtype=np.uint32).view(np.int8)
    spec = dict(I8, m=1, n=1, k=4, transa=1, with_c=True, alpha=1)
    case = Case(spec, 0)
    case.A, case.B = a.copy(), b.copy()
    case.Cm = np.array([k["c"]], dtype=np.uint32).view(np.int32).copy()
    case.alpha[:] = 1
    case.beta[:] = 1
    assert int(case.run_oracle()[0]) == k["out"]


@pytest.mark.parametrize("ta", [0, 1])
@pytest.mark.parametrize("tb", [0, 1])
@pytest.mark.parametrize("oa,ob,od", [(0, 0, 0), (1, 0, 0), (0, 1, 1), (1, 1, 1)])
def test_int8_layouts_against_numpy(ta, tb, oa, ob, od):
    m, n, k, batch = 7, 5, 12, 3
    spec = dict(I8, m=m, n=n, k=k, batch=batch, transa=ta, transb=tb, order_a=oa, order_b=ob, order_c=od,
                order_d=od, with_c=True)
    # padded leading dimensions and batch strides
    ar, ac = (k, m) if ta else (m, k)
    br, bc = (n, k) if tb else (k, n)
    spec["lda"] = (ar if oa == 0 else ac) + 3
    spec["ldb"] = (br if ob == 0 else bc) + 2
    spec["ldd"] = (m if od == 0 else n) + 4
    spec["ldc"] = (m if od == 0 else n) + 1
    spec["stride_a"] = spec["lda"] * (ac if oa == 0 else ar) + 5
    spec["stride_d"] = spec["ldd"] * (n if od == 0 else m) + 7
    case = Case(spec, 42)
    d = case.run_oracle()
    idx = case.logical_index()
    for b in range(batch):
        A, B = op_matrices(case, b)
        Cm = logical(case, case.Cm, "c", m, n, b)
        want = int(case.alpha[0]) * (A.astype(np.int64) @ B.astype(np.int64)) + int(case.beta[0]) * Cm.astype(np.int64)
        assert np.array_equal(d[idx[b]], want.astype(np.int32))
    mask = np.ones(d.size, bool)
    mask[idx.ravel()] = False
    assert (d[mask].view(np.uint8) == 0xCD).all(), "oracle wrote outside the logical matrix"


def test_int8_config1_shape_identity_and_transpose():
    # benchmark configuration 1: 256^3, A:N B:T column-major, alpha=1 beta=0, seed 0
    spec = dict(I8, m=256, n=256, k=256, transa=0, transb=1, alpha=1)
    case = Case(spec, 0)
    d = case.run_oracle().reshape(256, 256).T  # col-major storage -> [i, j]
    A, B = op_matrices(case)
    want = A.astype(np.int64) @ B.astype(np.int64)
    assert np.array_equal(d, want.astype(np.int32))
    # (AB)^T = B^T A^T through the API: swap operands and transposes, row-major output
    spec2 = dict(I8, m=256, n=256, k=256, transa=0, transb=1, alpha=1, order_d=1, order_c=1)
    case2 = Case(spec2, 0)
    case2.A, case2.B = case.B, case.A   # op(A2) = B (256x256 N), op(B2) = A^T
    d2 = case2.run_oracle().reshape(256, 256)  # row-major [i, j] of (B A^T)... compare via numpy
    A2, B2 = op_matrices(case2)
    assert np.array_equal(d2, (A2.astype(np.int64) @ B2.astype(np.int64)).astype(np.int32))
    # one-hot A picks rows of op(B)
    case3 = Case(dict(I8, m=4, n=6, k=8, transa=1, alpha=1), 1)
    case3.A[:] = 0
    Aop = np.zeros((4, 8), np.int8)
    for i in range(4):
        Aop[i, 2 * i] = 1
    case3.A = Aop.ravel().copy()  # transa=T col-major: stored k x m, element (k,i) at k + i*8 == row-major [i][k]
    d3 = case3.run_oracle().reshape(6, 4).T
    _, B3 = op_matrices(case3)
    assert np.array_equal(d3, B3[[0, 2, 4, 6], :].astype(np.int32))


def test_int32_accumulator_extremes_no_overflow():
    # |sum| <= K * 128 * 128 = 2^26 for K = 4096: the largest value config 2 can produce
    spec = dict(I8, m=2, n=2, k=4096, transa=1, alpha=1)
    case = Case(spec, 0)
    case.A[:] = -128
    case.B[:] = -128
    assert (case.run_oracle() == 4096 * 128 * 128).all()
    case.B[:] = 127
    assert (case.run_oracle() == -4096 * 128 * 127).all()


F8 = dict(a_type=abi.CUDA_R_8F_E4M3, b_type=abi.CUDA_R_8F_E4M3, d_type=abi.CUDA_R_32F,
          compute_type=abi.CUBLAS_COMPUTE_32F, scale_type=abi.CUDA_R_32F)


def test_fp8_tiny_exact_rational():
    spec = dict(F8, m=3, n=2, k=8, transa=1, alpha=1.0)
    case = Case(spec, 9)
    d = case.run_oracle().reshape(2, 3).T
    tab = oracle.decode_table("e4m3")
    A, B = op_matrices(case)
    for i in range(3):
        for j in range(2):
            acc = sum(Fraction(float(tab[A[i, kk]])) * Fraction(float(tab[B[kk, j]])) for kk in range(8))
            assert d[i, j] == np.float32(float(acc))


@pytest.mark.parametrize("at,bt", [(abi.CUDA_R_8F_E4M3, abi.CUDA_R_8F_E4M3), (abi.CUDA_R_8F_E5M2, abi.CUDA_R_8F_E4M3),
                                   (abi.CUDA_R_16BF, abi.CUDA_R_16BF), (abi.CUDA_R_16F, abi.CUDA_R_16F),
                                   (abi.CUDA_R_32F, abi.CUDA_R_32F)])
def test_float_gemm_against_numpy_float64(at, bt):
    spec = dict(F8, a_type=at, b_type=bt, m=33, n=17, k=64, transa=1, d_type=abi.CUDA_R_32F,
                epilogue=abi.CUBLASLT_EPILOGUE_RELU_BIAS, with_c=True, with_scalar_scales=True,
                with_cd_scales=True, lda=80, ldd=40)
    case = Case(spec, 21)
    d = case.run_oracle()
    A, B = op_matrices(case)
    Af, Bf = decode_storage(A, at), decode_storage(B, bt)
    Cf = logical(case, case.Cm, "c", 33, 17).astype(np.float64)
    bias = case.bias.astype(np.float64)
    x = case.alpha[0] * case.a_scale[0] * case.b_scale[0] * (Af @ Bf) + case.beta[0] * case.c_scale[0] * Cf + bias[:, None]
    want = np.maximum(x, 0) * case.d_scale[0]
    got = d[case.logical_index()[0]].astype(np.float64)
    assert np.max(np.abs(got - want)) <= 1e-5 * np.max(np.abs(want))


def test_mxfp4_block_scaled_against_numpy():
    m, n, k, batch = 9, 6, 96, 2
    spec = dict(a_type=abi.CUDA_R_4F_E2M1, b_type=abi.CUDA_R_4F_E2M1, d_type=abi.CUDA_R_16BF,
                compute_type=abi.CUBLAS_COMPUTE_32F, scale_type=abi.CUDA_R_32F, m=m, n=n, k=k, batch=batch,
                transa=1, a_scale_mode=abi.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0,
                b_scale_mode=abi.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0, alpha=1.0)
    case = Case(spec, 4)
    d = case.run_oracle()
    e2m1 = oracle.decode_table("e2m1").astype(np.float64)
    idx = case.logical_index()
    for b in range(batch):
        def deq(store, scales, nvec):
            out = np.empty((nvec, k))
            for v in range(nvec):
                off = (b * nvec * k + v * k) // 2
                by = store[off:off + k // 2]
                vals = np.empty(k)
                vals[0::2] = e2m1[by & 15]
                vals[1::2] = e2m1[by >> 4]
                out[v] = vals * np.repeat(2.0 ** (scales[b, v].astype(np.float64) - 127), 32)
            return out
        Af, Bf = deq(case.A, case.a_scale, m), deq(case.B, case.b_scale, n)
        want = Af @ Bf.T
        got = oracle.decode_bf16(d[idx[b]]).astype(np.float64)
        assert np.max(np.abs(got - want)) <= 2.0 ** -8 * np.max(np.abs(want)) + 1e-30


def test_w8a8_decode_epilogue_formula():
    # config 3 in miniature: alpha vector per output channel, outer-vector B scale per token, fp32 bias, bf16 out
    m, n, k = 48, 16, 128
    spec = dict(a_type=abi.CUDA_R_8I, b_type=abi.CUDA_R_8I, d_type=abi.CUDA_R_16BF,
                compute_type=abi.CUBLAS_COMPUTE_32I, scale_type=abi.CUDA_R_32F, m=m, n=n, k=k, transa=1,
                pointer_mode=abi.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO,
                b_scale_mode=abi.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F,
                epilogue=abi.CUBLASLT_EPILOGUE_BIAS, bias_type=abi.CUDA_R_32F,
                alpha_range=(0.001, 0.01), scale_range=(0.005, 0.02), bias_std=0.02)
    case = Case(spec, 2, int_dist="normal")
    d = case.run_oracle()
    A, B = op_matrices(case)
    acc = (A.astype(np.int64) @ B.astype(np.int64)).astype(np.float64)
    want = case.alpha.astype(np.float64)[:, None] * case.b_scale.astype(np.float64)[None, :] * acc + case.bias.astype(np.float64)[:, None]
    got = oracle.decode_bf16(d[case.logical_index()[0]]).astype(np.float64)
    assert np.max(np.abs(got - want) / np.maximum(np.abs(want), 1e-3)) <= 2.0 ** -8
    # the bias really is per row of D and the B scale per column: perturbing one entry moves one row / column
    case.bias[5] += 100.0
    d2 = oracle.decode_bf16(case.run_oracle()[case.logical_index()[0]])
    diff = np.abs(d2.astype(np.float64) - got) > 1.0
    assert diff[5].all() and not np.delete(diff, 5, axis=0).any()


def test_gelu_bias_order_and_int8_saturation():
    spec = dict(F8, m=4, n=3, k=32, transa=1, d_type=abi.CUDA_R_32F, epilogue=abi.CUBLASLT_EPILOGUE_GELU_BIAS, alpha=1.0)
    case = Case(spec, 8)
    d = case.run_oracle().reshape(3, 4).T
    A, B = op_matrices(case)
    x = decode_storage(A, abi.CUDA_R_8F_E4M3) @ decode_storage(B, abi.CUDA_R_8F_E4M3) + case.bias.astype(np.float64)[:, None]
    want = 0.5 * x * (1 + np.tanh(np.sqrt(2 / np.pi) * (x + 0.044715 * x ** 3)))
    assert np.max(np.abs(d - want)) <= 1e-5 * max(1.0, np.max(np.abs(want)))
    # int8 output: round to nearest even, saturate
    spec = dict(a_type=abi.CUDA_R_8I, b_type=abi.CUDA_R_8I, d_type=abi.CUDA_R_8I, compute_type=abi.CUBLAS_COMPUTE_32I,
                scale_type=abi.CUDA_R_32F, m=2, n=2, k=4, transa=1, alpha=0.5)
    case = Case(spec, 0)
    case.A = np.array([1, 0, 0, 0, 127, 127, 127, 127], dtype=np.int8)  # rows of op(A)
    case.B = np.array([5, 0, 0, 0, 127, 127, 127, 127], dtype=np.int8)  # columns of op(B)
    d = case.run_oracle().reshape(2, 2).T
    assert d[0, 0] == 2        # 0.5 * 5 = 2.5 -> 2 (even)
    assert d[1, 1] == 127      # 0.5 * 4*127*127 saturates
    assert d[1, 0] == 127 and d[0, 1] == 64   # 0.5*635=317.5 -> sat ; 0.5*127=63.5 -> 64


def test_oracle_rejects_bad_shapes():
    case = Case(dict(I8, m=4, n=4, k=4, alpha=1), 0)
    hp = lambda x: x.ctypes.data
    d = case.new_d()
    p = case.problem({"A": hp(case.A), "B": hp(case.B), "D": hp(d), "alpha": hp(case.alpha), "beta": hp(case.beta)})
    p.b.rows = 5
    assert oracle.gemm(p) == abi.CUBLAS_STATUS_INVALID_VALUE


@pytest.mark.parametrize("which", ["a", "b"])
@pytest.mark.parametrize("typ", [abi.CUDA_R_8I, abi.CUDA_R_16BF, abi.CUDA_R_8F_E4M3])
@pytest.mark.parametrize("ta,tb,oa,ob", [(1, 0, 0, 0), (0, 1, 0, 0), (0, 0, 1, 1)])
def test_bias_gradient_epilogues_against_numpy(which, typ, ta, tb, oa, ob):
    """BGRADA / BGRADB: the bias buffer receives the sums over K of op(A)'s rows / op(B)'s columns (numpy sums of
    the matrices read straight from the layout definition), per batch at the bias batch stride, in the bias data
    type; D is what the DEFAULT epilogue gives."""
    epi = abi.CUBLASLT_EPILOGUE_BGRADA if which == "a" else abi.CUBLASLT_EPILOGUE_BGRADB
    base = dict(a_type=typ, b_type=typ, d_type=abi.CUDA_R_32F, compute_type=abi.CUBLAS_COMPUTE_32F, scale_type=abi.CUDA_R_32F,
                alpha=1.0, m=19, n=11, k=48, transa=ta, transb=tb, order_a=oa, order_b=ob, batch=2, bias_batch_stride=24)
    if typ == abi.CUDA_R_8I:
        base.update(compute_type=abi.CUBLAS_COMPUTE_32I)
    case = Case(dict(base, epilogue=epi, bias_type=abi.CUDA_R_32F), 77)
    d = case.run_oracle()
    plain = Case(dict(base), 77)
    np.testing.assert_array_equal(d, plain.run_oracle())
    rows = 19 if which == "a" else 11
    for b in range(2):
        A, B = op_matrices(case, b)
        src = decode_storage(A, typ) if which == "a" else decode_storage(B, typ).T
        want = src.sum(axis=1)
        got = case.bgrad_ref[24 * b:24 * b + rows].astype(np.float64)
        assert np.max(np.abs(got - want)) <= 1e-6 * max(1.0, np.max(np.abs(want)))
    # what lies between the batches' vectors stays untouched
    assert (case.bgrad_ref[rows:24].view(np.uint32) == 0xCDCDCDCD).all()


def test_gelu_derivative_against_differences_and_limits():
    """oracle_dgelu is the derivative of oracle's GELU: central differences of the float64 tanh form, 1/2 at 0, 0 and
    1 far out, and gelu'(x) + gelu'(-x) = 1 (GELU(x) - GELU(-x) = x)"""
    L = oracle.lib()
    k0, k1 = 0.7978845608028654, 0.044715
    gelu = lambda x: 0.5 * x * (1.0 + np.tanh(k0 * (x + k1 * x ** 3)))
    for x in np.linspace(-6.0, 6.0, 241):
        h = 1e-5
        want = (gelu(x + h) - gelu(x - h)) / (2 * h)
        got = L.oracle_dgelu(C.c_float(x))
        assert abs(got - want) <= 2e-6, (x, got, want)
        assert abs(L.oracle_dgelu(C.c_float(x)) + L.oracle_dgelu(C.c_float(-x)) - 1.0) <= 1e-6
    assert L.oracle_dgelu(C.c_float(0.0)) == 0.5
    assert abs(L.oracle_dgelu(C.c_float(-30.0))) <= 1e-7 and abs(L.oracle_dgelu(C.c_float(30.0)) - 1.0) <= 1e-7


@pytest.mark.parametrize("dt", [abi.CUDA_R_32F, abi.CUDA_R_16BF])
@pytest.mark.parametrize("od", [0, 1])
def test_gelu_aux_and_dgelu_epilogues_against_numpy(dt, od):
    """GELU_AUX_BIAS: the aux matrix holds alpha * op(A) op(B) + bias (the GELU input) at its own leading dimension and
    batch stride, D its GELU; DGELU_BGRAD: D = (alpha * op(A) op(B) + beta * C) * gelu'(aux), the bias buffer the sums
    of D's rows.  Both against numpy float64 from the layout definitions."""
    k0, k1 = 0.7978845608028654, 0.044715
    gelu = lambda x: 0.5 * x * (1.0 + np.tanh(k0 * (x + k1 * x ** 3)))
    dgelu = lambda x: 0.5 * (1 + np.tanh(k0 * (x + k1 * x ** 3))) + 0.5 * x * (1 - np.tanh(k0 * (x + k1 * x ** 3)) ** 2) * k0 * (1 + 3 * k1 * x * x)
    m, n, k, lda_aux = 13, 9, 40, 16
    base = dict(a_type=abi.CUDA_R_16BF, b_type=abi.CUDA_R_16BF, d_type=dt, compute_type=abi.CUBLAS_COMPUTE_32F,
                scale_type=abi.CUDA_R_32F, alpha=0.25, m=m, n=n, k=k, transa=1, batch=2, order_c=od, order_d=od,
                aux_ld=lda_aux, aux_batch_stride=lda_aux * 16)
    tol = 1e-4 if dt == abi.CUDA_R_32F else 2.0 ** -8   # (the oracle evaluates GELU in float32: 1 + tanh cancels for x << 0)

    def logical(case, storage, ld, stride, b):
        i, j = np.meshgrid(np.arange(m), np.arange(n), indexing="ij")
        idx = (i * ld + j) if od else (j * ld + i)
        return decode_storage(storage[idx + b * stride], dt).astype(np.float64)

    fwd = Case(dict(base, epilogue=abi.CUBLASLT_EPILOGUE_GELU_AUX_BIAS, bias_type=abi.CUDA_R_32F), 91)
    d = fwd.run_oracle()
    _, ldd, sd = __import__("oracle.cases", fromlist=["_layout"])._layout(fwd.spec, "d", m, n)
    for b in range(2):
        A, B = op_matrices(fwd, b)
        x = 0.25 * decode_storage(A, abi.CUDA_R_16BF).astype(np.float64) @ decode_storage(B, abi.CUDA_R_16BF).astype(np.float64)
        x = x + fwd.bias.astype(np.float64)[:m, None]
        aux = logical(fwd, fwd.aux_ref, lda_aux, lda_aux * 16, b)
        assert np.max(np.abs(aux - x) / np.maximum(np.abs(x), 1e-3)) <= tol
        got = logical(fwd, d, ldd, sd, b)
        assert np.max(np.abs(got - gelu(x)) / np.maximum(np.abs(gelu(x)), 1e-2)) <= tol
    bwd = Case(dict(base, epilogue=abi.CUBLASLT_EPILOGUE_DGELU_BGRAD, bias_type=abi.CUDA_R_32F, bias_batch_stride=16, with_c=True), 92)
    d = bwd.run_oracle()
    for b in range(2):
        A, B = op_matrices(bwd, b)
        y = 0.25 * decode_storage(A, abi.CUDA_R_16BF).astype(np.float64) @ decode_storage(B, abi.CUDA_R_16BF).astype(np.float64)
        y = y + float(bwd.beta[0]) * logical(bwd, bwd.Cm, ldd, sd, b)
        want = y * dgelu(logical(bwd, bwd.aux, lda_aux, lda_aux * 16, b))
        got = logical(bwd, d, ldd, sd, b)
        assert np.max(np.abs(got - want) / np.maximum(np.abs(want), 1e-2)) <= tol
        sums = bwd.bgrad_ref[16 * b:16 * b + m].astype(np.float64)
        assert np.max(np.abs(sums - want.sum(axis=1))) <= 1e-5 * max(1.0, np.max(np.abs(want.sum(axis=1)))) + (0 if dt == abi.CUDA_R_32F else 0)
    assert (bwd.bgrad_ref[m:16].view(np.uint32) == 0xCDCDCDCD).all()
