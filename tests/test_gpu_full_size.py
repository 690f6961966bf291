"""benchmark configurations 4 and 5 at their full 8192^3 size.  The CPU oracle cannot finish the whole
problem in seconds, so it recomputes three 64-row slabs of D (first, an interior tile boundary, last):
for K-contiguous operands a slab of op(A) is a pointer offset, so the slab is itself a complete
cublasLtMatmul problem with the same B, scales and epilogue."""
import ctypes as C

import numpy as np
import pytest

import oracle
from oracle.cases import Case
from zluda_amd import abi

pytestmark = pytest.mark.gpu
K = abi


def slab_check(gpu_api, spec, seed, slabs, rows=64, **kw):
    import torch
    print("full-size case", spec, flush=True)
    case = Case(spec, seed, **kw)
    st, got, kern, _ = case.run_gpu(gpu_api)
    assert st == 0
    m, n, k = spec["m"], spec["n"], spec["k"]
    batch = spec.get("batch", 1)
    esz = np.dtype(case.d_np).itemsize
    bits = abi.TYPE_BITS[spec["a_type"]]
    for b in range(batch):
        for i0 in slabs:
            sub = Case.__new__(Case)
            sub.__dict__.update(case.__dict__)
            sub.spec = dict(spec, m=rows, batch=1, ldd=rows, ldc=rows)
            sub.batch = 1
            sub.dtot = rows * n
            a_off = (b * m * k + i0 * k) * bits // 8
            sub.A = case.A[a_off:]
            sub.B = case.B[(b * n * k) * bits // 8:]
            if case.a_scale is not None and case.a_scale.dtype == np.uint8:
                sub.a_scale = case.a_scale.reshape(batch, m, k // 32)[b, i0:i0 + rows].copy()
                sub.b_scale = case.b_scale.reshape(batch, n, k // 32)[b].copy()
            if case.bias is not None:
                sub.bias = case.bias[i0:i0 + rows].copy()
            ref = sub.run_oracle().reshape(n, rows)                       # column-major slab
            full = got[b * m * n:(b + 1) * m * n].reshape(n, m)[:, i0:i0 + rows]
            sub.compare(np.ascontiguousarray(full).ravel(), ref.ravel())
    return kern


def test_config4_fp8_8192_gelu_bias(gpu_api):
    spec = dict(a_type=K.CUDA_R_8F_E4M3, b_type=K.CUDA_R_8F_E4M3, d_type=K.CUDA_R_16BF, c_type=K.CUDA_R_16BF,
                compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F, transa=1, m=8192, n=8192, k=8192,
                epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS, bias_type=K.CUDA_R_16BF, f8_amax_quant=True,
                alpha=1.0, bias_std=0.02)
    # the configuration's own recipe: x ~ N(0,1), q = e4m3(x * 448 / max|x|), per-tensor scale = max|x| / 448,
    # bf16 bias ~ N(0, 0.02)
    kern = slab_check(gpu_api, spec, 3, [0, 4064, 8128])
    assert kern == K.ZLUDA_KERNEL_MFMA_F8


def test_config5_mxfp4_8192_batch4(gpu_api):
    spec = dict(a_type=K.CUDA_R_4F_E2M1, b_type=K.CUDA_R_4F_E2M1, d_type=K.CUDA_R_16BF, c_type=K.CUDA_R_16BF,
                compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F, transa=1, m=8192, n=8192, k=8192,
                batch=4, a_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0,
                b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0, alpha=1.0)
    kern = slab_check(gpu_api, spec, 4, [0, 8128], rows=32)
    assert kern == K.ZLUDA_KERNEL_MFMA_MXF4
