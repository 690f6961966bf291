"""Seeded random sweep over what cublasLtMatmul admits for the quantized types: shapes, transposes,
orders, leading dimensions, batches, epilogues, scale modes, pointer modes, C reads, with and without a
workspace -- every case through the planner's own choice and against the CPU oracle (int8 -> int32
bit-exact, floats within 1e-2).  The point is the seams between the kernel families (LDS-DMA MFMA tiles,
transposing tiles, streaming decode, split-K, generic) rather than any one of them."""
import numpy as np
import pytest

from oracle.cases import Case
from zluda_amd import abi

pytestmark = pytest.mark.gpu
K = abi


def random_spec(rng):
    kind = rng.choice(["i8", "i8f", "f8", "mx"], p=[0.3, 0.25, 0.3, 0.15])
    shape = rng.choice(["small", "skinny", "tiles"])
    if shape == "small":
        m, n = int(rng.integers(1, 200)), int(rng.integers(1, 200))
    elif shape == "skinny":
        m, n = int(rng.choice([256, 512, 1000, 2048])), int(rng.integers(1, 70))
        if rng.random() < 0.3:
            m, n = n, m
    else:
        m, n = int(rng.choice([128, 192, 256, 320, 512])), int(rng.choice([64, 128, 203, 256, 384]))
    kq = int(rng.choice([16, 64, 256]))                      # K granularity of the case
    k = kq * int(rng.integers(1, max(2, 2048 // kq)))
    if shape == "skinny" and rng.random() < 0.5:
        k = int(rng.choice([1024, 2048, 3072, 4096, 2624, 1104]))
    spec = dict(m=m, n=n, k=k)
    if kind == "mx":
        k = max(32, k // 32 * 32)
        spec.update(k=k, a_type=K.CUDA_R_4F_E2M1, b_type=K.CUDA_R_4F_E2M1, compute_type=K.CUBLAS_COMPUTE_32F,
                    scale_type=K.CUDA_R_32F, transa=1, transb=0,
                    a_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0,
                    b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0)
        spec["d_type"] = int(rng.choice([K.CUDA_R_16BF, K.CUDA_R_16F, K.CUDA_R_32F]))
    else:
        ta, tb = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        if rng.random() < 0.4:
            ta, tb = 1, 0                                    # the K-contiguous combination is the common one
        spec.update(transa=ta, transb=tb)
        if rng.random() < 0.25:
            spec.update(order_a=1, order_b=1)
        if kind == "i8":
            spec.update(a_type=K.CUDA_R_8I, b_type=K.CUDA_R_8I, d_type=K.CUDA_R_32I, compute_type=K.CUBLAS_COMPUTE_32I,
                        scale_type=K.CUDA_R_32I)
        elif kind == "i8f":
            spec.update(a_type=K.CUDA_R_8I, b_type=K.CUDA_R_8I, compute_type=K.CUBLAS_COMPUTE_32I, scale_type=K.CUDA_R_32F,
                        d_type=int(rng.choice([K.CUDA_R_16BF, K.CUDA_R_16F, K.CUDA_R_32F])), alpha_range=(0.001, 0.002))
        else:
            at, bt = K.CUDA_R_8F_E4M3, K.CUDA_R_8F_E4M3
            r = rng.random()
            if r < 0.1:
                at = K.CUDA_R_8F_E5M2
            elif r < 0.2:
                bt = K.CUDA_R_8F_E5M2
            spec.update(a_type=at, b_type=bt, compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F,
                        d_type=int(rng.choice([K.CUDA_R_16BF, K.CUDA_R_16F, K.CUDA_R_32F])))
    spec["c_type"] = spec["d_type"]
    if rng.random() < 0.3:
        spec.update(order_c=1, order_d=1)
    if rng.random() < 0.3:
        spec["batch"] = int(rng.integers(2, 4))
    if rng.random() < 0.3:
        spec["with_c"] = True
    # padded leading dimensions (multiples of 4 or 16 bytes, or odd ones: the planner must cope)
    def pad(x):
        return x + int(rng.choice([0, 0, 4, 16, 48, 3]))
    ta, tb = spec.get("transa", 0), spec.get("transb", 0)
    row_a, row_b = spec.get("order_a", 0) == 1, spec.get("order_b", 0) == 1
    a_rows, a_cols = (k, m) if ta else (m, k)
    b_rows, b_cols = (n, k) if tb else (k, n)
    if kind != "mx" and rng.random() < 0.4:
        spec["lda"] = pad(a_cols if row_a else a_rows)
        spec["ldb"] = pad(b_cols if row_b else b_rows)
    if rng.random() < 0.3:
        row_d = spec.get("order_d", 0) == 1
        spec["ldd"] = (n if row_d else m) + int(rng.choice([0, 8, 16, 5]))
        spec["ldc"] = (n if row_d else m) + int(rng.choice([0, 8, 16, 5]))
    if kind != "i8":
        epi = rng.choice(["none", "bias", "relu_bias", "gelu_bias", "gelu", "relu"])
        code = {"none": K.CUBLASLT_EPILOGUE_DEFAULT, "bias": K.CUBLASLT_EPILOGUE_BIAS, "relu_bias": K.CUBLASLT_EPILOGUE_RELU_BIAS,
                "gelu_bias": K.CUBLASLT_EPILOGUE_GELU_BIAS, "gelu": K.CUBLASLT_EPILOGUE_GELU, "relu": K.CUBLASLT_EPILOGUE_RELU}[epi]
        spec["epilogue"] = code
        if "bias" in epi:
            spec["bias_type"] = int(rng.choice([K.CUDA_R_32F, K.CUDA_R_16BF]))
        if kind != "mx":
            r = rng.random()
            if r < 0.3:
                spec.update(with_scalar_scales=True, scale_range=(0.05, 0.06) if kind == "f8" else (0.5, 1.5))
            elif r < 0.55:
                spec.update(a_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F,
                            b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F,
                            scale_range=(0.05, 0.06) if kind == "f8" else (0.5, 1.5))
            elif r < 0.7:
                spec.update(b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F,
                            scale_range=(0.05, 0.06) if kind == "f8" else (0.5, 1.5))
        pm = rng.random()
        if pm < 0.25:
            spec["pointer_mode"] = (K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_HOST if spec.get("with_c")
                                    else K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO)
        elif pm < 0.4 and spec.get("with_c"):    # a device-side beta may be non-zero: the call needs a C then
            spec["pointer_mode"] = K.CUBLASLT_POINTER_MODE_DEVICE
    elif rng.random() < 0.3 and spec.get("with_c"):
        spec["pointer_mode"] = K.CUBLASLT_POINTER_MODE_DEVICE
    return spec


@pytest.mark.parametrize("chunk", range(8))
def test_random_problems_against_the_oracle(gpu_api, chunk):
    rng = np.random.default_rng(9000 + chunk)
    families = {}
    for i in range(24):
        spec = random_spec(rng)
        seed = 9000 + chunk * 100 + i
        ws = int(rng.choice([0, 0, 64 << 20]))
        print("random case", chunk, i, spec, "workspace", ws, flush=True)
        case = Case(spec, seed, int_dist="normal" if rng.random() < 0.3 else "uniform")
        ref = case.run_oracle()
        st, got, kern, variant = case.run_gpu(gpu_api, workspace_bytes=ws)
        assert st == 0, "cublasLtMatmul status %d" % st
        case.compare(got, ref)
        families[kern] = families.get(kern, 0) + 1
    print("kernel families used:", families)
