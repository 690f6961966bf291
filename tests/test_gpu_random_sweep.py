"""Seeded random sweep on the GPU: problems drawn over every family of the library (int8 with integer and with
float scaling, fp8 in its three operand mixes, MXFP4, 16/32-bit floats), transposes, orders, padded and
unaligned leading dimensions, batches, pointer modes, scale modes, every epilogue incl. the bias gradients,
decode-like and split-K-like shapes, grids of several rounds of workgroups, with and without a workspace -- each through the planner's choice and
then through up to three other tile variants of the family it chose, all against the CPU oracle.  The draw
is deterministic (fixed seed), so a failure names a case that can be rerun."""
import json

import numpy as np
import pytest

from oracle.cases import Case
from zluda_amd import abi as K, cublaslt

pytestmark = pytest.mark.gpu
BIG = True   # include shapes of several tiles of the large variants
NVAR = {K.ZLUDA_KERNEL_MFMA_I8: 12, K.ZLUDA_KERNEL_MFMA_F8: 12, K.ZLUDA_KERNEL_MFMA_MXF4: 12, K.ZLUDA_KERNEL_MFMA_TR8: 4,
        K.ZLUDA_KERNEL_DECODE_W8A8: 21, K.ZLUDA_KERNEL_MFMA_H16: 12, K.ZLUDA_KERNEL_MFMA_TR16: 4}
RNG = None


EPIS = [K.CUBLASLT_EPILOGUE_DEFAULT, K.CUBLASLT_EPILOGUE_RELU, K.CUBLASLT_EPILOGUE_GELU, K.CUBLASLT_EPILOGUE_BIAS,
        K.CUBLASLT_EPILOGUE_RELU_BIAS, K.CUBLASLT_EPILOGUE_GELU_BIAS, K.CUBLASLT_EPILOGUE_BGRADA, K.CUBLASLT_EPILOGUE_BGRADB]


def pick(xs):
    return xs[int(RNG.integers(len(xs)))]


def dims():
    r = RNG.random()
    if r < 0.2:   # decode-like
        return int(RNG.integers(16, 3000)), int(RNG.integers(1, 49)), pick([1024, 2048, 2560, 3072, 3584, 4096, 960, 1536, 5120, 272, 8192, 11008, 13824])
    if r < 0.4:   # few tiles, long K (split-K)
        return int(RNG.integers(1, 200)), int(RNG.integers(1, 200)), pick([2048, 4096, 6144, 8192, 3000, 4112])
    if r < 0.5:
        return pick([256, 320, 512, 640]), pick([256, 384, 512]), pick([256, 512, 768, 1024])
    if r < 0.75 and BIG:
        return int(RNG.integers(200, 1500)), int(RNG.integers(200, 1500)), int(RNG.integers(64, 1200))
    if r < 0.81 and BIG:   # more workgroups than CUs for most tile shapes: later workgroups follow another one on their CU
        return int(RNG.integers(2000, 5000)), int(RNG.integers(1500, 4500)), int(RNG.integers(32, 420))
    return int(RNG.integers(1, 400)), int(RNG.integers(1, 400)), int(RNG.integers(1, 700))


def make(only=None):
    fam = only or pick(["i8i", "i8f", "i8f", "f8", "f8", "mx", "fl"])
    m, n, k = dims()
    s = dict(m=m, n=n, k=k)
    s["transa"], s["transb"] = int(RNG.integers(2)), int(RNG.integers(2))
    if RNG.random() < 0.5: s["transa"], s["transb"] = 1, 0
    for t in "abcd":
        if RNG.random() < 0.25: s["order_" + t] = 1
    if fam == "i8i":
        s.update(a_type=K.CUDA_R_8I, b_type=K.CUDA_R_8I, d_type=K.CUDA_R_32I, compute_type=K.CUBLAS_COMPUTE_32I, scale_type=K.CUDA_R_32I)
        if RNG.random() < 0.4: s["with_c"] = True
    elif fam == "i8f":
        s.update(a_type=K.CUDA_R_8I, b_type=K.CUDA_R_8I, d_type=pick([K.CUDA_R_16BF, K.CUDA_R_16F, K.CUDA_R_32F, K.CUDA_R_8I, K.CUDA_R_32I]),
                 compute_type=K.CUBLAS_COMPUTE_32I, scale_type=K.CUDA_R_32F, alpha_range=(0.001, 0.002))
    elif fam == "f8":
        at, bt = pick([(K.CUDA_R_8F_E4M3, K.CUDA_R_8F_E4M3), (K.CUDA_R_8F_E5M2, K.CUDA_R_8F_E4M3), (K.CUDA_R_8F_E4M3, K.CUDA_R_8F_E5M2)])
        s.update(a_type=at, b_type=bt, d_type=pick([K.CUDA_R_16BF, K.CUDA_R_16F, K.CUDA_R_32F, K.CUDA_R_8F_E4M3]), compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F)
    elif fam == "mx":
        k = max(32, k // 32 * 32)
        if RNG.random() < 0.6: k = max(256, k // 256 * 256)
        s.update(k=k, transa=1, transb=0, a_type=K.CUDA_R_4F_E2M1, b_type=K.CUDA_R_4F_E2M1, d_type=pick([K.CUDA_R_16BF, K.CUDA_R_32F]),
                 compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F, a_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0,
                 b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0)
        s.pop("order_a", None); s.pop("order_b", None)
    elif fam == "h16":   # the 16-bit operand types at full size: their MFMA, transposing and decode kernels
        t = pick([K.CUDA_R_16BF, K.CUDA_R_16F])
        s.update(a_type=t, b_type=t, d_type=pick([t, t, K.CUDA_R_32F, K.CUDA_R_16BF]), compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F,
                 alpha_range=(0.02, 0.05))
    else:
        t = pick([K.CUDA_R_16BF, K.CUDA_R_16F, K.CUDA_R_32F])
        s.update(a_type=t, b_type=t, d_type=pick([t, K.CUDA_R_32F]), compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F)
        s["m"], s["n"], s["k"] = min(m, 300), min(n, 300), min(s["k"], 600)
    m, n, k = s["m"], s["n"], s["k"]
    ta, tb = s["transa"], s["transb"]
    # leading dimensions: sometimes padded
    def ld(tag, rows, cols, mult):
        order = s.get("order_" + tag, 0)
        base = rows if order == 0 else cols
        r = RNG.random()
        if r < 0.5: return
        pad = int(RNG.integers(1, 40)) if r < 0.6 else (16 * int(RNG.integers(1, 4)) if r < 0.9 else 4 * int(RNG.integers(1, 9)))
        if mode16: pad = (pad + 15) // 16 * 16; v16 = (base + 15) // 16 * 16 - base; pad += v16
        v = base + pad
        if mult > 1: v = (v + mult - 1) // mult * mult
        s["ld" + tag] = v
    mult = 2 if fam == "mx" else 1
    mode16 = RNG.random() < 0.6
    if mode16 and fam != "fl":   # K-contiguous operands need K % 16 == 0 for the MFMA kernels
        s["k"] = k = max(16, k // 16 * 16) if fam != "mx" else k
    ld("a", k if ta else m, m if ta else k, mult); ld("b", n if tb else k, k if tb else n, mult)
    ld("c", m, n, 1); ld("d", m, n, 1)
    if RNG.random() < 0.25:
        s["batch"] = int(RNG.integers(2, 4))
    if fam != "i8i":
        if RNG.random() < 0.4: s["with_c"] = True
        epi = pick(EPIS)
        if fam == "mx" and epi in (K.CUBLASLT_EPILOGUE_BGRADA, K.CUBLASLT_EPILOGUE_BGRADB): epi = K.CUBLASLT_EPILOGUE_GELU_BIAS
        s["epilogue"] = epi
        if epi != K.CUBLASLT_EPILOGUE_DEFAULT and RNG.random() < 0.5:
            s["bias_type"] = pick([K.CUDA_R_32F, K.CUDA_R_16BF, K.CUDA_R_16F])
        bg = epi in (K.CUBLASLT_EPILOGUE_BGRADA, K.CUBLASLT_EPILOGUE_BGRADB)
        if s.get("batch", 1) > 1 and epi not in (K.CUBLASLT_EPILOGUE_DEFAULT, K.CUBLASLT_EPILOGUE_RELU, K.CUBLASLT_EPILOGUE_GELU) and RNG.random() < 0.5:
            s["bias_batch_stride"] = max(m, n) + int(RNG.integers(0, 9))
        pm = pick([K.CUBLASLT_POINTER_MODE_HOST] * 3 + [K.CUBLASLT_POINTER_MODE_DEVICE, K.CUBLASLT_POINTER_MODE_DEVICE_VECTOR,
                  K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO, K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_HOST])
        s["pointer_mode"] = pm
        if pm == K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO: s.pop("with_c", None)
        if pm in (K.CUBLASLT_POINTER_MODE_DEVICE, K.CUBLASLT_POINTER_MODE_DEVICE_VECTOR): s["with_c"] = True
        if bg and s.get("batch", 1) > 1: s["bias_batch_stride"] = max(m, n) + int(RNG.integers(0, 9))
        if fam in ("i8f", "f8") and not bg:
            r = RNG.random()
            if r < 0.3: s["with_scalar_scales"] = True
            elif r < 0.5 and fam == "i8f": s["b_scale_mode"] = K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F
            elif r < 0.6 and fam == "i8f": s["a_scale_mode"] = K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F
            if RNG.random() < 0.2 and fam == "f8": s["with_cd_scales"] = True
    return fam, s


@pytest.mark.parametrize("chunk", list(range(6)) + ["h16a", "h16b"])
def test_random_problems_against_the_oracle(gpu_api, chunk):
    global RNG
    only = None
    if isinstance(chunk, str):   # the same draw restricted to f16 / bf16 operands
        only, chunk = "h16", 6 + "ab".index(chunk[-1])
    RNG = np.random.default_rng(4200 + chunk)
    ran = 0
    for it in range(40):
        fam, spec = make(only)
        seed = 420000 + chunk * 1000 + it
        ws = pick([0, 0, 1 << 24])
        forced = pick([None, None, None, K.ZLUDA_KERNEL_GENERIC])
        print("case", chunk, it, "seed", seed, "workspace", ws, "forced family", forced, json.dumps(spec), flush=True)
        case = Case(spec, seed)
        ref = case.run_oracle()
        try:
            st, got, kern, var = case.run_gpu(gpu_api, forced_kernel=forced, workspace_bytes=ws)
        except cublaslt.CublasLtError as e:   # a combination the API refuses when the descriptors are built
            print("  refused:", e, flush=True)
            continue
        assert st == 0, "cublasLtMatmul status %d" % st
        ran += 1
        # one e4m3 step is 2^-3 of the value; int32 outputs of float-scaled problems may sit on a rounding boundary
        tol = 0.13 if spec["d_type"] == K.CUDA_R_8F_E4M3 else None
        check(case, spec, got, ref, tol)
        if case.bgrad:
            ints = spec["a_type"] == K.CUDA_R_8I and case.bgrad_type == K.CUDA_R_32F
            case.compare_bgrad(case.bgrad_got, case.bgrad_ref, exact=ints)
        if kern in NVAR and forced is None:
            for fv in RNG.permutation(NVAR[kern])[:3]:
                st, got, _, _ = case.run_gpu(gpu_api, forced_kernel=kern, forced_variant=int(fv), workspace_bytes=ws)
                print("  forced variant", int(fv), "status", st, flush=True)
                if st == 0:
                    check(case, spec, got, ref, tol)
    assert ran >= 30


def check(case, spec, got, ref, tol):
    if spec["d_type"] == K.CUDA_R_32I and spec["scale_type"] == K.CUDA_R_32F:
        # float epilogue rounded to int32: association differences may move a value across a .5 boundary
        idx = case.logical_index().ravel()
        assert np.max(np.abs(got[idx].astype(np.int64) - ref[idx].astype(np.int64))) <= 1
        return
    case.compare(got, ref, tol=tol)
