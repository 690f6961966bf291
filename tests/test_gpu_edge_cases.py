"""Edge cases of cublasLtMatmul through the planner's own choice (no forced kernel): degenerate and
ragged shapes, long K, many batches, in-place C == D, device-side scalars, error returns on a live
device.  Same bars as tests/test_gpu_parity.py."""
import ctypes as C

import numpy as np
import pytest

from oracle.cases import Case
from zluda_amd import abi
from zluda_amd.cublaslt import MatmulCall

pytestmark = pytest.mark.gpu
K = abi

I8 = dict(a_type=K.CUDA_R_8I, b_type=K.CUDA_R_8I, c_type=K.CUDA_R_32I, d_type=K.CUDA_R_32I,
          compute_type=K.CUBLAS_COMPUTE_32I, scale_type=K.CUDA_R_32I, transa=1)
F8 = dict(a_type=K.CUDA_R_8F_E4M3, b_type=K.CUDA_R_8F_E4M3, c_type=K.CUDA_R_16BF, d_type=K.CUDA_R_16BF,
          compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F, transa=1)
MX = dict(a_type=K.CUDA_R_4F_E2M1, b_type=K.CUDA_R_4F_E2M1, c_type=K.CUDA_R_16BF, d_type=K.CUDA_R_16BF,
          compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F, transa=1,
          a_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0, b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0)


def run(gpu_api, spec, seed, **kw):
    print("edge case", spec, flush=True)
    case = Case(spec, seed, **kw)
    ref = case.run_oracle()
    st, got, kern, variant = case.run_gpu(gpu_api)
    assert st == 0, "cublasLtMatmul status %d" % st
    case.compare(got, ref)
    return kern


@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (1, 1, 16), (1, 37, 5), (37, 1, 48), (3, 5, 7), (17, 33, 129), (255, 257, 16)])
def test_tiny_and_odd_int8_shapes(gpu_api, m, n, k):
    run(gpu_api, dict(I8, m=m, n=n, k=k), 300 + m)


@pytest.mark.parametrize("m,n,k", [(257, 255, 4112), (512, 256, 32768), (256, 512, 16)])
def test_int8_ragged_tiles_long_and_short_k(gpu_api, m, n, k):
    """partial tiles on both edges; K = 32768 (256 stages; |sum| <= 2^29, no overflow); K = one chunk"""
    assert run(gpu_api, dict(I8, m=m, n=n, k=k), 310) == K.ZLUDA_KERNEL_MFMA_I8


def test_int8_many_small_batches(gpu_api):
    run(gpu_api, dict(I8, m=64, n=48, k=80, batch=33, with_c=True), 320)


def test_fp8_and_mxfp4_ragged(gpu_api):
    assert run(gpu_api, dict(F8, m=300, n=130, k=464, epilogue=K.CUBLASLT_EPILOGUE_RELU_BIAS, with_c=True), 330) == K.ZLUDA_KERNEL_MFMA_F8
    # K = 256 * odd: scale rows of 8 * odd bytes (chunks run across row boundaries)
    assert run(gpu_api, dict(MX, m=130, n=300, k=1280, batch=3), 331) == K.ZLUDA_KERNEL_MFMA_MXF4
    assert run(gpu_api, dict(MX, m=256, n=256, k=256), 332) == K.ZLUDA_KERNEL_MFMA_MXF4
    # K not a multiple of 256: outside the MFMA family's contract, served by the generic kernel
    assert run(gpu_api, dict(MX, m=64, n=64, k=96), 333) == K.ZLUDA_KERNEL_GENERIC


def test_decode_shapes_around_the_limits(gpu_api):
    dec = dict(I8, c_type=K.CUDA_R_16BF, d_type=K.CUDA_R_16BF, scale_type=K.CUDA_R_32F, alpha_range=(0.001, 0.01))
    assert run(gpu_api, dict(dec, m=64, n=1, k=4096), 340, int_dist="normal") == K.ZLUDA_KERNEL_DECODE_W8A8
    assert run(gpu_api, dict(dec, m=4099, n=32, k=4096), 341, int_dist="normal") == K.ZLUDA_KERNEL_DECODE_W8A8   # rows % 4 != 0
    assert run(gpu_api, dict(dec, m=2048, n=3, k=11008), 342, int_dist="normal") == K.ZLUDA_KERNEL_DECODE_W8A8  # K under the 12288 cover
    assert run(gpu_api, dict(dec, m=512, n=16, k=4096, batch=3), 343, int_dist="normal") == K.ZLUDA_KERNEL_DECODE_W8A8
    # beyond 48 tokens the planner prefers small MFMA tiles (the decode family itself runs up to 64)
    assert run(gpu_api, dict(dec, m=2048, n=32, k=4096), 344, int_dist="normal") == K.ZLUDA_KERNEL_DECODE_W8A8
    assert run(gpu_api, dict(dec, m=2048, n=33, k=4096), 346, int_dist="normal") == K.ZLUDA_KERNEL_DECODE_W8A8
    assert run(gpu_api, dict(dec, m=2048, n=48, k=4096), 348, int_dist="normal") == K.ZLUDA_KERNEL_DECODE_W8A8
    assert run(gpu_api, dict(dec, m=2048, n=49, k=4096), 349, int_dist="normal") == K.ZLUDA_KERNEL_MFMA_I8
    assert run(gpu_api, dict(dec, m=2048, n=64, k=4096), 347, int_dist="normal") == K.ZLUDA_KERNEL_MFMA_I8
    # f16 output, ld > rows (the packed store needs ld % 4 == 0: 2052 qualifies, 2051 does not)
    for ld in (2052, 2051):
        run(gpu_api, dict(dec, c_type=K.CUDA_R_16F, d_type=K.CUDA_R_16F, m=2048, n=8, k=4096, ldd=ld, ldc=ld), 345, int_dist="normal")


def test_decode_k_between_the_stream_instantiations(gpu_api):
    """K values between the covers of the LDS-streaming decode kernel's instantiations run on the next larger one
    with the lanes past the end of K reading zero (whole 256-byte units past it are never multiplied), with the full
    decode epilogue: alpha vector, per-token scale, bias.  K outside every cover, or more activation fragments than
    the registers hold: MFMA tiles when they fill at least half of the CUs (with the K split through the workspace
    if there is one), the register-streaming decode kernel otherwise."""
    dec = dict(I8, c_type=K.CUDA_R_16BF, d_type=K.CUDA_R_16BF, scale_type=K.CUDA_R_32F,
               pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO,
               b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F, epilogue=K.CUBLASLT_EPILOGUE_BIAS,
               bias_type=K.CUDA_R_32F, alpha_range=(0.001, 0.01), scale_range=(0.005, 0.02), bias_std=0.02)
    DEC = K.ZLUDA_KERNEL_DECODE_W8A8
    assert run(gpu_api, dict(dec, m=8192, n=16, k=2624), 350, int_dist="normal") == DEC      # 3072 cover: tail inside a unit
    assert run(gpu_api, dict(dec, m=2048, n=16, k=2560), 351, int_dist="normal") == DEC      # 3072 cover: two whole units missing
    assert run(gpu_api, dict(dec, m=1000, n=5, k=3584, lda=3584 + 64), 353, int_dist="normal") == DEC    # 4096 cover
    assert run(gpu_api, dict(dec, m=5120, n=16, k=13824), 354, int_dist="normal") == DEC     # 14336 cover
    assert run(gpu_api, dict(dec, m=2048, n=29, k=3584), 355, int_dist="normal") == DEC      # two token blocks
    f8 = dict(a_type=K.CUDA_R_8F_E4M3, b_type=K.CUDA_R_8F_E4M3, c_type=K.CUDA_R_16BF, d_type=K.CUDA_R_16BF,
              compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F, transa=1, epilogue=K.CUBLASLT_EPILOGUE_BIAS,
              bias_type=K.CUDA_R_16BF, with_scalar_scales=True, scale_range=(0.05, 0.06))
    assert run(gpu_api, dict(f8, m=4096, n=16, k=11008), 356) == DEC                           # fp8, 12288 cover
    assert run(gpu_api, dict(f8, m=1000, n=7, k=2736), 357) == DEC                             # fp8, tail inside a 128-byte step
    spec = dict(dec, m=4096, n=32, k=11008)      # two token blocks x 24 steps: more fragments than the registers hold
    print("edge case", spec, "with a 64 MiB workspace", flush=True)
    case = Case(spec, 352, int_dist="normal")
    ref = case.run_oracle()
    st, got, kern, variant = case.run_gpu(gpu_api, workspace_bytes=64 << 20)
    assert st == 0 and kern == K.ZLUDA_KERNEL_MFMA_I8 and case.last_workspace_needed > 0
    case.compare(got, ref)
    st, got, kern, variant = case.run_gpu(gpu_api)          # no workspace: 64 tiles only, decode family
    assert st == 0 and kern == K.ZLUDA_KERNEL_DECODE_W8A8
    case.compare(got, ref)


def test_in_place_c_equals_d_and_device_scalars(gpu_api):
    """C == D with beta != 0 (allowed: ext/hipblaslt-sys/src/lib.rs:1166-1177), alpha/beta read from device memory"""
    import torch
    spec = dict(I8, m=384, n=256, k=512, with_c=True, pointer_mode=K.CUBLASLT_POINTER_MODE_DEVICE)
    case = Case(spec, 350)
    ref = case.run_oracle()
    keep, ptr, dt = case.upload()
    # start D as a copy of C and pass the same pointer for both
    nbytes = case.Cm.nbytes
    d_t = torch.frombuffer(bytearray(case.Cm.tobytes()), dtype=torch.uint8).cuda()
    call = MatmulCall(gpu_api, spec)
    alpha, beta = case.scalars(ptr)
    st = call.run(alpha, ptr["A"], ptr["B"], beta, d_t.data_ptr(), d_t.data_ptr(), None, 0, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    call.close()
    assert st == 0
    got = np.frombuffer(d_t.cpu().numpy().tobytes(), dtype=np.int32)
    assert nbytes == got.nbytes
    assert np.array_equal(got, ref)


def test_error_returns_with_a_live_device(gpu_api):
    import torch
    spec = dict(I8, m=256, n=256, k=256)
    call = MatmulCall(gpu_api, spec)
    a = torch.zeros(256 * 256, dtype=torch.int8, device="cuda:0")
    d = torch.zeros(256 * 256, dtype=torch.int32, device="cuda:0")
    one, zero = C.c_int32(1), C.c_int32(0)
    stream = torch.cuda.current_stream().cuda_stream
    assert call.run(one, a.data_ptr(), a.data_ptr(), zero, None, d.data_ptr(), None, 0, stream) == 0
    assert call.run(one, None, a.data_ptr(), zero, None, d.data_ptr(), None, 0, stream) == K.CUBLAS_STATUS_INVALID_VALUE
    assert call.run(None, a.data_ptr(), a.data_ptr(), zero, None, d.data_ptr(), None, 0, stream) == K.CUBLAS_STATUS_INVALID_VALUE
    two = C.c_int32(2)   # beta != 0 without C
    assert call.run(one, a.data_ptr(), a.data_ptr(), two, None, None, None, 0, stream) == K.CUBLAS_STATUS_INVALID_VALUE
    # a foreign algo token
    junk = abi.cublasLtMatmulAlgo_t()
    junk.data[0] = 0x1234
    call.algo = junk
    assert call.run(one, a.data_ptr(), a.data_ptr(), zero, None, d.data_ptr(), None, 0, stream) == K.CUBLAS_STATUS_INVALID_VALUE
    call.close()
    torch.cuda.synchronize()


@pytest.mark.parametrize("ta,tb", [(1, 0), (0, 0), (0, 1)])
def test_gemm_ex_entry_points(gpu_api, ta, tb):
    """cublasGemmEx / cublasGemmStridedBatchedEx semantics (C in/out, host scalars) on the same kernels:
    int8 -> int32 with beta != 0, batched with strides and padding; fp8 -> bf16"""
    import torch
    stream = torch.cuda.current_stream().cuda_stream
    for spec, seed in ((dict(I8, transa=ta, transb=tb, m=320, n=192, k=256, with_c=True, ldc=336, ldd=336), 360),
                       (dict(I8, transa=ta, transb=tb, m=96, n=80, k=144, with_c=True, batch=5), 361),
                       (dict(F8, transa=ta, transb=tb, m=256, n=128, k=384, with_c=True, alpha=1.0), 362)):
        print("gemm_ex case", spec, flush=True)
        case = Case(spec, seed)
        ref = case.run_oracle()
        keep, ptr, dt = case.upload()
        c_t = torch.frombuffer(bytearray(case.Cm.tobytes()), dtype=torch.uint8).cuda()   # C is overwritten
        m, n, k, batch = spec["m"], spec["n"], spec["k"], spec.get("batch", 1)
        lda = spec.get("lda", k if ta else m)
        ldb = spec.get("ldb", n if tb else k)
        ldc = spec.get("ldc", m)
        int_scale = spec["scale_type"] == K.CUDA_R_32I
        ct = C.c_int32 if int_scale else C.c_float
        alpha, beta = ct(case.alpha[0].item()), ct(case.beta[0].item())
        if batch == 1:
            st = gpu_api.zluda_gemm_ex(ta, tb, m, n, k, C.addressof(alpha), ptr["A"], spec["a_type"], lda, ptr["B"],
                                       spec["b_type"], ldb, C.addressof(beta), c_t.data_ptr(), spec["c_type"], ldc,
                                       spec["compute_type"], stream)
        else:
            st = gpu_api.zluda_gemm_strided_batched_ex(ta, tb, m, n, k, C.addressof(alpha), ptr["A"], spec["a_type"], lda,
                                                       lda * (m if ta else k), ptr["B"], spec["b_type"], ldb,
                                                       ldb * (k if tb else n), C.addressof(beta), c_t.data_ptr(),
                                                       spec["c_type"], ldc, ldc * n, batch, spec["compute_type"], stream)
        torch.cuda.synchronize()
        assert st == 0, "status %d" % st
        got = np.frombuffer(c_t.cpu().numpy().tobytes(), dtype=case.d_np)
        c0 = np.frombuffer(case.Cm.tobytes(), dtype=case.d_np)
        idx = case.logical_index().ravel()
        pad = np.ones(got.size, bool)
        pad[idx] = False
        assert np.array_equal(got[pad], c0[pad]), "padding of C between rows and ld was overwritten"
        merged = ref.copy()          # the oracle's D storage carries its own padding pattern
        merged[idx] = got[idx]
        case.compare(merged, ref)
    # degenerate sizes
    one = C.c_int32(1)
    assert gpu_api.zluda_gemm_ex(0, 0, 0, 4, 4, C.addressof(one), None, K.CUDA_R_8I, 1, None, K.CUDA_R_8I, 4,
                                 C.addressof(one), None, K.CUDA_R_32I, 1, K.CUBLAS_COMPUTE_32I, stream) == 0
    assert gpu_api.zluda_gemm_ex(0, 0, -1, 4, 4, C.addressof(one), None, K.CUDA_R_8I, 1, None, K.CUDA_R_8I, 4,
                                 C.addressof(one), None, K.CUDA_R_32I, 1, K.CUBLAS_COMPUTE_32I, stream) == K.CUBLAS_STATUS_INVALID_VALUE


def test_split_k_through_the_workspace(gpu_api):
    """few tiles, long K: with a workspace the planner splits K (partial tiles + reduce kernel);
    int8 stays bit-exact, the float epilogues keep their tolerance, every layout/epilogue feature
    goes through the second kernel"""
    ws = 64 << 20
    for spec, seed in ((dict(I8, m=1024, n=256, k=8192), 370),
                       (dict(I8, m=300, n=200, k=8208, with_c=True, batch=2, ldd=304, ldc=320), 371),
                       (dict(I8, transa=0, transb=1, order_a=1, order_b=1, order_c=1, order_d=1, m=192, n=320, k=8192, with_c=True), 372),
                       (dict(I8, c_type=K.CUDA_R_16BF, d_type=K.CUDA_R_16BF, scale_type=K.CUDA_R_32F, m=512, n=128, k=6144,
                             epilogue=K.CUBLASLT_EPILOGUE_RELU_BIAS, bias_type=K.CUDA_R_32F,
                             pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO,
                             b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F, alpha_range=(0.001, 0.002)), 373),
                       (dict(F8, m=640, n=256, k=8192, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS, with_scalar_scales=True,
                             scale_range=(0.02, 0.03)), 374)):
        print("split-K case", spec, flush=True)
        case = Case(spec, seed)
        ref = case.run_oracle()
        st, got, kern, variant = case.run_gpu(gpu_api, workspace_bytes=ws)
        assert st == 0 and kern in (K.ZLUDA_KERNEL_MFMA_I8, K.ZLUDA_KERNEL_MFMA_F8)
        assert case.last_workspace_needed and case.last_workspace_needed <= ws, "the planner did not split K"
        case.compare(got, ref)
    # MXFP4: the K shares are whole scale chunks (1024 elements); 8960 = 35 stages in 4 shares -> 12 + 12 + 11 + 0
    for spec, seed in ((dict(MX, m=512, n=64, k=8192), 376), (dict(MX, m=320, n=48, k=8960, batch=2), 377),
                       (dict(MX, m=1024, n=256, k=16384), 378)):
        print("split-K case", spec, flush=True)
        case = Case(spec, seed)
        ref = case.run_oracle()
        st, got, kern, variant = case.run_gpu(gpu_api, workspace_bytes=ws)
        assert st == 0 and kern == K.ZLUDA_KERNEL_MFMA_MXF4
        assert case.last_workspace_needed and case.last_workspace_needed <= ws, "the planner did not split K"
        case.compare(got, ref)
    # the same token with too little workspace at call time: the call must not use it
    case = Case(dict(I8, m=1024, n=256, k=8192), 375)
    ref = case.run_oracle()
    st, got, kern, variant = case.run_gpu(gpu_api, workspace_bytes=0)
    assert st == 0 and case.last_workspace_needed == 0
    case.compare(got, ref)
