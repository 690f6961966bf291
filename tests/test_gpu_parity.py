"""GPU parity: every kernel family and tile variant, through the exported C ABI, against the CPU
oracle on the same seeded inputs.  Integer outputs must be bit-exact (whole D storage including the
padding between rows and ld); float outputs within max |rel err| <= 1e-2 (bf16 output, fp32
accumulate) with the documented floor of 1e-2 * rms(ref)."""
import sys

import numpy as np
import pytest

from oracle.cases import Case
from zluda_amd import abi

pytestmark = pytest.mark.gpu
K = abi

I8 = dict(a_type=K.CUDA_R_8I, b_type=K.CUDA_R_8I, d_type=K.CUDA_R_32I, compute_type=K.CUBLAS_COMPUTE_32I,
          scale_type=K.CUDA_R_32I, transa=1)
I8F = dict(I8, d_type=K.CUDA_R_16BF, scale_type=K.CUDA_R_32F)
F8 = dict(a_type=K.CUDA_R_8F_E4M3, b_type=K.CUDA_R_8F_E4M3, d_type=K.CUDA_R_16BF, compute_type=K.CUBLAS_COMPUTE_32F,
          scale_type=K.CUDA_R_32F, transa=1)
MX = dict(a_type=K.CUDA_R_4F_E2M1, b_type=K.CUDA_R_4F_E2M1, d_type=K.CUDA_R_16BF, compute_type=K.CUBLAS_COMPUTE_32F,
          scale_type=K.CUDA_R_32F, transa=1, a_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0,
          b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0)
DECODE = dict(I8F, pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO,
              b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F, epilogue=K.CUBLASLT_EPILOGUE_BIAS,
              bias_type=K.CUDA_R_32F, alpha_range=(0.001, 0.01), scale_range=(0.005, 0.02), bias_std=0.02)


def check(gpu_api, spec, seed, kernel=None, variant=-1, expect_kernel=None, tol=None, **case_kw):
    print("case", spec, "seed", seed, "kernel", kernel, "variant", variant, flush=True)
    case = Case(spec, seed, **case_kw)
    ref = case.run_oracle()
    st, got, k, v = case.run_gpu(gpu_api, forced_kernel=kernel, forced_variant=variant)
    assert st == 0, "cublasLtMatmul status %d" % st
    if expect_kernel is not None:
        assert k == expect_kernel, "planner chose kernel %d" % k
    return case.compare(got, ref, tol)


# ---- int8 -> int32 MFMA, every tile variant --------------------------------
@pytest.mark.parametrize("variant", range(12))
@pytest.mark.parametrize("m,n,k", [(256, 256, 128), (300, 200, 144), (512, 384, 1024)])
def test_mfma_i8_variants(gpu_api, variant, m, n, k):
    check(gpu_api, dict(I8, m=m, n=n, k=k, lda=k + 16 if k == 144 else k), 10 + variant, K.ZLUDA_KERNEL_MFMA_I8, variant)


def test_mfma_i8_alpha_beta_batch_and_padding(gpu_api):
    spec = dict(I8, m=200, n=136, k=272, batch=3, with_c=True, ldd=208, ldc=204, lda=288, stride_d=208 * 136 + 48)
    for variant in (0, 1, 4, 6, 8, 9, 10, 11):
        check(gpu_api, spec, 3, K.ZLUDA_KERNEL_MFMA_I8, variant)
    # device scalars
    check(gpu_api, dict(spec, pointer_mode=K.CUBLASLT_POINTER_MODE_DEVICE), 4, K.ZLUDA_KERNEL_MFMA_I8, 1)


def test_mfma_i8_row_major_output_swaps(gpu_api):
    spec = dict(I8, transa=0, transb=1, order_a=1, order_b=1, order_c=1, order_d=1, m=192, n=320, k=256, with_c=True)
    check(gpu_api, spec, 5, K.ZLUDA_KERNEL_MFMA_I8, 1)
    check(gpu_api, spec, 5, K.ZLUDA_KERNEL_MFMA_I8, 4)
    check(gpu_api, spec, 5, K.ZLUDA_KERNEL_MFMA_I8, 8)
    check(gpu_api, spec, 5, K.ZLUDA_KERNEL_MFMA_I8, 11)


# full tiles take the register-direct / vectorised epilogues; cover each of them per tile shape
@pytest.mark.parametrize("variant", range(12))
def test_mfma_full_tile_epilogues(gpu_api, variant):
    full = dict(m=512, n=256, k=384)
    check(gpu_api, dict(I8, **full, alpha=1), 110, K.ZLUDA_KERNEL_MFMA_I8, variant)
    check(gpu_api, dict(I8, **full, alpha=3, ldd=528), 111, K.ZLUDA_KERNEL_MFMA_I8, variant)
    check(gpu_api, dict(I8, transa=0, transb=1, order_a=1, order_b=1, order_c=1, order_d=1, **full), 112,
          K.ZLUDA_KERNEL_MFMA_I8, variant)
    vec = dict(I8F, **full, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS, bias_type=K.CUDA_R_32F,
               pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO,
               a_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F,
               b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F,
               alpha_range=(0.001, 0.002), scale_range=(0.5, 1.5))
    for dt in (K.CUDA_R_16BF, K.CUDA_R_16F, K.CUDA_R_32F):
        check(gpu_api, dict(vec, d_type=dt, c_type=dt), 113, K.ZLUDA_KERNEL_MFMA_I8, variant)
        check(gpu_api, dict(vec, d_type=dt, c_type=dt, order_c=1, order_d=1, epilogue=K.CUBLASLT_EPILOGUE_RELU_BIAS), 114,
              K.ZLUDA_KERNEL_MFMA_I8, variant)
    check(gpu_api, dict(F8, **full, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS, with_scalar_scales=True), 115,
          K.ZLUDA_KERNEL_MFMA_F8, variant)
    if variant < 8:   # (variants 8 .., the 16x16 MFMA shapes, serve int8 and fp8)
        check(gpu_api, dict(MX, m=512, n=256, k=1024), 116, K.ZLUDA_KERNEL_MFMA_MXF4, variant)


@pytest.mark.parametrize("variant", range(12))
def test_mfma_ragged_token_count_keeps_the_fast_epilogues(gpu_api, variant):
    """M a multiple of every tile height, N ragged (tokens): the stores of the columns past the end fall
    outside the buffer window; padding, the next batch and the canary behind D must stay untouched"""
    rag = dict(m=768, n=203, k=256)
    check(gpu_api, dict(I8, **rag, alpha=1, batch=2, ldd=784), 410, K.ZLUDA_KERNEL_MFMA_I8, variant)
    vec = dict(I8F, **rag, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS, bias_type=K.CUDA_R_32F,
               pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO,
               a_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F,
               b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F,
               alpha_range=(0.001, 0.002), scale_range=(0.5, 1.5))
    for dt in (K.CUDA_R_16BF, K.CUDA_R_32F):
        check(gpu_api, dict(vec, d_type=dt, c_type=dt, batch=2), 411, K.ZLUDA_KERNEL_MFMA_I8, variant)
    check(gpu_api, dict(F8, **rag, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS, with_scalar_scales=True, batch=2), 412,
          K.ZLUDA_KERNEL_MFMA_F8, variant)
    # row-major D: the ragged dimension is M
    check(gpu_api, dict(F8, m=203, n=768, k=256, order_c=1, order_d=1, d_type=K.CUDA_R_16F, c_type=K.CUDA_R_16F), 413,
          K.ZLUDA_KERNEL_MFMA_F8, variant)


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 11])
def test_mfma_i8_float_epilogue(gpu_api, variant):
    spec = dict(I8F, m=260, n=140, k=512, epilogue=K.CUBLASLT_EPILOGUE_RELU_BIAS, bias_type=K.CUDA_R_32F,
                pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_HOST, with_c=True,
                a_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F,
                b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F,
                alpha_range=(0.001, 0.002), scale_range=(0.5, 1.5))
    check(gpu_api, spec, 6, K.ZLUDA_KERNEL_MFMA_I8, variant)
    # same with a row-major D (per-row vectors then run along the accumulator registers)
    check(gpu_api, dict(spec, order_c=1, order_d=1), 7, K.ZLUDA_KERNEL_MFMA_I8, variant)
    for dt in (K.CUDA_R_32F, K.CUDA_R_16F, K.CUDA_R_8I):
        check(gpu_api, dict(spec, d_type=dt, c_type=dt, alpha_range=(0.0001, 0.0002)), 8, K.ZLUDA_KERNEL_MFMA_I8, variant)


# ---- fp8 -------------------------------------------------------------------------------------------
@pytest.mark.parametrize("variant", range(12))
def test_mfma_f8_variants(gpu_api, variant):
    check(gpu_api, dict(F8, m=256, n=256, k=256), 20 + variant, K.ZLUDA_KERNEL_MFMA_F8, variant)
    check(gpu_api, dict(F8, m=320, n=272, k=400, lda=416, ldb=400, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS,
                        with_scalar_scales=True), 30 + variant, K.ZLUDA_KERNEL_MFMA_F8, variant)


@pytest.mark.parametrize("at,bt", [(K.CUDA_R_8F_E5M2, K.CUDA_R_8F_E4M3), (K.CUDA_R_8F_E4M3, K.CUDA_R_8F_E5M2)])
def test_mfma_f8_mixed_formats(gpu_api, at, bt):
    for variant in (0, 1, 8):
        check(gpu_api, dict(F8, a_type=at, b_type=bt, m=256, n=128, k=512, d_type=K.CUDA_R_32F), 40, K.ZLUDA_KERNEL_MFMA_F8, variant)
    check(gpu_api, dict(F8, a_type=at, b_type=bt, m=256, n=128, k=512, order_c=1, order_d=1), 41, K.ZLUDA_KERNEL_MFMA_F8, 1)


def test_four_wave_kernel_stages_every_vector_its_epilogue_reads(gpu_api):
    """variant 11 keeps its epilogue free of loads from memory: the vectors along D's unit stride (alpha[], A's outer
    scales, the bias in each of its types; for a row-major D B's outer scales) reach it through LDS.  Each of them alone
    and together, several tiles per workgroup (the staging area is reused), batches with odd strides (a 16-bit bias
    that starts on an odd element), and D's scale folded in."""
    base = dict(F8, m=1024, n=512, k=640, with_scalar_scales=True)
    v11 = (K.ZLUDA_KERNEL_MFMA_F8, 11)
    for i, bt in enumerate((K.CUDA_R_16BF, K.CUDA_R_16F, K.CUDA_R_32F)):
        for epi in (K.CUBLASLT_EPILOGUE_BIAS, K.CUBLASLT_EPILOGUE_GELU_BIAS):
            check(gpu_api, dict(base, epilogue=epi, bias_type=bt), 900 + i, *v11)
        check(gpu_api, dict(base, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS, bias_type=bt, batch=3, bias_batch_stride=1031,
                            with_cd_scales=True), 910 + i, *v11)
    vec = dict(base, pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO, alpha_range=(0.5, 1.5),
               a_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F)
    check(gpu_api, vec, 920, *v11)
    check(gpu_api, dict(vec, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS, bias_type=K.CUDA_R_16BF, batch=2, bias_batch_stride=1025,
                        pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_HOST, alpha_vector_batch_stride=1029),
          921, *v11)
    check(gpu_api, dict(base, pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO, alpha_range=(0.5, 1.5)), 922, *v11)
    # row-major D: the unit stride runs along N, and the vector along it is B's
    check(gpu_api, dict(base, order_c=1, order_d=1, b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F), 923, *v11)
    # a tile row that is partial along M takes the element-wise path in the same launch
    check(gpu_api, dict(vec, m=1100, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS, bias_type=K.CUDA_R_16F), 924, *v11)
    # scale vectors across D's unit stride: B's outer scales (per token), alone and with everything along the other way,
    # a ragged token count (the staged vector ends inside the tile), batches; for a row-major D alpha[] and A's scales
    tok = dict(base, b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F)
    check(gpu_api, tok, 925, *v11)
    check(gpu_api, dict(vec, b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F, n=459, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS,
                        bias_type=K.CUDA_R_32F, batch=2), 926, *v11)
    check(gpu_api, dict(vec, order_c=1, order_d=1, m=512, n=1024), 927, *v11)
    check(gpu_api, dict(vec, order_c=1, order_d=1, m=203, n=768, b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F), 928, *v11)
    # the same epilogues behind int8 operands (W8A8 with float scaling -> bf16)
    w8 = dict(I8F, m=1024, n=512, k=640, pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO, alpha_range=(0.001, 0.002),
              b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F, scale_range=(0.5, 1.5))
    i11 = (K.ZLUDA_KERNEL_MFMA_I8, 11)
    check(gpu_api, w8, 930, *i11)
    check(gpu_api, dict(w8, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS, bias_type=K.CUDA_R_32F, n=300, batch=2), 931, *i11)
    check(gpu_api, dict(w8, epilogue=K.CUBLASLT_EPILOGUE_BIAS, bias_type=K.CUDA_R_16BF, a_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F), 932, *i11)
    check(gpu_api, dict(I8F, m=768, n=512, k=2048, alpha_range=(0.001, 0.002)), 933, *i11)
    # ReLU and f16 output are run-time choices of the same two epilogues; a negative scale of D turns the clip around
    for i, dt in enumerate((K.CUDA_R_16F, K.CUDA_R_16BF)):
        check(gpu_api, dict(base, d_type=dt, c_type=dt, epilogue=K.CUBLASLT_EPILOGUE_RELU_BIAS, bias_type=K.CUDA_R_32F, with_cd_scales=True), 940 + i, *v11)
        check(gpu_api, dict(w8, d_type=dt, c_type=dt, epilogue=K.CUBLASLT_EPILOGUE_RELU), 942 + i, *i11)
    check(gpu_api, dict(base, d_type=K.CUDA_R_16F, c_type=K.CUDA_R_16F, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS, bias_type=K.CUDA_R_16F), 944, *v11)
    check(gpu_api, dict(vec, d_type=K.CUDA_R_16F, c_type=K.CUDA_R_16F), 945, *v11)
    check(gpu_api, dict(MX, m=512, n=512, k=2048, d_type=K.CUDA_R_16F, c_type=K.CUDA_R_16F, epilogue=K.CUBLASLT_EPILOGUE_RELU), 946, K.ZLUDA_KERNEL_MFMA_MXF4, 11)
    # f32 output: 16 bytes per lane straight from its four rows
    check(gpu_api, dict(vec, d_type=K.CUDA_R_32F, c_type=K.CUDA_R_32F, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS, bias_type=K.CUDA_R_32F, n=459), 947, *v11)
    check(gpu_api, dict(w8, d_type=K.CUDA_R_32F, c_type=K.CUDA_R_32F, epilogue=K.CUBLASLT_EPILOGUE_RELU, batch=2), 948, *i11)
    check(gpu_api, dict(MX, m=512, n=512, k=2048, d_type=K.CUDA_R_32F, c_type=K.CUDA_R_32F), 949, K.ZLUDA_KERNEL_MFMA_MXF4, 11)
    # either fp8 operand may be E5M2 (not both), whichever way D lies
    for i, (at, bt) in enumerate(((K.CUDA_R_8F_E5M2, K.CUDA_R_8F_E4M3), (K.CUDA_R_8F_E4M3, K.CUDA_R_8F_E5M2))):
        check(gpu_api, dict(base, a_type=at, b_type=bt, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS), 950 + i, *v11)
        check(gpu_api, dict(base, a_type=at, b_type=bt, order_c=1, order_d=1, m=512, n=768), 952 + i, *v11)


def test_four_wave_kernel_mxfp4(gpu_api):
    """variant 11 for MXFP4: scale chunks of four stages prefetched through two LDS buffers across tile boundaries.  One,
    two, three and five chunks per tile (odd counts flip the buffer a tile's first chunk lands in), grids of fewer
    workgroups than tiles, batches, a row-major D, GELU; tiles that are partial along M take the element-wise epilogue
    and restart the stream.  FP4 products and their fp32 sums of this size are exact: the results match the oracle's
    bf16 outputs bit for bit."""
    v11 = K.ZLUDA_KERNEL_MFMA_MXF4
    for i, (shape, grid) in enumerate([(dict(m=256, n=256, k=1024), None), (dict(m=512, n=256, k=2048), None),
                                       (dict(m=512, n=512, k=3072), 1), (dict(m=1024, n=768, k=2048), 3),
                                       (dict(m=768, n=512, k=1024, batch=3), 4), (dict(m=512, n=512, k=4096, order_c=1, order_d=1), 3),
                                       (dict(m=512, n=256, k=5120, alpha=0.5), 1), (dict(m=640, n=512, k=2048, ldd=648), 2),
                                       (dict(m=512, n=512, k=2048, epilogue=K.CUBLASLT_EPILOGUE_GELU), 2)]):
        spec = dict(MX, **shape)
        print("case", spec, "grid", grid, flush=True)
        case = Case(spec, 700 + i)
        ref = case.run_oracle()
        if grid is None:
            st, got, _, v = case.run_gpu(gpu_api, forced_kernel=v11, forced_variant=11)
        else:
            st, got, plan = case.run_gpu_plan(gpu_api, v11, 11, grid_x=grid)
            v = plan.variant
        assert st == 0 and v == 11
        case.compare(got, ref)


# ---- MXFP4 -----------------------------------------------------------------------------------------
@pytest.mark.parametrize("variant", range(8))
def test_mfma_mxf4_variants(gpu_api, variant):
    check(gpu_api, dict(MX, m=256, n=256, k=512), 50 + variant, K.ZLUDA_KERNEL_MFMA_MXF4, variant)
    check(gpu_api, dict(MX, m=288, n=160, k=768, batch=2), 60 + variant, K.ZLUDA_KERNEL_MFMA_MXF4, variant)


@pytest.mark.parametrize("variant", [4, 5, 6, 8, 9])
def test_last_real_stage_is_waited_for(gpu_api, variant):
    """tile variants with three or four LDS stages wait for a stage by counting the younger operations in
    flight; behind the last stage of K those are padding.  A padding instruction that is out of range as a
    whole completes without a memory round trip and retires ahead of older loads, so the last stage was
    read before it had landed, once in a while: padding is a real load now.  K just above the number of
    LDS stages, repeated, with other work in between."""
    import torch
    other = torch.randn(1 << 22, device="cuda:0")
    bkb = 64 if variant == 4 else 128
    for rep in range(6):
        other.mul_(1.0001)
        if variant < 8:   # (variants 8 .., the 16x16 MFMA shapes, serve int8 and fp8)
            check(gpu_api, dict(MX, m=512, n=256, k=1024), 116, K.ZLUDA_KERNEL_MFMA_MXF4, variant)
        check(gpu_api, dict(I8, m=512, n=256, k=5 * bkb, alpha=1), 117 + rep, K.ZLUDA_KERNEL_MFMA_I8, variant)
        check(gpu_api, dict(F8, m=512, n=256, k=5 * bkb), 118 + rep, K.ZLUDA_KERNEL_MFMA_F8, variant)


@pytest.mark.parametrize("variant", [3, 4, 5, 6])
def test_mfma_mxf4_more_workgroups_than_cus(gpu_api, variant):
    """grids of several rounds of workgroups per CU: a workgroup that follows another one on its CU sees other
    memory timings than the first (the deeper LDS rings of the small tiles once counted their scale loads into the
    waits for the data and multiplied blocks that had not landed)"""
    for rep in range(3):
        check(gpu_api, dict(MX, m=8000, n=256, k=2048, batch=3), 1160 + variant, K.ZLUDA_KERNEL_MFMA_MXF4, variant)
    if variant == 5:   # the same through split-K shares (504 workgroups)
        case = Case(dict(MX, m=1771, n=17, k=13824, batch=3, order_d=1), 1170)
        ref = case.run_oracle()
        for rep in range(3):
            st, got, _, v = case.run_gpu(gpu_api, forced_kernel=K.ZLUDA_KERNEL_MFMA_MXF4, forced_variant=5, workspace_bytes=1 << 24)
            assert st == 0 and v == 5
            case.compare(got, ref)


@pytest.mark.parametrize("family,kernel", [("i8", K.ZLUDA_KERNEL_MFMA_I8), ("f8", K.ZLUDA_KERNEL_MFMA_F8)])
def test_small_tiles_on_grids_of_several_rounds(gpu_api, family, kernel):
    """the 3- and 4-stage tile variants with more workgroups than CUs and a K tail"""
    base = I8 if family == "i8" else F8
    for variant in (4, 5, 6, 10):
        check(gpu_api, dict(base, m=8000, n=200, k=400 if family == "i8" else 272, batch=3), 1180 + variant, kernel, variant)


def test_mxf4_generic_agrees(gpu_api):
    check(gpu_api, dict(MX, m=96, n=80, k=384), 70, K.ZLUDA_KERNEL_GENERIC)


# ---- W8A8 decode -----------------------------------------------------------------------------------
@pytest.mark.parametrize("variant", range(4))
@pytest.mark.parametrize("tokens", [1, 7, 16])
def test_decode_variants(gpu_api, variant, tokens):
    nw, steps = [(8, 8), (8, 16), (4, 16), (4, 8)][variant]
    kfull = nw * steps * 64
    check(gpu_api, dict(DECODE, m=1000, n=tokens, k=kfull), 80 + variant, K.ZLUDA_KERNEL_DECODE_W8A8, variant, int_dist="normal")
    check(gpu_api, dict(DECODE, m=528, n=tokens, k=1088), 90 + variant, K.ZLUDA_KERNEL_DECODE_W8A8, variant, int_dist="normal")


@pytest.mark.parametrize("variant", [0, 3])
def test_decode_two_token_blocks_and_long_k(gpu_api, variant):
    check(gpu_api, dict(DECODE, m=640, n=32, k=4096 if variant == 0 else 2048), 100, K.ZLUDA_KERNEL_DECODE_W8A8, variant, int_dist="normal")
    check(gpu_api, dict(DECODE, m=400, n=17, k=9280), 101, K.ZLUDA_KERNEL_DECODE_W8A8, variant, int_dist="normal")   # several chunks


STREAM = {4: (8, 8), 5: (8, 16), 6: (8, 28), 7: (4, 8), 8: (8, 12), 9: (8, 24), 10: (4, 4), 11: (8, 20), 12: (4, 28),
          13: (4, 12), 14: (4, 20), 15: (8, 32)}


def check_small_grid(gpu_api, spec, seed, variant, grid_x, **case_kw):
    """through the inner launch layer with a grid of `grid_x` workgroups: several 16-row blocks per workgroup"""
    print("case", spec, "seed", seed, "variant", variant, "grid_x", grid_x, flush=True)
    case = Case(spec, seed, **case_kw)
    st, got, plan = case.run_gpu_plan(gpu_api, K.ZLUDA_KERNEL_DECODE_W8A8, variant, grid_x=grid_x)
    assert st == 0 and plan.kernel == K.ZLUDA_KERNEL_DECODE_W8A8 and plan.variant == variant
    case.compare(got, case.run_oracle())


@pytest.mark.parametrize("variant", sorted(STREAM))
def test_decode_stream_variants(gpu_api, variant):
    """weights streamed through LDS: every K the variant table serves, ragged row ranges (row count
    neither a multiple of 16 nor of the grid), several 16-row blocks per workgroup, 1..32 tokens"""
    nw, steps = STREAM[variant]
    k = nw * steps * 64
    check(gpu_api, dict(DECODE, m=1000, n=16, k=k), 120 + variant, K.ZLUDA_KERNEL_DECODE_W8A8, variant, int_dist="normal")
    # 7 workgroups: 142.86 rows each, 9 blocks, the last partial
    check_small_grid(gpu_api, dict(DECODE, m=1000, n=5, k=k, lda=k + 64), 140 + variant, variant, 7, int_dist="normal")
    # more tokens: blocks of 16, as many as the activation registers allow (blocks x steps <= 32)
    for blocks, tokens in ((2, 29), (3, 41), (4, 64)):
        if blocks * steps <= 32:
            check(gpu_api, dict(DECODE, m=332, n=tokens, k=k), 160 + variant, K.ZLUDA_KERNEL_DECODE_W8A8, variant, int_dist="normal")
            check(gpu_api, dict(I8, m=333, n=tokens - 1, k=k, with_c=True), 180 + variant, K.ZLUDA_KERNEL_DECODE_W8A8, variant)


@pytest.mark.parametrize("variant", sorted(STREAM))
def test_decode_stream_variants_fp8(gpu_api, variant):
    """the same kernel for e4m3 x e4m3 (v_mfma_f32_16x16x128_f8f6f4): per-tensor scales, bias, bf16 / f16 / f32
    outputs, ragged row ranges, 1..64 tokens, a C read"""
    nw, steps = STREAM[variant]
    k = nw * steps * 64
    DEC = K.ZLUDA_KERNEL_DECODE_W8A8
    f8 = dict(F8, epilogue=K.CUBLASLT_EPILOGUE_BIAS, bias_type=K.CUDA_R_16BF, with_scalar_scales=True, scale_range=(0.05, 0.06))
    check(gpu_api, dict(f8, m=1000, n=16, k=k), 420 + variant, DEC, variant)
    check_small_grid(gpu_api, dict(f8, m=1000, n=5, k=k, lda=k + 64, d_type=K.CUDA_R_16F), 440 + variant, variant, 7)
    check(gpu_api, dict(F8, m=333, n=3, k=k, with_c=True, d_type=K.CUDA_R_32F, c_type=K.CUDA_R_32F), 450 + variant, DEC, variant)
    for blocks, tokens in ((2, 29), (3, 41), (4, 64)):
        if blocks * steps <= 32:
            check(gpu_api, dict(f8, m=332, n=tokens, k=k, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS), 460 + variant, DEC, variant)


# The slab form of the stream kernel, up to 16 tokens and 4 blocks per workgroup: variant 16 = 4 waves x one 1 KiB unit
# (2048 < K <= 4096), variants 17..19 = 8 waves x 2..4 units of 512 bytes (K up to 8192, 12288, 16384).
SLAB_K = [(16, 4096), (16, 3072), (16, 2064), (16, 3600), (17, 8192), (17, 5120), (17, 4112), (18, 12288), (18, 11008),
          (18, 8208), (19, 16384), (19, 13824), (19, 12304)]


@pytest.mark.parametrize("variant,k", SLAB_K)
def test_decode_slab_variant(gpu_api, variant, k):
    """whole row segments through LDS: exact and short K (slabs that end inside a unit, a last slab shorter than the
    others, units that lie past the end altogether), ragged row ranges, 1..16 tokens, round-robin blocks plus a split
    remainder, both epilogues"""
    DEC = K.ZLUDA_KERNEL_DECODE_W8A8
    check(gpu_api, dict(DECODE, m=1000, n=16, k=k), 520, DEC, variant, int_dist="normal")
    check(gpu_api, dict(DECODE, m=1000, n=1, k=k, bias_type=K.CUDA_R_16BF), 521, DEC, variant, int_dist="normal")
    # 17 workgroups: 3 round-robin blocks each and 184 rows left, 2-3 quads per workgroup
    check_small_grid(gpu_api, dict(DECODE, m=1000, n=5, k=k, lda=k + 64), 522, variant, 17, int_dist="normal")
    # 16 workgroups, 1024 rows: exactly 4 rounds, nothing left
    check_small_grid(gpu_api, dict(DECODE, m=1024, n=16, k=k, d_type=K.CUDA_R_16F), 523, variant, 16, int_dist="normal")
    # element-wise epilogue: int32 with C, a row count that is no multiple of 4, f32 output with scalar factors
    check(gpu_api, dict(I8, m=333, n=15, k=k, with_c=True), 524, DEC, variant)
    check_small_grid(gpu_api, dict(I8, m=333, n=7, k=k, with_c=True, batch=2), 525, variant, 6)
    check(gpu_api, dict(I8F, m=402, n=9, k=k, d_type=K.CUDA_R_32F, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS, alpha_range=(0.001, 0.002)), 526, DEC, variant)
    # scalar alpha, no bias, packed store; tokens along M (weights are operand B)
    check(gpu_api, dict(I8F, m=640, n=12, k=k, alpha_range=(0.001, 0.002), batch=3), 527, DEC, variant)
    check(gpu_api, dict(I8F, transa=0, transb=1, order_a=1, order_b=1, order_c=1, order_d=1, m=11, n=2048, k=k,
                        epilogue=K.CUBLASLT_EPILOGUE_RELU_BIAS, bias_type=K.CUDA_R_16F, alpha_range=(0.001, 0.002)), 528, DEC, variant, int_dist="normal")


@pytest.mark.parametrize("variant,k", [(16, 4096), (16, 3072), (16, 2176), (17, 8192), (17, 4224), (18, 11008), (19, 13824), (19, 16384)])
def test_decode_slab_variant_fp8(gpu_api, variant, k):
    DEC = K.ZLUDA_KERNEL_DECODE_W8A8
    f8 = dict(F8, epilogue=K.CUBLASLT_EPILOGUE_BIAS, bias_type=K.CUDA_R_16BF, with_scalar_scales=True, scale_range=(0.05, 0.06))
    check(gpu_api, dict(f8, m=1000, n=16, k=k), 540, DEC, variant)
    check_small_grid(gpu_api, dict(f8, m=1000, n=5, k=k, lda=k + 64, d_type=K.CUDA_R_16F), 541, variant, 17)
    check(gpu_api, dict(F8, m=333, n=3, k=k, with_c=True, d_type=K.CUDA_R_32F, c_type=K.CUDA_R_32F), 542, DEC, variant)
    check(gpu_api, dict(f8, m=332, n=13, k=k, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS, bias_type=K.CUDA_R_32F), 543, DEC, variant)


@pytest.mark.parametrize("variant,k", [(20, 4096), (20, 3072), (20, 2064), (17, 8192), (17, 5120), (17, 4112)])
def test_decode_slab_two_token_blocks(gpu_api, variant, k):
    """17 .. 32 tokens on the 8-wave shapes of one or two units: ragged token counts, both epilogues, int8 and fp8,
    tokens along M, several blocks per workgroup with a split remainder"""
    DEC = K.ZLUDA_KERNEL_DECODE_W8A8
    check(gpu_api, dict(DECODE, m=1000, n=32, k=k), 560, DEC, variant, int_dist="normal")
    check(gpu_api, dict(DECODE, m=1000, n=17, k=k, bias_type=K.CUDA_R_16BF), 561, DEC, variant, int_dist="normal")
    check_small_grid(gpu_api, dict(DECODE, m=1000, n=29, k=k, lda=k + 64), 562, variant, 17, int_dist="normal")
    check_small_grid(gpu_api, dict(DECODE, m=1024, n=32, k=k, d_type=K.CUDA_R_16F), 563, variant, 16, int_dist="normal")
    check(gpu_api, dict(I8, m=333, n=31, k=k, with_c=True), 564, DEC, variant)
    check_small_grid(gpu_api, dict(I8, m=333, n=19, k=k, with_c=True, batch=2), 565, variant, 6)
    check(gpu_api, dict(I8F, transa=0, transb=1, order_a=1, order_b=1, order_c=1, order_d=1, m=27, n=2048, k=k,
                        epilogue=K.CUBLASLT_EPILOGUE_RELU_BIAS, bias_type=K.CUDA_R_16F, alpha_range=(0.001, 0.002)), 566, DEC, variant, int_dist="normal")
    f8 = dict(F8, epilogue=K.CUBLASLT_EPILOGUE_BIAS, bias_type=K.CUDA_R_16BF, with_scalar_scales=True, scale_range=(0.05, 0.06))
    check(gpu_api, dict(f8, m=1000, n=32, k=k), 567, DEC, variant)
    check_small_grid(gpu_api, dict(f8, m=1000, n=21, k=k, lda=k + 64, d_type=K.CUDA_R_16F, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS), 568, variant, 17)
    check(gpu_api, dict(F8, m=333, n=18, k=k, with_c=True, d_type=K.CUDA_R_32F, c_type=K.CUDA_R_32F), 569, DEC, variant)


def test_decode_slab_is_refused_outside_its_range(gpu_api):
    """more than 16 tokens, K beyond the cover or under the next smaller one, more rows than 4 blocks per workgroup hold"""
    DEC = K.ZLUDA_KERNEL_DECODE_W8A8
    for variant, spec in ((16, dict(DECODE, m=512, n=17, k=4096)), (16, dict(DECODE, m=512, n=16, k=4112)),
                          (16, dict(DECODE, m=512, n=16, k=2048)), (17, dict(DECODE, m=512, n=16, k=4096)),
                          (17, dict(DECODE, m=512, n=16, k=8208)), (19, dict(DECODE, m=512, n=16, k=12288)),
                          (19, dict(DECODE, m=512, n=17, k=16384)), (20, dict(DECODE, m=512, n=16, k=4096)),
                          (20, dict(DECODE, m=512, n=33, k=4096)), (17, dict(DECODE, m=512, n=33, k=8192))):
        st, _, _ = Case(spec, 550).run_gpu_plan(gpu_api, DEC, variant)
        assert st == K.CUBLAS_STATUS_NOT_SUPPORTED, (variant, spec, st)
    for variant, k in ((16, 4096), (18, 11008)):
        st, _, _ = Case(dict(DECODE, m=1000, n=4, k=k), 551).run_gpu_plan(gpu_api, DEC, variant, grid_x=12)   # 1000 > 12 * 64 rows
        assert st == K.CUBLAS_STATUS_NOT_SUPPORTED, st


def test_decode_fp8_planner_choice_and_orientation(gpu_api):
    DEC = K.ZLUDA_KERNEL_DECODE_W8A8
    check(gpu_api, dict(F8, m=14336, n=16, k=4096, with_scalar_scales=True, scale_range=(0.05, 0.06)), 470, expect_kernel=DEC)
    # row-major activations [tokens][K] x weights^T: tokens are rows of D
    check(gpu_api, dict(F8, transa=0, transb=1, order_a=1, order_b=1, order_c=1, order_d=1, m=16, n=2048, k=4096,
                        epilogue=K.CUBLASLT_EPILOGUE_BIAS, bias_type=K.CUDA_R_16BF), 471, expect_kernel=DEC)
    # what the family does not take: mixed formats, K under no instantiation's cover -> the MFMA tiles
    check(gpu_api, dict(F8, a_type=K.CUDA_R_8F_E5M2, m=2048, n=16, k=4096), 472, expect_kernel=K.ZLUDA_KERNEL_MFMA_F8)
    check(gpu_api, dict(F8, m=2048, n=16, k=1536), 473, expect_kernel=K.ZLUDA_KERNEL_MFMA_F8)
    check(gpu_api, dict(F8, m=2048, n=16, k=2624 + 64), 474, expect_kernel=DEC)     # under the 3072 cover


def test_decode_config3_shape_takes_the_stream_kernel(gpu_api):
    st_spec = dict(DECODE, m=14336, n=16, k=4096)
    check(gpu_api, st_spec, 2, expect_kernel=K.ZLUDA_KERNEL_DECODE_W8A8, int_dist="normal")


def test_decode_tokens_along_m_and_int32_out(gpu_api):
    # row-major activations [tokens][K] x weights^T: tokens are rows of D
    spec = dict(I8F, transa=0, transb=1, order_a=1, order_b=1, order_c=1, order_d=1, m=16, n=2048, k=4096,
                epilogue=K.CUBLASLT_EPILOGUE_BIAS, bias_type=K.CUDA_R_32F, alpha_range=(0.001, 0.002))
    check(gpu_api, spec, 110, expect_kernel=K.ZLUDA_KERNEL_DECODE_W8A8, int_dist="normal")
    check(gpu_api, dict(I8, m=2048, n=8, k=4096, with_c=True), 111, expect_kernel=K.ZLUDA_KERNEL_DECODE_W8A8)


# ---- generic kernel (layouts the MFMA kernels do not take) -------------------------------------------
@pytest.mark.parametrize("ta,tb,oa,ob,od", [(0, 1, 0, 0, 0), (0, 0, 0, 0, 1), (1, 1, 1, 0, 0), (0, 1, 1, 1, 1)])
def test_generic_layouts_int8(gpu_api, ta, tb, oa, ob, od):
    spec = dict(I8, transa=ta, transb=tb, order_a=oa, order_b=ob, order_c=od, order_d=od, m=150, n=90, k=77,
                batch=2, with_c=True)
    check(gpu_api, spec, 120, K.ZLUDA_KERNEL_GENERIC)


@pytest.mark.parametrize("t", [K.CUDA_R_32F, K.CUDA_R_16F, K.CUDA_R_16BF, K.CUDA_R_8F_E4M3])
def test_generic_float_types(gpu_api, t):
    spec = dict(a_type=t, b_type=t, d_type=K.CUDA_R_32F if t == K.CUDA_R_32F else K.CUDA_R_16BF,
                compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F, m=130, n=70, k=96, transb=1,
                epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS, with_c=True, with_cd_scales=True)
    # (f32 operands have no other kernel; the 16-bit and fp8 ones would go to their transposing MFMA kernels)
    check(gpu_api, spec, 130, K.ZLUDA_KERNEL_GENERIC, expect_kernel=K.ZLUDA_KERNEL_GENERIC, tol=2e-2 if t == K.CUDA_R_32F else None)


def test_misaligned_pointers_fall_back(gpu_api):
    case = Case(dict(I8, m=256, n=256, k=256), 140)
    ref = case.run_oracle()
    st, got, k, _ = case.run_gpu(gpu_api, offset_bytes=4)   # heuristic promised alignment; pointers are off by 4
    assert st == 0 and k == K.ZLUDA_KERNEL_MFMA_I8            # the token says MFMA, the call ran the generic kernel
    case.compare(got, ref)


# ---- benchmark configurations ---------------------------------------------------------------------------
def test_config1_int8_256_nt(gpu_api):
    check(gpu_api, dict(I8, transa=0, transb=1, m=256, n=256, k=256, alpha=1), 0, expect_kernel=K.ZLUDA_KERNEL_MFMA_TR8)
    check(gpu_api, dict(I8, transa=0, transb=1, m=256, n=256, k=256, alpha=1), 0, K.ZLUDA_KERNEL_GENERIC)


def test_config3_decode_full_size(gpu_api):
    check(gpu_api, dict(DECODE, m=14336, n=16, k=4096), 2, expect_kernel=K.ZLUDA_KERNEL_DECODE_W8A8, int_dist="normal")


def test_config2_int8_4096_full_size(gpu_api):
    check(gpu_api, dict(I8, m=4096, n=4096, k=4096, alpha=1), 1, expect_kernel=K.ZLUDA_KERNEL_MFMA_I8)
