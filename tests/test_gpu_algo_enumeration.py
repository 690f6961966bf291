"""The calls applications make around cublasLtMatmul when they do not use the heuristic, end to end on the
GPU (cuda_macros/src/cublaslt.rs:104-111, 162-176, 225-231, 397-518): descriptors built by the
cublasLt*Init_internal entry points in the caller's own storage (what the cublasLt*Init() inlines of the CUDA
header do), algorithms enumerated with cublasLtMatmulAlgoGetIds, a token made by cublasLtMatmulAlgoInit,
its tile variant chosen through cublasLtMatmulAlgoConfigSetAttribute(CUSTOM_OPTION), validated by
cublasLtMatmulAlgoCheck and handed to cublasLtMatmul.  Results against the CPU oracle."""
import ctypes as C

import numpy as np
import pytest

from oracle.cases import Case
from zluda_amd import abi

pytestmark = pytest.mark.gpu
K = abi

ALGO_CONFIG_ID, ALGO_CONFIG_CUSTOM_OPTION = 0, 5
ALGO_CAP_CUSTOM_OPTION_MAX = 7


def run_enumerated(api, spec, seed, want_family, variants):
    import torch
    case = Case(spec, seed)
    ref = case.run_oracle()
    m, n, k = spec["m"], spec["n"], spec["k"]
    ta, tb = spec.get("transa", 0), spec.get("transb", 0)

    handle = C.c_void_p()
    assert api.cublasLtCreate(C.byref(handle)) == 0
    # descriptors in caller storage: 256 bytes for the matmul descriptor, 64 for layouts and the preference
    desc, pref = C.create_string_buffer(256), C.create_string_buffer(64)
    lay = {t: C.create_string_buffer(64) for t in "abcd"}
    assert api.cublasLtMatmulDescInit_internal(desc, 256, spec["compute_type"], spec["scale_type"]) == 0
    assert api.cublasLtMatmulPreferenceInit_internal(pref, 64) == 0
    shapes = {"a": (spec["a_type"], k if ta else m, m if ta else k), "b": (spec["b_type"], n if tb else k, k if tb else n),
              "c": (spec.get("c_type", spec["d_type"]), m, n), "d": (spec["d_type"], m, n)}
    for t, (typ, rows, cols) in shapes.items():
        assert api.cublasLtMatrixLayoutInit_internal(lay[t], 64, typ, rows, cols, rows) == 0
    assert api.desc_set(desc, K.CUBLASLT_MATMUL_DESC_TRANSA, C.c_int32, ta) == 0
    assert api.desc_set(desc, K.CUBLASLT_MATMUL_DESC_TRANSB, C.c_int32, tb) == 0
    if "epilogue" in spec:
        assert api.desc_set(desc, K.CUBLASLT_MATMUL_DESC_EPILOGUE, C.c_uint32, spec["epilogue"]) == 0
    if "bias_type" in spec:
        assert api.desc_set(desc, K.CUBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, C.c_int32, spec["bias_type"]) == 0

    # enumerate the algorithm ids for this type combination; the family we want must be among them
    types = (spec["compute_type"], spec["scale_type"], spec["a_type"], spec["b_type"], spec.get("c_type", spec["d_type"]),
             spec["d_type"])
    ids, cnt = (C.c_int * 8)(), C.c_int(0)
    assert api.cublasLtMatmulAlgoGetIds(handle, *types, 8, ids, C.byref(cnt)) == 0
    assert want_family in ids[:cnt.value]

    keep, ptr, dt = case.upload()
    for attr, name in ((K.CUBLASLT_MATMUL_DESC_BIAS_POINTER, "bias"), (K.CUBLASLT_MATMUL_DESC_A_SCALE_POINTER, "a_scale"),
                       (K.CUBLASLT_MATMUL_DESC_B_SCALE_POINTER, "b_scale")):
        if ptr.get(name) is not None:
            assert api.desc_set(desc, attr, C.c_void_p, ptr[name]) == 0
    alpha, beta = case.scalars(ptr)
    stream = torch.cuda.current_stream().cuda_stream
    canary = torch.from_numpy(np.frombuffer(case.new_d().tobytes(), dtype=np.uint8).copy()).cuda()
    try:
        algo = abi.cublasLtMatmulAlgo_t()
        assert api.cublasLtMatmulAlgoInit(handle, *types, want_family, C.byref(algo)) == 0
        vmax, wrote = C.c_int32(), C.c_size_t()
        assert api.cublasLtMatmulAlgoCapGetAttribute(C.byref(algo), ALGO_CAP_CUSTOM_OPTION_MAX, C.byref(vmax), 4, C.byref(wrote)) == 0
        for variant in variants:
            # CUSTOM_OPTION: 0 leaves the tile variant to the planner, v + 1 selects variant v; the capability
            # attribute reports the largest value
            assert variant + 1 <= vmax.value
            print("enumerated algorithm: family %d, CUSTOM_OPTION %d" % (want_family, variant + 1), spec, flush=True)
            v = C.c_uint32(variant + 1)
            assert api.cublasLtMatmulAlgoConfigSetAttribute(C.byref(algo), ALGO_CONFIG_CUSTOM_OPTION, C.byref(v), 4) == 0
            res = abi.cublasLtMatmulHeuristicResult_t()
            assert api.cublasLtMatmulAlgoCheck(handle, desc, lay["a"], lay["b"], lay["c"], lay["d"], C.byref(algo), C.byref(res)) == 0
            assert res.state == 0 and res.workspaceSize == 0
            assert (res.algo.data[0] & 0xFFFFFFFF) == want_family and (res.algo.data[1] & 0xFFFFFFFF) == variant
            dt[case._guard:case._guard + canary.numel()] = canary
            st = api.cublasLtMatmul(handle, desc, C.addressof(alpha), ptr["A"], lay["a"], ptr["B"], lay["b"], C.addressof(beta),
                                    ptr["C"], lay["c"], ptr["D"], lay["d"], C.byref(res.algo), None, 0, stream)
            torch.cuda.synchronize()
            assert st == 0, "cublasLtMatmul status %d" % st
            case.compare(case.download(dt), ref)
    finally:
        assert api.cublasLtDestroy(handle) == 0


def test_int8_through_enumerated_algorithms(gpu_api):
    spec = dict(a_type=K.CUDA_R_8I, b_type=K.CUDA_R_8I, c_type=K.CUDA_R_32I, d_type=K.CUDA_R_32I,
                compute_type=K.CUBLAS_COMPUTE_32I, scale_type=K.CUDA_R_32I, transa=1, m=512, n=384, k=1024, alpha=1)
    run_enumerated(gpu_api, spec, 501, K.ZLUDA_KERNEL_MFMA_I8, [0, 3, 6, 8])
    run_enumerated(gpu_api, dict(spec, transa=0, transb=1), 502, K.ZLUDA_KERNEL_MFMA_TR8, [1, 2])
    run_enumerated(gpu_api, spec, 503, K.ZLUDA_KERNEL_GENERIC, [0])


def test_fp8_through_enumerated_algorithms(gpu_api):
    spec = dict(a_type=K.CUDA_R_8F_E4M3, b_type=K.CUDA_R_8F_E4M3, c_type=K.CUDA_R_16BF, d_type=K.CUDA_R_16BF,
                compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F, transa=1, m=512, n=256, k=768, alpha=1.0,
                epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS, bias_type=K.CUDA_R_16BF, with_scalar_scales=True)
    run_enumerated(gpu_api, spec, 511, K.ZLUDA_KERNEL_MFMA_F8, [0, 2, 5, 8])
