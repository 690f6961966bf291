"""The drop-in boundary without a GPU: the library loads, exports every symbol include/*.h declares,
and the host-side behaviour of handles, descriptors, attributes and the heuristic matches the
reference's (zluda_blaslt/src/impl.rs; the plumbing tests zluda_blas/src/impl.rs:469-560)."""
import ctypes as C
import os
import re

import pytest

from zluda_amd import abi
from zluda_amd.cublaslt import SIGNATURES, LAUNCH_SIGNATURES, MatmulCall

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NS = abi.CUBLAS_STATUS_NOT_SUPPORTED
IV = abi.CUBLAS_STATUS_INVALID_VALUE


def declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b((?:cublasLt|zluda_gemm_)\w+)\s*\(", text)) - {"cublasLtLoggerCallback_t"}


def test_every_declared_symbol_is_exported(api):
    names = declared("cublaslt_abi.h")
    assert len(names) == 45, sorted(names)           # cuda_macros/src/cublaslt.rs:4-583
    assert names == set(SIGNATURES)
    for n in sorted(names | declared("zluda_gemm_launch.h")):
        assert hasattr(api.lib, n), n
    assert declared("zluda_gemm_launch.h") == set(LAUNCH_SIGNATURES)


def test_soname_links_exist(api):
    d = os.path.dirname(api.path)
    for n in ("libcublaslt.so", "libcublasLt.so", "libcublasLt.so.11", "libcublasLt.so.12", "libcublasLt.so.13"):
        assert os.path.exists(os.path.join(d, n)), n   # zluda_blaslt/Cargo.toml:6-8, 21-23


def test_struct_sizes():
    assert C.sizeof(abi.cublasLtMatmulAlgo_t) == 64
    assert C.sizeof(abi.cublasLtMatmulHeuristicResult_t) == 96   # cuda_types/src/cublaslt.rs:4825-4841


def test_status_names(api):
    assert api.cublasLtGetStatusName(0) == b"CUBLAS_STATUS_SUCCESS"
    assert api.cublasLtGetStatusName(7) == b"CUBLAS_STATUS_INVALID_VALUE"
    assert api.cublasLtGetStatusString(15) == b"CUBLAS_STATUS_NOT_SUPPORTED"
    assert api.cublasLtGetStatusName(12345) == b"CUBLAS_STATUS_UNKNOWN"
    assert api.cublasLtGetVersion() == 130002
    v = C.c_int()
    assert api.cublasLtGetProperty(0, C.byref(v)) == 0 and v.value == 13


def test_handle_lifecycle_and_cookie(api):
    h = C.c_void_p()
    assert api.cublasLtCreate(C.byref(h)) == 0
    cookie = C.cast(h, C.POINTER(C.c_uint64))[0]
    assert cookie == abi.ZLUDA_BLASLT_HANDLE_COOKIE       # zluda_blaslt/src/impl.rs:24-26
    assert api.cublasLtDestroy(h) == 0
    assert api.cublasLtDestroy(h) == IV                   # cookie cleared: zluda_common/src/lib.rs:1076-1085
    assert api.cublasLtDestroy(None) == IV
    assert api.cublasLtCreate(None) == IV


def test_cublas_handle_is_accepted_in_place_of_lt_handle(api):
    """zluda_blas embeds an Lt handle as the first payload word of its own cookie-checked handle
    (zluda_blas/src/impl.rs:17-23); `can_pass_into_blaslt` and `lt_destroy_blas_handle`
    (zluda_blas/src/impl.rs:469-560) pass that handle to cublasLt* calls."""
    lt = C.c_void_p()
    assert api.cublasLtCreate(C.byref(lt)) == 0
    blas = (C.c_uint64 * 4)(abi.ZLUDA_BLAS_HANDLE_COOKIE, lt.value, 0, 0)
    blas_handle = C.cast(blas, C.c_void_p)
    # can_pass_into_blaslt: fp32 64x64x64, heuristic with the cuBLAS handle must succeed
    call = MatmulCall(api, dict(m=64, n=64, k=64, a_type=abi.CUDA_R_32F, b_type=abi.CUDA_R_32F, d_type=abi.CUDA_R_32F,
                                compute_type=abi.CUBLAS_COMPUTE_32F, scale_type=abi.CUDA_R_32F))
    res = abi.cublasLtMatmulHeuristicResult_t()
    cnt = C.c_int(0)
    st = api.cublasLtMatmulAlgoGetHeuristic(blas_handle, call.desc, call.a_desc, call.b_desc, call.c_desc,
                                            call.d_desc, call.pref, 1, C.byref(res), C.byref(cnt))
    assert st == 0 and cnt.value == 1 and res.state == 0
    call.close()
    # lt_destroy_blas_handle: destroying through the cuBLAS handle destroys the embedded Lt handle only
    assert api.cublasLtDestroy(blas_handle) == 0
    assert blas[0] == abi.ZLUDA_BLAS_HANDLE_COOKIE
    assert api.cublasLtDestroy(lt) == IV
    garbage = (C.c_uint64 * 4)(0x1234, 0, 0, 0)
    assert api.cublasLtDestroy(C.cast(garbage, C.c_void_p)) == IV


def test_matmul_desc_attributes(api):
    d = C.c_void_p()
    assert api.cublasLtMatmulDescCreate(C.byref(d), abi.CUBLAS_COMPUTE_32I, abi.CUDA_R_32I) == 0
    D = abi
    # accepted by the reference: zluda_blaslt/src/impl.rs:257-305
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_TRANSA, C.c_int32, D.CUBLAS_OP_T) == 0
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_TRANSB, C.c_int32, 7) == IV
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_EPILOGUE, C.c_uint32, D.CUBLASLT_EPILOGUE_GELU_BIAS) == 0
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_EPILOGUE, C.c_uint32, D.CUBLASLT_EPILOGUE_BGRADA) == 0
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_EPILOGUE, C.c_uint32, D.CUBLASLT_EPILOGUE_BGRADB) == 0
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_EPILOGUE, C.c_uint32, D.CUBLASLT_EPILOGUE_GELU_BIAS) == 0
    # every epilogue zluda_common/src/lib.rs:762-804 maps is taken; the ReLU bit-mask forms, which it does not map, are not
    for e in (D.CUBLASLT_EPILOGUE_GELU_AUX, D.CUBLASLT_EPILOGUE_GELU_AUX_BIAS, D.CUBLASLT_EPILOGUE_DGELU, D.CUBLASLT_EPILOGUE_DGELU_BGRAD):
        assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_EPILOGUE, C.c_uint32, e) == 0
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_EPILOGUE, C.c_uint32, D.CUBLASLT_EPILOGUE_RELU_AUX) == NS
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, C.c_int32, D.CUDA_R_16BF) == 0
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_BIAS_POINTER, C.c_void_p, 0x1000) == 0
    # SCALE_TYPE: size check then type check (impl.rs:263-272)
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_SCALE_TYPE, C.c_int64, D.CUDA_R_32F) == IV
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_SCALE_TYPE, C.c_int32, D.CUDA_R_16F) == NS
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_SCALE_TYPE, C.c_int32, D.CUDA_R_32F) == 0
    # the quantized path's additions
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_POINTER_MODE, C.c_int32, D.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO) == 0
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_POINTER_MODE, C.c_int32, 9) == IV
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_A_SCALE_POINTER, C.c_void_p, 0x2000) == 0
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_B_SCALE_MODE, C.c_int32, D.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F) == 0
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_A_SCALE_MODE, C.c_int32, D.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0) == 0
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_A_SCALE_MODE, C.c_int32, D.CUBLASLT_MATMUL_MATRIX_SCALE_VEC16_UE4M3) == NS
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_D_SCALE_MODE, C.c_int32, D.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F) == NS
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_ALPHA_VECTOR_BATCH_STRIDE, C.c_int64, 64) == 0
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_BIAS_BATCH_STRIDE, C.c_int64, 64) == 0
    # the aux matrix of the GELU_AUX / DGELU epilogues: pointer, leading dimension, batch stride; D's type only
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_EPILOGUE_AUX_POINTER, C.c_void_p, 0x1000) == 0
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_EPILOGUE_AUX_LD, C.c_int64, 4096) == 0
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_EPILOGUE_AUX_BATCH_STRIDE, C.c_int64, 1 << 24) == 0
    assert api.desc_set(d, D.CUBLASLT_MATMUL_DESC_EPILOGUE_AUX_LD, C.c_int32, 4096) == IV
    # EPILOGUE_AUX_DATA_TYPE: kept in the descriptor (a type other than D's is refused when the problem is planned)
    assert api.desc_set(d, 22, C.c_int32, D.CUDA_R_16BF) == 0 and api.desc_set(d, 22, C.c_int32, -1) == 0
    # everything else: NOT_SUPPORTED (impl.rs:302)
    assert api.desc_set(d, 23, C.c_void_p, 1) == NS   # EPILOGUE_AUX_SCALE_POINTER
    assert api.cublasLtMatmulDescSetAttribute(d, D.CUBLASLT_MATMUL_DESC_TRANSA, None, 4) == IV
    # get: value, size query, wrong size
    v, w = C.c_int32(), C.c_size_t()
    assert api.cublasLtMatmulDescGetAttribute(d, D.CUBLASLT_MATMUL_DESC_TRANSA, C.byref(v), 4, C.byref(w)) == 0
    assert v.value == D.CUBLAS_OP_T and w.value == 4
    assert api.cublasLtMatmulDescGetAttribute(d, D.CUBLASLT_MATMUL_DESC_BIAS_POINTER, None, 0, C.byref(w)) == 0 and w.value == 8
    assert api.cublasLtMatmulDescGetAttribute(d, D.CUBLASLT_MATMUL_DESC_TRANSA, C.byref(v), 2, C.byref(w)) == IV
    p = C.c_void_p()
    assert api.cublasLtMatmulDescGetAttribute(d, D.CUBLASLT_MATMUL_DESC_A_SCALE_POINTER, C.byref(p), 8, None) == 0 and p.value == 0x2000
    assert api.cublasLtMatmulDescDestroy(d) == 0
    assert api.cublasLtMatmulDescDestroy(None) == IV


def test_layout_and_preference_attributes(api):
    D = abi
    l = C.c_void_p()
    assert api.cublasLtMatrixLayoutCreate(C.byref(l), D.CUDA_R_8I, 128, 64, 128) == 0
    assert api.layout_set(l, D.CUBLASLT_MATRIX_LAYOUT_ORDER, C.c_int32, D.CUBLASLT_ORDER_ROW) == 0
    assert api.layout_set(l, D.CUBLASLT_MATRIX_LAYOUT_ORDER, C.c_int32, D.CUBLASLT_ORDER_COL32) == NS
    assert api.layout_set(l, D.CUBLASLT_MATRIX_LAYOUT_BATCH_COUNT, C.c_int32, 4) == 0
    assert api.layout_set(l, D.CUBLASLT_MATRIX_LAYOUT_BATCH_COUNT, C.c_int32, 0) == IV
    assert api.layout_set(l, D.CUBLASLT_MATRIX_LAYOUT_STRIDED_BATCH_OFFSET, C.c_int64, 8192) == 0
    assert api.layout_set(l, D.CUBLASLT_MATRIX_LAYOUT_TYPE, C.c_uint32, D.CUDA_R_4F_E2M1) == 0
    assert api.layout_set(l, D.CUBLASLT_MATRIX_LAYOUT_LD, C.c_int32, 128) == IV     # LD is int64
    assert api.layout_set(l, D.CUBLASLT_MATRIX_LAYOUT_PLANE_OFFSET, C.c_int64, 0) == NS
    v64, w = C.c_int64(), C.c_size_t()
    assert api.cublasLtMatrixLayoutGetAttribute(l, D.CUBLASLT_MATRIX_LAYOUT_STRIDED_BATCH_OFFSET, C.byref(v64), 8, C.byref(w)) == 0
    assert v64.value == 8192
    u = C.c_uint64()
    assert api.cublasLtMatrixLayoutGetAttribute(l, D.CUBLASLT_MATRIX_LAYOUT_ROWS, C.byref(u), 8, None) == 0 and u.value == 128
    assert api.cublasLtMatrixLayoutDestroy(l) == 0
    p = C.c_void_p()
    assert api.cublasLtMatmulPreferenceCreate(C.byref(p)) == 0
    assert api.pref_set(p, D.CUBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, C.c_uint64, 1 << 20) == 0
    assert api.pref_set(p, D.CUBLASLT_MATMUL_PREF_SEARCH_MODE, C.c_uint32, 0) == 0
    assert api.pref_set(p, D.CUBLASLT_MATMUL_PREF_MIN_ALIGNMENT_A_BYTES, C.c_uint32, 16) == 0   # impl.rs:346-353
    assert api.pref_set(p, 2, C.c_uint32, 0) == NS
    m = C.c_uint64()
    assert api.cublasLtMatmulPreferenceGetAttribute(p, D.CUBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, C.byref(m), 8, None) == 0
    assert m.value == 1 << 20
    assert api.cublasLtMatmulPreferenceDestroy(p) == 0


def test_unimplemented_exports_return_not_supported(api):
    # zluda_blaslt/src/lib.rs:44-70 + impl.rs:83-86 (release build)
    assert api.cublasLtLoggerSetLevel(1) == NS
    assert api.cublasLtLoggerForceDisable() == NS
    assert api.cublasLtLoggerOpenFile(b"/dev/null") == NS
    assert api.cublasLtHeuristicsCacheSetCapacity(8) == NS
    assert api.cublasLtMatrixTransformDescCreate(C.byref(C.c_void_p()), abi.CUDA_R_32F) == NS
    assert api.cublasLtMatrixTransformDescInit_internal(C.create_string_buffer(64), 64, abi.CUDA_R_32F) == NS
    assert api.cublasLtDisableCpuInstructionsSetMask(1) == 0
    assert api.cublasLtDisableCpuInstructionsSetMask(0) == 1


def test_init_internal_builds_descriptors_in_caller_storage(api):
    """the cublasLt*Init() inlines of the CUDA header pass their own opaque structs: 256 bytes for a matmul
    descriptor, 64 for a layout or a preference (cuda_types/src/cublaslt.rs:43-83)"""
    IV = abi.CUBLAS_STATUS_INVALID_VALUE
    desc, pref = C.create_string_buffer(256), C.create_string_buffer(64)
    lay = [C.create_string_buffer(64) for _ in range(3)]
    assert api.cublasLtMatmulDescInit_internal(desc, 256, abi.CUBLAS_COMPUTE_32I, abi.CUDA_R_32I) == 0
    assert api.cublasLtMatmulDescInit_internal(desc, 16, abi.CUBLAS_COMPUTE_32I, abi.CUDA_R_32I) == IV
    assert api.cublasLtMatmulDescInit_internal(None, 256, abi.CUBLAS_COMPUTE_32I, abi.CUDA_R_32I) == IV
    assert api.cublasLtMatmulPreferenceInit_internal(pref, 64) == 0
    assert api.cublasLtMatmulPreferenceInit_internal(None, 64) == IV
    assert api.cublasLtMatmulPreferenceInit_internal(pref, 8) == IV
    for buf, typ in zip(lay, (abi.CUDA_R_8I, abi.CUDA_R_8I, abi.CUDA_R_32I)):
        assert api.cublasLtMatrixLayoutInit_internal(buf, 64, typ, 512, 512, 512) == 0
    assert api.cublasLtMatrixLayoutInit_internal(lay[0], 32, abi.CUDA_R_8I, 512, 512, 512) == IV
    # they behave like created ones: attributes, heuristic
    op = C.c_int32(abi.CUBLAS_OP_T)
    assert api.cublasLtMatmulDescSetAttribute(desc, abi.CUBLASLT_MATMUL_DESC_TRANSA, C.byref(op), 4) == 0
    back, wrote = C.c_int32(-1), C.c_size_t()
    assert api.cublasLtMatmulDescGetAttribute(desc, abi.CUBLASLT_MATMUL_DESC_TRANSA, C.byref(back), 4, C.byref(wrote)) == 0
    assert back.value == abi.CUBLAS_OP_T and wrote.value == 4
    rows = C.c_uint64()
    assert api.cublasLtMatrixLayoutGetAttribute(lay[2], abi.CUBLASLT_MATRIX_LAYOUT_ROWS, C.byref(rows), 8, None) == 0
    assert rows.value == 512
    h = C.c_void_p()
    assert api.cublasLtCreate(C.byref(h)) == 0
    res = (abi.cublasLtMatmulHeuristicResult_t * 2)()
    n = C.c_int()
    assert api.cublasLtMatmulAlgoGetHeuristic(h, desc, lay[0], lay[1], lay[2], lay[2], pref, 2, res, C.byref(n)) == 0
    assert n.value == 2 and res[0].state == 0
    assert (res[0].algo.data[0] & 0xffffffff) == abi.ZLUDA_KERNEL_MFMA_I8
    assert api.cublasLtDestroy(h) == 0


def test_heuristic_tokens_and_algo_check(api):
    spec = dict(m=4096, n=4096, k=4096, a_type=abi.CUDA_R_8I, b_type=abi.CUDA_R_8I, d_type=abi.CUDA_R_32I,
                compute_type=abi.CUBLAS_COMPUTE_32I, scale_type=abi.CUDA_R_32I, transa=abi.CUBLAS_OP_T)
    call = MatmulCall(api, spec)
    assert len(call.heuristic) == 2                              # MFMA choice, then the generic kernel
    assert call.kernel == abi.ZLUDA_KERNEL_MFMA_I8
    assert call.heuristic[1].algo.data[0] & 0xFFFFFFFF == abi.ZLUDA_KERNEL_GENERIC
    assert call.heuristic[0].algo.data[0] >> 32 == abi.ZLUDA_ALGO_MAGIC
    assert call.heuristic[0].workspaceSize == 0 and call.heuristic[0].wavesCount > 0
    res = abi.cublasLtMatmulHeuristicResult_t()
    assert api.cublasLtMatmulAlgoCheck(call.handle, call.desc, call.a_desc, call.b_desc, call.c_desc, call.d_desc,
                                       C.byref(call.heuristic[0].algo), C.byref(res)) == 0
    assert res.algo.data[0] == call.heuristic[0].algo.data[0]
    bogus = abi.cublasLtMatmulAlgo_t()
    assert api.cublasLtMatmulAlgoCheck(call.handle, call.desc, call.a_desc, call.b_desc, call.c_desc, call.d_desc,
                                       C.byref(bogus), C.byref(res)) == IV
    # requestedAlgoCount = 1 returns one
    one = abi.cublasLtMatmulHeuristicResult_t()
    cnt = C.c_int()
    assert api.cublasLtMatmulAlgoGetHeuristic(call.handle, call.desc, call.a_desc, call.b_desc, None, call.d_desc,
                                              call.pref, 1, C.byref(one), C.byref(cnt)) == 0 and cnt.value == 1
    assert api.cublasLtMatmulAlgoGetHeuristic(call.handle, call.desc, call.a_desc, call.b_desc, None, call.d_desc,
                                              call.pref, 0, C.byref(one), C.byref(cnt)) == IV
    assert api.cublasLtMatmulAlgoGetHeuristic(None, call.desc, call.a_desc, call.b_desc, None, call.d_desc,
                                              call.pref, 1, C.byref(one), C.byref(cnt)) == IV
    call.close()


def test_heuristic_rejects_inconsistent_shapes(api):
    spec = dict(m=64, n=64, k=64, a_type=abi.CUDA_R_8I, b_type=abi.CUDA_R_8I, d_type=abi.CUDA_R_32I,
                compute_type=abi.CUBLAS_COMPUTE_32I, scale_type=abi.CUDA_R_32I)
    call = MatmulCall(api, spec)
    api.layout_set(call.b_desc, abi.CUBLASLT_MATRIX_LAYOUT_ROWS, C.c_uint64, 65)
    api.layout_set(call.b_desc, abi.CUBLASLT_MATRIX_LAYOUT_LD, C.c_int64, 65)
    res, cnt = abi.cublasLtMatmulHeuristicResult_t(), C.c_int()
    assert api.cublasLtMatmulAlgoGetHeuristic(call.handle, call.desc, call.a_desc, call.b_desc, call.c_desc,
                                              call.d_desc, call.pref, 1, C.byref(res), C.byref(cnt)) == IV
    call.close()


def test_matmul_without_device_fails_loudly(api):
    """There is no CPU fallback: without a HIP device cublasLtMatmul reports NOT_INITIALIZED."""
    if api.zluda_gemm_device_cu_count() != 0:
        pytest.skip("a HIP device is present")
    spec = dict(m=64, n=64, k=64, a_type=abi.CUDA_R_8I, b_type=abi.CUDA_R_8I, d_type=abi.CUDA_R_32I,
                compute_type=abi.CUBLAS_COMPUTE_32I, scale_type=abi.CUDA_R_32I)
    call = MatmulCall(api, spec)
    buf = (C.c_char * (64 * 64 * 4))()
    one, zero = C.c_int32(1), C.c_int32(0)
    st = call.run(one, C.addressof(buf), C.addressof(buf), zero, None, C.addressof(buf))
    assert st == abi.CUBLAS_STATUS_NOT_INITIALIZED
    call.close()


def test_algorithm_enumeration_and_configuration(api):
    """cublasLtMatmulAlgoGetIds / AlgoInit / AlgoCapGetAttribute / AlgoConfig{Set,Get}Attribute
    (cuda_macros/src/cublaslt.rs:397-518): ids are kernel families, the tile variant is CUSTOM_OPTION"""
    h = C.c_void_p()
    assert api.cublasLtCreate(C.byref(h)) == 0
    ids = (C.c_int * 8)()
    n = C.c_int(0)
    i8 = (abi.CUBLAS_COMPUTE_32I, abi.CUDA_R_32I, abi.CUDA_R_8I, abi.CUDA_R_8I, abi.CUDA_R_32I, abi.CUDA_R_32I)
    assert api.cublasLtMatmulAlgoGetIds(h, *i8, 8, ids, C.byref(n)) == 0
    assert sorted(ids[:n.value]) == [abi.ZLUDA_KERNEL_GENERIC, abi.ZLUDA_KERNEL_MFMA_I8, abi.ZLUDA_KERNEL_DECODE_W8A8,
                                     abi.ZLUDA_KERNEL_MFMA_TR8]
    assert api.cublasLtMatmulAlgoGetIds(h, *i8, 1, ids, C.byref(n)) == 0 and n.value == 1
    f8 = (abi.CUBLAS_COMPUTE_32F, abi.CUDA_R_32F, abi.CUDA_R_8F_E4M3, abi.CUDA_R_8F_E4M3, abi.CUDA_R_16BF, abi.CUDA_R_16BF)
    assert api.cublasLtMatmulAlgoGetIds(h, *f8, 8, ids, C.byref(n)) == 0
    assert sorted(ids[:n.value]) == [abi.ZLUDA_KERNEL_GENERIC, abi.ZLUDA_KERNEL_MFMA_F8, abi.ZLUDA_KERNEL_DECODE_W8A8,
                                     abi.ZLUDA_KERNEL_MFMA_TR8]
    f4 = (abi.CUBLAS_COMPUTE_32F, abi.CUDA_R_32F, abi.CUDA_R_4F_E2M1, abi.CUDA_R_4F_E2M1, abi.CUDA_R_16BF, abi.CUDA_R_16BF)
    assert api.cublasLtMatmulAlgoGetIds(h, *f4, 8, ids, C.byref(n)) == 0
    assert sorted(ids[:n.value]) == [abi.ZLUDA_KERNEL_GENERIC, abi.ZLUDA_KERNEL_MFMA_MXF4]
    for t in (abi.CUDA_R_16BF, abi.CUDA_R_16F):
        h16 = (abi.CUBLAS_COMPUTE_32F, abi.CUDA_R_32F, t, t, t, t)
        assert api.cublasLtMatmulAlgoGetIds(h, *h16, 8, ids, C.byref(n)) == 0
        assert sorted(ids[:n.value]) == [abi.ZLUDA_KERNEL_GENERIC, abi.ZLUDA_KERNEL_MFMA_H16, abi.ZLUDA_KERNEL_MFMA_TR16]
    f32 = (abi.CUBLAS_COMPUTE_32F, abi.CUDA_R_32F, abi.CUDA_R_32F, abi.CUDA_R_32F, abi.CUDA_R_32F, abi.CUDA_R_32F)
    assert api.cublasLtMatmulAlgoGetIds(h, *f32, 8, ids, C.byref(n)) == 0
    assert sorted(ids[:n.value]) == [abi.ZLUDA_KERNEL_GENERIC, abi.ZLUDA_KERNEL_MFMA_F32, abi.ZLUDA_KERNEL_MFMA_TR32]
    # a combination nothing runs
    bad = (abi.CUBLAS_COMPUTE_32I, abi.CUDA_R_32I, abi.CUDA_R_32F, abi.CUDA_R_32F, abi.CUDA_R_32I, abi.CUDA_R_32I)
    assert api.cublasLtMatmulAlgoGetIds(h, *bad, 8, ids, C.byref(n)) == 0 and n.value == 0

    algo = abi.cublasLtMatmulAlgo_t()
    assert api.cublasLtMatmulAlgoInit(h, *i8, abi.ZLUDA_KERNEL_MFMA_F8, C.byref(algo)) == IV
    assert api.cublasLtMatmulAlgoInit(h, *i8, abi.ZLUDA_KERNEL_MFMA_I8, C.byref(algo)) == 0
    assert api.cublasLtMatmulAlgoInit(None, *i8, abi.ZLUDA_KERNEL_MFMA_I8, C.byref(algo)) == IV

    def get(fn, attr, ctype):
        v, w = ctype(), C.c_size_t()
        assert fn(C.byref(algo), attr, C.addressof(v), C.sizeof(v), C.byref(w)) == 0 and w.value == C.sizeof(v)
        return v.value
    assert get(api.cublasLtMatmulAlgoConfigGetAttribute, 0, C.c_int32) == abi.ZLUDA_KERNEL_MFMA_I8      # ID
    assert get(api.cublasLtMatmulAlgoConfigGetAttribute, 5, C.c_uint32) == 0                            # CUSTOM_OPTION
    assert get(api.cublasLtMatmulAlgoConfigGetAttribute, 2, C.c_int32) == 1                             # SPLITK_NUM
    nvar = get(api.cublasLtMatmulAlgoCapGetAttribute, 7, C.c_int32)                                     # CUSTOM_OPTION_MAX
    assert nvar == api.zluda_gemm_variant_count(abi.ZLUDA_KERNEL_MFMA_I8) >= 4
    assert get(api.cublasLtMatmulAlgoCapGetAttribute, 3, C.c_int32) == 1                                # STRIDED_BATCH
    assert get(api.cublasLtMatmulAlgoCapGetAttribute, 16, C.c_uint32) == 16                             # MIN_ALIGNMENT_A
    w = C.c_size_t()
    assert api.cublasLtMatmulAlgoCapGetAttribute(C.byref(algo), 15, None, 0, C.byref(w)) == 0 and w.value == 8
    assert api.cublasLtMatmulAlgoCapGetAttribute(C.byref(algo), 99, None, 0, C.byref(w)) == IV

    def put(attr, ctype, value):
        v = ctype(value)
        return api.cublasLtMatmulAlgoConfigSetAttribute(C.byref(algo), attr, C.addressof(v), C.sizeof(v))
    assert put(5, C.c_uint32, 3) == 0 and get(api.cublasLtMatmulAlgoConfigGetAttribute, 5, C.c_uint32) == 3
    assert put(5, C.c_uint32, nvar + 1) == IV
    assert put(0, C.c_int32, 3) == IV            # the id is read-only
    assert put(2, C.c_int32, 4) == NS            # no split-K
    assert put(1, C.c_uint32, 0) == 0 and put(1, C.c_uint32, 7) == NS

    # the configured token runs through AlgoCheck like a heuristic result: variant 2 of the int8 family
    spec = dict(m=4096, n=4096, k=4096, a_type=abi.CUDA_R_8I, b_type=abi.CUDA_R_8I, d_type=abi.CUDA_R_32I,
                compute_type=abi.CUBLAS_COMPUTE_32I, scale_type=abi.CUDA_R_32I, transa=abi.CUBLAS_OP_T)
    call = MatmulCall(api, spec)
    res = abi.cublasLtMatmulHeuristicResult_t()
    assert api.cublasLtMatmulAlgoCheck(call.handle, call.desc, call.a_desc, call.b_desc, call.c_desc, call.d_desc, C.byref(algo), C.byref(res)) == 0
    assert res.algo.data[1] == 2 and res.state == 0
    call.close()
    # garbage tokens are rejected
    junk = abi.cublasLtMatmulAlgo_t()
    assert api.cublasLtMatmulAlgoConfigGetAttribute(C.byref(junk), 0, None, 0, C.byref(w)) == IV
    assert api.cublasLtDestroy(h) == 0
