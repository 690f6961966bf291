"""ctypes binding of libcublaslt.so: every export by its cuBLASLt name, status codes returned as
ints, exactly what a CUDA application (or the reference's `CublasLtApi` test trait,
zluda_blas/src/tests.rs:33-84) sees.  No torch types cross this boundary: device memory is passed as
integer addresses.

A process that also uses PyTorch must import torch before loading this library: torch ships its own
libamdhip64.so.7, and the library then binds to that already-loaded HIP runtime instead of bringing
a second one into the process (two runtimes do not share a device context).

There is no CPU path behind these calls: loading fails loudly when the library has not been built,
and cublasLtMatmul returns CUBLAS_STATUS_NOT_INITIALIZED when no HIP device is usable.
"""
import ctypes as C
import os

from . import abi
from .abi import cublasLtMatmulAlgo_t, cublasLtMatmulHeuristicResult_t

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libcublaslt.so")

_vp, _u32, _u64, _i64, _sz, _int = C.c_void_p, C.c_uint32, C.c_uint64, C.c_int64, C.c_size_t, C.c_int
_pvp, _psz, _pint = C.POINTER(C.c_void_p), C.POINTER(C.c_size_t), C.POINTER(C.c_int)
_palgo, _pres = C.POINTER(cublasLtMatmulAlgo_t), C.POINTER(cublasLtMatmulHeuristicResult_t)

# name -> (restype, argtypes); the 45 exports of cuda_macros/src/cublaslt.rs:4-583
SIGNATURES = {
    "cublasLtCreate": (_u32, [_pvp]),
    "cublasLtDestroy": (_u32, [_vp]),
    "cublasLtGetStatusName": (C.c_char_p, [_u32]),
    "cublasLtGetStatusString": (C.c_char_p, [_u32]),
    "cublasLtGetVersion": (_sz, []),
    "cublasLtGetCudartVersion": (_sz, []),
    "cublasLtGetProperty": (_u32, [_u32, _pint]),
    "cublasLtHeuristicsCacheGetCapacity": (_u32, [_psz]),
    "cublasLtHeuristicsCacheSetCapacity": (_u32, [_sz]),
    "cublasLtDisableCpuInstructionsSetMask": (C.c_uint, [C.c_uint]),
    "cublasLtMatmul": (_u32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _palgo, _vp, _sz, _vp]),
    "cublasLtMatrixTransform": (_u32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "cublasLtMatrixLayoutInit_internal": (_u32, [_vp, _sz, _u32, _u64, _u64, _i64]),
    "cublasLtMatrixLayoutCreate": (_u32, [_pvp, _u32, _u64, _u64, _i64]),
    "cublasLtMatrixLayoutDestroy": (_u32, [_vp]),
    "cublasLtMatrixLayoutSetAttribute": (_u32, [_vp, _u32, _vp, _sz]),
    "cublasLtMatrixLayoutGetAttribute": (_u32, [_vp, _u32, _vp, _sz, _psz]),
    "cublasLtMatmulDescInit_internal": (_u32, [_vp, _sz, _u32, _u32]),
    "cublasLtMatmulDescCreate": (_u32, [_pvp, _u32, _u32]),
    "cublasLtMatmulDescDestroy": (_u32, [_vp]),
    "cublasLtMatmulDescSetAttribute": (_u32, [_vp, _u32, _vp, _sz]),
    "cublasLtMatmulDescGetAttribute": (_u32, [_vp, _u32, _vp, _sz, _psz]),
    "cublasLtMatrixTransformDescInit_internal": (_u32, [_vp, _sz, _u32]),
    "cublasLtMatrixTransformDescCreate": (_u32, [_pvp, _u32]),
    "cublasLtMatrixTransformDescDestroy": (_u32, [_vp]),
    "cublasLtMatrixTransformDescSetAttribute": (_u32, [_vp, _u32, _vp, _sz]),
    "cublasLtMatrixTransformDescGetAttribute": (_u32, [_vp, _u32, _vp, _sz, _psz]),
    "cublasLtMatmulPreferenceInit_internal": (_u32, [_vp, _sz]),
    "cublasLtMatmulPreferenceCreate": (_u32, [_pvp]),
    "cublasLtMatmulPreferenceDestroy": (_u32, [_vp]),
    "cublasLtMatmulPreferenceSetAttribute": (_u32, [_vp, _u32, _vp, _sz]),
    "cublasLtMatmulPreferenceGetAttribute": (_u32, [_vp, _u32, _vp, _sz, _psz]),
    "cublasLtMatmulAlgoGetHeuristic": (_u32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _pres, _pint]),
    "cublasLtMatmulAlgoGetIds": (_u32, [_vp, _u32, _u32, _u32, _u32, _u32, _u32, _int, _pint, _pint]),
    "cublasLtMatmulAlgoInit": (_u32, [_vp, _u32, _u32, _u32, _u32, _u32, _u32, _int, _palgo]),
    "cublasLtMatmulAlgoCheck": (_u32, [_vp, _vp, _vp, _vp, _vp, _vp, _palgo, _pres]),
    "cublasLtMatmulAlgoCapGetAttribute": (_u32, [_palgo, _u32, _vp, _sz, _psz]),
    "cublasLtMatmulAlgoConfigSetAttribute": (_u32, [_palgo, _u32, _vp, _sz]),
    "cublasLtMatmulAlgoConfigGetAttribute": (_u32, [_palgo, _u32, _vp, _sz, _psz]),
    "cublasLtLoggerSetCallback": (_u32, [_vp]),
    "cublasLtLoggerSetFile": (_u32, [_vp]),
    "cublasLtLoggerOpenFile": (_u32, [C.c_char_p]),
    "cublasLtLoggerSetLevel": (_u32, [_int]),
    "cublasLtLoggerSetMask": (_u32, [_int]),
    "cublasLtLoggerForceDisable": (_u32, []),
}

# the inner launch layer (include/zluda_gemm_launch.h)
LAUNCH_SIGNATURES = {
    "zluda_gemm_plan_problem": (_u32, [C.POINTER(abi.zluda_gemm_problem), _u32, C.c_int32, _u32,
                                       C.POINTER(abi.zluda_gemm_plan)]),
    "zluda_gemm_launch": (_u32, [C.POINTER(abi.zluda_gemm_problem), C.POINTER(abi.zluda_gemm_plan), _vp]),
    "zluda_gemm_launch_noalloc": (_u32, [C.POINTER(abi.zluda_gemm_problem), C.POINTER(abi.zluda_gemm_plan), _vp]),
    "zluda_gemm_variant_count": (_u32, [_u32]),
    "zluda_gemm_ex": (_u32, [_u32, _u32, C.c_int32, C.c_int32, C.c_int32, _vp, _vp, _u32, C.c_int64, _vp, _u32, C.c_int64,
                             _vp, _vp, _u32, C.c_int64, _u32, _vp]),
    "zluda_gemm_strided_batched_ex": (_u32, [_u32, _u32, C.c_int32, C.c_int32, C.c_int32, _vp, _vp, _u32, C.c_int64, C.c_int64,
                                             _vp, _u32, C.c_int64, C.c_int64, _vp, _vp, _u32, C.c_int64, C.c_int64, C.c_int32,
                                             _u32, _vp]),
    "zluda_gemm_device_cu_count": (_u32, []),
}


class CublasLtError(RuntimeError):
    def __init__(self, status, what):
        super().__init__("%s failed with cublasStatus_t %d" % (what, status))
        self.status = status


class CublasLt:
    """The loaded library.  `api.cublasLtXxx(...)` calls the export and returns its status."""

    def __init__(self, path=None):
        path = path or _LIB_PATH
        if not os.path.exists(path):
            raise FileNotFoundError(
                "%s is missing: build it first (python -m zluda_amd.build); there is no fallback path" % path)
        self.path = path
        self.lib = C.CDLL(path)
        for name, (res, args) in list(SIGNATURES.items()) + list(LAUNCH_SIGNATURES.items()):
            fn = getattr(self.lib, name)  # AttributeError = a declared export is missing
            fn.restype, fn.argtypes = res, args
            setattr(self, name, fn)

    def check(self, status, what="cublasLt call"):
        if status != abi.CUBLAS_STATUS_SUCCESS:
            raise CublasLtError(status, what)

    # -- small conveniences over SetAttribute (value packing only; no logic) -------------------
    def set_attr(self, setter, obj, attr, ctype, value):
        v = ctype(value)
        return setter(obj, attr, C.addressof(v), C.sizeof(v))

    def desc_set(self, desc, attr, ctype, value):
        return self.set_attr(self.cublasLtMatmulDescSetAttribute, desc, attr, ctype, value)

    def layout_set(self, layout, attr, ctype, value):
        return self.set_attr(self.cublasLtMatrixLayoutSetAttribute, layout, attr, ctype, value)

    def pref_set(self, pref, attr, ctype, value):
        return self.set_attr(self.cublasLtMatmulPreferenceSetAttribute, pref, attr, ctype, value)


_cached = None


def load(path=None):
    """Loads (once) and returns the library binding."""
    global _cached
    if path is not None:
        return CublasLt(path)
    if _cached is None:
        _cached = CublasLt()
    return _cached


class MatmulCall:
    """One configured cublasLtMatmul: the descriptor sequence an application issues
    (cublasLtMatmulDescCreate / SetAttribute, 4x cublasLtMatrixLayoutCreate / SetAttribute,
    cublasLtMatmulPreferenceCreate, cublasLtMatmulAlgoGetHeuristic), kept so that the call can be
    replayed.  `spec` is a plain dict:

      m, n, k, batch           sizes (batch defaults to 1)
      a_type, b_type, c_type, d_type   cudaDataType numbers (c_type defaults to d_type)
      compute_type, scale_type
      transa, transb           CUBLAS_OP_*
      order_a/b/c/d            CUBLASLT_ORDER_* (default COL)
      lda, ldb, ldc, ldd       leading dimensions in elements (default: tight)
      stride_a/b/c/d           batch strides in elements (default: tight)
      pointer_mode, epilogue, bias_type
      a_scale_mode, b_scale_mode
    Device addresses are given at run() time.
    """

    def __init__(self, api, spec, forced_kernel=None, forced_variant=-1, max_workspace=0):
        self.api, self.spec = api, dict(spec)
        s = self.spec
        m, n, k = s["m"], s["n"], s["k"]
        batch = s.get("batch", 1)
        ta, tb = s.get("transa", abi.CUBLAS_OP_N), s.get("transb", abi.CUBLAS_OP_N)
        self.handle = C.c_void_p()
        api.check(api.cublasLtCreate(C.byref(self.handle)), "cublasLtCreate")
        self.desc = C.c_void_p()
        api.check(api.cublasLtMatmulDescCreate(C.byref(self.desc), s["compute_type"], s["scale_type"]),
                  "cublasLtMatmulDescCreate")
        D = abi
        api.check(api.desc_set(self.desc, D.CUBLASLT_MATMUL_DESC_TRANSA, C.c_int32, ta), "TRANSA")
        api.check(api.desc_set(self.desc, D.CUBLASLT_MATMUL_DESC_TRANSB, C.c_int32, tb), "TRANSB")
        if "pointer_mode" in s:
            api.check(api.desc_set(self.desc, D.CUBLASLT_MATMUL_DESC_POINTER_MODE, C.c_int32, s["pointer_mode"]), "POINTER_MODE")
        if "epilogue" in s:
            api.check(api.desc_set(self.desc, D.CUBLASLT_MATMUL_DESC_EPILOGUE, C.c_uint32, s["epilogue"]), "EPILOGUE")
        if "bias_type" in s:
            api.check(api.desc_set(self.desc, D.CUBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, C.c_int32, s["bias_type"]), "BIAS_DATA_TYPE")
        if "a_scale_mode" in s:
            api.check(api.desc_set(self.desc, D.CUBLASLT_MATMUL_DESC_A_SCALE_MODE, C.c_int32, s["a_scale_mode"]), "A_SCALE_MODE")
        if "b_scale_mode" in s:
            api.check(api.desc_set(self.desc, D.CUBLASLT_MATMUL_DESC_B_SCALE_MODE, C.c_int32, s["b_scale_mode"]), "B_SCALE_MODE")
        if "bias_batch_stride" in s:
            api.check(api.desc_set(self.desc, D.CUBLASLT_MATMUL_DESC_BIAS_BATCH_STRIDE, C.c_int64, s["bias_batch_stride"]), "BIAS_BATCH_STRIDE")
        if "aux_type" in s:
            api.check(api.desc_set(self.desc, D.CUBLASLT_MATMUL_DESC_EPILOGUE_AUX_DATA_TYPE, C.c_int32, s["aux_type"]), "EPILOGUE_AUX_DATA_TYPE")
        if "aux_ld" in s:
            api.check(api.desc_set(self.desc, D.CUBLASLT_MATMUL_DESC_EPILOGUE_AUX_LD, C.c_int64, s["aux_ld"]), "EPILOGUE_AUX_LD")
        if "aux_batch_stride" in s:
            api.check(api.desc_set(self.desc, D.CUBLASLT_MATMUL_DESC_EPILOGUE_AUX_BATCH_STRIDE, C.c_int64, s["aux_batch_stride"]), "EPILOGUE_AUX_BATCH_STRIDE")
        if "alpha_vector_batch_stride" in s:
            api.check(api.desc_set(self.desc, D.CUBLASLT_MATMUL_DESC_ALPHA_VECTOR_BATCH_STRIDE, C.c_int64,
                                   s["alpha_vector_batch_stride"]), "ALPHA_VECTOR_BATCH_STRIDE")

        def layout(tag, typ, rows, cols):
            order = s.get("order_" + tag, D.CUBLASLT_ORDER_COL)
            ld = s.get("ld" + tag, rows if order == D.CUBLASLT_ORDER_COL else cols)
            h = C.c_void_p()
            api.check(api.cublasLtMatrixLayoutCreate(C.byref(h), typ, rows, cols, ld), "cublasLtMatrixLayoutCreate")
            if order != D.CUBLASLT_ORDER_COL:
                api.check(api.layout_set(h, D.CUBLASLT_MATRIX_LAYOUT_ORDER, C.c_int32, order), "ORDER")
            if batch > 1 or ("stride_" + tag) in s:
                lead = cols if order == D.CUBLASLT_ORDER_COL else rows
                stride = s.get("stride_" + tag, ld * lead)
                api.check(api.layout_set(h, D.CUBLASLT_MATRIX_LAYOUT_BATCH_COUNT, C.c_int32, batch), "BATCH_COUNT")
                api.check(api.layout_set(h, D.CUBLASLT_MATRIX_LAYOUT_STRIDED_BATCH_OFFSET, C.c_int64, stride), "STRIDED_BATCH_OFFSET")
            return h

        self.a_desc = layout("a", s["a_type"], k if ta else m, m if ta else k)
        self.b_desc = layout("b", s["b_type"], n if tb else k, k if tb else n)
        self.c_desc = layout("c", s.get("c_type", s["d_type"]), m, n)
        self.d_desc = layout("d", s["d_type"], m, n)
        self.pref = C.c_void_p()
        api.check(api.cublasLtMatmulPreferenceCreate(C.byref(self.pref)), "cublasLtMatmulPreferenceCreate")
        api.check(api.pref_set(self.pref, D.CUBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, C.c_uint64, max_workspace), "MAX_WORKSPACE_BYTES")
        self.max_workspace = max_workspace
        self.algo = None
        if forced_kernel is not None:
            self.algo = cublasLtMatmulAlgo_t()
            self.algo.data[0] = (abi.ZLUDA_ALGO_MAGIC << 32) | forced_kernel
            self.algo.data[1] = forced_variant & 0xFFFFFFFF  # -1: the planner's own variant
            self.heuristic = None
        else:
            res = (cublasLtMatmulHeuristicResult_t * 4)()
            cnt = C.c_int(0)
            api.check(api.cublasLtMatmulAlgoGetHeuristic(self.handle, self.desc, self.a_desc, self.b_desc,
                                                         self.c_desc, self.d_desc, self.pref, 4, res, C.byref(cnt)),
                      "cublasLtMatmulAlgoGetHeuristic")
            self.heuristic = [res[i] for i in range(cnt.value)]
            self.algo = self.heuristic[0].algo

    @property
    def kernel(self):
        return int(self.algo.data[0] & 0xFFFFFFFF)

    @property
    def variant(self):
        return int(self.algo.data[1] & 0xFFFFFFFF)

    def set_pointers(self, bias=None, a_scale=None, b_scale=None, c_scale=None, d_scale=None, aux=None):
        api, D = self.api, abi
        for attr, val in ((D.CUBLASLT_MATMUL_DESC_BIAS_POINTER, bias),
                          (D.CUBLASLT_MATMUL_DESC_EPILOGUE_AUX_POINTER, aux),
                          (D.CUBLASLT_MATMUL_DESC_A_SCALE_POINTER, a_scale),
                          (D.CUBLASLT_MATMUL_DESC_B_SCALE_POINTER, b_scale),
                          (D.CUBLASLT_MATMUL_DESC_C_SCALE_POINTER, c_scale),
                          (D.CUBLASLT_MATMUL_DESC_D_SCALE_POINTER, d_scale)):
            if val is not None:
                api.check(api.desc_set(self.desc, attr, C.c_void_p, val), "pointer attribute %d" % attr)

    def run(self, alpha, A, B, beta, Cptr, Dptr, workspace=None, workspace_size=0, stream=None):
        """alpha/beta: host ctypes objects (POINTER_MODE_HOST) or integer device addresses."""
        def ptr(x):
            if x is None:
                return None
            return x if isinstance(x, int) else C.addressof(x)
        return self.api.cublasLtMatmul(self.handle, self.desc, ptr(alpha), A, self.a_desc, B, self.b_desc,
                                       ptr(beta), Cptr, self.c_desc, Dptr, self.d_desc,
                                       C.byref(self.algo) if self.algo is not None else None,
                                       workspace, workspace_size, stream)

    def close(self):
        api = self.api
        for h in (self.a_desc, self.b_desc, self.c_desc, self.d_desc):
            api.cublasLtMatrixLayoutDestroy(h)
        api.cublasLtMatmulPreferenceDestroy(self.pref)
        api.cublasLtMatmulDescDestroy(self.desc)
        api.cublasLtDestroy(self.handle)
