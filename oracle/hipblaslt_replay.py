"""Replays the reference's call sequence against libhipblaslt.so.  TEST INFRASTRUCTURE ONLY.

ZLUDA's cublasLtMatmul is a 1:1 forward to hipBLASLt (zluda_blaslt/src/impl.rs:157-196), with the
enum conversions of zluda_common/src/lib.rs:575-815.  This module issues exactly that sequence
(DescCreate -> SetAttribute -> 4x MatrixLayoutCreate -> AlgoGetHeuristic(…, 1, …) -> Matmul) from the
same `spec` dict the parity tests use, so that our kernels can be compared with "ZLUDA's existing
hipBLASLt-forwarded path" on a GPU box.  Attributes the reference rejects today (scale pointers,
scale modes, pointer mode: impl.rs:274-303) are forwarded with the mapping zluda_common already
declares (lib.rs:652-678) or, for the two it lacks, with hipBLASLt's own ids.

Needs a GPU; only tests/ and bench.py import it.
"""
import ctypes as C

from zluda_amd import abi

HIPBLAS_OP = {abi.CUBLAS_OP_N: 111, abi.CUBLAS_OP_T: 112, abi.CUBLAS_OP_C: 113}   # zluda_common/src/lib.rs:751-760
HIPBLAS_COMPUTE = {abi.CUBLAS_COMPUTE_32F: 2, abi.CUBLAS_COMPUTE_32I: 9}          # lib.rs:599-630
# layout attribute ids: ext/hipblaslt-sys/src/lib.rs:262-328
L_BATCH_COUNT, L_STRIDE, L_TYPE, L_ORDER, L_ROWS, L_COLS, L_LD = 0, 1, 2, 3, 4, 5, 6
# matmul desc attribute ids: ext/hipblaslt-sys/src/lib.rs:351-440 (+ 31/32 from the installed header)
D_TRANSA, D_TRANSB, D_EPILOGUE, D_BIAS_POINTER, D_BIAS_DATA_TYPE = 0, 1, 2, 3, 4
D_A_SCALE_POINTER, D_B_SCALE_POINTER, D_C_SCALE_POINTER, D_D_SCALE_POINTER = 5, 6, 7, 8
D_AUX_POINTER, D_AUX_LD, D_AUX_BATCH_STRIDE = 10, 11, 12
D_POINTER_MODE, D_A_SCALE_MODE, D_B_SCALE_MODE = 13, 31, 32
P_MAX_WORKSPACE = 1


class hipblasLtMatmulAlgo_t(C.Structure):
    _fields_ = [("data", C.c_uint8 * 16), ("max_workspace_bytes", C.c_size_t)]


class hipblasLtMatmulHeuristicResult_t(C.Structure):   # ext/hipblaslt-sys/src/lib.rs:634-671
    _fields_ = [("algo", hipblasLtMatmulAlgo_t), ("workspaceSize", C.c_size_t), ("state", C.c_int),
                ("wavesCount", C.c_float), ("reserved", C.c_int * 4)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        L = C.CDLL("libhipblaslt.so")
        vp, u32, sz = C.c_void_p, C.c_uint32, C.c_size_t
        sigs = {
            "hipblasLtCreate": [C.POINTER(vp)], "hipblasLtDestroy": [vp],
            "hipblasLtMatmulDescCreate": [C.POINTER(vp), u32, u32], "hipblasLtMatmulDescDestroy": [vp],
            "hipblasLtMatmulDescSetAttribute": [vp, u32, vp, sz],
            "hipblasLtMatrixLayoutCreate": [C.POINTER(vp), u32, C.c_uint64, C.c_uint64, C.c_int64],
            "hipblasLtMatrixLayoutDestroy": [vp], "hipblasLtMatrixLayoutSetAttribute": [vp, u32, vp, sz],
            "hipblasLtMatmulPreferenceCreate": [C.POINTER(vp)], "hipblasLtMatmulPreferenceDestroy": [vp],
            "hipblasLtMatmulPreferenceSetAttribute": [vp, u32, vp, sz],
            "hipblasLtMatmulAlgoGetHeuristic": [vp, vp, vp, vp, vp, vp, vp, C.c_int,
                                                C.POINTER(hipblasLtMatmulHeuristicResult_t), C.POINTER(C.c_int)],
            "hipblasLtMatmul": [vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, C.POINTER(hipblasLtMatmulAlgo_t), vp, sz, vp],
        }
        for name, args in sigs.items():
            f = getattr(L, name)
            f.restype, f.argtypes = C.c_int, args
        _lib = L
    return _lib


class Replay:
    """hipBLASLt configured from a MatmulCall-style spec.  `ok` is False when the heuristic returns
    no algorithm (the comparison point then does not exist for this configuration)."""

    def __init__(self, spec, workspace_bytes=64 << 20):
        import torch
        L = lib()
        s = dict(spec)
        self.spec = s
        m, n, k = s["m"], s["n"], s["k"]
        batch = s.get("batch", 1)
        ta, tb = s.get("transa", 0), s.get("transb", 0)
        self.handle, self.desc, self.pref = C.c_void_p(), C.c_void_p(), C.c_void_p()
        self.layouts = []
        self.ok, self.why = False, ""
        st = L.hipblasLtCreate(C.byref(self.handle))
        if st:
            self.why = "hipblasLtCreate=%d" % st
            return
        if s["compute_type"] not in HIPBLAS_COMPUTE:
            self.why = "compute type not mapped"
            return
        st = L.hipblasLtMatmulDescCreate(C.byref(self.desc), HIPBLAS_COMPUTE[s["compute_type"]], s["scale_type"])
        if st:
            self.why = "hipblasLtMatmulDescCreate=%d" % st
            return

        def dset(attr, ctype, val):
            v = ctype(val)
            r = L.hipblasLtMatmulDescSetAttribute(self.desc, attr, C.addressof(v), C.sizeof(v))
            if r:
                self.why += " desc attr %d -> %d;" % (attr, r)
            return r
        self._dset = dset
        bad = dset(D_TRANSA, C.c_int32, HIPBLAS_OP[ta]) | dset(D_TRANSB, C.c_int32, HIPBLAS_OP[tb])
        if "epilogue" in s:
            bad |= dset(D_EPILOGUE, C.c_uint32, s["epilogue"])
        if "bias_type" in s:
            bad |= dset(D_BIAS_DATA_TYPE, C.c_int32, s["bias_type"])
        if "pointer_mode" in s:
            pm = s["pointer_mode"]
            if pm == abi.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO:
                pm = abi.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_HOST   # hipBLASLt only has the BETA_HOST form
            bad |= dset(D_POINTER_MODE, C.c_int32, pm)
        if "aux_ld" in s:
            bad |= dset(D_AUX_LD, C.c_int64, s["aux_ld"])
            bad |= dset(D_AUX_BATCH_STRIDE, C.c_int64, s.get("aux_batch_stride", 0))
        if "a_scale_mode" in s:
            bad |= dset(D_A_SCALE_MODE, C.c_int32, s["a_scale_mode"])
        if "b_scale_mode" in s:
            bad |= dset(D_B_SCALE_MODE, C.c_int32, s["b_scale_mode"])
        if bad:
            return

        def layout(tag, typ, rows, cols):
            order = s.get("order_" + tag, 0)
            ld = s.get("ld" + tag, rows if order == 0 else cols)
            h = C.c_void_p()
            r = L.hipblasLtMatrixLayoutCreate(C.byref(h), typ, rows, cols, ld)
            if r:
                self.why += " layout %s -> %d;" % (tag, r)
                return None
            self.layouts.append(h)

            def lset(attr, ctype, val):
                v = ctype(val)
                return L.hipblasLtMatrixLayoutSetAttribute(h, attr, C.addressof(v), C.sizeof(v))
            if order != 0 and lset(L_ORDER, C.c_int32, order):
                self.why += " layout order;"
                return None
            if batch > 1:
                lead = cols if order == 0 else rows
                if lset(L_BATCH_COUNT, C.c_int32, batch) or lset(L_STRIDE, C.c_int64, s.get("stride_" + tag, ld * lead)):
                    self.why += " layout batch;"
                    return None
            return h
        self.a = layout("a", s["a_type"], k if ta else m, m if ta else k)
        self.b = layout("b", s["b_type"], n if tb else k, k if tb else n)
        self.c = layout("c", s.get("c_type", s["d_type"]), m, n)
        self.d = layout("d", s["d_type"], m, n)
        if None in (self.a, self.b, self.c, self.d):
            return
        L.hipblasLtMatmulPreferenceCreate(C.byref(self.pref))
        ws = C.c_uint64(workspace_bytes)
        L.hipblasLtMatmulPreferenceSetAttribute(self.pref, P_MAX_WORKSPACE, C.addressof(ws), 8)
        self.workspace = torch.empty(workspace_bytes, dtype=torch.uint8, device="cuda:0")
        self.workspace_bytes = workspace_bytes
        self.res = hipblasLtMatmulHeuristicResult_t()
        self._pointers_set = False

    def set_pointers(self, bias=None, a_scale=None, b_scale=None, c_scale=None, d_scale=None, aux=None):
        for attr, val in ((D_BIAS_POINTER, bias), (D_AUX_POINTER, aux), (D_A_SCALE_POINTER, a_scale), (D_B_SCALE_POINTER, b_scale),
                          (D_C_SCALE_POINTER, c_scale), (D_D_SCALE_POINTER, d_scale)):
            if val is not None and self._dset(attr, C.c_void_p, val):
                return False
        return True

    def find_algo(self):
        """the reference asks for requestedAlgoCount algorithms and uses the first (impl.rs:198-241)"""
        cnt = C.c_int(0)
        st = lib().hipblasLtMatmulAlgoGetHeuristic(self.handle, self.desc, self.a, self.b, self.c, self.d, self.pref,
                                                   1, C.byref(self.res), C.byref(cnt))
        self.ok = st == 0 and cnt.value >= 1
        if not self.ok:
            self.why += " heuristic status %d, %d algorithms" % (st, cnt.value)
        return self.ok

    def run(self, alpha, A, B, beta, Cptr, Dptr, stream=None):
        def ptr(x):
            return x if (x is None or isinstance(x, int)) else C.addressof(x)
        return lib().hipblasLtMatmul(self.handle, self.desc, ptr(alpha), A, self.a, B, self.b, ptr(beta),
                                     Cptr if Cptr is not None else Dptr, self.c, Dptr, self.d,
                                     C.byref(self.res.algo), self.workspace.data_ptr(), self.workspace_bytes, stream)

    def close(self):
        L = lib()
        for h in self.layouts:
            L.hipblasLtMatrixLayoutDestroy(h)
        if self.pref:
            L.hipblasLtMatmulPreferenceDestroy(self.pref)
        if self.desc:
            L.hipblasLtMatmulDescDestroy(self.desc)
        if self.handle:
            L.hipblasLtDestroy(self.handle)
