"""Loader of the CPU checker (oracle/ref_gemm.c).  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this package; nothing
under zluda_amd/ does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

from zluda_amd import abi

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "liboracle_gemm.so")


def build(force=False):
    cmd = ["make", "-C", HERE] + (["-B"] if force else [])
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode:
        raise RuntimeError("building the oracle failed:\n" + res.stdout)
    return LIB


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            build()
        L = C.CDLL(LIB)
        L.oracle_gemm.restype = C.c_uint32
        L.oracle_gemm.argtypes = [C.POINTER(abi.zluda_gemm_problem)]
        for name in ("e4m3", "e5m2", "e2m1", "ue8m0"):
            f = getattr(L, "oracle_decode_" + name)
            f.restype, f.argtypes = C.c_float, [C.c_uint8]
        for name in ("e4m3", "e5m2", "e2m1"):
            f = getattr(L, "oracle_encode_" + name)
            f.restype, f.argtypes = C.c_uint8, [C.c_float]
        L.oracle_encode_bf16.restype, L.oracle_encode_bf16.argtypes = C.c_uint16, [C.c_float]
        L.oracle_decode_bf16.restype, L.oracle_decode_bf16.argtypes = C.c_float, [C.c_uint16]
        L.oracle_encode_f16.restype, L.oracle_encode_f16.argtypes = C.c_uint16, [C.c_float]
        L.oracle_decode_f16.restype, L.oracle_decode_f16.argtypes = C.c_float, [C.c_uint16]
        L.oracle_gelu.restype, L.oracle_gelu.argtypes = C.c_float, [C.c_float]
        L.oracle_dgelu.restype, L.oracle_dgelu.argtypes = C.c_float, [C.c_float]
        for name in ("oracle_encode_e4m3_array", "oracle_encode_e5m2_array", "oracle_encode_bf16_array",
                     "oracle_decode_bf16_array", "oracle_encode_f16_array"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.oracle_quantize_mxfp4.restype = None
        L.oracle_quantize_mxfp4.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t]
        _lib = L
    return _lib


def _arr(fn, x, in_dtype, out_dtype):
    x = np.ascontiguousarray(x, dtype=in_dtype)
    y = np.empty(x.shape, dtype=out_dtype)
    fn(x.ctypes.data, y.ctypes.data, x.size)
    return y


def encode_e4m3(x):
    return _arr(lib().oracle_encode_e4m3_array, x, np.float32, np.uint8)


def encode_e5m2(x):
    return _arr(lib().oracle_encode_e5m2_array, x, np.float32, np.uint8)


def encode_bf16(x):
    return _arr(lib().oracle_encode_bf16_array, x, np.float32, np.uint16)


def decode_bf16(x):
    return _arr(lib().oracle_decode_bf16_array, x, np.uint16, np.float32)


def encode_f16(x):
    return _arr(lib().oracle_encode_f16_array, x, np.float32, np.uint16)


def quantize_mxfp4(x):
    """x: [rows, k] float32 -> (packed uint8 [rows, k/2], scales uint8 [rows, k/32])."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, k = x.shape
    q = np.empty((rows, k // 2), np.uint8)
    s = np.empty((rows, k // 32), np.uint8)
    lib().oracle_quantize_mxfp4(x.ctypes.data, q.ctypes.data, s.ctypes.data, rows, k)
    return q, s


def decode_table(name):
    """All codes of an 8-bit (or 4-bit) format as float32."""
    f = getattr(lib(), "oracle_decode_" + name)
    n = 16 if name == "e2m1" else 256
    return np.array([f(i) for i in range(n)], dtype=np.float32)


def gemm(problem):
    """Runs the CPU restatement on a zluda_gemm_problem whose pointers are all host pointers."""
    return lib().oracle_gemm(C.byref(problem))
