"""MI355X-native cublasLtMatmul for ZLUDA's quantized dense-GEMM path.

The product is the shared library zluda_amd/lib/libcublaslt.so (C ABI: include/cublaslt_abi.h).
This package only builds it (zluda_amd.build) and binds it with ctypes (zluda_amd.cublaslt) the
way the reference's test trait `CublasLtApi` does (zluda_blas/src/tests.rs:33-84).
"""
from . import abi  # noqa: F401
from .cublaslt import CublasLt, CublasLtError, load  # noqa: F401
