"""Concurrent use of the library from several host threads, each on its own stream with its own
handle and descriptors (the reference's contract: no global lock, lazily initialised backend, handles
and descriptors Send + Sync -- zluda_blaslt/src/impl.rs:7-12, 34-38).  Every result is compared with
the CPU oracle, so a race in the lazily built state (device properties, kernel modules) or a launch
on the wrong stream shows up as a mismatch."""
import threading

import pytest

from oracle.cases import Case
from zluda_amd import abi

pytestmark = pytest.mark.gpu
K = abi

I8 = dict(a_type=K.CUDA_R_8I, b_type=K.CUDA_R_8I, d_type=K.CUDA_R_32I, compute_type=K.CUBLAS_COMPUTE_32I,
          scale_type=K.CUDA_R_32I)
F8 = dict(a_type=K.CUDA_R_8F_E4M3, b_type=K.CUDA_R_8F_E4M3, d_type=K.CUDA_R_16BF, compute_type=K.CUBLAS_COMPUTE_32F,
          scale_type=K.CUDA_R_32F, transa=1)
SPECS = [
    dict(I8, transa=1, m=512, n=384, k=1024),                                       # LDS-DMA MFMA kernel
    dict(I8, transa=0, transb=1, m=300, n=212, k=272, lda=304, ldb=216),            # transposing MFMA kernel
    dict(I8, transa=1, d_type=K.CUDA_R_16BF, scale_type=K.CUDA_R_32F, m=2048, n=16, k=4096,
         pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO,
         b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F, epilogue=K.CUBLASLT_EPILOGUE_BIAS,
         bias_type=K.CUDA_R_32F, alpha_range=(0.001, 0.01), scale_range=(0.005, 0.02), bias_std=0.02),   # decode
    dict(F8, m=320, n=272, k=400, lda=416, ldb=400, epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS, with_scalar_scales=True),
    dict(I8, transa=1, m=96, n=80, k=72, lda=72, ldb=72),                           # generic kernel (K % 16 != 0)
]


def test_four_threads_four_streams(gpu_api):
    import torch
    cases = [Case(spec, 400 + i) for i, spec in enumerate(SPECS)]
    refs = [c.run_oracle() for c in cases]
    failures = []

    def worker(tid):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for it in range(6):
                    for j in range(len(cases)):
                        i = (j + tid) % len(cases)          # threads run different kernels at the same time
                        case = Case(SPECS[i], 400 + i)      # own buffers per call
                        st, got, kern, _ = case.run_gpu(gpu_api)
                        if st != 0:
                            failures.append("thread %d case %d: status %d" % (tid, i, st))
                            return
                        try:
                            case.compare(got, refs[i])
                        except AssertionError as e:
                            failures.append("thread %d iteration %d case %d kernel %d: %s" % (tid, it, i, kern, e))
                            return
        except Exception as e:  # noqa: BLE001 - reported through the list, the test fails below
            failures.append("thread %d: %s: %s" % (tid, type(e).__name__, e))

    print("concurrency: 4 threads x 6 rounds x %d cases" % len(cases), flush=True)
    threads = [threading.Thread(target=worker, args=(t,)) for t in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "a worker thread did not finish"
    assert not failures, "\n".join(failures)
