"""cublasLtMatmul under HIP graph capture: the launch layer only enqueues kernels (no allocation, no
memset, no synchronisation), so a serving loop can record its GEMMs once and replay them.  Five
calls of different kernel families -- including a split-K call, which is two kernels through the
caller's workspace, and a GELU_AUX_BIAS call, which is a GEMM kernel and an element-wise pass -- are
captured into one graph; it is replayed several times with fresh operand
contents between the replays, and every replay is checked against the CPU oracle."""
import numpy as np
import pytest

from oracle.cases import Case
from zluda_amd import abi
from zluda_amd.cublaslt import MatmulCall

pytestmark = pytest.mark.gpu
K = abi

I8 = dict(a_type=K.CUDA_R_8I, b_type=K.CUDA_R_8I, c_type=K.CUDA_R_32I, d_type=K.CUDA_R_32I,
          compute_type=K.CUBLAS_COMPUTE_32I, scale_type=K.CUDA_R_32I)
SPECS = [
    (dict(I8, transa=1, m=1024, n=256, k=8192), 64 << 20, K.ZLUDA_KERNEL_MFMA_I8),          # split-K + reduce kernel
    (dict(I8, transa=0, transb=1, m=300, n=212, k=272, lda=304, ldb=216), 0, K.ZLUDA_KERNEL_MFMA_TR8),
    (dict(I8, transa=1, c_type=K.CUDA_R_16BF, d_type=K.CUDA_R_16BF, scale_type=K.CUDA_R_32F, m=2048, n=16, k=4096,
          pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO,
          b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F, epilogue=K.CUBLASLT_EPILOGUE_BIAS,
          bias_type=K.CUDA_R_32F, alpha_range=(0.001, 0.01), scale_range=(0.005, 0.02), bias_std=0.02), 0,
     K.ZLUDA_KERNEL_DECODE_W8A8),
    # 24 tokens, K = 8192: the 8-wave slab shape with two token blocks
    (dict(I8, transa=1, c_type=K.CUDA_R_16BF, d_type=K.CUDA_R_16BF, scale_type=K.CUDA_R_32F, m=1000, n=24, k=8192,
          epilogue=K.CUBLASLT_EPILOGUE_RELU_BIAS, alpha_range=(0.0005, 0.001)), 0, K.ZLUDA_KERNEL_DECODE_W8A8),
    # GELU input kept: GEMM kernel into the aux matrix, then the element-wise pass into D
    (dict(a_type=K.CUDA_R_8F_E4M3, b_type=K.CUDA_R_8F_E4M3, c_type=K.CUDA_R_16F, d_type=K.CUDA_R_16F, compute_type=K.CUBLAS_COMPUTE_32F,
          scale_type=K.CUDA_R_32F, transa=1, m=384, n=264, k=512, epilogue=K.CUBLASLT_EPILOGUE_GELU_AUX_BIAS, aux_ld=400,
          with_scalar_scales=True, scale_range=(0.05, 0.06)), 0, K.ZLUDA_KERNEL_MFMA_F8),
]


def test_kernel_families_in_one_graph(gpu_api):
    import torch
    print("graph capture of", [s for s, _, _ in SPECS], flush=True)
    cases, calls, bufs = [], [], []
    for i, (spec, ws_bytes, want) in enumerate(SPECS):
        case = Case(spec, 500 + i, int_dist="normal" if want == K.ZLUDA_KERNEL_DECODE_W8A8 else "uniform")
        keep, ptr, dt = case.upload()
        call = MatmulCall(gpu_api, case.spec, max_workspace=ws_bytes)
        assert call.kernel == want
        call.set_pointers(bias=ptr["bias"], a_scale=ptr["a_scale"], b_scale=ptr["b_scale"],
                          c_scale=ptr["c_scale"], d_scale=ptr["d_scale"], aux=ptr["aux"])
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device="cuda:0")
        cases.append(case); calls.append(call); bufs.append((keep, ptr, dt, ws, ws_bytes))

    def enqueue(stream):
        for case, call, (keep, ptr, dt, ws, ws_bytes) in zip(cases, calls, bufs):
            alpha, beta = case.scalars(ptr)
            st = call.run(alpha, ptr["A"], ptr["B"], beta, ptr["C"], ptr["D"],
                          ws.data_ptr() if ws_bytes else None, ws_bytes, stream)
            assert st == 0, "cublasLtMatmul status %d" % st

    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        enqueue(side.cuda_stream)              # warm-up outside the capture (lazy module loading)
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            enqueue(torch.cuda.current_stream().cuda_stream)
    try:
        for replay in range(3):
            # fresh contents in the same buffers: A of every case is redrawn, D gets its canary back
            for i, (case, (keep, ptr, dt, ws, ws_bytes)) in enumerate(zip(cases, bufs)):
                fresh = Case(case.spec, 600 + 10 * replay + i,
                             int_dist="normal" if SPECS[i][2] == K.ZLUDA_KERNEL_DECODE_W8A8 else "uniform")
                case.A = fresh.A
                raw = np.frombuffer(case.A.tobytes(), dtype=np.uint8)
                keep[0][:raw.size] = torch.from_numpy(raw.copy()).to("cuda:0")
                canary = np.frombuffer(case.new_d().tobytes(), dtype=np.uint8)
                dt[:canary.size] = torch.from_numpy(canary.copy()).to("cuda:0")
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            for case, (keep, ptr, dt, ws, ws_bytes) in zip(cases, bufs):
                case.compare(case.download(dt), case.run_oracle())
                if case.aux_mode == 1:
                    case.compare_aux(keep[10][:case.aux.nbytes].cpu().numpy().view(case.aux.dtype).copy(), case.aux_ref)
    finally:
        for call in calls:
            call.close()
