"""zluda_gemm_launch_noalloc (include/zluda_gemm_launch.h): the launch entry point whose split-K scratch is an
array inside the library image.  Called through the C ABI and compared with zluda_gemm_launch running the
same plan with a caller-provided workspace: the same kernels run with the same split, so the outputs must be
bit-identical, for integer and for float problems.  Two calls in a row share the array; the second problem is
smaller, so stale partial tiles of the first call lie beside (and beyond) the ones it uses."""
import ctypes as C

import numpy as np
import pytest

from oracle.cases import Case
from zluda_amd import abi

pytestmark = pytest.mark.gpu
K = abi
SCRATCH = 32 << 20   # ZLUDA_GEMM_STATIC_SCRATCH_BYTES

I8 = dict(a_type=K.CUDA_R_8I, b_type=K.CUDA_R_8I, c_type=K.CUDA_R_32I, d_type=K.CUDA_R_32I,
          compute_type=K.CUBLAS_COMPUTE_32I, scale_type=K.CUDA_R_32I, transa=1, alpha=1)
F8 = dict(a_type=K.CUDA_R_8F_E4M3, b_type=K.CUDA_R_8F_E4M3, c_type=K.CUDA_R_16BF, d_type=K.CUDA_R_16BF,
          compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F, transa=1, alpha=1.0,
          epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS, bias_type=K.CUDA_R_16BF, with_scalar_scales=True)


def run_both(api, spec, seed, kernel):
    """returns (D through zluda_gemm_launch_noalloc, D through zluda_gemm_launch + workspace, plan)"""
    import torch
    case = Case(spec, seed)
    stream = torch.cuda.current_stream().cuda_stream
    outs = []
    plan_used = None
    for noalloc in (True, False):
        keep, ptr, dt = case.upload()
        ptrs = dict(ptr)
        ptrs["alpha"], ptrs["beta"] = case.alpha.ctypes.data, case.beta.ctypes.data
        p = case.problem(ptrs)
        p.workspace_size = SCRATCH
        plan = abi.zluda_gemm_plan()
        assert api.zluda_gemm_plan_problem(C.byref(p), kernel, -1, api.zluda_gemm_device_cu_count(), C.byref(plan)) == 0
        assert plan.grid_z > 1 and 0 < plan.workspace <= SCRATCH, "the case is meant to split K"
        if noalloc:
            p.workspace = None
            st = api.zluda_gemm_launch_noalloc(C.byref(p), C.byref(plan), stream)
        else:
            ws = torch.empty(plan.workspace, dtype=torch.uint8, device="cuda:0")
            p.workspace, p.workspace_size = ws.data_ptr(), plan.workspace
            st = api.zluda_gemm_launch(C.byref(p), C.byref(plan), stream)
        torch.cuda.synchronize()
        assert st == 0, "status %d" % st
        outs.append(case.download(dt))
        plan_used = plan
    return case, outs[0], outs[1], plan_used


def test_noalloc_matches_the_workspace_entry_point_twice_in_a_row(gpu_api):
    # first call: 8 splits of a 256 x 256 x 16384 int8 problem; second, smaller: fewer tiles, shorter K
    for spec, seed, kernel in ((dict(I8, m=256, n=256, k=16384), 701, K.ZLUDA_KERNEL_MFMA_I8),
                               (dict(I8, m=128, n=64, k=8192), 702, K.ZLUDA_KERNEL_MFMA_I8),
                               (dict(F8, m=512, n=48, k=8192), 703, K.ZLUDA_KERNEL_MFMA_F8),
                               (dict(F8, m=64, n=16, k=4096), 704, K.ZLUDA_KERNEL_MFMA_F8),
                               (dict(I8, transa=0, transb=1, m=256, n=128, k=4096), 705, K.ZLUDA_KERNEL_MFMA_TR8)):
        print("no-alloc case", spec, flush=True)
        case, got, want, plan = run_both(gpu_api, spec, seed, kernel)
        assert np.array_equal(got, want), "grid_z %d: the two entry points disagree" % plan.grid_z
        case.compare(got, case.run_oracle())


def test_noalloc_rejects_a_plan_beyond_the_scratch(gpu_api):
    import torch
    spec = dict(I8, m=256, n=256, k=16384)
    case = Case(spec, 706)
    keep, ptr, dt = case.upload()
    ptrs = dict(ptr)
    ptrs["alpha"], ptrs["beta"] = case.alpha.ctypes.data, case.beta.ctypes.data
    p = case.problem(ptrs)
    p.workspace_size = SCRATCH
    plan = abi.zluda_gemm_plan()
    assert gpu_api.zluda_gemm_plan_problem(C.byref(p), K.ZLUDA_KERNEL_MFMA_I8, -1, gpu_api.zluda_gemm_device_cu_count(), C.byref(plan)) == 0
    plan.workspace = SCRATCH + 1     # as if planned against a larger workspace
    st = gpu_api.zluda_gemm_launch_noalloc(C.byref(p), C.byref(plan), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert st == K.CUBLAS_STATUS_ALLOC_FAILED
    assert bool((dt[case._guard:case._guard + 64] == 0xCD).all()), "nothing may have been launched"


def test_noalloc_under_graph_capture_after_a_warm_up_call(gpu_api):
    """the entry point is for callers that record their GEMMs into a HIP graph: after one call outside the capture
    (which looks up the scratch array) a split-K call is captured and replayed three times with fresh operands in
    between, every replay against the workspace entry point's result for the same operands"""
    import torch
    spec = dict(I8, m=256, n=256, k=16384)
    case = Case(spec, 710)
    keep, ptr, dt = case.upload()
    ptrs = dict(ptr)
    ptrs["alpha"], ptrs["beta"] = case.alpha.ctypes.data, case.beta.ctypes.data
    p = case.problem(ptrs)
    p.workspace_size = SCRATCH
    plan = abi.zluda_gemm_plan()
    assert gpu_api.zluda_gemm_plan_problem(C.byref(p), K.ZLUDA_KERNEL_MFMA_I8, -1, gpu_api.zluda_gemm_device_cu_count(), C.byref(plan)) == 0
    assert plan.grid_z > 1
    p.workspace = None
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        assert gpu_api.zluda_gemm_launch_noalloc(C.byref(p), C.byref(plan), side.cuda_stream) == 0   # the warm-up call
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            assert gpu_api.zluda_gemm_launch_noalloc(C.byref(p), C.byref(plan), torch.cuda.current_stream().cuda_stream) == 0
    ws = torch.empty(plan.workspace, dtype=torch.uint8, device="cuda:0")
    for replay in range(3):
        fresh = Case(spec, 720 + replay)
        case.A = fresh.A
        raw = np.frombuffer(case.A.tobytes(), dtype=np.uint8)
        keep[0][:raw.size] = torch.from_numpy(raw.copy()).to("cuda:0")
        canary = np.frombuffer(case.new_d().tobytes(), dtype=np.uint8)
        dt[:canary.size] = torch.from_numpy(canary.copy()).to("cuda:0")
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = case.download(dt)
        dt[:canary.size] = torch.from_numpy(canary.copy()).to("cuda:0")
        p.workspace, p.workspace_size = ws.data_ptr(), plan.workspace
        assert gpu_api.zluda_gemm_launch(C.byref(p), C.byref(plan), torch.cuda.current_stream().cuda_stream) == 0
        torch.cuda.synchronize()
        p.workspace, p.workspace_size = None, SCRATCH
        assert np.array_equal(got, case.download(dt)), "replay %d" % replay
        case.compare(got, case.run_oracle())
