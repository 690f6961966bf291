#!/usr/bin/env python3
"""Benchmark of the cublasLtMatmul hot path on one MI355X.

A "step" is one cublasLtMatmul call (through the exported C ABI of zluda_amd/lib/libcublaslt.so) on
synthetic inputs that are already resident in HBM.  The headline line reports benchmark configuration 4
(fp8 e4m3, M=N=K=8192, per-tensor scales, bf16 bias + GELU, bf16 D): the 8192^3 size the metric is quoted
on.  The other benchmark configurations, the 8192^3 int8 case and configuration 5's problem at batch 1
ride along under "also", each with its own roofline figures and, when the installed hipBLASLt has a
solution, the time of the reference's hipBLASLt-forwarded path on the same buffers.

Timing: first an untimed stretch of calls of `--settle` seconds (default 0.5: the power management needs a few
hundred milliseconds of load to settle, and what a burst shows before that is up to 15 % off what a running job
sees), then W warm-up calls, then exactly K calls between two synchronisations (wall clock -> `value`); HIP
events on the launch stream split the K calls into five batches, and `roofline.kernel_ms` is the median
batch.  A one-wave probe kernel on a second stream samples the shader cycle counter against the real-time
counter during one more (untimed) batch: `clock_mhz_observed`, and `frac_at_observed_clock` = the
roofline fraction against the datasheet peak scaled to that clock (the peak assumes 2400 MHz).

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--settle SECONDS] [--workload c1|c2|c3|c4|c5|c5_b1|i8_8192|...] [--only]
                  [--also LIST] [--no-cpu] [--no-hipblaslt] [--copy-probe] [--sustained SECONDS] [--full]

The line the script prints stays under 8 KB: the headline's figures, then under "also" one compact entry per other
workload in the order the metric names them (decode, int8 8192^3, MXFP4, ...).  `roofline.vs_hipblaslt` is the
headline's rate over the hipBLASLt-forwarded path's on the same buffers, `roofline.decode_c3` the decode half of the
metric.  --full prints every workload's whole record instead (for profiles/ and notes).
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import numpy as np  # noqa: E402,F401
import torch  # noqa: E402  -- before libcublaslt.so: one HIP runtime (torch's libamdhip64.so.7) per process

from zluda_amd import abi, cublaslt  # noqa: E402
from zluda_amd.cublaslt import MatmulCall  # noqa: E402

K = abi
PEAK = {"i8": 5000.0, "f8": 5000.0, "f4": 10100.0, "bf16": 2500.0, "hbm": 8000.0}  # TOP/s, TFLOP/s, GB/s (MI355X datasheet)
PEAK_CLOCK_MHZ = 2400.0   # the shader clock the datasheet's matrix peaks are quoted at

I8 = dict(a_type=K.CUDA_R_8I, b_type=K.CUDA_R_8I, d_type=K.CUDA_R_32I, compute_type=K.CUBLAS_COMPUTE_32I,
          scale_type=K.CUDA_R_32I, transa=1)
WORKLOADS = {
    "c1": dict(name="int8xint8->int32 M=N=K=256 A:N B:T (benchmark configuration 1)", kind="i8",
               spec=dict(I8, m=256, n=256, k=256, transa=0, transb=1), steps=200),
    "c2": dict(name="int8xint8->int32 M=N=K=4096 A:T B:N (benchmark configuration 2)", kind="i8",
               spec=dict(I8, m=4096, n=4096, k=4096), steps=50),
    "i8_4096_nt": dict(name="int8xint8->int32 M=N=K=4096 A:N B:T (config 1's layout at config 2's size)", kind="i8",
                       spec=dict(I8, m=4096, n=4096, k=4096, transa=0, transb=1), steps=50),
    "i8_8192": dict(name="int8xint8->int32 M=N=K=8192 A:T B:N", kind="i8", spec=dict(I8, m=8192, n=8192, k=8192), steps=25),
    "c3": dict(name="W8A8 decode M=14336 N=16 K=4096 alpha-vec + per-token scale + fp32 bias -> bf16 (benchmark configuration 3)",
               kind="hbm", steps=200,
               spec=dict(I8, d_type=K.CUDA_R_16BF, scale_type=K.CUDA_R_32F, m=14336, n=16, k=4096,
                         pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO,
                         b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F,
                         epilogue=K.CUBLASLT_EPILOGUE_BIAS, bias_type=K.CUDA_R_32F)),
    "decode_k13824": dict(name="W8A8 decode M=5120 N=16 K=13824 alpha-vec + per-token scale + fp32 bias -> bf16 (configuration 3's "
                               "problem at a down-projection shape: few rows, long K)", kind="hbm", steps=200,
                          spec=dict(I8, d_type=K.CUDA_R_16BF, scale_type=K.CUDA_R_32F, m=5120, n=16, k=13824,
                                    pointer_mode=K.CUBLASLT_POINTER_MODE_ALPHA_DEVICE_VECTOR_BETA_ZERO,
                                    b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F,
                                    epilogue=K.CUBLASLT_EPILOGUE_BIAS, bias_type=K.CUDA_R_32F)),
    "c4": dict(name="fp8 e4m3 M=N=K=8192 per-tensor scales, bf16 bias + GELU -> bf16 (benchmark configuration 4)", kind="f8",
               steps=50,
               spec=dict(a_type=K.CUDA_R_8F_E4M3, b_type=K.CUDA_R_8F_E4M3, d_type=K.CUDA_R_16BF,
                         compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F, transa=1, m=8192, n=8192, k=8192,
                         epilogue=K.CUBLASLT_EPILOGUE_GELU_BIAS, bias_type=K.CUDA_R_16BF)),
    "c5": dict(name="MXFP4 (E2M1 + UE8M0/32) M=N=K=8192 batch 4 -> bf16 (benchmark configuration 5)", kind="f4", steps=10,
               spec=dict(a_type=K.CUDA_R_4F_E2M1, b_type=K.CUDA_R_4F_E2M1, d_type=K.CUDA_R_16BF,
                         compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F, transa=1, m=8192, n=8192, k=8192,
                         batch=4, a_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0,
                         b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0)),
    "c5_b1": dict(name="MXFP4 (E2M1 + UE8M0/32) M=N=K=8192 batch 1 -> bf16 (configuration 5's problem at the one batch "
                       "count the installed hipBLASLt takes)", kind="f4", steps=10,
                  spec=dict(a_type=K.CUDA_R_4F_E2M1, b_type=K.CUDA_R_4F_E2M1, d_type=K.CUDA_R_16BF,
                            compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F, transa=1, m=8192, n=8192, k=8192,
                            a_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0,
                            b_scale_mode=K.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0)),
    # not a benchmark configuration: the 16-bit operand type applications call cublasLtMatmul with most, on the same kernels
    "bf16_8192": dict(name="bf16xbf16->bf16 M=N=K=8192 A:T B:N", kind="bf16", steps=25,
                      spec=dict(a_type=K.CUDA_R_16BF, b_type=K.CUDA_R_16BF, d_type=K.CUDA_R_16BF,
                                compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F, transa=1, m=8192, n=8192, k=8192)),
    "bf16_8192_nn": dict(name="bf16xbf16->bf16 M=N=K=8192 A:N B:N (operand A transposed on its way into LDS)", kind="bf16", steps=25,
                         spec=dict(a_type=K.CUDA_R_16BF, b_type=K.CUDA_R_16BF, d_type=K.CUDA_R_16BF,
                                   compute_type=K.CUBLAS_COMPUTE_32F, scale_type=K.CUDA_R_32F, transa=0, m=8192, n=8192, k=8192)),
}
for _w in WORKLOADS.values():   # five equal batches
    _w["steps"] = max(5, _w["steps"] // 5 * 5)


# HBM bytes per launch of the dominant kernel come from the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
# this script whose summaries are committed under profiles/ (each counter scaled by what it reads for the
# 256 MiB copy of --copy-probe).  The line carries the figure and the file it was read from; a workload
# without a summary reports null.
PROFILE_OF = {"c1": "gemm_mfma_tr_i8_c1_256", "c2": "gemm_mfma_w4_i8_c2_4096", "i8_4096_nt": "gemm_mfma_tr_i8_4096_nt",
              "i8_8192": "gemm_mfma_w4_i8_8192", "c3": "decode_slab_c3", "c4": "gemm_mfma_w4_f8_c4_8192",
              "c5": "gemm_mfma_w4_mxf4_c5_8192x4", "c5_b1": "gemm_mfma_w4_mxf4_c5_8192_b1",
              "decode_k13824": "decode_slab_k13824", "bf16_8192": "gemm_mfma_w4_bf16_8192", "bf16_8192_nn": "gemm_mfma_tr_bf16_8192_nn"}


def measured_traffic(key):
    """(bytes per launch or None, file name or None) from profiles/<kernel>_<workload>.txt"""
    import re
    name = PROFILE_OF.get(key)
    if not name:
        return None, None
    path = os.path.join(ROOT, "profiles", name + ".txt")
    try:
        m = re.search(r"traffic = (\d+) bytes per dispatch", open(path).read())
    except OSError:
        return None, None
    return (int(m.group(1)), "profiles/%s.txt" % name) if m else (None, None)


def algorithmic(spec):
    """(ops, bytes) of one call: 2*M*N*K*batch and every operand/result byte exactly once."""
    m, n, k, b = spec["m"], spec["n"], spec["k"], spec.get("batch", 1)
    bits = K.TYPE_BITS
    by = b * (m * k * bits[spec["a_type"]] + n * k * bits[spec["b_type"]] + m * n * bits[spec["d_type"]]) // 8
    if spec.get("a_scale_mode") == K.CUBLASLT_MATMUL_MATRIX_SCALE_VEC32_UE8M0:
        by += b * (m + n) * (k // 32)
    if spec.get("b_scale_mode") == K.CUBLASLT_MATMUL_MATRIX_SCALE_OUTER_VEC_32F:
        by += n * 4
    if spec.get("pointer_mode", 0) >= K.CUBLASLT_POINTER_MODE_DEVICE_VECTOR:
        by += m * 4
    if "bias_type" in spec:
        by += m * bits[spec["bias_type"]] // 8
    if spec.get("kind_scalar_scales"):
        by += 8
    return 2 * m * n * k * b, by


class Buffers:
    """Synthetic device-resident inputs of one workload (torch is only the allocator here)."""

    def __init__(self, torch, key, spec, copies=1):
        dev = "cuda:0"
        g = torch.Generator(device=dev)
        g.manual_seed({"c2": 1, "c3": 2, "c4": 3, "c5": 4, "c5_b1": 4}.get(key, 5))
        decode = WORKLOADS[key]["kind"] == "hbm"
        m, n, k, b = spec["m"], spec["n"], spec["k"], spec.get("batch", 1)
        self.keep = []
        self.bias = self.a_scale = self.b_scale = self.alpha_dev = None
        at = spec["a_type"]
        if at == K.CUDA_R_8I:
            if decode:   # round(N(0,32)) clipped to +-127
                mk = lambda r: torch.clamp(torch.round(torch.randn(r, k, device=dev, generator=g) * 32), -127, 127).to(torch.int8)
            else:             # uniform [-128, 127]
                mk = lambda r: torch.randint(-128, 128, (r, k), device=dev, generator=g, dtype=torch.int8)
            self.A = [mk(m) for _ in range(copies)]
            self.B = mk(n)
        elif at == K.CUDA_R_16BF:   # N(0,1); an operand that is not transposed is stored [K][rows]
            mk = lambda r, t: torch.randn((r, k) if t else (k, r), device=dev, generator=g).to(torch.bfloat16)
            self.A = [mk(m, spec.get("transa", 0))]
            self.B = mk(n, not spec.get("transb", 0))
        elif at == K.CUDA_R_8F_E4M3:
            def mk(r):
                x = torch.randn(r, k, device=dev, generator=g)
                amax = x.abs().max()
                return (x * (448.0 / amax)).to(torch.float8_e4m3fn), (amax / 448.0).reshape(1).float()
            a, sa = mk(m)
            bq, sb = mk(n)
            self.A, self.B, self.a_scale, self.b_scale = [a], bq, sa, sb
        else:  # MXFP4: per 32-block e = floor(log2(max)) - 2, elements RNE to E2M1, low nibble = even k
            grid = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], device=dev)
            mids = (grid[:-1] + grid[1:]) / 2

            def mk(r):
                qs, ss = [], []
                for _ in range(b):
                    x = torch.randn(r, k // 32, 32, device=dev, generator=g)
                    e = torch.floor(torch.log2(x.abs().amax(dim=2, keepdim=True))) - 2
                    y = (x * torch.exp2(-e)).clamp(-6, 6)
                    idx = torch.bucketize(y.abs(), mids)   # nearest grid point (ties resolve downward: bench data only)
                    code = (idx | ((y < 0).to(idx.dtype) << 3)).to(torch.uint8).reshape(r, k)
                    qs.append(code[:, 0::2] | (code[:, 1::2] << 4))
                    ss.append((e.reshape(r, k // 32) + 127).to(torch.uint8))
                return torch.stack(qs).contiguous(), torch.stack(ss).contiguous()
            a, sa = mk(m)
            bq, sb = mk(n)
            self.A, self.B, self.a_scale, self.b_scale = [a], bq, sa, sb
        dt = {K.CUDA_R_32I: torch.int32, K.CUDA_R_16BF: torch.bfloat16}[spec["d_type"]]
        self.D = torch.empty(b * m * n, device=dev, dtype=dt)
        if decode:
            self.alpha_dev = torch.empty(m, device=dev).uniform_(0.001, 0.01, generator=g)
            self.b_scale = torch.empty(n, device=dev).uniform_(0.005, 0.02, generator=g)
            self.bias = torch.randn(m, device=dev, generator=g) * 0.02
        if key == "c4":
            self.bias = (torch.randn(m, device=dev, generator=g) * 0.02).to(torch.bfloat16)


NBATCH = 5


SETTLE_SECONDS = 0.5   # --settle: untimed stretch of calls in front of every measurement
DEFAULT_WARMUP = 10


def settle(torch, fn, seconds):
    """Back-to-back calls for `seconds` (no timing): under matrix load the part reaches its power cap after a few hundred
    milliseconds, and only then does a short measurement show what a long-running job sees.  Returns the calls made."""
    if seconds <= 0:
        return 0
    t0, n, chunk = time.perf_counter(), 0, 8
    while time.perf_counter() - t0 < seconds:
        for i in range(chunk):
            fn(n + i)
        n += chunk
        torch.cuda.synchronize()   # bounds the queue: the stretch ends when the clock says so, not thousands of calls later
        chunk = min(chunk * 2, 256)
    return n


def time_calls(torch, fn, steps, warmup, settle_s=None):
    """An untimed settle stretch, `warmup` untimed calls, then exactly `steps` calls between two synchronisations.
    Returns (wall seconds for the `steps` calls, median over NBATCH equal batches of the seconds per call by HIP
    events on the launch stream, [seconds per call of each batch], warm-up calls made, settle calls made)."""
    settled = settle(torch, fn, SETTLE_SECONDS if settle_s is None else settle_s)
    if warmup < 0:
        warmup = DEFAULT_WARMUP
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    nb = NBATCH if steps % NBATCH == 0 else 1
    per = steps // nb
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(nb + 1)]
    t0 = time.perf_counter()
    ev[0].record()
    for b in range(nb):
        for i in range(per):
            fn(b * per + i)
        ev[b + 1].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    batches = sorted(ev[b].elapsed_time(ev[b + 1]) * 1e-3 / per for b in range(nb))
    return wall, batches[len(batches) // 2], batches, warmup, settled


_probe = None


def load_probe():
    """the measurement helpers of zluda_amd/csrc/bench (None when not built)"""
    global _probe
    path = os.path.join(ROOT, "zluda_amd", "lib", "libzluda_bench_probe.so")
    if _probe is None and os.path.exists(path):
        _probe = C.CDLL(path)
        _probe.zluda_bench_clock_probe.argtypes = [C.c_void_p, C.c_uint64, C.c_void_p]
        _probe.zluda_bench_flat_read.argtypes = [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]
    return _probe


def flat_read_seconds(torch, buffers, steps, warmup):
    """A plain read of the same weight buffers, rotated the same way, one kernel launch each: the practical
    ceiling of a memory-bound kernel over these bytes on this GPU.  Seconds per launch, or None."""
    probe = load_probe()
    if probe is None:
        return None
    sink = torch.zeros(1, dtype=torch.int32, device="cuda:0")
    stream = torch.cuda.current_stream().cuda_stream

    def fn(i):
        t = buffers[i % len(buffers)]
        if probe.zluda_bench_flat_read(t.data_ptr(), t.numel() * t.element_size(), sink.data_ptr(), stream) != 0:
            raise RuntimeError("flat read launch failed")
    return time_calls(torch, fn, steps, warmup)[1]


def observed_clock_mhz(torch, fn, calls, seconds_per_call):
    """Shader clock held while `calls` more calls of `fn` run: a one-wave kernel on a second stream reads the
    shader cycle counter and the constant-rate real-time counter at both ends of ~80 % of that stretch.
    None when the helper library is missing."""
    if load_probe() is None:
        return None
    khz = _probe.zluda_bench_wall_clock_khz()
    if khz <= 0:
        return None
    out = torch.zeros(2, dtype=torch.int64, device="cuda:0")
    side = torch.cuda.Stream()
    ticks = int(max(calls * seconds_per_call * 0.8, 20e-6) * khz * 1e3)
    fn(0)   # the load is already running when the probe takes its first sample
    if _probe.zluda_bench_clock_probe(out.data_ptr(), ticks, side.cuda_stream) != 0:
        return None
    for i in range(calls):
        fn(i)
    torch.cuda.synchronize()
    cycles, rt = (int(x) for x in out.tolist())
    return cycles / (rt / (khz * 1e3)) / 1e6 if rt > 0 else None


SUSTAIN_SECONDS = 0.0   # --sustained: seconds of back-to-back calls per measurement (0 = off)


def sustained(torch, fn, seconds, per_batch=10):
    """The same call back to back for `seconds`, with the board power sampled from hwmon meanwhile: under matrix
    load the part sits at its power cap after a few hundred milliseconds, so what a long-running job sees is the
    time a kernel's ENERGY allows, not what a burst of a few dozen calls shows.  Returns microseconds per call,
    watts and millijoules per call over the second half of the run (watts None where hwmon is not readable)."""
    import glob
    import threading
    files = glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input")
    samples, stop = [], []

    def sampler():
        while not stop:
            try:
                samples.append((time.perf_counter(), int(open(files[0]).read()) / 1e6))
            except (OSError, ValueError, IndexError):
                return
            time.sleep(0.002)
    th = threading.Thread(target=sampler, daemon=True)
    torch.cuda.synchronize()
    th.start()
    t0, marks, n = time.perf_counter(), [], 0
    while time.perf_counter() - t0 < seconds:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(per_batch):
            fn(n + i)
        e1.record()
        n += per_batch
        e1.synchronize()
        marks.append((time.perf_counter(), e0.elapsed_time(e1) / per_batch * 1e3))
    stop.append(1)
    th.join()
    half = marks[len(marks) // 2:]
    us = sum(m[1] for m in half) / len(half)
    pw = [p for (t, p) in samples if half[0][0] <= t <= half[-1][0]]
    watts = sum(pw) / len(pw) if pw else None
    return {"seconds": seconds, "us_per_call": us, "watts": watts, "mj_per_call": us * watts * 1e-3 if watts else None}


def run_workload(torch, api, key, steps, warmup, with_hipblaslt):
    w = WORKLOADS[key]
    spec = w["spec"]
    ops, nbytes = algorithmic(spec)
    if key == "c4":
        nbytes += 8
    copies = 1
    decode = w["kind"] == "hbm"
    if decode:
        copies = 8   # 8 x 58.7 MB (or more) of weights > 256 MB Infinity Cache: every call streams from HBM
    buf = Buffers(torch, key, spec, copies)
    call = MatmulCall(api, spec)
    call.set_pointers(bias=buf.bias.data_ptr() if buf.bias is not None else None,
                      a_scale=buf.a_scale.data_ptr() if buf.a_scale is not None and not decode else None,
                      b_scale=buf.b_scale.data_ptr() if buf.b_scale is not None else None)
    int_scale = spec["scale_type"] == K.CUDA_R_32I
    one = C.c_int32(1) if int_scale else C.c_float(1.0)
    zero = C.c_int32(0) if int_scale else C.c_float(0.0)
    alpha = buf.alpha_dev.data_ptr() if buf.alpha_dev is not None else one
    stream = torch.cuda.current_stream().cuda_stream
    a_ptrs = [a.data_ptr() for a in buf.A]
    bp, dp = buf.B.data_ptr(), buf.D.data_ptr()

    def ours(i):
        st = call.run(alpha, a_ptrs[i % copies], bp, zero, None, dp, None, 0, stream)
        if st:
            raise RuntimeError("cublasLtMatmul status %d on workload %s" % (st, key))
    wall, per_call, batches, warmed, settled = time_calls(torch, ours, steps, warmup)
    bound = "hbm" if w["kind"] == "hbm" else "mfma"
    achieved = (nbytes / per_call / 1e9) if bound == "hbm" else (ops / per_call / 1e12)
    peak = PEAK[w["kind"]]
    traffic, traffic_file = measured_traffic(key)
    clock = observed_clock_mhz(torch, ours, max(steps // NBATCH, 4), per_call)
    res = {
        "workload": w["name"], "steps": steps, "warmup": warmed, "settle_s": SETTLE_SECONDS, "settle_calls": settled,
        "ms_per_step": wall / steps * 1e3,
        "tops": ops / (wall / steps) / 1e12, "gbps": nbytes / (wall / steps) / 1e9,
        "kernel": {"family": call.kernel, "variant": call.variant},
        "roofline": {"bound": bound, "achieved": achieved, "peak": peak, "unit": "GB/s" if bound == "hbm" else "TFLOP/s",
                     "frac": achieved / peak, "traffic": traffic, "traffic_source": traffic_file,
                     "kernel_ms": per_call * 1e3, "kernel_ms_batches": [b * 1e3 for b in batches],
                     "algorithmic_ops": ops, "algorithmic_bytes": nbytes, "clock_mhz_observed": clock},
    }
    if bound == "hbm":   # beside the streaming kernel: what a plain read of the same weights takes
        flat = flat_read_seconds(torch, buf.A, steps, warmup)
        if flat:
            res["roofline"]["flat_read_ms"] = flat * 1e3
            res["roofline"]["flat_read_gbps"] = sum(a.numel() for a in buf.A[:1]) / flat / 1e9
    if SUSTAIN_SECONDS > 0:
        res["sustained"] = sustained(torch, ours, SUSTAIN_SECONDS)
    if clock and bound == "mfma":   # what the datasheet peak comes to at the clock the part actually held
        res["roofline"]["frac_at_observed_clock"] = achieved / (peak * clock / PEAK_CLOCK_MHZ)
    if with_hipblaslt:
        res["hipblaslt_forwarded"] = time_hipblaslt(torch, spec, buf, alpha, zero, a_ptrs, copies, steps, warmup, ops, nbytes)
    call.close()
    return res


def time_hipblaslt(torch, spec, buf, alpha, zero, a_ptrs, copies, steps, warmup, ops, nbytes):
    """the reference's hipBLASLt-forwarded path on the same buffers (oracle.hipblaslt_replay)"""
    try:
        from oracle.hipblaslt_replay import Replay
        rp = Replay(spec)
        if rp.why:
            return {"available": False, "why": rp.why.strip()}
        key_c3 = buf.alpha_dev is not None
        ok = rp.set_pointers(bias=buf.bias.data_ptr() if buf.bias is not None else None,
                             a_scale=buf.a_scale.data_ptr() if buf.a_scale is not None and not key_c3 else None,
                             b_scale=buf.b_scale.data_ptr() if buf.b_scale is not None else None)
        if not ok or not rp.find_algo():
            why = rp.why.strip()
            rp.close()
            return {"available": False, "why": why}
        stream = torch.cuda.current_stream().cuda_stream
        bp, dp = buf.B.data_ptr(), buf.D.data_ptr()

        def theirs(i):
            st = rp.run(alpha, a_ptrs[i % copies], bp, zero, None, dp, stream)
            if st:
                raise RuntimeError("hipblasLtMatmul status %d" % st)
        wall, per_call, _, _, _ = time_calls(torch, theirs, steps, warmup)
        clock = observed_clock_mhz(torch, theirs, max(steps // NBATCH, 4), per_call)
        sus = sustained(torch, theirs, SUSTAIN_SECONDS) if SUSTAIN_SECONDS > 0 else None
        rp.close()
        return {"available": True, "sustained": sus, "ms_per_step": wall / steps * 1e3, "kernel_ms": per_call * 1e3, "clock_mhz_observed": clock,
                "tops": ops / per_call / 1e12, "gbps": nbytes / per_call / 1e9}
    except Exception as e:  # the comparison point is optional; the product numbers are not
        return {"available": False, "why": "%s: %s" % (type(e).__name__, e)}


def cpu_baseline(key, budget_s=12.0):
    """The CPU oracle (oracle/ref_gemm.c, OpenMP over all host cores) timed on a bounded sample of the
    workload: a slab of rows of D (full N and K, one batch), repeated until `budget_s` seconds of CPU
    work have been spent.  For a slab the rate is extrapolated to the whole problem (every row of D costs the
    same) and the sample text says so."""
    import oracle  # noqa: F401
    from oracle.cases import Case
    spec = dict(WORKLOADS[key]["spec"])
    full_m = spec["m"]
    rows = {"c1": full_m, "c2": full_m, "i8_4096_nt": full_m, "i8_8192": 2048, "c3": full_m, "decode_k13824": full_m, "c4": 256, "c5": 64, "c5_b1": 64,
            "bf16_8192": 256, "bf16_8192_nn": 256}[key]
    spec.update(m=rows, batch=1, alpha=1)
    decode = WORKLOADS[key]["kind"] == "hbm"
    case = Case(spec, 1, int_dist="normal" if decode else "uniform")
    case.run_oracle()   # page in, spin up the OpenMP team
    reps, dt = 0, 0.0
    while dt < budget_s and reps < 1000:
        t0 = time.perf_counter()
        case.run_oracle()
        dt += time.perf_counter() - t0
        reps += 1
    ops = 2 * rows * spec["n"] * spec["k"] * reps
    unit = "GB/s" if decode else "TOPS"
    val = (algorithmic(spec)[1] * reps / dt / 1e9) if decode else ops / dt / 1e12
    return {"value": val, "unit": unit, "cores": int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)),
            "kind": "port", "seconds": dt,
            "sample": "%d passes over %d of %d rows of D (full N=%d, K=%d, batch 1)%s, oracle/ref_gemm.c with OpenMP, "
                      "%.1f s of CPU time" % (reps, rows, full_m, spec["n"], spec["k"],
                                              "; rate of the slab, extrapolated to the whole problem" if rows < full_m else "", dt)}


ALSO_DEFAULT = ("c3", "i8_8192", "c5", "c5_b1", "c2", "c1", "i8_4096_nt", "decode_k13824")   # the order the metric names them in
ALSO_KEYS = {"c3": "decode_c3"}


def compact(res):
    """one workload's record cut down to what the line has room for"""
    r = res["roofline"]
    out = {"ms": round(r["kernel_ms"], 5), "frac": round(r["frac"], 4), "kernel": "%d/%d" % (res["kernel"]["family"], res["kernel"]["variant"])}
    if r["bound"] == "hbm":
        out["gbps"] = round(r["achieved"], 1)
        if "flat_read_gbps" in r:
            out["flat_read_gbps"] = round(r["flat_read_gbps"], 1)
    else:
        out["tops"] = round(r["achieved"], 1)
    if r.get("traffic"):
        out["traffic"] = r["traffic"]
    h = res.get("hipblaslt_forwarded")
    if h is not None:
        if h.get("available"):
            out["hipblaslt_ms"] = round(h["kernel_ms"], 5)
            out["vs_hipblaslt"] = round(h["kernel_ms"] / r["kernel_ms"], 3)
        else:
            out["hipblaslt"] = (h.get("why") or "unavailable")[:60]
    if res.get("sustained"):
        out["sustained_us"] = round(res["sustained"]["us_per_call"], 1)
    return out


def main():
    global SUSTAIN_SECONDS, SETTLE_SECONDS
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=0)
    ap.add_argument("--warmup", type=int, default=-1, help="untimed calls between the settle stretch and the timed calls (default %d)" % DEFAULT_WARMUP)
    ap.add_argument("--settle", type=float, default=SETTLE_SECONDS, metavar="SECONDS",
                    help="untimed stretch of calls in front of every measurement, whatever --warmup says: the power "
                         "management needs a few hundred milliseconds of load to settle (0 = off)")
    ap.add_argument("--workload", default="c4", choices=sorted(WORKLOADS))
    ap.add_argument("--only", action="store_true", help="skip the other workloads")
    ap.add_argument("--also", default=",".join(ALSO_DEFAULT), help="the other workloads to run, in order (default: %(default)s)")
    ap.add_argument("--full", action="store_true", help="whole records for every workload instead of the compact line")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-hipblaslt", action="store_true")
    ap.add_argument("--sustained", type=float, default=0.0, metavar="SECONDS",
                    help="also run every workload (and its hipBLASLt counterpart) back to back for this long with the "
                         "board power sampled from hwmon: time, watts and energy per call at the power cap")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also launch one plain elementwise copy of 256 MiB (int32 in, int32 out): the known-size "
                         "kernel that calibrates FETCH_SIZE / WRITE_SIZE in a rocprofv3 --pmc run")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (pass --gpus 1)")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a HIP device; there is no CPU path to benchmark")
    api = cublaslt.load()
    torch.cuda.init()
    SUSTAIN_SECONDS = args.sustained
    SETTLE_SECONDS = max(args.settle, 0.0)
    key = args.workload
    steps = args.steps or WORKLOADS[key]["steps"]
    if args.copy_probe:
        src = torch.ones(64 << 20, dtype=torch.int32, device="cuda:0")
        dst = torch.empty_like(src)
        torch.add(src, 1, out=dst)
        torch.cuda.synchronize()
        del src, dst
    head = run_workload(torch, api, key, steps, args.warmup, not args.no_hipblaslt)
    also = {}
    if not args.only:
        for other in [o for o in args.also.split(",") if o]:
            if other == key or other not in WORKLOADS:
                continue
            try:
                also[other] = run_workload(torch, api, other, WORKLOADS[other]["steps"], args.warmup, not args.no_hipblaslt)
            except Exception as e:
                also[other] = {"error": "%s: %s" % (type(e).__name__, e)}
            torch.cuda.empty_cache()
    unit = "GB/s" if WORKLOADS[key]["kind"] == "hbm" else "TOPS"
    roof = dict(head["roofline"])
    if not args.full:
        roof.pop("kernel_ms_batches", None)
    hb = head.get("hipblaslt_forwarded") or {}
    if hb.get("available"):
        # the reference's forwarded path on the same buffers, same timing: its rate and ours over it
        roof["hipblaslt_tops" if unit == "TOPS" else "hipblaslt_gbps"] = hb["tops"] if unit == "TOPS" else hb["gbps"]
        roof["vs_hipblaslt"] = hb["kernel_ms"] / head["roofline"]["kernel_ms"]
    elif hb:
        roof["hipblaslt"] = (hb.get("why") or "unavailable")[:80]
    c3 = also.get("c3")
    if c3 and "roofline" in c3:   # the decode half of the metric, where the driver keeps it
        r3 = c3["roofline"]
        roof["decode_c3"] = {"gbps": r3["achieved"], "frac": r3["frac"], "kernel_ms": r3["kernel_ms"], "peak": r3["peak"],
                             "flat_read_gbps": r3.get("flat_read_gbps")}
    line = {
        "metric": "cublasLtMatmul TOPS (int8/fp8/MXFP4, 8192^3) + decode GEMM HBM GB/s",
        "value": head["gbps"] if unit == "GB/s" else head["tops"], "unit": unit, "n_gpus": 1, "steps": steps,
        "warmup": head["warmup"], "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": {"i8": "int8", "hbm": "int8", "f8": "fp8_e4m3", "f4": "fp4_e2m1", "bf16": "bf16"}[WORKLOADS[key]["kind"]],
        "data": "synthetic", "config": {"workload": head["workload"], "kernel": head["kernel"]},
        "settle_s": head["settle_s"],
        "roofline": roof,
        "cpu_baseline": None if args.no_cpu else cpu_baseline(key),
        "sustained": head.get("sustained"),
        "device": torch.cuda.get_device_name(0), "cu_count": api.zluda_gemm_device_cu_count(),
        "also": also if args.full else {k: (v if "error" in v else compact(v)) for k, v in also.items()},
    }
    if args.full:
        line["hipblaslt_forwarded"] = head.get("hipblaslt_forwarded")
    print(json.dumps(line))


if __name__ == "__main__":
    main()
