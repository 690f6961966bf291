"""bench.py's contract, as far as it can be checked without a GPU: it measures one GPU and says so, it refuses
to run without a device (there is no CPU path to benchmark), its algorithmic work per launch is the figure the
roofline fraction is quoted on, and every rocprofv3 summary it reads its traffic figure from is committed."""
import os
import subprocess
import sys

import bench

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = run("--gpus", "2")
    assert r.returncode != 0 and "one GPU" in r.stderr


def test_no_device_no_numbers():
    import torch
    if torch.cuda.is_available():
        return
    r = run("--steps", "5")
    assert r.returncode != 0 and "HIP device" in r.stderr and r.stdout.strip() == ""


def test_algorithmic_work_per_launch():
    w = bench.WORKLOADS
    assert bench.algorithmic(w["c1"]["spec"]) == (2 * 256**3, 393216)
    assert bench.algorithmic(w["c2"]["spec"]) == (137438953472, 100663296)
    assert bench.algorithmic(w["c3"]["spec"]) == (1879048192, 59359296)
    ops, nbytes = bench.algorithmic(w["c4"]["spec"])
    assert (ops, nbytes + 8) == (1099511627776, 268451848)     # + the two fp32 scale factors, added by run_workload
    assert bench.algorithmic(w["c5"]["spec"]) == (4398046511104, 822083584)
    assert bench.algorithmic(w["c5_b1"]["spec"]) == (1099511627776, 205520896)


def test_every_traffic_figure_has_its_committed_summary():
    for key in bench.WORKLOADS:
        traffic, source = bench.measured_traffic(key)
        assert traffic and source and os.path.exists(os.path.join(ROOT, source)), key
        text = open(os.path.join(ROOT, source)).read()
        assert "rocprofv3 --kernel-trace --stats" in text and "rocprofv3 --pmc FETCH_SIZE" in text
