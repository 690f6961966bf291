"""The slab decode kernel waits for its first weight block with a counted s_waitcnt that assumes a fixed number of
epilogue factor loads in flight behind it (kSlabFactorLoads, kernels/decode_slab.hpp).  A compiler that merged or
dropped one of those loads would make that wait too lax, silently.  This compiles every packed-epilogue
instantiation for gfx950 (device code only, a few seconds) and counts the loads it really issues."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
KERNELS = os.path.join(ROOT, "zluda_amd", "csrc", "kernels")
KINDS = ("KIND_I8", "KIND_F8", "KIND_F16", "KIND_BF16")


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")
def test_every_packed_instantiation_issues_exactly_the_counted_factor_loads(tmp_path):
    header = open(os.path.join(KERNELS, "decode_slab.hpp")).read()
    counted = int(re.search(r"constexpr int kSlabFactorLoads = (\d+);", header).group(1))
    insts = ["%d, %s, %s" % (fast, kind, tail) for fast in (1, 2) for kind in KINDS for tail in ("false", "true")]
    insts += ["%d, %s, true, 8, 512, %d" % (fast, kind, q) for fast in (1, 2) for kind in KINDS for q in (2, 3, 4)]
    insts += ["%d, %s, true, 8, 512, %d, 2" % (fast, kind, q) for fast in (1, 2) for kind in KINDS for q in (1, 2)]
    src = tmp_path / "slab_counts.hip"
    src.write_text('#include <hip/hip_runtime.h>\n#include "decode_slab.hpp"\nusing namespace zluda_amd;\n' + "".join(
        "template __global__ void zluda_amd::decode_slab_kernel<%s>(DecodeParams);\n" % i for i in insts))
    out = tmp_path / "slab_counts.s"
    subprocess.run(["hipcc", "--offload-arch=gfx950", "-O3", "-std=c++17", "-I", KERNELS, "-Wno-unused-value",
                    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-S", "--cuda-device-only",
                    str(src), "-o", str(out)], check=True, stderr=subprocess.DEVNULL)
    found, name, n = {}, None, 0
    for line in open(out):
        m = re.match(r"^(_ZN9zluda_amd18decode_slab_kernel\w+):", line)
        if m:
            name, n = m.group(1), 0
        elif name:
            if "global_load_" in line:
                n += 1
            if "s_barrier" in line:      # everything in front of the reduction: the factor loads and nothing else
                found[name], name = n, None
    assert len(found) == len(insts), sorted(found)
    assert all(v == counted for v in found.values()), (counted, found)


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_no_issued_dma_instruction_is_wholly_out_of_range(tmp_path):
    """The counted waits of the slab kernel assume that loads retire in the order they were issued, which an instruction
    whose 64 lanes are all out of range does not do.  tests/host_c/slab_addr_check.cpp runs the kernel's own addressing
    functions (kernels/decode_slab_addr.hpp) on the host over every shape and K the launcher gives the kernel: every
    instruction has a lane in range, and the lanes in range fetch each K byte of each row exactly once."""
    exe = tmp_path / "slab_addr_check"
    subprocess.run(["g++", "-O2", "-std=c++17", os.path.join(ROOT, "tests", "host_c", "slab_addr_check.cpp"), "-o", str(exe)], check=True)
    res = subprocess.run([str(exe)], capture_output=True, text=True)
    assert res.returncode == 0, res.stdout
    assert int(res.stdout.split()[0]) > 300
