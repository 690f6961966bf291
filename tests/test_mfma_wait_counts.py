"""The pipelined MFMA kernels wait for a stage of their LDS ring with s_waitcnt vmcnt(N), N = the number of younger
vector memory instructions that may stay in flight.  A count that is one too high lets a wave multiply rows that have
not landed; it shows up as rare wrong results, if at all.  tests/host_c/mfma_wait_check.cpp replays the issue order of
every instantiated tile variant on the CPU with the kernels' own counts (kernels/mfma_wait_counts.hpp) and checks each
wait; here it is built and run, and run again against copies of the header with one count edited by one."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
KERNELS = os.path.join(ROOT, "zluda_amd", "csrc", "kernels")
NEEDED = ["tests/host_c/mfma_wait_check.cpp", "zluda_amd/csrc/planner.hpp", "zluda_amd/csrc/gemm_args.hpp",
          "zluda_amd/csrc/kernels/mfma_wait_counts.hpp", "include/cublaslt_abi.h", "include/zluda_gemm_launch.h"]

pytestmark = pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")


def build_and_run(tree, tmp_path, tag):
    exe = tmp_path / ("mfma_wait_check_" + tag)
    subprocess.run(["g++", "-O1", "-std=c++17", os.path.join(tree, "tests", "host_c", "mfma_wait_check.cpp"), "-o", str(exe)], check=True)
    return subprocess.run([str(exe)], capture_output=True, text=True)


def test_every_counted_wait_of_every_tile_variant():
    import tempfile, pathlib
    with tempfile.TemporaryDirectory() as d:
        res = build_and_run(ROOT, pathlib.Path(d), "ok")
    assert res.returncode == 0, res.stdout
    assert int(res.stdout.split()[0]) > 20000


MUTATIONS = [
    ("c.wait_prologue = (nstage - 1) * c.ndata;", "c.wait_prologue = (nstage - 1) * c.ndata + 1;"),
    ("c.wait_prologue = (nstage - 1) * c.ndata;", "c.wait_prologue = (nstage - 1) * c.ndata - 1;"),
    ("c.wait_stage = (nstage - 2) * c.ndata;", "c.wait_stage = (nstage - 2) * c.ndata + 1;"),
    ("c.wait_prologue = c.nload;", "c.wait_prologue = c.nload + 1;"),
    ("c.wait_prologue = c.nload;", "c.wait_prologue = c.nload - 1;"),
    ("c.wait_stage = 0;", "c.wait_stage = 1;"),
    ("? kl - 2 :", "? kl - 1 :"),
    ("c.ls = mx ? (c.sparts + c.nwv * (c.ch - nstage) - 1) / (c.nwv * (c.ch - nstage)) : 0;",
     "c.ls = mx ? (c.sparts + c.nwv * (c.ch - nstage) - 1) / (c.nwv * (c.ch - nstage)) - 1 : 0;"),
]


@pytest.mark.parametrize("index", range(len(MUTATIONS)))
def test_a_count_edited_by_one_is_caught(tmp_path, index):
    old, new = MUTATIONS[index]
    for rel in NEEDED:
        dst = tmp_path / rel
        dst.parent.mkdir(parents=True, exist_ok=True)
        shutil.copy(os.path.join(ROOT, rel), dst)
    header = tmp_path / "zluda_amd/csrc/kernels/mfma_wait_counts.hpp"
    text = header.read_text()
    assert text.count(old) == 1, old
    header.write_text(text.replace(old, new))
    res = build_and_run(str(tmp_path), tmp_path, "mut")
    assert res.returncode != 0, "the edit went unnoticed: %s" % new


def test_the_kernels_take_their_waits_from_the_checked_header():
    def waits(name):
        return re.findall(r"wait_vmcnt_barrier<([^>]*)>\(\)", open(os.path.join(KERNELS, name)).read())
    assert sorted(set(waits("gemm_mfma_pipe.hpp"))) == ["PC.wait_prologue", "PC.wait_stage"]
    assert sorted(set(waits("gemm_mfma_pipe16.hpp"))) == ["PC.wait_prologue", "PC.wait_stage"]
    assert set(waits("gemm_mfma_w4.hpp")) == {"0"}          # the four-wave kernel never counts
    tr = open(os.path.join(KERNELS, "gemm_mfma_tr.hpp")).read()
    assert "tail_from = tr_tail_from(" in tr
    # no other counted wait hides in inline assembly of these kernels
    for name in ("gemm_mfma_pipe.hpp", "gemm_mfma_pipe16.hpp", "gemm_mfma_w4.hpp", "gemm_mfma_tr.hpp"):
        src = open(os.path.join(KERNELS, name)).read()
        for n in re.findall(r'"s_waitcnt vmcnt\(([^)]*)\)', src):   # (inside assembly strings; comments may say vmcnt(n))
            assert n in ("0", "%0"), (name, n)
