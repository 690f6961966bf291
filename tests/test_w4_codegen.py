"""The four-wave kernel issues its MFMAs as inline assembly, which hides them from the compiler's hazard recogniser and
register allocator.  This test compiles its translation units to assembly (hipcc, device pass only, no GPU needed) and
checks what the kernel's comments promise about the compiler's output:
  * no accumulator (AGPR) is read by anything but an MFMA within the wait states the hardware needs after an MFMA wrote it
    (v_accvgpr_read, a store or a spill of an AGPR right behind an MFMA would read a stale value);
  * the K loop holds no spill code and no accumulator moves."""
import os
import re
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "zluda_amd", "csrc")
HIPCC = "/opt/rocm/bin/hipcc"
NEED = 18   # wait states between an 8-pass (16-pass) MFMA's issue and a VALU / memory read of its result: 11 (19) on gfx940-class parts


def assembly(unit):
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "k.s")
        cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "--cuda-device-only", "-S", os.path.join(CSRC, unit), "-o", out]
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        assert res.returncode == 0, res.stdout[-2000:]
        return open(out).read()


def kernels(text):
    """name -> instruction lines of every w4 kernel in the file"""
    out = {}
    for m in re.finditer(r"^(_ZN9zluda_amd19gemm_mfma_w4_kernel\w+):\s*;.*?\n(.*?)^\s*s_endpgm", text, re.S | re.M):
        lines = [l.strip() for l in m.group(2).split("\n")]
        out[m.group(1)] = [l for l in lines if l and not l.startswith(";") and not l.startswith(".") and not l.endswith(":")]
    return out


AGPR = re.compile(r"\ba(\d+)\b|\ba\[(\d+):(\d+)\]")


def agprs(operand_text):
    regs = set()
    for m in AGPR.finditer(operand_text):
        if m.group(1) is not None:
            regs.add(int(m.group(1)))
        else:
            regs.update(range(int(m.group(2)), int(m.group(3)) + 1))
    return regs


@pytest.mark.parametrize("unit", ["mfma_w4_f8.hip", "mfma_w4_i8.hip", "mfma_w4_mxf4.hip", "mfma_w4_bf16.hip"])
def test_nothing_reads_an_accumulator_too_soon_after_an_mfma(unit):
    found = kernels(assembly(unit))
    assert found, "no four-wave kernel in " + unit
    for name, ins in found.items():
        last_write = {}   # AGPR -> wait states since the MFMA that wrote it was issued
        n_mfma = 0
        for line in ins:
            op, _, rest = line.partition(" ")
            rest = rest.split(";")[0]
            if op.startswith("v_mfma"):
                n_mfma += 1
                dst = rest.split(",")[0]
                for r in last_write:
                    last_write[r] += 1
                for r in agprs(dst):
                    last_write[r] = 0
                continue
            states = 1
            if op == "s_nop":
                states = int(rest.strip()) + 1
            else:
                # any other instruction that names an AGPR as a source reads it
                ops = rest.split(",")
                srcs = ",".join(ops[1:]) if op.startswith(("v_accvgpr_read", "v_accvgpr_mov")) else rest
                if op.startswith(("scratch_load", "buffer_load", "global_load", "ds_read", "v_accvgpr_write")):
                    srcs = ",".join(ops[1:])
                for r in agprs(srcs):
                    assert last_write.get(r, NEED) >= NEED, "%s: `%s` reads a%d %d wait states after the MFMA that wrote it" % (
                        name, line, r, last_write[r])
            for r in last_write:
                last_write[r] += states
        assert n_mfma >= 256, name


def loop_body(body, name):
    """the K loop of a kernel: the blocks of the first inner loop that holds MFMAs, wherever the layout put them (the
    loop may hold forward branches -- the MXFP4 kernel decides per stage whether a scale instruction is due -- and its
    latch may sit in front of its header)"""
    blocks, cur = [], []
    for line in body.split("\n"):
        if re.match(r"^(\.LBB\d+_\d+:|; %bb\.\d+:)", line):
            blocks.append(cur)
            cur = []
        cur.append(line)
    blocks.append(cur)
    for b in blocks:
        head = "\n".join(b[:3])
        if "Inner Loop Header: Depth=2" not in head:
            continue
        label = b[0].split(":")[0].lstrip(".L")        # BB0_52
        mine = [x for x in blocks if x is b or re.search(r"Header=" + re.escape(label) + r" Depth=2", "\n".join(x[:3]))]
        text = "\n".join("\n".join(x) for x in mine)
        if "v_mfma" in text:
            return text
    raise AssertionError("no K loop found in " + name)


@pytest.mark.parametrize("unit", ["mfma_w4_f8.hip", "mfma_w4_i8.hip", "mfma_w4_mxf4.hip", "mfma_w4_bf16.hip"])
def test_the_k_loop_is_free_of_spills_and_accumulator_moves(unit):
    text = assembly(unit)
    mx = "mxf4" in unit
    n = 0
    for m in re.finditer(r"^(_ZN9zluda_amd19gemm_mfma_w4_kernel\w+):\s*;.*?\n(.*?)^\s*s_endpgm", text, re.S | re.M):
        hot = loop_body(m.group(2), m.group(1))
        n += 1
        assert hot.count("v_mfma") in (128, 256), "%s: %d MFMAs in the loop of two stages" % (m.group(1), hot.count("v_mfma"))
        for bad in ("scratch_", "v_accvgpr_") + (() if mx else ("v_readlane", "v_writelane")):
            assert bad not in hot, "%s: %s inside the K loop" % (m.group(1), bad)
        assert hot.count("ds_read_b128") == 64 and hot.count("s_barrier") == 2, m.group(1)
        # data DMA: 16 instructions per wave and stage; MXFP4: scale instructions on top (two in the stage that starts a
        # chunk, one in the next two, none in the fourth), its 16 + 16
        # two-byte scale fragments per stage, and nothing but the two barrier waits counts vector memory operations
        # (three sites: the odd stage of a pair never starts a chunk, which the compiler sees)
        assert hot.count("buffer_load_dwordx4") == (32 + 3 if mx else 32), (m.group(1), hot.count("buffer_load_dwordx4"))
        assert hot.count("ds_read_u16") == (32 if mx else 0), m.group(1)
        assert hot.count("s_waitcnt vmcnt") == 2, m.group(1)
    assert n >= 1
