"""Writes the golden fixtures that pin the oracle against the reference's own known-answer tests.

Runs only where the reference tree is mounted (it reads test DATA out of
ptx/src/test/spirv_run/mod.rs as text); the JSON files it writes are committed and are all the test
suite needs.

  ptx_cvt_kat.json      scalar conversion vectors (mod.rs:321-329) and the dp4a vector (mod.rs:480-484)
  mma_m16n8k32_s8.json  the int8 mma.sync result vector (mod.rs:890-918) together with the A, B, C
                        matrices its kernel feeds (mma_m16n8k32_s32_s8_s8_s32.ptx): thread t holds the
                        sixteen values in_j = 16 t + j, packs them four to a 32-bit register with the
                        (overlapping) shifts of the kernel's pack_u8 helper, and the registers are
                        placed in the 16x32 / 32x8 / 16x8 matrices by the PTX ISA fragment layout of
                        mma.m16n8k32 (.s8).
"""
import json
import os
import re
import sys

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))
src = open(os.path.join(REF, "ptx/src/test/spirv_run/mod.rs")).read()


def grab(name):
    m = re.search(r"test_ptx(?:_warp)?!\(\s*%s,\s*(.*?)\);" % re.escape(name), src, re.S)
    assert m, name
    return m.group(1)


def s8(b):
    b &= 0xFF
    return b - 256 if b >= 128 else b


kat = {
    "source": "ptx/src/test/spirv_run/mod.rs:321-329, 480-484",
    # cvt.rn.satfinite.e4m3x2.f32 d, a, b : a -> upper byte, b -> lower byte
    "e4m3x2_from_f32": {"in": [0.40625, 12.9], "out": 0x2D55},
    "e5m2x2_from_f32": {"in": [0.375, -5256.6], "out": 0x36ED},
    "f16x2_from_e4m3x2": {"in": 0x2D55, "out": 0x36804A80},
    "f16x2_from_e5m2x2": {"in": 0x36ED, "out": 0x3600ED00},
    "bf16x2_from_f32": {"in": [0.40625, 12.9], "out": 0x3ED0414E},
    # dp4a.s32.s32 d, a, b, c
    "dp4a_s32": {"a": 0x8E2DA590, "b": 0xEDEAEE14, "c": 0x248A9F70, "out": 613065134},
}
for key, text in (("e4m3x2_from_f32", grab("cvt_rn_satfinite_e4m3x2_f32")),
                  ("bf16x2_from_f32", grab("cvt_rn_bf16x2_f32"))):
    assert "0.40625" in text and "12.9" in text, (key, text)
assert "0x2D55" in grab("cvt_rn_satfinite_e4m3x2_f32") and "0x36ED" in grab("cvt_rn_satfinite_e5m2x2_f32")
assert "0x36804a80" in grab("cvt_rn_f16x2_e4m3x2") and "0x3600ED00" in grab("cvt_rn_f16x2_e5m2x2")
assert "0x3ED0414E" in grab("cvt_rn_bf16x2_f32") and "613065134" in grab("dp4a")
json.dump(kat, open(os.path.join(HERE, "ptx_cvt_kat.json"), "w"), indent=1)

# ---- mma.m16n8k32 -------------------------------------------------------------------------
expected = [int(x) for x in re.findall(r"-?\d+", grab("mma_m16n8k32_s32_s8_s8_s32").replace("i32", ""))]
assert len(expected) == 256, len(expected)


def pack_u8(v):  # the kernel's helper: 16-bit inputs shifted by 0/8/16/24 and OR-ed (they overlap)
    return (v[0] | (v[1] << 8) | (v[2] << 16) | (v[3] << 24)) & 0xFFFFFFFF


def bytes_of(reg):
    return [s8(reg >> (8 * i)) for i in range(4)]


warps = []
for w in range(2):  # 64 threads = two 32-lane warps, each an independent mma
    A = [[0] * 32 for _ in range(16)]
    B = [[0] * 8 for _ in range(32)]
    Cm = [[0] * 8 for _ in range(16)]
    Dm = [[0] * 8 for _ in range(16)]
    for lane in range(32):
        t = w * 32 + lane
        inp = [(t * 16 + j) & 0xFFFF for j in range(16)]
        a_regs = [pack_u8(inp[4 * r:4 * r + 4]) for r in range(4)]
        b_regs = [pack_u8(inp[0:4]), pack_u8(inp[0:4])]
        c_regs = [inp[0], inp[1], inp[2], inp[3]]
        gid, tig = lane >> 2, lane & 3
        a_vals = sum((bytes_of(r) for r in a_regs), [])  # a0..a15
        for i, v in enumerate(a_vals):
            row = gid if (i < 4 or 8 <= i < 12) else gid + 8
            col = tig * 4 + (i & 3) + (16 if i >= 8 else 0)
            A[row][col] = v
        b_vals = sum((bytes_of(r) for r in b_regs), [])  # b0..b7
        for i, v in enumerate(b_vals):
            row = tig * 4 + (i & 3) + (16 if i >= 4 else 0)
            B[row][gid] = v
        for i in range(4):
            row = gid if i < 2 else gid + 8
            col = tig * 2 + (i & 1)
            Cm[row][col] = c_regs[i]
            Dm[row][col] = expected[t * 4 + i]
    warps.append({"A": A, "B": B, "C": Cm, "D": Dm})
json.dump({"source": "ptx/src/test/spirv_run/mod.rs:890-918 + mma_m16n8k32_s32_s8_s8_s32.ptx",
           "m": 16, "n": 8, "k": 32, "warps": warps},
          open(os.path.join(HERE, "mma_m16n8k32_s8.json"), "w"))
print("wrote ptx_cvt_kat.json, mma_m16n8k32_s8.json")
