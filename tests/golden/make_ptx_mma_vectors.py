"""Writes tests/golden/ptx_mma_vectors.json: the expected outputs the reference's own tests hold for
its five `mma.sync` programs (ptx/src/test/spirv_run/mod.rs, the `test_ptx_warp!(mma_...)` entries;
each program runs as one block of 64 threads = two warps, ptx/src/test/spirv_run/mod.rs:105-113).
Only the number arrays are taken; the programs' input recipes are restated in oracle/ptx_mma.py.

    python tests/golden/make_ptx_mma_vectors.py [/root/reference]
"""
import json
import os
import re
import sys

NAMES = ["mma_m16n8k16_f32_f16_f16_f32", "mma_m16n8k16_f32_bf16_bf16_f32", "mma_m16n8k16_f32_bf16_bf16_f32_2x",
         "mma_m16n8k32_s32_s8_s8_s32", "mma_m16n8k32_s32_s8_s8_s32_interleave"]


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    text = open(os.path.join(ref, "ptx/src/test/spirv_run/mod.rs")).read()
    out = {}
    for name in NAMES:
        m = re.search(r"test_ptx_warp!\(\s*%s,\s*\[(.*?)\]\s*\);" % name, text, flags=re.S)
        body = m.group(1)
        is_float = "f32" in body.split(",")[0]
        values = [v.strip().replace("f32", "").replace("i32", "") for v in body.split(",") if v.strip()]
        out[name] = {"type": "f32" if is_float else "i32",
                     "values": [float(v) if is_float else int(v) for v in values]}
        print(name, out[name]["type"], len(values))
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "ptx_mma_vectors.json"), "w") as f:
        json.dump(out, f, indent=0, separators=(",", ":"))


if __name__ == "__main__":
    main()
