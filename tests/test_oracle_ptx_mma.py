"""Pins oracle/ptx_mma.py (fragment layouts of mma.sync m16n8k32.s8 and m16n8k16.f16/.bf16) against the
expected outputs of the reference's own five mma programs (ptx/src/test/spirv_run/mod.rs, extracted by
tests/golden/make_ptx_mma_vectors.py): every lane feeds different values, so a transposed operand, a
swapped register or a wrong element order changes the result."""
import json
import os

import numpy as np
import pytest

from oracle import ptx_mma

GOLD = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ptx_mma_vectors.json")))


@pytest.mark.parametrize("name", sorted(GOLD))
def test_reference_program_outputs(name):
    want = np.array(GOLD[name]["values"], np.float32 if GOLD[name]["type"] == "f32" else np.int32)
    results = [ptx_mma.mma_sync(kind, a, b, c) for kind, a, b, c in ptx_mma.program_inputs(name)]
    got = ptx_mma.program_output(name, results)
    assert len(got) >= len(want)          # the 2x program's expectation covers its first warp only
    np.testing.assert_array_equal(got[:len(want)], want)


def test_a_layout_mistake_would_show():
    # swapping the two B registers (K halves) must change the s8 program's result
    (kind, a, b, c), = ptx_mma.program_inputs("mma_m16n8k32_s32_s8_s8_s32_interleave")[1:2]
    assert not np.array_equal(ptx_mma.mma_sync(kind, a, b, c), ptx_mma.mma_sync(kind, a, b[..., ::-1], c))
