"""PTX mma.sync on gfx950 (include/zluda_ptx_mma.h).  CPU: the library and the device bitcode exist
and carry the names ZLUDA's compiler calls.  GPU: the reference's five mma programs
(ptx/src/test/spirv_run/mma_m16n8k*.ptx, inputs restated in oracle/ptx_mma.py) give the outputs the
reference's tests expect (tests/golden/ptx_mma_vectors.json) bit for bit, and seeded random fragments
match the CPU oracle -- through the MFMA path (both warps of a wavefront present) and the per-lane
path (32-thread blocks; only every other warp executing)."""
import json
import os

import numpy as np
import pytest

from oracle import ptx_mma as ref
from zluda_amd import ptx_mma

GOLD = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ptx_mma_vectors.json")))


def test_library_exports_the_host_entry():
    lib = ptx_mma.load()
    assert lib.zluda_ptx_mma_run(3, None, None, None, None, 64, 64, 0, None) == 7      # unknown kind
    assert lib.zluda_ptx_mma_run(0, 1, 1, 1, 1, 64, 48, 0, None) == 7                  # block not whole warps
    assert lib.zluda_ptx_mma_run(0, 1, 1, 1, 1, 96, 64, 0, None) == 7                  # threads not whole blocks


def test_bitcode_defines_the_functions_the_compiler_calls():
    data = open(ptx_mma.BITCODE_PATH, "rb").read()
    assert data[:4] == b"BC\xc0\xde"
    for name in ptx_mma.DEVICE_FUNCTIONS:
        assert name.encode() in data, name


def run_gpu(lib, kind, a, b, c, block, masked=0):
    import torch
    W = a.shape[0]
    ta = torch.from_numpy(a.astype(np.uint32).view(np.int32).reshape(-1)).cuda()
    tb = torch.from_numpy(b.astype(np.uint32).view(np.int32).reshape(-1)).cuda()
    tc = torch.from_numpy(np.ascontiguousarray(c).view(np.int32).reshape(-1)).cuda()
    td = torch.full_like(tc, 0x5A5A5A5A)
    st = lib.zluda_ptx_mma_run(kind, ta.data_ptr(), tb.data_ptr(), tc.data_ptr(), td.data_ptr(), W * 32, block, masked,
                               torch.cuda.current_stream().cuda_stream)
    assert st == 0
    torch.cuda.synchronize()
    return td.cpu().numpy().view(np.asarray(c).dtype).reshape(W, 32, 4)


@pytest.fixture(scope="module")
def lib(gpu_api):
    return ptx_mma.load()


@pytest.mark.gpu
@pytest.mark.parametrize("block", [64, 32])
@pytest.mark.parametrize("name", sorted(GOLD))
def test_reference_programs(lib, name, block):
    print("program", name, "block", block, flush=True)
    want = np.array(GOLD[name]["values"], np.float32 if GOLD[name]["type"] == "f32" else np.int32)
    results = [run_gpu(lib, kind, a, b, c, block) for kind, a, b, c in ref.program_inputs(name)]
    got = ref.program_output(name, results)
    np.testing.assert_array_equal(got[:len(want)], want)


def random_fragments(kind, warps, seed):
    rng = np.random.default_rng(seed)
    if kind == ref.S8:
        a = rng.integers(0, 2**32, (warps, 32, 4), dtype=np.uint64).astype(np.uint32)
        b = rng.integers(0, 2**32, (warps, 32, 2), dtype=np.uint64).astype(np.uint32)
        c = rng.integers(-2**31, 2**31, (warps, 32, 4), dtype=np.int64).astype(np.int32)   # wraps like the hardware
        return a, b, c
    # small integers: every product and partial sum is exact in fp32, so the order of summation is free
    bits = ref.bf16_bits_rne if kind == ref.BF16 else ref.f16_bits
    pack = lambda x: (bits(x[..., 1]) << 16 | bits(x[..., 0])).astype(np.uint32)
    a = pack(rng.integers(-16, 17, (warps, 32, 4, 2)).astype(np.float32))
    b = pack(rng.integers(-16, 17, (warps, 32, 2, 2)).astype(np.float32))
    c = rng.integers(-1000, 1001, (warps, 32, 4)).astype(np.float32)
    return a, b, c


@pytest.mark.gpu
@pytest.mark.parametrize("kind", [ref.S8, ref.F16, ref.BF16])
@pytest.mark.parametrize("block,masked", [(64, 0), (256, 0), (32, 0), (128, 1), (128, 2)])
def test_random_fragments_against_the_oracle(lib, kind, block, masked):
    print("kind", kind, "block", block, "masked", masked, flush=True)
    warps = 64
    a, b, c = random_fragments(kind, warps, 7000 + kind)
    want = ref.mma_sync(kind, a, b, c)
    if masked:   # masked 1: the odd warps of each block skip the instruction (d = c), masked 2: the even ones
        skip = (np.arange(warps) % (block // 32)) % 2 == (1 if masked == 1 else 0)
        want[skip] = c[skip]
    got = run_gpu(lib, kind, a, b, c, block, masked)
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.gpu
@pytest.mark.parametrize("kind", [ref.F16, ref.BF16])
@pytest.mark.parametrize("block,masked", [(64, 0), (32, 0), (128, 2)])
def test_arbitrary_floats_within_the_accumulation_bound(lib, kind, block, masked):
    """Non-integer f16 / bf16 fragments: the sum is no longer exact in fp32, the PTX ISA does not fix the
    order of accumulation, and the MFMA form (products summed by the matrix unit, c added last) and the
    per-lane form (c first, then a chain of fused multiply-adds) round differently.  Tolerance: the bound
    every fp32 accumulation order meets, (K + 1) * 2^-24 * (|A| * |B| + |C|) per element, K = 16."""
    print("kind", kind, "block", block, "masked", masked, flush=True)
    warps = 64
    rng = np.random.default_rng(7200 + kind)
    bits = ref.bf16_bits_rne if kind == ref.BF16 else ref.f16_bits
    pack = lambda x: (bits(x[..., 1]) << 16 | bits(x[..., 0])).astype(np.uint32)
    a = pack(rng.normal(0, 1, (warps, 32, 4, 2)).astype(np.float32))
    b = pack(rng.normal(0, 1, (warps, 32, 2, 2)).astype(np.float32))
    c = rng.normal(0, 4, (warps, 32, 4)).astype(np.float32)
    want, mag = ref.mma_sync_exact(kind, a, b, c)
    if masked:
        skip = (np.arange(warps) % (block // 32)) % 2 == 0
        want[skip] = c[skip]
    got = run_gpu(lib, kind, a, b, c, block, masked).astype(np.float64)
    err = np.abs(got - want)
    print("largest error / bound: %.3f" % float((err / (17 * 2.0**-24 * mag)).max()), flush=True)
    assert (err <= 17 * 2.0**-24 * mag).all()
    assert err.max() > 0   # the inputs do exercise rounding: an all-exact result means the case is too easy


@pytest.mark.gpu
@pytest.mark.parametrize("per_lane", [0, 1])
def test_chained_instructions(lib, per_lane):
    """the measurement entry point: c <- mma(a, b, c) three times, both forms, int8 (wraps exactly)"""
    import torch
    warps = 16
    a, b, c = random_fragments(ref.S8, warps, 7100)
    want = c
    for _ in range(3):
        want = ref.mma_sync(ref.S8, a, b, want)
    ta, tb, tc = (torch.from_numpy(x.view(np.int32).reshape(-1)).cuda() for x in (a, b, c))
    td = torch.zeros_like(tc)
    st = lib.zluda_ptx_mma_chain(ref.S8, ta.data_ptr(), tb.data_ptr(), tc.data_ptr(), td.data_ptr(), warps * 32, 128, 3,
                                 per_lane, torch.cuda.current_stream().cuda_stream)
    assert st == 0
    torch.cuda.synchronize()
    np.testing.assert_array_equal(td.cpu().numpy().reshape(warps, 32, 4), want)
