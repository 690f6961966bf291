"""CPU restatement of PTX `mma.sync.aligned` for the three shapes the reference lowers to device
functions (ptx/src/pass/replace_instructions_with_functions.rs:468-486 builds the names,
ptx/lib/zluda_ptx_impl.cpp:979-1079 implements them per lane):

    m16n8k32.row.col.s32.s8.s8.s32      m16n8k16.row.col.f32.f16.f16.f32      m16n8k16.row.col.f32.bf16.bf16.f32

Test infrastructure only.  A warp is 32 lanes; lane = 4 * g + t (g = "groupID", t = "threadID in
group").  With E = elements per 32-bit register (4 for s8, 2 for f16 / bf16), element e of register r
of a lane is, by the fragment layouts the PTX ISA publishes for these shapes,

    A (16 x K, row):   row g + 8 * (r & 1),   column t * E + e + 4 * E * (r >> 1)        r = 0..3
    B (K x 8, col):    row  t * E + e + 4 * E * r,   column g                             r = 0..1
    C, D (16 x 8):     row g + 8 * (r >> 1),  column 2 * t + (r & 1)                      r = 0..3

and D = A * B + C per warp.  Pinned by tests/test_oracle_ptx_mma.py against the expected outputs the
reference's tests hold for its five mma programs (tests/golden/ptx_mma_vectors.json), whose input
recipes `program_inputs` restates from the programs themselves
(ptx/src/test/spirv_run/mma_m16n8k*.ptx).
"""
import numpy as np

S8, F16, BF16 = 0, 1, 2
KINDS = {"s8": S8, "f16": F16, "bf16": BF16}


def bf16_bits_rne(x):
    """float32 -> bf16 bit pattern, round to nearest even (cvt.rn.bf16x2.f32)"""
    u = np.asarray(x, np.float32).view(np.uint32).astype(np.uint64)
    return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF).astype(np.uint32)


def f16_bits(x):
    return np.asarray(x, np.float32).astype(np.float16).view(np.uint16).astype(np.uint32)


def unpack(regs, kind):
    """uint32 [..., R] -> element values [..., R, E] (element 0 = least significant bits)"""
    regs = np.asarray(regs, np.uint32)
    if kind == S8:
        b = np.stack([(regs >> (8 * e)) & 0xFF for e in range(4)], -1).astype(np.uint8)
        return b.view(np.int8).astype(np.float64)
    h = np.stack([(regs >> (16 * e)) & 0xFFFF for e in range(2)], -1)
    if kind == F16:
        return h.astype(np.uint16).view(np.float16).astype(np.float64)
    return (h.astype(np.uint32) << 16).view(np.float32).astype(np.float64)


def _matrices(kind, a, b, c):
    """fragments -> (A [W,16,K], B [W,K,8], C [W,16,8]) in float64"""
    a, b = np.asarray(a, np.uint32), np.asarray(b, np.uint32)
    W = a.shape[0]
    E = 4 if kind == S8 else 2
    K = 8 * E
    av, bv = unpack(a, kind), unpack(b, kind)
    A = np.zeros((W, 16, K)); B = np.zeros((W, K, 8)); C = np.zeros((W, 16, 8))
    lane = np.arange(32); g, t = lane >> 2, lane & 3
    for r in range(4):
        for e in range(E):
            A[:, g + 8 * (r & 1), t * E + e + 4 * E * (r >> 1)] = av[:, :, r, e]
        C[:, g + 8 * (r >> 1), 2 * t + (r & 1)] = np.asarray(c)[:, :, r]
    for r in range(2):
        for e in range(E):
            B[:, t * E + e + 4 * E * r, g] = bv[:, :, r, e]
    return A, B, C


def _fragment(D):
    """D [W,16,8] -> the accumulator fragment [W,32,4]"""
    lane = np.arange(32); g, t = lane >> 2, lane & 3
    d = np.zeros((D.shape[0], 32, 4))
    for r in range(4):
        d[:, :, r] = D[:, g + 8 * (r >> 1), 2 * t + (r & 1)]
    return d


def mma_sync(kind, a, b, c):
    """a: uint32 [W, 32, 4], b: uint32 [W, 32, 2], c: int32 / float32 [W, 32, 4] -> d like c"""
    A, B, C = _matrices(kind, a, b, c)
    d = _fragment(A @ B + C)   # exact in float64 for int8 and for the value ranges the exact float tests use
    if kind == S8:
        return (d.astype(np.int64) & 0xFFFFFFFF).astype(np.uint32).view(np.int32)
    return d.astype(np.float32)


def mma_sync_exact(kind, a, b, c):
    """(d, mag) in float64, unrounded: d = A * B + C and mag = |A| * |B| + |C|, the sum of the magnitudes
    of the terms of each element.  Any fp32 accumulation of the K + 1 terms, in whatever order and with
    or without fused multiply-adds, stays within (K + 1) * 2^-24 * mag of d; the PTX ISA leaves the order
    open, so this is the bound a result for arbitrary float inputs is held to."""
    A, B, C = _matrices(kind, a, b, c)
    return _fragment(A @ B + C), _fragment(np.abs(A) @ np.abs(B) + np.abs(C))


def program_inputs(name, threads=64):
    """The register values each of the reference's mma test programs builds from %tid.x, as a list of
    (kind, a [W,32,4], b [W,32,2], c [W,32,4]) in the order the program stores the results."""
    tid = np.arange(threads, dtype=np.uint32)
    W = threads // 32
    if "s8" in name:
        # in_j = 16 tid + j (u16); pack_u8 ORs in0 | in1 << 8 | in2 << 16 | in3 << 24 without masking
        inj = [(16 * tid + j) & 0xFFFF for j in range(16)]
        pack = lambda q: (inj[4 * q] | (inj[4 * q + 1] << 8) | (inj[4 * q + 2] << 16) | (inj[4 * q + 3] << 24)).astype(np.uint32)
        a = [pack(q) for q in range(4)]
        c = np.stack(inj[:4], -1).astype(np.int32).reshape(W, 32, 4)
        st = lambda regs: np.stack(regs, -1).reshape(W, 32, len(regs))
        if name.endswith("interleave"):
            b0, b1 = pack(0), pack(1)
            fwd, rev = st(a), st(a[::-1])
            return [(S8, fwd, st([b0, b1]), c), (S8, rev, st([b1, b0]), c),
                    (S8, fwd, st([b1, b0]), c), (S8, rev, st([b0, b0]), c)]
        return [(S8, st(a), st([pack(0), pack(0)]), c)]
    kind = BF16 if "bf16" in name else F16
    bits = bf16_bits_rne if kind == BF16 else f16_bits
    inj = [(8.0 * tid + j).astype(np.float32) for j in range(8)]
    # cvt.rn.f16x2.f32 d, x, y : x -> upper half, y -> lower half
    pair = lambda x, y: ((bits(inj[x]) << 16) | bits(inj[y])).astype(np.uint32)
    st = lambda regs: np.stack(regs, -1).reshape(W, 32, len(regs))
    a = st([pair(0, 1), pair(2, 3), pair(4, 5), pair(6, 7)])
    out = [(kind, a, st([pair(0, 1), pair(2, 3)]), st(inj[:4]))]
    if name.endswith("2x"):
        out.append((kind, a, st([pair(4, 5), pair(6, 7)]), st(inj[4:])))
    return out


def program_output(name, results, threads=64):
    """Interleaves the per-mma results [W,32,4] the way the program stores them: thread-major"""
    return np.concatenate([np.asarray(r).reshape(threads, 4) for r in results], axis=1).reshape(-1)
