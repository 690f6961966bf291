"""ctypes binding of libzluda_ptx_mma.so (include/zluda_ptx_mma.h): runs the gfx950 device functions
for PTX `mma.sync` on fragments held in device memory.  Device memory crosses the boundary as integer
addresses; loading fails loudly when the library has not been built (there is no CPU path)."""
import ctypes as C
import os

S8, F16, BF16 = 0, 1, 2
_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libzluda_ptx_mma.so")
BITCODE_PATH = os.path.join(os.path.dirname(_LIB_PATH), "zluda_ptx_impl_mma.bc")
# the names ZLUDA's compiler emits calls to (ptx/src/pass/replace_instructions_with_functions.rs:468-486)
DEVICE_FUNCTIONS = ("__zluda_ptx_impl_mma_sync_aligned_m16n8k16_row_col_f32_f16_f16_f32",
                    "__zluda_ptx_impl_mma_sync_aligned_m16n8k16_row_col_f32_bf16_bf16_f32",
                    "__zluda_ptx_impl_mma_sync_aligned_m16n8k32_row_col_s32_s8_s8_s32")


def load():
    if not os.path.exists(_LIB_PATH):
        raise OSError("%s is not built: run zluda_amd.build.build()" % _LIB_PATH)
    lib = C.CDLL(_LIB_PATH)
    lib.zluda_ptx_mma_run.restype = C.c_uint32
    lib.zluda_ptx_mma_run.argtypes = [C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32,
                                      C.c_uint32, C.c_uint32, C.c_void_p]
    lib.zluda_ptx_mma_chain.restype = C.c_uint32
    lib.zluda_ptx_mma_chain.argtypes = [C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32,
                                        C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p]
    return lib


def measure(kind=S8, waves_per_cu=8, iters=2000, reps=5):
    """Times the dependent chain of zluda_ptx_mma_chain on the current device for the MFMA form and the
    per-lane form; returns {form: (ns per warp-level mma per CU slot, useful TOP/s over the chip)}."""
    import torch
    lib = load()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    threads = cus * waves_per_cu * 64
    a = torch.randint(-2**31, 2**31 - 1, (threads * 4,), dtype=torch.int32, device="cuda")
    b = torch.randint(-2**31, 2**31 - 1, (threads * 2,), dtype=torch.int32, device="cuda")
    c = torch.zeros(threads * 4, dtype=torch.int32, device="cuda")
    d = torch.empty_like(c)
    flops_per_mma = 2 * 16 * 8 * (32 if kind == S8 else 16)
    out = {}
    for form, per_lane in (("mfma", 0), ("per_lane", 1)):
        best = None
        for _ in range(reps + 1):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            st = lib.zluda_ptx_mma_chain(kind, a.data_ptr(), b.data_ptr(), c.data_ptr(), d.data_ptr(), threads, 256, iters,
                                         per_lane, torch.cuda.current_stream().cuda_stream)
            e1.record()
            assert st == 0
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1)
            best = ms if best is None else min(best, ms)
        warp_mmas = threads // 32 * iters
        out[form] = (best * 1e6 / iters, warp_mmas * flops_per_mma / (best * 1e-3) / 1e12)
    return out


if __name__ == "__main__":
    import torch  # noqa: F401
    for name, kind in (("s8 m16n8k32", S8), ("f16 m16n8k16", F16), ("bf16 m16n8k16", BF16)):
        for wpc in (4, 8, 16):
            r = measure(kind, wpc)
            print("%-14s %2d waves/CU: mfma form %7.1f ns per chained mma, %7.2f T(FL)OP/s; per-lane form %7.1f ns, %7.2f T(FL)OP/s"
                  % (name, wpc, r["mfma"][0], r["mfma"][1], r["per_lane"][0], r["per_lane"][1]), flush=True)
