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
    return lib
