// The launch entry point that allocates nothing: split-K partial tiles go to an array in device memory
// that is part of the library image instead of a caller workspace.
#include <atomic>
#include <hip/hip_runtime.h>

#include "launch_util.hpp"
#include "planner.hpp"

using namespace zluda_amd;

// Split-K partial tiles go to this array instead of a caller workspace.  Every device the library runs
// on holds its own copy (at its own address) until the process ends.  In host code the array's name is
// only a handle for hipGetSymbolAddress: the device address it returns is what kernels and copies get.
static __device__ __align__(256) unsigned char scratch[ZLUDA_GEMM_STATIC_SCRATCH_BYTES];

extern "C" uint32_t zluda_gemm_launch_noalloc(const zluda_gemm_problem *p, const zluda_gemm_plan *plan,
                                              void *stream) {
  if (!p || !plan) return CUBLAS_STATUS_INVALID_VALUE;
  if (plan->workspace > ZLUDA_GEMM_STATIC_SCRATCH_BYTES) return CUBLAS_STATUS_ALLOC_FAILED;  // more than the library holds
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) return CUBLAS_STATUS_NOT_INITIALIZED;
  if (dev < 0 || dev >= 64) return CUBLAS_STATUS_NOT_SUPPORTED;
  // once per device, with that device current: the address of this device's copy of the array
  static std::atomic<void *> scratch_of[64];  // zero-initialised; racing first calls store the same value
  void *ws = scratch_of[dev].load(std::memory_order_acquire);
  if (!ws) {
    // The look-up may load the code object, which is not something to do in the middle of a stream capture: a caller that
    // captures warms the entry point up with one call outside the capture first (any plan, even one that needs no scratch).
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing((hipStream_t)stream, &cap) != hipSuccess) return CUBLAS_STATUS_NOT_INITIALIZED;
    if (cap != hipStreamCaptureStatusNone) return CUBLAS_STATUS_NOT_SUPPORTED;
    void *ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return CUBLAS_STATUS_NOT_INITIALIZED;
    scratch_of[dev].store(ptr, std::memory_order_release);
    ws = ptr;
  }
  // nothing in the array has to start at zero: every split writes its whole partial tile before the
  // reduction kernel of the same call reads it
  return launch_planned(p, plan, ws, ZLUDA_GEMM_STATIC_SCRATCH_BYTES, stream);
}

