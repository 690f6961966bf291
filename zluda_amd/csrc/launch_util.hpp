// Kernel launch through hipLaunchKernel, whose own return value tells whether the launch was accepted.
// hipGetLastError() is never consulted: it would report (and clear) a sticky error left in the calling
// thread by unrelated HIP calls of the application.
#pragma once
#include <hip/hip_runtime.h>

#include <type_traits>

#include "../../include/cublaslt_abi.h"

namespace zluda_amd {

template <class... Params, class... Args>
inline uint32_t launch_kernel(void (*kernel)(Params...), dim3 grid, dim3 block, hipStream_t s, const Args &...args) {
  static_assert(sizeof...(Params) == sizeof...(Args), "one argument per kernel parameter");
  // (an argument of another type would be converted into a temporary that is gone before hipLaunchKernel reads it)
  static_assert((std::is_same_v<std::remove_cv_t<Params>, std::remove_cv_t<Args>> && ...), "arguments of exactly the kernel's parameter types");
  void *ptrs[] = {(void *)&static_cast<const Params &>(args)...};
  return hipLaunchKernel((const void *)kernel, grid, block, ptrs, 0, s) == hipSuccess ? CUBLAS_STATUS_SUCCESS
                                                                                    : CUBLAS_STATUS_EXECUTION_FAILED;
}

} // namespace zluda_amd
