// Measurement helper of bench.py, not part of libcublaslt.so: one wavefront that samples the shader
// cycle counter (s_memtime) against the constant-rate real-time counter (s_memrealtime) while other
// kernels run, so that the benchmark can state the shader clock the GPU actually held under the
// measured load.  The wave sleeps between samples and leaves after `ticks` real-time ticks
// (at most ~1 s worth, whatever the caller passes), so it always exits.
#include <hip/hip_runtime.h>
#include <stdint.h>

__global__ void clock_probe_kernel(uint64_t *out, uint64_t ticks) {
  if (threadIdx.x != 0) return;
  if (ticks > 100000000ull) ticks = 100000000ull;
  const uint64_t r0 = wall_clock64(), c0 = clock64();
  uint64_t r1 = r0;
  for (uint32_t spins = 0; spins < 40000000u && r1 - r0 < ticks; spins++) {
    __builtin_amdgcn_s_sleep(64);
    r1 = wall_clock64();
  }
  const uint64_t c1 = clock64();
  out[0] = c1 - c0;  // shader cycles
  out[1] = r1 - r0;  // real-time ticks
}

// out: two uint64 in device memory; ticks: length of the sample in real-time ticks; returns hipError_t
extern "C" __attribute__((visibility("default"))) int zluda_bench_clock_probe(uint64_t *out, uint64_t ticks, void *stream) {
  void *args[] = {&out, &ticks};
  return (int)hipLaunchKernel((const void *)clock_probe_kernel, dim3(1), dim3(64), args, 0, (hipStream_t)stream);
}

// real-time counter rate in kHz (0 on failure)
extern "C" __attribute__((visibility("default"))) int zluda_bench_wall_clock_khz(void) {
  int dev = 0, khz = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess) return 0;
  return khz;
}

// A flat read of `bytes` (a multiple of 16) bytes: every lane walks the buffer 16 bytes at a time, the whole
// grid one contiguous stripe per step -- the shortest time in which this GPU can pull that many bytes out of
// HBM with one kernel launch, i.e. the practical ceiling of a memory-bound kernel over the same data.  (Swept over
// 256 .. 7168 workgroups of 256 .. 1024 threads, 1 .. 8 loads in flight per lane, with and without the non-temporal
// hint, on 58.7 MB: 9.45 .. 9.7 us for every non-temporal shape with at least 16 waves per CU, 9.9 .. 10.3 without the
// hint; this shape reads 9.5.)
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(512) void flat_read_kernel(const u32x4 *src, uint64_t n16, uint32_t *sink) {
  uint32_t acc = 0;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (uint64_t)gridDim.x * blockDim.x) {
    const u32x4 v = __builtin_nontemporal_load(&src[i]);  // (read once: the hint is worth 5 %)
    acc ^= v[0] ^ v[1] ^ v[2] ^ v[3];
  }
  if (acc == 0x9e3779b9u) sink[0] = acc;  // (keeps the loads alive; practically never taken)
}

// src: device buffer of `bytes` bytes, sink: one device dword; returns hipError_t
extern "C" __attribute__((visibility("default"))) int zluda_bench_flat_read(const void *src, uint64_t bytes, uint32_t *sink, void *stream) {
  const u32x4 *s4 = (const u32x4 *)src;
  uint64_t n16 = bytes / 16;
  void *args[] = {&s4, &n16, &sink};
  return (int)hipLaunchKernel((const void *)flat_read_kernel, dim3(1024), dim3(512), args, 0, (hipStream_t)stream);
}
