// Shared host/device helpers for the flaggems_amd kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/flaggems_amd.h"
#include "../../include/flaggems_amd_probes.h"

namespace fg {

constexpr int kWave = 64;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

// Thread-local error text behind fg_last_error_string().
char* error_buffer();
constexpr size_t kErrorBufferBytes = 512;

#define FG_FAIL(code, ...)                                              \
  do {                                                                  \
    snprintf(::fg::error_buffer(), ::fg::kErrorBufferBytes, __VA_ARGS__); \
    return (code);                                                      \
  } while (0)

// Status of the most recent kernel launch made by this thread through FG_LAUNCH.  The launch call's own return
// value is kept, so that an error some other library left in the process-wide "last error" slot is neither taken
// for this launch's nor cleared.
hipError_t& launch_status();
int cu_count_or_default();  // compute units of the current device, 256 when it cannot be asked

template <typename T>
struct same_type { using type = T; };

// Launches `kern` with the given arguments (converted to the kernel's parameter types) and records the status.
template <typename... KArgs>
inline void launch(void (*kern)(KArgs...), dim3 grid, dim3 block, size_t lds_bytes, hipStream_t stream,
                   typename same_type<KArgs>::type... args) {
  void* params[] = {const_cast<void*>(static_cast<const void*>(&args))...};
  launch_status() = hipLaunchKernel(reinterpret_cast<const void*>(kern), grid, block, params, lds_bytes, stream);
}

#define FG_LAUNCH(kern, grid, block, lds_bytes, stream, ...) ::fg::launch(kern, grid, block, lds_bytes, stream, __VA_ARGS__)

// A failed launch also sets HIP's per-thread "last error", which would otherwise stay set after this library has
// reported the failure through its own status and be raised by the caller's next launch check at an unrelated
// operation: hipGetLastError() consumes it.  Nothing is read or cleared after a launch that succeeded.
#define FG_CHECK_LAUNCH(what)                                                       \
  do {                                                                              \
    hipError_t e_ = ::fg::launch_status();                                          \
    if (e_ != hipSuccess) {                                                         \
      (void)hipGetLastError();                                                      \
      FG_FAIL(FG_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e_));                \
    }                                                                               \
  } while (0)

// Kernels that use more than 64 KB of dynamic LDS need the limit raised once per device (the attribute belongs to
// the device's copy of the kernel).  `done` is one flag array per kernel set; a race sets the attribute twice.
constexpr int kMaxDevices = 64;
struct PerDeviceFlags { bool done[kMaxDevices]; };
inline hipError_t raise_dynamic_lds_limit(PerDeviceFlags& flags, int bytes, const void* k0, const void* k1 = nullptr,
                                          const void* k2 = nullptr) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const bool tracked = dev >= 0 && dev < kMaxDevices;
  if (tracked && flags.done[dev]) return hipSuccess;
  e = hipFuncSetAttribute(k0, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess && k1) e = hipFuncSetAttribute(k1, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess && k2) e = hipFuncSetAttribute(k2, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess && tracked) flags.done[dev] = true;
  return e;
}

__host__ __device__ inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

__device__ inline float bits_to_float(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ inline uint32_t float_to_bits(float f) { return __builtin_bit_cast(uint32_t, f); }

}  // namespace fg
