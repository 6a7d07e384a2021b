// Shared host/device helpers for the flaggems_amd kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/flaggems_amd.h"

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

#define FG_CHECK_LAUNCH(what)                                                       \
  do {                                                                              \
    hipError_t e_ = hipGetLastError();                                              \
    if (e_ != hipSuccess) FG_FAIL(FG_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e_)); \
  } while (0)

__host__ __device__ inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

__device__ inline float bits_to_float(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ inline uint32_t float_to_bits(float f) { return __builtin_bit_cast(uint32_t, f); }

}  // namespace fg
