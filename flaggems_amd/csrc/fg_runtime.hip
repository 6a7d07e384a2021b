// Library-wide pieces of the C ABI: version and thread-local error text.
#include "fg_common.h"

namespace fg {
char* error_buffer() {
  static thread_local char buf[kErrorBufferBytes] = {0};
  return buf;
}
int cu_count_or_default() {
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 256;
  return n;
}

hipError_t& launch_status() {
  static thread_local hipError_t status = hipSuccess;
  return status;
}
}  // namespace fg

extern "C" int fg_version(void) { return 100; }
extern "C" const char* fg_last_error_string(void) { return fg::error_buffer(); }

// 0 when `stream` is not being captured into a HIP graph, else the id of the capture in progress.  The host binding
// uses it to keep memory it allocated inside a capture (which belongs to that graph) apart from memory that
// outlives graphs.
extern "C" unsigned long long fg_stream_capture_id(void* stream) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  unsigned long long id = 0;
  if (hipStreamGetCaptureInfo((hipStream_t)stream, &status, &id) != hipSuccess) return 0;
  return status == hipStreamCaptureStatusActive ? (id != 0 ? id : ~0ull) : 0;
}

// ---------------------------------------------------------------------------------------------
// Measurement aid: the time a kernel needs merely to read `bytes` of device memory once (16-byte non-temporal loads,
// eight in flight per lane, all compute units).  The decode GEMMs are bound by reading their weights; benchmarks
// put their times next to this floor for a buffer of the same size.
// ---------------------------------------------------------------------------------------------
namespace fg {
namespace {
constexpr int kProbeThreads = 512, kProbeUnroll = 8;
__global__ __launch_bounds__(kProbeThreads) void stream_read_kernel(const u32x4* __restrict__ src, int64_t n16, uint32_t* sink) {
  const int64_t stride = (int64_t)gridDim.x * kProbeThreads;
  int64_t i = (int64_t)blockIdx.x * kProbeThreads + threadIdx.x;
  u32x4 acc = {0u, 0u, 0u, 0u};
  for (; i + (kProbeUnroll - 1) * stride < n16; i += kProbeUnroll * stride) {
    u32x4 v[kProbeUnroll];
#pragma unroll
    for (int j = 0; j < kProbeUnroll; ++j) v[j] = __builtin_nontemporal_load(src + i + j * stride);
#pragma unroll
    for (int j = 0; j < kProbeUnroll; ++j) acc ^= v[j];
  }
  for (; i < n16; i += stride) acc ^= __builtin_nontemporal_load(src + i);
  // the loads must not be optimised away; the store happens for no real input
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9E3779B9u && sink) sink[0] = acc.x;
}
}  // namespace
}  // namespace fg

extern "C" int fg_stream_read_probe(const void* src, size_t bytes, void* sink, void* stream) {
  using namespace fg;
  if (bytes == 0) return FG_OK;
  if (!src || (uintptr_t)src % 16 != 0) FG_FAIL(FG_ERR_INVALID_ARG, "fg_stream_read_probe: src must be a 16-byte aligned device pointer");
  const int64_t n16 = (int64_t)(bytes / 16);
  int blocks = cu_count_or_default() * 4;
  const int64_t want = (n16 + kProbeThreads - 1) / kProbeThreads;
  if (want < blocks) blocks = want > 0 ? (int)want : 1;
  FG_LAUNCH(stream_read_kernel, dim3((uint32_t)blocks), dim3(kProbeThreads), 0, (hipStream_t)stream,
            reinterpret_cast<const u32x4*>(src), n16, reinterpret_cast<uint32_t*>(sink));
  FG_CHECK_LAUNCH("stream_read_kernel");
  return FG_OK;
}
