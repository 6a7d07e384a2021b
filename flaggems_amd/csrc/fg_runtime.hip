// Library-wide pieces of the C ABI: version and thread-local error text.
#include "fg_common.h"

namespace fg {
char* error_buffer() {
  static thread_local char buf[kErrorBufferBytes] = {0};
  return buf;
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
