// Library-level entry points: ABI version and the thread-local error message.
#include "common.h"

namespace subspec {
static thread_local char g_error[512] = "";
void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}
}  // namespace subspec

extern "C" int subspec_abi_version(void) { return SUBSPEC_ABI_VERSION; }
extern "C" const char* subspec_last_error(void) { return subspec::g_error; }

// Host-to-device weight streaming: one asynchronous copy from pinned host memory on the caller's
// copy stream.  The caller owns ordering (events between the copy stream and the compute stream).
extern "C" int subspec_stream_copy_h2d(void* dst_device, const void* src_pinned_host, size_t bytes, void* stream) {
  if (!dst_device || !src_pinned_host) SUBSPEC_FAIL(SUBSPEC_ERR_ARG, "stream_copy_h2d: null pointer argument");
  if (bytes == 0) return SUBSPEC_OK;
  SUBSPEC_CHECK_HIP(hipMemcpyAsync(dst_device, src_pinned_host, bytes, hipMemcpyHostToDevice, (hipStream_t)stream));
  return SUBSPEC_OK;
}
