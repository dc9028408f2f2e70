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
constexpr int kProfileRing = 512;
static bool g_profile = false;
static hipEvent_t g_ev[kProfileRing][2];
static bool g_ev_made = false;
static int g_ev_next = 0;        // calls recorded since profiling was last enabled
DominantKernelTimer::DominantKernelTimer(hipStream_t st) : st_(st), on_(g_profile && g_ev_made && g_ev_next < kProfileRing) {
  if (on_) (void)hipEventRecord(g_ev[g_ev_next][0], st_);
}
DominantKernelTimer::~DominantKernelTimer() {
  if (on_) {
    (void)hipEventRecord(g_ev[g_ev_next][1], st_);
    ++g_ev_next;
  }
}
}  // namespace subspec

extern "C" int subspec_profile_enable(int on) {
  using namespace subspec;
  if (on && !g_ev_made) {
    for (int i = 0; i < kProfileRing; ++i) {
      SUBSPEC_CHECK_HIP(hipEventCreate(&g_ev[i][0]));
      SUBSPEC_CHECK_HIP(hipEventCreate(&g_ev[i][1]));
    }
    g_ev_made = true;
  }
  g_profile = on != 0;
  if (on) g_ev_next = 0;
  return SUBSPEC_OK;
}

extern "C" int subspec_profile_count(void) { return subspec::g_ev_next; }

extern "C" float subspec_profile_read_ms(int index) {
  using namespace subspec;
  if (!g_ev_made || index < 0 || index >= g_ev_next) return -1.f;
  if (hipEventSynchronize(g_ev[index][1]) != hipSuccess) return -1.f;
  float ms = -1.f;
  if (hipEventElapsedTime(&ms, g_ev[index][0], g_ev[index][1]) != hipSuccess) return -1.f;
  return ms;
}

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
