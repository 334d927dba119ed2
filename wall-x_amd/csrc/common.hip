// Error reporting and device queries shared by every entry point of libwallx_mi355.
#include "common.h"

#include <cstdarg>
#include <cstdio>

namespace wx {

static thread_local char g_error[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

static thread_local int g_gemm_path = 0;
void gemm_path_reset() { g_gemm_path = 0; }
void gemm_path_note(int bit) { g_gemm_path |= bit; }

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) return WX_OK;
  return fail(WX_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
}

int device_cu_count() {
  static thread_local int cached_dev = -1;
  static thread_local int cached_cus = 0;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  if (dev != cached_dev) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached_dev = dev;
    cached_cus = n;
  }
  return cached_cus;
}

}  // namespace wx

extern "C" const char* wx_last_error_string(void) { return wx::g_error; }
extern "C" int wx_last_gemm_path(void) { return wx::g_gemm_path; }
extern "C" int wx_abi_version(void) { return 1; }

extern "C" int wx_stream_capture_id(wx_stream_t stream, unsigned long long* id) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  unsigned long long cap = 0;
  if (hipStreamGetCaptureInfo(reinterpret_cast<hipStream_t>(stream), &status, &cap) != hipSuccess) {
    (void)hipGetLastError();
    return wx::fail(WX_ERR_LAUNCH, "wx_stream_capture_id: hipStreamGetCaptureInfo failed");
  }
  if (status != hipStreamCaptureStatusActive) cap = 0;
  if (id != nullptr) *id = cap;
  return status == hipStreamCaptureStatusActive ? 1 : 0;
}
