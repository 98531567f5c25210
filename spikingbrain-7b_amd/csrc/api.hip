// Error plumbing and version query of the C ABI.
#include <stdarg.h>
#include <stdio.h>

#include "common.h"

namespace {
thread_local char g_err[512] = "";
}

namespace sb_host {

void set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char *what) {
  const hipError_t e = hipGetLastError();
  if (e == hipSuccess) return SB_OK;
  set_error("%s: launch failed: %s", what, hipGetErrorString(e));
  return (int)e;
}

}  // namespace sb_host

extern "C" int sb_abi_version(void) { return SB_ABI_VERSION; }
extern "C" const char *sb_last_error(void) { return g_err; }

extern "C" int sb_stream_capture_id(void *stream, uint64_t *id) {
  if (!id) return sb_host::fail(SB_ERR_INVALID, "sb_stream_capture_id: null id");
  *id = 0;
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  unsigned long long seq = 0;
  const hipError_t e = hipStreamGetCaptureInfo((hipStream_t)stream, &status, &seq);
  if (e != hipSuccess) return sb_host::fail((int)e, "sb_stream_capture_id: %s", hipGetErrorString(e));
  if (status == hipStreamCaptureStatusActive) *id = seq ? (uint64_t)seq : ~(uint64_t)0;
  return SB_OK;
}
