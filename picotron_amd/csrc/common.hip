// Status plumbing shared by every entry point of libpicotron_amd.so.
#include "common.h"

#include <cstdarg>
#include <cstdio>

namespace pico {

static thread_local char g_last_error[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(PICO_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(e));
  return PICO_OK;
}

}  // namespace pico

extern "C" const char* pico_version(void) { return "picotron_amd 0.1 gfx950"; }
extern "C" const char* pico_last_error(void) { return pico::g_last_error; }
