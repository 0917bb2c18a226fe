// Host-side plumbing of the C ABI: thread-local error text, launch checking, version.
#include "device_utils.h"
#include "relax_amd.h"

namespace relax_amd {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: kernel launch failed: %s", what, hipGetErrorString(e));
    return RELAX_AMD_ELAUNCH;
  }
  return RELAX_AMD_OK;
}

}  // namespace relax_amd

extern "C" int relax_amd_version(void) { return RELAX_AMD_ABI_VERSION; }
extern "C" const char* relax_amd_last_error(void) { return relax_amd::g_error; }
