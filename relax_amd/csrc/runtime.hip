// Host-side plumbing of the C ABI: thread-local error text, launch checking, version.
#include <atomic>

#include "device_utils.h"
#include "loss_math.h"
#include "relax_amd.h"

namespace relax_amd {

static thread_local char g_error[512] = "";
static thread_local const char* g_last_kernel = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int check_launch(const char* what) {
  g_last_kernel = what;
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: kernel launch failed: %s", what, hipGetErrorString(e));
    return RELAX_AMD_ELAUNCH;
  }
  return RELAX_AMD_OK;
}

static std::atomic<int> g_kernel_choice{RELAX_AMD_KERNEL_AUTO};

int kernel_choice() { return g_kernel_choice.load(std::memory_order_relaxed); }

const char* policy_loss_args_size_error(const relax_amd_policy_loss_args* a) {
  return a->struct_size < sizeof(relax_amd_policy_loss_args)
             ? "args->struct_size is smaller than this library's relax_amd_policy_loss_args: set it to "
               "sizeof(relax_amd_policy_loss_args) and rebuild against the current header"
             : nullptr;
}

}  // namespace relax_amd

extern "C" int relax_amd_set_kernel_choice(int choice) {
  if (choice < RELAX_AMD_KERNEL_AUTO || choice > RELAX_AMD_KERNEL_RESIDENT) {
    relax_amd::set_error("set_kernel_choice: unknown choice %d", choice);
    return RELAX_AMD_EINVAL;
  }
  return relax_amd::g_kernel_choice.exchange(choice, std::memory_order_relaxed);
}

extern "C" int relax_amd_version(void) { return RELAX_AMD_ABI_VERSION; }
extern "C" const char* relax_amd_last_error(void) { return relax_amd::g_error; }
extern "C" const char* relax_amd_last_kernel(void) { return relax_amd::g_last_kernel; }
