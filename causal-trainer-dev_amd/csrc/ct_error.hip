#include "ct_error.h"

#include <stdarg.h>
#include <stdio.h>

namespace ct {

static thread_local char g_error[512] = "";
static thread_local ct_launch_hook g_hook = nullptr;
static thread_local void* g_hook_user = nullptr;

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* what) {
  hipError_t err = hipGetLastError();
  if (err == hipSuccess) return CT_OK;
  return fail(CT_LAUNCH_FAILED, "%s: %s", what, hipGetErrorString(err));
}

void notify_launch(const char* kernel, int phase, hipStream_t stream) {
  if (g_hook) g_hook(g_hook_user, kernel, phase, static_cast<void*>(stream));
}

}  // namespace ct

extern "C" void ct_set_launch_hook(ct_launch_hook hook, void* user) {
  ct::g_hook = hook;
  ct::g_hook_user = user;
}

extern "C" const char* ct_last_error(void) { return ct::g_error; }

extern "C" int32_t ct_abi_version(void) { return 2; }
