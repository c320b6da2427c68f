#include "ct_error.h"

#include <stdarg.h>
#include <stdint.h>
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

// Plain copy of `bytes` (a multiple of 16) with 16-byte accesses: the kernel of known traffic
// that hardware counters (FETCH_SIZE, WRITE_SIZE) are scaled against.
__global__ __launch_bounds__(256) void ct_calibration_copy_kernel(const uint4* src, uint4* dst,
                                                                  size_t count) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (size_t)gridDim.x * 256)
    dst[i] = src[i];
}

extern "C" int32_t ct_calibration_copy(void* stream, void* dst, const void* src, size_t bytes) {
  if (!dst || !src || bytes == 0 || bytes % 16 != 0 ||
      ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15u))
    return ct::fail(CT_INVALID_ARGUMENT, "ct_calibration_copy: pointers and size must be 16-byte multiples");
  ct::LaunchScope scope("ct_calibration_copy_kernel", (hipStream_t)stream);
  hipLaunchKernelGGL(ct_calibration_copy_kernel, dim3(256 * 16), dim3(256), 0, (hipStream_t)stream,
                     static_cast<const uint4*>(src), static_cast<uint4*>(dst), bytes / 16);
  return scope.done();
}

extern "C" void ct_set_launch_hook(ct_launch_hook hook, void* user) {
  ct::g_hook = hook;
  ct::g_hook_user = user;
}

extern "C" const char* ct_last_error(void) { return ct::g_error; }

extern "C" int32_t ct_abi_version(void) { return 3; }
