// Thread-local error text behind ct_last_error().
#pragma once

#include <hip/hip_runtime.h>

#include "../../include/ct_hotpath.h"

namespace ct {

// Records a formatted message for the calling thread and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// Returns CT_OK, or records the HIP error of the most recent launch.
int check_launch(const char* what);

// Calls the thread's launch hook (if any) around a kernel launch.
void notify_launch(const char* kernel, int phase, hipStream_t stream);

// Brackets one kernel launch with the launch hook; evaluates to the launch status.
struct LaunchScope {
  const char* kernel;
  hipStream_t stream;
  LaunchScope(const char* k, hipStream_t s) : kernel(k), stream(s) { notify_launch(kernel, 0, stream); }
  int done() {
    const int rc = check_launch(kernel);
    notify_launch(kernel, 1, stream);
    return rc;
  }
};

}  // namespace ct

#define CT_REQUIRE(cond, ...)                                          \
  do {                                                                 \
    if (!(cond)) return ::ct::fail(CT_INVALID_ARGUMENT, __VA_ARGS__);  \
  } while (0)
