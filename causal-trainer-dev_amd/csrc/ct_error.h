// Thread-local error text behind ct_last_error().
#pragma once

#include <hip/hip_runtime.h>

#include "../../include/ct_hotpath.h"

namespace ct {

// Records a formatted message for the calling thread and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// Returns CT_OK, or records the HIP error of the most recent launch.
int check_launch(const char* what);

}  // namespace ct

#define CT_REQUIRE(cond, ...)                                          \
  do {                                                                 \
    if (!(cond)) return ::ct::fail(CT_INVALID_ARGUMENT, __VA_ARGS__);  \
  } while (0)
