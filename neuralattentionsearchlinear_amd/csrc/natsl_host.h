// Host-side helpers shared by the C-ABI entry points.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>

#include "../../include/natsl.h"

namespace natsl {

char* error_buffer();  // thread-local, 512 bytes (defined in natsl_route.hip)

inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(NATSL_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return NATSL_OK;
}

inline int cdiv(int a, int b) { return (a + b - 1) / b; }

}  // namespace natsl
