// Shared host-side helpers for the C ABI translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdio>

#include "kvax_amd.h"

namespace kvax {

// Records a formatted message for kvax_last_error() and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(KVAX_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
  return KVAX_OK;
}

inline int cdiv(int a, int b) { return (a + b - 1) / b; }

}  // namespace kvax
