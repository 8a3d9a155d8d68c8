// Host-side helpers for the C-ABI entry points: status codes, error text, argument checks.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/hpfp8.h"

namespace hpfp8 {

char* error_buffer();  // thread-local, defined in capi.hip
int prepare_scratch();  // quantize.hip: resolves the no-allocation entry point's device memory on the current device

inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(HPFP8_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(e));
  return HPFP8_OK;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace hpfp8

#define HPFP8_REQUIRE(cond, code, ...) \
  do {                                 \
    if (!(cond)) return ::hpfp8::fail(code, __VA_ARGS__); \
  } while (0)
