// Host-side plumbing shared by every translation unit of libtorchtune_amd.so: error reporting across
// the C ABI, argument checks, and a few device helpers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/torchtune_amd.h"

namespace ttamd {

// Thread-local message returned by ttamd_last_error(); defined in capi.hip.
char* error_buffer();
constexpr int kErrorBufferBytes = 512;

inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), kErrorBufferBytes, fmt, ap);
  va_end(ap);
  return code;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

#define TT_REQUIRE(cond, ...)                                 \
  do {                                                        \
    if (!(cond)) return ::ttamd::fail(TTAMD_EINVAL, __VA_ARGS__); \
  } while (0)

// Call after a kernel launch: turns a launch failure into a C-ABI error code without synchronising.
inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TTAMD_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
  return TTAMD_OK;
}

inline bool is_pow2(int64_t v) { return v > 0 && (v & (v - 1)) == 0; }

constexpr int kWave = 64;  // CDNA wavefront width

}  // namespace ttamd
