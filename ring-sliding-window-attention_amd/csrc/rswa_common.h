// Shared host/device helpers for the rswa kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/rswa.h"

namespace rswa {

// ---- error reporting -------------------------------------------------------
char* last_error_buffer();  // thread-local, 512 bytes
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

#define RSWA_REQUIRE(cond, code, ...)      \
  do {                                     \
    if (!(cond)) return ::rswa::fail((code), __VA_ARGS__); \
  } while (0)

// A launch is bracketed by these two: the first drops whatever error an earlier, unrelated
// HIP call of this thread left behind, so that the second reports the launch's own only.
inline void clear_launch_error() { (void)hipGetLastError(); }
inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(RSWA_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return RSWA_OK;
}

// ---- vector types ----------------------------------------------------------
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8;
typedef __attribute__((__vector_size__(4 * sizeof(_Float16)))) _Float16 f16x4;
typedef __attribute__((__vector_size__(2 * sizeof(_Float16)))) _Float16 f16x2;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef __attribute__((__vector_size__(8 * sizeof(float)))) float f32x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4;

static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace rswa
