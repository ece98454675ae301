// Shared helpers of the gfx950 Marlin library: error reporting, vector types
// and the layout constants every kernel agrees on.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>

#include "sonar_marlin.h"

namespace sonar {

// ---- error reporting ------------------------------------------------------
char* last_error_buffer();  // thread-local, 512 bytes

inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(last_error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

#define SONAR_REQUIRE(cond, ...)                          \
  do {                                                    \
    if (!(cond)) return ::sonar::fail(SONAR_E_INVALID, __VA_ARGS__); \
  } while (0)

#define SONAR_HIP(expr)                                                     \
  do {                                                                      \
    hipError_t e_ = (expr);                                                 \
    if (e_ != hipSuccess)                                                   \
      return ::sonar::fail(SONAR_E_RUNTIME, "%s failed: %s", #expr,         \
                           hipGetErrorString(e_));                          \
  } while (0)

inline int launch_status(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess)
    return fail(SONAR_E_RUNTIME, "launch of %s failed: %s", what, hipGetErrorString(e));
  return SONAR_OK;
}

// ---- vector types ---------------------------------------------------------
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx2_t __attribute__((ext_vector_type(2)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
// address spaces of the asynchronous global -> LDS copy builtin
typedef __attribute__((address_space(3))) void lds_void_t;
typedef __attribute__((address_space(1))) const void glb_void_t;

// ---- layout constants -----------------------------------------------------
// Marlin order: tiles of 16 (k) x 64 (n), 128 words each, stored k-tile major.
constexpr int kMarlinTileK = 16;
constexpr int kMarlinTileN = 64;
constexpr int kMarlinTileWords = 128;
// gfx950 streaming order: 64-column strips, each a run of 32-row chunks of
// 256 words (1 KiB); lane L of a wavefront owns words 4L..4L+3 of a chunk.
constexpr int kStripN = 64;
constexpr int kChunkK = 32;
constexpr int kChunkWords = 256;

}  // namespace sonar
