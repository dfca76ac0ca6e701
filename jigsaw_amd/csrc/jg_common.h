// Shared helpers for the jigsaw HIP kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "../../include/jigsaw_hip.h"

namespace jg {

// Thread-local message of the most recent failure on this host thread.
char* last_error_buf();
void set_error(const char* fmt, ...);

#define JG_FAIL(code, ...)        \
  do {                            \
    ::jg::set_error(__VA_ARGS__); \
    return (code);                \
  } while (0)

#define JG_REQUIRE(cond, ...)                         \
  do {                                                \
    if (!(cond)) JG_FAIL(JG_ERR_BAD_ARG, __VA_ARGS__); \
  } while (0)

// Launch check: picks up a launch-time error without synchronising the device.
#define JG_CHECK_LAUNCH(name)                                              \
  do {                                                                     \
    hipError_t e__ = hipGetLastError();                                    \
    if (e__ != hipSuccess)                                                 \
      JG_FAIL(JG_ERR_LAUNCH, "%s: launch failed: %s", (name),              \
              hipGetErrorString(e__));                                     \
  } while (0)

static inline size_t dtype_size(int dtype) {
  switch (dtype) {
    case JG_F32: return 4;
    case JG_BF16: return 2;
    case JG_F16: return 2;
    default: return 0;
  }
}

// ---- bf16 <-> f32 (round to nearest even, NaN kept quiet), as torch rounds ----
__host__ __device__ static inline float bf16_to_f32(uint16_t h) {
  union { uint32_t u; float f; } c;
  c.u = ((uint32_t)h) << 16;
  return c.f;
}
__host__ __device__ static inline uint16_t f32_to_bf16(float f) {
  union { uint32_t u; float f; } c;
  c.f = f;
  if ((c.u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)0x7fc0;
  uint32_t r = c.u + 0x7fffu + ((c.u >> 16) & 1u);
  return (uint16_t)(r >> 16);
}

static inline int cdiv(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }

}  // namespace jg
