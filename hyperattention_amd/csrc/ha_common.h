// Shared host/device helpers for libhyperattn (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/hyperattn.h"

#define HA_WAVE 64

// ---- error reporting (host) -----------------------------------------------------------------
char* ha_error_buffer();  // thread-local, 512 bytes, defined in api.hip

static inline int ha_fail(int status, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(ha_error_buffer(), 512, fmt, ap);
  va_end(ap);
  return status;
}

static inline int ha_launch_status(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return ha_fail((int)e, "%s: launch failed: %s", what, hipGetErrorString(e));
  return HA_OK;
}

#define HA_REQUIRE(cond, status, ...)            \
  do {                                           \
    if (!(cond)) return ha_fail(status, __VA_ARGS__); \
  } while (0)

// ---- element types --------------------------------------------------------------------------
typedef _Float16 f16_t;
typedef __bf16 bf16_t;

typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T>
struct ElemTraits;
template <>
struct ElemTraits<f16_t> {
  typedef f16x8 vec8;
  typedef f16x4 vec4;
  typedef f16x2 vec2;
};
template <>
struct ElemTraits<bf16_t> {
  typedef bf16x8 vec8;
  typedef bf16x4 vec4;
  typedef bf16x2 vec2;
};

__device__ __forceinline__ float ha_to_float(f16_t v) { return (float)v; }
__device__ __forceinline__ float ha_to_float(bf16_t v) { return (float)v; }

// index loads of either width
__device__ __forceinline__ int ha_load_idx(const void* base, int64_t off, int is64) {
  // one load either way (row numbers fit the low word of a little-endian int64), so that the value
  // is not consumed by a select right behind the load
  return *reinterpret_cast<const int32_t*>(static_cast<const char*>(base) + (off << (is64 ? 3 : 2)));
}
