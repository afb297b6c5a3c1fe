// Shared host/device helpers of the KvsAll kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <type_traits>

#include "../../include/kge_hip.h"
#include "kge_host.h"

namespace kge {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

// ---- host-side error plumbing -------------------------------------------------------------
int set_error(int code, const char* fmt, ...);
void clear_error();

#define KGE_REQUIRE(cond, code, ...)                      \
  do {                                                    \
    if (!(cond)) return ::kge::set_error(code, __VA_ARGS__); \
  } while (0)

#define KGE_HIP_CHECK(expr)                                                              \
  do {                                                                                   \
    hipError_t _e = (expr);                                                              \
    if (_e != hipSuccess)                                                                \
      return ::kge::set_error(KGE_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(_e)); \
  } while (0)

#define KGE_LAUNCH_CHECK(name)                                                          \
  do {                                                                                  \
    hipError_t _e = hipGetLastError();                                                  \
    if (_e != hipSuccess)                                                               \
      return ::kge::set_error(KGE_ERR_HIP, "launch of %s failed: %s", name, hipGetErrorString(_e)); \
  } while (0)

// ---- MFMA 32x32 accumulator layout --------------------------------------------------------
// acc[i] of lane l holds output (row_of(i, l / 32), l % 32).
__device__ __forceinline__ int row_of(int i, int hf) { return ((i >> 2) << 3) + (hf << 2) + (i & 3); }

// Order-preserving map float -> uint32 (larger float <=> larger key); NaN is not handled.
__device__ __forceinline__ uint32_t f32_to_ordered(float f) {
  uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float ordered_to_f32(uint32_t k) {
  uint32_t u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
  return __uint_as_float(u);
}

// A threshold that every score equal to x beats in a float comparison (`s > just_below(x)` holds for s == x), as
// close below x as that allows.  One step down in the ordered encoding does it except around zero: the neighbour of
// +0 there is -0, which compares EQUAL to it, and the denormals next to them depend on the comparison honouring
// denormals; so for |x| below the smallest normal the answer is minus the smallest normal.  (-inf stays -inf.)
__device__ __forceinline__ float just_below(float x) {
  if (!(x > __uint_as_float(0xff800000u))) return x;                        // -inf, NaN
  if (__builtin_fabsf(x) < 1.17549435e-38f) return -1.17549435e-38f;
  return ordered_to_f32(f32_to_ordered(x) - 1u);
}

}  // namespace kge
