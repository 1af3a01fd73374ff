// Shared by every translation unit of libjpt_mi355.so: status codes, the
// thread-local error message and small device helpers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>

#include "jpt_mi355.h"

namespace jpt {

char* error_buffer();  // thread-local, 512 bytes (defined in api.cpp)

inline int32_t fail(int32_t code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

#define JPT_REQUIRE(cond, ...)                         \
  do {                                                 \
    if (!(cond)) return jpt::fail(JPT_E_BADARG, __VA_ARGS__); \
  } while (0)

// A HIP runtime call that must succeed.
#define JPT_HIP(call)                                                            \
  do {                                                                           \
    hipError_t jpt_hip_e = (call);                                               \
    if (jpt_hip_e != hipSuccess)                                                 \
      return jpt::fail(JPT_E_HIP, "%s: %s", #call, hipGetErrorString(jpt_hip_e)); \
  } while (0)

// Checks the launch that was just enqueued.
inline int32_t launch_status(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess)
    return fail(JPT_E_HIP, "%s: %s", what, hipGetErrorString(e));
  return JPT_OK;
}

inline int elem_size(int32_t dtype) {
  return dtype == JPT_BF16 ? 2 : dtype == JPT_F32 ? 4 : dtype == JPT_I8 ? 1 : 0;
}

inline bool aligned(const void* p, size_t a) {
  return (reinterpret_cast<uintptr_t>(p) % a) == 0;
}

// ---- device helpers --------------------------------------------------------

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) {
  return __uint_as_float(static_cast<uint32_t>(h) << 16);
}

// float32 -> bfloat16 bits, round to nearest even, NaN kept quiet.
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}

__device__ __forceinline__ float round_to_bf16(float f) {
  return bf16_bits_to_f32(f32_to_bf16_bits(f));
}

__device__ __forceinline__ float load_as_f32(const void* p, int64_t i, int dtype) {
  if (dtype == JPT_BF16) return bf16_bits_to_f32(static_cast<const uint16_t*>(p)[i]);
  if (dtype == JPT_F32) return static_cast<const float*>(p)[i];
  return static_cast<float>(static_cast<const int8_t*>(p)[i]);
}

__device__ __forceinline__ void store_from_f32(void* p, int64_t i, int dtype, float v) {
  if (dtype == JPT_BF16)
    static_cast<uint16_t*>(p)[i] = f32_to_bf16_bits(v);
  else
    static_cast<float*>(p)[i] = v;
}

}  // namespace jpt
