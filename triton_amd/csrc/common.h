// Shared declarations for the gfx950 kernels behind the C ABI of include/triton_amd.h.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/triton_amd.h"

namespace tk {

// Records a message for tk_last_error() and returns `code`.
int32_t fail(int32_t code, const char* fmt, ...);

inline int32_t check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TK_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return TK_OK;
}

inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;

// ---- scalar conversions usable on host and device --------------------------------------------
__host__ __device__ inline float bf16_bits_to_f32(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  __builtin_memcpy(&f, &u, 4);
  return f;
}

// fp32 -> bf16 bits, round to nearest even, NaN kept quiet (same as torch's cast).
__host__ __device__ inline uint16_t f32_to_bf16_bits(float f) {
  uint32_t u;
  __builtin_memcpy(&u, &f, 4);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
  uint32_t r = 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)((u + r) >> 16);
}

__device__ inline float f16_bits_to_f32(uint16_t b) {
  _Float16 h;
  __builtin_memcpy(&h, &b, 2);
  return (float)h;
}

__device__ inline uint16_t f32_to_f16_bits(float f) {
  _Float16 h = (_Float16)f;
  uint16_t b;
  __builtin_memcpy(&b, &h, 2);
  return b;
}

__device__ inline uint32_t f32_bits(float f) { return __builtin_bit_cast(uint32_t, f); }
__device__ inline float bits_f32(uint32_t u) { return __builtin_bit_cast(float, u); }

}  // namespace tk
