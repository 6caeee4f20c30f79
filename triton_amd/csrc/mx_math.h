// Scalar MX (microscaling) arithmetic shared by the quantise / dequantise kernels and the GEMM.
// Every function is `__host__ __device__` so the same code can be checked on the CPU.
//
// The conversions are closed forms of the bit algorithms in
// python/triton_kernels/triton_kernels/numerics_details/mxfp.py:251-327 (downcast) and :346-429 (upcast).
#pragma once
#include "common.h"

namespace tk {

__host__ __device__ inline uint32_t hd_f32_bits(float f) {
  uint32_t u;
  __builtin_memcpy(&u, &f, 4);
  return u;
}
__host__ __device__ inline float hd_bits_f32(uint32_t u) {
  float f;
  __builtin_memcpy(&f, &u, 4);
  return f;
}

// Largest finite / largest power-of-two magnitude of the element formats (mxfp.py:187-189,
// mxfp_details/_downcast_to_mxfp.py:13-30).
__host__ __device__ inline float mx_max_q(int kind) {
  return kind == TK_E2M1 ? 6.0f : (kind == TK_E4M3 ? 448.0f : 57344.0f);
}
__host__ __device__ inline float mx_max_pow2_q(int kind) {
  return kind == TK_E2M1 ? 4.0f : (kind == TK_E4M3 ? 256.0f : 32768.0f);
}

// Bit pattern (an fp32 power of two, or 0) of the dequantisation scale of a block whose largest
// magnitude is `absmax` (mxfp.py:255-268).
__host__ __device__ inline uint32_t mx_scale_bits(float absmax, int kind, int rounding) {
  if (rounding == TK_MX_ROUND_UP) {
    float d = absmax / mx_max_q(kind);
    return (hd_f32_bits(d) + 0x007FFFFFu) & 0x7F800000u;
  }
  float d = absmax / mx_max_pow2_q(kind);
  return hd_f32_bits(d) & 0x7F800000u;
}

// 1/scale, 0 for a zero scale (mxfp.py:278).  The scale is a power of two so the quotient is exact.
__host__ __device__ inline float mx_inv_scale(uint32_t sbits) {
  return sbits == 0 ? 0.0f : 1.0f / hd_bits_f32(sbits);
}

// fp32 -> e2m1 code (bit 3 sign, bits 2:1 exponent, bit 0 mantissa); round to nearest even, saturate to
// +-6, NaN/inf -> +-6 (mxfp.py:298-327).
//   |q| <  1 : multiples of 0.5  -> magic-number add rounds 2|q| to an integer in {0,1,2}
//   |q| >= 1 : one mantissa bit  -> integer round of the fp32 pattern at bit 22
__host__ __device__ inline uint32_t e2m1_code(float q) {
  uint32_t u = hd_f32_bits(q);
  uint32_t sign = (u >> 28) & 0x8u;
  uint32_t a = u & 0x7FFFFFFFu;
  uint32_t code;
  if (a < 0x3F800000u) {
    float t = hd_bits_f32(a) * 2.0f + 12582912.0f;
    code = hd_f32_bits(t) & 0x3u;
  } else {
    uint32_t r = a + 0x1FFFFFu + ((a >> 22) & 1u);
    code = (r >> 22) - 252u;
    code = code > 7u ? 7u : code;
  }
  return sign | code;
}

// fp32 (already clamped to +-448) -> OCP e4m3fn byte, round to nearest even.
__host__ __device__ inline uint32_t e4m3_byte(float q) {
  uint32_t u = hd_f32_bits(q);
  uint32_t sign = (u >> 24) & 0x80u;
  uint32_t a = u & 0x7FFFFFFFu;
  if (a > 0x7F800000u) return sign | 0x7Fu;  // NaN
  uint32_t code;
  if (a < 0x3C800000u) {  // below 2^-6: subnormal step 2^-9
    float t = hd_bits_f32(a) * 512.0f + 12582912.0f;
    code = hd_f32_bits(t) & 0xFu;
  } else {
    uint32_t r = a + 0x7FFFFu + ((a >> 20) & 1u);
    code = (r >> 20) - 960u;
    code = code > 0x7Eu ? 0x7Eu : code;
  }
  return sign | code;
}

// fp32 (already clamped to +-57344) -> OCP e5m2 byte, round to nearest even.
__host__ __device__ inline uint32_t e5m2_byte(float q) {
  uint32_t u = hd_f32_bits(q);
  uint32_t sign = (u >> 24) & 0x80u;
  uint32_t a = u & 0x7FFFFFFFu;
  if (a > 0x7F800000u) return sign | 0x7Fu;  // NaN
  uint32_t code;
  if (a < 0x38800000u) {  // below 2^-14: subnormal step 2^-16
    float t = hd_bits_f32(a) * 65536.0f + 12582912.0f;
    code = hd_f32_bits(t) & 0x7u;
  } else {
    uint32_t r = a + 0xFFFFFu + ((a >> 21) & 1u);
    code = (r >> 21) - 448u;
    code = code > 0x7Bu ? 0x7Bu : code;
  }
  return sign | code;
}

// NaN-propagating clamp to [-m, m] (torch.clamp keeps NaN, mxfp.py:295).
__host__ __device__ inline float mx_clamp(float q, float m) { return q > m ? m : (q < -m ? -m : q); }

// e2m1 code -> value as bf16 bits {0,.5,1,1.5,2,3,4,6} with the sign in bit 15 (mxfp.py:346-361).
__host__ __device__ inline uint32_t e2m1_to_bf16_bits(uint32_t code) {
  uint32_t c = code & 7u;
  uint32_t mag = c < 2u ? (c ? 0x3F00u : 0u) : 0x3F00u + (c << 6);
  return mag | ((code & 8u) << 12);
}

__host__ __device__ inline float e4m3_to_f32(uint32_t b) {
  uint32_t sign = (b & 0x80u) << 24;
  uint32_t e = (b >> 3) & 0xFu, m = b & 7u;
  if (e == 0xFu && m == 7u) return hd_bits_f32(sign | 0x7FC00000u);
  if (e == 0) return hd_bits_f32(sign | hd_f32_bits((float)m * 0.001953125f));  // m * 2^-9
  return hd_bits_f32(sign | ((e + 120u) << 23) | (m << 20));
}

__host__ __device__ inline float e5m2_to_f32(uint32_t b) {
  uint32_t sign = (b & 0x80u) << 24;
  uint32_t e = (b >> 2) & 0x1Fu, m = b & 3u;
  if (e == 0x1Fu) return hd_bits_f32(sign | 0x7F800000u | (m << 21));
  if (e == 0) return hd_bits_f32(sign | hd_f32_bits((float)m * 0.0000152587890625f));  // m * 2^-16
  return hd_bits_f32(sign | ((e + 112u) << 23) | (m << 21));
}

// Dequantised value in fp32: element * 2^(scale-127), clamped to +-max_finite; NaN is kept
// (mxfp.py:394-415).  `scale_byte` 0 gives scale bits 0 = 0.0f, 0xFF gives +inf.
__host__ __device__ inline float mx_dequant(float elem, uint32_t scale_byte, float max_finite, bool keep_inf) {
  float s = hd_bits_f32(scale_byte << 23);
  float v = elem * s;
  float c = v > max_finite ? max_finite : (v < -max_finite ? -max_finite : v);
  if (keep_inf) {
    uint32_t eb = hd_f32_bits(elem) & 0x7FFFFFFFu;
    if (eb == 0x7F800000u) c = elem;
  }
  return c;
}

}  // namespace tk
