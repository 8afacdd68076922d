// Narrow floating-point formats on the path: decode / encode as closed forms, usable on host
// and device.  Format constants as in the reference type table
// (python/triton/language/core.py:352-363: fp8e4nv = 1-4-3 bias 7, fp8e5 = 1-5-2 bias 15) and
// its conversion tests (python/test/unit/language/test_conversions.py:295-303); e2m1 and e8m0
// follow the OCP Microscaling Formats specification v1.0 (not present in the reference).
#pragma once
#include <stdint.h>
#include <string.h>
#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define MI355_HD __host__ __device__ inline
#else
#define MI355_HD inline
#endif

namespace mi355 {

MI355_HD float bits_to_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
MI355_HD uint32_t f32_to_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}

// e4m3fn: no infinity, NaN = S.1111.111, max finite 448, subnormal step 2^-9.
MI355_HD float e4m3_to_f32(uint8_t c) {
  uint32_t s = (uint32_t)(c >> 7) << 31, e = (c >> 3) & 15, m = c & 7;
  if (e == 15 && m == 7) return bits_to_f32(s | 0x7FC00000u);
  if (e == 0) {
    float v = (float)m * 0.001953125f;  // m * 2^-9, exact
    return bits_to_f32(f32_to_bits(v) | s);
  }
  return bits_to_f32(s | ((e + 120) << 23) | (m << 20));
}

// e5m2: IEEE-like (inf / NaN kept); it is the high byte of an fp16.
MI355_HD float e5m2_to_f32(uint8_t c) {
  uint32_t s = (uint32_t)(c >> 7) << 31, e = (c >> 2) & 31, m = c & 3;
  if (e == 31) return bits_to_f32(s | 0x7F800000u | (m << 21));
  if (e == 0) {
    float v = (float)m * 0.0000152587890625f;  // m * 2^-16, exact
    return bits_to_f32(f32_to_bits(v) | s);
  }
  return bits_to_f32(s | ((e + 112) << 23) | (m << 21));
}

// e2m1: codes 0..7 -> {0, .5, 1, 1.5, 2, 3, 4, 6}, bit 3 = sign.
MI355_HD float e2m1_to_f32(uint8_t c) {
  uint32_t s = (uint32_t)((c >> 3) & 1) << 31, e = (c >> 1) & 3, m = c & 1;
  if (e == 0) return bits_to_f32(s | (m ? 0x3F000000u : 0u));
  return bits_to_f32(s | ((e + 126) << 23) | (m << 22));
}

// e8m0: b -> 2^(b-127); 255 is NaN.  2^-127 is an fp32 subnormal and exact.
MI355_HD float e8m0_to_f32(uint8_t b) {
  if (b == 255) return bits_to_f32(0x7FC00000u);
  if (b == 0) return bits_to_f32(0x00400000u);
  return bits_to_f32((uint32_t)b << 23);
}

// fp32 -> fp8, round to nearest even, finite overflow saturates to the largest finite code
// (448 / 57344, the downcast maxima of test_conversions.py:307-329); NaN stays NaN.
MI355_HD uint8_t f32_to_fp8(float f, int ebits, int mbits, int bias, uint8_t max_code, uint8_t nan_code) {
  uint32_t u = f32_to_bits(f);
  uint8_t s = (uint8_t)((u >> 31) << 7);
  uint32_t a = u & 0x7FFFFFFFu;
  if (a > 0x7F800000u) return s | nan_code;
  int e = (int)(a >> 23) - 127;  // unbiased
  uint32_t mant = (a & 0x7FFFFFu) | 0x800000u;
  if (a < 0x00800000u) return s;  // fp32 subnormal -> 0
  int emin = 1 - bias;
  int shift = 23 - mbits;  // bits to drop for a normal result
  if (e < emin) shift += emin - e;
  if (shift > 31) return s;
  uint32_t kept = mant >> shift;
  uint32_t rem = mant & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (kept & 1u))) kept++;
  // kept now holds [implicit one | mantissa] for normals, or the subnormal mantissa
  uint32_t code;
  if (e < emin) {
    code = kept;  // may carry into the first normal: encoding is contiguous
  } else {
    code = ((uint32_t)(e + bias) << mbits) + (kept - (1u << mbits));
  }
  if (code > max_code) code = max_code;
  (void)ebits;
  return s | (uint8_t)code;
}
MI355_HD uint8_t f32_to_e4m3(float f) { return f32_to_fp8(f, 4, 3, 7, 0x7E, 0x7F); }
MI355_HD uint8_t f32_to_e5m2(float f) { return f32_to_fp8(f, 5, 2, 15, 0x7B, 0x7F); }

}  // namespace mi355
