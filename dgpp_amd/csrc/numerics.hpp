// Bit-exact scalar codecs shared by host encoders and device kernels: bf16, OCP E4M3FN,
// E2M1 and E8M0. Value semantics follow the reference's src/common/dtypes.hpp:83-190 and
// src/kernels/latent_format.hpp:117-162; the arithmetic here is this library's own
// (field manipulation instead of search loops, usable from device code).
#pragma once

#include <cmath>
#include <cstdint>
#include <cstring>

#if defined(__HIPCC__)
#define DGPP_HD __host__ __device__
#else
#define DGPP_HD
#endif

namespace dgpp_amd {

DGPP_HD inline uint32_t f32_bits(float f) {
  return __builtin_bit_cast(uint32_t, f);
}
DGPP_HD inline float bits_f32(uint32_t u) {
  return __builtin_bit_cast(float, u);
}

DGPP_HD inline float bf16_to_f32(uint16_t b) { return bits_f32(static_cast<uint32_t>(b) << 16); }

// Round to nearest even; NaN -> canonical quiet NaN with the sign kept.
DGPP_HD inline uint16_t f32_to_bf16(float f) {
  const uint32_t u = f32_bits(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return static_cast<uint16_t>(((u >> 16) & 0x8000u) | 0x7FC0u);
  return static_cast<uint16_t>((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

// OCP E4M3FN: bias 7, no infinities, 0x7F / 0xFF are NaN, subnormals m * 2^-9.
DGPP_HD inline float e4m3_to_f32(uint8_t v) {
  const uint32_t sign = static_cast<uint32_t>(v & 0x80u) << 24;
  const uint32_t e = (v >> 3) & 0xFu, m = v & 7u;
  if (e == 0xFu && m == 7u) return bits_f32(sign | 0x7FC00000u);
  if (e == 0u) return bits_f32(f32_bits(static_cast<float>(m) * 0.001953125f) | sign);
  return bits_f32(sign | ((e + 120u) << 23) | (m << 20));
}

// Saturating round-to-nearest-even encode: |x| > 448 clamps to 448, NaN -> 0x7F with the sign.
DGPP_HD inline uint8_t f32_to_e4m3(float f) {
  const uint32_t u = f32_bits(f);
  const uint8_t sign = static_cast<uint8_t>((u >> 24) & 0x80u);
  uint32_t a = u & 0x7FFFFFFFu;
  if (a > 0x7F800000u) return sign | 0x7Fu;
  if (a >= 0x43E00000u) return sign | 0x7Eu;  // >= 448
  if (a < 0x3C800000u) {                      // below 2^-6: the subnormal grid, quantum 2^-9
    // Adding 2^14 (ulp 2^-9 in fp32) rounds to nearest even on that grid; the count is the
    // low mantissa bits. 8 means "rounded up to the smallest normal", whose code is 8 too.
    const float r = bits_f32(a) + 16384.0f;
    return sign | static_cast<uint8_t>(f32_bits(r) & 0xFu);
  }
  // Normal range: keep 3 mantissa bits, round to nearest even on bit 20; a carry moves into
  // the exponent, which is the correct next binade.
  a += 0x7FFFFu + ((a >> 20) & 1u);
  const uint32_t code = ((a >> 20) & 0x7FFu) - (120u << 3);  // exponent rebias 127 -> 7
  return sign | static_cast<uint8_t>(code > 0x7Eu ? 0x7Eu : code);
}

// E2M1: magnitudes {0, .5, 1, 1.5, 2, 3, 4, 6}, bit 3 the sign.
DGPP_HD inline float e2m1_to_f32(uint8_t v) {
  const uint32_t c = v & 7u;
  // 2 * magnitude packed one nibble per code: 0,1,2,3,4,6,8,12.
  const uint32_t twice = (0xC8643210u >> (4u * c)) & 0xFu;
  const float mag = static_cast<float>(twice) * 0.5f;
  return (v & 8u) ? -mag : mag;
}

// Round to nearest on the E2M1 grid, ties to the even code, saturating; NaN saturates.
DGPP_HD inline uint8_t f32_to_e2m1(float f) {
  const uint32_t u = f32_bits(f);
  const uint8_t sign = static_cast<uint8_t>((u >> 28) & 8u);
  const uint32_t abits = u & 0x7FFFFFFFu;
  if (abits > 0x7F800000u) return sign | 7u;
  const float a = bits_f32(abits);
  // Midpoints between neighbours; a tie goes to the even code, so the comparison alternates
  // between <= (lower code even) and < (lower code odd).
  uint8_t c = 0;
  c += a > 0.25f;
  c += a >= 0.75f;
  c += a > 1.25f;
  c += a >= 1.75f;
  c += a > 2.5f;
  c += a >= 3.5f;
  c += a > 5.0f;
  return sign | c;
}

// E8M0: 2^(b - 127); 255 is NaN; 0 is 2^-127 (an fp32 subnormal).
DGPP_HD inline float e8m0_to_f32(uint8_t b) {
  if (b == 255u) return bits_f32(0x7FC00000u);
  if (b == 0u) return bits_f32(0x00400000u);
  return bits_f32(static_cast<uint32_t>(b) << 23);
}

// ceil(log2(x)) + 127 from the IEEE fields, clamped to 254.
DGPP_HD inline uint8_t e8m0_ceil_log2(float x) {
  const uint32_t u = f32_bits(x);
  const uint32_t b = ((u >> 23) & 0xFFu) + ((u & 0x7FFFFFu) != 0u ? 1u : 0u);
  return static_cast<uint8_t>(b > 254u ? 254u : b);
}

}  // namespace dgpp_amd
