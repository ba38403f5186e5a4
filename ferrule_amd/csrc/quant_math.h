// Closed forms of the reference's activation quantizers, usable from device code
// and from a host build (tests compile this header with g++ and compare it with
// the CPU checker over large input sets).
//
// What is being restated (crates/ferrule-model/src/checkpoint/encoding.rs):
//   :335-337  rounded_power_of_two_scale = 2^ceil(log2(amax / quant_max)) in f32
//   :339-387  quantize_fp8_e4m3fn_to_f32: a candidate search whose outcome is
//             "nearest E4M3 value; a mantissa tie rounds away from zero, except
//             that the tie between 2^e and 1.125*2^e keeps 2^e for e >= -5 (the
//             2^e candidate is met first and the comparison is strict), and the
//             tie 7.5*2^-9 keeps 7*2^-9"
//   :389-406  quantize_fp4_e2m1_to_f32: nearest of {0,.5,1,1.5,2,3,4,6}, ties to
//             the lower magnitude (ascending scan, strict comparison)
// The portable GPU kernel of the reference uses rintf instead of round
// (portable/entrypoints.cu:142-179); that variant is kRoundHalfEven here.
#pragma once

#include <math.h>
#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define FERRULE_HD __host__ __device__ __forceinline__
#else
#define FERRULE_HD static inline
#endif

namespace ferrule_quant {

constexpr uint32_t kRoundCpuReference = 0;
constexpr uint32_t kRoundHalfEven = 1;

FERRULE_HD uint32_t f2u(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
FERRULE_HD float u2f(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}

// ceil(log2f(q)) as an integer, q > 0 finite.  The f32 rounding of log2 matters
// only when q lies a few ulps above a power of two (then log2f may return the
// integer itself and the ceiling does not move up); that sliver is evaluated in
// double and rounded to f32 like the library routine.
FERRULE_HD int ceil_log2f(float q) {
  const uint32_t bits = f2u(q);
  int e = static_cast<int>((bits >> 23) & 0xffu) - 127;
  uint32_t frac = bits & 0x7fffffu;
  if (((bits >> 23) & 0xffu) == 0u) {
    // subnormal q: normalise
    int shift = 0;
    while ((frac & 0x800000u) == 0u) {
      frac <<= 1;
      ++shift;
    }
    frac &= 0x7fffffu;
    e = -126 - shift;
  }
  if (frac == 0u) return e;
  if (frac >= 256u) return e + 1;
  const double l = static_cast<double>(e) + log2(1.0 + static_cast<double>(frac) * 0x1p-23);
  const float lf = static_cast<float>(l);
  return static_cast<int>(ceilf(lf));
}

// E8M0 byte of rounded_power_of_two_scale(amax, quant_max); amax > 0 finite.
// The f32 value 2^n underflows to 0 below 2^-149 and overflows to +inf above
// 2^127 in the reference; both are outside what amax floors allow (>= 2^-126).
FERRULE_HD uint32_t scale_byte(float amax, float quant_max) {
  const int n = ceil_log2f(amax / quant_max);
  const int b = n + 127;
  return static_cast<uint32_t>(b < 0 ? 0 : b > 255 ? 255 : b);
}

FERRULE_HD float e8m0_value(uint32_t byte) { return u2f(byte == 0u ? (1u << 22) : (byte << 23)); }

// |v| already clamped to (0, 448] -> E4M3 code without sign.
FERRULE_HD uint32_t fp8_e4m3_encode_magnitude(float m, uint32_t mode) {
  const uint32_t bits = f2u(m);
  if (m >= 0.015625f) {  // normal range, 2^-6 ..= 448
    const uint32_t q = (bits >> 20) & 7u;
    const uint32_t rem = bits & 0xfffffu;
    const uint32_t biased = (bits >> 23) & 0xffu;
    bool up = rem > 0x80000u;
    if (rem == 0x80000u) {
      if (mode == kRoundHalfEven) {
        up = (q & 1u) != 0u;
      } else {
        up = !(q == 0u && biased >= 122u);
      }
    }
    const uint32_t rounded = (bits >> 20) + (up ? 1u : 0u);  // exponent|mantissa3, carry included
    // f32 biased exponent 121 (2^-6) is E4M3 exponent 1
    const uint32_t code = rounded - (120u << 3);
    return code > 0x7eu ? 0x7eu : code;
  }
  const float u = m * 512.0f;
  if (u > 7.5f) return 8u;  // 2^-6
  if (u == 7.5f) return 7u;
  if (mode == kRoundHalfEven) return static_cast<uint32_t>(rintf(u));
  return static_cast<uint32_t>(roundf(u));
}

// One element of simulate_fp8_..._activation_quant: x / scale, clamp, encode.
FERRULE_HD uint32_t fp8_e4m3_quantize_byte(float x, float scale, uint32_t mode) {
  float q = x / scale;
  q = q < -448.0f ? -448.0f : q > 448.0f ? 448.0f : q;  // NaN passes through
  const uint32_t sign = (f2u(q) >> 24) & 0x80u;
  if (q != q) return sign | 0x7fu;
  if (q == 0.0f) return sign;
  return sign | fp8_e4m3_encode_magnitude(fabsf(q), mode);
}

// The same byte as fp8_e4m3_quantize_byte(x, scale, mode) for a power-of-two scale given by its
// inverse (x * inv_scale equals x / scale exactly), without a branch: the register epilogues of
// the GEMMs quantise 64 values per lane and the branching form cost them more time than their
// K loops' tails.  Checked against the branching form over every f32 exponent/mantissa pattern
// that can matter (tests/test_quant_math_cpu.py).
FERRULE_HD uint32_t fp8_e4m3_quantize_byte_pow2(float x, float inv_scale, uint32_t mode) {
  float q = x * inv_scale;
  const bool nan = q != q;
  q = q < -448.0f ? -448.0f : q > 448.0f ? 448.0f : q;
  const uint32_t qbits = f2u(q);
  const uint32_t sign = (qbits >> 24) & 0x80u;
  const uint32_t bits = qbits & 0x7fffffffu;  // |q|
  // normal range: round the 20 dropped mantissa bits; a tie goes up when t = 1
  const uint32_t q3 = (bits >> 20) & 7u;
  const uint32_t t = mode == kRoundHalfEven ? (q3 & 1u) : ((q3 == 0u && (bits >> 23) >= 122u) ? 0u : 1u);
  const uint32_t rounded = (bits + 0x7ffffu + t) >> 20;  // exponent|mantissa3, carry included
  const uint32_t wide = rounded - (120u << 3);
  const uint32_t normal = wide > 0x7eu ? 0x7eu : wide;
  // subnormal range: the grid of 2^-9, half away from zero (u - floor(u) is exact), 7.5 -> 7
  const float u = u2f(bits) * 512.0f;
  const float fl = floorf(u);
  const float away = fl + ((u - fl) >= 0.5f ? 1.0f : 0.0f);
  const float r = mode == kRoundHalfEven ? rintf(u) : away;
  const uint32_t sub = u == 7.5f ? 7u : static_cast<uint32_t>(r);
  const uint32_t code = bits >= 0x3c800000u ? normal : sub;  // |q| >= 2^-6
  return nan ? (sign | 0x7fu) : (sign | code);
}

// 2^-(byte-127): the exact inverse of e8m0_value(byte) for bytes 1..253.
FERRULE_HD float e8m0_inverse(uint32_t byte) { return u2f((254u - byte) << 23); }

FERRULE_HD uint32_t fp4_e2m1_quantize_nibble(float x, float scale, bool signed_zero) {
  float q = x / scale;
  q = q < -6.0f ? -6.0f : q > 6.0f ? 6.0f : q;
  const uint32_t sign = (f2u(q) >> 28) & 8u;
  if (q != q) return signed_zero ? sign : 0u;  // non-finite passes through as a zero code
  if (q == 0.0f) return signed_zero ? sign : 0u;
  const float m = fabsf(q);
  const uint32_t idx = (m > 0.25f) + (m > 0.75f) + (m > 1.25f) + (m > 1.75f) + (m > 2.5f) +
                       (m > 3.5f) + (m > 5.0f);
  return sign | idx;
}

}  // namespace ferrule_quant
