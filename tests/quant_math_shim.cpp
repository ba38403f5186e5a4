// Host build of ferrule_amd/csrc/quant_math.h for CPU tests (compiled by
// tests/test_quant_math_cpu.py with g++; not part of the provider library).
#include <stddef.h>
#include <stdint.h>

#include "../ferrule_amd/csrc/quant_math.h"

extern "C" {
void shim_fp8_bytes(const float *x, size_t n, float scale, uint32_t mode, uint8_t *out) {
  for (size_t i = 0; i < n; ++i) out[i] = (uint8_t)ferrule_quant::fp8_e4m3_quantize_byte(x[i], scale, mode);
}
void shim_fp8_bytes_pow2(const float *x, size_t n, uint32_t scale_byte, uint32_t mode, uint8_t *out) {
  const float inv = ferrule_quant::e8m0_inverse(scale_byte);
  for (size_t i = 0; i < n; ++i) out[i] = (uint8_t)ferrule_quant::fp8_e4m3_quantize_byte_pow2(x[i], inv, mode);
}
void shim_fp4_nibbles(const float *x, size_t n, float scale, int signed_zero, uint8_t *out) {
  for (size_t i = 0; i < n; ++i) out[i] = (uint8_t)ferrule_quant::fp4_e2m1_quantize_nibble(x[i], scale, signed_zero != 0);
}
void shim_scale_bytes(const float *amax, size_t n, float quant_max, uint8_t *out) {
  for (size_t i = 0; i < n; ++i) out[i] = (uint8_t)ferrule_quant::scale_byte(amax[i], quant_max);
}
}
