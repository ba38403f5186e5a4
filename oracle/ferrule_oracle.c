/*
 * CPU restatement of Ferrule's reference arithmetic (see ferrule_oracle.h).
 * TEST INFRASTRUCTURE ONLY - never linked into the provider.
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math -fopenmp -shared -fPIC
 * (-ffp-contract=off matters: the reference rounds every multiply and add.)
 */
#include "ferrule_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ---- small Rust-semantics helpers ------------------------------------- */

/* f32::powi(2.0, n): repeated squaring, reciprocal for n<0; equals ldexpf for
 * every n the path uses (-127..128), including 2^-127 (subnormal) and 2^128
 * (+inf). */
static float pow2i(int n) { return ldexpf(1.0f, n); }

/* f32::clamp: NaN stays NaN. */
static float clampf(float v, float lo, float hi) {
  if (v < lo) return lo;
  if (v > hi) return hi;
  return v;
}

/* ---- encoding.rs ------------------------------------------------------- */

float fo_decode_fp4_e2m1_nibble(uint8_t nibble) {
  /* encoding.rs:14-30 */
  float magnitude;
  switch (nibble & 0x07) {
  case 0: magnitude = 0.0f; break;
  case 1: magnitude = 0.5f; break;
  case 2: magnitude = 1.0f; break;
  case 3: magnitude = 1.5f; break;
  case 4: magnitude = 2.0f; break;
  case 5: magnitude = 3.0f; break;
  case 6: magnitude = 4.0f; break;
  default: magnitude = 6.0f; break;
  }
  return (nibble & 0x08) ? -magnitude : magnitude;
}

void fo_decode_fp4_e2m1_packed_low_first(const uint8_t *bytes, size_t count,
                                         float *out) {
  /* encoding.rs:37-44 */
  for (size_t i = 0; i < count; ++i) {
    out[2 * i] = fo_decode_fp4_e2m1_nibble(bytes[i] & 0x0f);
    out[2 * i + 1] = fo_decode_fp4_e2m1_nibble(bytes[i] >> 4);
  }
}

float fo_decode_e8m0_scale(uint8_t byte) {
  /* encoding.rs:51-53 */
  return pow2i((int)byte - 127);
}

float fo_decode_fp8_e4m3fn_byte(uint8_t byte) {
  /* encoding.rs:61-75 */
  const float sign = (byte & 0x80) ? -1.0f : 1.0f;
  const int exponent = (byte >> 3) & 0x0f;
  const int mantissa = byte & 0x07;
  if (exponent == 0) {
    if (mantissa == 0) return sign * 0.0f;
    return sign * (float)mantissa * pow2i(-9);
  }
  if (exponent == 0x0f && mantissa == 0x07) return NAN;
  return sign * pow2i(exponent - 7) * (1.0f + (float)mantissa / 8.0f);
}

int fo_dequantize_fp4_e2m1_with_e8m0_scales(const uint8_t *weight,
                                            const uint8_t *scales,
                                            size_t out_features,
                                            size_t in_features,
                                            size_t block_size, float *out) {
  /* encoding.rs:82-140 */
  if (block_size == 0 || in_features % block_size != 0 || in_features % 2 != 0)
    return 1;
  const size_t packed_cols = in_features / 2;
  const size_t scale_cols = in_features / block_size;
  for (size_t row = 0; row < out_features; ++row) {
    for (size_t k = 0; k < in_features; ++k) {
      const uint8_t packed = weight[row * packed_cols + k / 2];
      const uint8_t nibble = (k % 2 == 0) ? (packed & 0x0f) : (packed >> 4);
      const float scale =
          fo_decode_e8m0_scale(scales[row * scale_cols + k / block_size]);
      out[row * in_features + k] = fo_decode_fp4_e2m1_nibble(nibble) * scale;
    }
  }
  return 0;
}

int fo_dequantize_fp8_e4m3fn_with_e8m0_scales(const uint8_t *weight,
                                              const uint8_t *scales,
                                              size_t out_features,
                                              size_t in_features,
                                              size_t block_m, size_t block_k,
                                              float *out) {
  /* encoding.rs:147-198 */
  if (block_m == 0 || block_k == 0) return 1;
  const size_t scale_cols = (in_features + block_k - 1) / block_k;
  for (size_t row = 0; row < out_features; ++row) {
    for (size_t col = 0; col < in_features; ++col) {
      const float scale = fo_decode_e8m0_scale(
          scales[(row / block_m) * scale_cols + col / block_k]);
      out[row * in_features + col] =
          fo_decode_fp8_e4m3fn_byte(weight[row * in_features + col]) * scale;
    }
  }
  return 0;
}

int fo_dequantize_fp8_e4m3fn_with_f32_scales(const uint8_t *weight,
                                             const float *scales,
                                             size_t out_features,
                                             size_t in_features, size_t block_m,
                                             size_t block_k, float *out) {
  /* loop of encoding.rs:186-196 with an f32 scale table */
  if (block_m == 0 || block_k == 0) return 1;
  const size_t scale_cols = (in_features + block_k - 1) / block_k;
  for (size_t row = 0; row < out_features; ++row) {
    for (size_t col = 0; col < in_features; ++col) {
      const float scale = scales[(row / block_m) * scale_cols + col / block_k];
      out[row * in_features + col] =
          fo_decode_fp8_e4m3fn_byte(weight[row * in_features + col]) * scale;
    }
  }
  return 0;
}

float fo_rounded_power_of_two_scale(float amax, float quant_max) {
  /* encoding.rs:335-337: 2.0f32.powf((amax / quant_max).log2().ceil()) */
  return powf(2.0f, ceilf(log2f(amax / quant_max)));
}

static float nearest_fp8_subnormal_positive(float magnitude) {
  /* encoding.rs:383-387 (f32::round = half away from zero = roundf) */
  const float step = pow2i(-9);
  float mantissa = roundf(magnitude / step);
  mantissa = clampf(mantissa, 0.0f, 7.0f);
  return mantissa * step;
}

static float nearest_fp8_e4m3fn_positive(float magnitude) {
  /* encoding.rs:348-381 */
  float best = nearest_fp8_subnormal_positive(magnitude);
  float best_err = fabsf(best - magnitude);
  const int exp_floor = (int)floorf(log2f(magnitude));
  for (int exp = exp_floor - 1; exp <= exp_floor + 1; ++exp) {
    if (exp < -6 || exp > 8) continue;
    const float scale = pow2i(exp);
    int mantissa = (int)roundf((magnitude / scale - 1.0f) * 8.0f);
    int candidate_exp = exp;
    if (mantissa < 0) continue;
    if (mantissa > 7) {
      candidate_exp += 1;
      mantissa = 0;
    }
    if (candidate_exp > 8) {
      candidate_exp = 8;
      mantissa = 6;
    }
    if (candidate_exp == 8 && mantissa > 6) mantissa = 6;
    const float candidate =
        pow2i(candidate_exp) * (1.0f + (float)mantissa / 8.0f);
    const float err = fabsf(candidate - magnitude);
    if (err < best_err) {
      best = candidate;
      best_err = err;
    }
  }
  return best;
}

float fo_quantize_fp8_e4m3fn_to_f32(float value) {
  /* encoding.rs:339-346 */
  if (!isfinite(value) || value == 0.0f) return value;
  const float sign = signbit(value) ? -1.0f : 1.0f;
  const float magnitude = fminf(fabsf(value), 448.0f);
  return sign * nearest_fp8_e4m3fn_positive(magnitude);
}

float fo_quantize_fp4_e2m1_to_f32(float value) {
  /* encoding.rs:389-406 */
  static const float MAGNITUDES[8] = {0.0f, 0.5f, 1.0f, 1.5f,
                                      2.0f, 3.0f, 4.0f, 6.0f};
  if (!isfinite(value) || value == 0.0f) return value;
  const float sign = signbit(value) ? -1.0f : 1.0f;
  const float magnitude = fminf(fabsf(value), 6.0f);
  float best = MAGNITUDES[0];
  float best_err = fabsf(magnitude - best);
  for (int i = 1; i < 8; ++i) {
    const float err = fabsf(magnitude - MAGNITUDES[i]);
    if (err < best_err) {
      best = MAGNITUDES[i];
      best_err = err;
    }
  }
  return sign * best;
}

static int act_quant_shape_ok(size_t len, size_t row_width, size_t block_size) {
  if (row_width == 0 || block_size == 0 || row_width % block_size != 0) return 0;
  if (len % row_width != 0) return 0;
  return 1;
}

static float block_amax(const float *block, size_t n) {
  /* .fold(0.0, |acc, v| acc.max(v.abs())) - f32::max ignores NaN like fmaxf */
  float amax = 0.0f;
  for (size_t i = 0; i < n; ++i) amax = fmaxf(amax, fabsf(block[i]));
  return amax;
}

int fo_simulate_fp8_act_quant_in_place(float *values, size_t len,
                                       size_t row_width, size_t block_size) {
  /* encoding.rs:207-242 */
  if (!act_quant_shape_ok(len, row_width, block_size)) return 1;
  for (size_t start = 0; start < len; start += block_size) {
    float *block = values + start;
    const float amax = fmaxf(block_amax(block, block_size), 1e-4f);
    const float scale = fo_rounded_power_of_two_scale(amax, 448.0f);
    for (size_t i = 0; i < block_size; ++i) {
      const float quantized = fo_quantize_fp8_e4m3fn_to_f32(
          clampf(block[i] / scale, -448.0f, 448.0f));
      block[i] = quantized * scale;
    }
  }
  return 0;
}

int fo_simulate_fp4_act_quant_in_place(float *values, size_t len,
                                       size_t row_width, size_t block_size) {
  /* encoding.rs:249-284 */
  if (!act_quant_shape_ok(len, row_width, block_size)) return 1;
  for (size_t start = 0; start < len; start += block_size) {
    float *block = values + start;
    const float amax =
        fmaxf(block_amax(block, block_size), 6.0f * pow2i(-126));
    const float scale = fo_rounded_power_of_two_scale(amax, 6.0f);
    for (size_t i = 0; i < block_size; ++i) {
      const float quantized =
          fo_quantize_fp4_e2m1_to_f32(clampf(block[i] / scale, -6.0f, 6.0f));
      block[i] = quantized * scale;
    }
  }
  return 0;
}

/* value already on the E4M3 grid (or zero / non-finite) -> byte */
static uint8_t fp8_grid_value_to_byte(float q) {
  uint32_t bits;
  memcpy(&bits, &q, 4);
  const uint8_t sign = (bits >> 31) ? 0x80 : 0x00;
  const float m = fabsf(q);
  if (m == 0.0f) return sign;
  if (!isfinite(q)) return sign | 0x7f;
  if (m < pow2i(-6)) return sign | (uint8_t)(m * 512.0f);
  const int exponent = (int)((bits >> 23) & 0xff) - 127 + 7;
  return sign | (uint8_t)(exponent << 3) | (uint8_t)((bits >> 20) & 7);
}

static uint8_t e8m0_byte_of_power_of_two(float scale) {
  /* scale is an exact power of two (or 0/inf after f32 under/overflow) */
  uint32_t bits;
  memcpy(&bits, &scale, 4);
  const uint32_t e = (bits >> 23) & 0xff;
  if (e == 0) return 0; /* 2^-127 and below are carried as byte 0 */
  return (uint8_t)e;    /* 255 for +inf */
}

int fo_pack_fp8_act(const float *values, size_t len, size_t row_width,
                    size_t block_size, uint8_t *packed, uint8_t *scales) {
  if (!act_quant_shape_ok(len, row_width, block_size)) return 1;
  for (size_t start = 0, b = 0; start < len; start += block_size, ++b) {
    const float *block = values + start;
    const float amax = fmaxf(block_amax(block, block_size), 1e-4f);
    const float scale = fo_rounded_power_of_two_scale(amax, 448.0f);
    scales[b] = e8m0_byte_of_power_of_two(scale);
    for (size_t i = 0; i < block_size; ++i) {
      const float q = fo_quantize_fp8_e4m3fn_to_f32(
          clampf(block[i] / scale, -448.0f, 448.0f));
      packed[start + i] = fp8_grid_value_to_byte(q);
    }
  }
  return 0;
}

static uint8_t fp4_grid_value_to_nibble(float q) {
  const uint8_t sign = signbit(q) ? 8 : 0;
  const float m = fabsf(q);
  if (!(m == m) || isinf(m)) return sign; /* non-finite passes through as 0 */
  static const float MAGNITUDES[8] = {0.0f, 0.5f, 1.0f, 1.5f,
                                      2.0f, 3.0f, 4.0f, 6.0f};
  for (uint8_t i = 0; i < 8; ++i)
    if (m == MAGNITUDES[i]) return sign | i;
  return sign;
}

int fo_pack_fp4_act(const float *values, size_t len, size_t row_width,
                    size_t block_size, uint8_t *packed, uint8_t *scales) {
  if (!act_quant_shape_ok(len, row_width, block_size) || block_size % 2 != 0)
    return 1;
  for (size_t start = 0, b = 0; start < len; start += block_size, ++b) {
    const float *block = values + start;
    const float amax =
        fmaxf(block_amax(block, block_size), 6.0f * pow2i(-126));
    const float scale = fo_rounded_power_of_two_scale(amax, 6.0f);
    scales[b] = e8m0_byte_of_power_of_two(scale);
    for (size_t i = 0; i < block_size; i += 2) {
      const uint8_t lo = fp4_grid_value_to_nibble(
          fo_quantize_fp4_e2m1_to_f32(clampf(block[i] / scale, -6.0f, 6.0f)));
      const uint8_t hi = fp4_grid_value_to_nibble(fo_quantize_fp4_e2m1_to_f32(
          clampf(block[i + 1] / scale, -6.0f, 6.0f)));
      packed[(start + i) / 2] = (uint8_t)(lo | (hi << 4));
    }
  }
  return 0;
}

/* ---- math.rs ----------------------------------------------------------- */

float fo_round_to_bf16(float value) {
  /* models/common/math.rs:7-14 */
  uint32_t bits;
  memcpy(&bits, &value, 4);
  uint32_t out;
  if ((bits & 0x7fffffffu) > 0x7f800000u) {
    out = (((bits >> 16) | 0x0040u) & 0xffffu) << 16;
  } else {
    const uint32_t rounding_bias = 0x7fffu + ((bits >> 16) & 1u);
    out = (bits + rounding_bias) & 0xffff0000u;
  }
  float r;
  memcpy(&r, &out, 4);
  return r;
}

uint16_t fo_bf16_bits(float value) {
  const float r = fo_round_to_bf16(value);
  uint32_t bits;
  memcpy(&bits, &r, 4);
  return (uint16_t)(bits >> 16);
}

/* ---- weight.rs --------------------------------------------------------- */

void fo_matvec_row_major(const float *weights, size_t rows, size_t cols,
                         const float *input, float *output) {
  /* weight.rs:440-451 */
  for (size_t row = 0; row < rows; ++row) {
    float acc = 0.0f;
    const size_t offset = row * cols;
    for (size_t col = 0; col < cols; ++col) {
      acc += weights[offset + col] * input[col];
    }
    output[row] = acc;
  }
}

int fo_linear_fp4_matvec(const uint8_t *weight, const uint8_t *scales,
                         size_t out_features, size_t in_features,
                         size_t block_size, const float *input, float *output,
                         int threads) {
  if (block_size == 0 || in_features % block_size != 0 ||
      in_features % 2 != 0 || block_size % 2 != 0)
    return 1;
  const size_t packed_cols = in_features / 2;
  const size_t scale_cols = in_features / block_size;
  float decode[16];
  for (int i = 0; i < 16; ++i) decode[i] = fo_decode_fp4_e2m1_nibble((uint8_t)i);
#pragma omp parallel for schedule(static) num_threads(threads > 1 ? threads : 1)
  for (long row = 0; row < (long)out_features; ++row) {
    const uint8_t *wrow = weight + (size_t)row * packed_cols;
    const uint8_t *srow = scales + (size_t)row * scale_cols;
    float acc = 0.0f;
    for (size_t b = 0; b < scale_cols; ++b) {
      const float scale = fo_decode_e8m0_scale(srow[b]);
      float table[16]; /* decode(nibble) * scale, the dequantized weight */
      for (int i = 0; i < 16; ++i) table[i] = decode[i] * scale;
      const size_t k0 = b * block_size;
      for (size_t k = k0; k < k0 + block_size; k += 2) {
        const uint8_t byte = wrow[k / 2];
        acc += table[byte & 0x0f] * input[k];
        acc += table[byte >> 4] * input[k + 1];
      }
    }
    output[row] = acc;
  }
  return 0;
}

int fo_linear_fp8_matvec(const uint8_t *weight, const void *scales,
                         int scale_kind, size_t out_features,
                         size_t in_features, size_t block_m, size_t block_k,
                         const float *input, float *output, int threads) {
  if (block_m == 0 || block_k == 0) return 1;
  const size_t scale_cols = (in_features + block_k - 1) / block_k;
  float decode[256];
  for (int i = 0; i < 256; ++i) decode[i] = fo_decode_fp8_e4m3fn_byte((uint8_t)i);
#pragma omp parallel for schedule(static) num_threads(threads > 1 ? threads : 1)
  for (long row = 0; row < (long)out_features; ++row) {
    const uint8_t *wrow = weight + (size_t)row * in_features;
    const size_t srow = ((size_t)row / block_m) * scale_cols;
    float acc = 0.0f;
    for (size_t b = 0; b < scale_cols; ++b) {
      const float scale =
          scale_kind == FO_SCALE_F32
              ? ((const float *)scales)[srow + b]
              : fo_decode_e8m0_scale(((const uint8_t *)scales)[srow + b]);
      const size_t k0 = b * block_k;
      const size_t k1 = k0 + block_k < in_features ? k0 + block_k : in_features;
      for (size_t k = k0; k < k1; ++k) {
        const float w = decode[wrow[k]] * scale;
        acc += w * input[k];
      }
    }
    output[row] = acc;
  }
  return 0;
}

int fo_linear_fp4_matvec_materialized(const uint8_t *weight,
                                      const uint8_t *scales,
                                      size_t out_features, size_t in_features,
                                      size_t block_size, const float *input,
                                      float *output) {
  float *w = (float *)malloc(out_features * in_features * sizeof(float));
  if (!w) return 2;
  int rc = fo_dequantize_fp4_e2m1_with_e8m0_scales(
      weight, scales, out_features, in_features, block_size, w);
  if (rc == 0) fo_matvec_row_major(w, out_features, in_features, input, output);
  free(w);
  return rc;
}

int fo_linear_fp8_matvec_materialized(const uint8_t *weight, const void *scales,
                                      int scale_kind, size_t out_features,
                                      size_t in_features, size_t block_m,
                                      size_t block_k, const float *input,
                                      float *output) {
  float *w = (float *)malloc(out_features * in_features * sizeof(float));
  if (!w) return 2;
  int rc = scale_kind == FO_SCALE_F32
               ? fo_dequantize_fp8_e4m3fn_with_f32_scales(
                     weight, (const float *)scales, out_features, in_features,
                     block_m, block_k, w)
               : fo_dequantize_fp8_e4m3fn_with_e8m0_scales(
                     weight, (const uint8_t *)scales, out_features, in_features,
                     block_m, block_k, w);
  if (rc == 0) fo_matvec_row_major(w, out_features, in_features, input, output);
  free(w);
  return rc;
}

/* ---- executor.rs / routed.rs / ffn.rs ---------------------------------- */

float fo_silu(float x) {
  /* executor.rs:179-181 */
  return x / (1.0f + expf(-x));
}

int fo_expert_execute_fp4(const uint8_t *gate_w, const uint8_t *gate_s,
                          const uint8_t *up_w, const uint8_t *up_s,
                          const uint8_t *down_w, const uint8_t *down_s,
                          size_t hidden, size_t intermediate,
                          size_t block_size, const float *input,
                          float route_weight, float swiglu_limit,
                          size_t act_quant_block, float *output,
                          float *hidden_out, int threads) {
  /* executor.rs:82-124 */
  int rc = 0;
  float *x = (float *)malloc(hidden * sizeof(float));
  float *gate = (float *)malloc(intermediate * sizeof(float));
  float *up = (float *)malloc(intermediate * sizeof(float));
  float *h = (float *)malloc(intermediate * sizeof(float));
  if (!x || !gate || !up || !h) {
    rc = 2;
    goto done;
  }
  memcpy(x, input, hidden * sizeof(float));
  if (act_quant_block) { /* quantized_input: row_width = input.len() */
    rc = fo_simulate_fp8_act_quant_in_place(x, hidden, hidden, act_quant_block);
    if (rc) goto done;
  }
  rc = fo_linear_fp4_matvec(gate_w, gate_s, intermediate, hidden, block_size, x,
                            gate, threads);
  if (rc) goto done;
  rc = fo_linear_fp4_matvec(up_w, up_s, intermediate, hidden, block_size, x, up,
                            threads);
  if (rc) goto done;
  if (swiglu_limit > 0.0f) {
    for (size_t i = 0; i < intermediate; ++i) {
      gate[i] = fminf(gate[i], swiglu_limit);
      up[i] = clampf(up[i], -swiglu_limit, swiglu_limit);
    }
  }
  for (size_t i = 0; i < intermediate; ++i) {
    h[i] = fo_silu(gate[i]) * up[i] * route_weight;
  }
  if (act_quant_block) {
    rc = fo_simulate_fp8_act_quant_in_place(h, intermediate, intermediate,
                                            act_quant_block);
    if (rc) goto done;
  }
  if (hidden_out) memcpy(hidden_out, h, intermediate * sizeof(float));
  rc = fo_linear_fp4_matvec(down_w, down_s, hidden, intermediate, block_size, h,
                            output, threads);
done:
  free(x);
  free(gate);
  free(up);
  free(h);
  return rc;
}

void fo_accumulate_routes(const float *route_outputs, size_t routes,
                          size_t width, const float *shared, float *out) {
  /* routed.rs:85-110, 183-201 */
  if (routes == 0) {
    for (size_t i = 0; i < width; ++i) out[i] = 0.0f;
  } else {
    memcpy(out, route_outputs, width * sizeof(float));
    for (size_t r = 1; r < routes; ++r) {
      const float *v = route_outputs + r * width;
      for (size_t i = 0; i < width; ++i) out[i] += v[i];
    }
  }
  if (shared) {
    for (size_t i = 0; i < width; ++i) out[i] += shared[i];
  }
}

void fo_swiglu_ffn_f32(const float *gate, const float *up, const float *down,
                       size_t hidden, size_t intermediate, const float *input,
                       float output_scale, float swiglu_limit, float *output) {
  /* ffn.rs:24-48 */
  float *g = (float *)malloc(intermediate * sizeof(float));
  float *u = (float *)malloc(intermediate * sizeof(float));
  float *h = (float *)malloc(intermediate * sizeof(float));
  fo_matvec_row_major(gate, intermediate, hidden, input, g);
  fo_matvec_row_major(up, intermediate, hidden, input, u);
  if (swiglu_limit > 0.0f) {
    for (size_t i = 0; i < intermediate; ++i) {
      g[i] = fminf(g[i], swiglu_limit);
      u[i] = clampf(u[i], -swiglu_limit, swiglu_limit);
    }
  }
  for (size_t i = 0; i < intermediate; ++i)
    h[i] = fo_silu(g[i]) * u[i] * output_scale;
  fo_matvec_row_major(down, hidden, intermediate, h, output);
  free(g);
  free(u);
  free(h);
}

void fo_reduce_routes_ranked(const float *route_output, size_t tokens,
                             size_t routes_per_token, size_t hidden,
                             float *output) {
  /* portable/entrypoints.cu:1604-1610 */
  for (size_t t = 0; t < tokens; ++t) {
    for (size_t h = 0; h < hidden; ++h) {
      float result = output[t * hidden + h];
      for (size_t rank = 0; rank < routes_per_token; ++rank) {
        result += route_output[(t * routes_per_token + rank) * hidden + h];
      }
      output[t * hidden + h] = fo_round_to_bf16(result);
    }
  }
}

/* ---- router ------------------------------------------------------------- */

float fo_stable_softplus(float value) {
  /* routing.rs:367-372: total_cmp(&20.0) == Greater => value, else exp().ln_1p().
   * total_cmp puts a positive NaN above 20 as well. */
  if (value > 20.0f) return value;
  if (value != value) {
    uint32_t bits;
    memcpy(&bits, &value, 4);
    if ((bits >> 31) == 0) return value;
  }
  return log1pf(expf(value));
}

/* f32::total_cmp as an ordered integer key (larger key = greater value) */
static int64_t total_order_key(float v) {
  int32_t bits;
  memcpy(&bits, &v, 4);
  bits ^= (int32_t)(((uint32_t)(bits >> 31)) >> 1);
  return bits;
}

int fo_router_route_sqrt_softplus(const float *logits, size_t experts,
                                  const float *bias,
                                  const int64_t *hash_experts, size_t hash_len,
                                  size_t top_k, float route_scale,
                                  int32_t *indices, float *weights,
                                  float *scores_out, float *selection_out) {
  /* routing.rs:209-289 */
  if (experts == 0) return 1;
  if (top_k == 0 || top_k > experts) return 1;
  if (!isfinite(route_scale)) return 1;
  for (size_t e = 0; e < experts; ++e) {
    if (!isfinite(logits[e])) return 1;
  }
  if (bias) {
    for (size_t e = 0; e < experts; ++e) {
      if (!isfinite(bias[e])) return 1;
    }
  }
  if (hash_experts) {
    if (hash_len < top_k) return 1;
    for (size_t rank = 0; rank < top_k; ++rank) {
      if (hash_experts[rank] < 0 || (size_t)hash_experts[rank] >= experts) return 1;
      for (size_t before = 0; before < rank; ++before) {
        if (hash_experts[before] == hash_experts[rank]) return 1;
      }
    }
  }
  /* routing.rs:297-303 */
  float *scores = (float *)malloc(experts * sizeof(float));
  size_t *chosen = (size_t *)malloc(top_k * sizeof(size_t));
  for (size_t e = 0; e < experts; ++e) scores[e] = sqrtf(fo_stable_softplus(logits[e]));
  if (hash_experts) {
    for (size_t rank = 0; rank < top_k; ++rank) chosen[rank] = (size_t)hash_experts[rank];
  } else {
    /* routing.rs:305-331: a full sort by (selection desc, expert asc), truncated.
     * The order is strict (experts are distinct), so picking the best remaining
     * expert top_k times gives the same prefix. */
    unsigned char *taken = (unsigned char *)calloc(experts, 1);
    for (size_t rank = 0; rank < top_k; ++rank) {
      size_t best = experts;
      int64_t best_key = 0;
      for (size_t e = 0; e < experts; ++e) {
        if (taken[e]) continue;
        const float selection = scores[e] + (bias ? bias[e] : 0.0f);
        const int64_t key = total_order_key(selection);
        if (best == experts || key > best_key) {
          best = e;
          best_key = key;
        }
      }
      taken[best] = 1;
      chosen[rank] = best;
    }
    free(taken);
  }
  /* routing.rs:160-178 */
  float sum = 0.0f;
  for (size_t rank = 0; rank < top_k; ++rank) {
    weights[rank] = scores[chosen[rank]];
    sum += weights[rank];
  }
  int rc = 0;
  if (sum <= 0.0f || !isfinite(sum)) {
    rc = 1;
  } else {
    for (size_t rank = 0; rank < top_k; ++rank) weights[rank] /= sum;
    for (size_t rank = 0; rank < top_k; ++rank) weights[rank] *= route_scale;
    for (size_t rank = 0; rank < top_k; ++rank) {
      indices[rank] = (int32_t)chosen[rank];
      if (scores_out) scores_out[rank] = scores[chosen[rank]];
      if (selection_out) {
        selection_out[rank] = scores[chosen[rank]] + (bias ? bias[chosen[rank]] : 0.0f);
      }
    }
  }
  free(chosen);
  free(scores);
  return rc;
}

static float device_softplus(float value) {
  /* portable/entrypoints.cu:103-111 */
  if (value > 20.0f) return value;
  if (value < -20.0f) return expf(value);
  return log1pf(expf(value));
}

static void device_insert_topk(float value, int32_t candidate, float *best_values,
                               int32_t *best_indices, uint32_t k) {
  /* portable/entrypoints.cu:770-791 */
  uint32_t position = k;
  while (position > 0) {
    const uint32_t previous = position - 1;
    if (value < best_values[previous] ||
        (value == best_values[previous] && best_indices[previous] >= 0 &&
         candidate >= best_indices[previous])) {
      break;
    }
    --position;
  }
  if (position < k) {
    for (uint32_t move = k - 1; move > position; --move) {
      best_values[move] = best_values[move - 1];
      best_indices[move] = best_indices[move - 1];
    }
    best_values[position] = value;
    best_indices[position] = candidate;
  }
}

void fo_router_kernel_rows(uint32_t kind, uint32_t rows, uint32_t columns,
                           uint32_t k, uint32_t hash_rows,
                           uint32_t hash_columns, uint32_t flags,
                           float route_scale, const float *logits,
                           const float *bias, const int32_t *token_ids,
                           const int32_t *hash_table, void *indices_out,
                           float *weights) {
  /* portable/entrypoints.cu:793-884, one "thread" per row */
  if (k == 0 || k > 64) return;
  int32_t *indices = (int32_t *)indices_out;
  for (uint32_t row = 0; row < rows; ++row) {
    float best_values[64];
    int32_t best_indices[64];
    for (uint32_t i = 0; i < k; ++i) {
      best_values[i] = -INFINITY;
      best_indices[i] = -1;
    }
    const float *line = logits + (size_t)row * columns;
    if (kind == 1) {
      for (uint32_t e = 0; e < columns; ++e) {
        const float score = sqrtf(fmaxf(device_softplus(line[e]), 0.0f));
        const float selection = score + ((flags & 1u) ? bias[e] : 0.0f);
        device_insert_topk(selection, (int32_t)e, best_values, best_indices, k);
      }
      float sum = 0.0f;
      for (uint32_t rank = 0; rank < k; ++rank) {
        const int32_t e = best_indices[rank];
        const float score = e >= 0 ? sqrtf(fmaxf(device_softplus(line[e]), 0.0f)) : 0.0f;
        best_values[rank] = score;
        sum += score;
      }
      for (uint32_t rank = 0; rank < k; ++rank) {
        indices[(size_t)row * k + rank] = best_indices[rank];
        weights[(size_t)row * k + rank] =
            sum > 0.0f && isfinite(sum) ? best_values[rank] / sum * route_scale : 0.0f;
      }
    } else if (kind == 2) {
      const int32_t token = token_ids[row];
      if (token < 0 || (uint32_t)token >= hash_rows) continue;
      float sum = 0.0f;
      int ok = 1;
      for (uint32_t rank = 0; rank < k; ++rank) {
        const int32_t e = hash_table[(size_t)token * hash_columns + rank];
        if (e < 0 || (uint32_t)e >= columns) {
          ok = 0;
          break;
        }
        const float score = sqrtf(fmaxf(device_softplus(line[e]), 0.0f));
        best_indices[rank] = e;
        best_values[rank] = score;
        sum += score;
      }
      if (!ok) continue;
      for (uint32_t rank = 0; rank < k; ++rank) {
        indices[(size_t)row * k + rank] = best_indices[rank];
        weights[(size_t)row * k + rank] =
            sum > 0.0f && isfinite(sum) ? best_values[rank] / sum * route_scale : 0.0f;
      }
    } else {
      for (uint32_t e = 0; e < columns; ++e) {
        device_insert_topk(line[e], (int32_t)e, best_values, best_indices, k);
      }
      for (uint32_t rank = 0; rank < k; ++rank) {
        const size_t out = (size_t)row * k + rank;
        if (kind == 3) {
          ((float *)indices_out)[out] = (float)best_indices[rank];
        } else {
          indices[out] = best_indices[rank];
        }
        weights[out] = best_values[rank];
      }
    }
  }
}

/* ---- expert slot table ---------------------------------------------------- */

void fo_expert_table_publish(uint32_t kind, uint32_t expert, uint32_t slot,
                             int32_t generation, const uint64_t values[6],
                             uint64_t *table, uint32_t slot_capacity,
                             int32_t *expert_to_slot,
                             int32_t *expert_generations,
                             int32_t *slot_generations) {
  /* portable/entrypoints.cu:1270-1300 */
  if (kind == 1) {
    for (int m = 0; m < 6; ++m) table[(size_t)m * slot_capacity + slot] = values[m];
    slot_generations[slot] = generation;
    expert_to_slot[expert] = (int32_t)slot;
    expert_generations[expert] = generation;
  } else {
    expert_to_slot[expert] = -1;
    expert_generations[expert] = 0;
    for (int m = 0; m < 6; ++m) table[(size_t)m * slot_capacity + slot] = 0;
    slot_generations[slot] = generation;
  }
}

void fo_expert_resolve_init(int32_t *miss_control, uint32_t miss_capacity,
                            uint32_t route_capacity) {
  /* portable/entrypoints.cu:1301-1307 */
  const size_t count = (size_t)miss_capacity + route_capacity + 2;
  for (size_t i = 0; i < count; ++i) miss_control[i] = i < 2 ? 0 : -1;
}

void fo_expert_resolve(const int32_t *expert_ids, uint32_t route_count,
                       uint32_t expert_capacity, uint32_t slot_capacity,
                       uint32_t miss_capacity, const int32_t *expert_to_slot,
                       const int32_t *expert_generations,
                       const int32_t *slot_generations, int32_t *route_slots,
                       int32_t *route_generations, int32_t *miss_markers,
                       int32_t *miss_control) {
  /* portable/entrypoints.cu:1311-1340 */
  for (uint32_t route = 0; route < route_count; ++route) {
    const int32_t expert = expert_ids[route];
    int32_t slot = -1, generation = 0;
    if (expert >= 0 && (uint32_t)expert < expert_capacity) {
      const int32_t mapped = expert_to_slot[expert];
      const int32_t expert_generation = expert_generations[expert];
      if (mapped >= 0 && (uint32_t)mapped < slot_capacity &&
          expert_generation > 0 &&
          slot_generations[mapped] == expert_generation) {
        slot = mapped;
        generation = expert_generation;
      }
    }
    route_slots[route] = slot;
    route_generations[route] = generation;
    miss_markers[route] = slot < 0 ? 1 : 0;
    miss_control[2 + (size_t)miss_capacity + route] = expert;
    if (slot < 0) {
      const int32_t miss = miss_control[0]++;
      if (miss >= 0 && (uint32_t)miss < miss_capacity) {
        miss_control[2 + miss] = expert;
      } else {
        miss_control[1] |= 1;
      }
    }
  }
}

int32_t fo_expert_gather_dispatch(uint32_t route_count, uint32_t slot_capacity,
                                  int32_t active_value, const uint64_t *table,
                                  const int32_t *slot_generations,
                                  const int32_t *route_slots,
                                  const int32_t *route_generations,
                                  const float *router_weights,
                                  const int32_t *active_markers,
                                  uint64_t *outputs, float *output_route_weights,
                                  int32_t *expert_ids) {
  /* portable/entrypoints.cu:1341-1379; dispatch_error starts at 0 (:2011-2017) */
  int32_t error = 0;
  for (uint32_t route = 0; route < route_count; ++route) {
    const int32_t slot = route_slots[route];
    const int32_t generation = route_generations[route];
    const int active = active_markers[route] == active_value;
    const int current = slot >= 0 && (uint32_t)slot < slot_capacity &&
                        generation > 0 && slot_generations[slot] == generation;
    int good = active && current;
    for (int m = 0; m < 6; ++m) {
      const uint64_t value = current ? table[(size_t)m * slot_capacity + slot] : 0;
      outputs[(size_t)m * route_count + route] = value;
      good = good && value != 0;
    }
    if (active && !good) error |= 1;
    output_route_weights[route] = good ? router_weights[route] : 0.0f;
    expert_ids[route] = good ? (int32_t)route : -1;
  }
  return error;
}

/* ---- hyper-connection producer ------------------------------------------- */

static float hc_sigmoid(float x) {
  /* hyper_connection.rs:425-427 */
  return 1.0f / (1.0f + expf(-x));
}

int fo_hc_split_sinkhorn(const float *mixes, size_t tokens, size_t hc,
                         size_t sinkhorn_iters, float eps, const float *scale,
                         const float *base, float *pre, float *post, float *comb) {
  /* hyper_connection.rs:175-262 */
  if (hc == 0 || sinkhorn_iters == 0 || !(eps > 0.0f)) return 1;
  const size_t mix_hc = (2 + hc) * hc;
  for (size_t token = 0; token < tokens; ++token) {
    const float *mix = mixes + token * mix_hc;
    for (size_t j = 0; j < hc; ++j) {
      pre[token * hc + j] = hc_sigmoid(mix[j] * scale[0] + base[j]) + eps;
      post[token * hc + j] = 2.0f * hc_sigmoid(mix[hc + j] * scale[1] + base[hc + j]);
    }
    float *cm = comb + token * hc * hc;
    for (size_t row = 0; row < hc; ++row) {
      float row_max = -INFINITY;
      for (size_t col = 0; col < hc; ++col) {
        const float value = mix[2 * hc + row * hc + col] * scale[2] + base[2 * hc + row * hc + col];
        cm[row * hc + col] = value;
        row_max = fmaxf(row_max, value);
      }
      float row_sum = 0.0f;
      for (size_t col = 0; col < hc; ++col) {
        cm[row * hc + col] = expf(cm[row * hc + col] - row_max);
        row_sum += cm[row * hc + col];
      }
      for (size_t col = 0; col < hc; ++col) cm[row * hc + col] = cm[row * hc + col] / row_sum + eps;
    }
    /* normalize_comb_cols / normalize_comb_rows: hyper_connection.rs:398-414 */
    for (size_t iteration = 0; iteration < sinkhorn_iters; ++iteration) {
      if (iteration > 0) {
        for (size_t row = 0; row < hc; ++row) {
          float sum = 0.0f;
          for (size_t col = 0; col < hc; ++col) sum += cm[row * hc + col];
          for (size_t col = 0; col < hc; ++col) cm[row * hc + col] /= sum + eps;
        }
      }
      for (size_t col = 0; col < hc; ++col) {
        float sum = 0.0f;
        for (size_t row = 0; row < hc; ++row) sum += cm[row * hc + col];
        for (size_t row = 0; row < hc; ++row) cm[row * hc + col] /= sum + eps;
      }
    }
  }
  return 0;
}

int fo_hc_pre(const float *state, size_t tokens, size_t hc, size_t hidden,
              size_t sinkhorn_iters, float eps, float norm_eps,
              const float *function, const float *scale, const float *base,
              float *mixes, float *raw_dots, float *pre, float *post, float *comb,
              float *hidden_out) {
  /* hyper_connection.rs:264-311 */
  if (hc == 0 || hidden == 0 || sinkhorn_iters == 0 || !(eps > 0.0f) || !(norm_eps > 0.0f)) return 1;
  const size_t mix_hc = (2 + hc) * hc, hc_dim = hc * hidden;
  for (size_t token = 0; token < tokens; ++token) {
    const float *x = state + token * hc_dim;
    float squares = 0.0f;
    for (size_t i = 0; i < hc_dim; ++i) squares += x[i] * x[i];
    const float rms = 1.0f / sqrtf(squares / (float)hc_dim + norm_eps);
    for (size_t row = 0; row < mix_hc; ++row) {
      const float *w = function + row * hc_dim;
      float dot = 0.0f;
      for (size_t i = 0; i < hc_dim; ++i) dot += w[i] * x[i];
      if (raw_dots) raw_dots[token * mix_hc + row] = dot;
      mixes[token * mix_hc + row] = dot * rms;
    }
  }
  if (fo_hc_split_sinkhorn(mixes, tokens, hc, sinkhorn_iters, eps, scale, base, pre, post, comb)) return 1;
  for (size_t token = 0; token < tokens; ++token) {
    float *h = hidden_out + token * hidden;
    for (size_t d = 0; d < hidden; ++d) h[d] = 0.0f;
    for (size_t copy = 0; copy < hc; ++copy) {
      const float weight = pre[token * hc + copy];
      const float *s = state + (token * hc + copy) * hidden;
      for (size_t d = 0; d < hidden; ++d) h[d] += weight * s[d];
    }
  }
  return 0;
}

int fo_rms_norm(const float *input, const float *weight, size_t len, float eps,
                float *out) {
  /* models/common/math.rs:22-42: (sum / len + eps).sqrt().recip() */
  if (len == 0) return 1;
  float squares = 0.0f;
  for (size_t i = 0; i < len; ++i) squares += input[i] * input[i];
  const float scale = 1.0f / sqrtf(squares / (float)len + eps);
  for (size_t i = 0; i < len; ++i) out[i] = input[i] * scale * weight[i];
  return 0;
}

int fo_hc_producer(const float *state, size_t tokens, size_t hc, size_t hidden,
                   size_t sinkhorn_iters, float eps, float norm_eps,
                   float layer_rms_eps, int bf16_boundaries,
                   const float *function, const float *scale, const float *base,
                   const float *layer_rms_weight, float *raw_dots, float *pre,
                   float *post, float *comb, float *hidden_out, float *normalized,
                   uint8_t *packed, uint8_t *scales) {
  if (hidden % 128 != 0) return 1;
  float *mixes = (float *)malloc(tokens * (2 + hc) * hc * sizeof(float));
  int rc = fo_hc_pre(state, tokens, hc, hidden, sinkhorn_iters, eps, norm_eps, function, scale, base, mixes,
                     raw_dots, pre, post, comb, hidden_out);
  free(mixes);
  if (rc) return rc;
  for (size_t token = 0; token < tokens && !rc; ++token) {
    float *h = hidden_out + token * hidden, *n = normalized + token * hidden;
    if (bf16_boundaries) {
      for (size_t d = 0; d < hidden; ++d) h[d] = fo_round_to_bf16(h[d]);
    }
    rc = fo_rms_norm(h, layer_rms_weight, hidden, layer_rms_eps, n);
    if (bf16_boundaries) {
      for (size_t d = 0; d < hidden; ++d) n[d] = fo_round_to_bf16(n[d]);
    }
  }
  if (rc) return rc;
  return fo_pack_fp8_act(normalized, tokens * hidden, hidden, 128, packed, scales);
}

/* ---- error-bound arithmetic for the parity tests (see the header): sum |w| v in double */
int fo_abs_linear_fp4(const uint8_t *weight, const uint8_t *scales,
                      size_t out_features, size_t in_features, size_t block_size,
                      const double *v, double *out, int threads) {
  if (block_size == 0 || in_features % block_size != 0 || block_size % 2 != 0) return 1;
  const size_t packed_cols = in_features / 2;
  const size_t scale_cols = in_features / block_size;
  double magnitude[16];
  for (int i = 0; i < 16; ++i) magnitude[i] = fabs((double)fo_decode_fp4_e2m1_nibble((uint8_t)i));
#pragma omp parallel for schedule(static) num_threads(threads > 1 ? threads : 1)
  for (long row = 0; row < (long)out_features; ++row) {
    const uint8_t *wrow = weight + (size_t)row * packed_cols;
    const uint8_t *srow = scales + (size_t)row * scale_cols;
    double acc = 0.0;
    for (size_t b = 0; b < scale_cols; ++b) {
      const double scale = (double)fo_decode_e8m0_scale(srow[b]);
      double part = 0.0;
      const size_t k0 = b * block_size;
      for (size_t k = k0; k < k0 + block_size; k += 2) {
        const uint8_t byte = wrow[k / 2];
        part += magnitude[byte & 0x0f] * v[k] + magnitude[byte >> 4] * v[k + 1];
      }
      acc += part * scale;
    }
    out[row] = acc;
  }
  return 0;
}

int fo_abs_linear_fp8(const uint8_t *weight, const void *scales, int scale_kind,
                      size_t out_features, size_t in_features, size_t block_m,
                      size_t block_k, const double *v, double *out, int threads) {
  if (block_m == 0 || block_k == 0) return 1;
  const size_t scale_cols = (in_features + block_k - 1) / block_k;
  double magnitude[256];
  for (int i = 0; i < 256; ++i) {
    const float d = fo_decode_fp8_e4m3fn_byte((uint8_t)i);
    magnitude[i] = d != d ? 0.0 : fabs((double)d);
  }
#pragma omp parallel for schedule(static) num_threads(threads > 1 ? threads : 1)
  for (long row = 0; row < (long)out_features; ++row) {
    const uint8_t *wrow = weight + (size_t)row * in_features;
    const size_t srow = ((size_t)row / block_m) * scale_cols;
    double acc = 0.0;
    for (size_t b = 0; b < scale_cols; ++b) {
      const double scale = scale_kind == FO_SCALE_F32
                               ? fabs((double)((const float *)scales)[srow + b])
                               : (double)fo_decode_e8m0_scale(((const uint8_t *)scales)[srow + b]);
      double part = 0.0;
      const size_t k1 = (b + 1) * block_k < in_features ? (b + 1) * block_k : in_features;
      for (size_t k = b * block_k; k < k1; ++k) part += magnitude[wrow[k]] * v[k];
      acc += part * scale;
    }
    out[row] = acc;
  }
  return 0;
}
