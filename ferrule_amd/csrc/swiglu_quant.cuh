// Register epilogue shared by the gate/up GEMMs (routed experts and the dense shared FFN):
//   h = silu(gate) * up * weight          (clamped first when swiglu_limit > 0)
//   (hq, hs) = FP8-E4M3 / UE8M0 quantisation of h in blocks of 128 along the intermediate dimension
// with the CPU quantiser's rules (crates/ferrule-model/src/checkpoint/encoding.rs:207-242:
// amax floored at 1e-4, scale 2^ceil(log2(amax/448)), its tie rule).  A wave of the GEMM holds
// 128 consecutive features of S::NT token tiles, i.e. exactly one quantisation block per token:
// 32 values in each of the four lanes (i, g=0..3) of a token.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ferrule_hip_provider.h"
#include "mx_gemm.cuh"
#include "quant_math.h"

namespace ferrule_hip {

// row_info(t, r, live, row, weight): for the wave's token tile t, tile-local token row r ->
// whether it exists, its row in the hq/hs arrays and its multiplier (route weight or the FFN's
// output scale).
template <typename S, typename RowInfo>
__device__ __forceinline__ void swiglu_quantize_store(f32x4_t (&acc)[2][S::NF][S::NT], uint32_t lane, uint32_t wave,
                                                      uint32_t f0, uint32_t intermediate_size, float swiglu_limit,
                                                      uint8_t *hq, uint8_t *hs, float *hidden_f32,
                                                      int32_t *error_flag, RowInfo row_info) {
  static_assert(S::NF == 8, "one wave = one 128-wide activation quantisation block");
  const uint32_t i = lane & 15u, g = lane >> 4;
  const uint32_t wf = wave % S::WAVES_F, wt = wave / S::WAVES_F;
  const uint32_t fbase = f0 + wf * 128u;
  if (fbase >= intermediate_size) return;
  const uint32_t scale_cols = intermediate_size >> 7;
#pragma unroll
  for (int t = 0; t < S::NT; ++t) {
    const uint32_t r = S::token_row(wt, t) + i;  // row inside the tile
    bool live;
    size_t row;
    float weight;
    row_info(t, r, live, row, weight);
    float h[S::NF][4];
    float amax = 0.0f;
    bool bad = false;
#pragma unroll
    for (int f = 0; f < S::NF; ++f) {
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        float gate = acc[0][f][t][v];
        float up = acc[1][f][t][v];
        if (swiglu_limit > 0.0f) {
          gate = fminf(gate, swiglu_limit);
          up = fminf(swiglu_limit, fmaxf(-swiglu_limit, up));
        }
        float value = silu_fast(gate) * up * weight;
        if (!(fabsf(value) <= 3.4028234e38f)) {  // NaN or inf: sm103/grouped_fp4_moe.cuh:611-614
          value = 0.0f;
          bad = live;
        }
        h[f][v] = value;
        amax = fmaxf(amax, fabsf(value));
      }
    }
    // the other three lanes of this token hold the rest of the 128-wide block
    amax = fmaxf(amax, __shfl_xor(amax, 16));
    amax = fmaxf(amax, __shfl_xor(amax, 32));
    const uint32_t sbyte = ferrule_quant::scale_byte(fmaxf(amax, 1.0e-4f), 448.0f);
    // amax is floored at 1e-4 and finite: the byte lies in [105, 247] and the inverse is exact
    const float inv_scale = ferrule_quant::e8m0_inverse(sbyte);
    if (bad && error_flag != nullptr) atomicOr(error_flag, 1);
    // The bytes come from the hardware converter (round to nearest even) wherever that is the
    // CPU quantiser's byte: the two differ only where a value sits exactly half way between two
    // codes (the CPU rule sends most ties away from zero), and such a value has its low 19
    // mantissa bits clear.  If any live lane of the wave holds one (next to never with real
    // activations), the token fragment is encoded once more by the exact routine; the software
    // encoder for all 64 values of a lane cost 7 of this epilogue's 12 microseconds.
    uint32_t packed[S::NF];
    uint32_t low_bits = 0xffffffffu;
#pragma unroll
    for (int f = 0; f < S::NF; ++f) {   // h is finite (see above)
      packed[f] = e4m3_bytes_rne(h[f][0] * inv_scale, h[f][1] * inv_scale, h[f][2] * inv_scale, h[f][3] * inv_scale,
                                 low_bits);
    }
    if (__ballot(live && low_bits == 0u) != 0ull) {
#pragma unroll
      for (int f = 0; f < S::NF; ++f) {
        packed[f] = 0;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          packed[f] |= ferrule_quant::fp8_e4m3_quantize_byte_pow2(h[f][v], inv_scale, FERRULE_HIP_FP8_ROUND_CPU_REFERENCE)
                       << (8 * v);
        }
      }
    }
    if (!live) continue;
    uint8_t *out = hq + row * intermediate_size + fbase + g * 4u;
#pragma unroll
    for (int f = 0; f < S::NF; ++f) {
      *reinterpret_cast<uint32_t *>(out + f * 16) = packed[f];
      if (hidden_f32 != nullptr) {
        *reinterpret_cast<float4 *>(hidden_f32 + row * intermediate_size + fbase + f * 16 + g * 4u) =
            make_float4(h[f][0], h[f][1], h[f][2], h[f][3]);
      }
    }
    if (g == 0u) hs[row * scale_cols + (fbase >> 7)] = static_cast<uint8_t>(sbyte);
  }
}

}  // namespace ferrule_hip
