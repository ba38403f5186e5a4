// Drop-in for ferrule_core_moe_launch, kinds on the quantized MoE path
// (abi/core_provider.h:493; kernel portable/entrypoints.cu:1515-1612):
//   2  WEIGHTED_SWIGLU_F32        hidden = gate*sigmoid(gate)*up*route_weight, with the clamp
//                                 gate=min(gate,L), up in [-L,L] when L > 0
//   7  REDUCE_ROUTES              out[t,h] = bf16(out[t,h] + sum_rank route_output[t*k+rank,h])
//   8  REDUCE_EXPERT_GROUP_ROUTES as 7, but NaN for a token with a missing route or when the
//                                 error flag is raised
// The combine is a strict rank-ordered fp32 left fold starting from the value already in
// `output` (the shared-expert prefix), one BF16 rounding at the end, result held in f32 -
// exactly portable/entrypoints.cu:1604-1610.  Elementwise and HBM bound: each thread owns
// four consecutive h so route_output is read with 16-byte loads.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ferrule_hip_provider.h"
#include "numeric.cuh"
#include "quant_math.h"

namespace ferrule_hip {
namespace {

template <typename T>
__device__ __forceinline__ T *ptr(uint64_t address) {
  return global_ptr<T>(address);
}

__global__ __launch_bounds__(256) void weighted_swiglu_kernel(FerruleHipMoeArgs a) {
  const uint64_t index = static_cast<uint64_t>(blockIdx.x) * 256u + threadIdx.x;
  const uint64_t total = static_cast<uint64_t>(a.experts) * a.batch_columns * a.n;
  if (index >= total) return;
  float gate = ptr<const float>(a.gate)[index];
  float up = ptr<const float>(a.up)[index];
  if (a.swiglu_limit > 0.0f) {
    gate = fminf(gate, a.swiglu_limit);
    up = fminf(a.swiglu_limit, fmaxf(-a.swiglu_limit, up));
  }
  const uint32_t route = static_cast<uint32_t>(index / a.n);
  const float route_weight = a.route_weights != 0 ? ptr<const float>(a.route_weights)[route] : a.route_weight;
  // the CPU path's silu(gate) * up * route_weight (executor.rs:113-117)
  float value = silu_ref(gate) * up * route_weight;
  if (a.route_weights != 0 && value == value && fabsf(value) <= 3.4028234e38f && value != 0.0f) {
    // portable/entrypoints.cu:1533-1536: with per-route weights the value is snapped to the
    // (unscaled) E4M3 grid; the CPU path's tie rule is used
    const uint32_t code = ferrule_quant::fp8_e4m3_quantize_byte(value, 1.0f, FERRULE_HIP_FP8_ROUND_CPU_REFERENCE);
    value = fp8_e4m3_decode(code);
  }
  ptr<float>(a.hidden_values)[index] = value;
}

template <bool CHECK>
__global__ __launch_bounds__(256) void reduce_routes_kernel(FerruleHipMoeArgs a) {
  // one thread per 4 consecutive hidden elements when hidden % 4 == 0, else per element
  const bool vec = (a.hidden & 3u) == 0u;
  const uint32_t per_row = vec ? a.hidden >> 2 : a.hidden;
  const uint64_t index = static_cast<uint64_t>(blockIdx.x) * 256u + threadIdx.x;
  if (index >= static_cast<uint64_t>(a.tokens) * per_row) return;
  const uint32_t token = static_cast<uint32_t>(index / per_row);
  const uint32_t h0 = static_cast<uint32_t>(index % per_row) * (vec ? 4u : 1u);
  float *out = ptr<float>(a.output) + static_cast<size_t>(token) * a.hidden + h0;
  const uint32_t width = vec ? 4u : 1u;
  bool complete = true;
  if constexpr (CHECK) {
    complete = ptr<const int32_t>(a.route_error)[0] == 0;
    for (uint32_t rank = 0; rank < a.routes_per_token; ++rank) {
      complete &= ptr<const int32_t>(a.route_written)[token * a.routes_per_token + rank] != 0;
    }
  }
  if (!complete) {
    for (uint32_t e = 0; e < width; ++e) out[e] = __uint_as_float(0x7fc00000u);
    return;
  }
  const float *routes = ptr<const float>(a.route_output);
  if (vec) {
    float4 acc = *reinterpret_cast<const float4 *>(out);
    // route rows are read once: eight nontemporal loads in flight, added in rank order
    typedef float f32x4v __attribute__((ext_vector_type(4)));
    const f32x4v *first = reinterpret_cast<const f32x4v *>(routes + static_cast<size_t>(token) * a.routes_per_token * a.hidden + h0);
    const size_t stride = a.hidden >> 2;
    for (uint32_t rank0 = 0; rank0 < a.routes_per_token; rank0 += 8u) {
      f32x4v v[8];
#pragma unroll
      for (uint32_t j = 0; j < 8u; ++j) {
        v[j] = f32x4v{0.f, 0.f, 0.f, 0.f};
        if (rank0 + j < a.routes_per_token) v[j] = __builtin_nontemporal_load(first + (rank0 + j) * stride);
      }
#pragma unroll
      for (uint32_t j = 0; j < 8u; ++j) {
        if (rank0 + j < a.routes_per_token) {
          acc.x += v[j][0]; acc.y += v[j][1]; acc.z += v[j][2]; acc.w += v[j][3];
        }
      }
    }
    *reinterpret_cast<float4 *>(out) =
        make_float4(bf16_round(acc.x), bf16_round(acc.y), bf16_round(acc.z), bf16_round(acc.w));
  } else {
    float acc = out[0];
    for (uint32_t rank = 0; rank < a.routes_per_token; ++rank) {
      const size_t route = static_cast<size_t>(token) * a.routes_per_token + rank;
      acc += routes[route * a.hidden + h0];
    }
    out[0] = bf16_round(acc);
  }
}

}  // namespace
}  // namespace ferrule_hip

extern "C" int32_t ferrule_hip_core_moe_launch(const FerruleHipMoeArgs *args) {
  using namespace ferrule_hip;
  if (args == nullptr) return 1;  // hipErrorInvalidValue, as portable/entrypoints.cu:1542-1547
  const FerruleHipMoeArgs &a = *args;
  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(a.stream));
  clear_launch_error();
  if (a.kind == FERRULE_HIP_MOE_WEIGHTED_SWIGLU_F32) {
    const uint64_t total = static_cast<uint64_t>(a.experts) * a.batch_columns * a.n;
    if (a.gate == 0 || a.up == 0 || a.hidden_values == 0) return 1;
    if (total == 0) return 0;
    weighted_swiglu_kernel<<<static_cast<uint32_t>((total + 255u) / 256u), 256, 0, stream>>>(a);
  } else if (a.kind == FERRULE_HIP_MOE_REDUCE_ROUTES || a.kind == FERRULE_HIP_MOE_REDUCE_EXPERT_GROUP_ROUTES) {
    if (a.route_output == 0 || a.output == 0 || a.hidden == 0) return 1;
    const bool check = a.kind == FERRULE_HIP_MOE_REDUCE_EXPERT_GROUP_ROUTES;
    if (check && (a.route_written == 0 || a.route_error == 0)) return 1;
    const uint32_t per_row = (a.hidden & 3u) == 0u ? a.hidden >> 2 : a.hidden;
    const uint64_t total = static_cast<uint64_t>(a.tokens) * per_row;
    if (total == 0) return 0;
    const uint32_t grid = static_cast<uint32_t>((total + 255u) / 256u);
    if (check) {
      reduce_routes_kernel<true><<<grid, 256, 0, stream>>>(a);
    } else {
      reduce_routes_kernel<false><<<grid, 256, 0, stream>>>(a);
    }
  } else {
    return 1;
  }
  return static_cast<int32_t>(take_launch_error());
}
