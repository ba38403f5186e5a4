// Drop-in for ferrule_core_router_launch (abi/core_provider.h:486; kernel
// portable/entrypoints.cu:770-884): the step that turns router logits into the expert ids
// and route weights the expert-group route plan consumes, without leaving the device.
//   1  ROUTER_TOPK            score = sqrt(max(softplus(logit), 0)); pick the k largest
//                             score + bias (bias only with flags & 1), equal values in
//                             ascending expert order; weight = score / sum * route_scale
//                             with the sum folded left to right in rank order
//   2  ROUTER_HASH            ids come from hash_table[token_ids[row], 0..k); same weights;
//                             a row with a bad token id or table entry is left untouched
//   3  VOCAB_TOPK_F32_INDEX   plain top-k of the logits, ids as f32, weights = the values
//   4  VOCAB_TOPK_I32_INDEX   as 3 with int32 ids
//
// The reference runs one thread per row: a serial scan of the row (strided over rows, so
// uncoalesced) with an insertion sort in thread-private arrays.  Here ONE WAVE owns a row:
//   * lane l holds columns l, l + 64, ... in registers (coalesced 256-byte wave loads): a 32-bit
//     key, the order-preserving image of the selection value, and the value that the outputs
//     need (the score without bias, or the logit for plain top-k);
//   * a round takes the wave maximum of the keys (a per-lane maximum over registers, four DPP
//     steps inside each row of 16 lanes, a scalar maximum over the four rows), then the wave
//     minimum of the columns that hold it - the reference's tie rule: value descending, column
//     ascending among equal values (-0 and +0 are equal, as for its operator==) - and clears
//     that one key.  The owner lane broadcasts the column's score with one v_readlane, so no
//     score is computed twice;
//   * lane r keeps rank r, so the left fold of the sum (a readlane per rank), the division and
//     the 4-byte stores run on k lanes at once.
// A slot beyond the number of columns gets id -1 (and score 0 / value -inf), as the
// reference's sentinel entries do.  NaN selection values (only reachable through a NaN
// bias or inf - inf; the CPU router rejects such inputs, routing.rs:247-262) rank above
// every number here; the reference's insertion order for them depends on the scan
// position and is not reproduced.
//
// Rows wider than 64 * kMaxCandidatesPerLane columns keep nothing in registers: rank r is the
// largest 64-bit key (value image, ~column) strictly below rank r-1's, recomputed from memory in
// every round (correct, k times the loads; the host side of the score router caps experts at
// 512, context.rs:7148-7155, which the register form covers).
//
// softplus is log1p(exp(x)) as in the reference; log1p(e) is evaluated as log(u) * e / (u - 1)
// with u = fl(1 + e), which is log1p to about two ulp at a third of the instructions of the
// library's double-float log1pf (the kernel is VALU bound: 8 MB of logits are 1 us of HBM time).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ferrule_hip_provider.h"
#include "numeric.cuh"

namespace ferrule_hip {
namespace {

constexpr uint32_t kWavesPerWorkgroup = 4;
constexpr int kMaxCandidatesPerLane = 8;

template <typename T>
__device__ __forceinline__ T *ptr(uint64_t address) {
  return global_ptr<T>(address);
}

// portable/entrypoints.cu:103-111
__device__ __forceinline__ float softplus_ref(float value) {
  if (value > 20.0f) return value;
  const float e = expf(value);
  if (value < -20.0f) return e;
  const float u = 1.0f + e;
  const float d = u - 1.0f;  // the part of e that made it into u; 0 when e is below half an ulp of 1
  return d == 0.0f ? e : logf(u) * (e / d);
}

__device__ __forceinline__ float router_score(float logit) {
  return sqrtf(fmaxf(softplus_ref(logit), 0.0f));
}

// Larger key <=> earlier rank.  High word: the float mapped to an unsigned integer in
// numeric order (-0 folded onto +0, NaN on top); low word: ~column, so that the lower
// column wins among equal values.  A real candidate never has key 0 (the high word of
// -inf is 0x007fffff), which is what "no candidate" uses.
__device__ __forceinline__ uint32_t order_key(float value) {
  uint32_t bits = __float_as_uint(value);
  if (bits == 0x80000000u) bits = 0u;
  uint32_t order = (bits & 0x80000000u) != 0u ? ~bits : (bits | 0x80000000u);
  if (value != value) order = 0xfffffffeu;  // below the "nothing chosen yet" bound of round 0
  return order;
}

__device__ __forceinline__ uint64_t selection_key(float value, uint32_t column) {
  return (static_cast<uint64_t>(order_key(value)) << 32) | static_cast<uint32_t>(~column);
}

__device__ __forceinline__ uint64_t max_u64(uint64_t a, uint64_t b) { return a > b ? a : b; }

template <int CTRL>
__device__ __forceinline__ uint64_t dpp_u64(uint64_t v) {
  const int lo = __builtin_amdgcn_update_dpp(0, static_cast<int>(static_cast<uint32_t>(v)), CTRL, 0xf, 0xf, false);
  const int hi = __builtin_amdgcn_update_dpp(0, static_cast<int>(static_cast<uint32_t>(v >> 32)), CTRL, 0xf, 0xf, false);
  return (static_cast<uint64_t>(static_cast<uint32_t>(hi)) << 32) | static_cast<uint32_t>(lo);
}

// Maximum over the 64 lanes, returned wave-uniform.  Inside a row of 16 lanes: quad
// permutes [1,0,3,2] and [2,3,0,1], then half-row and row mirrors; across the four rows
// the values are read into scalar registers.
__device__ __forceinline__ uint64_t wave_max_u64(uint64_t v) {
  v = max_u64(v, dpp_u64<0xb1>(v));
  v = max_u64(v, dpp_u64<0x4e>(v));
  v = max_u64(v, dpp_u64<0x141>(v));
  v = max_u64(v, dpp_u64<0x140>(v));
  uint64_t best = 0;
#pragma unroll
  for (int row = 0; row < 4; ++row) {
    const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(v)), row * 16));
    const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(static_cast<uint32_t>(v >> 32)), row * 16));
    best = max_u64(best, (static_cast<uint64_t>(hi) << 32) | lo);
  }
  return best;
}

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
  return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), CTRL, 0xf, 0xf, false));
}

__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
  v = max(v, dpp_u32<0xb1>(v));
  v = max(v, dpp_u32<0x4e>(v));
  v = max(v, dpp_u32<0x141>(v));
  v = max(v, dpp_u32<0x140>(v));
  uint32_t best = 0;
#pragma unroll
  for (int row = 0; row < 4; ++row) {
    best = max(best, static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), row * 16)));
  }
  return best;
}

__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v) { return ~wave_max_u32(~v); }

// kind 1: SCORE = true; kinds 3/4: SCORE = false
template <bool SCORE>
__device__ __forceinline__ float selection_value(const FerruleHipRouterArgs &a, float logit, uint32_t column) {
  if constexpr (SCORE) {
    const float score = router_score(logit);
    return score + ((a.flags & 1u) != 0u ? ptr<const float>(a.bias)[column] : 0.0f);
  } else {
    return logit;
  }
}

// CPL > 0: the row's keys live in registers, columns <= 64 * CPL.  CPL == 0: any width,
// keys recomputed per round.
template <int CPL, bool SCORE>
__global__ __launch_bounds__(64 * kWavesPerWorkgroup) void router_select_kernel(FerruleHipRouterArgs a) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t row = blockIdx.x * kWavesPerWorkgroup + (threadIdx.x >> 6);
  if (row >= a.rows) return;  // wave-uniform
  const float *line = ptr<const float>(a.logits) + static_cast<uint64_t>(row) * a.columns;

  int32_t chosen = -1;  // lane r ends up with rank r
  // what the outputs need of the chosen column: its score without bias, or its logit
  float picked = SCORE ? 0.0f : __uint_as_float(0xff800000u);
  if constexpr (CPL > 0) {
    uint32_t keys[CPL];
    float payload[CPL];
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
      const uint32_t column = static_cast<uint32_t>(c) * 64u + lane;
      keys[c] = 0u;
      payload[c] = 0.0f;
      if (column < a.columns) {
        const float logit = line[column];
        if constexpr (SCORE) {
          payload[c] = router_score(logit);
          keys[c] = order_key(payload[c] + ((a.flags & 1u) != 0u ? ptr<const float>(a.bias)[column] : 0.0f));
        } else {
          payload[c] = logit;
          keys[c] = order_key(logit);
        }
      }
    }
    for (uint32_t rank = 0; rank < a.k; ++rank) {
      uint32_t best = keys[0];
#pragma unroll
      for (int c = 1; c < CPL; ++c) best = max(best, keys[c]);
      best = wave_max_u32(best);
      if (best == 0u) break;  // wave-uniform: the row is exhausted, later ranks keep -1
      uint32_t column = 0xffffffffu;
#pragma unroll
      for (int c = CPL - 1; c >= 0; --c) column = keys[c] == best ? static_cast<uint32_t>(c) * 64u + lane : column;
      column = wave_min_u32(column);
      const uint32_t mine = column - lane;  // c * 64 in the owner lane only
      float value = 0.0f;
#pragma unroll
      for (int c = 0; c < CPL; ++c) {
        const bool owner = mine == static_cast<uint32_t>(c) * 64u;
        value = owner ? payload[c] : value;
        keys[c] = owner ? 0u : keys[c];
      }
      value = __uint_as_float(static_cast<uint32_t>(
          __builtin_amdgcn_readlane(static_cast<int>(__float_as_uint(value)), static_cast<int>(column & 63u))));
      if (lane == rank) {
        chosen = static_cast<int32_t>(column);
        picked = value;
      }
    }
  } else {
    uint64_t previous = ~0ull;
    for (uint32_t rank = 0; rank < a.k; ++rank) {
      uint64_t best = 0;
      for (uint32_t column = lane; column < a.columns; column += 64u) {
        const uint64_t key = selection_key(selection_value<SCORE>(a, line[column], column), column);
        best = max_u64(best, key < previous ? key : 0ull);
      }
      best = wave_max_u64(best);
      if (lane == rank && best != 0ull) chosen = static_cast<int32_t>(~static_cast<uint32_t>(best));
      previous = best;  // 0 once the row is exhausted: every later round finds nothing
    }
    if (chosen >= 0) picked = SCORE ? router_score(line[chosen]) : line[chosen];
  }

  const bool live = lane < a.k;
  const uint64_t out = static_cast<uint64_t>(row) * a.k + lane;
  if constexpr (SCORE) {
    // portable/entrypoints.cu:816-839: the chosen columns' scores (the reference evaluates them
    // again from the logits, which gives the same values), summed in rank order, one division
    // and one multiplication per weight
    const float score = live ? picked : 0.0f;
    float sum = 0.0f;
    for (uint32_t rank = 0; rank < a.k; ++rank) {
      sum += __uint_as_float(static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(__float_as_uint(score)), rank)));
    }
    if (live) {
      ptr<int32_t>(a.indices)[out] = chosen;
      const bool usable = sum > 0.0f && sum <= 3.4028234e38f;
      ptr<float>(a.weights)[out] = usable ? score / sum * a.route_scale : 0.0f;
    }
  } else {
    if (live) {
      if (a.kind == FERRULE_HIP_VOCAB_TOPK_F32_INDEX) {
        ptr<float>(a.indices)[out] = static_cast<float>(chosen);
      } else {
        ptr<int32_t>(a.indices)[out] = chosen;
      }
      ptr<float>(a.weights)[out] = picked;
    }
  }
}

// kind 2 (portable/entrypoints.cu:840-866): one wave per row, lane r = rank r
__global__ __launch_bounds__(64 * kWavesPerWorkgroup) void router_hash_kernel(FerruleHipRouterArgs a) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t row = blockIdx.x * kWavesPerWorkgroup + (threadIdx.x >> 6);
  if (row >= a.rows) return;  // wave-uniform
  const int32_t token = ptr<const int32_t>(a.token_ids)[row];
  if (token < 0 || static_cast<uint32_t>(token) >= a.hash_rows) return;  // wave-uniform
  const bool live = lane < a.k;
  int32_t expert = 0;
  if (live) expert = ptr<const int32_t>(a.hash_table)[static_cast<uint64_t>(token) * a.hash_columns + lane];
  const bool bad = live && (expert < 0 || static_cast<uint32_t>(expert) >= a.columns);
  if (__any(bad)) return;
  const float *line = ptr<const float>(a.logits) + static_cast<uint64_t>(row) * a.columns;
  const float score = live ? router_score(line[expert]) : 0.0f;
  float sum = 0.0f;
  for (uint32_t rank = 0; rank < a.k; ++rank) {
    sum += __uint_as_float(static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(__float_as_uint(score)), rank)));
  }
  if (live) {
    const uint64_t out = static_cast<uint64_t>(row) * a.k + lane;
    ptr<int32_t>(a.indices)[out] = expert;
    const bool usable = sum > 0.0f && sum <= 3.4028234e38f;
    ptr<float>(a.weights)[out] = usable ? score / sum * a.route_scale : 0.0f;
  }
}

template <bool SCORE>
void launch_select(const FerruleHipRouterArgs &a, uint32_t grid, hipStream_t stream) {
  constexpr uint32_t block = 64 * kWavesPerWorkgroup;
  if (a.columns <= 64u) {
    router_select_kernel<1, SCORE><<<grid, block, 0, stream>>>(a);
  } else if (a.columns <= 128u) {
    router_select_kernel<2, SCORE><<<grid, block, 0, stream>>>(a);
  } else if (a.columns <= 256u) {
    router_select_kernel<4, SCORE><<<grid, block, 0, stream>>>(a);
  } else if (a.columns <= 64u * kMaxCandidatesPerLane) {
    router_select_kernel<kMaxCandidatesPerLane, SCORE><<<grid, block, 0, stream>>>(a);
  } else {
    router_select_kernel<0, SCORE><<<grid, block, 0, stream>>>(a);
  }
}

}  // namespace
}  // namespace ferrule_hip

extern "C" int32_t ferrule_hip_core_router_launch(const FerruleHipRouterArgs *args) {
  using namespace ferrule_hip;
  if (args == nullptr) return 1;  // hipErrorInvalidValue, as portable/entrypoints.cu:1970-1973
  const FerruleHipRouterArgs &a = *args;
  if (a.kind < FERRULE_HIP_ROUTER_TOPK || a.kind > FERRULE_HIP_VOCAB_TOPK_I32_INDEX) return 1;
  // the reference kernel returns at once for these shapes and the launch reports success
  // (portable/entrypoints.cu:795-797)
  if (a.rows == 0 || a.k == 0 || a.k > 64u) return 0;
  if (a.logits == 0 || a.indices == 0 || a.weights == 0) return 1;
  if (a.kind == FERRULE_HIP_ROUTER_TOPK && (a.flags & 1u) != 0u && a.bias == 0) return 1;
  if (a.kind == FERRULE_HIP_ROUTER_HASH && (a.token_ids == 0 || a.hash_table == 0 || a.hash_columns < a.k)) return 1;
  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(a.stream));
  clear_launch_error();
  const uint32_t grid = (a.rows + kWavesPerWorkgroup - 1u) / kWavesPerWorkgroup;
  if (a.kind == FERRULE_HIP_ROUTER_TOPK) {
    launch_select<true>(a, grid, stream);
  } else if (a.kind == FERRULE_HIP_ROUTER_HASH) {
    router_hash_kernel<<<grid, 64 * kWavesPerWorkgroup, 0, stream>>>(a);
  } else {
    launch_select<false>(a, grid, stream);
  }
  return static_cast<int32_t>(take_launch_error());
}
