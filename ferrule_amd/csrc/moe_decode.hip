// Decode MoE layer over MXFP4 experts with BF16 activations (no activation quantisation).
//
// Semantics, per route (token t, rank j, expert e, router weight w):
//   gate = W1_e x_t, up = W3_e x_t          fp32 accumulation
//   clamp when swiglu_limit > 0:  gate = min(gate, L), up = clamp(up, -L, L)
//   h    = silu(gate) * up * w              (left to right, fp32)
//   y    = W2_e h                           fp32 accumulation
// which is CpuReferenceExpertExecutor::execute with its default construction
// (crates/ferrule-model/src/moe/executor.rs:82-124); then per token the routes are summed
// in rank order (crates/ferrule-model/src/moe/routed.rs:85-110) on top of an optional f32
// prefix, and rounded once to BF16 (crates/ferrule-model/src/models/common/math.rs:7-14).
//
// Three launches:
//   gate_up : grid (I/64, groups); a workgroup = 4 waves, each wave owns one 16-row tile of
//             W1 and the same tile of W3 and walks ALL of K, so no cross-wave reduction is
//             needed and SwiGLU * weight is applied straight from the accumulators.
//   down    : grid (H/64, groups); each wave owns one 16-row tile of W2; h is consumed as
//             hi + lo BF16 halves (two MFMAs per weight fragment) so the fp32 h of the
//             reference is represented to 2^-17 instead of being rounded to BF16.
//   combine : rank-ordered fp32 fold + single BF16 writeback.
// Data movement: every weight byte is read once with 16-byte non-temporal loads, DEPTH K
// blocks ahead per wave (register ring).  The activations of the (up to 16) tokens routed
// to the expert are staged through LDS in 512-wide K chunks, double buffered, shared by the
// four waves; the next chunk's global loads are in flight while the current one is used.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ferrule_hip_provider.h"
#include "numeric.cuh"
#include "skinny_core.cuh"

namespace ferrule_hip {
namespace {

constexpr uint32_t kRowPad = 8;           // BF16 elements of padding per LDS row (16 bytes)
constexpr uint32_t kTokenTile = 16;
constexpr uint32_t kWaves = 4;

struct MoeParams {
  const int32_t *active_expert_slots;
  const int32_t *expert_route_indptr;
  const int32_t *route_token_indices;
  const int32_t *route_indices;
  const float *route_weights;
  const int32_t *host_scalars;
  const uint64_t *gate_ptrs, *gate_scale_ptrs, *up_ptrs, *up_scale_ptrs, *down_ptrs, *down_scale_ptrs;
  const uint16_t *input;
  float *route_output;
  int32_t *route_written;
  int32_t *route_error;
  const float *prefix;
  uint16_t *output;
  uint16_t *hidden_hi;
  uint16_t *hidden_lo;
  uint32_t active_group_count, slot_capacity, num_tokens, num_routes, routes_per_token;
  uint32_t input_size, intermediate_size, hidden_size, flags;
  float swiglu_limit;
};

// Geometry of the activation staging for a chunk of CKB K blocks (CKB*128 BF16 per row):
// a row is CKB*16 pieces of 16 bytes; the 256 threads cover 256/(CKB*16) rows per pass.
template <int CKB>
struct StageGeometry {
  static constexpr uint32_t kChunk = CKB * 128u;
  static constexpr uint32_t kLdsRow = kChunk + kRowPad;
  static constexpr uint32_t kPiecesPerRow = CKB * 16u;
  static constexpr uint32_t kRowsPerPass = 256u / kPiecesPerRow;
  static constexpr int kPasses = kTokenTile / kRowsPerPass;
  __device__ static uint32_t row(int pass) { return pass * kRowsPerPass + threadIdx.x / kPiecesPerRow; }
  __device__ static uint32_t piece() { return threadIdx.x % kPiecesPerRow; }
};

template <int NX, int CKB>
struct StageRegs {
  u32x4_t v[NX][StageGeometry<CKB>::kPasses];
};

template <int NX, int CKB>
__device__ __forceinline__ void stage_load(StageRegs<NX, CKB> &regs,
                                           const uint16_t *(&src)[NX][StageGeometry<CKB>::kPasses],
                                           uint32_t chunk, uint32_t k) {
  using G = StageGeometry<CKB>;
  const uint32_t k0 = chunk * G::kChunk + G::piece() * 8u;
  const u32x4_t zero4 = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int s = 0; s < NX; ++s) {
#pragma unroll
    for (int pass = 0; pass < G::kPasses; ++pass) {
      regs.v[s][pass] = zero4;
      if (src[s][pass] != nullptr && k0 < k) regs.v[s][pass] = load16(src[s][pass] + k0);
    }
  }
}

template <int NX, int CKB>
__device__ __forceinline__ void stage_store(const StageRegs<NX, CKB> &regs, uint16_t *xs, uint32_t buffer) {
  using G = StageGeometry<CKB>;
#pragma unroll
  for (int s = 0; s < NX; ++s) {
#pragma unroll
    for (int pass = 0; pass < G::kPasses; ++pass) {
      uint16_t *dst = xs + ((buffer * NX + s) * kTokenTile + G::row(pass)) * G::kLdsRow + G::piece() * 8u;
      *reinterpret_cast<u32x4_t *>(dst) = regs.v[s][pass];
    }
  }
}

template <int NX, int CKB>
__device__ __forceinline__ void lds_read_x(XFrag<NX> &f, const uint16_t *xs, uint32_t buffer, uint32_t kk,
                                           uint32_t r, uint32_t g) {
  using G = StageGeometry<CKB>;
#pragma unroll
  for (int s = 0; s < NX; ++s) {
    const uint16_t *src = xs + ((buffer * NX + s) * kTokenTile + r) * G::kLdsRow + kk * 128u + g * 32u;
#pragma unroll
    for (int d = 0; d < 4; ++d) f.x[s][d] = *reinterpret_cast<const u32x4_t *>(src + 8 * d);
  }
}

// One token tile: acc[m] += W_m[16 rows, K] * X[K, <=16 tokens].  Every wave of the
// workgroup must call this (barriers inside); `active` waves own a row tile.
template <int NMAT, int NX, int DEPTH, int CKB>
__device__ __forceinline__ void rowstream_tile(const Fp4Operands<NMAT, NX> &op,
                                               const uint16_t *(&src)[NX][StageGeometry<CKB>::kPasses],
                                               uint16_t *xs, bool active, uint32_t lane,
                                               f32x4_t (&acc)[NMAT]) {
  static_assert(DEPTH % CKB == 0, "the ring is addressed with the unrolled block index");
  using G = StageGeometry<CKB>;
  constexpr int kChunksPerRound = DEPTH / CKB;
  const uint32_t r = lane & 15u;
  const uint32_t g = lane >> 4;
  const uint32_t kblocks = op.k >> 7;
  const uint32_t nchunks = (op.k + G::kChunk - 1u) / G::kChunk;
  Fp4WFrag<NMAT> ring[DEPTH];
  StageRegs<NX, CKB> stage;

  stage_load(stage, src, 0u, op.k);
  if (active) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (static_cast<uint32_t>(d) < kblocks) fp4_load_w(ring[d], op, d, g);
    }
  }
  stage_store(stage, xs, 0u);
  __syncthreads();

  for (uint32_t c0 = 0; c0 < nchunks; c0 += kChunksPerRound) {
#pragma unroll
    for (int cc = 0; cc < kChunksPerRound; ++cc) {
      const uint32_t c = c0 + cc;
      if (c < nchunks) {
        const bool more = c + 1u < nchunks;
        if (more) stage_load(stage, src, c + 1u, op.k);
        if (active) {
#pragma unroll
          for (int kk = 0; kk < CKB; ++kk) {
            const uint32_t kb = c * CKB + kk;
            if (kb < kblocks) {
              XFrag<NX> xf;
              lds_read_x<NX, CKB>(xf, xs, c & 1u, kk, r, g);
              fp4_mac(ring[cc * CKB + kk], xf, acc);
              if (kb + DEPTH < kblocks) fp4_load_w(ring[cc * CKB + kk], op, kb + DEPTH, g);
            }
          }
        }
        if (more) stage_store(stage, xs, (c + 1u) & 1u);
        __syncthreads();
      }
    }
  }
}

__device__ __forceinline__ uint32_t live_groups(const MoeParams &p) {
  uint32_t groups = p.active_group_count;
  if (p.host_scalars != nullptr) {
    const int32_t planned = p.host_scalars[0];
    groups = planned < 0 ? 0u : min(groups, static_cast<uint32_t>(planned));
  }
  return groups;
}

template <int DEPTH>
__global__ __launch_bounds__(256) void moe_gate_up_kernel(MoeParams p) {
  constexpr int CKB = 4;
  using G = StageGeometry<CKB>;
  __shared__ __attribute__((aligned(16))) uint16_t xs[2 * 1 * kTokenTile * G::kLdsRow];
  const uint32_t group = blockIdx.y;
  if (group >= live_groups(p)) return;
  const int32_t slot = p.active_expert_slots[group];
  if (slot < 0 || static_cast<uint32_t>(slot) >= p.slot_capacity) {
    if (threadIdx.x == 0) atomicOr(p.route_error, 1);
    return;
  }
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t r = lane & 15u;
  const uint32_t g = lane >> 4;
  const uint32_t tile = blockIdx.x * kWaves + wave;
  const bool active = tile * 16u < p.intermediate_size;
  const uint32_t wrow = min(tile * 16u + r, p.intermediate_size - 1u);
  const uint32_t row_begin = static_cast<uint32_t>(p.expert_route_indptr[group]);
  const uint32_t row_end = static_cast<uint32_t>(p.expert_route_indptr[group + 1]);

  Fp4Operands<2, 1> op;
  const uint8_t *gate_w = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(p.gate_ptrs[slot]));
  const uint8_t *gate_s = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(p.gate_scale_ptrs[slot]));
  const uint8_t *up_w = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(p.up_ptrs[slot]));
  const uint8_t *up_s = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(p.up_scale_ptrs[slot]));
  op.wrow[0] = gate_w + static_cast<size_t>(wrow) * (p.input_size >> 1);
  op.srow[0] = gate_s + static_cast<size_t>(wrow) * (p.input_size >> 5);
  op.wrow[1] = up_w + static_cast<size_t>(wrow) * (p.input_size >> 1);
  op.srow[1] = up_s + static_cast<size_t>(wrow) * (p.input_size >> 5);
  op.xrow[0] = nullptr;
  op.k = p.input_size;

  for (uint32_t t0 = row_begin; t0 < row_end; t0 += kTokenTile) {
    const uint32_t m = min(kTokenTile, row_end - t0);
    const uint16_t *src[1][G::kPasses];
#pragma unroll
    for (int pass = 0; pass < G::kPasses; ++pass) {
      const uint32_t row = G::row(pass);
      src[0][pass] = nullptr;
      if (row < m) {
        const int32_t token = p.route_token_indices[t0 + row];
        if (token >= 0 && static_cast<uint32_t>(token) < p.num_tokens) {
          src[0][pass] = p.input + static_cast<size_t>(token) * p.input_size;
        }
      }
    }
    f32x4_t acc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    rowstream_tile<2, 1, DEPTH, CKB>(op, src, xs, active, lane, acc);
    if (active && r < m) {
      const float weight = p.route_weights[t0 + r];
      uint32_t hi[4], lo[4];
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        float gate = acc[0][v];
        float up = acc[1][v];
        if (p.swiglu_limit > 0.0f) {
          gate = fminf(gate, p.swiglu_limit);
          up = fminf(p.swiglu_limit, fmaxf(-p.swiglu_limit, up));
        }
        const float h = silu_ref(gate) * up * weight;
        hi[v] = bf16_rne_bits(h);
        lo[v] = bf16_rne_bits(h - bf16_bits_to_f32(hi[v]));
      }
      const size_t o = static_cast<size_t>(t0 + r) * p.intermediate_size + tile * 16u + g * 4u;
      *reinterpret_cast<uint2 *>(p.hidden_hi + o) = make_uint2(hi[0] | (hi[1] << 16), hi[2] | (hi[3] << 16));
      *reinterpret_cast<uint2 *>(p.hidden_lo + o) = make_uint2(lo[0] | (lo[1] << 16), lo[2] | (lo[3] << 16));
    }
  }
}

template <int DEPTH>
__global__ __launch_bounds__(256) void moe_down_kernel(MoeParams p) {
  constexpr int CKB = 2;
  using G = StageGeometry<CKB>;
  __shared__ __attribute__((aligned(16))) uint16_t xs[2 * 2 * kTokenTile * G::kLdsRow];
  const uint32_t group = blockIdx.y;
  if (group >= live_groups(p)) return;
  const int32_t slot = p.active_expert_slots[group];
  if (slot < 0 || static_cast<uint32_t>(slot) >= p.slot_capacity) return;  // flagged by gate_up
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t r = lane & 15u;
  const uint32_t g = lane >> 4;
  const uint32_t tile = blockIdx.x * kWaves + wave;
  const bool active = tile * 16u < p.hidden_size;
  const uint32_t wrow = min(tile * 16u + r, p.hidden_size - 1u);
  const uint32_t row_begin = static_cast<uint32_t>(p.expert_route_indptr[group]);
  const uint32_t row_end = static_cast<uint32_t>(p.expert_route_indptr[group + 1]);

  Fp4Operands<1, 2> op;
  const uint8_t *down_w = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(p.down_ptrs[slot]));
  const uint8_t *down_s = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(p.down_scale_ptrs[slot]));
  op.wrow[0] = down_w + static_cast<size_t>(wrow) * (p.intermediate_size >> 1);
  op.srow[0] = down_s + static_cast<size_t>(wrow) * (p.intermediate_size >> 5);
  op.xrow[0] = nullptr;
  op.xrow[1] = nullptr;
  op.k = p.intermediate_size;

  for (uint32_t t0 = row_begin; t0 < row_end; t0 += kTokenTile) {
    const uint32_t m = min(kTokenTile, row_end - t0);
    const uint16_t *src[2][G::kPasses];
#pragma unroll
    for (int pass = 0; pass < G::kPasses; ++pass) {
      const uint32_t row = G::row(pass);
      const bool valid = row < m;
      src[0][pass] = valid ? p.hidden_hi + static_cast<size_t>(t0 + row) * p.intermediate_size : nullptr;
      src[1][pass] = valid ? p.hidden_lo + static_cast<size_t>(t0 + row) * p.intermediate_size : nullptr;
    }
    f32x4_t acc[1] = {{0.f, 0.f, 0.f, 0.f}};
    rowstream_tile<1, 2, DEPTH, CKB>(op, src, xs, active, lane, acc);
    if (active && r < m) {
      const int32_t route = p.route_indices[t0 + r];
      if (route >= 0 && static_cast<uint32_t>(route) < p.num_routes) {
        float *out = p.route_output + static_cast<size_t>(route) * p.hidden_size + tile * 16u + g * 4u;
        *reinterpret_cast<float4 *>(out) = make_float4(acc[0][0], acc[0][1], acc[0][2], acc[0][3]);
        if (tile == 0u && g == 0u) p.route_written[route] = 1;
      }
    }
  }
}

// output[t,h] = bf16(prefix[t,h] + sum over ranks in order); NaN when a route of the token
// was not produced or the error flag is up (portable/entrypoints.cu:1591-1603).
__global__ __launch_bounds__(256) void moe_combine_kernel(MoeParams p) {
  const uint32_t per_row = p.hidden_size >> 2;
  const uint64_t index = static_cast<uint64_t>(blockIdx.x) * 256u + threadIdx.x;
  if (index >= static_cast<uint64_t>(p.num_tokens) * per_row) return;
  const uint32_t token = static_cast<uint32_t>(index / per_row);
  const uint32_t h0 = static_cast<uint32_t>(index % per_row) * 4u;
  bool complete = p.route_error[0] == 0;
  for (uint32_t rank = 0; rank < p.routes_per_token; ++rank) {
    complete &= p.route_written[token * p.routes_per_token + rank] != 0;
  }
  uint16_t *out = p.output + static_cast<size_t>(token) * p.hidden_size + h0;
  if (!complete) {
    *reinterpret_cast<uint2 *>(out) = make_uint2(0x7fc07fc0u, 0x7fc07fc0u);
    return;
  }
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  uint32_t first = 0;
  if (p.prefix != nullptr) {
    acc = *reinterpret_cast<const float4 *>(p.prefix + static_cast<size_t>(token) * p.hidden_size + h0);
  } else if (p.routes_per_token > 0) {
    // routed.rs:183-201: the first route initialises the accumulator
    acc = *reinterpret_cast<const float4 *>(
        p.route_output + static_cast<size_t>(token) * p.routes_per_token * p.hidden_size + h0);
    first = 1;
  }
  for (uint32_t rank = first; rank < p.routes_per_token; ++rank) {
    const size_t route = static_cast<size_t>(token) * p.routes_per_token + rank;
    const float4 v = *reinterpret_cast<const float4 *>(p.route_output + route * p.hidden_size + h0);
    acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
  }
  const uint32_t b0 = bf16_rne_bits(acc.x), b1 = bf16_rne_bits(acc.y);
  const uint32_t b2 = bf16_rne_bits(acc.z), b3 = bf16_rne_bits(acc.w);
  *reinterpret_cast<uint2 *>(out) = make_uint2(b0 | (b1 << 16), b2 | (b3 << 16));
}

inline uint64_t align256(uint64_t v) { return (v + 255u) & ~static_cast<uint64_t>(255u); }

inline uint64_t hidden_plane_bytes(const FerruleHipMoeDecodeArgs &a) {
  return align256(static_cast<uint64_t>(a.total_routed_rows) * a.intermediate_size * 2u);
}

int32_t validate(const FerruleHipMoeDecodeArgs *a) {
  if (a == nullptr) return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->active_group_count == 0 || a->slot_capacity == 0 || a->active_group_count > a->slot_capacity)
    return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->total_routed_rows == 0 || a->num_tokens == 0 || a->num_routes == 0 || a->routes_per_token == 0)
    return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->num_routes != a->num_tokens * a->routes_per_token) return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->input_size == 0 || a->intermediate_size == 0 || a->hidden_size == 0)
    return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->input_size % 128u != 0 || a->intermediate_size % 128u != 0 || a->hidden_size % 16u != 0)
    return FERRULE_HIP_UNSUPPORTED;
  if (a->active_group_count > 65535u) return FERRULE_HIP_UNSUPPORTED;
  const uint64_t ptrs[] = {a->active_expert_slots, a->expert_route_indptr, a->route_token_indices,
                           a->route_indices, a->route_weights, a->gate_ptrs, a->gate_scale_ptrs,
                           a->up_ptrs, a->up_scale_ptrs, a->down_ptrs, a->down_scale_ptrs,
                           a->input_bf16, a->route_output, a->route_written, a->route_error, a->workspace};
  for (uint64_t v : ptrs) {
    if (v == 0) return FERRULE_HIP_INVALID_ARGUMENT;
  }
  if ((a->input_bf16 & 15u) || (a->route_output & 15u) || (a->workspace & 255u))
    return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->flags & FERRULE_HIP_MOE_DECODE_COMBINE) {
    if (a->output == 0 || (a->output & 7u)) return FERRULE_HIP_INVALID_ARGUMENT;
    if ((a->flags & FERRULE_HIP_MOE_DECODE_PREFIX_F32) && (a->prefix_f32 == 0 || (a->prefix_f32 & 15u)))
      return FERRULE_HIP_INVALID_ARGUMENT;
  }
  if (a->workspace_bytes < 2u * hidden_plane_bytes(*a)) return FERRULE_HIP_INVALID_ARGUMENT;
  return FERRULE_HIP_SUCCESS;
}

template <typename T>
T *as_ptr(uint64_t v) {
  return reinterpret_cast<T *>(static_cast<uintptr_t>(v));
}

}  // namespace
}  // namespace ferrule_hip

using namespace ferrule_hip;

extern "C" uint64_t ferrule_hip_moe_decode_workspace_size(const FerruleHipMoeDecodeArgs *args) {
  if (args == nullptr || args->total_routed_rows == 0 || args->intermediate_size == 0) return 0;
  return 2u * hidden_plane_bytes(*args);
}

extern "C" int32_t ferrule_hip_moe_decode_can_implement(const FerruleHipMoeDecodeArgs *args) {
  return validate(args);
}

extern "C" int32_t ferrule_hip_moe_decode_launch(const FerruleHipMoeDecodeArgs *args) {
  const int32_t status = validate(args);
  if (status != FERRULE_HIP_SUCCESS) return status;
  const FerruleHipMoeDecodeArgs &a = *args;
  MoeParams p;
  p.active_expert_slots = as_ptr<const int32_t>(a.active_expert_slots);
  p.expert_route_indptr = as_ptr<const int32_t>(a.expert_route_indptr);
  p.route_token_indices = as_ptr<const int32_t>(a.route_token_indices);
  p.route_indices = as_ptr<const int32_t>(a.route_indices);
  p.route_weights = as_ptr<const float>(a.route_weights);
  p.host_scalars = as_ptr<const int32_t>(a.host_scalars);
  p.gate_ptrs = as_ptr<const uint64_t>(a.gate_ptrs);
  p.gate_scale_ptrs = as_ptr<const uint64_t>(a.gate_scale_ptrs);
  p.up_ptrs = as_ptr<const uint64_t>(a.up_ptrs);
  p.up_scale_ptrs = as_ptr<const uint64_t>(a.up_scale_ptrs);
  p.down_ptrs = as_ptr<const uint64_t>(a.down_ptrs);
  p.down_scale_ptrs = as_ptr<const uint64_t>(a.down_scale_ptrs);
  p.input = as_ptr<const uint16_t>(a.input_bf16);
  p.route_output = as_ptr<float>(a.route_output);
  p.route_written = as_ptr<int32_t>(a.route_written);
  p.route_error = as_ptr<int32_t>(a.route_error);
  p.prefix = (a.flags & FERRULE_HIP_MOE_DECODE_PREFIX_F32) ? as_ptr<const float>(a.prefix_f32) : nullptr;
  p.output = as_ptr<uint16_t>(a.output);
  p.hidden_hi = as_ptr<uint16_t>(a.workspace);
  p.hidden_lo = as_ptr<uint16_t>(a.workspace + hidden_plane_bytes(a));
  p.active_group_count = a.active_group_count;
  p.slot_capacity = a.slot_capacity;
  p.num_tokens = a.num_tokens;
  p.num_routes = a.num_routes;
  p.routes_per_token = a.routes_per_token;
  p.input_size = a.input_size;
  p.intermediate_size = a.intermediate_size;
  p.hidden_size = a.hidden_size;
  p.flags = a.flags;
  p.swiglu_limit = a.swiglu_limit;

  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(a.stream));
  clear_launch_error();
  const dim3 gate_grid((a.intermediate_size / 16u + kWaves - 1u) / kWaves, a.active_group_count);
  if (!(a.flags & FERRULE_HIP_MOE_DECODE_SKIP_GATE_UP)) moe_gate_up_kernel<4><<<gate_grid, 256, 0, stream>>>(p);
  const dim3 down_grid((a.hidden_size / 16u + kWaves - 1u) / kWaves, a.active_group_count);
  if (!(a.flags & FERRULE_HIP_MOE_DECODE_SKIP_DOWN)) moe_down_kernel<4><<<down_grid, 256, 0, stream>>>(p);
  if (a.flags & FERRULE_HIP_MOE_DECODE_COMBINE) {
    const uint64_t total = static_cast<uint64_t>(a.num_tokens) * (a.hidden_size / 4u);
    moe_combine_kernel<<<static_cast<uint32_t>((total + 255u) / 256u), 256, 0, stream>>>(p);
  }
  return take_launch_error() == hipSuccess ? FERRULE_HIP_SUCCESS : FERRULE_HIP_LAUNCH_FAILED;
}
