// Dense FP8 SwiGLU FFN over packed rows: drop-in for ferrule_cutlass_shared_ffn_*
// (abi/cutlass_provider.h:113-142, 407-410; kernel capabilities/shared_ffn.cuh:295-594).
//   gate/up   one GEMM on the scaled MFMA: W1 and W3 tiles share every token fragment; the
//             register epilogue applies SwiGLU x output_scale and the FP8-K128 activation
//             quantiser (the same epilogue as the routed experts)
//   down      the FP8 block GEMM of fp8_gemm.hip with unrounded fp32 output (or += output)
// Arithmetic follows SwiGluFfn::reference_execute (crates/ferrule-model/src/ffn.rs:24-48) with the
// FP8-K128 activation quantisation policy in front of both projections (weight.rs:63-108).
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include "../../include/ferrule_hip_provider.h"
#include "fp8_gemm.h"
#include "mx_gemm.cuh"
#include "swiglu_quant.cuh"

namespace ferrule_hip {
namespace {

// 2 matrices x 128 features x 128 tokens per workgroup; a wave = 128 features x 32 tokens
template <int NSTAGE>
using FfnShape = GemmShape<kMfmaFmtFp8, 2, 8, 2, 1, 4, NSTAGE>;

struct FfnParams {
  const uint8_t *x, *xs, *gate, *gate_s, *up, *up_s;
  float *hidden_f32;
  uint8_t *hq, *hs;
  uint32_t rows, input_size, intermediate_size;
  float output_scale, swiglu_limit;
};

template <typename S>
__host__ __device__ constexpr uint32_t ffn_lds_bytes(uint32_t cols) {
  return S::NSTAGE * S::kStageBytes + ((S::TM * cols + 15u) & ~15u) + 2u * cols * 4u;
}

template <typename S>
__global__ __launch_bounds__(S::kThreads) void shared_ffn_gate_up_kernel(FfnParams p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t tiles_t = (p.rows + S::TM - 1) / S::TM;
  uint32_t id = blockIdx.x;
  const uint32_t per = gridDim.x >> 3;  // contiguous runs per XCD, token tiles fastest
  if (id < per * 8u) id = (id & 7u) * per + (id >> 3);
  const uint32_t t0 = (id % tiles_t) * S::TM;
  const uint32_t f0 = (id / tiles_t) * S::FN;
  const uint32_t cols = p.input_size >> 7;

  uint8_t *stages = lds;
  uint8_t *xsc = lds + S::NSTAGE * S::kStageBytes;
  uint32_t *wsc = reinterpret_cast<uint32_t *>(xsc + ((S::TM * cols + 15u) & ~15u));  // [2][cols]

  // operands from the tile's first rows on: the lane offsets of the cursors are 32-bit
  GemmOperands<2> op;
  op.x = p.x + static_cast<size_t>(t0) * p.input_size;
  op.w[0] = p.gate + static_cast<size_t>(f0) * p.input_size;
  op.w[1] = p.up + static_cast<size_t>(f0) * p.input_size;
  op.wscale[0] = op.wscale[1] = nullptr;
  op.k = p.input_size;
  GemmCursors<S> cur;
  gemm_init_cursors<S>(
      cur, op, wave, lane, [&](uint32_t r) { return (min(t0 + r, p.rows - 1u) - t0) * p.input_size; },
      [&](uint32_t, uint32_t r) { return (min(f0 + r, p.intermediate_size - 1u) - f0) * p.input_size; },
      [&](uint32_t, uint32_t) { return 0u; });
  // the first stages go out first; the scale tables are staged under their latency
  gemm_prologue<S>(cur, stages, p.input_size >> 7, wave);
  for (uint32_t idx = threadIdx.x; idx < S::TM * cols; idx += S::kThreads) {
    const uint32_t row = idx / cols, c = idx - row * cols;
    xsc[idx] = p.xs[static_cast<size_t>(min(t0 + row, p.rows - 1u)) * cols + c];
  }
  for (uint32_t idx = threadIdx.x; idx < 2u * cols; idx += S::kThreads) {
    const uint32_t mat = idx / cols, c = idx - mat * cols;
    wsc[idx] = (mat == 0u ? p.gate_s : p.up_s)[static_cast<size_t>(f0 >> 7) * cols + c];
  }
  __syncthreads();   // the tables; the stages are waited for by the K loop

  f32x4_t acc[2][S::NF][S::NT];
#pragma unroll
  for (int mat = 0; mat < 2; ++mat) {
#pragma unroll
    for (int f = 0; f < S::NF; ++f) {
#pragma unroll
      for (int t = 0; t < S::NT; ++t) acc[mat][f][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
  }
  const uint32_t i = lane & 15u;
  const uint32_t wt = wave / S::WAVES_F;
  const uint8_t *my_xsc = xsc + (S::token_row(wt, 0) + i) * cols;
  gemm_mainloop<S, WScaleMode::Byte, true>(
      acc, cur, stages, p.input_size >> 7, wave, lane,
      [&](int t, uint32_t kb) { return static_cast<uint32_t>(my_xsc[t * 16 * cols + kb]); },
      [&](int mat, uint32_t kb) { return wsc[mat * cols + kb]; });

  swiglu_quantize_store<S>(acc, lane, wave, f0, p.intermediate_size, p.swiglu_limit, p.hq, p.hs, p.hidden_f32,
                           nullptr, [&](int, uint32_t r, bool &live, size_t &row, float &weight) {
                             live = t0 + r < p.rows;
                             row = t0 + r;
                             weight = p.output_scale;
                           });
}

constexpr uint32_t kMaxLds = 160u * 1024u;

bool aligned16(uint64_t address) { return address != 0 && (address & 15u) == 0; }

}  // namespace
}  // namespace ferrule_hip

using namespace ferrule_hip;

// capabilities/shared_ffn.cuh:530-575
extern "C" int32_t ferrule_hip_shared_ffn_can_implement(const FerruleHipSharedFfnArgs *args) {
  if (args == nullptr) return FERRULE_HIP_INVALID_ARGUMENT;
  const FerruleHipSharedFfnArgs &a = *args;
  if (!aligned16(a.input_fp8) || !aligned16(a.input_ue8m0) || !aligned16(a.gate_weight_fp8) ||
      !aligned16(a.gate_weight_ue8m0) || !aligned16(a.up_weight_fp8) || !aligned16(a.up_weight_ue8m0) ||
      !aligned16(a.down_weight_fp8) || !aligned16(a.down_weight_ue8m0) || !aligned16(a.hidden_f32) ||
      !aligned16(a.hidden_fp8) || !aligned16(a.hidden_ue8m0) || !aligned16(a.output_f32)) {
    return FERRULE_HIP_INVALID_ARGUMENT;
  }
  if (a.rows == 0 || a.input_size == 0 || a.intermediate_size == 0 || a.output_size == 0 ||
      (a.input_size % 128u) != 0 || (a.intermediate_size % 128u) != 0 || (a.output_size % 16u) != 0) {
    return FERRULE_HIP_INVALID_ARGUMENT;
  }
  if (a.gate_block_m != 128u || a.gate_block_k != 128u || a.up_block_m != 128u || a.up_block_k != 128u ||
      a.down_block_m != 128u || a.down_block_k != 128u) {
    return FERRULE_HIP_INVALID_ARGUMENT;
  }
  if (!isfinite(a.output_scale) || !isfinite(a.swiglu_limit)) return FERRULE_HIP_INVALID_ARGUMENT;
  if ((a.flags & ~(FERRULE_HIP_SHARED_FFN_ACCUMULATE | FERRULE_HIP_SHARED_FFN_TILE_SCHEDULE)) != 0) {
    return FERRULE_HIP_INVALID_ARGUMENT;
  }
  if (ffn_lds_bytes<FfnShape<2>>(a.input_size >> 7) > kMaxLds ||
      fp8_gemm_lds_bytes_small(a.intermediate_size >> 7) > kMaxLds) {
    return FERRULE_HIP_UNSUPPORTED;
  }
  return FERRULE_HIP_SUCCESS;
}

extern "C" int32_t ferrule_hip_shared_ffn_launch(const FerruleHipSharedFfnArgs *args) {
  const int32_t status = ferrule_hip_shared_ffn_can_implement(args);
  if (status != FERRULE_HIP_SUCCESS) return status;
  const FerruleHipSharedFfnArgs &a = *args;
  auto ptr = [](uint64_t v) { return reinterpret_cast<void *>(static_cast<uintptr_t>(v)); };
  FfnParams p;
  p.x = static_cast<const uint8_t *>(ptr(a.input_fp8));
  p.xs = static_cast<const uint8_t *>(ptr(a.input_ue8m0));
  p.gate = static_cast<const uint8_t *>(ptr(a.gate_weight_fp8));
  p.gate_s = static_cast<const uint8_t *>(ptr(a.gate_weight_ue8m0));
  p.up = static_cast<const uint8_t *>(ptr(a.up_weight_fp8));
  p.up_s = static_cast<const uint8_t *>(ptr(a.up_weight_ue8m0));
  p.hidden_f32 = static_cast<float *>(ptr(a.hidden_f32));
  p.hq = static_cast<uint8_t *>(ptr(a.hidden_fp8));
  p.hs = static_cast<uint8_t *>(ptr(a.hidden_ue8m0));
  p.rows = a.rows;
  p.input_size = a.input_size;
  p.intermediate_size = a.intermediate_size;
  p.output_scale = a.output_scale;
  p.swiglu_limit = a.swiglu_limit;
  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(a.stream));
  const uint32_t cols = a.input_size >> 7;
  const uint32_t tiles = ((a.rows + 127u) / 128u) * ((a.intermediate_size + 127u) / 128u);
  Fp8GemmParams d;
  d.x = p.hq;
  d.xs = p.hs;
  d.w = static_cast<const uint8_t *>(ptr(a.down_weight_fp8));
  d.ws = ptr(a.down_weight_ue8m0);
  d.out = ptr(a.output_f32);
  d.m = a.rows;
  d.n = a.output_size;
  d.k = a.intermediate_size;
  d.cols = a.intermediate_size >> 7;
  const int down_mode = (a.flags & FERRULE_HIP_SHARED_FFN_ACCUMULATE) ? kGemmOutF32Accumulate : kGemmOutF32Raw;
  const bool tiles_only = (a.flags & FERRULE_HIP_SHARED_FFN_TILE_SCHEDULE) != 0;
  if (!tiles_only && fp8_rows_applies(a.rows, a.input_size) && fp8_rows_applies(a.rows, a.intermediate_size)) {
    // Decode rows (the reference's small-M form: capabilities/shared_ffn.cuh:477-523): three launches
    // that each stream their operand once over every CU - gate/up with 8 features of both matrices
    // per wave and h in f32, the FP8-K128 quantiser of h (the same bytes as the tiled kernel's
    // register epilogue: both are the CPU quantiser's), the down projection.
    int32_t status = fp8_rows_swiglu_run(p.x, p.xs, p.gate, p.gate_s, p.up, p.up_s, p.hidden_f32, a.rows, a.input_size,
                                         a.intermediate_size, a.output_scale, a.swiglu_limit, a.stream);
    if (status != FERRULE_HIP_SUCCESS) return status;
    FerruleHipQuantizeArgs q = {};
    q.kind = FERRULE_HIP_QUANTIZE_FP8_PACKED;
    q.value_len = a.rows * a.intermediate_size;
    q.row_width = a.intermediate_size;
    q.block_size = 128u;
    q.reserved = FERRULE_HIP_FP8_ROUND_CPU_REFERENCE;
    q.values = a.hidden_f32;
    q.packed = a.hidden_fp8;
    q.scales = a.hidden_ue8m0;
    q.stream = a.stream;
    if (ferrule_hip_core_quantize_launch(&q) != 0) return FERRULE_HIP_LAUNCH_FAILED;
    return fp8_gemm_run(d, false, down_mode, a.stream);
  }
  clear_launch_error();
  hipError_t err;
  if (ffn_lds_bytes<FfnShape<3>>(cols) <= kMaxLds) {
    using S = FfnShape<3>;
    auto kernel = shared_ffn_gate_up_kernel<S>;
    const uint32_t lds = ffn_lds_bytes<S>(cols);
    err = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                              static_cast<int>(lds));
    if (err == hipSuccess) kernel<<<tiles, S::kThreads, lds, stream>>>(p);
  } else {
    using S = FfnShape<2>;
    auto kernel = shared_ffn_gate_up_kernel<S>;
    const uint32_t lds = ffn_lds_bytes<S>(cols);
    err = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                              static_cast<int>(lds));
    if (err == hipSuccess) kernel<<<tiles, S::kThreads, lds, stream>>>(p);
  }
  if (err != hipSuccess) {
    g_last_hip_error = static_cast<int32_t>(err);
    return FERRULE_HIP_LAUNCH_FAILED;
  }
  if (take_launch_error() != 0) return FERRULE_HIP_LAUNCH_FAILED;
  return fp8_gemm_run(d, false, down_mode, a.stream, tiles_only);
}
