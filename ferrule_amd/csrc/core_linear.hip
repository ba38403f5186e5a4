// Drop-in for ferrule_core_linear_launch, quantized kinds only
// (abi/core_provider.h:477; kernel portable/entrypoints.cu:208-284):
//   kind 4  FP8_E4M3_E8M0           x f32 [batch,k]
//   kind 8  FP8_E4M3_E8M0_FROM_F32  x f32, quantized per (row, block_k) block on the fly
//   kind 5  FP8_E4M3_E8M0_PACKED    x e4m3 [batch,k] + e8m0 [batch, scale_cols], K128 blocks
// Output is f32 [batch,n].  The reference runs one thread per output walking K
// sequentially; here one wavefront owns one weight row, its 64 lanes read the row
// coalesced, and the partial sums are folded with a wave reduction.  Scale blocks of
// any size are accepted, as in the reference.  Kind 5 with whole 128-wide K blocks and
// 16-byte aligned operands goes to the FP8 GEMM schedules instead (see the launch).
//
// Arithmetic: the CPU path (crates/ferrule-model/src/checkpoint/weight.rs:154-173,
// :440-451) multiplies the dequantized weight (decode * 2^s, exact) with the
// activation and accumulates in fp32; the on-the-fly activation quantizer follows
// crates/ferrule-model/src/checkpoint/encoding.rs:207-242 via quant_math.h.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ferrule_hip_provider.h"
#include "fp8_gemm.h"
#include "numeric.cuh"
#include "quant_math.h"

namespace ferrule_hip {
namespace {

constexpr uint32_t kMaxBatchPerPass = 8;

template <int KIND>
__global__ __launch_bounds__(256) void core_linear_kernel(FerruleHipLinearArgs args) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t row = blockIdx.x * 4u + (threadIdx.x >> 6);
  if (row >= args.n) return;
  const uint8_t *weight = global_ptr<const uint8_t>(args.weight) +
                          static_cast<size_t>(row) * args.k;
  const uint8_t *wscale = global_ptr<const uint8_t>(args.weight_scales);
  const float *x_f32 = global_ptr<const float>(args.x);
  const uint8_t *x_u8 = global_ptr<const uint8_t>(args.x);
  const uint8_t *x_scales = global_ptr<const uint8_t>(args.x_scales);
  float *output = global_ptr<float>(args.output);
  const uint32_t block_m = KIND == FERRULE_HIP_LINEAR_FP8_E4M3_E8M0_PACKED ? 128u : args.block_m;
  const uint32_t block_k = KIND == FERRULE_HIP_LINEAR_FP8_E4M3_E8M0_PACKED ? 128u : args.block_k;
  const size_t scale_row = static_cast<size_t>(row / block_m) * args.scale_cols;

  for (uint32_t b0 = 0; b0 < args.batch; b0 += kMaxBatchPerPass) {
    float acc[kMaxBatchPerPass];
#pragma unroll
    for (uint32_t b = 0; b < kMaxBatchPerPass; ++b) acc[b] = 0.f;
    for (uint32_t block = 0; block < args.scale_cols; ++block) {
      const float ws = e8m0_to_f32(wscale[scale_row + block]);
      const uint32_t begin = block * block_k;
      const uint32_t end = min(args.k, begin + block_k);
      float xs[kMaxBatchPerPass];
#pragma unroll
      for (uint32_t b = 0; b < kMaxBatchPerPass; ++b) {
        xs[b] = 1.0f;
        if (b0 + b >= args.batch) continue;
        if constexpr (KIND == FERRULE_HIP_LINEAR_FP8_E4M3_E8M0_FROM_F32) {
          float amax = 0.f;
          for (uint32_t col = begin + lane; col < end; col += 64u) {
            amax = fmaxf(amax, fabsf(x_f32[static_cast<size_t>(b0 + b) * args.k + col]));
          }
          amax = fmaxf(wave_max(amax), 1e-4f);
          xs[b] = ferrule_quant::e8m0_value(ferrule_quant::scale_byte(amax, 448.0f));
        } else if constexpr (KIND == FERRULE_HIP_LINEAR_FP8_E4M3_E8M0_PACKED) {
          xs[b] = e8m0_to_f32(x_scales[static_cast<size_t>(b0 + b) * args.scale_cols + block]);
        }
      }
      for (uint32_t col = begin + lane; col < end; col += 64u) {
        const float w = fp8_e4m3_decode(weight[col]) * ws;  // exact: power-of-two scale
#pragma unroll
        for (uint32_t b = 0; b < kMaxBatchPerPass; ++b) {
          if (b0 + b >= args.batch) continue;
          const size_t xi = static_cast<size_t>(b0 + b) * args.k + col;
          float xv;
          if constexpr (KIND == FERRULE_HIP_LINEAR_FP8_E4M3_E8M0) {
            xv = x_f32[xi];
          } else if constexpr (KIND == FERRULE_HIP_LINEAR_FP8_E4M3_E8M0_FROM_F32) {
            const uint32_t code = ferrule_quant::fp8_e4m3_quantize_byte(
                x_f32[xi], xs[b], FERRULE_HIP_FP8_ROUND_CPU_REFERENCE);
            xv = fp8_e4m3_decode(code) * xs[b];
          } else {
            xv = fp8_e4m3_decode(x_u8[xi]) * xs[b];
          }
          acc[b] = fmaf(w, xv, acc[b]);
        }
      }
    }
#pragma unroll
    for (uint32_t b = 0; b < kMaxBatchPerPass; ++b) {
      const float sum = wave_sum(acc[b]);
      if (lane == 0u && b0 + b < args.batch) {
        output[static_cast<size_t>(b0 + b) * args.n + row] = sum;
      }
    }
  }
}

}  // namespace
}  // namespace ferrule_hip

extern "C" int32_t ferrule_hip_core_linear_launch(const FerruleHipLinearArgs *args) {
  using namespace ferrule_hip;
  // reference: portable/entrypoints.cu:1880-1888 (invalid => cudaErrorInvalidValue = 1)
  if (args == nullptr || args->batch == 0 || args->n == 0) return 1;
  if (args->k == 0 || args->scale_cols == 0 || args->x == 0 || args->weight == 0 ||
      args->weight_scales == 0 || args->output == 0)
    return 1;
  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(args->stream));
  clear_launch_error();
  const uint32_t grid = (args->n + 3u) / 4u;
  switch (args->kind) {
  case FERRULE_HIP_LINEAR_FP8_E4M3_E8M0:
    if (args->block_m == 0 || args->block_k == 0) return 1;
    core_linear_kernel<FERRULE_HIP_LINEAR_FP8_E4M3_E8M0><<<grid, 256, 0, stream>>>(*args);
    break;
  case FERRULE_HIP_LINEAR_FP8_E4M3_E8M0_FROM_F32:
    if (args->block_m == 0 || args->block_k == 0) return 1;
    core_linear_kernel<FERRULE_HIP_LINEAR_FP8_E4M3_E8M0_FROM_F32><<<grid, 256, 0, stream>>>(*args);
    break;
  case FERRULE_HIP_LINEAR_FP8_E4M3_E8M0_PACKED: {
    if (args->x_scales == 0) return 1;
    // The prepacked FP8-K128 linear is the second half of the activation-quantisation policy
    // (pack, then this; crates/ferrule-backend/src/cuda/context.rs:10694-10785) and runs for every
    // dense quantized linear of a decode step.  With whole 128-wide K blocks and aligned operands it is
    // the contraction of the FP8 GEMM entry points, so it takes their schedules: up to 32 rows stream
    // the weights once, more rows run MFMA tiles; unrounded f32 out.  Anything else keeps the
    // one-wave-per-row kernel.
    const uint64_t all = args->x | args->x_scales | args->weight | args->weight_scales | args->output;
    if ((args->k % 128u) == 0 && args->scale_cols == args->k / 128u && (all & 15u) == 0 && args->batch <= 8u * 65535u &&
        fp8_gemm_lds_bytes_small(args->scale_cols) <= 160u * 1024u &&
        static_cast<uint64_t>((args->batch + 127u) / 128u) * ((args->n + 127u) / 128u) <= 0x3fffffffull) {
      Fp8GemmParams p;
      p.x = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(args->x));
      p.xs = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(args->x_scales));
      p.w = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(args->weight));
      p.ws = reinterpret_cast<const void *>(static_cast<uintptr_t>(args->weight_scales));
      p.out = reinterpret_cast<void *>(static_cast<uintptr_t>(args->output));
      p.m = args->batch;
      p.n = args->n;
      p.k = args->k;
      p.cols = args->scale_cols;
      return fp8_gemm_run(p, false, kGemmOutF32Raw, args->stream) == FERRULE_HIP_SUCCESS ? 0 : 1;
    }
    core_linear_kernel<FERRULE_HIP_LINEAR_FP8_E4M3_E8M0_PACKED><<<grid, 256, 0, stream>>>(*args);
    break;
  }
  default:
    return 1;  // the unquantized kinds are not part of this provider
  }
  return static_cast<int32_t>(take_launch_error());
}
