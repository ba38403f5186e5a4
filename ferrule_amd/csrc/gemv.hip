// Decode GEMV for FP8-e4m3 (block scaled) and MXFP4 (e2m1 + e8m0/32) weights with
// BF16 activations, fp32 accumulation and one BF16 writeback.
//
// Semantics: LinearWeight::reference_matvec per activation row
// (crates/ferrule-model/src/checkpoint/weight.rs:154-173) then round_to_bf16
// (crates/ferrule-model/src/models/common/math.rs:7-14).
//
// Shape of the kernel ("skinny" MFMA GEMV):
//   * a workgroup owns 16 consecutive weight rows; its waves split K in 128-wide
//     blocks (wave w takes blocks w, w+WAVES, ...), so the workgroup's loads of a
//     row are contiguous;
//   * lane (r = lane%16, g = lane/16) loads 16 bytes of row r with one
//     global_load_dwordx4: 32 FP4 values = exactly one E8M0 scale block, or 16
//     FP8 values;
//   * the packed values are expanded to BF16 *exactly* by the gfx950 converters
//     (v_cvt_scalef32_pk_bf16_fp4 / _fp8; the E8M0 scale is applied by the same
//     instruction - e2m1/e4m3 times a power of two is representable in BF16);
//   * v_mfma_f32_16x16x32_bf16 multiplies the 16x32 weight fragment with the
//     32x16 activation fragment (tokens padded to 16 columns).  Products of two
//     BF16 numbers are exact in fp32, so the only rounding is the fp32
//     accumulation, as in the reference;
//   * F32 block scales cannot ride in the converter: the MFMA chain of one
//     128-wide K block lands in a block accumulator that is folded in with one
//     FMA per accumulator register (acc += scale * block);
//   * waves are reduced through LDS, then one BF16 (or f32) store per output.
// The kernel streams every weight byte exactly once; activations (a few KB) come
// from L2.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ferrule_hip_provider.h"
#include "numeric.cuh"
#include "skinny_core.cuh"

namespace ferrule_hip {
namespace {

struct GemvParams {
  const uint8_t *weight;
  const uint8_t *scales;
  const uint16_t *x;
  void *output;
  uint32_t batch;
  uint32_t n;
  uint32_t k;
  uint32_t scale_cols;
  uint32_t block_m;
  uint32_t block_k;
  uint32_t flags;
};

template <int FMT, int SCALE, int WAVES, int DEPTH, int XDEPTH, bool BLOCK_MAJOR = false>
__global__ __launch_bounds__(WAVES * 64) void skinny_gemv_kernel(GemvParams p) {
  __shared__ float red[WAVES][256];
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t r = lane & 15u;
  const uint32_t g = lane >> 4;
  const uint32_t row0 = blockIdx.x * 16u;
  const uint32_t row = min(row0 + r, p.n - 1u);
  const uint32_t kblocks = (p.k + 127u) >> 7;

  for (uint32_t b0 = 0; b0 < p.batch; b0 += 16u) {
    const uint32_t token = b0 + r;
    const uint16_t *xrow = token < p.batch ? p.x + static_cast<size_t>(token) * p.k : nullptr;
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};

    if constexpr (FMT == kFp4) {
      Fp4Operands<1, 1> op;
      if constexpr (BLOCK_MAJOR) {  // n % 16 == 0 and k % 128 == 0 (checked on the host)
        op.wrow[0] = p.weight + static_cast<size_t>(row0) * (p.k >> 1) + r * 64u + g * 16u;
        op.srow[0] = p.scales + static_cast<size_t>(row0) * (p.k >> 5) + r * 4u;
      } else {
        op.wrow[0] = p.weight + static_cast<size_t>(row) * (p.k >> 1);
        op.srow[0] = p.scales + static_cast<size_t>(row) * p.scale_cols;
      }
      op.xrow[0] = xrow;
      op.k = p.k;
      f32x4_t a[1] = {acc};
      fp4_stream<BLOCK_MAJOR, 1, 1, DEPTH, XDEPTH>(op, wave, WAVES, kblocks, g, a);
      acc = a[0];
    } else {
      Fp8Operands op;
      op.wrow = BLOCK_MAJOR ? p.weight + static_cast<size_t>(row0) * p.k + r * 64u + g * 16u
                            : p.weight + static_cast<size_t>(row) * p.k;
      // block_k % 128 == 0 (checked on the host).
      // E8M0: any block_m (the scale rides in each lane's converter).
      // F32 : one scale per (16-row tile, K block), so block_m % 16 == 0.
      op.srow = SCALE == kE8m0
                    ? static_cast<const void *>(p.scales + static_cast<size_t>(row / p.block_m) * p.scale_cols)
                    : static_cast<const void *>(reinterpret_cast<const float *>(p.scales) +
                                                static_cast<size_t>(row0 / p.block_m) * p.scale_cols);
      op.xrow = xrow;
      op.k = p.k;
      op.kb_per_scale = p.block_k >> 7;
      fp8_stream<SCALE, BLOCK_MAJOR, DEPTH, XDEPTH>(op, wave, WAVES, kblocks, g, acc);
    }

    // acc[v] of lane l is (weight row 4*(l/16)+v, token l%16)
#pragma unroll
    for (int v = 0; v < 4; ++v) red[wave][v * 64 + lane] = acc[v];
    __syncthreads();
    if (threadIdx.x < 256u) {
      const uint32_t tok = threadIdx.x >> 4;
      const uint32_t rr = threadIdx.x & 15u;
      const uint32_t idx = (rr & 3u) * 64u + (rr >> 2) * 16u + tok;
      float sum = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) sum += red[w][idx];
      const uint32_t orow = row0 + rr;
      const uint32_t otok = b0 + tok;
      if (orow < p.n && otok < p.batch) {
        const size_t o = static_cast<size_t>(otok) * p.n + orow;
        if (p.flags & FERRULE_HIP_GEMV_OUTPUT_F32) {
          static_cast<float *>(p.output)[o] = sum;
        } else {
          static_cast<uint16_t *>(p.output)[o] = bf16_rne_bits(sum);
        }
      }
    }
    __syncthreads();
  }
}

// Generic shapes (odd K, odd scale blocks): one wave per weight row, software
// decode, fp32 FMA, up to 8 activation rows per pass.
template <int FMT, int SCALE>
__global__ __launch_bounds__(256) void generic_gemv_kernel(GemvParams p) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t row = blockIdx.x * 4u + (threadIdx.x >> 6);
  if (row >= p.n) return;
  for (uint32_t b0 = 0; b0 < p.batch; b0 += 8u) {
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (uint32_t col = lane; col < p.k; col += 64u) {
      float w;
      if constexpr (FMT == kFp4) {
        const uint32_t byte = p.weight[static_cast<size_t>(row) * (p.k >> 1) + (col >> 1)];
        const uint32_t nib = (col & 1u) ? (byte >> 4) : (byte & 15u);
        w = fp4_e2m1_decode(nib) *
            e8m0_to_f32(p.scales[static_cast<size_t>(row) * p.scale_cols + col / p.block_k]);
      } else {
        const float d = fp8_e4m3_decode(p.weight[static_cast<size_t>(row) * p.k + col]);
        const size_t si = static_cast<size_t>(row / p.block_m) * p.scale_cols + col / p.block_k;
        const float s = SCALE == kF32 ? reinterpret_cast<const float *>(p.scales)[si]
                                      : e8m0_to_f32(p.scales[si]);
        w = d * s;
      }
#pragma unroll
      for (uint32_t b = 0; b < 8u; ++b) {
        if (b0 + b < p.batch) {
          acc[b] = fmaf(w, bf16_bits_to_f32(p.x[static_cast<size_t>(b0 + b) * p.k + col]), acc[b]);
        }
      }
    }
#pragma unroll
    for (uint32_t b = 0; b < 8u; ++b) {
      const float sum = wave_sum(acc[b]);
      if (lane == 0u && b0 + b < p.batch) {
        const size_t o = static_cast<size_t>(b0 + b) * p.n + row;
        if (p.flags & FERRULE_HIP_GEMV_OUTPUT_F32) {
          static_cast<float *>(p.output)[o] = sum;
        } else {
          static_cast<uint16_t *>(p.output)[o] = bf16_rne_bits(sum);
        }
      }
    }
  }
}

// Element-wise dequantisation through the same converters the GEMV uses.
template <int FMT, int SCALE>
__global__ __launch_bounds__(256) void dequant_kernel(GemvParams p) {
  // one thread per packed dword
  const size_t dword = static_cast<size_t>(blockIdx.x) * 256u + threadIdx.x;
  float *out = static_cast<float *>(p.output);
  if constexpr (FMT == kFp4) {
    const size_t dwords_per_row = p.k >> 3;
    if (dword >= static_cast<size_t>(p.n) * dwords_per_row) return;
    const uint32_t row = static_cast<uint32_t>(dword / dwords_per_row);
    const uint32_t k0 = static_cast<uint32_t>(dword % dwords_per_row) * 8u;
    const uint32_t packed = reinterpret_cast<const uint32_t *>(p.weight)[dword];
    const float sc = e8m0_to_f32(p.scales[static_cast<size_t>(row) * p.scale_cols + k0 / p.block_k]);
    const bf16x8_t v = expand_fp4_dword(packed, sc);
#pragma unroll
    for (int e = 0; e < 8; ++e) out[static_cast<size_t>(row) * p.k + k0 + e] = static_cast<float>(v[e]);
  } else {
    const size_t dwords_per_row = p.k >> 2;
    if (dword >= static_cast<size_t>(p.n) * dwords_per_row) return;
    const uint32_t row = static_cast<uint32_t>(dword / dwords_per_row);
    const uint32_t k0 = static_cast<uint32_t>(dword % dwords_per_row) * 4u;
    const uint32_t packed = reinterpret_cast<const uint32_t *>(p.weight)[dword];
    const size_t si = static_cast<size_t>(row / p.block_m) * p.scale_cols + k0 / p.block_k;
    float sc = 1.0f;
    float post = 1.0f;
    if constexpr (SCALE == kE8m0) {
      sc = e8m0_to_f32(p.scales[si]);
    } else {
      post = reinterpret_cast<const float *>(p.scales)[si];
    }
    const bf16x2_t a0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(packed, sc, false);
    const bf16x2_t a1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(packed, sc, true);
    float v[4] = {static_cast<float>(a0[0]), static_cast<float>(a0[1]), static_cast<float>(a1[0]),
                  static_cast<float>(a1[1])};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      out[static_cast<size_t>(row) * p.k + k0 + e] = SCALE == kF32 ? v[e] * post : v[e];
    }
  }
}

inline bool aligned16(uint64_t p) { return p != 0 && (p & 15u) == 0; }

// Shapes the MFMA kernel takes; everything else valid goes to the generic kernel.
bool skinny_ok(const FerruleHipQuantGemvArgs &a) {
  if (a.weight_format == kFp4) return a.k % 32u == 0u && a.block_k == 32u;
  if (a.k % 16u != 0u) return false;
  if (a.block_k % 128u != 0u) return false;
  return a.scale_kind == kE8m0 || a.block_m % 16u == 0u;
}

int32_t validate(const FerruleHipQuantGemvArgs *a, bool need_x) {
  if (a == nullptr) return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->weight_format != kFp4 && a->weight_format != kFp8) return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->scale_kind != kE8m0 && a->scale_kind != kF32) return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->n == 0 || a->k == 0 || a->block_m == 0 || a->block_k == 0) return FERRULE_HIP_INVALID_ARGUMENT;
  if (need_x && a->batch == 0) return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->scale_cols != (a->k + a->block_k - 1) / a->block_k) return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->weight_format == kFp4) {
    // the MX contract: one E8M0 scale per 32 contiguous K elements of one row
    if (a->scale_kind != kE8m0 || a->block_m != 1 || a->k % 2u != 0 || a->k % a->block_k != 0)
      return FERRULE_HIP_INVALID_ARGUMENT;
    if (a->block_k % 8u != 0) return FERRULE_HIP_UNSUPPORTED;
  }
  if (!aligned16(a->weight) || !aligned16(a->weight_scales) || !aligned16(a->output))
    return FERRULE_HIP_INVALID_ARGUMENT;
  if (need_x && !aligned16(a->x)) return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->flags & FERRULE_HIP_GEMV_BLOCK_MAJOR_WEIGHTS) {
    // only the decode GEMV reads the prepared order, and only whole tiles of it
    if (!need_x) return FERRULE_HIP_INVALID_ARGUMENT;
    if (a->weight_format == kFp4 && a->block_k != 32u) return FERRULE_HIP_INVALID_ARGUMENT;
    if (a->n % 16u != 0 || a->k % 128u != 0 || !skinny_ok(*a)) return FERRULE_HIP_UNSUPPORTED;
  }
  return FERRULE_HIP_SUCCESS;
}

GemvParams make_params(const FerruleHipQuantGemvArgs &a) {
  GemvParams p;
  p.weight = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(a.weight));
  p.scales = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(a.weight_scales));
  p.x = reinterpret_cast<const uint16_t *>(static_cast<uintptr_t>(a.x));
  p.output = reinterpret_cast<void *>(static_cast<uintptr_t>(a.output));
  p.batch = a.batch;
  p.n = a.n;
  p.k = a.k;
  p.scale_cols = a.scale_cols;
  p.block_m = a.block_m;
  p.block_k = a.block_k;
  p.flags = a.flags;
  return p;
}

template <int FMT, int SCALE, bool BLOCK_MAJOR = false>
void launch_skinny(const GemvParams &p, hipStream_t stream) {
  const uint32_t tiles = (p.n + 15u) / 16u;
  const uint32_t kblocks = (p.k + 127u) / 128u;
  // few row tiles: split K wider so every CU still has many loads in flight
  if (tiles <= 1024u && kblocks >= 16u) {
    skinny_gemv_kernel<FMT, SCALE, 16, 4, 2, BLOCK_MAJOR><<<tiles, 1024, 0, stream>>>(p);
  } else if (tiles <= 4096u && kblocks >= 8u) {
    skinny_gemv_kernel<FMT, SCALE, 8, 4, 2, BLOCK_MAJOR><<<tiles, 512, 0, stream>>>(p);
  } else {
    skinny_gemv_kernel<FMT, SCALE, 4, 4, 2, BLOCK_MAJOR><<<tiles, 256, 0, stream>>>(p);
  }
}

}  // namespace
}  // namespace ferrule_hip

using namespace ferrule_hip;

extern "C" int32_t ferrule_hip_quant_gemv_can_implement(const FerruleHipQuantGemvArgs *args) {
  return validate(args, true);
}

extern "C" int32_t ferrule_hip_quant_gemv_launch(const FerruleHipQuantGemvArgs *args) {
  const int32_t status = validate(args, true);
  if (status != FERRULE_HIP_SUCCESS) return status;
  const GemvParams p = make_params(*args);
  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(args->stream));
  clear_launch_error();
  if (skinny_ok(*args)) {
    if (args->weight_format == kFp4 && (args->flags & FERRULE_HIP_GEMV_BLOCK_MAJOR_WEIGHTS)) {
      launch_skinny<kFp4, kE8m0, true>(p, stream);
    } else if (args->weight_format == kFp4) {
      launch_skinny<kFp4, kE8m0>(p, stream);
    } else if (args->flags & FERRULE_HIP_GEMV_BLOCK_MAJOR_WEIGHTS) {
      if (args->scale_kind == kE8m0) {
        launch_skinny<kFp8, kE8m0, true>(p, stream);
      } else {
        launch_skinny<kFp8, kF32, true>(p, stream);
      }
    } else if (args->scale_kind == kE8m0) {
      launch_skinny<kFp8, kE8m0>(p, stream);
    } else {
      launch_skinny<kFp8, kF32>(p, stream);
    }
  } else {
    const uint32_t blocks = (p.n + 3u) / 4u;
    if (args->weight_format == kFp4) {
      generic_gemv_kernel<kFp4, kE8m0><<<blocks, 256, 0, stream>>>(p);
    } else if (args->scale_kind == kE8m0) {
      generic_gemv_kernel<kFp8, kE8m0><<<blocks, 256, 0, stream>>>(p);
    } else {
      generic_gemv_kernel<kFp8, kF32><<<blocks, 256, 0, stream>>>(p);
    }
  }
  return take_launch_error() == hipSuccess ? FERRULE_HIP_SUCCESS : FERRULE_HIP_LAUNCH_FAILED;
}

extern "C" int32_t ferrule_hip_dequant_launch(const FerruleHipQuantGemvArgs *args) {
  const int32_t status = validate(args, false);
  if (status != FERRULE_HIP_SUCCESS) return status;
  if (args->weight_format == kFp4 ? (args->k % 8u != 0) : (args->k % 4u != 0 || args->block_k % 4u != 0))
    return FERRULE_HIP_UNSUPPORTED;
  const GemvParams p = make_params(*args);
  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(args->stream));
  clear_launch_error();
  const size_t dwords = static_cast<size_t>(p.n) * (args->weight_format == kFp4 ? p.k / 8u : p.k / 4u);
  const uint32_t blocks = static_cast<uint32_t>((dwords + 255u) / 256u);
  if (args->weight_format == kFp4) {
    dequant_kernel<kFp4, kE8m0><<<blocks, 256, 0, stream>>>(p);
  } else if (args->scale_kind == kE8m0) {
    dequant_kernel<kFp8, kE8m0><<<blocks, 256, 0, stream>>>(p);
  } else {
    dequant_kernel<kFp8, kF32><<<blocks, 256, 0, stream>>>(p);
  }
  return take_launch_error() == hipSuccess ? FERRULE_HIP_SUCCESS : FERRULE_HIP_LAUNCH_FAILED;
}
