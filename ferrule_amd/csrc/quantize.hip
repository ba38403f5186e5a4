// Activation packers: f32 rows -> E4M3 bytes + E8M0 scale per block (kind 5) and
// f32 rows -> packed E2M1 nibbles + E8M0 scale per block (kind 4).
//
// Drop-in for ferrule_core_quantize_launch (abi/core_provider.h:481; kernel
// portable/entrypoints.cu:342-448).  Arithmetic follows the CPU reference
// (crates/ferrule-model/src/checkpoint/encoding.rs:207-284, 335-406) through the
// closed forms in quant_math.h; `reserved` = FERRULE_HIP_FP8_ROUND_HALF_EVEN selects
// the portable GPU kernel's rintf variant instead.
//
// The kernel is memory bound (4 B in, 1 or 0.5 B out per element): each thread
// loads one float4, the block maximum is reduced with wave shuffles inside the
// group of block_size/4 threads, and one dword / one 16-bit word is stored.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ferrule_hip_diagnostics.h"
#include "../../include/ferrule_hip_provider.h"
#include "numeric.cuh"
#include "quant_math.h"

namespace ferrule_hip {
namespace {

using namespace ferrule_quant;

// GROUP = threads per quantization block = block_size / 4 (power of two, <= 64)
template <int KIND, int GROUP>
__global__ __launch_bounds__(256) void quantize_vec_kernel(FerruleHipQuantizeArgs args) {
  const uint64_t thread = static_cast<uint64_t>(blockIdx.x) * 256u + threadIdx.x;
  const uint64_t quads = args.value_len / 4u;
  const bool active = thread < quads;
  const float *values = global_ptr<const float>(args.values) +
                        args.value_offset;
  float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
  if (active) v = reinterpret_cast<const float4 *>(values)[thread];
  float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
#pragma unroll
  for (int offset = GROUP / 2; offset > 0; offset >>= 1) {
    amax = fmaxf(amax, __shfl_xor(amax, offset, 64));
  }
  const bool cpu_rule = args.reserved != FERRULE_HIP_FP8_ROUND_HALF_EVEN;
  uint32_t byte;
  if constexpr (KIND == FERRULE_HIP_QUANTIZE_FP8_PACKED) {
    amax = fmaxf(amax, 1e-4f);
    byte = scale_byte(amax, 448.0f);
  } else {
    if (cpu_rule) {
      amax = fmaxf(amax, 6.0f * 0x1p-126f);
      byte = scale_byte(amax, 6.0f);
    } else {
      // portable/entrypoints.cu:113-121: 127 for an all-zero or non-finite block
      byte = (amax > 0.0f && amax <= 3.4028234e38f) ? scale_byte(amax, 6.0f) : 127u;
    }
  }
  if (!active) return;
  const float scale = e8m0_value(byte);
  if ((thread % GROUP) == 0u) {
    global_ptr<uint8_t>(args.scales)[thread / GROUP] =
        static_cast<uint8_t>(byte);
  }
  if constexpr (KIND == FERRULE_HIP_QUANTIZE_FP8_PACKED) {
    const uint32_t mode = args.reserved;
    uint32_t packed;
    if (byte >= 1u && byte <= 253u) {  // the scale has an exact f32 inverse: hardware converter, exact at ties
      packed = e4m3_bytes_exact(v.x, v.y, v.z, v.w, e8m0_inverse(byte), mode);
    } else {  // non-finite block maximum
      packed = fp8_e4m3_quantize_byte(v.x, scale, mode) | (fp8_e4m3_quantize_byte(v.y, scale, mode) << 8) |
               (fp8_e4m3_quantize_byte(v.z, scale, mode) << 16) | (fp8_e4m3_quantize_byte(v.w, scale, mode) << 24);
    }
    global_ptr<uint32_t>(args.packed)[thread] = packed;
  } else {
    const uint32_t packed = fp4_e2m1_quantize_nibble(v.x, scale, cpu_rule) |
                            (fp4_e2m1_quantize_nibble(v.y, scale, cpu_rule) << 4) |
                            (fp4_e2m1_quantize_nibble(v.z, scale, cpu_rule) << 8) |
                            (fp4_e2m1_quantize_nibble(v.w, scale, cpu_rule) << 12);
    global_ptr<uint16_t>(args.packed)[thread] =
        static_cast<uint16_t>(packed);
  }
}

// FP8, blocks of 128: sixteen values per thread as four 16-byte pieces, each piece one of 64 consecutive
// ones of the wave (a wave instruction fetches 1 KB in one stretch), so a block is half a wave of one
// piece.  Four loads in flight per thread: the four-values-per-thread form above keeps one load in
// flight per thread and reaches 2.3 TB/s on a 4096 x 7168 f32 matrix, this one is bound by HBM.
__global__ __launch_bounds__(256) void quantize_fp8_k128_wide_kernel(FerruleHipQuantizeArgs args) {
  typedef float f32x4v __attribute__((ext_vector_type(4)));
  const uint32_t lane = threadIdx.x & 63u;
  const uint64_t wave = static_cast<uint64_t>(blockIdx.x) * 4u + (threadIdx.x >> 6);
  const uint64_t pieces = args.value_len / 4u;   // a multiple of 32: whole blocks
  const f32x4v *src = reinterpret_cast<const f32x4v *>(
      global_ptr<const float>(args.values) + args.value_offset);
  uint64_t piece[4];
  bool active[4];
  f32x4v v[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    piece[j] = wave * 256u + static_cast<uint32_t>(j) * 64u + lane;
    active[j] = piece[j] < pieces;   // uniform over the 32 lanes of a block
    v[j] = __builtin_nontemporal_load(src + (active[j] ? piece[j] : 0u));
  }
  const uint32_t mode = args.reserved;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float amax = fmaxf(fmaxf(fabsf(v[j][0]), fabsf(v[j][1])), fmaxf(fabsf(v[j][2]), fabsf(v[j][3])));
#pragma unroll
    for (int offset = 16; offset > 0; offset >>= 1) amax = fmaxf(amax, __shfl_xor(amax, offset, 64));
    const uint32_t byte = scale_byte(fmaxf(amax, 1e-4f), 448.0f);
    if (!active[j]) continue;
    if ((lane & 31u) == 0u) {
      global_ptr<uint8_t>(args.scales)[piece[j] >> 5] = static_cast<uint8_t>(byte);
    }
    uint32_t packed;
    if (byte >= 1u && byte <= 253u) {  // the scale has an exact f32 inverse: hardware converter, exact at ties
      packed = e4m3_bytes_exact(v[j][0], v[j][1], v[j][2], v[j][3], e8m0_inverse(byte), mode);
    } else {  // non-finite block maximum
      const float scale = e8m0_value(byte);
      packed = fp8_e4m3_quantize_byte(v[j][0], scale, mode) | (fp8_e4m3_quantize_byte(v[j][1], scale, mode) << 8) |
               (fp8_e4m3_quantize_byte(v[j][2], scale, mode) << 16) | (fp8_e4m3_quantize_byte(v[j][3], scale, mode) << 24);
    }
    global_ptr<uint32_t>(args.packed)[piece[j]] = packed;
  }
}

// Any block size: one thread per quantization block, as the reference kernel.
template <int KIND>
__global__ __launch_bounds__(256) void quantize_scalar_kernel(FerruleHipQuantizeArgs args) {
  const uint64_t block_index = static_cast<uint64_t>(blockIdx.x) * 256u + threadIdx.x;
  if (block_index >= args.value_len / args.block_size) return;
  const float *input = global_ptr<const float>(args.values) +
                       args.value_offset;
  const uint64_t begin = block_index * args.block_size;
  const bool cpu_rule = args.reserved != FERRULE_HIP_FP8_ROUND_HALF_EVEN;
  float amax = 0.0f;
  for (uint32_t i = 0; i < args.block_size; ++i) amax = fmaxf(amax, fabsf(input[begin + i]));
  uint32_t byte;
  if constexpr (KIND == FERRULE_HIP_QUANTIZE_FP8_PACKED) {
    byte = scale_byte(fmaxf(amax, 1e-4f), 448.0f);
  } else if (cpu_rule) {
    byte = scale_byte(fmaxf(amax, 6.0f * 0x1p-126f), 6.0f);
  } else {
    byte = (amax > 0.0f && amax <= 3.4028234e38f) ? scale_byte(amax, 6.0f) : 127u;
  }
  const float scale = e8m0_value(byte);
  global_ptr<uint8_t>(args.scales)[block_index] =
      static_cast<uint8_t>(byte);
  if constexpr (KIND == FERRULE_HIP_QUANTIZE_FP8_PACKED) {
    uint8_t *packed = global_ptr<uint8_t>(args.packed);
    for (uint32_t i = 0; i < args.block_size; ++i) {
      packed[begin + i] = static_cast<uint8_t>(fp8_e4m3_quantize_byte(input[begin + i], scale, args.reserved));
    }
  } else {
    uint8_t *packed = global_ptr<uint8_t>(args.packed);
    for (uint32_t i = 0; i < args.block_size; i += 2) {
      const uint32_t lo = fp4_e2m1_quantize_nibble(input[begin + i], scale, cpu_rule);
      const uint32_t hi = fp4_e2m1_quantize_nibble(input[begin + i + 1], scale, cpu_rule);
      packed[(begin + i) / 2] = static_cast<uint8_t>(lo | (hi << 4));
    }
  }
}

template <int KIND>
void launch_quantize(const FerruleHipQuantizeArgs &a, hipStream_t stream) {
  const bool vec = (a.value_offset % 4u == 0u) && (a.values % 16u == 0u) && (a.packed % 4u == 0u);
  const uint64_t quads = a.value_len / 4u;
  const uint32_t grid = static_cast<uint32_t>((quads + 255u) / 256u);
  // the wide form needs a matrix that fills the machine with sixteen values per thread (a 512 x 7168 one
  // takes 10 us in it against 8 us four values per thread)
  if (KIND == FERRULE_HIP_QUANTIZE_FP8_PACKED && vec && a.block_size == 128u && a.packed % 16u == 0u &&
      a.value_len >= (8u << 20)) {
    const uint64_t groups = a.value_len / 16u;
    quantize_fp8_k128_wide_kernel<<<static_cast<uint32_t>((groups + 255u) / 256u), 256, 0, stream>>>(a);
  } else if (vec && a.block_size == 32u) {
    quantize_vec_kernel<KIND, 8><<<grid, 256, 0, stream>>>(a);
  } else if (vec && a.block_size == 64u) {
    quantize_vec_kernel<KIND, 16><<<grid, 256, 0, stream>>>(a);
  } else if (vec && a.block_size == 128u) {
    quantize_vec_kernel<KIND, 32><<<grid, 256, 0, stream>>>(a);
  } else if (vec && a.block_size == 256u) {
    quantize_vec_kernel<KIND, 64><<<grid, 256, 0, stream>>>(a);
  } else {
    const uint64_t blocks = a.value_len / a.block_size;
    quantize_scalar_kernel<KIND><<<static_cast<uint32_t>((blocks + 255u) / 256u), 256, 0, stream>>>(a);
  }
}

// Every f32 pattern, both rounding rules: e4m3_bytes_exact against the software encoder (any
// pattern), and the converter alone against it on the finite ones.  counts[0] = differences of the
// former plus differences of the latter on patterns with any of the low 19 bits set (must be 0),
// counts[1] = one such pattern + 1, counts[2] = differences of the converter alone on patterns with
// those bits clear (the ties that go to the exact routine).
__global__ __launch_bounds__(256) void fp8_converter_selftest_kernel(unsigned long long *counts) {
  const uint32_t lane_pattern = blockIdx.x * 256u + threadIdx.x;   // the grid covers 2^24 threads
  unsigned long long wrong = 0, ties = 0, example = 0;
  for (uint32_t high = 0; high < 256u; ++high) {
    const uint32_t pattern = (high << 24) | lane_pattern;
    const float q = __uint_as_float(pattern);
    for (uint32_t mode = 0; mode < 2u; ++mode) {   // FERRULE_HIP_FP8_ROUND_CPU_REFERENCE, _HALF_EVEN
      const uint32_t exact = ferrule_quant::fp8_e4m3_quantize_byte_pow2(q, 1.0f, mode);
      // the complete routine (converter + fallback), any pattern, NaNs and infinities included
      if ((e4m3_bytes_exact(q, q, q, q, 1.0f, mode) & 0xffu) != exact) {
        ++wrong;
        example = static_cast<unsigned long long>(pattern) + 1ull;
      }
      if (!(fabsf(q) <= 3.4028234e38f)) continue;
      // the converter alone, finite patterns
      uint32_t low_bits = 0xffffffffu;
      const uint32_t fast = e4m3_bytes_rne(q, q, q, q, low_bits) & 0xffu;
      if (fast != exact) {
        if ((pattern & 0x7ffffu) != 0u) {
          ++wrong;
          example = static_cast<unsigned long long>(pattern) + 1ull;
        } else {
          ++ties;
        }
      }
    }
  }
  if (wrong != 0) {
    atomicAdd(&counts[0], wrong);
    atomicMax(&counts[1], example);
  }
  if (ties != 0) atomicAdd(&counts[2], ties);
}

}  // namespace
}  // namespace ferrule_hip

extern "C" int32_t ferrule_hip_fp8_converter_selftest_launch(uint64_t counts, uint64_t stream_bits) {
  using namespace ferrule_hip;
  if (counts == 0 || (counts & 7u) != 0) return FERRULE_HIP_INVALID_ARGUMENT;
  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(stream_bits));
  clear_launch_error();
  fp8_converter_selftest_kernel<<<1u << 16, 256, 0, stream>>>(
      reinterpret_cast<unsigned long long *>(static_cast<uintptr_t>(counts)));
  return take_launch_error() == hipSuccess ? FERRULE_HIP_SUCCESS : FERRULE_HIP_LAUNCH_FAILED;
}

extern "C" int32_t ferrule_hip_core_quantize_launch(const FerruleHipQuantizeArgs *args) {
  using namespace ferrule_hip;
  // reference: invalid => cudaErrorInvalidValue (1), portable/entrypoints.cu:1914-1916
  if (args == nullptr || args->block_size == 0 || args->row_width == 0) return 1;
  if (args->kind != FERRULE_HIP_QUANTIZE_FP8_PACKED && args->kind != FERRULE_HIP_QUANTIZE_FP4_PACKED) return 1;
  if (args->row_width % args->block_size != 0 || args->value_len % args->row_width != 0) return 1;
  if (args->kind == FERRULE_HIP_QUANTIZE_FP4_PACKED && args->block_size % 2u != 0) return 1;
  if (args->values == 0 || args->packed == 0 || args->scales == 0) return 1;
  if (args->value_len == 0) return 0;
  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(args->stream));
  clear_launch_error();
  if (args->kind == FERRULE_HIP_QUANTIZE_FP8_PACKED) {
    launch_quantize<FERRULE_HIP_QUANTIZE_FP8_PACKED>(*args, stream);
  } else {
    launch_quantize<FERRULE_HIP_QUANTIZE_FP4_PACKED>(*args, stream);
  }
  return static_cast<int32_t>(take_launch_error());
}
