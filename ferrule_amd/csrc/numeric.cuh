// Device-side numeric helpers shared by every kernel of the provider (gfx950 only).
//
// Formats (crates/ferrule-model/src/checkpoint/encoding.rs:14-75):
//   E2M1 nibble  s mmm  -> {0,.5,1,1.5,2,3,4,6}, low nibble of a byte = even k
//   E4M3FN byte  s eeee mmm, bias 7, 0x7f/0xff NaN, max 448
//   E8M0 byte    2^(b-127); b=0 -> 2^-127, b=255 -> +inf (not NaN, as the reference)
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "quant_math.h"

namespace ferrule_hip {

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef int i32x4_t __attribute__((ext_vector_type(4)));
typedef int i32x8_t __attribute__((ext_vector_type(8)));

// A device address that arrives as an integer (the argument blocks of the C ABI), as a pointer the
// compiler knows to be global memory.  A plain integer-to-pointer cast gives a generic pointer:
// loads and stores through it become FLAT instructions, which count on the LDS counter as well,
// so every wait around them is for memory and LDS together.
template <typename T>
__device__ __forceinline__ T *global_ptr(uint64_t address) {
  typedef __attribute__((address_space(1))) T global_t;
  return (T *)reinterpret_cast<global_t *>(static_cast<uintptr_t>(address));
}

// 2^(b-127) built from bits; identical to the reference's GPU twin
// (portable/entrypoints.cu:63-66) and to f32::powi on the CPU path.
__device__ __forceinline__ float e8m0_to_f32(uint32_t byte) {
  return __uint_as_float(byte == 0u ? (1u << 22) : (byte << 23));
}

// models/common/math.rs:7-14 / portable/entrypoints.cu:72-79
__device__ __forceinline__ uint16_t bf16_rne_bits(float value) {
  const uint32_t bits = __float_as_uint(value);
  if ((bits & 0x7fffffffu) > 0x7f800000u) {
    return static_cast<uint16_t>((bits >> 16) | 0x0040u);
  }
  const uint32_t rounding_bias = 0x7fffu + ((bits >> 16) & 1u);
  return static_cast<uint16_t>((bits + rounding_bias) >> 16);
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) {
  return __uint_as_float(bits16 << 16);
}

__device__ __forceinline__ float bf16_round(float value) {
  return bf16_bits_to_f32(bf16_rne_bits(value));
}

// Software decoders (used by generic-shape kernels and as the definition the
// hardware converters are tested against).
__device__ __forceinline__ float fp4_e2m1_decode(uint32_t nibble) {
  // magnitudes 0,.5,1,1.5,2,3,4,6 as f32: exponent/mantissa assembled from bits
  const uint32_t m = nibble & 7u;
  // value = m<2 ? m*0.5 : (1 + (m&1)*0.5) * 2^((m>>1)-1)
  const uint32_t bits = m == 0u   ? 0u
                        : m == 1u ? 0x3f000000u
                                  : (((m >> 1) + 126u) << 23) | ((m & 1u) << 22);
  return __uint_as_float(bits | ((nibble & 8u) << 28));
}

__device__ __forceinline__ float fp8_e4m3_decode(uint32_t byte) {
  const uint32_t sign = (byte & 0x80u) << 24;
  const uint32_t exponent = (byte >> 3) & 0x0fu;
  const uint32_t mantissa = byte & 7u;
  if (exponent == 0u) {
    // subnormal: mantissa * 2^-9 (exact in f32)
    return __uint_as_float(__float_as_uint(static_cast<float>(mantissa) * 0.001953125f) | sign);
  }
  if (exponent == 15u && mantissa == 7u) {
    return __uint_as_float(0x7fc00000u);
  }
  return __uint_as_float(sign | ((exponent + 120u) << 23) | (mantissa << 20));
}

// silu as the CPU path writes it: x / (1 + exp(-x))
// (crates/ferrule-model/src/moe/executor.rs:179-181)
__device__ __forceinline__ float silu_ref(float x) { return x / (1.0f + expf(-x)); }

// silu with the hardware's exp2 and reciprocal (a handful of instructions against some thirty-five
// for the library exp and an IEEE division).  A few ulp for moderate x; exp(-x) is formed from the
// rounded product x * log2(e), so the relative error grows with |x| (about (8 + |x|) * 2^-24, which is
// what the parity bounds of its users allow): bounded, not ulp-pinned.  For kernels that evaluate it for
// many values per lane: the gate/up GEMM epilogues, whose 64 values per lane were VALU bound with
// silu_ref and whose result goes to an E4M3 quantiser, and the dense decode FFN's down
// projection, where every workgroup forms the whole hidden row.  The decode MoE layer, one value
// per accumulator register, keeps silu_ref.
__device__ __forceinline__ float silu_fast(float x) {
  return x * __builtin_amdgcn_rcpf(1.0f + __expf(-x));
}

// Wave-wide sum over 64 lanes.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, 64);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) v = fmaxf(v, __shfl_xor(v, offset, 64));
  return v;
}

// Four finite values -> four E4M3 bytes (byte v = value v) by the hardware converter: clamped to
// +-448 like the CPU quantiser, round to nearest EVEN.  That is the CPU quantiser's byte
// (quant_math.h, FERRULE_HIP_FP8_ROUND_CPU_REFERENCE) for every value that does not sit exactly
// half way between two codes; a value that does has the low 19 bits of its f32 pattern clear,
// which `low_bits` tracks (the minimum over the values seen of pattern & 0x7ffff).  Checked over
// every f32 pattern by ferrule_hip_fp8_converter_selftest_launch.
__device__ __forceinline__ uint32_t e4m3_bytes_rne(float q0, float q1, float q2, float q3, uint32_t &low_bits) {
  q0 = __builtin_amdgcn_fmed3f(q0, -448.0f, 448.0f);
  q1 = __builtin_amdgcn_fmed3f(q1, -448.0f, 448.0f);
  q2 = __builtin_amdgcn_fmed3f(q2, -448.0f, 448.0f);
  q3 = __builtin_amdgcn_fmed3f(q3, -448.0f, 448.0f);
  low_bits = min(min(low_bits, __float_as_uint(q0) & 0x7ffffu), __float_as_uint(q1) & 0x7ffffu);
  low_bits = min(min(low_bits, __float_as_uint(q2) & 0x7ffffu), __float_as_uint(q3) & 0x7ffffu);
  int pair = __builtin_amdgcn_cvt_pk_fp8_f32(q0, q1, 0, false);
  pair = __builtin_amdgcn_cvt_pk_fp8_f32(q2, q3, pair, true);
  return static_cast<uint32_t>(pair);
}

// Four values times a power-of-two inverse scale -> four E4M3 bytes with the CPU quantiser's rule
// `mode` (FERRULE_HIP_FP8_ROUND_*), any inputs: the hardware converter's bytes, and the exact
// routine for this thread's four when one of them is a tie candidate or not finite (a NaN makes
// the sum NaN, an infinity makes it infinite or NaN).
__device__ __forceinline__ uint32_t e4m3_bytes_exact(float x0, float x1, float x2, float x3, float inv_scale,
                                                     uint32_t mode) {
  const float q0 = x0 * inv_scale, q1 = x1 * inv_scale, q2 = x2 * inv_scale, q3 = x3 * inv_scale;
  uint32_t low_bits = 0xffffffffu;
  uint32_t packed = e4m3_bytes_rne(q0, q1, q2, q3, low_bits);
  const float sum = (q0 + q1) + (q2 + q3);
  if (low_bits == 0u || !(fabsf(sum) <= 3.4028234e38f)) {
    packed = ferrule_quant::fp8_e4m3_quantize_byte_pow2(x0, inv_scale, mode) |
             (ferrule_quant::fp8_e4m3_quantize_byte_pow2(x1, inv_scale, mode) << 8) |
             (ferrule_quant::fp8_e4m3_quantize_byte_pow2(x2, inv_scale, mode) << 16) |
             (ferrule_quant::fp8_e4m3_quantize_byte_pow2(x3, inv_scale, mode) << 24);
  }
  return packed;
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also makes the compiler
// drain every outstanding global load it knows of (s_waitcnt vmcnt(0)), which would empty a
// weight prefetch ring at every barrier; here only LDS operations are fenced.  Neither barrier
// waits for loads issued from inline assembly (lds_dma4 / lds_dma16): the compiler does not count
// those, and whoever issues them waits with wait_vmcnt() before the barrier that publishes them.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Barrier for stages that are filled by direct global->LDS loads.  A release fence on LDS makes
// the compiler wait for EVERY outstanding direct-to-LDS load of the wave (they write LDS), i.e.
// s_waitcnt vmcnt(0) at each barrier, which serialises a multi-stage prefetch into one stage.
// Here the wave has already waited (in-order vmcnt) for exactly the loads that must have landed,
// its own LDS reads of the stage being released were consumed by MFMAs and are therefore
// complete, and LDS itself is coherent inside the CU, so the bare barrier is sufficient; the
// compiler does not move memory operations across it.
__device__ __forceinline__ void stage_barrier() {
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
}

// Launch status without inheriting a stale error: HIP keeps the last error of the
// calling thread until somebody reads it, and the caller's own runtime calls (a
// failed peer query, a not-ready event) may have left one behind.
//   clear_launch_error();  kernel<<<...>>>(...);  return take_launch_error();
// The raw hipError_t of the last failed launch of the calling thread is kept for
// ferrule_hip_last_error_code().
extern thread_local int32_t g_last_hip_error;
inline void clear_launch_error() { (void)hipGetLastError(); }
inline hipError_t take_launch_error() {
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) g_last_hip_error = static_cast<int32_t>(e);
  return e;
}

}  // namespace ferrule_hip
