// Building blocks shared by the decode GEMV and the decode MoE kernels: the gfx950 scaled
// converters (packed FP4 / FP8 -> BF16 with the block scale applied, exact) and typed global
// loads.
//
// Operand layout of v_mfma_f32_16x16x32_bf16 as these kernels use it:
//   lane l = (r = l%16, g = l/16)
//   A operand (weights): row r of a 16-row tile, 8 consecutive k per MFMA
//   B operand (activations): activation row r ("token" column), the same 8 k
//   accumulator: acc[v] of lane l = (weight row 4*g + v, token r)
// Each lane owns 16 bytes of packed weights per 128-wide K block (32 FP4 = one E8M0 scale
// block, or 16 FP8).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ferrule_hip_provider.h"
#include "numeric.cuh"

namespace ferrule_hip {

constexpr int kFp8 = FERRULE_HIP_WEIGHT_FP8_E4M3;
constexpr int kFp4 = FERRULE_HIP_WEIGHT_MXFP4_E2M1;
constexpr int kE8m0 = FERRULE_HIP_SCALE_E8M0;
constexpr int kF32 = FERRULE_HIP_SCALE_F32;

__device__ __forceinline__ bf16x8_t expand_fp4_dword(uint32_t packed, float scale) {
  const bf16x2_t a0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(packed, scale, 0);
  const bf16x2_t a1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(packed, scale, 1);
  const bf16x2_t a2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(packed, scale, 2);
  const bf16x2_t a3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(packed, scale, 3);
  bf16x8_t out;
  out[0] = a0[0]; out[1] = a0[1]; out[2] = a1[0]; out[3] = a1[1];
  out[4] = a2[0]; out[5] = a2[1]; out[6] = a3[0]; out[7] = a3[1];
  return out;
}

__device__ __forceinline__ bf16x8_t expand_fp8_dwords(uint32_t lo, uint32_t hi, float scale) {
  const bf16x2_t a0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, scale, false);
  const bf16x2_t a1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, scale, true);
  const bf16x2_t a2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, scale, false);
  const bf16x2_t a3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, scale, true);
  bf16x8_t out;
  out[0] = a0[0]; out[1] = a0[1]; out[2] = a1[0]; out[3] = a1[1];
  out[4] = a2[0]; out[5] = a2[1]; out[6] = a3[0]; out[7] = a3[1];
  return out;
}

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ bf16x8_t as_bf16x8(const u32x4_t &v) {
  union {
    u32x4_t u;
    bf16x8_t b;
  } c;
  c.u = v;
  return c.b;
}

// Pointers that arrive as integers (slot tables) have no address space the compiler can see,
// and it would emit flat loads, which also count against the LDS counter; these helpers say
// "global" explicitly.
typedef const __attribute__((address_space(1))) u32x4_t *global_u32x4_ptr;
typedef const __attribute__((address_space(1))) uint32_t *global_u32_ptr;
typedef const __attribute__((address_space(1))) uint8_t *global_u8_ptr;

// Weights are read exactly once: keep them out of the way of the activations in cache.
__device__ __forceinline__ u32x4_t load_stream16(const void *p) {
  return __builtin_nontemporal_load((global_u32x4_ptr)(p));
}
__device__ __forceinline__ u32x4_t load16(const void *p) { return *(global_u32x4_ptr)(p); }
__device__ __forceinline__ uint32_t load4(const void *p) { return *(global_u32_ptr)(p); }
__device__ __forceinline__ uint32_t load1(const void *p) { return *(global_u8_ptr)(p); }

}  // namespace ferrule_hip
