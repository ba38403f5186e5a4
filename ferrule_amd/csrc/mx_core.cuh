// MX building blocks for the scaled-MFMA kernels (gfx950 v_mfma_scale_f32_16x16x128_f8f6f4).
//
// Why this exists: expanding MXFP4 to BF16 on the VALU costs ~11 cycles per converter
// instruction (2 values), i.e. about 350 VALU cycles per KB of weights and SIMD - measured,
// it caps a streaming kernel near half of HBM bandwidth.  The scaled MFMA consumes the
// packed E2M1 nibbles and their E8M0 block scales directly (32 cycles per 16x128 tile), so
// the weights never touch the VALU.  Its other operand must be an 8/6/4-bit float, so BF16
// (or f32) activations are first split into a short sum of MX-FP8 terms:
//     x ~ sum_t  q_t * 2^(s_t - 127),   q_t in E4M3, one E8M0 scale s_t per 32 elements.
// Each term takes the leading 4 significant bits of what is left, by truncation, so the
// remainder after every term is known exactly and each term's scale is at most 1/16 of the
// one before.  The split is a truncation, not an identity, and the callers choose the
// number of terms for the error they can afford:
//   2 terms of a BF16 value: exact for every element that is normal in its first term
//     (at least 2^-13 of its 32-block maximum); a smaller element loses less than 2^-20 of
//     that maximum;
//   4 terms of an f32 value: every element is held to better than 2^-15 of its 32-block
//     maximum (16 significant bits of the largest element).
// sum_k w*x is then the sum over terms of MFMA results, all accumulated in fp32; the
// truncation enters the result as sum_k |w_k| * (what was cut from x_k).
//
// Operand layout of the 16x16x128 instruction, lane l = (i = l%16, g = l/16), measured on
// the device with one-hot operands:
//   4-bit operand (4 VGPRs): row/column i, k in [32g, 32g+32), low nibble first - a lane's
//      16-byte load of an MXFP4 row IS its operand;
//   8-bit operand (8 VGPRs): row/column i, VGPRs 0-3 hold k in [16g, 16g+16) and VGPRs 4-7
//      hold k in [64+16g, 64+16g+16) (two 64-wide halves, 16 consecutive k per lane each);
//   scale: the byte supplied by lane (i, g) applies to k in [32g, 32g+32) of row/column i
//      for either operand width - for MXFP4 that is exactly the block the lane holds;
//   D: acc[v] of lane l = (row 4g+v, column i).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "numeric.cuh"
#include "skinny_core.cuh"

namespace ferrule_hip {

typedef __attribute__((address_space(3))) void lds_void_t;

// s_waitcnt vmcnt(n) for a run-time n (the instruction takes an immediate).
__device__ __forceinline__ void wait_vmcnt(uint32_t n) {
#define FERRULE_VMCNT_CASE(N) \
  case N: __builtin_amdgcn_s_waitcnt(0x0f70 | ((N) & 0xf) | (((N) >> 4) << 14)); break;
  switch (n) {
    FERRULE_VMCNT_CASE(0) FERRULE_VMCNT_CASE(1) FERRULE_VMCNT_CASE(2) FERRULE_VMCNT_CASE(3)
    FERRULE_VMCNT_CASE(4) FERRULE_VMCNT_CASE(5) FERRULE_VMCNT_CASE(6) FERRULE_VMCNT_CASE(7)
    FERRULE_VMCNT_CASE(8) FERRULE_VMCNT_CASE(9) FERRULE_VMCNT_CASE(10) FERRULE_VMCNT_CASE(11)
    FERRULE_VMCNT_CASE(12) FERRULE_VMCNT_CASE(13) FERRULE_VMCNT_CASE(14) FERRULE_VMCNT_CASE(15)
    FERRULE_VMCNT_CASE(16) FERRULE_VMCNT_CASE(17) FERRULE_VMCNT_CASE(18) FERRULE_VMCNT_CASE(19)
    FERRULE_VMCNT_CASE(20) FERRULE_VMCNT_CASE(21) FERRULE_VMCNT_CASE(22) FERRULE_VMCNT_CASE(23)
    FERRULE_VMCNT_CASE(24) FERRULE_VMCNT_CASE(25) FERRULE_VMCNT_CASE(26) FERRULE_VMCNT_CASE(27)
    FERRULE_VMCNT_CASE(28) FERRULE_VMCNT_CASE(29) FERRULE_VMCNT_CASE(30) FERRULE_VMCNT_CASE(31)
    FERRULE_VMCNT_CASE(32) FERRULE_VMCNT_CASE(33) FERRULE_VMCNT_CASE(34) FERRULE_VMCNT_CASE(35)
    FERRULE_VMCNT_CASE(36) FERRULE_VMCNT_CASE(37) FERRULE_VMCNT_CASE(38) FERRULE_VMCNT_CASE(39)
    FERRULE_VMCNT_CASE(40) FERRULE_VMCNT_CASE(41) FERRULE_VMCNT_CASE(42) FERRULE_VMCNT_CASE(43)
    FERRULE_VMCNT_CASE(44) FERRULE_VMCNT_CASE(45) FERRULE_VMCNT_CASE(46) FERRULE_VMCNT_CASE(47)
    FERRULE_VMCNT_CASE(48) FERRULE_VMCNT_CASE(49) FERRULE_VMCNT_CASE(50) FERRULE_VMCNT_CASE(51)
    FERRULE_VMCNT_CASE(52) FERRULE_VMCNT_CASE(53) FERRULE_VMCNT_CASE(54) FERRULE_VMCNT_CASE(55)
    FERRULE_VMCNT_CASE(56) FERRULE_VMCNT_CASE(57) FERRULE_VMCNT_CASE(58) FERRULE_VMCNT_CASE(59)
    FERRULE_VMCNT_CASE(60) FERRULE_VMCNT_CASE(61) FERRULE_VMCNT_CASE(62)
  default: __builtin_amdgcn_s_waitcnt(0x0f70); break;
  }
#undef FERRULE_VMCNT_CASE
}

// Direct global->LDS load of 16 (or 4) bytes per lane: lane l's bytes land at lds_base + l*size.
// Issued as inline assembly on purpose.  The compiler's wait-count bookkeeping files the
// builtin form under the LDS counter as well, as an event that may complete out of order, and
// from then on every wait for an ordinary ds_read becomes lgkmcnt(0) - the fragment reads of a
// K step can no longer be pipelined against the MFMAs.  The loads are tracked by hand instead:
// they return in order on vmcnt, and every consumer waits with wait_vmcnt() before the barrier
// that publishes a stage.  (A compiler-inserted vmcnt wait can only become stricter by the
// extra outstanding loads, never weaker.)  lds_base must be wave-uniform.
__device__ __forceinline__ void lds_dma16(const void *src, void *lds_base) {
  const uint32_t base = __builtin_amdgcn_readfirstlane(
      static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_void_t *)(lds_base))));
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void lds_dma4(const void *src, void *lds_base) {
  const uint32_t base = __builtin_amdgcn_readfirstlane(
      static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_void_t *)(lds_base))));
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dword %0, off" : : "v"(src), "s"(base) : "memory", "m0");
}
// The same with the address split into a wave-uniform base (scalar registers) and a 32-bit
// offset per lane.
// A pointer the compiler may hold in vector registers, moved to scalar ones (no-ops when it is
// there already): what the "s" operand of the loads below takes.
__device__ __forceinline__ const void *uniform_pointer(const void *p) {
  const uint64_t bits = reinterpret_cast<uintptr_t>(p);
  const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(bits));
  const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(bits >> 32));
  return reinterpret_cast<const void *>(static_cast<uintptr_t>((static_cast<uint64_t>(hi) << 32) | lo));
}
__device__ __forceinline__ void lds_dma16(const void *uniform_base, uint32_t lane_offset, void *lds_base) {
  const uint32_t base = __builtin_amdgcn_readfirstlane(
      static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_void_t *)(lds_base))));
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1"
               : : "v"(lane_offset), "s"(uniform_pointer(uniform_base)), "s"(base) : "memory", "m0");
}
// the same for data that is read once (weights of a streaming kernel): nontemporal, it does not push
// what other waves share out of L2
__device__ __forceinline__ void lds_dma16_stream(const void *uniform_base, uint32_t lane_offset, void *lds_base) {
  const uint32_t base = __builtin_amdgcn_readfirstlane(
      static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_void_t *)(lds_base))));
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1 nt"
               : : "v"(lane_offset), "s"(uniform_pointer(uniform_base)), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void lds_dma4(const void *uniform_base, uint32_t lane_offset, void *lds_base) {
  const uint32_t base = __builtin_amdgcn_readfirstlane(
      static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_void_t *)(lds_base))));
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %0, %1"
               : : "v"(lane_offset), "s"(uniform_pointer(uniform_base)), "s"(base) : "memory", "m0");
}

constexpr int kMfmaFmtFp8 = 0;  // e4m3
constexpr int kMfmaFmtFp4 = 4;  // e2m1

__device__ __forceinline__ i32x8_t make_a_fp4(const u32x4_t &w) {
  i32x8_t a = {static_cast<int>(w[0]), static_cast<int>(w[1]), static_cast<int>(w[2]), static_cast<int>(w[3]),
               0, 0, 0, 0};
  return a;
}

// lo = the 16 bytes at k [16g, 16g+16), hi = the 16 bytes at k [64+16g, 64+16g+16)
__device__ __forceinline__ i32x8_t make_b_fp8(const u32x4_t &lo, const u32x4_t &hi) {
  i32x8_t b = {static_cast<int>(lo[0]), static_cast<int>(lo[1]), static_cast<int>(lo[2]), static_cast<int>(lo[3]),
               static_cast<int>(hi[0]), static_cast<int>(hi[1]), static_cast<int>(hi[2]), static_cast<int>(hi[3])};
  return b;
}

// acc += (fp4 A with scale byte sa) x (fp8 B with scale byte sb); scales in byte 0 of sa/sb
__device__ __forceinline__ f32x4_t mfma_fp4_fp8(const i32x8_t &a, const i32x8_t &b, const f32x4_t &acc,
                                                uint32_t sa, uint32_t sb) {
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, acc, kMfmaFmtFp4, kMfmaFmtFp8, 0,
                                                          static_cast<int>(sa), 0, static_cast<int>(sb));
}

// ---------------------------------------------------------------------------
// One term of the split of a 32-element block, for the N = 8 elements one of the block's
// four lanes holds: takes the leading 4 significant bits (relative to the block's own scale)
// out of r[] and leaves the exact remainder in r[].  packed[N/4] = the lane's E4M3 bytes,
// returns the block's E8M0 scale byte.  The block maximum is taken over the four lanes with two
// xor-shuffles (the lanes of a block are adjacent).
// ---------------------------------------------------------------------------
template <int N>
__device__ __forceinline__ uint32_t mx_split_term(float (&r)[N], uint32_t (&packed)[N / 4]) {
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < N; ++i) amax = fmaxf(amax, fabsf(r[i]));
  static_assert(N == 8, "four lanes of eight elements per 32-element block");
  amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
  amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
  const uint32_t eb = (__float_as_uint(amax) >> 23) & 0xffu;
  // scale 2^(eb-127-7): the block maximum lands in [128, 256) < 448
  int sbyte = static_cast<int>(eb) - 7;
  sbyte = sbyte < 1 ? 1 : sbyte > 253 ? 253 : sbyte;
  const float s = __uint_as_float(static_cast<uint32_t>(sbyte) << 23);
  const float inv_s = __uint_as_float(static_cast<uint32_t>(254 - sbyte) << 23);
#pragma unroll
  for (int v = 0; v < N / 4; ++v) packed[v] = 0u;
#pragma unroll
  for (int i = 0; i < N; ++i) {
    const float v = r[i] * inv_s;  // exact: power of two
    const float a = fabsf(v);
    const uint32_t sign = (__float_as_uint(v) >> 24) & 0x80u;
    uint32_t code;
    float kept;
    if (!(a < 512.0f)) {  // inf / NaN input
      code = 0x7fu;
      kept = a;
    } else if (a >= 0.015625f) {
      const uint32_t bits = __float_as_uint(a);
      code = (bits >> 20) - (120u << 3);  // truncate to 3 mantissa bits
      kept = __uint_as_float(bits & 0xfff00000u);
    } else {
      const uint32_t m = static_cast<uint32_t>(a * 512.0f);  // subnormal grid, toward zero
      code = m;
      kept = static_cast<float>(m) * 0.001953125f;
    }
    packed[i >> 2] |= (sign | code) << (8 * (i & 3));
    r[i] = sign ? r[i] + kept * s : r[i] - kept * s;  // exact remainder
  }
  return amax == 0.0f ? 127u : static_cast<uint32_t>(sbyte);
}

// x [rows, k] (BF16 bits or f32) -> q [TERMS][plane_rows][k] bytes, s [TERMS][plane_rows][k/32]
// bytes; only the first `rows` rows of every term plane are written.
// Four adjacent lanes per 32-element block, eight elements each (one thread per block left most
// CUs idle at decode sizes: 64 tokens x 7168 are 14 336 blocks).  The grid covers whole blocks, so
// the four lanes of a block are always all active.
template <typename IN, int TERMS>
__global__ __launch_bounds__(256) void mx_split_kernel(const IN *__restrict__ x, uint8_t *__restrict__ q,
                                                       uint8_t *__restrict__ s, uint32_t rows, uint32_t plane_rows,
                                                       uint32_t k) {
  const uint32_t blocks_per_row = k >> 5;
  const uint64_t piece = static_cast<uint64_t>(blockIdx.x) * 256u + threadIdx.x;  // 8 elements
  const uint64_t block = piece >> 2;
  const bool live = block < static_cast<uint64_t>(rows) * blocks_per_row;
  // lanes past the end still take part in the shuffles of their own (dead) block
  const uint64_t at = live ? piece * 8u : 0u;
  float r[8];
  if constexpr (sizeof(IN) == 2) {
    const u32x4_t d = *reinterpret_cast<const u32x4_t *>(x + at);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      r[2 * e] = __uint_as_float(d[e] << 16);
      r[2 * e + 1] = __uint_as_float(d[e] & 0xffff0000u);
    }
  } else {
    const float4 *src = reinterpret_cast<const float4 *>(x + at);
    const float4 d0 = src[0], d1 = src[1];
    r[0] = d0.x; r[1] = d0.y; r[2] = d0.z; r[3] = d0.w;
    r[4] = d1.x; r[5] = d1.y; r[6] = d1.z; r[7] = d1.w;
  }
  const uint64_t plane_q = static_cast<uint64_t>(plane_rows) * k;
  const uint64_t plane_s = static_cast<uint64_t>(plane_rows) * blocks_per_row;
#pragma unroll
  for (int t = 0; t < TERMS; ++t) {
    uint32_t packed[2];
    const uint32_t scale = mx_split_term(r, packed);
    if (live) {
      *reinterpret_cast<uint2 *>(q + t * plane_q + at) = make_uint2(packed[0], packed[1]);
      if ((piece & 3u) == 0u) s[t * plane_s + block] = static_cast<uint8_t>(scale);
    }
  }
}

}  // namespace ferrule_hip
