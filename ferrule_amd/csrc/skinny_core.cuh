// The streaming inner loop shared by the decode GEMV and the decode MoE kernels.
//
// One wavefront multiplies a 16-row weight tile by up to 16 activation rows over
// the K blocks (128 wide) assigned to it, with v_mfma_f32_16x16x32_bf16:
//   lane l = (r = l%16, g = l/16)
//   A operand (weights): row r of the tile, 8 consecutive k per MFMA
//   B operand (activations): activation row r ("token" column), same 8 k
//   accumulator: acc[v] of lane l = (weight row 4*g + v, token r)
// Each lane owns 16 bytes of packed weights per K block (32 FP4 = one E8M0 scale
// block, or 16 FP8), expands them to BF16 with the gfx950 scaled converters (exact)
// and feeds four (FP4) or two (FP8) MFMAs.
//
// Memory-level parallelism is explicit: fragments for DEPTH K blocks are requested
// before the first one is consumed (a ring of register fragments, fully unrolled),
// because a decode GEMV is a single pass over its weights and the only way to reach
// HBM bandwidth is to have every wave's bytes in flight as early as possible.
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

// ---------------------------------------------------------------------------
// MXFP4: NMAT weight matrices share the activations; NX activation sets (e.g. the
// BF16 high and low halves of an f32 vector) share the weights.
//
// Two rings with different depths: weight fragments come from HBM and are requested
// DEPTH blocks ahead; activation fragments come from L2 and are requested one block
// ahead (they are 4x larger per lane, so a deep ring of them would spill).
// ---------------------------------------------------------------------------
template <int NMAT>
struct Fp4WFrag {
  u32x4_t w[NMAT];
  uint32_t sb[NMAT];
};

template <int NX>
struct XFrag {
  u32x4_t x[NX][4];
};

template <int NMAT, int NX>
struct Fp4Operands {
  // row-major: this lane's weight row start ([k/2] bytes) and scale row start ([k/32] bytes);
  // block-major (16-row tiles of [K block][row][64 B] and [K block][row][4 B], k % 128 == 0):
  // this lane's 16 bytes and its row's scale dword in K block 0 of the tile
  const uint8_t *wrow[NMAT];
  const uint8_t *srow[NMAT];
  const uint16_t *xrow[NX];    // this lane's activation row (BF16) or nullptr (zero column)
  uint32_t k;                  // multiple of 32
};

template <bool BLOCK_MAJOR, int NMAT, int NX>
__device__ __forceinline__ void fp4_load_w(Fp4WFrag<NMAT> &f, const Fp4Operands<NMAT, NX> &op,
                                           uint32_t kblock, uint32_t g) {
  if constexpr (BLOCK_MAJOR) {
    // one wave load = 1 KiB of consecutive bytes; the scale dword of the row holds the bytes of
    // the four 32-wide groups, lane group g takes its own
#pragma unroll
    for (int m = 0; m < NMAT; ++m) {
      f.w[m] = load_stream16(op.wrow[m] + kblock * 1024u);
      f.sb[m] = (load4(op.srow[m] + kblock * 64u) >> (8u * g)) & 0xffu;
    }
    return;
  }
  const uint32_t k0 = kblock * 128u + g * 32u;  // lane covers k0 .. k0+31
  const u32x4_t zero4 = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int m = 0; m < NMAT; ++m) {
    f.w[m] = zero4;
    f.sb[m] = 127u;
    if (k0 < op.k) {
      f.w[m] = load_stream16(op.wrow[m] + (k0 >> 1));
      f.sb[m] = load1(op.srow[m] + (k0 >> 5));
    }
  }
}

// x covers 32 consecutive k (FP4 lane span) as 4 x 16 bytes per activation set
template <int NMAT, int NX>
__device__ __forceinline__ void fp4_load_x(XFrag<NX> &f, const Fp4Operands<NMAT, NX> &op,
                                           uint32_t kblock, uint32_t g) {
  const uint32_t k0 = kblock * 128u + g * 32u;
  const u32x4_t zero4 = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int s = 0; s < NX; ++s) {
#pragma unroll
    for (int d = 0; d < 4; ++d) f.x[s][d] = zero4;
    if (k0 < op.k && op.xrow[s] != nullptr) {
#pragma unroll
      for (int d = 0; d < 4; ++d) f.x[s][d] = load16(op.xrow[s] + k0 + 8 * d);
    }
  }
}

template <int NMAT, int NX>
__device__ __forceinline__ void fp4_mac(const Fp4WFrag<NMAT> &wf, const XFrag<NX> &xf,
                                        f32x4_t (&acc)[NMAT]) {
#pragma unroll
  for (int m = 0; m < NMAT; ++m) {
    const float sc = e8m0_to_f32(wf.sb[m]);
    const uint32_t w[4] = {wf.w[m][0], wf.w[m][1], wf.w[m][2], wf.w[m][3]};
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const bf16x8_t a = expand_fp4_dword(w[d], sc);
#pragma unroll
      for (int s = 0; s < NX; ++s) {
        acc[m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, as_bf16x8(xf.x[s][d]), acc[m], 0, 0, 0);
      }
    }
  }
}

// K blocks first, first+stride, ... < kblocks; DEPTH weight fragments and XDEPTH
// activation fragments in flight (XDEPTH divides DEPTH; XDEPTH == DEPTH requests
// everything up front, which is what a one-shot launch wants).
template <bool BLOCK_MAJOR, int NMAT, int NX, int DEPTH, int XDEPTH>
__device__ __forceinline__ void fp4_stream(const Fp4Operands<NMAT, NX> &op, uint32_t first,
                                           uint32_t stride, uint32_t kblocks, uint32_t g,
                                           f32x4_t (&acc)[NMAT]) {
  static_assert(DEPTH % XDEPTH == 0, "ring slots are addressed with the unrolled index");
  Fp4WFrag<NMAT> wring[DEPTH];
  XFrag<NX> xring[XDEPTH];
#pragma unroll
  for (int d = 0; d < XDEPTH; ++d) {
    const uint32_t j = first + d * stride;
    if (j < kblocks) fp4_load_x(xring[d], op, j, g);
  }
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) {
    const uint32_t j = first + d * stride;
    if (j < kblocks) fp4_load_w<BLOCK_MAJOR>(wring[d], op, j, g);
  }
  for (uint32_t base = first; base < kblocks; base += DEPTH * stride) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const uint32_t j = base + d * stride;
      if (j < kblocks) {
        fp4_mac(wring[d], xring[d % XDEPTH], acc);
        const uint32_t next_x = j + XDEPTH * stride;
        if (next_x < kblocks) fp4_load_x(xring[d % XDEPTH], op, next_x, g);
        const uint32_t next_w = j + DEPTH * stride;
        if (next_w < kblocks) fp4_load_w<BLOCK_MAJOR>(wring[d], op, next_w, g);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// FP8 e4m3, one weight matrix, one activation set.
// ---------------------------------------------------------------------------
struct Fp8WFrag {
  u32x4_t w[2];
  float sc[1];  // scale of this lane's row (E8M0) or of the tile (F32) for this K block
};

struct Fp8Operands {
  // row-major: this lane's weight row start ([k] bytes); block-major (16-row tiles of
  // [64-byte K cell][row][64 B], k % 128 == 0): this lane's 16 bytes of cell 0 of the tile
  const uint8_t *wrow;
  const void *srow;      // scale row of this lane's row (E8M0 bytes) or of the tile (f32)
  const uint16_t *xrow;
  uint32_t k;            // multiple of 16
  uint32_t kb_per_scale; // block_k / 128: K blocks covered by one scale (block_k % 128 == 0)
};

template <int SCALE, bool BLOCK_MAJOR>
__device__ __forceinline__ void fp8_load_w(Fp8WFrag &f, const Fp8Operands &op, uint32_t kblock, uint32_t g) {
  const u32x4_t zero4 = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    if constexpr (BLOCK_MAJOR) {  // one wave load = the 1 KiB cell (kblock, u) of the tile
      f.w[u] = load_stream16(op.wrow + (kblock * 2u + u) * 1024u);
    } else {
      const uint32_t k0 = kblock * 128u + u * 64u + g * 16u;  // lane covers k0 .. k0+15
      f.w[u] = zero4;
      if (k0 < op.k) f.w[u] = load_stream16(op.wrow + k0);
    }
  }
  const uint32_t si = op.kb_per_scale == 1u ? kblock : kblock / op.kb_per_scale;
  if constexpr (SCALE == kF32) {
    f.sc[0] = static_cast<const float *>(op.srow)[si];
  } else {
    f.sc[0] = e8m0_to_f32(static_cast<const uint8_t *>(op.srow)[si]);
  }
}

// x[2u], x[2u+1]: the 16 k of half u as 2 x 16 bytes
__device__ __forceinline__ void fp8_load_x(XFrag<1> &f, const Fp8Operands &op, uint32_t kblock, uint32_t g) {
  const u32x4_t zero4 = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const uint32_t k0 = kblock * 128u + u * 64u + g * 16u;
    f.x[0][2 * u] = zero4;
    f.x[0][2 * u + 1] = zero4;
    if (k0 < op.k && op.xrow != nullptr) {
      f.x[0][2 * u] = load16(op.xrow + k0);
      f.x[0][2 * u + 1] = load16(op.xrow + k0 + 8);
    }
  }
}

template <int SCALE>
__device__ __forceinline__ void fp8_mac(const Fp8WFrag &f, const XFrag<1> &xf, f32x4_t &acc) {
  if constexpr (SCALE == kE8m0) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(expand_fp8_dwords(f.w[u][0], f.w[u][1], f.sc[0]),
                                                    as_bf16x8(xf.x[0][2 * u]), acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(expand_fp8_dwords(f.w[u][2], f.w[u][3], f.sc[0]),
                                                    as_bf16x8(xf.x[0][2 * u + 1]), acc, 0, 0, 0);
    }
  } else {
    // the f32 scale covers the whole 128 block: MFMA chain into a block accumulator,
    // then acc += scale * block (one FMA per accumulator register)
    f32x4_t blk = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      blk = __builtin_amdgcn_mfma_f32_16x16x32_bf16(expand_fp8_dwords(f.w[u][0], f.w[u][1], 1.0f),
                                                    as_bf16x8(xf.x[0][2 * u]), blk, 0, 0, 0);
      blk = __builtin_amdgcn_mfma_f32_16x16x32_bf16(expand_fp8_dwords(f.w[u][2], f.w[u][3], 1.0f),
                                                    as_bf16x8(xf.x[0][2 * u + 1]), blk, 0, 0, 0);
    }
#pragma unroll
    for (int v = 0; v < 4; ++v) acc[v] = fmaf(f.sc[0], blk[v], acc[v]);
  }
}

template <int SCALE, bool BLOCK_MAJOR, int DEPTH, int XDEPTH>
__device__ __forceinline__ void fp8_stream(const Fp8Operands &op, uint32_t first, uint32_t stride,
                                           uint32_t kblocks, uint32_t g, f32x4_t &acc) {
  static_assert(DEPTH % XDEPTH == 0, "ring slots are addressed with the unrolled index");
  Fp8WFrag wring[DEPTH];
  XFrag<1> xring[XDEPTH];
#pragma unroll
  for (int d = 0; d < XDEPTH; ++d) {
    const uint32_t j = first + d * stride;
    if (j < kblocks) fp8_load_x(xring[d], op, j, g);
  }
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) {
    const uint32_t j = first + d * stride;
    if (j < kblocks) fp8_load_w<SCALE, BLOCK_MAJOR>(wring[d], op, j, g);
  }
  for (uint32_t base = first; base < kblocks; base += DEPTH * stride) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const uint32_t j = base + d * stride;
      if (j < kblocks) {
        fp8_mac<SCALE>(wring[d], xring[d % XDEPTH], acc);
        const uint32_t next_x = j + XDEPTH * stride;
        if (next_x < kblocks) fp8_load_x(xring[d % XDEPTH], op, next_x, g);
        const uint32_t next_w = j + DEPTH * stride;
        if (next_w < kblocks) fp8_load_w<SCALE, BLOCK_MAJOR>(wring[d], op, next_w, g);
      }
    }
  }
}

}  // namespace ferrule_hip
