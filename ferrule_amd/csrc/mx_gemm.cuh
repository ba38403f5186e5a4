// Tiled GEMM core on the gfx950 scaled MFMA (v_mfma_scale_f32_16x16x128_f8f6f4):
//     Y[token, feature] = sum_k X[token, k] * W[feature, k]
// X is MX-FP8 (E4M3 bytes, one E8M0 scale per row and 128-wide K block), W is FP8 (E4M3, one
// scale per 128x128 block) or MXFP4 (E2M1 nibbles, one E8M0 scale per row and 32 k).  Both
// operands are K-major, so a weight row fragment is the MFMA's A operand and a token row
// fragment its B operand; accumulator register v of lane (i, g) is (feature 4g+v, token i),
// i.e. each lane ends up with four consecutive features of one token.
//
// One workgroup owns FN features x TM tokens (per weight matrix; up to NMAT matrices share
// the token fragments, e.g. gate and up).  Its waves form a WAVES_F x WAVES_T grid, each wave
// holds NF x NT accumulator tiles.  K advances 128 per step through an NSTAGE-deep ring of
// LDS stages that are filled with direct global->LDS loads (no VGPR staging): every wave
// issues the same number of loads per stage, so "stage s has landed" is an in-order vmcnt
// wait of the wave followed by one workgroup barrier, and the barrier also proves that the
// stage about to be refilled has been left by everybody.
//
// LDS layout of a stage: X rows of 128 bytes, then weight rows of 128 (FP8) or 64 (FP4)
// bytes, then for FP4 the rows' four scale bytes.  16-byte pieces are XOR-swizzled with the
// row index so that the 16 lanes of one ds_read_b128 phase hit 16 different bank groups:
//   128-byte rows: piece p of row r sits at slot p ^ ((r >> 1) & 7)
//    64-byte rows: piece p of row r sits at slot p ^ ((r >> 2) & 3)
// The swizzle costs nothing: a direct-to-LDS load writes lane l at base + 16*l, so it is
// applied to the lane's SOURCE address instead.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mx_core.cuh"
#include "numeric.cuh"
#include "skinny_core.cuh"

namespace ferrule_hip {

template <int WFMT_, int NMAT_, int NF_, int NT_, int WAVES_F_, int WAVES_T_, int NSTAGE_>
struct GemmShape {
  static constexpr int WFMT = WFMT_, NMAT = NMAT_, NF = NF_, NT = NT_;
  static constexpr int WAVES_F = WAVES_F_, WAVES_T = WAVES_T_, NSTAGE = NSTAGE_;
  static constexpr bool kFp4W = WFMT == kMfmaFmtFp4;
  static constexpr int kWaves = WAVES_F * WAVES_T;
  static constexpr int kThreads = kWaves * 64;
  static constexpr int FN = WAVES_F * NF * 16;  // features per workgroup and matrix
  static constexpr int TM = WAVES_T * NT * 16;  // tokens per workgroup
  static constexpr int kWRow = kFp4W ? 64 : 128;  // bytes of a weight row per K step
  static constexpr int kWPieces = kWRow / 16;
  static constexpr int kXBytes = TM * 128;
  static constexpr int kWBytes = NMAT * FN * kWRow;
  static constexpr int kSBytes = kFp4W ? NMAT * FN * 4 : 0;
  static constexpr int kStageBytes = kXBytes + kWBytes + kSBytes;
  // wave-wide load instructions per stage, by region
  static constexpr int kXInstr = kXBytes / 1024;
  static constexpr int kWInstr = kWBytes / 1024;
  static constexpr int kSInstr = kSBytes / 256;
  static_assert(kXInstr % kWaves == 0 && kWInstr % kWaves == 0 && kSInstr % kWaves == 0,
                "every wave issues the same loads per stage");
  static constexpr int kXSlots = kXInstr / kWaves;
  static constexpr int kWSlots = kWInstr / kWaves;
  static constexpr int kSSlots = kSInstr / kWaves;
  static constexpr int kSlots = kXSlots + kWSlots + kSSlots;  // loads per wave and stage
  static_assert((NSTAGE - 1) * kSlots <= 48, "vmcnt is a 6-bit counter");
  static_assert(NF * 16 <= 128, "a wave's features stay inside one 128-row scale block");
};

// What the core needs to know about the operands.  Row resolvers return the byte offset of a
// row from the operand's base, already clamped to a valid row.
template <int NMAT>
struct GemmOperands {
  const uint8_t *x;            // E4M3 rows
  const uint8_t *w[NMAT];      // weight rows
  const uint8_t *wscale[NMAT]; // FP4: [n, k/32] row scales; FP8: unused by the core
  uint32_t k;                  // multiple of 128
};

// Per-lane source cursors of the wave's loads for one stage; advanced by a constant per
// region after every stage.
template <typename S>
struct GemmCursors {
  const uint8_t *src[S::kSlots];
};

// xrow(r) / wrow(mat, r): byte offset of workgroup-local row r's first k (clamped rows for
// r beyond the problem); srow(mat, r): offset of its scale bytes.
template <typename S, typename XRow, typename WRow, typename SRow>
__device__ __forceinline__ void gemm_init_cursors(GemmCursors<S> &c, const GemmOperands<S::NMAT> &op,
                                                  uint32_t wave, uint32_t lane, XRow xrow, WRow wrow,
                                                  SRow srow) {
#pragma unroll
  for (int i = 0; i < S::kXSlots; ++i) {
    const uint32_t q = (i * S::kWaves + wave) * 64u + lane;  // 16-byte slot of the X region
    const uint32_t row = q >> 3, slot = q & 7u;
    const uint32_t piece = slot ^ ((row >> 1) & 7u);
    c.src[i] = op.x + xrow(row) + piece * 16u;
  }
#pragma unroll
  for (int i = 0; i < S::kWSlots; ++i) {
    const uint32_t q = (i * S::kWaves + wave) * 64u + lane;
    const uint32_t row = q / S::kWPieces, slot = q % S::kWPieces;
    const uint32_t piece = S::kFp4W ? slot ^ ((row >> 2) & 3u) : slot ^ ((row >> 1) & 7u);
    const uint32_t mat = row / S::FN, r = row % S::FN;
    const uint8_t *base = op.w[0];
#pragma unroll
    for (int m = 1; m < S::NMAT; ++m) base = mat == static_cast<uint32_t>(m) ? op.w[m] : base;
    c.src[S::kXSlots + i] = base + wrow(mat, r) + piece * 16u;
  }
#pragma unroll
  for (int i = 0; i < S::kSSlots; ++i) {
    const uint32_t row = (i * S::kWaves + wave) * 64u + lane;
    const uint32_t mat = row / S::FN, r = row % S::FN;
    const uint8_t *base = op.wscale[0];
#pragma unroll
    for (int m = 1; m < S::NMAT; ++m) base = mat == static_cast<uint32_t>(m) ? op.wscale[m] : base;
    c.src[S::kXSlots + S::kWSlots + i] = base + srow(mat, r);
  }
}

template <typename S>
__device__ __forceinline__ void gemm_issue_stage(GemmCursors<S> &c, uint8_t *stage, uint32_t wave) {
#pragma unroll
  for (int i = 0; i < S::kXSlots; ++i) {
    uint8_t *dst = stage + (i * S::kWaves + wave) * 1024u;
    __builtin_amdgcn_global_load_lds((global_u8_ptr)(c.src[i]), (lds_void_t *)(dst), 16, 0, 0);
    c.src[i] += 128;
  }
#pragma unroll
  for (int i = 0; i < S::kWSlots; ++i) {
    uint8_t *dst = stage + S::kXBytes + (i * S::kWaves + wave) * 1024u;
    __builtin_amdgcn_global_load_lds((global_u8_ptr)(c.src[S::kXSlots + i]), (lds_void_t *)(dst), 16, 0, 0);
    c.src[S::kXSlots + i] += S::kWRow;
  }
#pragma unroll
  for (int i = 0; i < S::kSSlots; ++i) {
    uint8_t *dst = stage + S::kXBytes + S::kWBytes + (i * S::kWaves + wave) * 256u;
    __builtin_amdgcn_global_load_lds((global_u8_ptr)(c.src[S::kXSlots + S::kWSlots + i]), (lds_void_t *)(dst), 4, 0,
                                     0);
    c.src[S::kXSlots + S::kWSlots + i] += 4;
  }
}

// One weight scale per (wave, K block) for FP8 weights: `Byte` = an E8M0 byte folded into the
// MFMA, `Float` = an f32 factor applied to the K block's partial sums on the VALU.
enum class WScaleMode { PerRow32 /* FP4 */, Byte, Float };

// Accumulate all K steps.  x_scale(t, kb) -> scale byte of this lane's token in token tile t;
// w_block_scale(mat, kb) -> uint32_t byte (Byte) or float bits (Float) for this wave.
template <typename S, WScaleMode MODE, typename XScale, typename WBlockScale>
__device__ __forceinline__ void gemm_mainloop(f32x4_t (&acc)[S::NMAT][S::NF][S::NT], GemmCursors<S> &cur,
                                              uint8_t *stages, uint32_t nk, uint32_t wave, uint32_t lane,
                                              XScale x_scale, WBlockScale w_block_scale) {
  const uint32_t i = lane & 15u, g = lane >> 4;
  const uint32_t wf = wave % S::WAVES_F, wt = wave / S::WAVES_F;
  // this lane's fragment addresses inside a stage
  uint32_t x_lo[S::NT], x_hi[S::NT];
#pragma unroll
  for (int t = 0; t < S::NT; ++t) {
    const uint32_t row = (wt * S::NT + t) * 16u + i;
    const uint32_t swz = (row >> 1) & 7u;
    x_lo[t] = row * 128u + ((g ^ swz) << 4);
    x_hi[t] = row * 128u + (((4u + g) ^ swz) << 4);
  }
  uint32_t w_lo[S::NMAT][S::NF], w_hi[S::NMAT][S::NF], w_sc[S::NMAT][S::NF];
#pragma unroll
  for (int m = 0; m < S::NMAT; ++m) {
#pragma unroll
    for (int f = 0; f < S::NF; ++f) {
      const uint32_t row = m * S::FN + (wf * S::NF + f) * 16u + i;
      if constexpr (S::kFp4W) {
        w_lo[m][f] = S::kXBytes + row * 64u + ((g ^ ((row >> 2) & 3u)) << 4);
        w_hi[m][f] = 0;
        w_sc[m][f] = S::kXBytes + S::kWBytes + row * 4u + g;
      } else {
        const uint32_t swz = (row >> 1) & 7u;
        w_lo[m][f] = S::kXBytes + row * 128u + ((g ^ swz) << 4);
        w_hi[m][f] = S::kXBytes + row * 128u + (((4u + g) ^ swz) << 4);
        w_sc[m][f] = 0;
      }
    }
  }

  // prologue: NSTAGE-1 stages in flight
#pragma unroll
  for (int s = 0; s < S::NSTAGE - 1; ++s) {
    if (static_cast<uint32_t>(s) < nk) gemm_issue_stage<S>(cur, stages + s * S::kStageBytes, wave);
  }
  uint32_t buf = 0, fill = S::NSTAGE - 1;
  for (uint32_t s = 0; s < nk; ++s) {
    // stages younger than s that may stay in flight
    const uint32_t younger = min(static_cast<uint32_t>(S::NSTAGE - 2), nk - 1u - s);
    if (younger == S::NSTAGE - 2) {
      wait_vmcnt((S::NSTAGE - 2) * S::kSlots);
    } else {
      wait_vmcnt(younger * S::kSlots);
    }
    lds_barrier();
    if (s + (S::NSTAGE - 1) < nk) {
      gemm_issue_stage<S>(cur, stages + fill * S::kStageBytes, wave);
      fill = fill + 1u == S::NSTAGE ? 0u : fill + 1u;
    }
    const uint8_t *st = stages + buf * S::kStageBytes;
    buf = buf + 1u == S::NSTAGE ? 0u : buf + 1u;

    i32x8_t xb[S::NT];
    uint32_t sx[S::NT];
#pragma unroll
    for (int t = 0; t < S::NT; ++t) {
      xb[t] = make_b_fp8(*reinterpret_cast<const u32x4_t *>(st + x_lo[t]),
                         *reinterpret_cast<const u32x4_t *>(st + x_hi[t]));
      sx[t] = x_scale(t, s);
    }
#pragma unroll
    for (int m = 0; m < S::NMAT; ++m) {
      uint32_t wsc = 0;
      if constexpr (MODE != WScaleMode::PerRow32) wsc = w_block_scale(m, s);
#pragma unroll
      for (int f = 0; f < S::NF; ++f) {
        i32x8_t wa;
        uint32_t sw;
        if constexpr (S::kFp4W) {
          wa = make_a_fp4(*reinterpret_cast<const u32x4_t *>(st + w_lo[m][f]));
          sw = st[w_sc[m][f]];
        } else {
          wa = make_b_fp8(*reinterpret_cast<const u32x4_t *>(st + w_lo[m][f]),
                          *reinterpret_cast<const u32x4_t *>(st + w_hi[m][f]));
          sw = MODE == WScaleMode::Byte ? wsc : 127u;
        }
#pragma unroll
        for (int t = 0; t < S::NT; ++t) {
          if constexpr (MODE == WScaleMode::Float) {
            const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
            const f32x4_t part = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                wa, xb[t], zero, S::WFMT, kMfmaFmtFp8, 0, static_cast<int>(sw), 0, static_cast<int>(sx[t]));
            const float ws = __uint_as_float(wsc);
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[m][f][t][v] = fmaf(part[v], ws, acc[m][f][t][v]);
          } else {
            acc[m][f][t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                wa, xb[t], acc[m][f][t], S::WFMT, kMfmaFmtFp8, 0, static_cast<int>(sw), 0,
                static_cast<int>(sx[t]));
          }
        }
      }
    }
  }
  lds_barrier();  // nobody reads the stages any more (the caller may reuse the LDS)
}

}  // namespace ferrule_hip
