// Decode-row schedule of the FP8 x FP8 block-scaled GEMM: at most 32 activation rows.
//
// The reference's fp8_projection is a small-M kernel (grid (ceil(N/16), ceil(M/8)), hundreds of
// CTAs at one row; capabilities/fp8_projection.cuh:424-497) and "native providers own row-count
// schedule dispatch" (src/cuda/provider.rs:46-49).  The 128 x 128 MFMA tile of fp8_gemm.hip puts
// a 7168 x 7168 matrix on 56 workgroups when there is one row: the kernel is then bound by how few
// loads are in flight, not by HBM.  Here the problem is what it is at this size, a stream over
// the weights:
//
//   one wave = 16 weight rows (features) x all of K.  Per 128-wide K block the wave's 16 rows x 128
//   bytes are the A operand of v_mfma_scale_f32_16x16x128_f8f6f4 (lane (i, g) holds k [16g, 16g+16)
//   and [64+16g, 64+16g+16) of row i); the B operand is the same two pieces of activation row
//   min(i, m-1) (m x K bytes, shared by every wave through L2); the E8M0 scales of both ride in the
//   instruction.  17 to 32 rows are two such MFMAs per K block that share the weight operand.
//   Operands reach the lanes through a ring of LDS slots private to the wave, filled by direct
//   global->LDS loads of whole cache lines (RowsSlot); there is no barrier, and nothing is shared
//   between waves, so a launch of N/16 single-wave workgroups spreads over every CU.
//
// An output element is the same chain of K-block MFMAs (and, with f32 weight scales, the same
// v_fma folds) as in the tiled kernel, so the two schedules give the same bits; the row count
// alone decides which one runs.
//
// The shared FFN's gate/up stage (capabilities/shared_ffn.cuh:477-523 is the reference's small-M
// form) uses the same stream with rows 0-7 of the A operand taken from W1 and rows 8-15 from W3:
// one MFMA per K block yields gate and up of 8 features, a wave owns 8 features of both
// matrices, and an intermediate size of 2048 is 256 waves instead of 16 workgroups.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ferrule_hip_provider.h"
#include "fp8_gemm.h"
#include "mx_gemm.cuh"

namespace ferrule_hip {
namespace {

constexpr int kOutSwiGlu = 16;  // epilogue selector beside the kGemmOut* modes

struct RowsParams {
  const uint8_t *x;    // E4M3 [m, k]
  const uint8_t *xs;   // UE8M0 [m, cols]
  const uint8_t *w[2]; // E4M3 [n, k]
  const void *ws[2];   // UE8M0 or f32 [ceil(n/128), cols]
  void *out[2];
  uint32_t n[2];       // n[1] = 0: one matrix
  uint32_t m, k, cols; // cols = k / 128 >= 4
  float output_scale, swiglu_limit;  // SwiGLU epilogue only
};

// One ring slot in LDS: a window of four consecutive K blocks of the wave's 16 weight rows and of the
// activation rows, and the scales of those four blocks.  Everything arrives by direct global->LDS
// loads whose wave instruction covers whole cache lines: 8 weight rows x 128 bytes, or 2 activation
// rows x 512 bytes (the four K blocks of a row are consecutive).  Loading the MFMA fragments straight
// into registers instead makes every wave instruction touch 16 rows x 64 bytes, half a line per row,
// and such an instruction costs the CU's address path about 65 cycles against 17 (measured, data in
// L2): that, not HBM, bounded the earlier form of this kernel from a few rows on (7168 x 7168: 16 us at
// 16 rows, 24 us at 32).
// XI = activation load instructions per slot = staged rows / 2: 1, 2, 4, 6, 8, 12, 16 for up to 2, 4, 8, 12, 16,
// 24, 32 activation rows: no more activation loads than the rows need.  (vmcnt's 6 bits would allow up to six
// slots at one row; three measure best, see the launcher.)
// The 16-byte pieces of every 128-byte row segment are XOR-swizzled on the SOURCE address (piece
// s ^ (row & 7) lands in slot s), so the fragment reads of 16 rows hit different banks.
// WAVES = waves per workgroup.  With 8 and more activation rows the activations are as many bytes per
// wave as the weights, and every wave fetching all of them makes the launch ask L2 for twice to three
// times the weight bytes; two waves (32 features) then share one copy of a slot's activation rows, each
// loading half of it, with a workgroup barrier before a slot is read and before it is refilled.
template <int XI, int WAVES>
struct RowsSlot {
  static constexpr int TT = XI > 8 ? 2 : 1;               // MFMAs per K block (16 activation rows each)
  static constexpr uint32_t kStagedRows = 2u * XI;
  static constexpr uint32_t kWBytes = 4u * 16u * 128u;     // per wave: [K block][row][128]
  static constexpr uint32_t kXBytes = kStagedRows * 512u;  // shared: [row][K block][128]
  static constexpr int kXLoads = XI / WAVES;               // activation loads per wave and slot
  static constexpr int kScaleLoads = TT;                   // per wave: dword-per-lane loads (see fill)
  static constexpr uint32_t kScaleBytes = 256u * kScaleLoads;
  static constexpr uint32_t kBytes = WAVES * kWBytes + kXBytes + WAVES * kScaleBytes;
  static constexpr int kLoads = 8 + kXLoads + kScaleLoads; // wave instructions per fill
  static constexpr int kGroups = 62 / kLoads < 3 ? 62 / kLoads : 3;
  static_assert(XI % WAVES == 0 && kGroups * kBytes <= 160u * 1024u, "LDS");
};

// Slot::kGroups ring slots are in flight per wave.  All loads of the kernel are direct-to-LDS loads,
// issued as inline assembly and counted by hand: they return in issue order among themselves (not
// with respect to register loads, which is why the scales travel the same way).
template <WScaleMode MODE, int OUT, int XI, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void fp8_rows_kernel(RowsParams p) {
  using Slot = RowsSlot<XI, WAVES>;
  constexpr int GROUPS = Slot::kGroups, TT = Slot::TT;
  constexpr uint32_t kDepth = 4u * GROUPS;
  static_assert(GROUPS * Slot::kLoads <= 63, "vmcnt is a 6-bit counter");
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = WAVES == 1 ? 0u : __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t i = lane & 15u, g = lane >> 4;
  // this wave's tile of 16 weight rows; a wave beyond the last tile (an odd number of tiles, two waves
  // per workgroup) repeats the last one, because it shares the barriers and the activation loads, and
  // stores nothing
  uint32_t mat, f0, n;
  bool spare;
  if constexpr (OUT == kOutSwiGlu) {
    const uint32_t tiles = p.n[0] >> 3;
    const uint32_t tile = blockIdx.x * WAVES + wave;
    spare = tile >= tiles;
    mat = 0u;       // rows 0-7 of the tile: W1 (gate) rows f0.., rows 8-15: W3 (up) rows f0..
    f0 = min(tile, tiles - 1u) * 8u;
    n = p.n[0];
  } else {
    const uint32_t tiles0 = (p.n[0] + 15u) >> 4, tiles = tiles0 + ((p.n[1] + 15u) >> 4);
    uint32_t tile = blockIdx.x * WAVES + wave;
    spare = tile >= tiles;
    tile = min(tile, tiles - 1u);
    mat = tile >= tiles0 ? 1u : 0u;   // wave-uniform
    f0 = (tile - mat * tiles0) * 16u;
    n = mat ? p.n[1] : p.n[0];
  }
  const uint32_t nk = p.k >> 7;

  // Sources of the payload loads: a wave-uniform base per instruction (the window's first K block,
  // computed on the scalar unit) plus this lane's constant 32-bit offset.
  //   weights: instruction h of a K block covers tile rows 8h .. 8h+7; lane l takes row 8h + l/8, slot l%8
  //   activations: instruction h covers staged rows 2h, 2h+1; lane l takes row 2h + l/32, K block (l%32)/8
  //   of the window, slot l%8
  const uint32_t s8 = lane & 7u;
  const uint8_t *wbase[2];
  uint32_t woff[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const uint32_t r8 = lane >> 3;
    const uint32_t piece = (s8 ^ r8) * 16u;       // (row & 7) == r8 for every 8-row instruction
    if constexpr (OUT == kOutSwiGlu) {
      wbase[h] = p.w[h] + static_cast<size_t>(f0) * p.k;
      woff[h] = (min(f0 + r8, n - 1u) - f0) * p.k + piece;
    } else {
      wbase[h] = (mat ? p.w[1] : p.w[0]) + static_cast<size_t>(f0) * p.k;
      woff[h] = (min(f0 + 8u * h + r8, n - 1u) - f0) * p.k + piece;
    }
  }
  uint32_t xoff[Slot::kXLoads];   // this wave's share of the slot's activation loads
#pragma unroll
  for (int h = 0; h < Slot::kXLoads; ++h) {
    const uint32_t staged = 2u * (wave * Slot::kXLoads + h) + (lane >> 5);
    xoff[h] = min(staged, p.m - 1u) * p.k + ((lane >> 3) & 3u) * 128u + ((s8 ^ (staged & 7u)) * 16u);
  }

  // Sources of the scale loads (64-bit addresses per lane; aligned dwords, because the four scale
  // bytes of a window start at any byte).  Per 16 activation rows one load: lanes 0-15 the dword that
  // holds the first scale byte of the window of row `lane`, lanes 16-31 the following dword, and in the
  // first load lanes 32-35 the weight scales (f32: the four scales; bytes: the two dwords around the
  // window, of the gate or only matrix in lanes 32-33 and of the up matrix in lanes 34-35).  A dword
  // that is not needed is read from a valid address all the same.
  const uint32_t wblock = f0 >> 7;
  const uint8_t *const ws_row = static_cast<const uint8_t *>(mat ? p.ws[1] : p.ws[0]) +
                                static_cast<size_t>(wblock) * p.cols * (MODE == WScaleMode::Float ? 4u : 1u);
  const uint8_t *const ws_row2 = OUT == kOutSwiGlu ? static_cast<const uint8_t *>(p.ws[1]) +
                                                         static_cast<size_t>(wblock) * p.cols
                                                   : ws_row;
  auto aligned_dword = [](const uint8_t *at, uint32_t which) {
    const uintptr_t a = reinterpret_cast<uintptr_t>(at);
    // the second dword only when the four bytes straddle: otherwise it could lie past the buffer
    return reinterpret_cast<const uint8_t *>((a & ~static_cast<uintptr_t>(3)) + ((which && (a & 3u)) ? 4u : 0u));
  };

  // First K block of the window that serves the group starting at K block kb0: the window must end
  // inside the row, so the last groups of a K that is no multiple of four (and the fills past the end
  // of K, which nobody reads) take the row's last four blocks.  A fill always issues the same loads,
  // so the wait counts below are constants.
  auto window_of = [&](uint32_t kb0) { return min(kb0, nk - 4u); };
  auto fill = [&](uint32_t slot, uint32_t kb0) {
    uint8_t *const base = lds + slot * Slot::kBytes;
    const uint32_t sb = window_of(kb0);
    const size_t at = static_cast<size_t>(sb) * 128u;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        lds_dma16_stream(wbase[h] + at + j * 128, woff[h], base + wave * Slot::kWBytes + j * 2048 + h * 1024);
      }
    }
#pragma unroll
    for (int h = 0; h < Slot::kXLoads; ++h) {
      lds_dma16(p.x + at, xoff[h], base + WAVES * Slot::kWBytes + (wave * Slot::kXLoads + h) * 1024);
    }
    uint8_t *const scales = base + WAVES * Slot::kWBytes + Slot::kXBytes + wave * Slot::kScaleBytes;
#pragma unroll
    for (int t = 0; t < TT; ++t) {
      const uint32_t row = min(static_cast<uint32_t>(t) * 16u + i, p.m - 1u);
      const uint8_t *from = aligned_dword(p.xs + static_cast<size_t>(row) * p.cols + sb, g & 1u);
      if (t == 0 && lane >= 32u) {
        const uint32_t q = lane - 32u;
        if constexpr (MODE == WScaleMode::Float) {
          from = ws_row + static_cast<size_t>(sb + min(q, 3u)) * 4u;
        } else {
          from = aligned_dword(((q & 2u) ? ws_row2 : ws_row) + sb, q & 1u);
        }
      }
      lds_dma4(from, scales + t * 256);
    }
  };

  f32x4_t acc[TT];
#pragma unroll
  for (int t = 0; t < TT; ++t) acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  // this lane's fragment addresses inside a K block of the weight region and inside a staged row
  const uint32_t w_lo = i * 128u + ((g ^ (i & 7u)) * 16u), w_hi = i * 128u + (((4u + g) ^ (i & 7u)) * 16u);
  uint32_t x_lo[TT], x_hi[TT], xs_at[TT];
#pragma unroll
  for (int t = 0; t < TT; ++t) {
    // a lane whose activation row is not staged (beyond m, rounded up to two) reads the last staged row
    const uint32_t staged = min(static_cast<uint32_t>(t) * 16u + i, Slot::kStagedRows - 1u);
    x_lo[t] = staged * 512u + ((g ^ (staged & 7u)) * 16u);
    x_hi[t] = staged * 512u + (((4u + g) ^ (staged & 7u)) * 16u);
    // where this lane's scale window starts, in bytes from the (16-byte aligned) scale array, before the
    // window's first column is added: the low two bits of the sum are its offset inside the aligned dwords
    xs_at[t] = min(static_cast<uint32_t>(t) * 16u + i, p.m - 1u) * p.cols;
  }
  const uint32_t ws_at = wblock * p.cols;
  // K block `sel` of the window in ring slot `slot`; the window starts at K block sb.  With f32 weight
  // scales the K block's products come back in `fresh` (and the scale in `fresh_scale`) for fold().
  auto consume = [&](uint32_t slot, uint32_t sel, uint32_t sb, f32x4_t (&fresh)[TT], float &fresh_scale) {
    const uint8_t *const base = lds + slot * Slot::kBytes;
    const uint8_t *const wk = base + wave * Slot::kWBytes + sel * 2048u;
    const i32x8_t wa = make_b_fp8(*reinterpret_cast<const u32x4_t *>(wk + w_lo),
                                  *reinterpret_cast<const u32x4_t *>(wk + w_hi));
    const uint32_t *const sc = reinterpret_cast<const uint32_t *>(base + WAVES * Slot::kWBytes + Slot::kXBytes +
                                                                  wave * Slot::kScaleBytes);
    int sw_byte = 0;
    float ws = 0.0f;
    if constexpr (MODE == WScaleMode::Float) {
      ws = __uint_as_float(sc[32u + sel]);
    } else {
      // SwiGLU: tile rows 8-15 (lanes i >= 8) belong to the up matrix, whose dwords lanes 34, 35 fetched
      const uint32_t pair = (OUT == kOutSwiGlu && i >= 8u) ? 34u : 32u;
      const uint32_t window = __builtin_amdgcn_alignbyte(sc[pair + 1u], sc[pair], (ws_at + sb) & 3u);
      sw_byte = static_cast<int>(window >> (8u * sel));
    }
#pragma unroll
    for (int t = 0; t < TT; ++t) {
      const uint8_t *const xk = base + WAVES * Slot::kWBytes + sel * 128u;
      const i32x8_t xb = make_b_fp8(*reinterpret_cast<const u32x4_t *>(xk + x_lo[t]),
                                    *reinterpret_cast<const u32x4_t *>(xk + x_hi[t]));
      const uint32_t window = __builtin_amdgcn_alignbyte(sc[t * 64 + 16u + i], sc[t * 64 + i], (xs_at[t] + sb) & 3u);
      const int sx = static_cast<int>(window >> (8u * sel));   // the instruction takes byte 0
      if constexpr (MODE == WScaleMode::Float) {
        // f32 weight scales cannot ride in the instruction: a fresh product per K block, folded
        // with one v_fma per value (the tiled kernel's arithmetic)
        const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
        fresh[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wa, xb, zero, kMfmaFmtFp8, kMfmaFmtFp8, 0, 127,
                                                                     0, sx);
        fresh_scale = ws;
      } else {
        acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wa, xb, acc[t], kMfmaFmtFp8, kMfmaFmtFp8, 0,
                                                                  sw_byte, 0, sx);
      }
    }
  };
  auto fold = [&](const f32x4_t (&fresh)[TT], float ws) {
    if constexpr (MODE == WScaleMode::Float) {
#pragma unroll
      for (int t = 0; t < TT; ++t) {
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[t][v] = fmaf(fresh[t][v], ws, acc[t][v]);
      }
    }
  };

#pragma unroll
  for (int r = 0; r < GROUPS; ++r) fill(static_cast<uint32_t>(r), 4u * r);
  uint32_t kb0 = 0;
  for (; kb0 + kDepth <= nk; kb0 += kDepth) {   // whole rings: every window starts at its group's first block
#pragma unroll
    for (int r = 0; r < GROUPS; ++r) {
      wait_vmcnt((GROUPS - 1) * Slot::kLoads);   // slot r has landed; the younger slots are still in flight
      if constexpr (WAVES > 1) stage_barrier();  // ... the other wave's half of its activations too
      asm volatile("" ::: "memory");
      const uint32_t sb = kb0 + 4u * r;
      // the slot's four products first, then their folds in K order: a fold right behind its own MFMA
      // would sit out the instruction's latency four (eight) times per slot
      f32x4_t fresh[4][TT];
      float fresh_scale[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) consume(static_cast<uint32_t>(r), static_cast<uint32_t>(j), sb, fresh[j], fresh_scale[j]);
#pragma unroll
      for (int j = 0; j < 4; ++j) fold(fresh[j], fresh_scale[j]);
      __builtin_amdgcn_sched_barrier(0);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the slot's last fragments are in registers
      if constexpr (WAVES > 1) stage_barrier();  // ... in both waves: the refill overwrites shared rows
      fill(static_cast<uint32_t>(r), sb + kDepth);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  // what is left of K: fewer than kDepth blocks, all of them in the ring; no more fills
#pragma unroll
  for (int r = 0; r < GROUPS; ++r) {
    const uint32_t first = kb0 + 4u * r;
    if (first < nk) {   // the same in every wave of the workgroup
      wait_vmcnt((GROUPS - 1 - r) * Slot::kLoads);
      if constexpr (WAVES > 1) stage_barrier();
      asm volatile("" ::: "memory");
      const uint32_t sb = window_of(first);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (first + j < nk) {
          f32x4_t fresh[TT];
          float fresh_scale = 0.0f;
          consume(static_cast<uint32_t>(r), first + j - sb, sb, fresh, fresh_scale);
          fold(fresh, fresh_scale);
        }
      }
    }
  }
  wait_vmcnt(0);   // nothing may still be writing this workgroup's LDS when it ends

  // acc[t][v] = (weight row 4g + v of the tile, activation row 16 t + i)
#pragma unroll
  for (int t = 0; t < TT; ++t) {
    const uint32_t token = static_cast<uint32_t>(t) * 16u + i;
    const f32x4_t a = acc[t];
    if constexpr (OUT == kOutSwiGlu) {
      // lanes g = 0, 1 hold gate of features f0 + 4g + v, lanes g + 2 the up values of the same ones
      f32x4_t up;
#pragma unroll
      for (int v = 0; v < 4; ++v) up[v] = __shfl_xor(a[v], 32, 64);
      if (spare || g >= 2u || token >= p.m) continue;
      float h[4];
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        // the arithmetic of swiglu_quantize_store (swiglu_quant.cuh), value for value
        float gate = a[v], u = up[v];
        if (p.swiglu_limit > 0.0f) {
          gate = fminf(gate, p.swiglu_limit);
          u = fminf(p.swiglu_limit, fmaxf(-p.swiglu_limit, u));
        }
        float value = silu_fast(gate) * u * p.output_scale;
        if (!(fabsf(value) <= 3.4028234e38f)) value = 0.0f;
        h[v] = value;
      }
      const uint32_t feat = f0 + g * 4u;
      if (feat < n) {   // n is a multiple of 128: whole quads
        *reinterpret_cast<float4 *>(static_cast<float *>(p.out[0]) + static_cast<size_t>(token) * n + feat) =
            make_float4(h[0], h[1], h[2], h[3]);
      }
    } else {
      if (spare || token >= p.m) continue;
      void *const output = mat ? p.out[1] : p.out[0];
      const uint32_t feat = f0 + g * 4u;
      const size_t at = static_cast<size_t>(token) * n + feat;
      if (feat + 3u < n && (n & 3u) == 0u) {
        if constexpr (OUT == kGemmOutBf16) {
          const uint32_t lo = bf16_rne_bits(a[0]) | (static_cast<uint32_t>(bf16_rne_bits(a[1])) << 16);
          const uint32_t hi = bf16_rne_bits(a[2]) | (static_cast<uint32_t>(bf16_rne_bits(a[3])) << 16);
          *reinterpret_cast<uint2 *>(static_cast<uint16_t *>(output) + at) = make_uint2(lo, hi);
        } else if constexpr (OUT == kGemmOutF32Rounded) {
          *reinterpret_cast<float4 *>(static_cast<float *>(output) + at) =
              make_float4(bf16_round(a[0]), bf16_round(a[1]), bf16_round(a[2]), bf16_round(a[3]));
        } else {
          float4 *dst = reinterpret_cast<float4 *>(static_cast<float *>(output) + at);
          float4 v = make_float4(a[0], a[1], a[2], a[3]);
          if constexpr (OUT == kGemmOutF32Accumulate) {
            const float4 old = *dst;
            v = make_float4(old.x + v.x, old.y + v.y, old.z + v.z, old.w + v.w);
          }
          *dst = v;
        }
      } else {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          if (feat + v < n) {
            if constexpr (OUT == kGemmOutBf16) {
              static_cast<uint16_t *>(output)[at + v] = static_cast<uint16_t>(bf16_rne_bits(a[v]));
            } else if constexpr (OUT == kGemmOutF32Rounded) {
              static_cast<float *>(output)[at + v] = bf16_round(a[v]);
            } else if constexpr (OUT == kGemmOutF32Accumulate) {
              static_cast<float *>(output)[at + v] += a[v];
            } else {
              static_cast<float *>(output)[at + v] = a[v];
            }
          }
        }
      }
    }
  }
}

// Measured on N = K = 7168 with f32 block scales, kernel alone, plain loads: 1 / 8 / 16 / 32 rows 10.7 / 10.9 / 12.3-12.7 /
// 16.2 us (the register-load form: 11.4 / 13.4 / 16.0 / 23.8 us).  Three ring slots; four to six slots
// (up to 48 KB of weights in flight per wave at one row) are 2-10 % slower, two about the same.
// The weights are loaded nontemporally (one row 10.7 -> 9.8 us, 16 rows 12.6 -> 12.1 us, 32 rows unchanged); the
// activations, which every wave reads, are not.
// From 9 rows on two waves share a slot's activation rows (16 rows 12.1 -> 10.6 us, 32 rows 16.2 -> 13.8 us: the
// launch asks L2 for 77 and 102 MB instead of 102 and 154 MB, and the time follows those bytes at about 7.3 TB/s).
template <WScaleMode MODE, int OUT, int XI, int WAVES>
void launch_rows_kernel(const RowsParams &p, uint32_t tiles, hipStream_t stream) {
  using Slot = RowsSlot<XI, WAVES>;
  constexpr uint32_t kLds = Slot::kGroups * Slot::kBytes;
  auto kernel = fp8_rows_kernel<MODE, OUT, XI, WAVES>;
  if (kLds > 64u * 1024u) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(kLds)) != hipSuccess) {
      return;   // the launch error is picked up by the caller
    }
  }
  kernel<<<(tiles + WAVES - 1u) / WAVES, 64 * WAVES, kLds, stream>>>(p);
}

// `tiles` = 16-feature tiles of both matrices (SwiGLU: 8-feature tiles of the pair)
template <WScaleMode MODE, int OUT>
void launch_rows_out(const RowsParams &p, uint32_t tiles, hipStream_t stream) {
  if (p.m <= 2u) {
    launch_rows_kernel<MODE, OUT, 1, 1>(p, tiles, stream);
  } else if (p.m <= 4u) {
    launch_rows_kernel<MODE, OUT, 2, 1>(p, tiles, stream);
  } else if (p.m <= 8u) {
    launch_rows_kernel<MODE, OUT, 4, 1>(p, tiles, stream);
  } else if (p.m <= 12u) {
    launch_rows_kernel<MODE, OUT, 6, 2>(p, tiles, stream);
  } else if (p.m <= 16u) {
    launch_rows_kernel<MODE, OUT, 8, 2>(p, tiles, stream);
  } else if (p.m <= 24u) {
    launch_rows_kernel<MODE, OUT, 12, 2>(p, tiles, stream);
  } else {
    launch_rows_kernel<MODE, OUT, 16, 2>(p, tiles, stream);
  }
}

template <WScaleMode MODE>
void launch_rows(const RowsParams &p, int out_mode, uint32_t grid, hipStream_t stream) {
  switch (out_mode) {
    case kGemmOutBf16: launch_rows_out<MODE, kGemmOutBf16>(p, grid, stream); break;
    case kGemmOutF32Raw: launch_rows_out<MODE, kGemmOutF32Raw>(p, grid, stream); break;
    case kGemmOutF32Accumulate: launch_rows_out<MODE, kGemmOutF32Accumulate>(p, grid, stream); break;
    default: launch_rows_out<MODE, kGemmOutF32Rounded>(p, grid, stream); break;
  }
}

int32_t finish_launch() { return take_launch_error() == hipSuccess ? FERRULE_HIP_SUCCESS : FERRULE_HIP_LAUNCH_FAILED; }

}  // namespace

// at least four K blocks: the scales of a group are fetched as one four-column window of the row
bool fp8_rows_applies(uint32_t rows, uint32_t k) { return rows >= 1u && rows <= kFp8RowsMax && k >= 512u; }

int32_t fp8_rows_run(const Fp8GemmParams &g, bool f32_scales, int out_mode, uint64_t stream_bits) {
  RowsParams p;
  p.x = g.x;
  p.xs = g.xs;
  p.w[0] = g.w;
  p.ws[0] = g.ws;
  p.out[0] = g.out;
  p.n[0] = g.n;
  p.w[1] = g.n2 ? g.w2 : g.w;
  p.ws[1] = g.n2 ? g.ws2 : g.ws;
  p.out[1] = g.n2 ? g.out2 : g.out;
  p.n[1] = g.n2;
  p.m = g.m;
  p.k = g.k;
  p.cols = g.cols;
  p.output_scale = 1.0f;
  p.swiglu_limit = 0.0f;
  const uint32_t grid = ((g.n + 15u) >> 4) + ((g.n2 + 15u) >> 4);
  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(stream_bits));
  clear_launch_error();
  if (f32_scales) {
    launch_rows<WScaleMode::Float>(p, out_mode, grid, stream);
  } else {
    launch_rows<WScaleMode::Byte>(p, out_mode, grid, stream);
  }
  return finish_launch();
}

int32_t fp8_rows_swiglu_run(const uint8_t *x, const uint8_t *xs, const uint8_t *gate, const uint8_t *gate_s,
                            const uint8_t *up, const uint8_t *up_s, float *hidden_f32, uint32_t rows,
                            uint32_t input_size, uint32_t intermediate_size, float output_scale, float swiglu_limit,
                            uint64_t stream_bits) {
  RowsParams p;
  p.x = x;
  p.xs = xs;
  p.w[0] = gate;
  p.ws[0] = gate_s;
  p.w[1] = up;
  p.ws[1] = up_s;
  p.out[0] = p.out[1] = hidden_f32;
  p.n[0] = p.n[1] = intermediate_size;
  p.m = rows;
  p.k = input_size;
  p.cols = input_size >> 7;
  p.output_scale = output_scale;
  p.swiglu_limit = swiglu_limit;
  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(stream_bits));
  clear_launch_error();
  launch_rows_out<WScaleMode::Byte, kOutSwiGlu>(p, intermediate_size / 8u, stream);
  return finish_launch();
}

}  // namespace ferrule_hip
