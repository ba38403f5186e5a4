// FP8 x FP8 block-scaled GEMM for packed verification / prefill rows:
//   y[row, n] = bf16_round( sum_kb  (sum_{k in kb} a[row,k] * w[n,k]) * w_scale[n/128, kb] * a_scale[row, kb] )
// Drop-ins for ferrule_cutlass_fp8_projection_* and ferrule_cutlass_fp8_query_a_kv_*
// (abi/cutlass_provider.h:391-398; kernel capabilities/fp8_projection.cuh:318-416) plus the
// general entry with F32 weight scales / BF16 output.
//
// MFMA bound.  The K128 scale blocks are exactly the K extent of one
// v_mfma_scale_f32_16x16x128_f8f6f4, so E8M0 scales of both operands ride inside the
// instruction (exact powers of two, same value as the reference's fp32 multiplies) and the
// accumulation over K blocks happens in the MFMA accumulator.  F32 weight scales cannot be
// folded: each K block is then a fresh MFMA (C = 0) whose four partial sums are fused into the
// running sum with one v_fma each.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "../../include/ferrule_hip_provider.h"
#include "fp8_gemm.h"
#include "mx_gemm.cuh"

namespace ferrule_hip {
namespace {

// 128 x 128 per workgroup, three stages: fills 256 CUs from M = 512 upwards.  Eight waves of
// 64 x 32: with one workgroup per CU the K loop is bound by its per-step latencies, and two
// waves per SIMD overlap them (M = 512: 46 -> 40 us with E8M0 scales, 63 -> 42 us with f32).
using ShapeSmall = GemmShape<kMfmaFmtFp8, 1, 4, 2, 2, 4, 3>;
static_assert(!ShapeSmall::SPREAD_T, "the token scale rows of a wave are addressed as t * 16 rows from its first");
// 256 features x 256 tokens, two stages: half the operand traffic per flop; used as soon as it
// yields enough workgroups to occupy most of the 256 CUs.  Eight waves of 128 x 64 rather than
// four of 128 x 128: two waves per SIMD cover each other's waits (measured +5..9 %).
using ShapeLarge = GemmShape<kMfmaFmtFp8, 1, 8, 4, 2, 4, 2>;
constexpr uint64_t kLargeMinTiles = 192;
// 64 features x 128 tokens, four stages, eight waves of 32 x 32: for launches that would put at most half
// of the CUs to work with the 128 x 128 shape (33 to 128 rows against a 7168-row matrix are 56 of them),
// where the time is set by how many workgroups stream the weights and not by the tile's arithmetic.
using ShapeNarrow = GemmShape<kMfmaFmtFp8, 1, 2, 2, 2, 4, 4>;
static_assert(!ShapeNarrow::SPREAD_T, "the token scale rows of a wave are addressed as t * 16 rows from its first");
static_assert(ShapeNarrow::FN == 64 && 128 % ShapeNarrow::FN == 0, "a narrow tile lies inside one 128-row scale block");

template <typename S>
__host__ __device__ constexpr uint32_t gemm_lds_bytes(uint32_t cols) {
  // stages, token scale bytes [TM][cols], weight block scales [FN/128][cols] as dwords
  return S::NSTAGE * S::kStageBytes + ((S::TM * cols + 15u) & ~15u) + ((S::FN + 127) / 128) * cols * 4u;
}

// Half of ShapeLarge's tile along the tokens, three stages.  When the last round of large tiles
// would occupy at most half of the CUs, each of its tiles is cut into two of these (into four of
// ShapeSmall when it would occupy at most a quarter): the round then runs on all CUs and ends in a
// fraction of the time (an output element is the same chain of K-block MFMAs whatever tile it
// belongs to, so the bits do not change).
using ShapeLargeTail = GemmShape<kMfmaFmtFp8, 1, 4, 4, 4, 2, 3>;
static_assert(!ShapeLargeTail::SPREAD_T, "the token scale rows of a wave are addressed as t * 16 rows from its first");
constexpr uint32_t kCus = 256;

// Into how many pieces (1, 2 or 4) each tile of the last round of large tiles is cut: quarters
// (the 128 x 128 shape) when they fit the CUs in one round, else halves, else the tiles stay whole.
__host__ __device__ constexpr uint32_t last_round_pieces(uint32_t tiles, bool can_cut) {
  const uint32_t last = tiles % kCus;
  if (!can_cut || tiles <= kCus || last == 0) return 1;
  return 4 * last <= kCus ? 4 : 2 * last <= kCus ? 2 : 1;
}

struct GemmTile {
  uint32_t t0, f0, n;  // first token row, first feature of the matrix, its features
  const uint8_t *weight;
  const void *weight_scales;
  void *output;
};

// Tile of shape S of virtual block `id`, in the order described in the kernel.
template <typename S>
__device__ __forceinline__ GemmTile gemm_tile_of(const Fp8GemmParams &p, uint32_t id) {
  const uint32_t tiles_t = (p.m + S::TM - 1) / S::TM;
  const uint32_t tiles_f1 = (p.n + S::FN - 1) / S::FN;
  const uint32_t tiles_f = tiles_f1 + (p.n2 + S::FN - 1) / S::FN;  // feature tiles of both matrices
  constexpr uint32_t kPanel = 4;
  const uint32_t nb = tiles_t * tiles_f;
  const uint32_t per = nb >> 3;
  if (id < per * 8u) id = (id & 7u) * per + (id >> 3);
  const uint32_t panel = id / (kPanel * tiles_f);
  const uint32_t in_panel = id - panel * (kPanel * tiles_f);
  const uint32_t panel_t0 = panel * kPanel;
  const uint32_t panel_rows = min(kPanel, tiles_t - panel_t0);
  const uint32_t ft = in_panel / panel_rows;
  // the tile's matrix: feature tiles of the second one follow those of the first
  const bool second = ft >= tiles_f1;
  GemmTile tile;
  tile.t0 = (panel_t0 + in_panel % panel_rows) * S::TM;
  tile.f0 = (second ? ft - tiles_f1 : ft) * S::FN;
  tile.n = second ? p.n2 : p.n;
  tile.weight = second ? p.w2 : p.w;
  tile.weight_scales = second ? p.ws2 : p.ws;
  tile.output = second ? p.out2 : p.out;
  return tile;
}

// One output tile: FN features from f0 on x TM tokens from t0 on.
template <typename S, WScaleMode MODE, int OUT>
__device__ __forceinline__ void fp8_gemm_tile(const Fp8GemmParams &p, const GemmTile &tile, uint8_t *lds) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t t0 = tile.t0, f0 = tile.f0, n = tile.n;
  const uint8_t *const weight = tile.weight;
  const void *const weight_scales = tile.weight_scales;
  void *const output = tile.output;

  uint8_t *stages = lds;
  uint8_t *xsc = lds + S::NSTAGE * S::kStageBytes;
  uint32_t *wsc = reinterpret_cast<uint32_t *>(xsc + ((S::TM * p.cols + 15u) & ~15u));

  // operands from the tile's first rows on: the lane offsets of the cursors are 32-bit
  GemmOperands<1> op;
  op.x = p.x + static_cast<size_t>(t0) * p.k;
  op.w[0] = weight + static_cast<size_t>(f0) * p.k;
  op.wscale[0] = nullptr;
  op.k = p.k;
  GemmCursors<S> cur;
  gemm_init_cursors<S>(
      cur, op, wave, lane,
      [&](uint32_t r) { return (min(t0 + r, p.m - 1u) - t0) * p.k; },
      [&](uint32_t, uint32_t r) { return (min(f0 + r, n - 1u) - f0) * p.k; },
      [&](uint32_t, uint32_t) { return 0u; });
  // the first stages go out first; the scale tables are staged under their latency
  gemm_prologue<S>(cur, stages, p.k >> 7, wave);

  // token scales of the tile, [TM][cols] bytes: dwords when the rows allow it.  A thread's copies
  // are fetched together and stored afterwards (a load and its store per pass would put one memory
  // latency per pass in front of the K loop).
  if ((p.cols & 3u) == 0u) {
    const uint32_t dcols = p.cols >> 2;
    const uint32_t total = S::TM * dcols;
    for (uint32_t base = 0; base < total; base += 4u * S::kThreads) {
      uint32_t v[4];
#pragma unroll
      for (uint32_t j = 0; j < 4u; ++j) {
        const uint32_t idx = min(base + j * S::kThreads + threadIdx.x, total - 1u);
        const uint32_t row = idx / dcols, c = idx - row * dcols;
        const uint32_t token = min(t0 + row, p.m - 1u);
        v[j] = reinterpret_cast<const uint32_t *>(p.xs + static_cast<size_t>(token) * p.cols)[c];
      }
#pragma unroll
      for (uint32_t j = 0; j < 4u; ++j) {
        const uint32_t idx = base + j * S::kThreads + threadIdx.x;
        if (idx < total) reinterpret_cast<uint32_t *>(xsc)[idx] = v[j];
      }
    }
  } else {
    for (uint32_t idx = threadIdx.x; idx < S::TM * p.cols; idx += S::kThreads) {
      const uint32_t row = idx / p.cols, c = idx - row * p.cols;
      const uint32_t token = min(t0 + row, p.m - 1u);
      xsc[idx] = p.xs[static_cast<size_t>(token) * p.cols + c];
    }
  }
  const uint32_t nblk = (n + 127u) >> 7;
  for (uint32_t idx = threadIdx.x; idx < ((S::FN + 127) / 128) * p.cols; idx += S::kThreads) {
    const uint32_t b = idx / p.cols, c = idx - b * p.cols;
    const uint32_t blk = min((f0 >> 7) + b, nblk - 1u);
    if constexpr (MODE == WScaleMode::Float) {
      wsc[idx] = reinterpret_cast<const uint32_t *>(weight_scales)[static_cast<size_t>(blk) * p.cols + c];
    } else {
      wsc[idx] = reinterpret_cast<const uint8_t *>(weight_scales)[static_cast<size_t>(blk) * p.cols + c];
    }
  }
  __syncthreads();   // the tables; the stages are waited for by the K loop

  f32x4_t acc[1][S::NF][S::NT];
#pragma unroll
  for (int f = 0; f < S::NF; ++f) {
#pragma unroll
    for (int t = 0; t < S::NT; ++t) acc[0][f][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
  const uint32_t i = lane & 15u, g = lane >> 4;
  const uint32_t wf = wave % S::WAVES_F, wt = wave / S::WAVES_F;
  const uint8_t *my_xsc = xsc + (S::token_row(wt, 0) + i) * p.cols;
  const uint32_t *my_wsc = wsc + ((wf * S::NF * 16u) >> 7) * p.cols;
  auto x_scale = [&](int t, uint32_t kb) { return static_cast<uint32_t>(my_xsc[t * 16 * p.cols + kb]); };
  auto w_block_scale = [&](int, uint32_t kb) { return my_wsc[kb]; };
  if constexpr (S::NSTAGE >= 3) {
    // waves w and w + kWaves/2 share a SIMD: the second half of the waves runs half a K step behind
    if (wave >= static_cast<uint32_t>(S::kWaves / 2)) {
      gemm_mainloop<S, MODE, true, S::NT, false, 2>(acc, cur, stages, p.k >> 7, wave, lane, x_scale, w_block_scale);
    } else {
      gemm_mainloop<S, MODE, true, S::NT, false, 1>(acc, cur, stages, p.k >> 7, wave, lane, x_scale, w_block_scale);
    }
  } else {
    gemm_mainloop<S, MODE, true>(acc, cur, stages, p.k >> 7, wave, lane, x_scale, w_block_scale);
  }

#pragma unroll
  for (int t = 0; t < S::NT; ++t) {
    const uint32_t token = t0 + S::token_row(wt, t) + i;
    if (token >= p.m) continue;
#pragma unroll
    for (int f = 0; f < S::NF; ++f) {
      const uint32_t feat = f0 + (wf * S::NF + f) * 16u + g * 4u;
      const f32x4_t a = acc[0][f][t];
      const size_t at = static_cast<size_t>(token) * n + feat;
      if (feat + 3u < n && (n & 3u) == 0u) {
        if constexpr (OUT == kGemmOutBf16) {
          const uint32_t lo = bf16_rne_bits(a[0]) | (static_cast<uint32_t>(bf16_rne_bits(a[1])) << 16);
          const uint32_t hi = bf16_rne_bits(a[2]) | (static_cast<uint32_t>(bf16_rne_bits(a[3])) << 16);
          *reinterpret_cast<uint2 *>(reinterpret_cast<uint16_t *>(output) + at) = make_uint2(lo, hi);
        } else if constexpr (OUT == kGemmOutF32Rounded) {
          *reinterpret_cast<float4 *>(reinterpret_cast<float *>(output) + at) =
              make_float4(bf16_round(a[0]), bf16_round(a[1]), bf16_round(a[2]), bf16_round(a[3]));
        } else {
          float4 *dst = reinterpret_cast<float4 *>(reinterpret_cast<float *>(output) + at);
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
              reinterpret_cast<uint16_t *>(output)[at + v] = static_cast<uint16_t>(bf16_rne_bits(a[v]));
            } else if constexpr (OUT == kGemmOutF32Rounded) {
              reinterpret_cast<float *>(output)[at + v] = bf16_round(a[v]);
            } else if constexpr (OUT == kGemmOutF32Accumulate) {
              reinterpret_cast<float *>(output)[at + v] += a[v];
            } else {
              reinterpret_cast<float *>(output)[at + v] = a[v];
            }
          }
        }
      }
    }
  }
}

// Workgroups are dealt round-robin to the 8 XCDs (each with its own L2): blocks are renumbered so
// that one XCD gets a contiguous run of tiles.  Inside the run, tiles are ordered in panels of four
// token tiles (token tile fastest, then feature tile): the ~32 workgroups that run on an XCD at the
// same time then cover about 4 x 8 tiles and share both operands' K slices through that L2, instead
// of one weight tile and every token tile.  Blocks from `whole` on (none when Half is S) own a piece
// of a tile each, a half (along the tokens, shape Half) or a quarter (shape Quarter); the pieces of a
// tile are eight blocks apart, i.e. on the same XCD.
template <typename S, typename Half, typename Quarter, WScaleMode MODE, int OUT>
__global__ __launch_bounds__(S::kThreads) void fp8_block_gemm_kernel(Fp8GemmParams p, uint32_t whole, uint32_t pieces) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  if constexpr (std::is_same<S, Half>::value) {
    fp8_gemm_tile<S, MODE, OUT>(p, gemm_tile_of<S>(p, blockIdx.x), lds);
  } else {
    static_assert(Half::FN == S::FN && 2 * Half::TM == S::TM && 2 * Quarter::FN == S::FN && 2 * Quarter::TM == S::TM &&
                      Half::kThreads == S::kThreads && Quarter::kThreads == S::kThreads,
                  "two halves or four quarters cover one tile, run by the same workgroup size");
    if (blockIdx.x < whole) {
      fp8_gemm_tile<S, MODE, OUT>(p, gemm_tile_of<S>(p, blockIdx.x), lds);
      return;
    }
    // pieces in groups of 8 tiles (one per XCD) x pieces; a last group of fewer tiles keeps a tile's pieces side by side
    const uint32_t q = blockIdx.x - whole, per_group = 8u * pieces;
    const uint32_t group = q / per_group, i = q - group * per_group;
    const uint32_t cut_tiles = (gridDim.x - whole) / pieces;
    const bool complete = cut_tiles - group * 8u >= 8u;
    const uint32_t tile_index = group * 8u + (complete ? (i & 7u) : i / pieces);
    const uint32_t piece = complete ? (i >> 3) : i % pieces;
    GemmTile tile = gemm_tile_of<S>(p, whole + tile_index);
    if (pieces == 2u) {
      tile.t0 += piece * Half::TM;
      if (tile.t0 >= p.m) return;  // a ragged tile that ends inside its first half
      fp8_gemm_tile<Half, MODE, OUT>(p, tile, lds);
    } else {
      tile.t0 += (piece & 1u) * Quarter::TM;
      tile.f0 += (piece >> 1) * Quarter::FN;
      if (tile.t0 >= p.m || tile.f0 >= tile.n) return;
      fp8_gemm_tile<Quarter, MODE, OUT>(p, tile, lds);
    }
  }
}

constexpr uint32_t kMaxLds = 160u * 1024u;

template <typename S, typename Half, typename Quarter, WScaleMode MODE, int OUT>
hipError_t launch_shape(const Fp8GemmParams &p, hipStream_t stream) {
  constexpr bool kCanCut = !std::is_same<S, Half>::value;
  const uint32_t tiles = ((p.m + S::TM - 1) / S::TM) * ((p.n + S::FN - 1) / S::FN + (p.n2 + S::FN - 1) / S::FN);
  const uint32_t pieces = last_round_pieces(
      tiles, kCanCut && gemm_lds_bytes<Half>(p.cols) <= kMaxLds && gemm_lds_bytes<Quarter>(p.cols) <= kMaxLds);
  const uint32_t whole = pieces == 1u ? tiles : tiles - tiles % kCus;
  uint32_t lds = gemm_lds_bytes<S>(p.cols);
  if (pieces == 2u) lds = max(lds, gemm_lds_bytes<Half>(p.cols));
  if (pieces == 4u) lds = max(lds, gemm_lds_bytes<Quarter>(p.cols));
  auto kernel = fp8_block_gemm_kernel<S, Half, Quarter, MODE, OUT>;
  hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
  if (err != hipSuccess) return err;
  kernel<<<whole + pieces * (tiles - whole), S::kThreads, lds, stream>>>(p, whole, pieces);
  return hipSuccess;
}

template <WScaleMode MODE, int OUT>
hipError_t launch_mode(const Fp8GemmParams &p, hipStream_t stream) {
  // the large tile only when it still yields at least one workgroup per CU
  const uint64_t large_tiles =
      static_cast<uint64_t>((p.m + ShapeLarge::TM - 1) / ShapeLarge::TM) *
      ((p.n + ShapeLarge::FN - 1) / ShapeLarge::FN + (p.n2 + ShapeLarge::FN - 1) / ShapeLarge::FN);
  if (large_tiles >= kLargeMinTiles && gemm_lds_bytes<ShapeLarge>(p.cols) <= kMaxLds) {
    return launch_shape<ShapeLarge, ShapeLargeTail, ShapeSmall, MODE, OUT>(p, stream);
  }
  const uint64_t small_tiles =
      static_cast<uint64_t>((p.m + ShapeSmall::TM - 1) / ShapeSmall::TM) *
      ((p.n + ShapeSmall::FN - 1) / ShapeSmall::FN + (p.n2 + ShapeSmall::FN - 1) / ShapeSmall::FN);
  if (2u * small_tiles <= kCus && gemm_lds_bytes<ShapeNarrow>(p.cols) <= kMaxLds) {
    return launch_shape<ShapeNarrow, ShapeNarrow, ShapeNarrow, MODE, OUT>(p, stream);
  }
  return launch_shape<ShapeSmall, ShapeSmall, ShapeSmall, MODE, OUT>(p, stream);
}

bool aligned16(uint64_t address) { return address != 0 && (address & 15u) == 0; }

// capabilities/fp8_projection.cuh:67-97 plus what the LDS budget of this kernel adds
int32_t validate(uint32_t rows, uint32_t n, uint32_t k, uint32_t scale_cols, uint64_t a, uint64_t as, uint64_t w,
                 uint64_t ws, uint64_t out) {
  if (!aligned16(a) || !aligned16(as) || !aligned16(w) || !aligned16(ws) || !aligned16(out)) {
    return FERRULE_HIP_INVALID_ARGUMENT;
  }
  if (rows == 0 || rows > 8u * 65535u || n == 0 || k == 0 || (k & 127u) != 0 || scale_cols != k / 128u) {
    return FERRULE_HIP_INVALID_ARGUMENT;
  }
  if (gemm_lds_bytes<ShapeSmall>(scale_cols) > kMaxLds) return FERRULE_HIP_UNSUPPORTED;
  // one workgroup per tile on a 1-D grid (two matrices of one launch stay below 2^31 together)
  const uint64_t small_tiles = static_cast<uint64_t>((rows + ShapeSmall::TM - 1) / ShapeSmall::TM) *
                               ((static_cast<uint64_t>(n) + ShapeSmall::FN - 1) / ShapeSmall::FN);
  if (small_tiles > 0x3fffffffull) return FERRULE_HIP_UNSUPPORTED;
  return FERRULE_HIP_SUCCESS;
}

template <WScaleMode MODE>
hipError_t launch_out(const Fp8GemmParams &p, int out_mode, hipStream_t stream) {
  switch (out_mode) {
    case kGemmOutBf16: return launch_mode<MODE, kGemmOutBf16>(p, stream);
    case kGemmOutF32Raw: return launch_mode<MODE, kGemmOutF32Raw>(p, stream);
    case kGemmOutF32Accumulate: return launch_mode<MODE, kGemmOutF32Accumulate>(p, stream);
    default: return launch_mode<MODE, kGemmOutF32Rounded>(p, stream);
  }
}

}  // namespace

int32_t fp8_gemm_run(const Fp8GemmParams &p, bool f32_scales, int out_mode, uint64_t stream_bits, bool tiles_only) {
  if (!tiles_only && fp8_rows_applies(p.m, p.k)) return fp8_rows_run(p, f32_scales, out_mode, stream_bits);
  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(stream_bits));
  clear_launch_error();
  const hipError_t err = f32_scales ? launch_out<WScaleMode::Float>(p, out_mode, stream)
                                    : launch_out<WScaleMode::Byte>(p, out_mode, stream);
  if (err != hipSuccess) {
    g_last_hip_error = static_cast<int32_t>(err);
    return FERRULE_HIP_LAUNCH_FAILED;
  }
  return take_launch_error() == 0 ? FERRULE_HIP_SUCCESS : FERRULE_HIP_LAUNCH_FAILED;
}

uint32_t fp8_gemm_lds_bytes_small(uint32_t scale_cols) { return gemm_lds_bytes<ShapeSmall>(scale_cols); }

namespace {
int32_t run(const Fp8GemmParams &p, bool f32_scales, bool out_bf16, uint64_t stream_bits, bool tiles_only = false) {
  return fp8_gemm_run(p, f32_scales, out_bf16 ? kGemmOutBf16 : kGemmOutF32Rounded, stream_bits, tiles_only);
}
}  // namespace
}  // namespace ferrule_hip

using namespace ferrule_hip;

extern "C" int32_t ferrule_hip_fp8_block_gemm_can_implement(const FerruleHipFp8BlockGemmArgs *args) {
  if (args == nullptr) return FERRULE_HIP_INVALID_ARGUMENT;
  if (args->weight_scale_kind != FERRULE_HIP_SCALE_E8M0 && args->weight_scale_kind != FERRULE_HIP_SCALE_F32) {
    return FERRULE_HIP_INVALID_ARGUMENT;
  }
  if ((args->flags & ~(FERRULE_HIP_GEMM_OUTPUT_BF16 | FERRULE_HIP_GEMM_TILE_SCHEDULE)) != 0) {
    return FERRULE_HIP_INVALID_ARGUMENT;
  }
  return validate(args->rows, args->n, args->k, args->scale_cols, args->activation_fp8, args->activation_ue8m0,
                  args->weight_fp8, args->weight_scales, args->output);
}

extern "C" int32_t ferrule_hip_fp8_block_gemm_launch(const FerruleHipFp8BlockGemmArgs *args) {
  const int32_t status = ferrule_hip_fp8_block_gemm_can_implement(args);
  if (status != FERRULE_HIP_SUCCESS) return status;
  Fp8GemmParams p;
  p.x = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(args->activation_fp8));
  p.xs = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(args->activation_ue8m0));
  p.w = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(args->weight_fp8));
  p.ws = reinterpret_cast<const void *>(static_cast<uintptr_t>(args->weight_scales));
  p.out = reinterpret_cast<void *>(static_cast<uintptr_t>(args->output));
  p.m = args->rows;
  p.n = args->n;
  p.k = args->k;
  p.cols = args->scale_cols;
  return run(p, args->weight_scale_kind == FERRULE_HIP_SCALE_F32, (args->flags & FERRULE_HIP_GEMM_OUTPUT_BF16) != 0,
             args->stream, (args->flags & FERRULE_HIP_GEMM_TILE_SCHEDULE) != 0);
}

extern "C" int32_t ferrule_hip_fp8_query_a_kv_can_implement(const FerruleHipFp8QueryAKvArgs *args) {
  if (args == nullptr) return FERRULE_HIP_INVALID_ARGUMENT;
  const int32_t first = validate(args->rows, args->n1, args->k, args->scale_cols, args->activation_fp8,
                                 args->activation_ue8m0, args->query_a_weight_fp8, args->query_a_weight_ue8m0,
                                 args->query_a_output_f32);
  if (first != FERRULE_HIP_SUCCESS) return first;
  return validate(args->rows, args->n2, args->k, args->scale_cols, args->activation_fp8, args->activation_ue8m0,
                  args->kv_weight_fp8, args->kv_weight_ue8m0, args->kv_output_f32);
}

static int32_t launch_projection(const FerruleHipFp8QueryAKvArgs *args, bool second) {
  Fp8GemmParams p;
  p.x = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(args->activation_fp8));
  p.xs = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(args->activation_ue8m0));
  p.w = reinterpret_cast<const uint8_t *>(
      static_cast<uintptr_t>(second ? args->kv_weight_fp8 : args->query_a_weight_fp8));
  p.ws = reinterpret_cast<const void *>(
      static_cast<uintptr_t>(second ? args->kv_weight_ue8m0 : args->query_a_weight_ue8m0));
  p.out = reinterpret_cast<void *>(static_cast<uintptr_t>(second ? args->kv_output_f32 : args->query_a_output_f32));
  p.m = args->rows;
  p.n = second ? args->n2 : args->n1;
  p.k = args->k;
  p.cols = args->scale_cols;
  return run(p, false, false, args->stream);
}

extern "C" int32_t ferrule_hip_fp8_query_a_kv_launch(const FerruleHipFp8QueryAKvArgs *args) {
  const int32_t status = ferrule_hip_fp8_query_a_kv_can_implement(args);
  if (status != FERRULE_HIP_SUCCESS) return status;
  // both projections in ONE launch: the KV matrix's feature tiles follow QueryA's in the same grid,
  // so the two share the activation rows in L2 and fill the machine together
  Fp8GemmParams p;
  p.x = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(args->activation_fp8));
  p.xs = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(args->activation_ue8m0));
  p.w = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(args->query_a_weight_fp8));
  p.ws = reinterpret_cast<const void *>(static_cast<uintptr_t>(args->query_a_weight_ue8m0));
  p.out = reinterpret_cast<void *>(static_cast<uintptr_t>(args->query_a_output_f32));
  p.w2 = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(args->kv_weight_fp8));
  p.ws2 = reinterpret_cast<const void *>(static_cast<uintptr_t>(args->kv_weight_ue8m0));
  p.out2 = reinterpret_cast<void *>(static_cast<uintptr_t>(args->kv_output_f32));
  p.m = args->rows;
  p.n = args->n1;
  p.n2 = args->n2;
  p.k = args->k;
  p.cols = args->scale_cols;
  return run(p, false, false, args->stream);
}

// implementations/cutlass/entrypoints.cu:1234-1253
extern "C" int32_t ferrule_hip_fp8_projection_can_implement(const FerruleHipFp8QueryAKvArgs *args) {
  if (args == nullptr) return FERRULE_HIP_INVALID_ARGUMENT;
  if (args->n2 != 0u || args->kv_weight_fp8 != 0u || args->kv_weight_ue8m0 != 0u || args->kv_output_f32 != 0u ||
      args->scale_cols != args->k / 128u) {
    return FERRULE_HIP_INVALID_ARGUMENT;
  }
  return validate(args->rows, args->n1, args->k, args->scale_cols, args->activation_fp8, args->activation_ue8m0,
                  args->query_a_weight_fp8, args->query_a_weight_ue8m0, args->query_a_output_f32);
}

extern "C" int32_t ferrule_hip_fp8_projection_launch(const FerruleHipFp8QueryAKvArgs *args) {
  const int32_t status = ferrule_hip_fp8_projection_can_implement(args);
  if (status != FERRULE_HIP_SUCCESS) return status;
  return launch_projection(args, false);
}
