// Decode-row schedule of the FP8 x FP8 block-scaled GEMM: at most 32 activation rows.
//
// The reference's fp8_projection is a small-M kernel (grid (ceil(N/16), ceil(M/8)), hundreds of
// CTAs at one row; capabilities/fp8_projection.cuh:424-497) and "native providers own row-count
// schedule dispatch" (src/cuda/provider.rs:46-49).  The 128 x 128 MFMA tile of fp8_gemm.hip puts
// a 7168 x 7168 matrix on 56 workgroups when there is one row: the kernel is then bound by how few
// loads are in flight, not by HBM.  Here the problem is what it is at this size, a stream over
// the weights:
//
//   one wave = 16 weight rows (features) x all of K.  Per 128-wide K block the wave's two
//   16-byte loads per lane ARE the A operand of v_mfma_scale_f32_16x16x128_f8f6f4 (lane (i, g)
//   holds k [16g, 16g+16) and [64+16g, 64+16g+16) of row i); the B operand is the same two
//   pieces of activation row min(i, m-1), fetched from L2 (m x K bytes, shared by every wave); the
//   E8M0 scales of both ride in the instruction.  17 to 32 rows are two such MFMAs per K block
//   that share the weight operand.  A ring of kDepth K blocks of loads per wave is
//   in flight at any time; there is no LDS, no barrier, and nothing is shared between waves, so a
//   launch of N/16 single-wave workgroups spreads over every CU.
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

// Loads of any alignment (the scale bytes of four K blocks as one dword, four f32 scales as one
// 16-byte load): global memory takes them at full speed.
typedef uint32_t u32_any_t __attribute__((aligned(1)));
typedef uint32_t u32x4_any_t __attribute__((ext_vector_type(4), aligned(4)));
typedef const __attribute__((address_space(1))) u32_any_t *global_u32_any_ptr;
typedef const __attribute__((address_space(1))) u32x4_any_t *global_u32x4_any_ptr;

// Four consecutive K blocks of one wave: the weight rows, TT x 16 activation rows, their scales.
template <WScaleMode MODE, int TT>
struct RowsGroup {
  u32x4_t wlo[4], whi[4], xlo[TT][4], xhi[TT][4];
  uint32_t sx4[TT];  // activation scale bytes of K blocks sb .. sb+3 (sb = the group's first block, clamped)
  u32x4_t sw;        // Byte: [0] = the weight block scale bytes of the same four; Float: four f32 scales
};

// GROUPS groups of four K blocks are in flight per wave (8 + 8 TT payload and 1 + TT scale loads each:
// vmcnt is a 6-bit counter).  TT = 1: up to 16 activation rows; TT = 2: up to 32, as two MFMAs per K
// block that share the weight operand.
template <WScaleMode MODE, int OUT, int GROUPS, int TT, bool STREAM>
__global__ __launch_bounds__(64) void fp8_rows_kernel(RowsParams p) {
  constexpr uint32_t kDepth = 4u * GROUPS;
  static_assert(GROUPS * (9 + 9 * TT) <= 63, "vmcnt is a 6-bit counter");
  const uint32_t lane = threadIdx.x;
  const uint32_t i = lane & 15u, g = lane >> 4;
  // this lane's weight row
  uint32_t mat, f0, feature, n;
  if constexpr (OUT == kOutSwiGlu) {
    mat = i >> 3;   // rows 0-7: W1 (gate), rows 8-15: W3 (up)
    f0 = blockIdx.x * 8u;
    feature = f0 + (i & 7u);
    n = p.n[0];
  } else {
    const uint32_t tiles0 = (p.n[0] + 15u) >> 4;
    mat = blockIdx.x >= tiles0 ? 1u : 0u;   // wave-uniform
    f0 = (blockIdx.x - mat * tiles0) * 16u;
    feature = f0 + i;
    n = mat ? p.n[1] : p.n[0];
  }
  const uint32_t wrow = min(feature, n - 1u);
  const uint8_t *const wp = (mat ? p.w[1] : p.w[0]) + static_cast<size_t>(wrow) * p.k + g * 16u;
  const uint8_t *xp[TT], *xsp[TT];
#pragma unroll
  for (int t = 0; t < TT; ++t) {
    const uint32_t xrow = min(static_cast<uint32_t>(t) * 16u + i, p.m - 1u);
    xp[t] = p.x + static_cast<size_t>(xrow) * p.k + g * 16u;
    xsp[t] = p.xs + static_cast<size_t>(xrow) * p.cols;
  }
  const uint8_t *const wsp = static_cast<const uint8_t *>(mat ? p.ws[1] : p.ws[0]) +
                             static_cast<size_t>(wrow >> 7) * p.cols * (MODE == WScaleMode::Float ? 4u : 1u);
  const uint32_t nk = p.k >> 7;

  // First scale column of the group that starts at K block kb0: the four scales are fetched as one
  // window that must end inside the row.
  auto scale_base = [&](uint32_t kb0) { return min(kb0, nk - 4u); };
  // Loads of K blocks kb0 .. kb0+3.  Beyond the last K block the payload loads read the start of
  // the activation row instead (valid, cached, never used): a group always issues the same
  // loads, none of them in a branch, so the compiler's wait counts stay exact.
  auto fill = [&](RowsGroup<MODE, TT> &s, uint32_t kb0) {
    const uint32_t sb = scale_base(kb0);
#pragma unroll
    for (int t = 0; t < TT; ++t) s.sx4[t] = *(global_u32_any_ptr)(xsp[t] + sb);
    if constexpr (MODE == WScaleMode::Float) {
      s.sw = *(global_u32x4_any_ptr)(wsp + static_cast<size_t>(sb) * 4u);
    } else {
      s.sw[0] = *(global_u32_any_ptr)(wsp + sb);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t kb = kb0 + static_cast<uint32_t>(j);
      const bool live = kb < nk;
      const size_t at = live ? static_cast<size_t>(kb) * 128u : 0u;
#pragma unroll
      for (int t = 0; t < TT; ++t) {
        s.xlo[t][j] = load16(xp[t] + at);
        s.xhi[t][j] = load16(xp[t] + at + 64u);
      }
      const uint8_t *wsrc = live ? wp + at : xp[0];
      s.wlo[j] = STREAM ? load_stream16(wsrc) : load16(wsrc);
      s.whi[j] = STREAM ? load_stream16(wsrc + 64u) : load16(wsrc + 64u);
    }
  };

  f32x4_t acc[TT];
#pragma unroll
  for (int t = 0; t < TT; ++t) acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  // K block j of a group; `sel` = its position in the group's scale window
  auto consume = [&](const RowsGroup<MODE, TT> &s, int j, uint32_t sel) {
    const i32x8_t wa = make_b_fp8(s.wlo[j], s.whi[j]);
#pragma unroll
    for (int t = 0; t < TT; ++t) {
      const i32x8_t xb = make_b_fp8(s.xlo[t][j], s.xhi[t][j]);
      const int sx = static_cast<int>(s.sx4[t] >> (8u * sel));   // the instruction takes byte 0
      if constexpr (MODE == WScaleMode::Float) {
        // f32 weight scales cannot ride in the instruction: a fresh product per K block, folded
        // with one v_fma per value (the tiled kernel's arithmetic)
        const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
        const f32x4_t fresh = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wa, xb, zero, kMfmaFmtFp8,
                                                                               kMfmaFmtFp8, 0, 127, 0, sx);
        const uint32_t bits = sel == 0u ? s.sw[0] : sel == 1u ? s.sw[1] : sel == 2u ? s.sw[2] : s.sw[3];
        const float ws = __uint_as_float(bits);
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[t][v] = fmaf(fresh[v], ws, acc[t][v]);
      } else {
        acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wa, xb, acc[t], kMfmaFmtFp8, kMfmaFmtFp8, 0,
                                                                  static_cast<int>(s.sw[0] >> (8u * sel)), 0, sx);
      }
    }
  };

  RowsGroup<MODE, TT> ring[GROUPS];
#pragma unroll
  for (int r = 0; r < GROUPS; ++r) {
    // in ring order: loads return in the order of issue, and group 0 is needed first
    fill(ring[r], 4u * r);
    __builtin_amdgcn_sched_barrier(0);
  }
  uint32_t kb0 = 0;
  for (; kb0 + kDepth <= nk; kb0 += kDepth) {   // whole rings
#pragma unroll
    for (int r = 0; r < GROUPS; ++r) {
#pragma unroll
      for (int j = 0; j < 4; ++j) consume(ring[r], j, static_cast<uint32_t>(j));
      __builtin_amdgcn_sched_barrier(0);
      fill(ring[r], kb0 + 4u * r + kDepth);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  // what is left of K: fewer than kDepth blocks, all of them in the ring
#pragma unroll
  for (int r = 0; r < GROUPS; ++r) {
    const uint32_t first = kb0 + 4u * r;
    const uint32_t sb = scale_base(first);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (first + j < nk) consume(ring[r], j, first + j - sb);
    }
  }

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
      if (g >= 2u || token >= p.m) continue;
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
      if (token >= p.m) continue;
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

// Measured on N = K = 7168 (one row / sixteen rows, kernel alone): 2, 3, 4 groups with plain loads
// 11.4 / 11.1 / 11.7 us and 16.7 / 16.0 / 16.8 us; with nontemporal weight loads 13.1 / 13.0 / 13.4 us
// and 18.2 / 17.4 / 18.3 us (a wave load covers 16 rows x 64 bytes here, and half a cache line per row
// is the pattern on which the nontemporal hint costs bandwidth instead of saving it).
constexpr int kGroups = 3;       // up to 16 rows: 12 K blocks (24 KB of weights) in flight per wave
constexpr int kGroupsWide = 2;   // 17 to 32 rows: 8 K blocks (twice the activation registers per block)
constexpr bool kStream = false;  // plain weight loads

template <WScaleMode MODE, int OUT>
void launch_rows_out(const RowsParams &p, uint32_t grid, hipStream_t stream) {
  if (p.m <= 16u) {
    fp8_rows_kernel<MODE, OUT, kGroups, 1, kStream><<<grid, 64, 0, stream>>>(p);
  } else {
    fp8_rows_kernel<MODE, OUT, kGroupsWide, 2, kStream><<<grid, 64, 0, stream>>>(p);
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
