// Drop-in for ferrule_cutlass_hc_producer_{can_implement,launch}
// (abi/cutlass_provider.h:76-106, 403-406; kernel
// implementations/cutlass/capabilities/hyper_connection.cuh:30-75, 505-743): the producer of
// the FP8 activations that the GEMMs of a layer read.  Per token row, in one launch:
//   mix[24]        = function[24, 4*H] . state[4*H]                   (raw dot products)
//   rms            = 1 / sqrt(mean(state^2) + hc_norm_eps)
//   pre, post, comb= sigmoid / softmax + Sinkhorn split of mix * rms  (hyper_connection.rs:175-262)
//   hidden[H]      = sum_copy pre[copy] * state[copy]                 (hyper_connection.rs:300-309)
//   normalized[H]  = hidden * 1/sqrt(mean(hidden^2) + layer_rms_eps) * weight   (math.rs:22-42)
//   packed, scales = FP8-E4M3 bytes with one E8M0 scale per 128 values  (encoding.rs:207-242)
// The arithmetic is the CPU chain's (layer.rs:416-422): products and sums in f32, no BF16
// rounding between the stages, the CPU quantiser's tie rule.  `reserved` = 1 selects the CUDA
// provider's variant instead, which rounds hidden and normalized to BF16
// (hyper_connection.cuh:626, 653).  Sums run in another order than either reference (the CUDA
// provider hands the dot products to a library GEMM whose order is unspecified as well).
//
// Two launches, like the reference (a library GEMM, then one kernel), none of them a library call:
//   hc_mix_kernel       the 24 dot products per row on the FP32 MFMA (v_mfma_f32_32x32x2_f32:
//                       exact f32 products, f32 accumulation).  A workgroup owns 32 token rows
//                       and one slice of K; its four waves split the slice and add their 32x32
//                       tiles through LDS.  Every lane streams 64 contiguous bytes of its row per
//                       step, so state rows are fetched in whole 128-byte lines.  With few rows K
//                       is cut into up to 64 slices so that a decode batch still spreads the
//                       1.5 MB function matrix over many CUs; slice partials go to the caller's
//                       workspace (the reference's contract sizes it for 64 partials per value,
//                       hyper_connection.cuh:480-483) and are added in slice order, so results do
//                       not depend on scheduling.
//   hc_producer_kernel  one workgroup per row keeps the whole state row (4*H floats: 64 KB at
//                       H = 4096) in registers - thread t owns dimensions 4t..4t+3 of every
//                       1024-wide slice, of all four copies - so the sums of squares, the split,
//                       the weighted copy sum, RMSNorm and the quantiser all work from registers
//                       and the row is read once.  A 128-value quantisation block is 32 adjacent
//                       lanes: its maximum is four DPP steps and one cross-row shuffle.
// (A first version computed the dot products in the row kernel as well, streaming the function
// matrix from L2 once per row pair: 461 us for 8192 rows, bound by that L2 stream at one wave per
// SIMD.)
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <initializer_list>

#include "../../include/ferrule_hip_provider.h"
#include "numeric.cuh"
#include "quant_math.h"

namespace ferrule_hip {
namespace {

constexpr uint32_t kHc = 4;
constexpr uint32_t kMix = 24;
constexpr uint32_t kThreads = 256;
constexpr uint32_t kSlice = 1024;  // dimensions covered by one float4 per thread

typedef float f32x4v __attribute__((ext_vector_type(4)));

template <typename T>
__device__ __forceinline__ T *ptr(uint64_t address) {
  return global_ptr<T>(address);
}

// hyper_connection.rs:425-427
__device__ __forceinline__ float hc_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __uint_as_float(static_cast<uint32_t>(
      __builtin_amdgcn_update_dpp(0, static_cast<int>(__float_as_uint(v)), CTRL, 0xf, 0xf, false)));
}

// One row's split (hyper_connection.rs:175-262) by the first wave of the workgroup: lane l < 24
// holds mix[l], so lanes 0-3 make pre, 4-7 post, and lanes 8-23 are the 4x4 comb matrix, one row
// per quad.  Row sums fetch their four terms with quad broadcasts, column sums with shuffles,
// and add them in index order, as the CPU loops do.  (One thread doing all of it took about 9 us per row: 24
// exponentials and 150 divisions in one dependent chain, with the other waves at a barrier.)
__device__ __forceinline__ void split_sinkhorn_wave(uint32_t lane, float raw, float rms, const float *scale,
                                                    const float *base, float eps, uint32_t iters, bool live,
                                                    float *pre_lds, float *pre, float *post, float *comb_out) {
#pragma clang fp contract(off)  // the CPU rounds every multiply and add separately
  const uint32_t l = min(lane, kMix - 1u);
  const float mix = raw * rms;
  const float affine = mix * scale[l < kHc ? 0u : (l < 2u * kHc ? 1u : 2u)] + base[l];
  if (lane < 2u * kHc) {
    const float sig = hc_sigmoid(affine);
    if (lane < kHc) {
      const float p = sig + eps;
      pre_lds[lane] = p;
      if (live) pre[lane] = p;
    } else if (live) {
      post[lane - kHc] = 2.0f * sig;
    }
  }
  // comb: every lane runs the shuffles, only lanes 8..23 hold meaningful values
  const int col = static_cast<int>(lane & 3u);
  // a comb row is a quad of lanes: its four terms arrive by quad broadcasts (DPP), in column order
  float row_max = fmaxf(fmaxf(dpp_f32<0x00>(affine), dpp_f32<0x55>(affine)), fmaxf(dpp_f32<0xaa>(affine), dpp_f32<0xff>(affine)));
  float value = expf(affine - row_max);
  float sum = dpp_f32<0x00>(value);
  sum += dpp_f32<0x55>(value);
  sum += dpp_f32<0xaa>(value);
  sum += dpp_f32<0xff>(value);
  value = value / sum + eps;
  for (uint32_t iteration = 0; iteration < iters; ++iteration) {
    if (iteration > 0) {
      sum = dpp_f32<0x00>(value);
      sum += dpp_f32<0x55>(value);
      sum += dpp_f32<0xaa>(value);
      sum += dpp_f32<0xff>(value);
      value /= sum + eps;
    }
    sum = __shfl(value, 8 + col, 64);
#pragma unroll
    for (int r = 1; r < 4; ++r) sum += __shfl(value, 8 + 4 * r + col, 64);
    value /= sum + eps;
  }
  if (live && lane >= 2u * kHc && lane < kMix) comb_out[lane - 2u * kHc] = value;
}


// Sum of one value per thread over the workgroup's 256 threads, the same bits in every thread:
// four DPP steps leave every row of 16 lanes with its sum, the 16 row sums meet in LDS and are
// added in index order.  `slots` is 16 floats.
__device__ __forceinline__ float block_sum_scalar(float v, float *slots) {
  v += dpp_f32<0xb1>(v);
  v += dpp_f32<0x4e>(v);
  v += dpp_f32<0x141>(v);
  v += dpp_f32<0x140>(v);
  if ((threadIdx.x & 15u) == 0u) slots[threadIdx.x >> 4] = v;
  __syncthreads();
  float sum = 0.0f;
#pragma unroll
  for (uint32_t i = 0; i < kThreads / 16u; ++i) sum += slots[i];
  __syncthreads();
  return sum;
}

// maximum over the 32 adjacent lanes that hold one 128-value block
__device__ __forceinline__ float max_over_32_lanes(float v) {
  v = fmaxf(v, dpp_f32<0xb1>(v));   // quad_perm [1,0,3,2]
  v = fmaxf(v, dpp_f32<0x4e>(v));   // quad_perm [2,3,0,1]
  v = fmaxf(v, dpp_f32<0x141>(v));  // row_half_mirror
  v = fmaxf(v, dpp_f32<0x140>(v));  // row_mirror
  return fmaxf(v, __shfl_xor(v, 16, 64));
}

typedef float f32x16v __attribute__((ext_vector_type(16)));

// Raw dot products of 32 token rows with the 24 function rows over one slice of K, on the FP32
// MFMA.  v_mfma_f32_32x32x2_f32 takes A[i][k] from lane (i = l % 32, k = l / 32), B[k][j] from
// lane (j = l % 32, k = l / 32) and leaves D[8 * (v / 4) + 4 * (l / 32) + v % 4][l % 32] in
// register v.  Here i = function row (24 of 32 used, the rest repeat row 23 and are dropped),
// j = token row; lane (row, half) holds 16 consecutive k at offset 16 * half of a 32-wide step and
// the e-th instruction of a step multiplies element e of both halves - any pairing of k values
// is valid as long as A and B use the same one.
//
// Operands go through LDS so that memory is read in whole kilobytes: K advances in chunks of 256
// floats, a wave-wide load instruction fetches 1 KB of ONE row (eight token rows and six function
// rows per wave and chunk), the chunk is written to LDS with a row stride of 260 words (the
// 16-byte fragment reads of eight consecutive rows then cover all 32 banks) and each wave
// multiplies two of the chunk's eight 32-wide steps.  The next chunk's loads are in flight in
// registers meanwhile.  Reading the operands straight from memory in MFMA layout (32 rows x
// 128 bytes per wave load) reached 2.6 TB/s whatever the order of the steps.
// Chunk c of slice y is global chunk c * ksplit + y, so the slices of a tile, adjacent in dispatch
// order, work side by side on the same rows.
// KC = floats of K per chunk: 256 (1 KB per row and load, two workgroups per CU by LDS; used) or 128
// (two rows of 512 B per load, five workgroups per CU; measured no faster: 150 against 146 us).
template <uint32_t KC>
__global__ __launch_bounds__(kThreads) void hc_mix_kernel(FerruleHipHcProducerArgs a, float *partials, uint32_t ksplit) {
  constexpr uint32_t kChunk = KC, kPad = KC + 4u;
  constexpr uint32_t kLanesPerRow = KC / 4u, kRowsPerLoad = 64u / kLanesPerRow;
  constexpr int kStateLoads = 8 / kRowsPerLoad, kFunctionLoads = 6 / kRowsPerLoad, kStepsPerWave = KC / 128u;
  __shared__ __attribute__((aligned(16))) float st[32 * kPad];
  __shared__ __attribute__((aligned(16))) float fn[kMix * kPad];
  const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
  const uint32_t column = lane & 31u, half = lane >> 5;
  const uint32_t k_total = kHc * a.hidden;
  const uint32_t my_chunks = k_total / (kChunk * ksplit);  // whole by the choice of ksplit
  const uint32_t slice = blockIdx.x, tile = blockIdx.y;

  const float *srow[kStateLoads], *frow[kFunctionLoads];
  const uint32_t sub_row = lane / kLanesPerRow, sub_col = 4u * (lane % kLanesPerRow);
#pragma unroll
  for (int i = 0; i < kStateLoads; ++i) {
    const uint32_t token = min(tile * 32u + 8u * wave + static_cast<uint32_t>(i) * kRowsPerLoad + sub_row, a.rows - 1u);
    srow[i] = ptr<const float>(a.state_f32) + static_cast<size_t>(token) * k_total + sub_col;
  }
#pragma unroll
  for (int i = 0; i < kFunctionLoads; ++i) {
    frow[i] = ptr<const float>(a.function_row_major_f32) + static_cast<size_t>(6u * wave + static_cast<uint32_t>(i) * kRowsPerLoad + sub_row) * k_total + sub_col;
  }
  f32x4v rs[kStateLoads], rf[kFunctionLoads];  // native vectors: arrays of HIP's float4 class stayed in scratch memory
  {
    const uint32_t k0 = slice * kChunk;
#pragma unroll
    for (int i = 0; i < kStateLoads; ++i) rs[i] = *reinterpret_cast<const f32x4v *>(srow[i] + k0);
#pragma unroll
    for (int i = 0; i < kFunctionLoads; ++i) rf[i] = *reinterpret_cast<const f32x4v *>(frow[i] + k0);
  }

  f32x16v acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
  const float *a_frag = fn + min(column, kMix - 1u) * kPad + 16u * half;
  const float *b_frag = st + column * kPad + 16u * half;
  for (uint32_t c = 0; c < my_chunks; ++c) {
#pragma unroll
    for (int i = 0; i < kStateLoads; ++i) *reinterpret_cast<f32x4v *>(st + (8u * wave + static_cast<uint32_t>(i) * kRowsPerLoad + sub_row) * kPad + sub_col) = rs[i];
#pragma unroll
    for (int i = 0; i < kFunctionLoads; ++i) *reinterpret_cast<f32x4v *>(fn + (6u * wave + static_cast<uint32_t>(i) * kRowsPerLoad + sub_row) * kPad + sub_col) = rf[i];
    __syncthreads();
    {
      // the next chunk's loads fly under this chunk's MFMAs; the last round reloads its own chunk
      const uint32_t k0 = (min(c + 1u, my_chunks - 1u) * ksplit + slice) * kChunk;
#pragma unroll
      for (int i = 0; i < kStateLoads; ++i) rs[i] = *reinterpret_cast<const f32x4v *>(srow[i] + k0);
#pragma unroll
      for (int i = 0; i < kFunctionLoads; ++i) rf[i] = *reinterpret_cast<const f32x4v *>(frow[i] + k0);
    }
#pragma unroll
    for (uint32_t ss = 0; ss < kStepsPerWave; ++ss) {
      const uint32_t k = 32u * (kStepsPerWave * wave + ss);
#pragma unroll
      for (uint32_t q = 0; q < 4; ++q) {
        const f32x4v fa = *reinterpret_cast<const f32x4v *>(a_frag + k + 4u * q);
        const f32x4v fb = *reinterpret_cast<const f32x4v *>(b_frag + k + 4u * q);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[0], fb[0], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[1], fb[1], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[2], fb[2], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[3], fb[3], acc, 0, 0, 0);
      }
    }
    __syncthreads();  // everybody has left the chunk before it is overwritten
  }
  // the four waves' 32x32 tiles, added through LDS (the token tile's storage is free now)
  float *tiles = st;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const uint32_t out = 8u * (static_cast<uint32_t>(v) >> 2) + 4u * half + (static_cast<uint32_t>(v) & 3u);
    tiles[wave * 1024u + out * 32u + column] = acc[v];
  }
  __syncthreads();
  for (uint32_t index = threadIdx.x; index < kMix * 32u; index += kThreads) {
    const uint32_t out = index >> 5, row = tile * 32u + (index & 31u);
    if (row < a.rows) {
      const float sum = (tiles[index] + tiles[1024u + index]) + (tiles[2048u + index] + tiles[3072u + index]);
      partials[(static_cast<size_t>(slice) * a.rows + row) * kMix + out] = sum;
    }
  }
}

// NJ = hidden / 1024.  `partials` holds ksplit slices of [rows, 24] raw dot products (it is
// mix_f32 itself when ksplit is 1).
template <int NJ>
__global__ __launch_bounds__(kThreads) void hc_producer_kernel(FerruleHipHcProducerArgs a, const float *partials,
                                                               uint32_t ksplit) {
#pragma clang fp contract(off)  // the CPU rounds every multiply and add separately
  constexpr int R = 1;  // rows per workgroup
  __shared__ __attribute__((aligned(16))) float lds[16u + kMix + kHc + 8u * kMix];
  constexpr uint32_t kHidden = NJ * kSlice;
  constexpr uint32_t kHcHidden = kHc * kHidden;
  float *partial = lds;          // [16]: block_sum_scalar's slots
  float *dots = partial + 16u;    // [24]
  float *pre_lds = dots + kMix;   // [4]
  float *group_sums = pre_lds + kHc;  // [8][24]

  const uint32_t t = threadIdx.x;
  const uint32_t row0 = blockIdx.x * R;
  const bool bf16_boundaries = (a.reserved & 1u) != 0u;
  const float *state = ptr<const float>(a.state_f32);

  // the rows' state, read once; a row beyond the problem repeats the last one and stores nothing
  float4 s[R][kHc][NJ];
  uint32_t row_of[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    row_of[r] = min(row0 + r, a.rows - 1u);
    const float *base = state + static_cast<size_t>(row_of[r]) * kHcHidden + 4u * t;
#pragma unroll
    for (uint32_t c = 0; c < kHc; ++c) {
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const f32x4v v = __builtin_nontemporal_load(reinterpret_cast<const f32x4v *>(base + c * kHidden + j * kSlice));
        s[r][c][j] = make_float4(v[0], v[1], v[2], v[3]);
      }
    }
  }

  // the row's 24 raw dot products: the slice partials (at most 64) are fetched by 192 threads at
  // once, eight independent loads each, and added in a fixed order (slices g, g + 8, ... per
  // group g, then the groups); one thread per value walking the slices cost a load latency per
  // slice, 10 us at 64 slices
  if (t < kMix * 8u) {
    const uint32_t value = t % kMix, group = t / kMix;
    float part[8];
#pragma unroll
    for (uint32_t i = 0; i < 8; ++i) {
      const uint32_t slice = group + 8u * i;
      part[i] = slice < ksplit ? partials[(static_cast<size_t>(slice) * a.rows + row_of[0]) * kMix + value] : 0.0f;
    }
    float sum = part[0];
#pragma unroll
    for (uint32_t i = 1; i < 8; ++i) sum += part[i];
    group_sums[group * kMix + value] = sum;
  }
  __syncthreads();
  if (t < kMix) {
    float sum = group_sums[t];
#pragma unroll
    for (uint32_t g = 1; g < 8; ++g) sum += group_sums[g * kMix + t];
    dots[t] = sum;
  }

  float squares[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    float sum = 0.0f;
#pragma unroll
    for (uint32_t c = 0; c < kHc; ++c) {
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const float4 v = s[r][c][j];
        sum += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
      }
    }
    squares[r] = sum;
  }
  const float state_squares = block_sum_scalar(squares[0], partial);

  // the first wave turns the 24 dots into the split
  if (t < 64u) {
    const bool live = row0 < a.rows;
    const uint32_t row = row_of[0];
    const float raw = dots[min(t, kMix - 1u)];
    if (live && t < kMix) ptr<float>(a.mix_f32)[static_cast<size_t>(row) * kMix + t] = raw;
    // rms_factor, hyper_connection.rs:416-419
    const float rms = 1.0f / sqrtf(state_squares / static_cast<float>(kHcHidden) + a.hc_norm_eps);
    split_sinkhorn_wave(t, raw, rms, ptr<const float>(a.hc_scale_f32), ptr<const float>(a.hc_base_f32), a.hc_eps,
                        a.sinkhorn_iters, live, pre_lds, ptr<float>(a.split_pre_f32) + static_cast<size_t>(row) * kHc,
                        ptr<float>(a.split_post_f32) + static_cast<size_t>(row) * kHc,
                        ptr<float>(a.split_comb_f32) + static_cast<size_t>(row) * kHc * kHc);
  }
  __syncthreads();

  // hidden = sum over copies of pre * state, multiply and add rounded separately as on the CPU
  // (contraction is off in this function)
  float4 h[R][NJ];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      float4 out = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
      for (uint32_t c = 0; c < kHc; ++c) {
        const float w = pre_lds[r * kHc + c];
        out.x = out.x + w * s[r][c][j].x;
        out.y = out.y + w * s[r][c][j].y;
        out.z = out.z + w * s[r][c][j].z;
        out.w = out.w + w * s[r][c][j].w;
      }
      if (bf16_boundaries) out = make_float4(bf16_round(out.x), bf16_round(out.y), bf16_round(out.z), bf16_round(out.w));
      h[r][j] = out;
      sum += out.x * out.x + out.y * out.y + out.z * out.z + out.w * out.w;
      if (row0 + r < a.rows) {
        const f32x4v packed_out = {out.x, out.y, out.z, out.w};
        __builtin_nontemporal_store(packed_out, reinterpret_cast<f32x4v *>(ptr<float>(a.hidden_f32) + static_cast<size_t>(row0 + r) * kHidden + j * kSlice + 4u * t));
      }
    }
    squares[r] = sum;
  }
  const float hidden_squares = block_sum_scalar(squares[0], partial);

  // RMSNorm with the layer weight, then the FP8-K128 quantiser
  const float *weight = ptr<const float>(a.layer_rms_weight_f32);
#pragma unroll
  for (int r = 0; r < R; ++r) {
    // math.rs:34-36: (sum / len + eps).sqrt().recip()
    const float scale = 1.0f / sqrtf(hidden_squares / static_cast<float>(kHidden) + a.layer_rms_eps);
    const bool live = row0 + r < a.rows;
    const size_t out_row = static_cast<size_t>(row0 + r);
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const uint32_t d = j * kSlice + 4u * t;
      const float4 w = *reinterpret_cast<const float4 *>(weight + d);
      float4 n;
      n.x = h[r][j].x * scale * w.x;
      n.y = h[r][j].y * scale * w.y;
      n.z = h[r][j].z * scale * w.z;
      n.w = h[r][j].w * scale * w.w;
      if (bf16_boundaries) n = make_float4(bf16_round(n.x), bf16_round(n.y), bf16_round(n.z), bf16_round(n.w));
      // encoding.rs:207-242: block maximum floored at 1e-4, power-of-two scale, nearest E4M3
      float amax = fmaxf(fmaxf(fabsf(n.x), fabsf(n.y)), fmaxf(fabsf(n.z), fabsf(n.w)));
      amax = fmaxf(max_over_32_lanes(amax), 1.0e-4f);
      uint32_t byte = 127u;  // a non-finite maximum keeps the unit scale (hyper_connection.cuh:193-196)
      if (amax <= 3.4028234e38f) byte = ferrule_quant::scale_byte(amax, 448.0f);
      // byte lies in [105, 247] or is 127: the scale has an exact f32 inverse
      const uint32_t codes = e4m3_bytes_exact(n.x, n.y, n.z, n.w, ferrule_quant::e8m0_inverse(byte),
                                              FERRULE_HIP_FP8_ROUND_CPU_REFERENCE);
      if (live) {
        const f32x4v packed_n = {n.x, n.y, n.z, n.w};
        __builtin_nontemporal_store(packed_n, reinterpret_cast<f32x4v *>(ptr<float>(a.normalized_f32) + out_row * kHidden + d));
        __builtin_nontemporal_store(codes, reinterpret_cast<uint32_t *>(ptr<uint8_t>(a.packed_e4m3) + out_row * kHidden + d));
        if ((t & 31u) == 0u) ptr<uint8_t>(a.scales_ue8m0)[out_row * (kHidden / 128u) + (d >> 7)] = static_cast<uint8_t>(byte);
      }
    }
  }
}

bool aligned16(uint64_t address) { return address != 0 && (address & 15u) == 0; }

FerruleHipStatus validate(const FerruleHipHcProducerArgs &a) {
  // hyper_connection.cuh:461-496, with the hidden size free in steps of 1024 and no workspace
  if (a.rows == 0 || a.rows > 32u * 65535u || a.hc != kHc || a.mix != kMix || a.reserved > 1u || a.sinkhorn_iters == 0) {
    return FERRULE_HIP_INVALID_ARGUMENT;
  }
  const bool finite = a.hc_eps > 0.0f && a.hc_eps <= 3.4028234e38f && a.hc_norm_eps > 0.0f &&
                      a.hc_norm_eps <= 3.4028234e38f && a.layer_rms_eps >= 0.0f && a.layer_rms_eps <= 3.4028234e38f;
  if (!finite) return FERRULE_HIP_INVALID_ARGUMENT;
  for (uint64_t p : {a.state_f32, a.function_row_major_f32, a.hc_scale_f32, a.hc_base_f32, a.layer_rms_weight_f32,
                     a.mix_f32, a.hidden_f32, a.normalized_f32, a.packed_e4m3, a.scales_ue8m0, a.split_pre_f32,
                     a.split_post_f32, a.split_comb_f32}) {
    if (!aligned16(p)) return FERRULE_HIP_INVALID_ARGUMENT;
  }
  if (a.hidden == 0 || a.hidden % kSlice != 0 || a.hidden > 8u * kSlice) return FERRULE_HIP_UNSUPPORTED;
  return FERRULE_HIP_SUCCESS;
}

// K slices of the mix kernel: enough workgroups to give every CU four, a power of two up to 64 that
// gives every slice whole 256-wide chunks, within what the caller's workspace holds.
uint32_t choose_ksplit(const FerruleHipHcProducerArgs &a) {
  const uint32_t tiles = (a.rows + 31u) / 32u;
  const uint32_t chunks = kHc * a.hidden / 256u;
  uint32_t ksplit = 1;
  while (ksplit < 64u && chunks % (ksplit * 2u) == 0u && tiles * ksplit < 1024u) ksplit *= 2u;
  const uint64_t per_slice = static_cast<uint64_t>(a.rows) * kMix * sizeof(float);
  while (ksplit > 1u && (a.workspace == 0 || (a.workspace & 15u) != 0 || per_slice * ksplit > a.workspace_bytes)) {
    ksplit /= 2u;
  }
  return ksplit;
}

template <int NJ>
void launch_rows(const FerruleHipHcProducerArgs &a, hipStream_t stream) {
  const uint32_t ksplit = choose_ksplit(a);
  float *partials = reinterpret_cast<float *>(static_cast<uintptr_t>(ksplit > 1u ? a.workspace : a.mix_f32));
  // slices of one tile are adjacent in dispatch order: they run at the same time on the same rows
  hc_mix_kernel<256><<<dim3(ksplit, (a.rows + 31u) / 32u), kThreads, 0, stream>>>(a, partials, ksplit);
  hc_producer_kernel<NJ><<<a.rows, kThreads, 0, stream>>>(a, partials, ksplit);
}

}  // namespace
}  // namespace ferrule_hip

extern "C" int32_t ferrule_hip_hc_producer_can_implement(const FerruleHipHcProducerArgs *args) {
  if (args == nullptr) return FERRULE_HIP_INVALID_ARGUMENT;
  return ferrule_hip::validate(*args);
}

extern "C" int32_t ferrule_hip_hc_producer_launch(const FerruleHipHcProducerArgs *args) {
  using namespace ferrule_hip;
  if (args == nullptr) return FERRULE_HIP_INVALID_ARGUMENT;
  const FerruleHipStatus status = validate(*args);
  if (status != FERRULE_HIP_SUCCESS) return status;
  const FerruleHipHcProducerArgs &a = *args;
  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(a.stream));
  clear_launch_error();
  switch (a.hidden / kSlice) {
    case 1: launch_rows<1>(a, stream); break;
    case 2: launch_rows<2>(a, stream); break;
    case 3: launch_rows<3>(a, stream); break;
    case 4: launch_rows<4>(a, stream); break;
    case 5: launch_rows<5>(a, stream); break;
    case 6: launch_rows<6>(a, stream); break;
    case 7: launch_rows<7>(a, stream); break;
    default: launch_rows<8>(a, stream); break;
  }
  return take_launch_error() == 0 ? FERRULE_HIP_SUCCESS : FERRULE_HIP_LAUNCH_FAILED;
}
