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
// The reference is a library GEMM followed by one kernel that reads the state a second time.
// Here a workgroup keeps the whole state row (4*H floats: 64 KB at H = 4096) in registers -
// thread t owns dimensions 4t..4t+3 of every 1024-wide slice, of all four copies - so the
// state is read from HBM exactly once and every later stage (both sums of squares, the mix,
// the weighted copy sum, RMSNorm, the quantiser) works from registers.  The function matrix
// (24 x 4*H floats, 1.5 MB at H = 4096) is shared by all rows and streams from L2; with two
// rows per workgroup every 16-byte piece of it feeds eight FMAs.  A 128-value quantisation
// block is 32 adjacent lanes: its maximum is four DPP steps and one cross-row shuffle.
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
  return reinterpret_cast<T *>(static_cast<uintptr_t>(address));
}

// Sum over the workgroup's 256 threads of `count` values per thread; partial[thread][count]
// in LDS, result[count] in LDS.  Thread t < 4 * count adds one quarter of one value's
// partials, consecutive lanes reading consecutive words.
template <uint32_t COUNT>
__device__ __forceinline__ void block_sum(const float (&mine)[COUNT], float *partial, float *quarters, float *result) {
  const uint32_t t = threadIdx.x;
#pragma unroll
  for (uint32_t c = 0; c < COUNT; ++c) partial[t * COUNT + c] = mine[c];
  __syncthreads();
  for (uint32_t item = t; item < 4u * COUNT; item += kThreads) {
    const uint32_t value = item % COUNT, quarter = item / COUNT;
    float sum = 0.0f;
#pragma unroll 8
    for (uint32_t i = 0; i < kThreads / 4u; ++i) sum += partial[(quarter * (kThreads / 4u) + i) * COUNT + value];
    quarters[item] = sum;
  }
  __syncthreads();
  if (t < COUNT) result[t] = (quarters[t] + quarters[COUNT + t]) + (quarters[2u * COUNT + t] + quarters[3u * COUNT + t]);
  __syncthreads();
}

// hyper_connection.rs:425-427
__device__ __forceinline__ float hc_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }

// One row's split (hyper_connection.rs:175-262), by one thread.  mix = raw dots * rms.
__device__ void split_sinkhorn(const float *raw, float rms, const float *scale, const float *base, float eps,
                               uint32_t iters, float *pre_lds, float *pre, float *post, float *comb_out) {
#pragma clang fp contract(off)  // the CPU rounds every multiply and add; only the explicit fmaf calls fuse
  float mix[kMix];
#pragma unroll
  for (uint32_t i = 0; i < kMix; ++i) mix[i] = raw[i] * rms;
#pragma unroll
  for (uint32_t j = 0; j < kHc; ++j) {
    const float p = hc_sigmoid(mix[j] * scale[0] + base[j]) + eps;
    pre_lds[j] = p;
    pre[j] = p;
    post[j] = 2.0f * hc_sigmoid(mix[kHc + j] * scale[1] + base[kHc + j]);
  }
  float comb[kHc * kHc];
#pragma unroll
  for (uint32_t row = 0; row < kHc; ++row) {
    float row_max = __uint_as_float(0xff800000u);
#pragma unroll
    for (uint32_t col = 0; col < kHc; ++col) {
      const float value = mix[2 * kHc + row * kHc + col] * scale[2] + base[2 * kHc + row * kHc + col];
      comb[row * kHc + col] = value;
      row_max = fmaxf(row_max, value);
    }
    float row_sum = 0.0f;
#pragma unroll
    for (uint32_t col = 0; col < kHc; ++col) {
      comb[row * kHc + col] = expf(comb[row * kHc + col] - row_max);
      row_sum += comb[row * kHc + col];
    }
#pragma unroll
    for (uint32_t col = 0; col < kHc; ++col) comb[row * kHc + col] = comb[row * kHc + col] / row_sum + eps;
  }
  for (uint32_t iteration = 0; iteration < iters; ++iteration) {
    if (iteration > 0) {
#pragma unroll
      for (uint32_t row = 0; row < kHc; ++row) {
        float sum = 0.0f;
#pragma unroll
        for (uint32_t col = 0; col < kHc; ++col) sum += comb[row * kHc + col];
#pragma unroll
        for (uint32_t col = 0; col < kHc; ++col) comb[row * kHc + col] /= sum + eps;
      }
    }
#pragma unroll
    for (uint32_t col = 0; col < kHc; ++col) {
      float sum = 0.0f;
#pragma unroll
      for (uint32_t row = 0; row < kHc; ++row) sum += comb[row * kHc + col];
#pragma unroll
      for (uint32_t row = 0; row < kHc; ++row) comb[row * kHc + col] /= sum + eps;
    }
  }
#pragma unroll
  for (uint32_t i = 0; i < kHc * kHc; ++i) comb_out[i] = comb[i];
}

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __uint_as_float(static_cast<uint32_t>(
      __builtin_amdgcn_update_dpp(0, static_cast<int>(__float_as_uint(v)), CTRL, 0xf, 0xf, false)));
}

// maximum over the 32 adjacent lanes that hold one 128-value block
__device__ __forceinline__ float max_over_32_lanes(float v) {
  v = fmaxf(v, dpp_f32<0xb1>(v));   // quad_perm [1,0,3,2]
  v = fmaxf(v, dpp_f32<0x4e>(v));   // quad_perm [2,3,0,1]
  v = fmaxf(v, dpp_f32<0x141>(v));  // row_half_mirror
  v = fmaxf(v, dpp_f32<0x140>(v));  // row_mirror
  return fmaxf(v, __shfl_xor(v, 16, 64));
}

// NJ = hidden / 1024; R = rows per workgroup
template <int NJ, int R>
__global__ __launch_bounds__(kThreads) void hc_producer_kernel(FerruleHipHcProducerArgs a) {
#pragma clang fp contract(off)  // the CPU rounds every multiply and add; only the explicit fmaf calls fuse
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr uint32_t kHidden = NJ * kSlice;
  constexpr uint32_t kHcHidden = kHc * kHidden;
  constexpr uint32_t kValues = kMix * R;  // widest block_sum of the kernel
  float *partial = lds;                               // [256][kValues]
  float *quarters = partial + kThreads * kValues;     // [4 * kValues]
  float *dots = quarters + 4u * kValues;              // [kValues]: mix[o * R + r]
  float *scalars = dots + kValues;                    // [R]: sums of squares
  float *pre_lds = scalars + R;                       // [R][4]

  const uint32_t t = threadIdx.x;
  const uint32_t row0 = blockIdx.x * R;
  const bool bf16_boundaries = (a.reserved & 1u) != 0u;
  const float *state = ptr<const float>(a.state_f32);
  const float *function = ptr<const float>(a.function_row_major_f32);

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

  // raw dot products with the 24 function rows, eight rows at a time, plus the state's squares
  float acc[kValues];
#pragma unroll
  for (uint32_t o = 0; o < kMix; ++o) {
    float sum[R];
#pragma unroll
    for (int r = 0; r < R; ++r) sum[r] = 0.0f;
    const float *frow = function + static_cast<size_t>(o) * kHcHidden + 4u * t;
#pragma unroll
    for (uint32_t c = 0; c < kHc; ++c) {
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const float4 f = *reinterpret_cast<const float4 *>(frow + c * kHidden + j * kSlice);
#pragma unroll
        for (int r = 0; r < R; ++r) {
          sum[r] = fmaf(f.x, s[r][c][j].x, sum[r]);
          sum[r] = fmaf(f.y, s[r][c][j].y, sum[r]);
          sum[r] = fmaf(f.z, s[r][c][j].z, sum[r]);
          sum[r] = fmaf(f.w, s[r][c][j].w, sum[r]);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) acc[o * R + r] = sum[r];
  }
  block_sum<kValues>(acc, partial, quarters, dots);

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
  block_sum<R>(squares, partial, quarters, scalars);

  // one thread per row (in different waves) turns the 24 dots into the split
  if ((t & 63u) == 0u && (t >> 6) < static_cast<uint32_t>(R)) {
    const uint32_t r = t >> 6;
    if (row0 + r < a.rows) {
      const uint32_t row = row0 + r;
      float raw[kMix];
#pragma unroll
      for (uint32_t o = 0; o < kMix; ++o) {
        raw[o] = dots[o * R + r];
        ptr<float>(a.mix_f32)[static_cast<size_t>(row) * kMix + o] = raw[o];
      }
      // rms_factor, hyper_connection.rs:416-419
      const float rms = 1.0f / sqrtf(scalars[r] / static_cast<float>(kHcHidden) + a.hc_norm_eps);
      split_sinkhorn(raw, rms, ptr<const float>(a.hc_scale_f32), ptr<const float>(a.hc_base_f32), a.hc_eps,
                     a.sinkhorn_iters, pre_lds + r * kHc, ptr<float>(a.split_pre_f32) + static_cast<size_t>(row) * kHc,
                     ptr<float>(a.split_post_f32) + static_cast<size_t>(row) * kHc,
                     ptr<float>(a.split_comb_f32) + static_cast<size_t>(row) * kHc * kHc);
    } else {
#pragma unroll
      for (uint32_t c = 0; c < kHc; ++c) pre_lds[r * kHc + c] = 0.0f;
    }
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
        *reinterpret_cast<float4 *>(ptr<float>(a.hidden_f32) + static_cast<size_t>(row0 + r) * kHidden + j * kSlice + 4u * t) = out;
      }
    }
    squares[r] = sum;
  }
  block_sum<R>(squares, partial, quarters, scalars);

  // RMSNorm with the layer weight, then the FP8-K128 quantiser
  const float *weight = ptr<const float>(a.layer_rms_weight_f32);
#pragma unroll
  for (int r = 0; r < R; ++r) {
    // math.rs:34-36: (sum / len + eps).sqrt().recip()
    const float scale = 1.0f / sqrtf(scalars[r] / static_cast<float>(kHidden) + a.layer_rms_eps);
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
      const float q = ferrule_quant::e8m0_value(byte);
      const uint32_t codes = ferrule_quant::fp8_e4m3_quantize_byte(n.x, q, FERRULE_HIP_FP8_ROUND_CPU_REFERENCE) |
                             (ferrule_quant::fp8_e4m3_quantize_byte(n.y, q, FERRULE_HIP_FP8_ROUND_CPU_REFERENCE) << 8) |
                             (ferrule_quant::fp8_e4m3_quantize_byte(n.z, q, FERRULE_HIP_FP8_ROUND_CPU_REFERENCE) << 16) |
                             (ferrule_quant::fp8_e4m3_quantize_byte(n.w, q, FERRULE_HIP_FP8_ROUND_CPU_REFERENCE) << 24);
      if (live) {
        *reinterpret_cast<float4 *>(ptr<float>(a.normalized_f32) + out_row * kHidden + d) = n;
        *reinterpret_cast<uint32_t *>(ptr<uint8_t>(a.packed_e4m3) + out_row * kHidden + d) = codes;
        if ((t & 31u) == 0u) ptr<uint8_t>(a.scales_ue8m0)[out_row * (kHidden / 128u) + (d >> 7)] = static_cast<uint8_t>(byte);
      }
    }
  }
}

template <int R>
constexpr uint32_t lds_bytes() {
  return (kThreads * kMix * R + 4u * kMix * R + kMix * R + R + R * kHc) * sizeof(float);
}

bool aligned16(uint64_t address) { return address != 0 && (address & 15u) == 0; }

FerruleHipStatus validate(const FerruleHipHcProducerArgs &a) {
  // hyper_connection.cuh:461-496, with the hidden size free in steps of 1024 and no workspace
  if (a.rows == 0 || a.hc != kHc || a.mix != kMix || a.reserved > 1u || a.sinkhorn_iters == 0) {
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

template <int NJ>
hipError_t launch_rows(const FerruleHipHcProducerArgs &a, hipStream_t stream) {
  // two rows per workgroup once there are enough rows to fill the machine either way: half the
  // L2 traffic for the function matrix.  Above H = 4096 a row pair no longer fits the registers.
  if (NJ <= 4 && a.rows >= 1024u) {
    auto kernel = hc_producer_kernel<(NJ <= 4 ? NJ : 1), 2>;
    hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes<2>()));
    if (err != hipSuccess) return err;
    kernel<<<(a.rows + 1u) / 2u, kThreads, lds_bytes<2>(), stream>>>(a);
  } else {
    hc_producer_kernel<NJ, 1><<<a.rows, kThreads, lds_bytes<1>(), stream>>>(a);
  }
  return hipSuccess;
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
  hipError_t err = hipSuccess;
  switch (a.hidden / kSlice) {
    case 1: err = launch_rows<1>(a, stream); break;
    case 2: err = launch_rows<2>(a, stream); break;
    case 3: err = launch_rows<3>(a, stream); break;
    case 4: err = launch_rows<4>(a, stream); break;
    case 5: err = launch_rows<5>(a, stream); break;
    case 6: err = launch_rows<6>(a, stream); break;
    case 7: err = launch_rows<7>(a, stream); break;
    default: err = launch_rows<8>(a, stream); break;
  }
  if (err != hipSuccess) return FERRULE_HIP_LAUNCH_FAILED;
  return take_launch_error() == 0 ? FERRULE_HIP_SUCCESS : FERRULE_HIP_LAUNCH_FAILED;
}
