// Decode GEMV for FP8-e4m3 (block scaled) and MXFP4 (e2m1 + e8m0/32) weights with
// BF16 activations, fp32 accumulation and one BF16 writeback.
//
// Semantics: LinearWeight::reference_matvec per activation row
// (crates/ferrule-model/src/checkpoint/weight.rs:154-173) then round_to_bf16
// (crates/ferrule-model/src/models/common/math.rs:7-14).
//
// Shape of the kernel ("skinny" MFMA GEMV):
//   * a workgroup owns 16 consecutive weight rows of one matrix; K is cut into CHUNKS of
//     consecutive k (512 k of MXFP4 = 4 K blocks, 256 k of FP8 = 2 K blocks) and K slice v is
//     the chunks v, v + slices, ...; with one row tile per CU a wave owns one slice (every byte
//     of the matrix is requested at once), with several per CU a wave walks two or four of them;
//   * a 15 MB matrix is 2 us of HBM time, so the kernel is shaped by what happens around the
//     stream.  Measured with in-kernel timestamps: every vector memory instruction of a wave
//     costs the CU's address path about 16 cycles whatever it fetches, loads return in issue
//     order, and a fragment of activations fetched per (lane, MFMA) from L2 costs four
//     instructions per K block against one for the weights.  Hence, per chunk:
//       1. the wave's slice of every activation row with ONE 16-byte-per-lane load per row,
//          issued first so that it returns first,
//       2. one scale dword per lane (MXFP4: row r, K block g of the chunk; the four lanes of a
//          row hold the chunk's sixteen scale bytes and exchange them by shuffles),
//       3. the weights: one 16-byte load per lane and K block (two for FP8), nontemporal on the
//          block-major order,
//       4. the activation slices are parked in a wave-private strip of LDS (no barrier) and read
//          back as MFMA fragments while the weights are still in flight;
//   * lane (r = lane%16, g = lane/16) holds 32 FP4 values = exactly one E8M0 scale block, or
//     16 FP8 values, of row r; they are expanded to BF16 *exactly* by the gfx950 converters
//     (v_cvt_scalef32_pk_bf16_fp4 / _fp8; the E8M0 scale is applied by the same instruction);
//   * v_mfma_f32_16x16x32_bf16 multiplies the 16x32 weight fragment with the 32x16 activation
//     fragment (up to 8 tokens per pass, the other columns are zero).  Products of two BF16
//     numbers are exact in fp32, so the only rounding is the fp32 accumulation, as in the
//     reference;
//   * F32 block scales cannot ride in the converter: the MFMA chain of one 128-wide K block
//     lands in a block accumulator that is folded in with one FMA per accumulator register
//     (acc += scale * block);
//   * waves are reduced through LDS in wave order, then one BF16 (or f32) store per output.
// A launch may cover several matrices (ferrule_hip_quant_gemv_multi_launch): the launch,
// address set-up and drain of a decode-sized kernel cost about as much as streaming one matrix.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>

#include "../../include/ferrule_hip_provider.h"
#include "numeric.cuh"
#include "skinny_core.cuh"

namespace ferrule_hip {
namespace {

struct GemvParams {
  const uint8_t *weight;
  const uint8_t *scales;
  const void *x;          // BF16 [batch, k]; SwiGLU-input form: f32 [batch, k] gate sums
  void *output;
  uint32_t batch;
  uint32_t n;
  uint32_t k;
  uint32_t scale_cols;
  uint32_t block_m;
  uint32_t block_k;
  uint32_t flags;
  // SwiGLU-input form only: the up sums beside `x` (the gate sums), and the activation's scalars
  const float *x_up;
  float swiglu_limit;
  float output_scale;
};

constexpr uint32_t kMaxMatrices = FERRULE_HIP_GEMV_MULTI_MAX;
constexpr uint32_t kMaxWaves = 16;

// Kernel argument of a launch over several matrices: workgroup b serves tile (b - tile_begin[m])
// of the matrix m with tile_begin[m] <= b < tile_begin[m + 1].  CAP = matrices the block has room
// for: launches of up to kSmallLaunch matrices take the small block (0.7 KB of kernel arguments
// instead of 2.7 KB; eight matrices measured 22.1 against 23.3 us).
constexpr uint32_t kSmallLaunch = 8;
template <uint32_t CAP>
struct GemvLaunchT {
  uint32_t count;
  uint32_t waves;    // waves of a workgroup
  uint32_t slices;   // K slices of a row tile (a multiple of the waves, or equal to them)
  uint32_t uniform_tiles;   // row tiles per matrix when all matrices have the same number, else 0
  uint32_t tile_begin[CAP + 1];
  GemvParams m[CAP];
};
using GemvLaunch = GemvLaunchT<kMaxMatrices>;
static_assert(sizeof(GemvLaunch) <= 4096, "kernel arguments");

// What a workgroup does with its 16 rows:
//   Plain       y = W x    BF16 activations, BF16 or f32 out
//   SwigluInput y = W h    h = silu(gate) * up * scale computed in f32 from two f32 rows when the
//                          activation slices are parked (clamped first when swiglu_limit > 0); each
//                          h row is split exactly into three BF16 rows (8 + 8 + 8 significant bits)
//                          that take three MFMA columns, and their results are added at the end
enum class GemvForm { Plain, SwigluInput };

template <int FMT, GemvForm FORM>
struct Chunk {
  // K blocks per chunk: the SwiGLU-input form parks three strips per row, so half as many as the
  // plain MXFP4 form
  static constexpr uint32_t kBlocks = (FMT == kFp4 && FORM == GemvForm::Plain) ? 4u : 2u;
  static constexpr uint32_t kElements = kBlocks * 128u;             // k per chunk
  static constexpr uint32_t kStripBytes = kElements * 2u + 16u;     // one BF16 row slice + bank skew
  static constexpr uint32_t kLanes = kElements / 8u;                // lanes that hold a piece of a slice
};

// LDS: [waves][strips][strip bytes] activation slices, then [K slices][64 lanes][4] partial sums.
inline uint32_t gemv_lds_bytes(uint32_t strip_bytes, uint32_t waves, uint32_t strips, uint32_t slices) {
  return ((waves * strips * strip_bytes + 255u) & ~255u) + slices * 1024u;
}

// Rows [16 tile, 16 tile + 16) of one matrix by a workgroup of `waves` waves, T
// activation strips (MFMA columns) per pass over the weights.
//
// Two rules shape this code (both measured, each worth most of a microsecond of a 6 us kernel):
//   * everything the first loads need comes out of ONE round of scalar loads of the kernel
//     argument (the workgroup size travels in the argument for that reason, and the token loop
//     is entered unconditionally: batch >= 1 is checked on the host);
//   * every global load of a chunk is issued unconditionally in straight-line code (addresses
//     are clamped into the operand, results of absent pieces replaced by zero afterwards).  A
//     load inside a branch makes the compiler's wait counts conservative: the activation slices
//     would be "waited for" together with the weights issued after them, and nothing would
//     overlap the HBM latency.
// Activation rows beyond the batch are clamped to its last row: their MFMA columns repeat that
// row's result and are never stored; columns beyond T multiply by zero.
template <int FMT, int SCALE, bool BLOCK_MAJOR, int T, GemvForm FORM>
//
// The K extent is cut into `slices` K slices (slice v = chunks v, v + slices, ...), each summed on its
// own in fp32 and the slices added in slice order at the end.  A workgroup has as many waves as
// slices, or a half or a quarter of them, each wave then doing several slices one after the other:
// the bits of a result depend on `slices` only, not on the shape of the workgroup.
__device__ __forceinline__ void skinny_gemv_tile(const GemvParams &p, uint32_t tile, uint32_t waves, uint32_t slices) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  using C = Chunk<FMT, FORM>;
  constexpr int NMAT = 1;
  constexpr bool XF32 = FORM == GemvForm::SwigluInput;
  constexpr int TOKENS = XF32 ? T / 3 : T;   // activation rows per pass
  static_assert(!XF32 || T % 3 == 0, "three strips per f32 row");
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t r = lane & 15u;
  const uint32_t g = lane >> 4;
  const uint32_t row0 = tile * 16u;
  const uint32_t row = min(row0 + r, p.n - 1u);
  const uint32_t kblocks = p.k >> 7;   // k % 128 == 0 (checked on the host)
  const uint32_t chunks = (kblocks + C::kBlocks - 1u) / C::kBlocks;
  // strips of this wave; the partial sums live behind the strips
  uint8_t *strip = lds + wave * (T * C::kStripBytes);
  float *red = reinterpret_cast<float *>(lds + ((waves * T * C::kStripBytes + 255u) & ~255u));
  const u32x4_t zero4 = {0u, 0u, 0u, 0u};
  const uint8_t *frag = strip + min(r, static_cast<uint32_t>(T - 1)) * C::kStripBytes;
  const uint8_t *const wbase[1] = {p.weight};
  const uint8_t *const sbase[1] = {p.scales};

  uint32_t b0 = 0;
  do {
    const uint32_t tokens = min(p.batch - b0, static_cast<uint32_t>(TOKENS));
    for (uint32_t slice = wave; slice < slices; slice += waves) {
    f32x4_t acc[NMAT];
#pragma unroll
    for (int m = 0; m < NMAT; ++m) acc[m] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    for (uint32_t chunk = slice; chunk < chunks; chunk += slices) {
      const uint32_t kb0 = chunk * C::kBlocks;
      // 1. activation slices: lane l holds k [chunk * kElements + 8 l, + 8) of every row
      u32x4_t xv[TOKENS][XF32 ? 4 : 1];   // SwiGLU input: 8 gate sums, then 8 up sums
      const uint32_t xk = chunk * C::kElements + lane * 8u;
      const bool x_live = lane < C::kLanes && xk < p.k;
      const uint32_t xk_clamped = min(xk, p.k - 8u);
      auto load_x = [&]() {
#pragma unroll
        for (int t = 0; t < TOKENS; ++t) {
          const uint32_t token = min(b0 + static_cast<uint32_t>(t), p.batch - 1u);
          if constexpr (XF32) {
            const size_t at = static_cast<size_t>(token) * p.k + xk_clamped;
            xv[t][0] = load16(static_cast<const float *>(p.x) + at);
            xv[t][1] = load16(static_cast<const float *>(p.x) + at + 4);
            xv[t][2] = load16(p.x_up + at);
            xv[t][3] = load16(p.x_up + at + 4);
          } else {
            xv[t][0] = load16(static_cast<const uint16_t *>(p.x) + static_cast<size_t>(token) * p.k + xk_clamped);
          }
        }
      };
      // loads return in issue order: the activation slices must be requested before the weights,
      // or parking them would wait for the whole chunk.  (The other order, weights first so that a
      // batch of four or eight rows does not hold the weight requests back, measured slower: 6.2
      // against 6.1 us at four rows, 7.1 against 6.5 us at eight.)
      load_x();
      __builtin_amdgcn_sched_barrier(0);
      // 2. scales.  MXFP4: the dword of (row r, K block kb0 + g) = the bytes of its four 32-wide
      //    groups (with fewer than four K blocks per chunk the upper lane groups repeat the last).
      //    FP8: one scale per lane and K block; block_k % 128 == 0 (checked on the host);
      //    E8M0: the scale of this lane's row (any block_m) rides in the converter;
      //    F32 : one scale per (16-row tile, K block), so block_m % 16 == 0.
      uint32_t sdw[NMAT];
      float sc8[NMAT][C::kBlocks];
      // 3. weights.  MXFP4: lane (r, g) of K block kb0 + j holds k [32 g, 32 g + 32) of row r;
      //    FP8: lane (r, g) of half u of K block kb0 + j holds k [64 u + 16 g, + 16) of row r
      u32x4_t w[NMAT][C::kBlocks][FMT == kFp4 ? 1 : 2];
#pragma unroll
      for (int m = 0; m < NMAT; ++m) {
        if constexpr (FMT == kFp4) {
          const uint32_t skb = min(kb0 + min(g, C::kBlocks - 1u), kblocks - 1u);
          if constexpr (BLOCK_MAJOR) {
            sdw[m] = load4(sbase[m] + static_cast<size_t>(row0) * (p.k >> 5) + skb * 64u + r * 4u);
          } else {
            sdw[m] = load4(sbase[m] + static_cast<size_t>(row) * p.scale_cols + skb * 4u);
          }
#pragma unroll
          for (uint32_t j = 0; j < C::kBlocks; ++j) {
            const uint32_t kb = min(kb0 + j, kblocks - 1u);
            if constexpr (BLOCK_MAJOR) {
              w[m][j][0] = load_stream16(wbase[m] + static_cast<size_t>(row0) * (p.k >> 1) + kb * 1024u + r * 64u + g * 16u);
            } else {
              w[m][j][0] = load_stream16(wbase[m] + static_cast<size_t>(row) * (p.k >> 1) + kb * 64u + g * 16u);
            }
          }
        } else {
          const uint32_t kb_per_scale = p.block_k >> 7;
#pragma unroll
          for (uint32_t j = 0; j < C::kBlocks; ++j) {
            const uint32_t kb = min(kb0 + j, kblocks - 1u);
            const uint32_t si = kb_per_scale == 1u ? kb : kb / kb_per_scale;
            if constexpr (SCALE == kF32) {
              sc8[m][j] = reinterpret_cast<const float *>(sbase[m])[static_cast<size_t>(row0 / p.block_m) * p.scale_cols + si];
            } else {
              sc8[m][j] = e8m0_to_f32(load1(sbase[m] + static_cast<size_t>(row / p.block_m) * p.scale_cols + si));
            }
#pragma unroll
            for (uint32_t u = 0; u < 2u; ++u) {
              if constexpr (BLOCK_MAJOR) {
                w[m][j][u] = load_stream16(wbase[m] + static_cast<size_t>(row0) * p.k + (kb * 2u + u) * 1024u + r * 64u + g * 16u);
              } else {
                w[m][j][u] = load_stream16(wbase[m] + static_cast<size_t>(row) * p.k + kb * 128u + u * 64u + g * 16u);
              }
            }
          }
        }
      }
      // 4. park the activation slices, fetch fragments and scale bytes while the weights fly
      if (lane < C::kLanes) {
#pragma unroll
        for (int t = 0; t < TOKENS; ++t) {
          if constexpr (XF32) {
            // SwiGluFfn::reference_execute (crates/ferrule-model/src/ffn.rs:33-47): clamp, then
            // silu(gate) * up * output_scale, left to right in f32 (silu_fast: every workgroup
            // forms the whole row, and silu_ref would cost it half a microsecond per row);
            // h = hi + mid + lo with every term a BF16 value (8 + 8 + 8 significant bits, exact)
            u32x4_t term[3];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              float gate = __uint_as_float(xv[t][e >> 2][e & 3]);
              float up = __uint_as_float(xv[t][2 + (e >> 2)][e & 3]);
              if (p.swiglu_limit > 0.0f) {
                gate = fminf(gate, p.swiglu_limit);
                up = fminf(fmaxf(up, -p.swiglu_limit), p.swiglu_limit);
              }
              const float v = x_live ? silu_fast(gate) * up * p.output_scale : 0.0f;
              const uint32_t hi = __float_as_uint(v) & 0xffff0000u;
              const float r1 = v - __uint_as_float(hi);
              const uint32_t mid = __float_as_uint(r1) & 0xffff0000u;
              const uint32_t lo = __float_as_uint(r1 - __uint_as_float(mid)) & 0xffff0000u;
              const uint32_t parts[3] = {hi, mid, lo};
#pragma unroll
              for (int c = 0; c < 3; ++c) {
                if ((e & 1) == 0) term[c][e >> 1] = parts[c] >> 16;
                else term[c][e >> 1] |= parts[c];
              }
            }
#pragma unroll
            for (int c = 0; c < 3; ++c)
              *reinterpret_cast<u32x4_t *>(strip + (3 * t + c) * C::kStripBytes + lane * 16u) = term[c];
          } else {
            *reinterpret_cast<u32x4_t *>(strip + t * C::kStripBytes + lane * 16u) = x_live ? xv[t][0] : zero4;
          }
        }
      }
      uint32_t sbyte[NMAT][C::kBlocks];
      u32x4_t xf[C::kBlocks][4];
#pragma unroll
      for (uint32_t j = 0; j < C::kBlocks; ++j) {
        if constexpr (FMT == kFp4) {
#pragma unroll
          for (int m = 0; m < NMAT; ++m)
            sbyte[m][j] = (static_cast<uint32_t>(__shfl(static_cast<int>(sdw[m]), static_cast<int>(r + 16u * j), 64)) >> (8u * g)) & 0xffu;
        }
#pragma unroll
        for (uint32_t q = 0; q < 4u; ++q) xf[j][q] = zero4;
      }
      // An LDS read costs its lanes, but a branch around the reads costs the schedule: measured, all lanes
      // reading (the clamped row, a broadcast) is the faster form up to four rows, the masked form at eight.
      if (T < 8 || r < static_cast<uint32_t>(T)) {
#pragma unroll
        for (uint32_t j = 0; j < C::kBlocks; ++j) {
#pragma unroll
          for (uint32_t q = 0; q < 4u; ++q) {
            // MXFP4: MFMA q of the block takes k [32 g + 8 q, + 8); FP8: q = 2 u + half, k [64 u + 16 g + 8 half, + 8)
            const uint32_t at = FMT == kFp4 ? g * 64u + q * 16u : (q >> 1) * 128u + g * 32u + (q & 1u) * 16u;
            xf[j][q] = *reinterpret_cast<const u32x4_t *>(frag + j * 256u + at);
          }
        }
      }
      // nothing that touches a weight register may be scheduled above this line: it would pull
      // the wait for the first weight block (HBM latency) in front of the LDS traffic
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int m = 0; m < NMAT; ++m) {
#pragma unroll
        for (uint32_t j = 0; j < C::kBlocks; ++j) {
          const bool live = kb0 + j < kblocks;   // a chunk may end before its last K block
          if constexpr (FMT == kFp4) {
            const float sc = e8m0_to_f32(sbyte[m][j]);
            const u32x4_t wj = live ? w[m][j][0] : zero4;
#pragma unroll
            for (uint32_t q = 0; q < 4u; ++q) {
              acc[m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(expand_fp4_dword(wj[q], sc), as_bf16x8(xf[j][q]), acc[m], 0, 0, 0);
            }
          } else {
            const u32x4_t w0 = live ? w[m][j][0] : zero4;
            const u32x4_t w1 = live ? w[m][j][1] : zero4;
            if constexpr (SCALE == kE8m0) {
              const float sc = sc8[m][j];
              acc[m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(expand_fp8_dwords(w0[0], w0[1], sc), as_bf16x8(xf[j][0]), acc[m], 0, 0, 0);
              acc[m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(expand_fp8_dwords(w0[2], w0[3], sc), as_bf16x8(xf[j][1]), acc[m], 0, 0, 0);
              acc[m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(expand_fp8_dwords(w1[0], w1[1], sc), as_bf16x8(xf[j][2]), acc[m], 0, 0, 0);
              acc[m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(expand_fp8_dwords(w1[2], w1[3], sc), as_bf16x8(xf[j][3]), acc[m], 0, 0, 0);
            } else {
              // the f32 scale covers the whole 128 block: MFMA chain into a block accumulator,
              // then acc += scale * block (one FMA per accumulator register)
              f32x4_t blk = {0.f, 0.f, 0.f, 0.f};
              blk = __builtin_amdgcn_mfma_f32_16x16x32_bf16(expand_fp8_dwords(w0[0], w0[1], 1.0f), as_bf16x8(xf[j][0]), blk, 0, 0, 0);
              blk = __builtin_amdgcn_mfma_f32_16x16x32_bf16(expand_fp8_dwords(w0[2], w0[3], 1.0f), as_bf16x8(xf[j][1]), blk, 0, 0, 0);
              blk = __builtin_amdgcn_mfma_f32_16x16x32_bf16(expand_fp8_dwords(w1[0], w1[1], 1.0f), as_bf16x8(xf[j][2]), blk, 0, 0, 0);
              blk = __builtin_amdgcn_mfma_f32_16x16x32_bf16(expand_fp8_dwords(w1[2], w1[3], 1.0f), as_bf16x8(xf[j][3]), blk, 0, 0, 0);
#pragma unroll
              for (int v = 0; v < 4; ++v) acc[m][v] = fmaf(sc8[m][j], blk[v], acc[m][v]);
            }
          }
        }
      }
    }

    // acc[v] of lane l is (weight row 4*(l/16)+v, column l%16); slices are added in slice order
    *reinterpret_cast<f32x4_t *>(red + (slice * 64u + lane) * 4u) = acc[0];
    }
    __syncthreads();
    if (threadIdx.x < 16u * TOKENS) {
      const uint32_t tok = threadIdx.x >> 4;
      const uint32_t rr = threadIdx.x & 15u;
      // the sum over the K slices of (row rr, column c)
      auto column = [&](uint32_t c) {
        const uint32_t src = ((rr >> 2) * 16u + c) * 4u + (rr & 3u);
        float part[kMaxWaves];
#pragma unroll
        for (uint32_t w = 0; w < kMaxWaves; ++w) part[w] = red[min(w, slices - 1u) * 256u + src];
        float sum = 0.f;
#pragma unroll
        for (uint32_t w = 0; w < kMaxWaves; ++w) sum += w < slices ? part[w] : 0.f;   // + 0 of an absent slice changes nothing
        return sum;
      };
      const uint32_t orow = row0 + rr;
      const size_t o = static_cast<size_t>(b0 + tok) * p.n + orow;
      const bool store = orow < p.n && tok < tokens;
      float sum;
      if constexpr (XF32) {
        sum = (column(3u * tok) + column(3u * tok + 1u)) + column(3u * tok + 2u);
      } else {
        sum = column(tok);
      }
      if (store) {
        if (p.flags & FERRULE_HIP_GEMV_OUTPUT_F32) {
          static_cast<float *>(p.output)[o] = sum;
        } else {
          static_cast<uint16_t *>(p.output)[o] = bf16_rne_bits(sum);
        }
      }
    }
    b0 += TOKENS;
    if (b0 >= p.batch) break;
    __syncthreads();   // the partial sums are rewritten by the next pass
  } while (true);
}

template <int FMT, int SCALE, bool BLOCK_MAJOR, int T, GemvForm FORM>
__global__ __launch_bounds__(kMaxWaves * 64) void skinny_gemv_kernel(GemvParams p, uint32_t waves, uint32_t slices) {
  skinny_gemv_tile<FMT, SCALE, BLOCK_MAJOR, T, FORM>(p, blockIdx.x, waves, slices);
}

// Several matrices: one more round of scalar loads to fetch the block of this workgroup's matrix.
template <int FMT, int SCALE, bool BLOCK_MAJOR, int T, uint32_t CAP>
__global__ __launch_bounds__(kMaxWaves * 64) void skinny_gemv_multi_kernel(GemvLaunchT<CAP> launch) {
  // Both look-ups are computed and one is selected, without a branch: everything they read then
  // comes out of ONE round of scalar loads of the kernel argument (a branch on uniform_tiles made
  // it a round of its own, about 0.4 us per workgroup).
  uint32_t count = launch.count, waves = launch.waves, slices = launch.slices, uniform = launch.uniform_tiles;
  uint32_t begin[CAP];
#pragma unroll
  for (uint32_t m = 1; m < CAP; ++m) begin[m] = launch.tile_begin[m];
  // the head of the block and the whole prefix table are in registers HERE, fetched in one round
  // (the table is loaded in pieces: one entry of each piece is named)
  asm volatile("" : "+s"(count), "+s"(waves), "+s"(slices), "+s"(uniform), "+s"(begin[1]));
  if constexpr (CAP > 8u) {
    asm volatile("" : "+s"(begin[CAP / 2 + 1]), "+s"(begin[3 * CAP / 4 + 1]), "+s"(begin[7 * CAP / 8 + 1]), "+s"(begin[CAP - 1]));
  }
  uint32_t which = 0, first = 0;
#pragma unroll
  for (uint32_t m = 1; m < CAP; ++m) {
    const bool at_or_past = blockIdx.x >= begin[m];   // tile_begin[m] = all tiles for m >= count
    which = at_or_past ? m : which;
    first = at_or_past ? begin[m] : first;
  }
  // every matrix has the same number of row tiles (the usual case: the experts or projections of
  // one layer): one division instead of the walk over the prefix table
  const uint32_t quotient = blockIdx.x / (uniform != 0u ? uniform : 1u);
  which = uniform != 0u ? quotient : which;
  first = uniform != 0u ? quotient * uniform : first;
  which = which < count ? which : count - 1u;
  skinny_gemv_tile<FMT, SCALE, BLOCK_MAJOR, T, GemvForm::Plain>(launch.m[which], blockIdx.x - first, waves, slices);
}

// Generic shapes (odd K, odd scale blocks): one wave per weight row, software
// decode, fp32 FMA, up to 8 activation rows per pass.
template <int FMT, int SCALE>
__global__ __launch_bounds__(256) void generic_gemv_kernel(GemvParams p) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t row = blockIdx.x * 4u + (threadIdx.x >> 6);
  if (row >= p.n) return;
  for (uint32_t b0 = 0; b0 < p.batch; b0 += 8u) {
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (uint32_t col = lane; col < p.k; col += 64u) {
      float w;
      if constexpr (FMT == kFp4) {
        const uint32_t byte = p.weight[static_cast<size_t>(row) * (p.k >> 1) + (col >> 1)];
        const uint32_t nib = (col & 1u) ? (byte >> 4) : (byte & 15u);
        w = fp4_e2m1_decode(nib) *
            e8m0_to_f32(p.scales[static_cast<size_t>(row) * p.scale_cols + col / p.block_k]);
      } else {
        const float d = fp8_e4m3_decode(p.weight[static_cast<size_t>(row) * p.k + col]);
        const size_t si = static_cast<size_t>(row / p.block_m) * p.scale_cols + col / p.block_k;
        const float s = SCALE == kF32 ? reinterpret_cast<const float *>(p.scales)[si]
                                      : e8m0_to_f32(p.scales[si]);
        w = d * s;
      }
#pragma unroll
      for (uint32_t b = 0; b < 8u; ++b) {
        if (b0 + b < p.batch) {
          acc[b] = fmaf(w, bf16_bits_to_f32(static_cast<const uint16_t *>(p.x)[static_cast<size_t>(b0 + b) * p.k + col]), acc[b]);
        }
      }
    }
#pragma unroll
    for (uint32_t b = 0; b < 8u; ++b) {
      const float sum = wave_sum(acc[b]);
      if (lane == 0u && b0 + b < p.batch) {
        const size_t o = static_cast<size_t>(b0 + b) * p.n + row;
        if (p.flags & FERRULE_HIP_GEMV_OUTPUT_F32) {
          static_cast<float *>(p.output)[o] = sum;
        } else {
          static_cast<uint16_t *>(p.output)[o] = bf16_rne_bits(sum);
        }
      }
    }
  }
}

// Element-wise dequantisation through the same converters the GEMV uses.
template <int FMT, int SCALE>
__global__ __launch_bounds__(256) void dequant_kernel(GemvParams p) {
  // one thread per packed dword
  const size_t dword = static_cast<size_t>(blockIdx.x) * 256u + threadIdx.x;
  float *out = static_cast<float *>(p.output);
  if constexpr (FMT == kFp4) {
    const size_t dwords_per_row = p.k >> 3;
    if (dword >= static_cast<size_t>(p.n) * dwords_per_row) return;
    const uint32_t row = static_cast<uint32_t>(dword / dwords_per_row);
    const uint32_t k0 = static_cast<uint32_t>(dword % dwords_per_row) * 8u;
    const uint32_t packed = reinterpret_cast<const uint32_t *>(p.weight)[dword];
    const float sc = e8m0_to_f32(p.scales[static_cast<size_t>(row) * p.scale_cols + k0 / p.block_k]);
    const bf16x8_t v = expand_fp4_dword(packed, sc);
#pragma unroll
    for (int e = 0; e < 8; ++e) out[static_cast<size_t>(row) * p.k + k0 + e] = static_cast<float>(v[e]);
  } else {
    const size_t dwords_per_row = p.k >> 2;
    if (dword >= static_cast<size_t>(p.n) * dwords_per_row) return;
    const uint32_t row = static_cast<uint32_t>(dword / dwords_per_row);
    const uint32_t k0 = static_cast<uint32_t>(dword % dwords_per_row) * 4u;
    const uint32_t packed = reinterpret_cast<const uint32_t *>(p.weight)[dword];
    const size_t si = static_cast<size_t>(row / p.block_m) * p.scale_cols + k0 / p.block_k;
    float sc = 1.0f;
    float post = 1.0f;
    if constexpr (SCALE == kE8m0) {
      sc = e8m0_to_f32(p.scales[si]);
    } else {
      post = reinterpret_cast<const float *>(p.scales)[si];
    }
    const bf16x2_t a0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(packed, sc, false);
    const bf16x2_t a1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(packed, sc, true);
    float v[4] = {static_cast<float>(a0[0]), static_cast<float>(a0[1]), static_cast<float>(a1[0]),
                  static_cast<float>(a1[1])};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      out[static_cast<size_t>(row) * p.k + k0 + e] = SCALE == kF32 ? v[e] * post : v[e];
    }
  }
}

inline bool aligned16(uint64_t p) { return p != 0 && (p & 15u) == 0; }

// Shapes the MFMA kernel takes; everything else valid goes to the generic kernel.
bool skinny_ok(const FerruleHipQuantGemvArgs &a) {
  if (a.k % 128u != 0u) return false;   // whole K blocks: no load of the MFMA kernel is conditional
  if (a.weight_format == kFp4) return a.block_k == 32u;
  if (a.block_k % 128u != 0u) return false;
  return a.scale_kind == kE8m0 || a.block_m % 16u == 0u;
}

int32_t validate(const FerruleHipQuantGemvArgs *a, bool need_x) {
  if (a == nullptr) return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->weight_format != kFp4 && a->weight_format != kFp8) return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->scale_kind != kE8m0 && a->scale_kind != kF32) return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->n == 0 || a->k == 0 || a->block_m == 0 || a->block_k == 0) return FERRULE_HIP_INVALID_ARGUMENT;
  if (need_x && a->batch == 0) return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->scale_cols != (a->k + a->block_k - 1) / a->block_k) return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->weight_format == kFp4) {
    // the MX contract: one E8M0 scale per 32 contiguous K elements of one row
    if (a->scale_kind != kE8m0 || a->block_m != 1 || a->k % 2u != 0 || a->k % a->block_k != 0)
      return FERRULE_HIP_INVALID_ARGUMENT;
    if (a->block_k % 8u != 0) return FERRULE_HIP_UNSUPPORTED;
  }
  if (!aligned16(a->weight) || !aligned16(a->weight_scales) || !aligned16(a->output))
    return FERRULE_HIP_INVALID_ARGUMENT;
  if (need_x && !aligned16(a->x)) return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->flags & FERRULE_HIP_GEMV_BLOCK_MAJOR_WEIGHTS) {
    // only the decode GEMV reads the prepared order, and only whole tiles of it
    if (!need_x) return FERRULE_HIP_INVALID_ARGUMENT;
    if (a->weight_format == kFp4 && a->block_k != 32u) return FERRULE_HIP_INVALID_ARGUMENT;
    if (a->n % 16u != 0 || a->k % 128u != 0 || !skinny_ok(*a)) return FERRULE_HIP_UNSUPPORTED;
  }
  return FERRULE_HIP_SUCCESS;
}

GemvParams make_params(const FerruleHipQuantGemvArgs &a) {
  GemvParams p;
  p.weight = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(a.weight));
  p.scales = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(a.weight_scales));
  p.x = reinterpret_cast<const uint16_t *>(static_cast<uintptr_t>(a.x));
  p.output = reinterpret_cast<void *>(static_cast<uintptr_t>(a.output));
  p.batch = a.batch;
  p.n = a.n;
  p.k = a.k;
  p.scale_cols = a.scale_cols;
  p.block_m = a.block_m;
  p.block_k = a.block_k;
  p.flags = a.flags;
  p.x_up = nullptr;
  p.swiglu_limit = 0.0f;
  p.output_scale = 1.0f;
  return p;
}

// The MFMA kernels' dynamic LDS goes beyond the 64 KiB a kernel gets by default.
template <typename Kernel>
hipError_t allow_large_lds(Kernel kernel, std::once_flag &once, hipError_t &result, uint32_t bytes) {
  std::call_once(once, [&] {
    result = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                 static_cast<int>(bytes));
  });
  return result;
}

template <int FMT, GemvForm FORM>
uint32_t waves_for(uint32_t k, uint32_t threads_for_the_sum) {
  const uint32_t chunks = (k / 128u + Chunk<FMT, FORM>::kBlocks - 1u) / Chunk<FMT, FORM>::kBlocks;
  const uint32_t least = (threads_for_the_sum + 63u) / 64u;
  const uint32_t waves = chunks > least ? chunks : least;
  return waves > kMaxWaves ? kMaxWaves : waves;
}

// Waves per workgroup for a launch of `tiles` row tiles.  With one tile per CU a workgroup wants as
// many waves as the K extent has chunks (every byte of the matrix is requested at once).  A launch
// with several tiles per CU (several matrices, or a tall one) does better with smaller workgroups,
// two or four to a CU: while one reduces and stores, the others stream (eight MXFP4 matrices of
// 4096 x 7168 in one launch: 31 us with 14-wave workgroups, 25 us with 7 waves, 22.5 us with 4).
// Three or five workgroups per CU (15 waves) measured worse than two.
inline uint32_t waves_for_tiles(uint32_t waves, uint64_t tiles, uint32_t threads_for_the_sum) {
  const uint32_t least = (threads_for_the_sum + 63u) / 64u;
  const uint32_t share = tiles >= 1024u ? 4u : (tiles >= 512u ? 2u : 1u);
  const uint32_t fewer = (waves + share - 1u) / share;
  return fewer >= least ? fewer : waves;
}

// One matrix in the given form, T strips per pass.
template <int FMT, int SCALE, bool BLOCK_MAJOR, int T, GemvForm FORM>
hipError_t launch_form_t(const GemvParams &p, hipStream_t stream) {
  constexpr uint32_t kTokens = FORM == GemvForm::SwigluInput ? T / 3 : T;
  static std::once_flag once;
  static hipError_t attribute = hipSuccess;
  const hipError_t e = allow_large_lds(skinny_gemv_kernel<FMT, SCALE, BLOCK_MAJOR, T, FORM>, once, attribute,
                                       gemv_lds_bytes(Chunk<FMT, FORM>::kStripBytes, kMaxWaves, T, kMaxWaves));
  if (e != hipSuccess) return e;
  const uint32_t slices = waves_for<FMT, FORM>(p.k, 16u * kTokens);
  const uint32_t waves = waves_for_tiles(slices, (p.n + 15u) / 16u, 16u * kTokens);
  const uint32_t lds = gemv_lds_bytes(Chunk<FMT, FORM>::kStripBytes, waves, T, slices);
  skinny_gemv_kernel<FMT, SCALE, BLOCK_MAJOR, T, FORM><<<(p.n + 15u) / 16u, waves * 64u, lds, stream>>>(p, waves, slices);
  return hipSuccess;
}

template <int FMT, int SCALE, bool BLOCK_MAJOR, int T, uint32_t CAP>
hipError_t launch_multi_t(const GemvLaunch &all, hipStream_t stream) {
  static std::once_flag once;
  static hipError_t attribute = hipSuccess;
  const hipError_t e = allow_large_lds(skinny_gemv_multi_kernel<FMT, SCALE, BLOCK_MAJOR, T, CAP>, once, attribute,
                                       gemv_lds_bytes(Chunk<FMT, GemvForm::Plain>::kStripBytes, kMaxWaves, T, kMaxWaves));
  if (e != hipSuccess) return e;
  GemvLaunchT<CAP> launch;
  launch.count = all.count;
  launch.uniform_tiles = all.uniform_tiles;
  for (uint32_t m = 0; m < CAP; ++m) {
    launch.m[m] = all.m[m];
    launch.tile_begin[m] = all.tile_begin[m];
  }
  launch.tile_begin[CAP] = all.tile_begin[all.count];   // all tiles
  uint32_t waves = 1;
  for (uint32_t m = 0; m < launch.count; ++m) {
    const uint32_t need = waves_for<FMT, GemvForm::Plain>(launch.m[m].k, 16u * T);
    waves = need > waves ? need : waves;
  }
  launch.slices = waves;
  waves = waves_for_tiles(waves, all.tile_begin[all.count], 16u * T);
  launch.waves = waves;
  const uint32_t lds = gemv_lds_bytes(Chunk<FMT, GemvForm::Plain>::kStripBytes, waves, T, launch.slices);
  skinny_gemv_multi_kernel<FMT, SCALE, BLOCK_MAJOR, T, CAP><<<all.tile_begin[all.count], waves * 64u, lds, stream>>>(launch);
  return hipSuccess;
}

template <int FMT, int SCALE, bool BLOCK_MAJOR, int T>
hipError_t launch_skinny_t(GemvLaunch &launch, hipStream_t stream) {
  if (launch.count == 1u) return launch_form_t<FMT, SCALE, BLOCK_MAJOR, T, GemvForm::Plain>(launch.m[0], stream);
  if (launch.count <= kSmallLaunch) return launch_multi_t<FMT, SCALE, BLOCK_MAJOR, T, kSmallLaunch>(launch, stream);
  return launch_multi_t<FMT, SCALE, BLOCK_MAJOR, T, kMaxMatrices>(launch, stream);
}

// T = activation rows per pass: the smallest of 1, 2, 4, 8 that holds the largest batch of the launch.
template <int FMT, int SCALE, bool BLOCK_MAJOR>
hipError_t launch_skinny(GemvLaunch &launch, hipStream_t stream) {
  uint32_t tokens = 1;
  for (uint32_t m = 0; m < launch.count; ++m) tokens = launch.m[m].batch > tokens ? launch.m[m].batch : tokens;
  if (tokens <= 1u) return launch_skinny_t<FMT, SCALE, BLOCK_MAJOR, 1>(launch, stream);
  if (tokens <= 2u) return launch_skinny_t<FMT, SCALE, BLOCK_MAJOR, 2>(launch, stream);
  if (tokens <= 4u) return launch_skinny_t<FMT, SCALE, BLOCK_MAJOR, 4>(launch, stream);
  return launch_skinny_t<FMT, SCALE, BLOCK_MAJOR, 8>(launch, stream);
}

// The down projection of a dense FFN: SwiGLU of the gate and up sums on the way in.
template <int FMT, int SCALE, bool BLOCK_MAJOR>
hipError_t launch_swiglu_down(const GemvParams &down, hipStream_t stream) {
  const uint32_t b = down.batch;
  if (b <= 1u) return launch_form_t<FMT, SCALE, BLOCK_MAJOR, 3, GemvForm::SwigluInput>(down, stream);
  if (b <= 2u) return launch_form_t<FMT, SCALE, BLOCK_MAJOR, 6, GemvForm::SwigluInput>(down, stream);
  // four rows per pass over the weights (five need spilled registers at the 128 a 16-wave workgroup gets)
  return launch_form_t<FMT, SCALE, BLOCK_MAJOR, 12, GemvForm::SwigluInput>(down, stream);
}

// One launch for `count` matrices of one weight format, scale kind and weight order.
int32_t launch_matrices(const FerruleHipQuantGemvArgs *const *args, uint32_t count) {
  const FerruleHipQuantGemvArgs &first = *args[0];
  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(first.stream));
  clear_launch_error();
  if (!skinny_ok(first)) {
    // odd shapes: one generic launch per matrix
    for (uint32_t m = 0; m < count; ++m) {
      const GemvParams p = make_params(*args[m]);
      const uint32_t blocks = (p.n + 3u) / 4u;
      if (args[m]->weight_format == kFp4) {
        generic_gemv_kernel<kFp4, kE8m0><<<blocks, 256, 0, stream>>>(p);
      } else if (args[m]->scale_kind == kE8m0) {
        generic_gemv_kernel<kFp8, kE8m0><<<blocks, 256, 0, stream>>>(p);
      } else {
        generic_gemv_kernel<kFp8, kF32><<<blocks, 256, 0, stream>>>(p);
      }
    }
    return take_launch_error() == hipSuccess ? FERRULE_HIP_SUCCESS : FERRULE_HIP_LAUNCH_FAILED;
  }
  GemvLaunch launch;
  launch.count = count;
  uint64_t tiles = 0;
  for (uint32_t m = 0; m < kMaxMatrices; ++m) {
    launch.tile_begin[m] = static_cast<uint32_t>(tiles);
    if (m < count) {
      launch.m[m] = make_params(*args[m]);
      tiles += (launch.m[m].n + 15u) / 16u;
    } else {
      launch.m[m] = launch.m[0];
    }
  }
  launch.uniform_tiles = (launch.m[0].n + 15u) / 16u;
  for (uint32_t m = 1; m < count; ++m) {
    if ((launch.m[m].n + 15u) / 16u != launch.uniform_tiles) launch.uniform_tiles = 0;
  }
  launch.tile_begin[kMaxMatrices] = static_cast<uint32_t>(tiles);
  for (uint32_t m = count; m <= kMaxMatrices; ++m) launch.tile_begin[m] = static_cast<uint32_t>(tiles);
  if (tiles > 0x7fffffffull) return FERRULE_HIP_UNSUPPORTED;
  const bool block_major = (first.flags & FERRULE_HIP_GEMV_BLOCK_MAJOR_WEIGHTS) != 0;
  hipError_t e;
  if (first.weight_format == kFp4) {
    e = block_major ? launch_skinny<kFp4, kE8m0, true>(launch, stream) : launch_skinny<kFp4, kE8m0, false>(launch, stream);
  } else if (first.scale_kind == kE8m0) {
    e = block_major ? launch_skinny<kFp8, kE8m0, true>(launch, stream) : launch_skinny<kFp8, kE8m0, false>(launch, stream);
  } else {
    e = block_major ? launch_skinny<kFp8, kF32, true>(launch, stream) : launch_skinny<kFp8, kF32, false>(launch, stream);
  }
  if (e != hipSuccess) {
    g_last_hip_error = static_cast<int32_t>(e);
    return FERRULE_HIP_LAUNCH_FAILED;
  }
  return take_launch_error() == hipSuccess ? FERRULE_HIP_SUCCESS : FERRULE_HIP_LAUNCH_FAILED;
}

int32_t validate_multi(const FerruleHipQuantGemvMultiArgs *a) {
  if (a == nullptr || a->count == 0 || a->matrices == 0) return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->count > kMaxMatrices) return FERRULE_HIP_UNSUPPORTED;
  const FerruleHipQuantGemvArgs *list = reinterpret_cast<const FerruleHipQuantGemvArgs *>(static_cast<uintptr_t>(a->matrices));
  for (uint32_t m = 0; m < a->count; ++m) {
    const int32_t status = validate(&list[m], true);
    if (status != FERRULE_HIP_SUCCESS) return status;
    // one kernel instantiation and one stream per launch
    if (list[m].weight_format != list[0].weight_format || list[m].scale_kind != list[0].scale_kind ||
        ((list[m].flags ^ list[0].flags) & FERRULE_HIP_GEMV_BLOCK_MAJOR_WEIGHTS) != 0 || list[m].stream != list[0].stream ||
        skinny_ok(list[m]) != skinny_ok(list[0]))
      return FERRULE_HIP_INVALID_ARGUMENT;
  }
  return FERRULE_HIP_SUCCESS;
}

// The three linears of the dense decode FFN as GEMV blocks (gate, up: [intermediate, input];
// down: [output, intermediate]), for the shared validation.
void ffn_linears(const FerruleHipDenseFfnDecodeArgs &a, FerruleHipQuantGemvArgs (&out)[3]) {
  const uint64_t weights[3] = {a.gate_weight, a.up_weight, a.down_weight};
  const uint64_t scales[3] = {a.gate_scales, a.up_scales, a.down_scales};
  for (int i = 0; i < 3; ++i) {
    FerruleHipQuantGemvArgs &l = out[i];
    l.weight_format = a.weight_format;
    l.scale_kind = a.scale_kind;
    l.batch = a.batch;
    l.n = i < 2 ? a.intermediate_size : a.output_size;
    l.k = i < 2 ? a.input_size : a.intermediate_size;
    l.block_m = a.block_m;
    l.block_k = a.block_k;
    l.scale_cols = a.block_k == 0 ? 0 : (l.k + a.block_k - 1u) / a.block_k;
    l.flags = (a.flags & FERRULE_HIP_GEMV_BLOCK_MAJOR_WEIGHTS) | (i == 2 ? (a.flags & FERRULE_HIP_GEMV_OUTPUT_F32) : FERRULE_HIP_GEMV_OUTPUT_F32);
    l.reserved = 0;
    // gate sums [batch, intermediate] f32, then the up sums
    const uint64_t up_sums = a.hidden_f32 + static_cast<uint64_t>(a.batch) * a.intermediate_size * sizeof(float);
    l.x = i < 2 ? a.x : a.hidden_f32;
    l.weight = weights[i];
    l.weight_scales = scales[i];
    l.output = i == 0 ? a.hidden_f32 : (i == 1 ? up_sums : a.output);
    l.stream = a.stream;
  }
}

int32_t validate_ffn(const FerruleHipDenseFfnDecodeArgs *a) {
  if (a == nullptr) return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->input_size == 0 || a->intermediate_size == 0 || a->output_size == 0) return FERRULE_HIP_INVALID_ARGUMENT;
  if (!(a->swiglu_limit >= 0.0f)) return FERRULE_HIP_INVALID_ARGUMENT;
  FerruleHipQuantGemvArgs linears[3];
  ffn_linears(*a, linears);
  for (const FerruleHipQuantGemvArgs &l : linears) {
    const int32_t status = validate(&l, true);
    if (status != FERRULE_HIP_SUCCESS) return status;
    if (!skinny_ok(l)) return FERRULE_HIP_UNSUPPORTED;   // whole 128-wide K blocks only
  }
  return FERRULE_HIP_SUCCESS;
}

}  // namespace
}  // namespace ferrule_hip

using namespace ferrule_hip;

extern "C" int32_t ferrule_hip_dense_ffn_decode_can_implement(const FerruleHipDenseFfnDecodeArgs *args) {
  return validate_ffn(args);
}

extern "C" int32_t ferrule_hip_dense_ffn_decode_launch(const FerruleHipDenseFfnDecodeArgs *args) {
  const int32_t status = validate_ffn(args);
  if (status != FERRULE_HIP_SUCCESS) return status;
  FerruleHipQuantGemvArgs linears[3];
  ffn_linears(*args, linears);
  // gate and up in one launch (twice the workgroups of either: a decode FFN's intermediate size
  // alone does not fill the machine), f32 sums out
  const FerruleHipQuantGemvArgs *first[2] = {&linears[0], &linears[1]};
  const int32_t sums = launch_matrices(first, 2);
  if (sums != FERRULE_HIP_SUCCESS) return sums;
  GemvParams down = make_params(linears[2]);
  down.x_up = reinterpret_cast<const float *>(static_cast<uintptr_t>(linears[1].output));
  down.swiglu_limit = args->swiglu_limit;
  down.output_scale = args->output_scale;
  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(args->stream));
  const bool block_major = (args->flags & FERRULE_HIP_GEMV_BLOCK_MAJOR_WEIGHTS) != 0;
  clear_launch_error();
  hipError_t e;
  if (args->weight_format == kFp4) {
    e = block_major ? launch_swiglu_down<kFp4, kE8m0, true>(down, stream) : launch_swiglu_down<kFp4, kE8m0, false>(down, stream);
  } else if (args->scale_kind == kE8m0) {
    e = block_major ? launch_swiglu_down<kFp8, kE8m0, true>(down, stream) : launch_swiglu_down<kFp8, kE8m0, false>(down, stream);
  } else {
    e = block_major ? launch_swiglu_down<kFp8, kF32, true>(down, stream) : launch_swiglu_down<kFp8, kF32, false>(down, stream);
  }
  if (e != hipSuccess) {
    g_last_hip_error = static_cast<int32_t>(e);
    return FERRULE_HIP_LAUNCH_FAILED;
  }
  return take_launch_error() == hipSuccess ? FERRULE_HIP_SUCCESS : FERRULE_HIP_LAUNCH_FAILED;
}

extern "C" int32_t ferrule_hip_quant_gemv_can_implement(const FerruleHipQuantGemvArgs *args) {
  return validate(args, true);
}

extern "C" int32_t ferrule_hip_quant_gemv_launch(const FerruleHipQuantGemvArgs *args) {
  const int32_t status = validate(args, true);
  if (status != FERRULE_HIP_SUCCESS) return status;
  return launch_matrices(&args, 1);
}

extern "C" int32_t ferrule_hip_quant_gemv_multi_can_implement(const FerruleHipQuantGemvMultiArgs *args) {
  return validate_multi(args);
}

extern "C" int32_t ferrule_hip_quant_gemv_multi_launch(const FerruleHipQuantGemvMultiArgs *args) {
  const int32_t status = validate_multi(args);
  if (status != FERRULE_HIP_SUCCESS) return status;
  const FerruleHipQuantGemvArgs *list = reinterpret_cast<const FerruleHipQuantGemvArgs *>(static_cast<uintptr_t>(args->matrices));
  const FerruleHipQuantGemvArgs *each[kMaxMatrices];
  for (uint32_t m = 0; m < args->count; ++m) each[m] = &list[m];
  return launch_matrices(each, args->count);
}

extern "C" int32_t ferrule_hip_dequant_launch(const FerruleHipQuantGemvArgs *args) {
  const int32_t status = validate(args, false);
  if (status != FERRULE_HIP_SUCCESS) return status;
  if (args->weight_format == kFp4 ? (args->k % 8u != 0) : (args->k % 4u != 0 || args->block_k % 4u != 0))
    return FERRULE_HIP_UNSUPPORTED;
  const GemvParams p = make_params(*args);
  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(args->stream));
  clear_launch_error();
  const size_t dwords = static_cast<size_t>(p.n) * (args->weight_format == kFp4 ? p.k / 8u : p.k / 4u);
  const uint32_t blocks = static_cast<uint32_t>((dwords + 255u) / 256u);
  if (args->weight_format == kFp4) {
    dequant_kernel<kFp4, kE8m0><<<blocks, 256, 0, stream>>>(p);
  } else if (args->scale_kind == kE8m0) {
    dequant_kernel<kFp8, kE8m0><<<blocks, 256, 0, stream>>>(p);
  } else {
    dequant_kernel<kFp8, kF32><<<blocks, 256, 0, stream>>>(p);
  }
  return take_launch_error() == hipSuccess ? FERRULE_HIP_SUCCESS : FERRULE_HIP_LAUNCH_FAILED;
}
