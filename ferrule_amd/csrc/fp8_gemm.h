// Internal interface of the FP8 block-scaled GEMM (fp8_gemm.hip) for the other entry points
// of the library that end in such a GEMM (the shared FFN's down projection).
#pragma once

#include <stdint.h>

namespace ferrule_hip {

struct Fp8GemmParams {
  const uint8_t *x;   // E4M3 [m, k]
  const uint8_t *xs;  // UE8M0 [m, k/128]
  const uint8_t *w;   // E4M3 [n, k]
  const void *ws;     // UE8M0 or f32 [ceil(n/128), k/128]
  void *out;          // [m, n]
  uint32_t m, n, k, cols;
  // an optional second weight matrix over the same activations in the same launch (n2 = 0: none)
  const uint8_t *w2 = nullptr;
  const void *ws2 = nullptr;
  void *out2 = nullptr;
  uint32_t n2 = 0;
};

constexpr int kGemmOutF32Rounded = 0;     // f32 holding BF16-rounded values (fp8_projection.cuh:398-414)
constexpr int kGemmOutBf16 = 1;
constexpr int kGemmOutF32Raw = 2;         // unrounded fp32 sums
constexpr int kGemmOutF32Accumulate = 3;  // out += unrounded fp32 sums

// FerruleHipStatus; validation is the caller's.  The row count decides the schedule: up to
// kFp8RowsMax rows stream the weights once, one wave per 16 features (fp8_rows.hip), more rows
// run MFMA tiles of 128 or 256 rows (fp8_gemm.hip); `tiles_only` keeps the tiles for any row
// count.  Both give the same bits for a row.
constexpr uint32_t kFp8RowsMax = 32;
int32_t fp8_gemm_run(const Fp8GemmParams &p, bool f32_scales, int out_mode, uint64_t stream_bits,
                     bool tiles_only = false);
uint32_t fp8_gemm_lds_bytes_small(uint32_t scale_cols);

// fp8_rows.hip
bool fp8_rows_applies(uint32_t rows, uint32_t k);
int32_t fp8_rows_run(const Fp8GemmParams &p, bool f32_scales, int out_mode, uint64_t stream_bits);
// hidden_f32 [rows, intermediate] = silu(x W1^T) * (x W3^T) * output_scale (clamped first when
// swiglu_limit > 0; non-finite values stored as 0), E8M0 block scales, rows <= kFp8RowsMax
int32_t fp8_rows_swiglu_run(const uint8_t *x, const uint8_t *xs, const uint8_t *gate, const uint8_t *gate_s,
                            const uint8_t *up, const uint8_t *up_s, float *hidden_f32, uint32_t rows,
                            uint32_t input_size, uint32_t intermediate_size, float output_scale, float swiglu_limit,
                            uint64_t stream_bits);

}  // namespace ferrule_hip
