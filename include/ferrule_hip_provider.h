/*
 * ferrule_hip_provider.h - C ABI of the MI355X (gfx950) quantized-weight matmul
 * provider for Ferrule.
 *
 * Contract (the same one Ferrule's native providers obey,
 * docs/ARCHITECTURE.md:265-293): every entry point takes ONE pointer to a POD
 * argument block; device pointers and the hipStream_t are carried as uint64_t;
 * the caller owns streams, device memory and workspace and keeps them alive for
 * the asynchronous work; the provider allocates nothing, never synchronises the
 * host, keeps no request state and never picks a semantic fallback.
 *
 * Two families of entry points:
 *   (1) drop-ins for reference symbols: the argument block is byte-identical to
 *       the reference struct named in the comment (sizes and offsets are
 *       static_assert-ed below) and the return convention is the reference's;
 *   (2) decode-path entry points that have no reference symbol, because the
 *       reference has no BF16-activation GEMV and no MXFP4 GEMV at all
 *       (crates/ferrule-backend/src/cuda/context.rs:10909-10911, 10981-10983).
 *
 * Return conventions:
 *   ferrule_hip_core_* : int32_t hipError_t, 0 = ok, 1 = hipErrorInvalidValue
 *                        (reference: cudaError_t, portable/entrypoints.cu:34-36).
 *   everything else    : FerruleHipStatus, numerically equal to
 *                        FerruleCutlassStatus (abi/cutlass_provider.h:26-31).
 */
#ifndef FERRULE_HIP_PROVIDER_H_
#define FERRULE_HIP_PROVIDER_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* abi/cutlass_provider.h:26-31 */
typedef enum FerruleHipStatus {
  FERRULE_HIP_SUCCESS = 0,
  FERRULE_HIP_INVALID_ARGUMENT = 2,
  FERRULE_HIP_LAUNCH_FAILED = 3,
  FERRULE_HIP_UNSUPPORTED = 4,
} FerruleHipStatus;

/* Kernel ids and manifest: abi/cutlass_provider.h:14-35. A bit is set only if
 * that operation is fully implemented by this library. */
#define FERRULE_HIP_KERNEL_FP8_QUERY_A_KV 1u
#define FERRULE_HIP_KERNEL_SHARED_FFN 4u
#define FERRULE_HIP_KERNEL_GROUPED_FP4_MOE 5u
#define FERRULE_HIP_KERNEL_FP8_PROJECTION 10u
/* ids above 32 are HIP-only capabilities with no reference id */
#define FERRULE_HIP_KERNEL_QUANT_GEMV 33u
#define FERRULE_HIP_KERNEL_MOE_DECODE 34u
#define FERRULE_HIP_KERNEL_FP8_BLOCK_GEMM 35u
#define FERRULE_HIP_KERNEL_BIT(id) (1ull << ((id) - 1u))

typedef struct FerruleHipProviderManifest {
  uint64_t kernel_mask;
} FerruleHipProviderManifest;

/* replaces ferrule_cutlass_provider_manifest (abi/cutlass_provider.h:390) */
FerruleHipProviderManifest ferrule_hip_provider_manifest(void);

/* Diagnostic with no reference counterpart: the raw hipError_t behind the calling
 * thread's most recent FERRULE_HIP_LAUNCH_FAILED (0 if none). Ferrule's error text
 * carries the native code (crates/ferrule-backend/src/cuda/cutlass.rs:2938-2963). */
int32_t ferrule_hip_last_error_code(void);

/* ------------------------------------------------------------------------ */
/* (1) drop-ins for ferrule_core_* (abi/core_provider.h)                     */
/* ------------------------------------------------------------------------ */

/* abi/core_provider.h:11-19 (only the quantized kinds are implemented) */
typedef enum FerruleHipLinearKind {
  FERRULE_HIP_LINEAR_FP8_E4M3_E8M0 = 4,
  FERRULE_HIP_LINEAR_FP8_E4M3_E8M0_PACKED = 5,
  FERRULE_HIP_LINEAR_FP8_E4M3_E8M0_FROM_F32 = 8,
} FerruleHipLinearKind;

/* byte-identical to FerruleCoreLinearArgs, abi/core_provider.h:21-37 (88 B) */
typedef struct FerruleHipLinearArgs {
  uint32_t kind;
  uint32_t batch;
  uint32_t n;
  uint32_t k;
  uint32_t scale_cols;
  uint32_t block_m;
  uint32_t block_k;
  uint32_t packed_offset;
  uint32_t scale_offset;
  uint64_t x;             /* kind 4/8: f32 [batch,k]; kind 5: e4m3 [batch,k] */
  uint64_t x_scales;      /* kind 5: e8m0 [batch, scale_cols] */
  uint64_t weight;        /* e4m3 [n,k] */
  uint64_t weight_scales; /* e8m0 [ceil(n/block_m), scale_cols] */
  uint64_t output;        /* f32 [batch,n] */
  uint64_t stream;
} FerruleHipLinearArgs;

/* replaces ferrule_core_linear_launch (abi/core_provider.h:477; kernel
 * portable/entrypoints.cu:208-284, kinds 4, 5, 8). Other kinds return 1. */
int32_t ferrule_hip_core_linear_launch(const FerruleHipLinearArgs *args);

/* abi/core_provider.h:79-85 (packed kinds only) */
typedef enum FerruleHipQuantizeKind {
  FERRULE_HIP_QUANTIZE_FP4_PACKED = 4,
  FERRULE_HIP_QUANTIZE_FP8_PACKED = 5,
} FerruleHipQuantizeKind;

/* `reserved` of the reference struct selects the FP8 tie rule. The reference is
 * three-way inconsistent here: its CPU path rounds the mantissa half away from
 * zero (crates/ferrule-model/src/checkpoint/encoding.rs:348-381), its portable
 * GPU kernel uses rintf (portable/entrypoints.cu:142-179). 0 (what a caller
 * that zeroes `reserved` gets) = the CPU path, which is the parity contract. */
#define FERRULE_HIP_FP8_ROUND_CPU_REFERENCE 0u
#define FERRULE_HIP_FP8_ROUND_HALF_EVEN 1u

/* byte-identical to FerruleCoreQuantizeArgs, abi/core_provider.h:87-99 (64 B) */
typedef struct FerruleHipQuantizeArgs {
  uint32_t kind;
  uint32_t value_offset;
  uint32_t value_len;
  uint32_t row_width;
  uint32_t block_size;
  uint32_t rope_dim;
  uint32_t reserved; /* FERRULE_HIP_FP8_ROUND_* */
  uint64_t values;   /* f32 [value_len] */
  uint64_t packed;   /* kind 5: e4m3 [value_len]; kind 4: e2m1 [value_len/2] */
  uint64_t scales;   /* e8m0 [value_len / block_size] */
  uint64_t stream;
} FerruleHipQuantizeArgs;

/* replaces ferrule_core_quantize_launch (abi/core_provider.h:481; kernel
 * portable/entrypoints.cu:342-448, kinds 4 and 5). */
int32_t ferrule_hip_core_quantize_launch(const FerruleHipQuantizeArgs *args);

/* ------------------------------------------------------------------------ */
/* (2) decode GEMV: no reference symbol                                      */
/* ------------------------------------------------------------------------ */

typedef enum FerruleHipWeightFormat {
  FERRULE_HIP_WEIGHT_FP8_E4M3 = 1,  /* [n,k] bytes */
  FERRULE_HIP_WEIGHT_MXFP4_E2M1 = 2 /* [n,k/2] bytes, low nibble = even k */
} FerruleHipWeightFormat;

typedef enum FerruleHipScaleKind {
  FERRULE_HIP_SCALE_E8M0 = 0, /* 1 byte, 2^(b-127); what Ferrule's checkpoints carry */
  FERRULE_HIP_SCALE_F32 = 1   /* 4 bytes; FP8 only */
} FerruleHipScaleKind;

#define FERRULE_HIP_GEMV_OUTPUT_F32 1u /* flags bit0: write f32 instead of bf16 */

/* y[b,n] = bf16( sum_k x[b,k] * dequant(W)[n,k] ), fp32 accumulation.
 * Semantics: LinearWeight::reference_matvec
 * (crates/ferrule-model/src/checkpoint/weight.rs:154-173) applied to each row
 * of x, followed by round_to_bf16 (models/common/math.rs:7-14).
 * MXFP4: block_m = 1, block_k = 32, scales e8m0 [n, k/32].
 * FP8  : scales [ceil(n/block_m), ceil(k/block_k)], e8m0 bytes or f32.
 * Pointers 16-byte aligned. */
typedef struct FerruleHipQuantGemvArgs {
  uint32_t weight_format; /* FerruleHipWeightFormat */
  uint32_t scale_kind;    /* FerruleHipScaleKind */
  uint32_t batch;
  uint32_t n;
  uint32_t k;
  uint32_t block_m;
  uint32_t block_k;
  uint32_t scale_cols;
  uint32_t flags;
  uint32_t reserved;
  uint64_t x;             /* bf16 [batch,k] */
  uint64_t weight;
  uint64_t weight_scales;
  uint64_t output;        /* bf16 (or f32) [batch,n] */
  uint64_t stream;
} FerruleHipQuantGemvArgs;

int32_t ferrule_hip_quant_gemv_can_implement(const FerruleHipQuantGemvArgs *args);
int32_t ferrule_hip_quant_gemv_launch(const FerruleHipQuantGemvArgs *args);

/* Test/diagnostic entry: element-wise dequantisation of a weight to f32 [n,k],
 * computed with exactly the device conversion path the GEMV/GEMM kernels use.
 * Semantics: dequantize_fp4_e2m1_with_e8m0_scales / dequantize_fp8_e4m3fn_with_e8m0_scales
 * (crates/ferrule-model/src/checkpoint/encoding.rs:82-198). Uses the
 * FerruleHipQuantGemvArgs block: x and batch are ignored, output is f32 [n,k]. */
int32_t ferrule_hip_dequant_launch(const FerruleHipQuantGemvArgs *args);

#ifdef __cplusplus
} /* extern "C" */

#define FERRULE_HIP_ASSERT_LAYOUT(type, size, first_u64, first_u64_offset,     \
                                  stream_offset)                               \
  static_assert(sizeof(type) == size, #type " size mismatch");                 \
  static_assert(alignof(type) == alignof(uint64_t), #type " alignment");       \
  static_assert(offsetof(type, first_u64) == first_u64_offset,                 \
                #type " first uint64_t offset mismatch");                      \
  static_assert(offsetof(type, stream) == stream_offset,                       \
                #type " stream offset mismatch")

/* abi/core_provider.h:512-535 */
FERRULE_HIP_ASSERT_LAYOUT(FerruleHipLinearArgs, 88, x, 40, 80);
FERRULE_HIP_ASSERT_LAYOUT(FerruleHipQuantizeArgs, 64, values, 32, 56);
FERRULE_HIP_ASSERT_LAYOUT(FerruleHipQuantGemvArgs, 80, x, 40, 72);
static_assert(sizeof(FerruleHipProviderManifest) == 8, "manifest size");
#endif

#endif /* FERRULE_HIP_PROVIDER_H_ */
