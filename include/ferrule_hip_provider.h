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
#define FERRULE_HIP_KERNEL_DENSE_FFN_DECODE 36u
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

/* Build identity with no reference counterpart (the reference links statically from
 * the same checkout, docs/ARCHITECTURE.md:271-274, so it cannot go stale): a
 * NUL-terminated hexadecimal sha256 of every source and header this library was
 * compiled from, for a host that loads the library dynamically to refuse one built
 * from other argument-block layouts. "unknown" when built without the digest. */
const char *ferrule_hip_source_digest(void);

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

/* abi/core_provider.h:347-353 */
typedef enum FerruleHipExpertGroupRoutePlanKind {
  FERRULE_HIP_EXPERT_GROUP_ROUTE_INIT_INVOCATION = 1,
  FERRULE_HIP_EXPERT_GROUP_ROUTE_INIT_PLAN = 2,
  FERRULE_HIP_EXPERT_GROUP_ROUTE_COUNT = 3,
  FERRULE_HIP_EXPERT_GROUP_ROUTE_COMPACT = 4,
  FERRULE_HIP_EXPERT_GROUP_ROUTE_SCATTER = 5,
  /* No reference counterpart: kinds 2..5 in ONE launch (one workgroup), preceded by the flag
   * half of kind 1 (route_written[0..route_count) = 0, route_error = 0; route_output is NOT
   * cleared - ferrule_hip_moe_decode_launch never reads a route it has not written).  Every
   * plan buffer ends up exactly as after kinds 2,3,4,5.  For decode batches:
   * route_count <= 2048 and slot_capacity <= 1024, hipErrorInvalidValue (1) beyond. */
  FERRULE_HIP_EXPERT_GROUP_ROUTE_FUSED_DECODE_PLAN = 16,
} FerruleHipExpertGroupRoutePlanKind;

#define FERRULE_HIP_FUSED_PLAN_MAX_ROUTES 2048u

/* byte-identical to FerruleCoreExpertGroupRoutePlanArgs, abi/core_provider.h:355-382
 * (184 B). All metadata arrays are int32 except router_weights/route_weights/
 * route_output (f32). */
typedef struct FerruleHipExpertGroupRoutePlanArgs {
  uint32_t kind;
  uint32_t route_count;
  uint32_t routes_per_token;
  uint32_t slot_capacity;
  uint32_t route_capacity;
  uint32_t output_elements;
  uint32_t small_group_row_limit;
  uint64_t route_slots;
  uint64_t route_generations;
  uint64_t router_weights;
  uint64_t slot_generations;
  uint64_t slot_counts;
  uint64_t slot_route_offsets;
  uint64_t slot_cursors;
  uint64_t active_expert_slots;
  uint64_t active_group_generations;
  uint64_t expert_route_indptr;
  uint64_t expert_route_counts;
  uint64_t route_token_indices;
  uint64_t route_indices;
  uint64_t route_weights;
  uint64_t host_scalars; /* int32[4]: groups, small groups, max rows, total rows */
  uint64_t route_output;
  uint64_t route_written;
  uint64_t route_error;
  uint64_t stream;
} FerruleHipExpertGroupRoutePlanArgs;

/* replaces ferrule_core_expert_group_route_plan_launch (abi/core_provider.h:490;
 * kernel portable/entrypoints.cu:1382-1513). Same five kinds, same outputs; the
 * compaction is a parallel scan instead of one thread, and rows inside a group are
 * in ascending route order (the reference's order is atomic-cursor nondeterministic,
 * so any order is within its contract). slot_capacity <= 1024. */
int32_t ferrule_hip_core_expert_group_route_plan_launch(
    const FerruleHipExpertGroupRoutePlanArgs *args);

/* abi/core_provider.h:384-390 (only the kinds on the quantized MoE path) */
typedef enum FerruleHipMoeKind {
  FERRULE_HIP_MOE_WEIGHTED_SWIGLU_F32 = 2,
  FERRULE_HIP_MOE_REDUCE_ROUTES = 7,
  FERRULE_HIP_MOE_REDUCE_EXPERT_GROUP_ROUTES = 8,
} FerruleHipMoeKind;

/* byte-identical to FerruleCoreMoeArgs, abi/core_provider.h:392-429 (248 B) */
typedef struct FerruleHipMoeArgs {
  uint32_t kind;
  uint32_t n;
  uint32_t k;
  uint32_t batch_columns;
  uint32_t experts;
  uint32_t tokens;
  uint32_t routes_per_token;
  uint32_t output_offset;
  uint32_t hidden;
  float route_weight;
  float swiglu_limit;
  uint64_t input;
  uint64_t input_scales;
  uint64_t gate_ptrs;
  uint64_t gate_scale_ptrs;
  uint64_t up_ptrs;
  uint64_t up_scale_ptrs;
  uint64_t down_ptrs;
  uint64_t down_scale_ptrs;
  uint64_t gate;
  uint64_t up;
  uint64_t route_weights;
  uint64_t hidden_values;
  uint64_t hidden_packed;
  uint64_t hidden_scales;
  uint64_t expert_output;
  uint64_t resident_output;
  uint64_t materialized_output;
  uint64_t route_slots;
  uint64_t materialized_route_slots;
  uint64_t miss_markers;
  uint64_t route_output;
  uint64_t route_written;
  uint64_t route_error;
  uint64_t output;
  uint64_t stream;
} FerruleHipMoeArgs;

/* replaces ferrule_core_moe_launch for kinds 2, 7, 8 (abi/core_provider.h:493;
 * kernel portable/entrypoints.cu:1515-1612): weighted SwiGLU on f32 gate/up, and the
 * rank-ordered fp32 combine of route outputs into the (f32-held, BF16-rounded)
 * output, kind 8 writing NaN for tokens with a missing route. */
int32_t ferrule_hip_core_moe_launch(const FerruleHipMoeArgs *args);

/* abi/core_provider.h:204-209 */
typedef enum FerruleHipRouterKind {
  FERRULE_HIP_ROUTER_TOPK = 1,
  FERRULE_HIP_ROUTER_HASH = 2,
  FERRULE_HIP_VOCAB_TOPK_F32_INDEX = 3,
  FERRULE_HIP_VOCAB_TOPK_I32_INDEX = 4,
} FerruleHipRouterKind;

/* byte-identical to FerruleCoreRouterArgs, abi/core_provider.h:211-228 (96 B) */
typedef struct FerruleHipRouterArgs {
  uint32_t kind;
  uint32_t rows;
  uint32_t columns;
  uint32_t k;            /* 1..64; 0 or more than 64 is a successful no-op, as in the reference */
  uint32_t hash_rows;
  uint32_t hash_columns;
  uint32_t flags;        /* bit 0: add bias[column] to the selection value (kind 1) */
  float route_scale;
  uint32_t reserved;
  uint64_t logits;       /* f32 [rows, columns] */
  uint64_t bias;         /* f32 [columns], kind 1 with flags & 1 */
  uint64_t token_ids;    /* i32 [rows], kind 2 */
  uint64_t hash_table;   /* i32 [hash_rows, hash_columns], kind 2 */
  uint64_t indices;      /* i32 [rows, k] (f32 for kind 3) */
  uint64_t weights;      /* f32 [rows, k] */
  uint64_t stream;
} FerruleHipRouterArgs;

/* replaces ferrule_core_router_launch (abi/core_provider.h:486; kernel
 * portable/entrypoints.cu:770-884, launch :1969-1977): sqrt-softplus score top-k or
 * hash-table routing with normalised, scaled route weights (kinds 1, 2), and the plain
 * top-k of a row (kinds 3, 4).  The outputs are the route ids and weights that the
 * expert-group route plan reads, so a layer's routing never leaves the device.  Null
 * args, an unknown kind or a null pointer that the kind reads returns 1. */
int32_t ferrule_hip_core_router_launch(const FerruleHipRouterArgs *args);

/* abi/core_provider.h:294-300 */
typedef enum FerruleHipExpertTableKind {
  FERRULE_HIP_EXPERT_INSTALL = 1,
  FERRULE_HIP_EXPERT_EVICT = 2,
  FERRULE_HIP_EXPERT_INITIALIZE_RESOLVE = 3,
  FERRULE_HIP_EXPERT_RESOLVE = 4,
  FERRULE_HIP_EXPERT_GATHER_DISPATCH = 5,
} FerruleHipExpertTableKind;

/* byte-identical to FerruleCoreExpertTableArgs, abi/core_provider.h:302-345 (296 B) */
typedef struct FerruleHipExpertTableArgs {
  uint32_t kind;
  uint32_t route_count;
  uint32_t expert_capacity;
  uint32_t slot_capacity;
  uint32_t miss_capacity;
  uint32_t route_capacity;
  uint32_t expert;
  uint32_t slot;
  int32_t generation;
  int32_t active_value;
  uint32_t reserved;
  uint64_t gate_weights;        /* u64 [slot_capacity]: the slot table, six pointer arrays */
  uint64_t gate_scales;
  uint64_t up_weights;
  uint64_t up_scales;
  uint64_t down_weights;
  uint64_t down_scales;
  uint64_t expert_to_slot;      /* i32 [expert_capacity], -1 = not resident */
  uint64_t expert_generations;  /* i32 [expert_capacity], 0 = not resident */
  uint64_t slot_generations;    /* i32 [slot_capacity] */
  uint64_t expert_ids;          /* i32 [routes]: kind 4 in; kind 5 out (route index or -1) */
  uint64_t route_slots;         /* i32 [routes]: kind 4 out, kind 5 in */
  uint64_t route_generations;   /* i32 [routes]: kind 4 out, kind 5 in */
  uint64_t miss_markers;        /* i32 [routes] */
  uint64_t miss_control;        /* i32 [2 + miss_capacity + route_capacity]: count, overflow,
                                   missing ids, then every route's expert id */
  uint64_t router_weights;      /* f32 [routes], kind 5 */
  uint64_t active_markers;      /* i32 [routes], kind 5 */
  uint64_t output_gate_weights; /* u64 [routes], kind 5 ... */
  uint64_t output_gate_scales;
  uint64_t output_up_weights;
  uint64_t output_up_scales;
  uint64_t output_down_weights;
  uint64_t output_down_scales;
  uint64_t output_route_weights; /* f32 [routes] */
  uint64_t dispatch_error;       /* i32 [1] */
  uint64_t gate_weight_value;    /* kind 1: the six pointers to publish */
  uint64_t gate_scale_value;
  uint64_t up_weight_value;
  uint64_t up_scale_value;
  uint64_t down_weight_value;
  uint64_t down_scale_value;
  uint64_t stream;
} FerruleHipExpertTableArgs;

/* replaces ferrule_core_expert_table_launch (abi/core_provider.h:490; kernel
 * portable/entrypoints.cu:1268-1380, launch :2006-2027), kinds 1-5: publish and retire
 * slot bindings, resolve router expert ids to (slot, generation) with a bounded miss
 * list, gather per-route dispatch pointers.  Beyond the reference's null check, kinds
 * 1/2 return 1 for an expert or slot outside the capacities given in the block (the
 * kernel would write out of bounds), and every kind returns 1 for a null pointer among
 * the arrays it touches. */
int32_t ferrule_hip_core_expert_table_launch(const FerruleHipExpertTableArgs *args);

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
/* flags bit1 (quant_gemv only): weight (and, for MXFP4, weight_scales) address the block-major
 * order written by ferrule_hip_prepare_mxfp4_block_major / ferrule_hip_prepare_fp8_block_major;
 * n % 16 == 0, k % 128 == 0, FP8 block_k % 128 == 0 */
#define FERRULE_HIP_GEMV_BLOCK_MAJOR_WEIGHTS 2u

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

/* Several independent decode linears in ONE launch, in the role of
 * ferrule_core_dual_linear_launch / ferrule_core_grouped_linear_launch
 * (abi/core_provider.h:39-77, 478-480; portable/entrypoints.cu:286-340), which run
 * two projections of one activation, or the grouped output projection, in a single
 * kernel: a decode-sized GEMV spends as long on launch, address set-up and drain as
 * on streaming its weights, and that cost is paid once per launch.
 * `matrices` is a HOST pointer to `count` (1..FERRULE_HIP_GEMV_MULTI_MAX)
 * FerruleHipQuantGemvArgs blocks, read during the call only; each matrix has its own
 * shape, activations, batch and output, all share weight_format, scale_kind, the
 * block-major flag and the stream (of the first block).  Results are those of `count`
 * single launches, bit for bit (launches with many row tiles run smaller workgroups, which
 * changes no sum: a row's K slices are added in a fixed order). */
#define FERRULE_HIP_GEMV_MULTI_MAX 32u
typedef struct FerruleHipQuantGemvMultiArgs {
  uint32_t count;
  uint32_t reserved;
  uint64_t matrices; /* host address of FerruleHipQuantGemvArgs[count] */
} FerruleHipQuantGemvMultiArgs;

int32_t ferrule_hip_quant_gemv_multi_can_implement(const FerruleHipQuantGemvMultiArgs *args);
int32_t ferrule_hip_quant_gemv_multi_launch(const FerruleHipQuantGemvMultiArgs *args);

/* Dense SwiGLU FFN for a decode batch in GEMV form, HBM bound (no reference symbol; the
 * reference runs its shared FFN for M in {1, 2, 4, 8, 17} rows on the tensor-core path,
 * capabilities/shared_ffn.cuh:477-523):
 *   gate = W1 x, up = W3 x (fp32 accumulate); clamp when swiglu_limit > 0;
 *   hidden = silu(gate) * up * output_scale (f32, no rounding, no activation quantisation);
 *   y = W2 hidden (fp32 accumulate), one BF16 (or f32) writeback
 * i.e. SwiGluFfn::reference_execute (crates/ferrule-model/src/ffn.rs:24-48) over quantized
 * LinearWeights (checkpoint/weight.rs:154-173).  Two launches: gate and up as two matrices of
 * one GEMV launch (twice the workgroups of either, f32 sums out); the down projection computes
 * the hidden values from those sums as it stages them and splits each exactly into three BF16
 * rows.  The hidden values themselves are never stored.  The three linears share
 * weight_format, scale_kind, block_m / block_k and the weight order; input_size and
 * intermediate_size are multiples of 128.  `hidden_f32` is scratch between the two launches
 * (caller-owned, 16-byte aligned): f32 [2, batch, intermediate_size], the gate sums followed
 * by the up sums.
 * flags: FERRULE_HIP_GEMV_OUTPUT_F32, FERRULE_HIP_GEMV_BLOCK_MAJOR_WEIGHTS as above. */
typedef struct FerruleHipDenseFfnDecodeArgs {
  uint32_t weight_format; /* FerruleHipWeightFormat */
  uint32_t scale_kind;    /* FerruleHipScaleKind */
  uint32_t batch;
  uint32_t input_size;        /* k of gate / up */
  uint32_t intermediate_size; /* n of gate / up, k of down */
  uint32_t output_size;       /* n of down */
  uint32_t block_m;
  uint32_t block_k;
  uint32_t flags;
  uint32_t reserved;
  float swiglu_limit;
  float output_scale;
  uint64_t x;             /* bf16 [batch, input_size] */
  uint64_t gate_weight;
  uint64_t gate_scales;
  uint64_t up_weight;
  uint64_t up_scales;
  uint64_t down_weight;
  uint64_t down_scales;
  uint64_t hidden_f32;    /* f32 [2, batch, intermediate_size]: gate sums, up sums */
  uint64_t output;        /* bf16 (or f32) [batch, output_size] */
  uint64_t stream;
} FerruleHipDenseFfnDecodeArgs;

int32_t ferrule_hip_dense_ffn_decode_can_implement(const FerruleHipDenseFfnDecodeArgs *args);
int32_t ferrule_hip_dense_ffn_decode_launch(const FerruleHipDenseFfnDecodeArgs *args);

/* Test/diagnostic entry: element-wise dequantisation of a weight to f32 [n,k],
 * computed with exactly the device conversion path the GEMV/GEMM kernels use.
 * Semantics: dequantize_fp4_e2m1_with_e8m0_scales / dequantize_fp8_e4m3fn_with_e8m0_scales
 * (crates/ferrule-model/src/checkpoint/encoding.rs:82-198). Uses the
 * FerruleHipQuantGemvArgs block: x and batch are ignored, output is f32 [n,k]. */
int32_t ferrule_hip_dequant_launch(const FerruleHipQuantGemvArgs *args);

/* ------------------------------------------------------------------------ */
/* (2b) decode MoE layer: no reference symbol                                */
/* ------------------------------------------------------------------------ */

#define FERRULE_HIP_MOE_DECODE_COMBINE 1u      /* flags bit0: also write `output` */
#define FERRULE_HIP_MOE_DECODE_PREFIX_F32 2u   /* flags bit1: start the combine from prefix_f32 */
#define FERRULE_HIP_MOE_DECODE_SKIP_GATE_UP 4u /* flags bit2: hidden workspace already holds h */
#define FERRULE_HIP_MOE_DECODE_SKIP_DOWN 8u    /* flags bit3: stop after gate/up (+ combine if asked) */
/* flags bit4: every expert weight and scale pointer of the table addresses the block-major
 * order written by ferrule_hip_prepare_mxfp4_block_major (below) instead of the row-major
 * checkpoint order */
#define FERRULE_HIP_MOE_DECODE_BLOCK_MAJOR_WEIGHTS 16u

/* Routed MXFP4 experts over BF16 activations without activation quantisation:
 *   gate = W1 x, up = W3 x (fp32 accumulate); clamp when swiglu_limit > 0;
 *   h = silu(gate) * up * route_weight;  y_route = W2 h (fp32 accumulate)
 *   output[t,:] = bf16( prefix[t,:] + sum_rank y_route[t*k + rank, :] )   (rank order)
 * i.e. CpuReferenceExpertExecutor::execute with its default construction
 * (crates/ferrule-model/src/moe/executor.rs:82-124) per route, then the routed
 * accumulate (crates/ferrule-model/src/moe/routed.rs:85-110) and one BF16 round.
 * The group / row metadata and the slot pointer tables are exactly those of
 * FerruleCutlassGroupedFp4MoeArgs (abi/cutlass_provider.h:337-376), produced by the
 * route-plan entry above; weight scales are the LINEAR [n, k/32] E8M0 bytes.
 * `active_group_count` bounds the launch grid; when `host_scalars` is non-zero the
 * kernels read the true group count from host_scalars[0] on the device, so no host
 * round trip is needed between the plan and this launch.  Any upper bound of the active
 * groups is correct (the plan's capacity, say); the layer also chooses its launches from
 * it (num_routes <= 5 * active_group_count: packed kernels only, which take a long
 * expert's rows 8 at a time and stream its weights once per 8 rows), so a host that
 * knows the real count should pass it.
 * Workspace: ferrule_hip_moe_decode_workspace_size bytes, 256-byte aligned. */
typedef struct FerruleHipMoeDecodeArgs {
  uint32_t active_group_count;
  uint32_t slot_capacity;
  uint32_t total_routed_rows; /* capacity of the row arrays (>= real row count) */
  uint32_t num_tokens;
  uint32_t num_routes;
  uint32_t routes_per_token;
  uint32_t input_size;        /* H: k of gate/up, multiple of 512 */
  uint32_t intermediate_size; /* I: n of gate/up, k of down, multiple of 256 */
  uint32_t hidden_size;       /* n of down: a multiple of 128, or of 16 when at most 128 */
  uint32_t flags;
  float swiglu_limit;
  uint32_t reserved;

  uint64_t active_expert_slots;
  uint64_t expert_route_indptr;
  uint64_t route_token_indices;
  uint64_t route_indices;
  uint64_t route_weights;
  uint64_t host_scalars;

  uint64_t gate_ptrs;
  uint64_t gate_scale_ptrs;
  uint64_t up_ptrs;
  uint64_t up_scale_ptrs;
  uint64_t down_ptrs;
  uint64_t down_scale_ptrs;

  uint64_t input_bf16;   /* [num_tokens, input_size] */
  uint64_t route_output; /* f32 [num_routes, hidden_size] */
  uint64_t route_written;
  uint64_t route_error;
  uint64_t prefix_f32;   /* optional f32 [num_tokens, hidden_size] (shared-expert output) */
  uint64_t output;       /* bf16 [num_tokens, hidden_size] */

  uint64_t workspace;
  uint64_t workspace_bytes;
  uint64_t stream;
} FerruleHipMoeDecodeArgs;

/* Reads scalar fields only (pointers may be zero), like
 * ferrule_cutlass_grouped_fp4_moe_workspace_size (abi/cutlass_provider.h:446-449). */
uint64_t ferrule_hip_moe_decode_workspace_size(const FerruleHipMoeDecodeArgs *args);
int32_t ferrule_hip_moe_decode_can_implement(const FerruleHipMoeDecodeArgs *args);
int32_t ferrule_hip_moe_decode_launch(const FerruleHipMoeDecodeArgs *args);

/* ferrule_hip_moe_decode_launch for callers that cannot allocate device memory (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): the
 * same block, kernels and results, with the workspace regions taken from a fixed array
 * in the library's device image instead of the caller.  No counterpart in the reference,
 * whose callers always own the workspace (abi/cutlass_provider.h:446-449).
 *   - `workspace` and `workspace_bytes` must be zero; inputs and outputs are the caller's.
 *   - FERRULE_HIP_UNSUPPORTED when ferrule_hip_moe_decode_workspace_size(args) exceeds
 *     FERRULE_HIP_MOE_DECODE_STATIC_WORKSPACE_BYTES (16 MiB: e.g. 64 tokens x top-8 at
 *     input 7168 / intermediate 2048 needs 9.2 MiB); nothing is launched then.
 *   - Calls no hipMalloc / hipFree or any allocating routine.  The first call on a device
 *     looks the array's address up (hipGetSymbolAddress) with that device current: make
 *     that call outside stream capture, with the device of `stream` current.
 *   - Every call on one GPU shares that GPU's array.  Calls on one stream are ordered by
 *     the stream.  A call on another stream while the previous call's work has not
 *     completed returns FERRULE_HIP_UNSUPPORTED and launches nothing (an event recorded
 *     behind every launch is queried; the event is created once per GPU with the array's
 *     address).  Under stream capture the check is skipped: calls captured into graphs
 *     that may replay at the same time on one GPU race, and ordering them is the graph
 *     owner's business.  Each GPU holds
 *     its 16 MiB copy until the process ends.  The array keeps the previous call's
 *     contents; no output of the layer depends on a workspace byte that the same call has
 *     not written (rows of dropped routes may be read as stale values, which nothing consumes). */
#define FERRULE_HIP_MOE_DECODE_STATIC_WORKSPACE_BYTES (16u << 20)
int32_t ferrule_hip_moe_decode_launch_static_workspace(const FerruleHipMoeDecodeArgs *args);

/* Weight preparation for FERRULE_HIP_MOE_DECODE_BLOCK_MAJOR_WEIGHTS: no reference symbol; it
 * plays the part ferrule_cutlass_prepare_mxfp4_sfb (abi/cutlass_provider.h:454-456) plays for
 * the CUDA provider - a one-off reorder when an expert's weights are installed in a slot.
 * A [n, k] MXFP4 matrix is seen as n/16 tiles of 16 rows by k/128 K blocks; a row holds 64
 * payload bytes and 4 scale bytes per K block.
 *   source      payload [tile][row][kblock][64 B]   scales [tile][row][kblock][4 B]  (row-major)
 *   destination payload [tile][kblock][row][64 B]   scales [tile][kblock][row][4 B]
 * so the 16 rows x 64 B one wavefront fetches for one scaled MFMA are 1 KiB of consecutive
 * bytes. Sizes are unchanged (n*k/2 and n*k/32 bytes). n % 16 == 0, k % 128 == 0; pointers 16-byte
 * aligned; destination must not overlap source. */
typedef struct FerruleHipPrepareMxfp4BlockMajorArgs {
  uint32_t n;
  uint32_t k;
  uint64_t weight_source;      /* packed E2M1 [n, k/2] */
  uint64_t scale_source;       /* UE8M0 [n, k/32] */
  uint64_t weight_destination; /* n*k/2 bytes */
  uint64_t scale_destination;  /* n*k/32 bytes */
  uint64_t stream;
} FerruleHipPrepareMxfp4BlockMajorArgs;

int32_t ferrule_hip_prepare_mxfp4_block_major(const FerruleHipPrepareMxfp4BlockMajorArgs *args);

/* The same reorder for an FP8 [n, k] matrix (no reference symbol; one-off at artifact upload):
 * 16-row tiles of k/64 cells of 64 bytes per row, source [tile][row][cell][64 B], destination
 * [tile][cell][row][64 B]. Block scales are not touched. n % 16 == 0, k % 128 == 0. Read by
 * ferrule_hip_quant_gemv_launch with FERRULE_HIP_GEMV_BLOCK_MAJOR_WEIGHTS. */
typedef struct FerruleHipPrepareFp8BlockMajorArgs {
  uint32_t n;
  uint32_t k;
  uint64_t weight_source;      /* E4M3 [n, k] */
  uint64_t weight_destination; /* n*k bytes, no overlap with the source */
  uint64_t stream;
} FerruleHipPrepareFp8BlockMajorArgs;

int32_t ferrule_hip_prepare_fp8_block_major(const FerruleHipPrepareFp8BlockMajorArgs *args);

/* ------------------------------------------------------------------------ */
/* (3) packed verification / prefill GEMM on the scaled MFMA                 */
/* ------------------------------------------------------------------------ */

/* byte-identical to FerruleCutlassFp8QueryAKvArgs, abi/cutlass_provider.h:41-56 (96 B).
 * activation_fp8 E4M3 [rows,k] with UE8M0 scales [rows, scale_cols] (K128 blocks); each
 * weight E4M3 [n,k] with UE8M0 scales [ceil(n/128), scale_cols]; outputs f32 [rows,n]
 * holding BF16-rounded values:
 *   y = bf16_round( sum_kb (sum_{k in kb} a*w) * w_scale[n/128,kb] * a_scale[row,kb] )
 * (capabilities/fp8_projection.cuh:318-416). */
typedef struct FerruleHipFp8QueryAKvArgs {
  uint32_t rows;
  uint32_t n1;
  uint32_t n2;
  uint32_t k;
  uint32_t scale_cols;
  uint64_t activation_fp8;
  uint64_t activation_ue8m0;
  uint64_t query_a_weight_fp8;
  uint64_t query_a_weight_ue8m0;
  uint64_t kv_weight_fp8;
  uint64_t kv_weight_ue8m0;
  uint64_t query_a_output_f32;
  uint64_t kv_output_f32;
  uint64_t stream;
} FerruleHipFp8QueryAKvArgs;

/* replace ferrule_cutlass_fp8_query_a_kv_{can_implement,launch} (abi/cutlass_provider.h:391-394):
 * both projections of one activation, in ONE launch (the KV matrix's feature tiles follow
 * QueryA's in the same grid); results equal two ferrule_hip_fp8_projection launches bit for bit. */
int32_t ferrule_hip_fp8_query_a_kv_can_implement(const FerruleHipFp8QueryAKvArgs *args);
int32_t ferrule_hip_fp8_query_a_kv_launch(const FerruleHipFp8QueryAKvArgs *args);
/* replace ferrule_cutlass_fp8_projection_{can_implement,launch} (abi/cutlass_provider.h:395-398;
 * implementations/cutlass/entrypoints.cu:1234-1265): single projection, n2 and the kv fields
 * must be zero and scale_cols == k/128. */
int32_t ferrule_hip_fp8_projection_can_implement(const FerruleHipFp8QueryAKvArgs *args);
int32_t ferrule_hip_fp8_projection_launch(const FerruleHipFp8QueryAKvArgs *args);

#define FERRULE_HIP_GEMM_OUTPUT_BF16 1u /* flags bit0: write bf16 instead of bf16-rounded f32 */
/* flags bit1: always the MFMA tile schedule.  The FP8 x FP8 entry points (projection, query_a_kv,
 * block GEMM, shared FFN) choose their schedule from the row count, as the reference's native
 * providers do (crates/ferrule-backend/src/cuda/provider.rs:46-49): up to 32 rows stream the
 * weights once with one wave per 16 output features (the reference's small-M kernel is
 * capabilities/fp8_projection.cuh:424-497), more rows run 128- or 256-row MFMA tiles.  A row's
 * result has the same bits in either schedule; this bit exists so that a test can say so. */
#define FERRULE_HIP_GEMM_TILE_SCHEDULE 2u

/* General FP8 block-scaled GEMM with no reference symbol: the same contraction with either
 * E8M0 or F32 weight scales per 128x128 block (the checkpoint layout of
 * dequantize_fp8_e4m3fn_with_e8m0_scales, crates/ferrule-model/src/checkpoint/encoding.rs:147-198,
 * and its f32-scale variant) and a BF16 or f32 output. The activation is the output of
 * ferrule_hip_core_quantize_launch kind 5 (E4M3 bytes + one UE8M0 byte per 128 k). */
typedef struct FerruleHipFp8BlockGemmArgs {
  uint32_t rows;
  uint32_t n;
  uint32_t k;                 /* multiple of 128 */
  uint32_t scale_cols;        /* k / 128 */
  uint32_t weight_scale_kind; /* FerruleHipScaleKind */
  uint32_t flags;
  uint64_t activation_fp8;
  uint64_t activation_ue8m0;
  uint64_t weight_fp8;
  uint64_t weight_scales;
  uint64_t output;
  uint64_t stream;
} FerruleHipFp8BlockGemmArgs;

int32_t ferrule_hip_fp8_block_gemm_can_implement(const FerruleHipFp8BlockGemmArgs *args);
int32_t ferrule_hip_fp8_block_gemm_launch(const FerruleHipFp8BlockGemmArgs *args);

/* byte-identical to FerruleCutlassGroupedFp4MoeArgs, abi/cutlass_provider.h:337-376 (224 B).
 * Routed MXFP4 experts over packed FP8 rows (prefill / verification):
 *   per routed row r of group g (expert slot s = active_expert_slots[g]):
 *     x      = input_fp8[route_token_indices[r]] with its UE8M0 K128 scales
 *     gate   = W1[s] x, up = W3[s] x                       (fp32 accumulation)
 *     h      = silu(gate) * up * route_weights[r], clamped first when swiglu_limit > 0
 *     hq     = FP8-E4M3 / UE8M0 quantisation of h in blocks of 128 along the intermediate
 *              dimension (simulate_fp8_e4m3fn_e8m0_activation_quant, encoding.rs:207-242)
 *     route_output[route_indices[r], :] = W2[s] hq         (fp32), route_written[..] = 1
 * which is CpuReferenceExpertExecutor::execute with Fp8E4M3WithE8M0Scale{128} activation
 * quantisation (crates/ferrule-model/src/moe/executor.rs:82-124).  Unlike the CUDA provider
 * (sm103/grouped_fp4_moe.cuh:618-690) gate, up and h are NOT rounded to BF16 in between: the
 * CPU path is the contract.  A non-finite h is stored as 0 and raises route_error, as there.
 * small_group_count, max_group_rows, *_generations are accepted and not needed.
 * Weight scale pointers address storage prepared by ferrule_hip_prepare_mxfp4_sfb. */
typedef struct FerruleHipGroupedFp4MoeArgs {
  uint32_t active_group_count;
  uint32_t small_group_count;
  uint32_t slot_capacity;
  uint32_t max_group_rows;
  uint32_t total_routed_rows;
  uint32_t num_tokens;
  uint32_t num_routes;
  uint32_t input_size;
  uint32_t intermediate_size;
  uint32_t hidden_size;
  float swiglu_limit;

  uint64_t active_expert_slots;
  uint64_t active_group_generations;
  uint64_t expert_route_indptr;
  uint64_t expert_route_counts;
  uint64_t route_token_indices;
  uint64_t route_indices;
  uint64_t route_weights;

  uint64_t slot_generations;
  uint64_t gate_ptrs;
  uint64_t gate_scale_ptrs;
  uint64_t up_ptrs;
  uint64_t up_scale_ptrs;
  uint64_t down_ptrs;
  uint64_t down_scale_ptrs;

  uint64_t input_fp8;
  uint64_t input_ue8m0;

  uint64_t route_output;
  uint64_t route_written;
  uint64_t route_error;

  uint64_t workspace;
  uint64_t workspace_bytes;
  uint64_t stream;
} FerruleHipGroupedFp4MoeArgs;

/* replace ferrule_cutlass_grouped_fp4_moe_{workspace_size,can_implement,launch}
 * (abi/cutlass_provider.h:446-453). workspace_size reads scalar fields only.
 * can_implement answers FERRULE_HIP_UNSUPPORTED when the input plane (num_tokens x input_size
 * bytes) or one expert matrix (intermediate_size x input_size / 2, hidden_size x
 * intermediate_size / 2 bytes) reaches 4 GiB: rows of both are addressed with 32-bit offsets. */
uint64_t ferrule_hip_grouped_fp4_moe_workspace_size(const FerruleHipGroupedFp4MoeArgs *args);
int32_t ferrule_hip_grouped_fp4_moe_can_implement(const FerruleHipGroupedFp4MoeArgs *args);
int32_t ferrule_hip_grouped_fp4_moe_launch(const FerruleHipGroupedFp4MoeArgs *args);
/* The same launch for a slot table whose weight AND scale pointers address the block-major order
 * written by ferrule_hip_prepare_mxfp4_block_major, so that ONE prepared copy of an expert serves
 * the decode layer (ferrule_hip_moe_decode_launch with its block-major flag) and this prefill
 * path; the reference likewise prepares an expert once per slot (context.rs:5185-5204).  A
 * separate symbol and not a flag: the 224-byte block is the reference's, without a spare field.
 * Results are bit-identical to ferrule_hip_grouped_fp4_moe_launch on the checkpoint order. */
int32_t ferrule_hip_grouped_fp4_moe_block_major_launch(const FerruleHipGroupedFp4MoeArgs *args);

/* byte-identical to FerruleCutlassPrepareMxfp4SfbArgs, abi/cutlass_provider.h:381-388 (40 B) */
typedef struct FerruleHipPrepareMxfp4SfbArgs {
  uint32_t n;
  uint32_t k;
  uint32_t reserved0;
  uint64_t linear_source;        /* UE8M0 [n, k/32] */
  uint64_t prepared_destination; /* ferrule_hip_mxfp4_sfb_storage_bytes(n, k) bytes */
  uint64_t stream;
} FerruleHipPrepareMxfp4SfbArgs;

/* replace ferrule_cutlass_mxfp4_sfb_storage_bytes / ferrule_cutlass_prepare_mxfp4_sfb
 * (abi/cutlass_provider.h:454-456). The prepared layout of this provider is the linear
 * [n, k/32] layout itself (a lane's scale byte sits beside the lane's weight bytes in the
 * scaled MFMA, so no interleave is needed): storage is n*k/32 bytes and prepare is a copy. */
uint64_t ferrule_hip_mxfp4_sfb_storage_bytes(uint32_t n, uint32_t k);
int32_t ferrule_hip_prepare_mxfp4_sfb(const FerruleHipPrepareMxfp4SfbArgs *args);

#define FERRULE_HIP_SHARED_FFN_ACCUMULATE 1u /* flags bit0: output += result (shared_ffn.cuh:45-46) */
/* flags bit1: always the MFMA tile schedule (see FERRULE_HIP_GEMM_TILE_SCHEDULE); without it up
 * to 32 rows take the decode-row schedule, the counterpart of the reference's small-M kernels
 * (capabilities/shared_ffn.cuh:477-523).  Same bits either way. */
#define FERRULE_HIP_SHARED_FFN_TILE_SCHEDULE 2u

/* byte-identical to FerruleCutlassSharedFfnArgs, abi/cutlass_provider.h:113-142 (160 B).
 * Dense FP8 SwiGLU FFN over packed rows, all weights E4M3 with UE8M0 128x128 block scales:
 *   gate = W1 x, up = W3 x (fp32);  clamp when swiglu_limit > 0
 *   h = silu(gate) * up * output_scale            (SwiGluFfn::reference_execute, ffn.rs:24-48)
 *   (hidden_fp8, hidden_ue8m0) = FP8-K128 activation quantisation of h  (the act-quant policy
 *                                 of the down projection, weight.rs:63-108)
 *   output_f32 (+)= W2 hq                          (fp32, not rounded)
 * hidden_f32 [rows, intermediate] receives the unquantised h. Unlike the CUDA provider
 * (capabilities/shared_ffn.cuh:295-475) there are no BF16 roundings between the stages: the
 * CPU path is the contract. */
typedef struct FerruleHipSharedFfnArgs {
  uint64_t input_fp8;
  uint64_t input_ue8m0;
  uint64_t gate_weight_fp8;
  uint64_t gate_weight_ue8m0;
  uint64_t up_weight_fp8;
  uint64_t up_weight_ue8m0;
  uint64_t down_weight_fp8;
  uint64_t down_weight_ue8m0;
  uint64_t hidden_f32;
  uint64_t hidden_fp8;
  uint64_t hidden_ue8m0;
  uint64_t output_f32;

  uint32_t rows;
  uint32_t input_size;
  uint32_t intermediate_size;
  uint32_t output_size;

  uint32_t gate_block_m;
  uint32_t gate_block_k;
  uint32_t up_block_m;
  uint32_t up_block_k;
  uint32_t down_block_m;
  uint32_t down_block_k;

  float output_scale;
  float swiglu_limit;
  uint32_t flags;
  uint64_t stream;
} FerruleHipSharedFfnArgs;

/* replace ferrule_cutlass_shared_ffn_{can_implement,launch} (abi/cutlass_provider.h:407-410) */
int32_t ferrule_hip_shared_ffn_can_implement(const FerruleHipSharedFfnArgs *args);
int32_t ferrule_hip_shared_ffn_launch(const FerruleHipSharedFfnArgs *args);

/* ------------------------------------------------------------------------ */
/* hyper-connection producer                                                  */
/* ------------------------------------------------------------------------ */

#define FERRULE_HIP_KERNEL_HYPER_CONNECTION_PRODUCER 3u /* abi/cutlass_provider.h:16 */
#define FERRULE_HIP_HC_PRODUCER_BF16_BOUNDARIES 1u       /* FerruleHipHcProducerArgs.reserved */

/* byte-identical to FerruleCutlassHcProducerArgs, abi/cutlass_provider.h:76-106 (168 B) */
typedef struct FerruleHipHcProducerArgs {
  uint32_t rows;
  uint32_t hc;             /* 4 */
  uint32_t hidden;         /* multiple of 1024, at most 8192 (the reference: 4096 only) */
  uint32_t mix;            /* 24 = (2 + hc) * hc */
  uint32_t sinkhorn_iters; /* at least 1 */
  float hc_eps;
  float hc_norm_eps;
  float layer_rms_eps;
  uint32_t reserved;       /* 0: the CPU chain, no BF16 rounding between the stages;
                              1: hidden and normalized rounded to BF16 as the CUDA provider does */
  uint64_t state_f32;               /* [rows, 4, hidden] */
  uint64_t function_row_major_f32;  /* [24, 4 * hidden] */
  uint64_t hc_scale_f32;            /* [3] */
  uint64_t hc_base_f32;             /* [24] */
  uint64_t layer_rms_weight_f32;    /* [hidden] */
  uint64_t mix_f32;                 /* out [rows, 24]: the raw dot products */
  uint64_t workspace;               /* unused here; may be 0 */
  uint64_t workspace_bytes;
  uint64_t hidden_f32;              /* out [rows, hidden] */
  uint64_t normalized_f32;          /* out [rows, hidden] */
  uint64_t packed_e4m3;             /* out [rows, hidden] */
  uint64_t scales_ue8m0;            /* out [rows, hidden / 128] */
  uint64_t split_pre_f32;           /* out [rows, 4] */
  uint64_t split_post_f32;          /* out [rows, 4] */
  uint64_t split_comb_f32;          /* out [rows, 4, 4] */
  uint64_t stream;
} FerruleHipHcProducerArgs;

/* replace ferrule_cutlass_hc_producer_{can_implement,launch} (abi/cutlass_provider.h:403-406;
 * implementations/cutlass/capabilities/hyper_connection.cuh:461-743): HC mix and split,
 * weighted copy sum, layer RMSNorm and FP8-K128 packing of `rows` token rows in one launch
 * that reads the state once.  All pointers except workspace must be non-null and 16-byte
 * aligned.  INVALID_ARGUMENT for a bad block, UNSUPPORTED for a hidden size outside the
 * supported set. */
int32_t ferrule_hip_hc_producer_can_implement(const FerruleHipHcProducerArgs *args);
int32_t ferrule_hip_hc_producer_launch(const FerruleHipHcProducerArgs *args);

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
FERRULE_HIP_ASSERT_LAYOUT(FerruleHipDenseFfnDecodeArgs, 128, x, 48, 120);
static_assert(sizeof(FerruleHipQuantGemvMultiArgs) == 16 && offsetof(FerruleHipQuantGemvMultiArgs, matrices) == 8,
              "FerruleHipQuantGemvMultiArgs layout");
FERRULE_HIP_ASSERT_LAYOUT(FerruleHipExpertGroupRoutePlanArgs, 184, route_slots, 32, 176);
FERRULE_HIP_ASSERT_LAYOUT(FerruleHipMoeArgs, 248, input, 48, 240);
FERRULE_HIP_ASSERT_LAYOUT(FerruleHipRouterArgs, 96, logits, 40, 88);
FERRULE_HIP_ASSERT_LAYOUT(FerruleHipHcProducerArgs, 168, state_f32, 40, 160);
static_assert(offsetof(FerruleHipHcProducerArgs, mix_f32) == 80, "mix offset");
FERRULE_HIP_ASSERT_LAYOUT(FerruleHipExpertTableArgs, 296, gate_weights, 48, 288);
static_assert(offsetof(FerruleHipExpertTableArgs, route_slots) == 128, "route_slots offset");
static_assert(offsetof(FerruleHipExpertTableArgs, output_gate_weights) == 176, "output gate offset");
static_assert(offsetof(FerruleHipExpertTableArgs, gate_weight_value) == 240, "value offset");
FERRULE_HIP_ASSERT_LAYOUT(FerruleHipMoeDecodeArgs, 216, active_expert_slots, 48, 208);
FERRULE_HIP_ASSERT_LAYOUT(FerruleHipFp8QueryAKvArgs, 96, activation_fp8, 24, 88);
FERRULE_HIP_ASSERT_LAYOUT(FerruleHipFp8BlockGemmArgs, 72, activation_fp8, 24, 64);
FERRULE_HIP_ASSERT_LAYOUT(FerruleHipGroupedFp4MoeArgs, 224, active_expert_slots, 48, 216);
FERRULE_HIP_ASSERT_LAYOUT(FerruleHipPrepareMxfp4SfbArgs, 40, linear_source, 16, 32);
FERRULE_HIP_ASSERT_LAYOUT(FerruleHipPrepareMxfp4BlockMajorArgs, 48, weight_source, 8, 40);
FERRULE_HIP_ASSERT_LAYOUT(FerruleHipPrepareFp8BlockMajorArgs, 32, weight_source, 8, 24);
FERRULE_HIP_ASSERT_LAYOUT(FerruleHipSharedFfnArgs, 160, input_fp8, 0, 152);
static_assert(offsetof(FerruleHipExpertGroupRoutePlanArgs, active_expert_slots) == 88, "route plan layout");
static_assert(offsetof(FerruleHipExpertGroupRoutePlanArgs, expert_route_indptr) == 104, "route plan layout");
static_assert(offsetof(FerruleHipExpertGroupRoutePlanArgs, host_scalars) == 144, "route plan layout");
static_assert(offsetof(FerruleHipExpertGroupRoutePlanArgs, route_output) == 152, "route plan layout");
static_assert(sizeof(FerruleHipProviderManifest) == 8, "manifest size");
#endif

#endif /* FERRULE_HIP_PROVIDER_H_ */
