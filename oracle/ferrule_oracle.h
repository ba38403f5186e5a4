/*
 * CPU restatement of Ferrule's reference arithmetic for the quantized-weight
 * matmul path.  TEST INFRASTRUCTURE ONLY: this library is the checker that the
 * parity tests, the smoke check and the benchmark's CPU-baseline leg call.  The
 * shipped provider never links, loads or calls anything declared here.
 *
 * Every function names the reference file:line it follows (paths relative to
 * the Ferrule checkout).  Arithmetic is plain IEEE binary32 with separately
 * rounded multiply and add (the reference is Rust, which never contracts to
 * FMA), so this file must be compiled with -ffp-contract=off.
 *
 * Pinning status (what fixes each function besides its own formula):
 *   decode tables, dequant, act-quant, bf16 rounding, matvec, expert SwiGLU,
 *   routed accumulate, dense SwiGLU FFN, ranked combine: pinned by the
 *   reference's own known-answer tests, transcribed as values in
 *   tests/test_oracle_golden.py, plus closed forms and brute force there.
 *   fo_rounded_power_of_two_scale: pinned on the BF16-valued input grid and on
 *   the reference vectors; for arbitrary f32 amax within 1 ulp above a power of
 *   two it depends on the platform log2f -> "parity unpinned" for those inputs.
 *   fo_silu: last-ulp behaviour of expf is platform dependent -> covered by the
 *   2-BF16-ulp output tolerance, not bit-pinned ("parity unpinned" at 1 ulp).
 *   fo_dequantize_fp8_e4m3fn_with_f32_scales and the F32-scale matvec: the
 *   reference has no F32-scale implementation; this is the closed form
 *   decode(w) * scale in the reference's operation order ("parity unpinned"
 *   against reference-held vectors, pinned by brute force and float64 bounds).
 *   fo_router_*: selection is pinned by the reference's literal index vectors
 *   (routing.rs tests, dsv4_decode_topk_boundary.rs hash test) and by numpy's
 *   stable lexsort; scores by float64 log1p/exp/sqrt of numpy to 2 ulp.  The last
 *   ulp of expf/log1pf is platform dependent ("parity unpinned" at 1 ulp, as for
 *   fo_silu); weights are compared at a few ulp, indices exactly wherever the
 *   selection scores are further apart than that.
 *   fo_expert_*: integer bookkeeping, pinned by the literal expectations of the
 *   reference's slot-table tests (expert_group_route_plan.rs:29-107,
 *   context.rs:2309-2440) transcribed in tests/test_expert_table_oracle.py.
 *   fo_hc_*, fo_rms_norm: pinned by the reference's own expectations
 *   (hyper_connection.rs:433-453, 470-484), by an independent float64 numpy evaluation of
 *   the same formulas and by the doubly-stochastic invariant of the Sinkhorn result; the
 *   last ulp of expf is platform dependent ("parity unpinned" at 1 ulp, as for fo_silu).
 */
#ifndef FERRULE_ORACLE_H_
#define FERRULE_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { FO_SCALE_E8M0 = 0, FO_SCALE_F32 = 1 };

/* crates/ferrule-model/src/checkpoint/encoding.rs:14-30 */
float fo_decode_fp4_e2m1_nibble(uint8_t nibble);
/* encoding.rs:37-44 */
void fo_decode_fp4_e2m1_packed_low_first(const uint8_t *bytes, size_t count,
                                         float *out);
/* encoding.rs:51-53 */
float fo_decode_e8m0_scale(uint8_t byte);
/* encoding.rs:61-75 */
float fo_decode_fp8_e4m3fn_byte(uint8_t byte);
/* encoding.rs:82-140; returns 0 ok, 1 on the reference's shape errors */
int fo_dequantize_fp4_e2m1_with_e8m0_scales(const uint8_t *weight,
                                            const uint8_t *scales,
                                            size_t out_features,
                                            size_t in_features,
                                            size_t block_size, float *out);
/* encoding.rs:147-198 */
int fo_dequantize_fp8_e4m3fn_with_e8m0_scales(const uint8_t *weight,
                                              const uint8_t *scales,
                                              size_t out_features,
                                              size_t in_features,
                                              size_t block_m, size_t block_k,
                                              float *out);
/* Same loop as encoding.rs:186-196 with an f32 scale table (no reference twin). */
int fo_dequantize_fp8_e4m3fn_with_f32_scales(const uint8_t *weight,
                                             const float *scales,
                                             size_t out_features,
                                             size_t in_features, size_t block_m,
                                             size_t block_k, float *out);
/* encoding.rs:335-337 */
float fo_rounded_power_of_two_scale(float amax, float quant_max);
/* encoding.rs:339-346 (+348-387) */
float fo_quantize_fp8_e4m3fn_to_f32(float value);
/* encoding.rs:389-406 */
float fo_quantize_fp4_e2m1_to_f32(float value);
/* encoding.rs:207-242 */
int fo_simulate_fp8_act_quant_in_place(float *values, size_t len,
                                       size_t row_width, size_t block_size);
/* encoding.rs:249-284 */
int fo_simulate_fp4_act_quant_in_place(float *values, size_t len,
                                       size_t row_width, size_t block_size);
/* Byte-level form of encoding.rs:207-242: the same scale and the same
 * quantized values, emitted as E4M3 bytes + E8M0 scale bytes. */
int fo_pack_fp8_act(const float *values, size_t len, size_t row_width,
                    size_t block_size, uint8_t *packed, uint8_t *scales);
/* Byte-level form of encoding.rs:249-284 (low nibble = even k). */
int fo_pack_fp4_act(const float *values, size_t len, size_t row_width,
                    size_t block_size, uint8_t *packed, uint8_t *scales);

/* crates/ferrule-model/src/models/common/math.rs:7-14 */
float fo_round_to_bf16(float value);
uint16_t fo_bf16_bits(float value);

/* crates/ferrule-model/src/checkpoint/weight.rs:440-451 */
void fo_matvec_row_major(const float *weights, size_t rows, size_t cols,
                         const float *input, float *output);

/* weight.rs:154-173 with the FP4 format (dequant, then matvec), written so
 * that no f32 matrix is materialised: every product is still
 * (decode*scale)*x[col], added left to right.  threads<=1 is serial. */
int fo_linear_fp4_matvec(const uint8_t *weight, const uint8_t *scales,
                         size_t out_features, size_t in_features,
                         size_t block_size, const float *input, float *output,
                         int threads);
/* weight.rs:154-173 with the FP8 format; scale_kind selects E8M0 bytes or f32. */
int fo_linear_fp8_matvec(const uint8_t *weight, const void *scales,
                         int scale_kind, size_t out_features,
                         size_t in_features, size_t block_m, size_t block_k,
                         const float *input, float *output, int threads);
/* As the reference really runs (weight.rs:165-172): materialise the whole f32
 * matrix on every call, then matvec.  Used only as the timed CPU baseline. */
int fo_linear_fp4_matvec_materialized(const uint8_t *weight,
                                      const uint8_t *scales,
                                      size_t out_features, size_t in_features,
                                      size_t block_size, const float *input,
                                      float *output);
int fo_linear_fp8_matvec_materialized(const uint8_t *weight, const void *scales,
                                      int scale_kind, size_t out_features,
                                      size_t in_features, size_t block_m,
                                      size_t block_k, const float *input,
                                      float *output);

/* crates/ferrule-model/src/moe/executor.rs:179-181 */
float fo_silu(float x);
/* executor.rs:82-124.  act_quant_block = 0 means no activation quantization
 * (the default construction); otherwise Fp8E4M3WithE8M0Scale{block}. */
int fo_expert_execute_fp4(const uint8_t *gate_w, const uint8_t *gate_s,
                          const uint8_t *up_w, const uint8_t *up_s,
                          const uint8_t *down_w, const uint8_t *down_s,
                          size_t hidden, size_t intermediate,
                          size_t block_size, const float *input,
                          float route_weight, float swiglu_limit,
                          size_t act_quant_block, float *output,
                          float *hidden_out /* nullable: [intermediate] */,
                          int threads);
/* crates/ferrule-model/src/moe/routed.rs:85-110, 183-201: out = sum over routes
 * in router order (first route initialises), then + shared (nullable). */
void fo_accumulate_routes(const float *route_outputs, size_t routes,
                          size_t width, const float *shared, float *out);
/* crates/ferrule-model/src/ffn.rs:24-48 for f32 linears. */
void fo_swiglu_ffn_f32(const float *gate, const float *up, const float *down,
                       size_t hidden, size_t intermediate, const float *input,
                       float output_scale, float swiglu_limit, float *output);

/* GPU-side combine semantics that the provider's reducer mirrors:
 * crates/ferrule-backend/native/cuda/implementations/portable/entrypoints.cu:1583-1611
 * out[t,h] = bf16(out[t,h] + route_output[t*k+0,h] + ... ) strict left fold. */
void fo_reduce_routes_ranked(const float *route_output, size_t tokens,
                             size_t routes_per_token, size_t hidden,
                             float *output);

/* ---- router (the step before the route plan) ----------------------------- */

/* crates/ferrule-model/src/moe/routing.rs:367-372 */
float fo_stable_softplus(float value);
/* ExpertRouterPolicy::route with RouterScoreFunction::SqrtSoftplus and
 * normalize_non_softmax_weights = true, routing.rs:135-191: validation
 * (routing.rs:209-289), scores sqrt(softplus) (routing.rs:297-303), selection
 * ScoreTopK = sort by (selection score descending in total order, expert
 * ascending) (routing.rs:305-331) or Hash = the first top_k ids of hash_experts
 * when that pointer is non-null (routing.rs:153-158); weights = gathered scores /
 * their left-to-right sum * route_scale.  Outputs are [top_k]; scores and
 * selection_scores are nullable.  Returns 0, or 1 where the reference returns Err. */
int fo_router_route_sqrt_softplus(const float *logits, size_t experts,
                                  const float *bias /* nullable */,
                                  const int64_t *hash_experts /* nullable */,
                                  size_t hash_len, size_t top_k,
                                  float route_scale, int32_t *indices,
                                  float *weights, float *scores,
                                  float *selection_scores);
/* Sequential restatement of the device router, one row after the other:
 * crates/ferrule-backend/native/cuda/implementations/portable/entrypoints.cu:770-884
 * (insert_topk + router_kernel) with softplus of entrypoints.cu:103-111.
 * kind 1 score top-k, 2 hash, 3/4 plain top-k of the logits with f32/i32 indices.
 * Rows that the kernel leaves untouched (bad token id or table entry) are left
 * untouched here.  indices is int32 [rows,k] (float for kind 3). */
void fo_router_kernel_rows(uint32_t kind, uint32_t rows, uint32_t columns,
                           uint32_t k, uint32_t hash_rows,
                           uint32_t hash_columns, uint32_t flags,
                           float route_scale, const float *logits,
                           const float *bias, const int32_t *token_ids,
                           const int32_t *hash_table, void *indices,
                           float *weights);

/* ---- expert slot table (between the router's ids and the route plan's slots) -------- */

/* Device side, crates/ferrule-backend/native/cuda/implementations/portable/entrypoints.cu
 * :1268-1300 (kinds INSTALL = 1 / EVICT = 2).  table is u64 [6][slot_capacity] in the order
 * gate weight, gate scale, up weight, up scale, down weight, down scale. */
void fo_expert_table_publish(uint32_t kind, uint32_t expert, uint32_t slot,
                             int32_t generation, const uint64_t values[6],
                             uint64_t *table, uint32_t slot_capacity,
                             int32_t *expert_to_slot,
                             int32_t *expert_generations,
                             int32_t *slot_generations);
/* entrypoints.cu:1301-1307 */
void fo_expert_resolve_init(int32_t *miss_control, uint32_t miss_capacity,
                            uint32_t route_capacity);
/* entrypoints.cu:1311-1340, routes visited in ascending order (the reference's miss-list
 * order is the order in which its threads reach an atomicAdd, i.e. unspecified). */
void fo_expert_resolve(const int32_t *expert_ids, uint32_t route_count,
                       uint32_t expert_capacity, uint32_t slot_capacity,
                       uint32_t miss_capacity, const int32_t *expert_to_slot,
                       const int32_t *expert_generations,
                       const int32_t *slot_generations, int32_t *route_slots,
                       int32_t *route_generations, int32_t *miss_markers,
                       int32_t *miss_control);
/* entrypoints.cu:1341-1379 with the flag reset of :2011-2017; outputs is u64
 * [6][route_count]; returns dispatch_error. */
int32_t fo_expert_gather_dispatch(uint32_t route_count, uint32_t slot_capacity,
                                  int32_t active_value, const uint64_t *table,
                                  const int32_t *slot_generations,
                                  const int32_t *route_slots,
                                  const int32_t *route_generations,
                                  const float *router_weights,
                                  const int32_t *active_markers,
                                  uint64_t *outputs, float *output_route_weights,
                                  int32_t *expert_ids);

/* ---- hyper-connection producer (the maker of the FP8 activations the GEMMs read) ---- */

/* crates/ferrule-model/src/hyper_connection.rs:175-262 hc_split_sinkhorn_reference.
 * mixes [tokens, (2+hc)*hc], scale [3], base [(2+hc)*hc] -> pre [tokens, hc],
 * post [tokens, hc], comb [tokens, hc, hc].  Returns 1 on the reference's errors. */
int fo_hc_split_sinkhorn(const float *mixes, size_t tokens, size_t hc,
                         size_t sinkhorn_iters, float eps, const float *scale,
                         const float *base, float *pre, float *post, float *comb);
/* hyper_connection.rs:264-311 hc_pre_reference (rms_factor :416-419, dot :421-423):
 * state [tokens, hc, hidden], function [(2+hc)*hc, hc*hidden] -> mixes (already times the
 * state's rms factor), the split, hidden [tokens, hidden].  raw_dots (nullable) receives the
 * dot products before the rms factor. */
int fo_hc_pre(const float *state, size_t tokens, size_t hc, size_t hidden,
              size_t sinkhorn_iters, float eps, float norm_eps,
              const float *function, const float *scale, const float *base,
              float *mixes, float *raw_dots, float *pre, float *post, float *comb,
              float *hidden_out);
/* crates/ferrule-model/src/models/common/math.rs:22-42 rms_norm, one row. */
int fo_rms_norm(const float *input, const float *weight, size_t len, float eps,
                float *out);
/* The CPU chain the producer fuses (models/deepseek_v4/layer.rs:416-422, 1016-1030):
 * hc_pre -> rms_norm with the layer weight -> FP8-K128 activation packing
 * (encoding.rs:207-242).  bf16_boundaries != 0 additionally rounds hidden and normalized
 * to BF16 where the CUDA provider does
 * (native/cuda/implementations/cutlass/capabilities/hyper_connection.cuh:626, 653). */
int fo_hc_producer(const float *state, size_t tokens, size_t hc, size_t hidden,
                   size_t sinkhorn_iters, float eps, float norm_eps,
                   float layer_rms_eps, int bf16_boundaries,
                   const float *function, const float *scale, const float *base,
                   const float *layer_rms_weight, float *raw_dots, float *pre,
                   float *post, float *comb, float *hidden_out, float *normalized,
                   uint8_t *packed, uint8_t *scales);

/* ---- error-bound arithmetic for the parity tests (NOT a restatement of any reference
 * function): out[row] = sum_k |dequant(W)[row,k]| * v[k] in double, v >= 0.  With
 * v = |x| this is the A = sum|w x| of the forward-error bound of an fp32 dot product
 * summed in any order; with other non-negative vectors it carries an input perturbation
 * through the linear map.  Same formats and layouts as the matvecs above. */
int fo_abs_linear_fp4(const uint8_t *weight, const uint8_t *scales,
                      size_t out_features, size_t in_features, size_t block_size,
                      const double *v, double *out, int threads);
int fo_abs_linear_fp8(const uint8_t *weight, const void *scales, int scale_kind,
                      size_t out_features, size_t in_features, size_t block_m,
                      size_t block_k, const double *v, double *out, int threads);

#ifdef __cplusplus
}
#endif
#endif
