/* Diagnostic entry points of libferrule_hip.so: test hooks with no counterpart in the reference's
 * provider ABI.  A drop-in host binds nothing from this header; the library exports these
 * symbols so that the device code behind the product entry points (hardware FP8 converter with
 * its software fallback, the MX split of the decode layer's activations, the unquantised hidden
 * rows of the grouped MoE) can be checked in isolation against the CPU checker. */
#ifndef FERRULE_HIP_DIAGNOSTICS_H_
#define FERRULE_HIP_DIAGNOSTICS_H_

#include "ferrule_hip_provider.h"

#ifdef __cplusplus
extern "C" {
#endif

/* The quantisers and the GEMM epilogues take their E4M3 bytes from the hardware converter
 * wherever it yields the software encoder's byte (the CPU quantiser's rule or round-half-even),
 * and the software encoder elsewhere.  This launch runs every f32 pattern through both, for both
 * rules.  counts: u64[3], zeroed by the caller; after the launch
 * [0] = differences of the complete routine (any pattern) plus differences of the converter alone
 * on finite patterns with any of the low 19 bits set (0, or the fast path is wrong), [1] = one such
 * pattern + 1, [2] = differences of the converter alone on patterns with those bits clear (the
 * ties, which go to the software encoder). */
int32_t ferrule_hip_fp8_converter_selftest_launch(uint64_t counts, uint64_t stream);

/* The grouped MoE launch (ferrule_hip_grouped_fp4_moe_launch), additionally storing the
 * unquantised h as f32 [total_routed_rows, intermediate_size] at hidden_f32 (the reference has
 * a debug_down_input pointer inside its kernel, sm103/grouped_fp4_moe.cuh:599-624). */
int32_t ferrule_hip_grouped_fp4_moe_debug_launch(const FerruleHipGroupedFp4MoeArgs *args, uint64_t hidden_f32);

/* The decode MoE layer's activation split on its own: x [rows, k] -> a sum of MX-FP8 terms,
 * q [terms][rows][k] E4M3 bytes and s [terms][rows][k/32] E8M0 bytes, by truncation
 * (term t takes the leading 4 significant bits of what terms 0..t-1 left, under the scale
 * 2^(exponent of the block's largest remainder - 7)).  input_kind 0 = BF16 input with 2 terms
 * (the layer's x), 1 = f32 input with 4 terms (its hidden rows); k a multiple of 32. */
typedef struct FerruleHipMxSplitArgs {
  uint32_t rows;
  uint32_t k;
  uint32_t input_kind;
  uint32_t reserved;
  uint64_t input;
  uint64_t q;
  uint64_t s;
  uint64_t stream;
} FerruleHipMxSplitArgs;
int32_t ferrule_hip_mx_split_launch(const FerruleHipMxSplitArgs *args);

#ifdef __cplusplus
} /* extern "C" */
static_assert(sizeof(FerruleHipMxSplitArgs) == 48, "FerruleHipMxSplitArgs layout");
#endif

#endif /* FERRULE_HIP_DIAGNOSTICS_H_ */
