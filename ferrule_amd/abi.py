"""ctypes mirror of ``include/ferrule_hip_provider.h`` (and of the diagnostic entry points of
``include/ferrule_hip_diagnostics.h``) and the library loader.

This plays the role of Ferrule's ``#[repr(C)]`` mirrors
(crates/ferrule-backend/src/cuda/kernels.rs:115-576,
crates/ferrule-backend/src/cuda/cutlass.rs:156-535): plain-old-data argument
blocks, device pointers and the stream carried as ``u64``.

The library is never built implicitly on the call path: if
``libferrule_hip.so`` is missing, loading raises.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libferrule_hip.so")

# FerruleHipStatus
SUCCESS = 0
INVALID_ARGUMENT = 2
LAUNCH_FAILED = 3
UNSUPPORTED = 4

WEIGHT_FP8_E4M3 = 1
WEIGHT_MXFP4_E2M1 = 2
SCALE_E8M0 = 0
SCALE_F32 = 1
GEMV_OUTPUT_F32 = 1
GEMV_BLOCK_MAJOR_WEIGHTS = 2
GEMV_MULTI_MAX = 32
MOE_DECODE_STATIC_WORKSPACE_BYTES = 16 << 20

KERNEL_FP8_QUERY_A_KV = 1
KERNEL_HYPER_CONNECTION_PRODUCER = 3
KERNEL_SHARED_FFN = 4
KERNEL_GROUPED_FP4_MOE = 5
KERNEL_FP8_PROJECTION = 10
KERNEL_QUANT_GEMV = 33
KERNEL_MOE_DECODE = 34
KERNEL_FP8_BLOCK_GEMM = 35
KERNEL_DENSE_FFN_DECODE = 36

LINEAR_FP8_E4M3_E8M0 = 4
LINEAR_FP8_E4M3_E8M0_PACKED = 5
LINEAR_FP8_E4M3_E8M0_FROM_F32 = 8
QUANTIZE_FP4_PACKED = 4
QUANTIZE_FP8_PACKED = 5
FP8_ROUND_CPU_REFERENCE = 0
FP8_ROUND_HALF_EVEN = 1

u32, u64, f32 = C.c_uint32, C.c_uint64, C.c_float


def kernel_bit(kernel_id: int) -> int:
    return 1 << (kernel_id - 1)


class ProviderManifest(C.Structure):
    _fields_ = [("kernel_mask", u64)]


class LinearArgs(C.Structure):
    """FerruleHipLinearArgs == FerruleCoreLinearArgs (88 bytes)."""
    _fields_ = [("kind", u32), ("batch", u32), ("n", u32), ("k", u32), ("scale_cols", u32),
                ("block_m", u32), ("block_k", u32), ("packed_offset", u32), ("scale_offset", u32),
                ("x", u64), ("x_scales", u64), ("weight", u64), ("weight_scales", u64),
                ("output", u64), ("stream", u64)]


class QuantizeArgs(C.Structure):
    """FerruleHipQuantizeArgs == FerruleCoreQuantizeArgs (64 bytes)."""
    _fields_ = [("kind", u32), ("value_offset", u32), ("value_len", u32), ("row_width", u32),
                ("block_size", u32), ("rope_dim", u32), ("reserved", u32),
                ("values", u64), ("packed", u64), ("scales", u64), ("stream", u64)]


class QuantGemvArgs(C.Structure):
    """FerruleHipQuantGemvArgs (80 bytes)."""
    _fields_ = [("weight_format", u32), ("scale_kind", u32), ("batch", u32), ("n", u32), ("k", u32),
                ("block_m", u32), ("block_k", u32), ("scale_cols", u32), ("flags", u32),
                ("reserved", u32),
                ("x", u64), ("weight", u64), ("weight_scales", u64), ("output", u64), ("stream", u64)]


class DenseFfnDecodeArgs(C.Structure):
    """FerruleHipDenseFfnDecodeArgs (128 bytes)."""
    _fields_ = [("weight_format", u32), ("scale_kind", u32), ("batch", u32), ("input_size", u32),
                ("intermediate_size", u32), ("output_size", u32), ("block_m", u32), ("block_k", u32), ("flags", u32),
                ("reserved", u32), ("swiglu_limit", f32), ("output_scale", f32),
                ("x", u64), ("gate_weight", u64), ("gate_scales", u64), ("up_weight", u64), ("up_scales", u64),
                ("down_weight", u64), ("down_scales", u64), ("hidden_f32", u64), ("output", u64), ("stream", u64)]


class QuantGemvMultiArgs(C.Structure):
    """FerruleHipQuantGemvMultiArgs (16 bytes): `matrices` is the HOST address of `count` QuantGemvArgs."""
    _fields_ = [("count", u32), ("reserved", u32), ("matrices", u64)]


class ExpertGroupRoutePlanArgs(C.Structure):
    """FerruleHipExpertGroupRoutePlanArgs == FerruleCoreExpertGroupRoutePlanArgs (184 bytes)."""
    _fields_ = [("kind", u32), ("route_count", u32), ("routes_per_token", u32), ("slot_capacity", u32),
                ("route_capacity", u32), ("output_elements", u32), ("small_group_row_limit", u32),
                ("route_slots", u64), ("route_generations", u64), ("router_weights", u64),
                ("slot_generations", u64), ("slot_counts", u64), ("slot_route_offsets", u64),
                ("slot_cursors", u64), ("active_expert_slots", u64), ("active_group_generations", u64),
                ("expert_route_indptr", u64), ("expert_route_counts", u64), ("route_token_indices", u64),
                ("route_indices", u64), ("route_weights", u64), ("host_scalars", u64),
                ("route_output", u64), ("route_written", u64), ("route_error", u64), ("stream", u64)]


class MoeArgs(C.Structure):
    """FerruleHipMoeArgs == FerruleCoreMoeArgs (248 bytes)."""
    _fields_ = [("kind", u32), ("n", u32), ("k", u32), ("batch_columns", u32), ("experts", u32),
                ("tokens", u32), ("routes_per_token", u32), ("output_offset", u32), ("hidden", u32),
                ("route_weight", f32), ("swiglu_limit", f32),
                ("input", u64), ("input_scales", u64), ("gate_ptrs", u64), ("gate_scale_ptrs", u64),
                ("up_ptrs", u64), ("up_scale_ptrs", u64), ("down_ptrs", u64), ("down_scale_ptrs", u64),
                ("gate", u64), ("up", u64), ("route_weights", u64), ("hidden_values", u64),
                ("hidden_packed", u64), ("hidden_scales", u64), ("expert_output", u64),
                ("resident_output", u64), ("materialized_output", u64), ("route_slots", u64),
                ("materialized_route_slots", u64), ("miss_markers", u64), ("route_output", u64),
                ("route_written", u64), ("route_error", u64), ("output", u64), ("stream", u64)]


class RouterArgs(C.Structure):
    """FerruleHipRouterArgs == FerruleCoreRouterArgs (96 bytes)."""
    _fields_ = [("kind", u32), ("rows", u32), ("columns", u32), ("k", u32), ("hash_rows", u32),
                ("hash_columns", u32), ("flags", u32), ("route_scale", f32), ("reserved", u32),
                ("logits", u64), ("bias", u64), ("token_ids", u64), ("hash_table", u64),
                ("indices", u64), ("weights", u64), ("stream", u64)]


class ExpertTableArgs(C.Structure):
    """FerruleHipExpertTableArgs == FerruleCoreExpertTableArgs (296 bytes)."""
    _fields_ = [("kind", u32), ("route_count", u32), ("expert_capacity", u32), ("slot_capacity", u32),
                ("miss_capacity", u32), ("route_capacity", u32), ("expert", u32), ("slot", u32),
                ("generation", C.c_int32), ("active_value", C.c_int32), ("reserved", u32),
                ("gate_weights", u64), ("gate_scales", u64), ("up_weights", u64), ("up_scales", u64),
                ("down_weights", u64), ("down_scales", u64), ("expert_to_slot", u64),
                ("expert_generations", u64), ("slot_generations", u64), ("expert_ids", u64),
                ("route_slots", u64), ("route_generations", u64), ("miss_markers", u64), ("miss_control", u64),
                ("router_weights", u64), ("active_markers", u64), ("output_gate_weights", u64),
                ("output_gate_scales", u64), ("output_up_weights", u64), ("output_up_scales", u64),
                ("output_down_weights", u64), ("output_down_scales", u64), ("output_route_weights", u64),
                ("dispatch_error", u64), ("gate_weight_value", u64), ("gate_scale_value", u64),
                ("up_weight_value", u64), ("up_scale_value", u64), ("down_weight_value", u64),
                ("down_scale_value", u64), ("stream", u64)]


class HcProducerArgs(C.Structure):
    """FerruleHipHcProducerArgs == FerruleCutlassHcProducerArgs (168 bytes)."""
    _fields_ = [("rows", u32), ("hc", u32), ("hidden", u32), ("mix", u32), ("sinkhorn_iters", u32),
                ("hc_eps", f32), ("hc_norm_eps", f32), ("layer_rms_eps", f32), ("reserved", u32),
                ("state_f32", u64), ("function_row_major_f32", u64), ("hc_scale_f32", u64), ("hc_base_f32", u64),
                ("layer_rms_weight_f32", u64), ("mix_f32", u64), ("workspace", u64), ("workspace_bytes", u64),
                ("hidden_f32", u64), ("normalized_f32", u64), ("packed_e4m3", u64), ("scales_ue8m0", u64),
                ("split_pre_f32", u64), ("split_post_f32", u64), ("split_comb_f32", u64), ("stream", u64)]


class MoeDecodeArgs(C.Structure):
    """FerruleHipMoeDecodeArgs (216 bytes)."""
    _fields_ = [("active_group_count", u32), ("slot_capacity", u32), ("total_routed_rows", u32),
                ("num_tokens", u32), ("num_routes", u32), ("routes_per_token", u32), ("input_size", u32),
                ("intermediate_size", u32), ("hidden_size", u32), ("flags", u32), ("swiglu_limit", f32),
                ("reserved", u32),
                ("active_expert_slots", u64), ("expert_route_indptr", u64), ("route_token_indices", u64),
                ("route_indices", u64), ("route_weights", u64), ("host_scalars", u64),
                ("gate_ptrs", u64), ("gate_scale_ptrs", u64), ("up_ptrs", u64), ("up_scale_ptrs", u64),
                ("down_ptrs", u64), ("down_scale_ptrs", u64),
                ("input_bf16", u64), ("route_output", u64), ("route_written", u64), ("route_error", u64),
                ("prefix_f32", u64), ("output", u64),
                ("workspace", u64), ("workspace_bytes", u64), ("stream", u64)]


ROUTE_INIT_INVOCATION, ROUTE_INIT_PLAN, ROUTE_COUNT, ROUTE_COMPACT, ROUTE_SCATTER = 1, 2, 3, 4, 5
ROUTE_FUSED_DECODE_PLAN, FUSED_PLAN_MAX_ROUTES = 16, 2048
EXPERT_INSTALL, EXPERT_EVICT, EXPERT_INITIALIZE_RESOLVE, EXPERT_RESOLVE, EXPERT_GATHER_DISPATCH = 1, 2, 3, 4, 5
HC_PRODUCER_BF16_BOUNDARIES = 1
ROUTER_TOPK, ROUTER_HASH, VOCAB_TOPK_F32_INDEX, VOCAB_TOPK_I32_INDEX = 1, 2, 3, 4
ROUTER_MAX_TOP_K, ROUTER_TOPK_MAX_EXPERTS, VOCAB_TOPK_MAX_K = 64, 512, 40  # context.rs:7148-7162, 7302-7310
MOE_WEIGHTED_SWIGLU_F32, MOE_REDUCE_ROUTES, MOE_REDUCE_EXPERT_GROUP_ROUTES = 2, 7, 8
MOE_DECODE_COMBINE, MOE_DECODE_PREFIX_F32, MOE_DECODE_SKIP_GATE_UP, MOE_DECODE_SKIP_DOWN = 1, 2, 4, 8
MOE_DECODE_BLOCK_MAJOR_WEIGHTS = 16
SMALL_GROUP_ROW_LIMIT = 192      # crates/ferrule-backend/src/cuda/context.rs:1683
WORKSPACE_ALIGNMENT = 256        # context.rs:1684

# symbol -> (restype, argtypes); every prototype of the header appears here and
# tests/test_abi.py checks the two lists against each other.
class Fp8QueryAKvArgs(C.Structure):
    """FerruleHipFp8QueryAKvArgs == FerruleCutlassFp8QueryAKvArgs (96 bytes)."""
    _fields_ = [("rows", u32), ("n1", u32), ("n2", u32), ("k", u32), ("scale_cols", u32),
                ("activation_fp8", u64), ("activation_ue8m0", u64), ("query_a_weight_fp8", u64),
                ("query_a_weight_ue8m0", u64), ("kv_weight_fp8", u64), ("kv_weight_ue8m0", u64),
                ("query_a_output_f32", u64), ("kv_output_f32", u64), ("stream", u64)]


class Fp8BlockGemmArgs(C.Structure):
    """FerruleHipFp8BlockGemmArgs (72 bytes); no reference counterpart."""
    _fields_ = [("rows", u32), ("n", u32), ("k", u32), ("scale_cols", u32), ("weight_scale_kind", u32),
                ("flags", u32), ("activation_fp8", u64), ("activation_ue8m0", u64), ("weight_fp8", u64),
                ("weight_scales", u64), ("output", u64), ("stream", u64)]


class GroupedFp4MoeArgs(C.Structure):
    """FerruleHipGroupedFp4MoeArgs == FerruleCutlassGroupedFp4MoeArgs (224 bytes)."""
    _fields_ = [("active_group_count", u32), ("small_group_count", u32), ("slot_capacity", u32),
                ("max_group_rows", u32), ("total_routed_rows", u32), ("num_tokens", u32), ("num_routes", u32),
                ("input_size", u32), ("intermediate_size", u32), ("hidden_size", u32), ("swiglu_limit", f32),
                ("active_expert_slots", u64), ("active_group_generations", u64), ("expert_route_indptr", u64),
                ("expert_route_counts", u64), ("route_token_indices", u64), ("route_indices", u64),
                ("route_weights", u64), ("slot_generations", u64), ("gate_ptrs", u64), ("gate_scale_ptrs", u64),
                ("up_ptrs", u64), ("up_scale_ptrs", u64), ("down_ptrs", u64), ("down_scale_ptrs", u64),
                ("input_fp8", u64), ("input_ue8m0", u64), ("route_output", u64), ("route_written", u64),
                ("route_error", u64), ("workspace", u64), ("workspace_bytes", u64), ("stream", u64)]


class PrepareMxfp4SfbArgs(C.Structure):
    """FerruleHipPrepareMxfp4SfbArgs == FerruleCutlassPrepareMxfp4SfbArgs (40 bytes)."""
    _fields_ = [("n", u32), ("k", u32), ("reserved0", u32), ("linear_source", u64),
                ("prepared_destination", u64), ("stream", u64)]


class PrepareMxfp4BlockMajorArgs(C.Structure):
    """FerruleHipPrepareMxfp4BlockMajorArgs (48 bytes)."""
    _fields_ = [("n", u32), ("k", u32), ("weight_source", u64), ("scale_source", u64),
                ("weight_destination", u64), ("scale_destination", u64), ("stream", u64)]


class PrepareFp8BlockMajorArgs(C.Structure):
    """FerruleHipPrepareFp8BlockMajorArgs (32 bytes)."""
    _fields_ = [("n", u32), ("k", u32), ("weight_source", u64), ("weight_destination", u64), ("stream", u64)]


class MxSplitArgs(C.Structure):
    """FerruleHipMxSplitArgs (48 bytes; include/ferrule_hip_diagnostics.h)."""
    _fields_ = [("rows", u32), ("k", u32), ("input_kind", u32), ("reserved", u32), ("input", u64), ("q", u64),
                ("s", u64), ("stream", u64)]


class SharedFfnArgs(C.Structure):
    """FerruleHipSharedFfnArgs == FerruleCutlassSharedFfnArgs (160 bytes)."""
    _fields_ = [("input_fp8", u64), ("input_ue8m0", u64), ("gate_weight_fp8", u64), ("gate_weight_ue8m0", u64),
                ("up_weight_fp8", u64), ("up_weight_ue8m0", u64), ("down_weight_fp8", u64),
                ("down_weight_ue8m0", u64), ("hidden_f32", u64), ("hidden_fp8", u64), ("hidden_ue8m0", u64),
                ("output_f32", u64), ("rows", u32), ("input_size", u32), ("intermediate_size", u32),
                ("output_size", u32), ("gate_block_m", u32), ("gate_block_k", u32), ("up_block_m", u32),
                ("up_block_k", u32), ("down_block_m", u32), ("down_block_k", u32), ("output_scale", f32),
                ("swiglu_limit", f32), ("flags", u32), ("stream", u64)]


SHARED_FFN_ACCUMULATE = 1
SHARED_FFN_TILE_SCHEDULE = 2
GEMM_OUTPUT_BF16 = 1
GEMM_TILE_SCHEDULE = 2
FP8_ROWS_MAX = 32   # rows up to which the FP8 x FP8 entries take the decode-row schedule

PROTOTYPES = {
    "ferrule_hip_provider_manifest": (ProviderManifest, []),
    "ferrule_hip_last_error_code": (C.c_int32, []),
    "ferrule_hip_source_digest": (C.c_char_p, []),
    "ferrule_hip_quant_gemv_can_implement": (C.c_int32, [C.POINTER(QuantGemvArgs)]),
    "ferrule_hip_quant_gemv_launch": (C.c_int32, [C.POINTER(QuantGemvArgs)]),
    "ferrule_hip_quant_gemv_multi_can_implement": (C.c_int32, [C.POINTER(QuantGemvMultiArgs)]),
    "ferrule_hip_quant_gemv_multi_launch": (C.c_int32, [C.POINTER(QuantGemvMultiArgs)]),
    "ferrule_hip_dense_ffn_decode_can_implement": (C.c_int32, [C.POINTER(DenseFfnDecodeArgs)]),
    "ferrule_hip_dense_ffn_decode_launch": (C.c_int32, [C.POINTER(DenseFfnDecodeArgs)]),
    "ferrule_hip_dequant_launch": (C.c_int32, [C.POINTER(QuantGemvArgs)]),
    "ferrule_hip_core_linear_launch": (C.c_int32, [C.POINTER(LinearArgs)]),
    "ferrule_hip_core_quantize_launch": (C.c_int32, [C.POINTER(QuantizeArgs)]),
    "ferrule_hip_fp8_converter_selftest_launch": (C.c_int32, [C.c_uint64, C.c_uint64]),
    "ferrule_hip_mx_split_launch": (C.c_int32, [C.POINTER(MxSplitArgs)]),
    "ferrule_hip_core_expert_group_route_plan_launch": (C.c_int32, [C.POINTER(ExpertGroupRoutePlanArgs)]),
    "ferrule_hip_core_moe_launch": (C.c_int32, [C.POINTER(MoeArgs)]),
    "ferrule_hip_core_router_launch": (C.c_int32, [C.POINTER(RouterArgs)]),
    "ferrule_hip_hc_producer_can_implement": (C.c_int32, [C.POINTER(HcProducerArgs)]),
    "ferrule_hip_hc_producer_launch": (C.c_int32, [C.POINTER(HcProducerArgs)]),
    "ferrule_hip_core_expert_table_launch": (C.c_int32, [C.POINTER(ExpertTableArgs)]),
    "ferrule_hip_moe_decode_workspace_size": (C.c_uint64, [C.POINTER(MoeDecodeArgs)]),
    "ferrule_hip_moe_decode_can_implement": (C.c_int32, [C.POINTER(MoeDecodeArgs)]),
    "ferrule_hip_moe_decode_launch": (C.c_int32, [C.POINTER(MoeDecodeArgs)]),
    "ferrule_hip_moe_decode_launch_static_workspace": (C.c_int32, [C.POINTER(MoeDecodeArgs)]),
    "ferrule_hip_fp8_query_a_kv_can_implement": (C.c_int32, [C.POINTER(Fp8QueryAKvArgs)]),
    "ferrule_hip_fp8_query_a_kv_launch": (C.c_int32, [C.POINTER(Fp8QueryAKvArgs)]),
    "ferrule_hip_fp8_projection_can_implement": (C.c_int32, [C.POINTER(Fp8QueryAKvArgs)]),
    "ferrule_hip_fp8_projection_launch": (C.c_int32, [C.POINTER(Fp8QueryAKvArgs)]),
    "ferrule_hip_fp8_block_gemm_can_implement": (C.c_int32, [C.POINTER(Fp8BlockGemmArgs)]),
    "ferrule_hip_fp8_block_gemm_launch": (C.c_int32, [C.POINTER(Fp8BlockGemmArgs)]),
    "ferrule_hip_shared_ffn_can_implement": (C.c_int32, [C.POINTER(SharedFfnArgs)]),
    "ferrule_hip_shared_ffn_launch": (C.c_int32, [C.POINTER(SharedFfnArgs)]),
    "ferrule_hip_grouped_fp4_moe_workspace_size": (C.c_uint64, [C.POINTER(GroupedFp4MoeArgs)]),
    "ferrule_hip_grouped_fp4_moe_can_implement": (C.c_int32, [C.POINTER(GroupedFp4MoeArgs)]),
    "ferrule_hip_grouped_fp4_moe_launch": (C.c_int32, [C.POINTER(GroupedFp4MoeArgs)]),
    "ferrule_hip_grouped_fp4_moe_block_major_launch": (C.c_int32, [C.POINTER(GroupedFp4MoeArgs)]),
    "ferrule_hip_grouped_fp4_moe_debug_launch": (C.c_int32, [C.POINTER(GroupedFp4MoeArgs), C.c_uint64]),
    "ferrule_hip_mxfp4_sfb_storage_bytes": (C.c_uint64, [C.c_uint32, C.c_uint32]),
    "ferrule_hip_prepare_mxfp4_sfb": (C.c_int32, [C.POINTER(PrepareMxfp4SfbArgs)]),
    "ferrule_hip_prepare_mxfp4_block_major": (C.c_int32, [C.POINTER(PrepareMxfp4BlockMajorArgs)]),
    "ferrule_hip_prepare_fp8_block_major": (C.c_int32, [C.POINTER(PrepareFp8BlockMajorArgs)]),
}

_lib = None


class ProviderLibraryMissing(RuntimeError):
    pass


class ProviderLibraryStale(RuntimeError):
    pass


def load() -> C.CDLL:
    """dlopen the provider. Raises if it has not been built (python -m ferrule_amd.build)."""
    global _lib
    if _lib is not None:
        return _lib
    # This Python host borrows torch's streams and device memory, so both must share
    # ONE HIP runtime.  torch ships its own libamdhip64.so.7; whichever copy is loaded
    # first serves every later request for that SONAME, and kernels registered with a
    # second runtime see no device (hipErrorNoDevice).  Load torch's first.
    import torch  # noqa: F401

    if not os.path.exists(LIB_PATH):
        raise ProviderLibraryMissing(
            f"{LIB_PATH} is missing: build it with `python -m ferrule_amd.build` "
            "(there is no CPU fallback for the provider)")
    lib = C.CDLL(LIB_PATH)
    # a library compiled from other sources (or other argument-block layouts) than the
    # ones on disk would misread the blocks this module builds: refuse it
    from . import build as _build

    try:
        digest_fn = lib.ferrule_hip_source_digest
    except AttributeError as exc:
        raise ProviderLibraryStale(f"{LIB_PATH} predates the source digest: rebuild it with "
                                   "`python -m ferrule_amd.build`") from exc
    digest_fn.restype = C.c_char_p
    built_from = digest_fn().decode()
    if built_from != _build.source_digest():
        raise ProviderLibraryStale(
            f"{LIB_PATH} was built from other sources than those on disk (digest {built_from[:12]}... "
            f"!= {_build.source_digest()[:12]}...): rebuild it with `python -m ferrule_amd.build`")
    for name, (res, args) in PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib
