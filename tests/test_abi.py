"""CPU-side checks of the C ABI: the library loads without a GPU, exports every
symbol the header declares, the ctypes mirrors have the reference's sizes, and
argument validation (which touches no device) returns the documented codes."""
import ctypes as C
import os
import re

import pytest

from ferrule_amd import abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
import glob

# every header under include/: the provider ABI and the diagnostic entry points
HEADER = "\n".join(open(path).read() for path in sorted(glob.glob(os.path.join(ROOT, "include", "*.h"))))


def declared_symbols():
    return sorted(set(re.findall(r"\b(ferrule_hip_[a-z0-9_]+)\s*\(", HEADER)))


def test_library_loads_and_exports_every_declared_symbol():
    lib = abi.load()
    names = declared_symbols()
    assert names, "no prototypes found in the header"
    for name in names:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
        assert name in abi.PROTOTYPES, f"{name} has no ctypes prototype"
    assert sorted(abi.PROTOTYPES) == names


def test_pod_layouts_match_the_reference_sizes():
    # abi/core_provider.h:512-535
    assert C.sizeof(abi.LinearArgs) == 88 and abi.LinearArgs.x.offset == 40 and abi.LinearArgs.stream.offset == 80
    assert C.sizeof(abi.QuantizeArgs) == 64 and abi.QuantizeArgs.values.offset == 32
    assert abi.QuantizeArgs.stream.offset == 56
    assert C.sizeof(abi.QuantGemvArgs) == 80 and abi.QuantGemvArgs.x.offset == 40
    assert C.sizeof(abi.ProviderManifest) == 8
    for m in re.finditer(r"FERRULE_HIP_ASSERT_LAYOUT\((\w+),\s*(\d+),\s*(\w+),\s*(\d+),\s*(\d+)\)", HEADER):
        name, size, first, first_off, stream_off = m.groups()
        cls = getattr(abi, name.replace("FerruleHip", ""))
        assert C.sizeof(cls) == int(size), name
        assert getattr(cls, first).offset == int(first_off), name
        assert cls.stream.offset == int(stream_off), name


def test_manifest_sets_only_implemented_bits():
    mask = abi.load().ferrule_hip_provider_manifest().kernel_mask
    assert mask & abi.kernel_bit(abi.KERNEL_QUANT_GEMV)
    known = 0
    for name in dir(abi):
        if name.startswith("KERNEL_") and isinstance(getattr(abi, name), int):
            known |= abi.kernel_bit(getattr(abi, name))
    assert mask & ~known == 0


def _gemv_args(**kw):
    a = abi.QuantGemvArgs()
    base = dict(weight_format=abi.WEIGHT_MXFP4_E2M1, scale_kind=abi.SCALE_E8M0, batch=1, n=64, k=256,
                block_m=1, block_k=32, scale_cols=8, x=0x1000, weight=0x2000, weight_scales=0x3000,
                output=0x4000)
    base.update(kw)
    for key, value in base.items():
        setattr(a, key, value)
    return a


def test_gemv_validation_codes_without_touching_a_device():
    lib = abi.load()
    ok = lib.ferrule_hip_quant_gemv_can_implement
    assert ok(None) == abi.INVALID_ARGUMENT
    assert ok(C.byref(_gemv_args())) == abi.SUCCESS
    assert ok(C.byref(_gemv_args(batch=0))) == abi.INVALID_ARGUMENT
    assert ok(C.byref(_gemv_args(weight=0))) == abi.INVALID_ARGUMENT
    assert ok(C.byref(_gemv_args(weight=0x2008))) == abi.INVALID_ARGUMENT      # 16-byte alignment
    assert ok(C.byref(_gemv_args(scale_cols=7))) == abi.INVALID_ARGUMENT
    assert ok(C.byref(_gemv_args(weight_format=9))) == abi.INVALID_ARGUMENT
    assert ok(C.byref(_gemv_args(scale_kind=abi.SCALE_F32))) == abi.INVALID_ARGUMENT   # MXFP4 is E8M0 only
    assert ok(C.byref(_gemv_args(k=250, scale_cols=8))) == abi.INVALID_ARGUMENT
    fp8 = dict(weight_format=abi.WEIGHT_FP8_E4M3, block_m=128, block_k=128, scale_cols=2)
    assert ok(C.byref(_gemv_args(**fp8))) == abi.SUCCESS
    assert ok(C.byref(_gemv_args(scale_kind=abi.SCALE_F32, **fp8))) == abi.SUCCESS
    # launch re-validates (reference: cutlass.rs:2851-2861) and must not reach the device
    assert lib.ferrule_hip_quant_gemv_launch(C.byref(_gemv_args(n=0))) == abi.INVALID_ARGUMENT


def test_provider_context_refuses_to_run_without_a_gpu():
    import torch

    from ferrule_amd.provider import HipArtifactOperatorContext

    if torch.cuda.is_available():
        pytest.skip("GPU present")
    with pytest.raises(RuntimeError):
        HipArtifactOperatorContext()


def test_shape_storage_lengths_follow_the_reference_rules():
    from ferrule_amd.provider import HipArtifactLinearShape as S

    assert S.fp4_e2m1_packed_with_e8m0_scale(4096, 7168).storage_lengths() == (14680064, 917504)
    assert S.fp8_e4m3_with_e8m0_scale(4096, 4096).storage_lengths() == (16777216, 1024)
    assert S.fp8_e4m3_with_f32_scale(4096, 4096).storage_lengths() == (16777216, 4096)
    assert S.fp8_e4m3_with_e8m0_scale(2, 3, 1, 2).storage_lengths() == (6, 4)     # weight.rs:505-535
    with pytest.raises(ValueError):
        S.fp4_e2m1_packed_with_e8m0_scale(4, 48).storage_lengths()


def test_fp8_gemm_validation_codes_without_touching_a_device():
    # capabilities/fp8_projection.cuh:67-97 and implementations/cutlass/entrypoints.cu:1234-1253
    lib = abi.load()

    def qkv(**kw):
        base = dict(rows=4, n1=256, n2=0, k=256, scale_cols=2, activation_fp8=0x1000, activation_ue8m0=0x2000,
                    query_a_weight_fp8=0x3000, query_a_weight_ue8m0=0x4000, query_a_output_f32=0x5000)
        base.update(kw)
        return C.byref(abi.Fp8QueryAKvArgs(**base))

    proj = lib.ferrule_hip_fp8_projection_can_implement
    assert proj(None) == abi.INVALID_ARGUMENT
    assert proj(qkv()) == abi.SUCCESS
    assert proj(qkv(n2=8)) == abi.INVALID_ARGUMENT                    # single projection: kv fields must be zero
    assert proj(qkv(kv_output_f32=0x6000)) == abi.INVALID_ARGUMENT
    assert proj(qkv(k=200, scale_cols=1)) == abi.INVALID_ARGUMENT     # k % 128
    assert proj(qkv(scale_cols=3)) == abi.INVALID_ARGUMENT
    assert proj(qkv(rows=0)) == abi.INVALID_ARGUMENT
    assert proj(qkv(rows=8 * 65535 + 1)) == abi.INVALID_ARGUMENT      # kMaxRows
    assert proj(qkv(activation_fp8=0x1004)) == abi.INVALID_ARGUMENT   # 16-byte alignment
    both = lib.ferrule_hip_fp8_query_a_kv_can_implement
    assert both(qkv()) == abi.INVALID_ARGUMENT                        # n2 == 0
    assert both(qkv(n2=64, kv_weight_fp8=0x6000, kv_weight_ue8m0=0x7000, kv_output_f32=0x8000)) == abi.SUCCESS
    assert lib.ferrule_hip_fp8_projection_launch(qkv(rows=0)) == abi.INVALID_ARGUMENT

    def gemm(**kw):
        base = dict(rows=4, n=256, k=256, scale_cols=2, weight_scale_kind=abi.SCALE_F32, flags=abi.GEMM_OUTPUT_BF16,
                    activation_fp8=0x1000, activation_ue8m0=0x2000, weight_fp8=0x3000, weight_scales=0x4000,
                    output=0x5000)
        base.update(kw)
        return C.byref(abi.Fp8BlockGemmArgs(**base))

    ok = lib.ferrule_hip_fp8_block_gemm_can_implement
    assert ok(gemm()) == abi.SUCCESS
    assert ok(gemm(weight_scale_kind=7)) == abi.INVALID_ARGUMENT
    assert ok(gemm(flags=abi.GEMM_TILE_SCHEDULE)) == abi.SUCCESS
    assert ok(gemm(flags=4)) == abi.INVALID_ARGUMENT
    assert ok(gemm(k=65536, scale_cols=512)) == abi.UNSUPPORTED        # token scales of a tile exceed LDS
    assert ok(gemm(rows=8 * 65535, n=1 << 30)) == abi.UNSUPPORTED      # more 128x128 tiles than a 1-D grid holds
    assert ok(gemm(rows=8 * 65535, n=18432)) == abi.SUCCESS


def test_shared_ffn_and_grouped_moe_validation_codes_without_touching_a_device():
    lib = abi.load()

    def ffn(**kw):
        base = dict(input_fp8=0x1000, input_ue8m0=0x2000, gate_weight_fp8=0x3000, gate_weight_ue8m0=0x4000,
                    up_weight_fp8=0x5000, up_weight_ue8m0=0x6000, down_weight_fp8=0x7000, down_weight_ue8m0=0x8000,
                    hidden_f32=0x9000, hidden_fp8=0xA000, hidden_ue8m0=0xB000, output_f32=0xC000, rows=3,
                    input_size=256, intermediate_size=128, output_size=64, gate_block_m=128, gate_block_k=128,
                    up_block_m=128, up_block_k=128, down_block_m=128, down_block_k=128, output_scale=1.0,
                    swiglu_limit=0.0, flags=0)
        base.update(kw)
        return C.byref(abi.SharedFfnArgs(**base))

    ok = lib.ferrule_hip_shared_ffn_can_implement
    assert ok(None) == abi.INVALID_ARGUMENT
    assert ok(ffn()) == abi.SUCCESS
    assert ok(ffn(flags=abi.SHARED_FFN_ACCUMULATE)) == abi.SUCCESS
    assert ok(ffn(flags=abi.SHARED_FFN_TILE_SCHEDULE)) == abi.SUCCESS  # schedule choice, no reference counterpart
    assert ok(ffn(flags=4)) == abi.INVALID_ARGUMENT                    # shared_ffn.cuh kKnownFlags
    assert ok(ffn(gate_block_k=64)) == abi.INVALID_ARGUMENT            # kUnsupportedArtifactBlocks
    assert ok(ffn(intermediate_size=96)) == abi.INVALID_ARGUMENT
    assert ok(ffn(output_size=40)) == abi.INVALID_ARGUMENT
    assert ok(ffn(output_scale=float("inf"))) == abi.INVALID_ARGUMENT
    assert ok(ffn(hidden_fp8=0)) == abi.INVALID_ARGUMENT
    assert lib.ferrule_hip_shared_ffn_launch(ffn(rows=0)) == abi.INVALID_ARGUMENT

    def moe(**kw):
        base = dict(active_group_count=2, small_group_count=2, slot_capacity=4, max_group_rows=5, total_routed_rows=8,
                    num_tokens=4, num_routes=8, input_size=256, intermediate_size=128, hidden_size=64, swiglu_limit=0.0)
        base.update(kw)
        return abi.GroupedFp4MoeArgs(**base)

    size = lib.ferrule_hip_grouped_fp4_moe_workspace_size
    assert size(None) == 0
    need = size(C.byref(moe()))                     # scalar fields only, every pointer zero
    assert need > 8 * 128 and need % 256 == 0
    assert size(C.byref(moe(hidden_size=72))) == 0   # hidden % 64 (grouped_fp4_moe.cuh:206-229)
    assert size(C.byref(moe(total_routed_rows=9))) == 0      # more rows than routes
    assert size(C.byref(moe(total_routed_rows=1))) == 0      # fewer rows than groups
    can = lib.ferrule_hip_grouped_fp4_moe_can_implement
    assert can(C.byref(moe())) == abi.INVALID_ARGUMENT        # null pointers
    fields = ("active_expert_slots", "expert_route_indptr", "route_token_indices", "route_indices", "route_weights",
              "gate_ptrs", "gate_scale_ptrs", "up_ptrs", "up_scale_ptrs", "down_ptrs", "down_scale_ptrs", "input_fp8",
              "input_ue8m0", "route_output", "route_written", "route_error", "workspace")
    pointers = {name: 0x10000 * (i + 1) for i, name in enumerate(fields)}
    assert can(C.byref(moe(workspace_bytes=need, **pointers))) == abi.SUCCESS
    # rows of the input plane and of one expert matrix are addressed with 32-bit offsets
    huge = moe(num_tokens=1 << 20, num_routes=1 << 20, total_routed_rows=1 << 20, max_group_rows=1 << 20,
               input_size=4096, **pointers)
    huge.workspace_bytes = size(C.byref(huge))
    assert huge.workspace_bytes > 0 and can(C.byref(huge)) == abi.UNSUPPORTED
    wide = moe(hidden_size=1 << 20, intermediate_size=8192, **pointers)
    wide.workspace_bytes = size(C.byref(wide))
    assert wide.workspace_bytes > 0 and can(C.byref(wide)) == abi.UNSUPPORTED
    assert lib.ferrule_hip_mxfp4_sfb_storage_bytes(2048, 7168) == 2048 * 7168 // 32
    assert lib.ferrule_hip_mxfp4_sfb_storage_bytes(2048, 100) == 0
    bad = abi.PrepareMxfp4SfbArgs(n=16, k=64, reserved0=1, linear_source=0x1000, prepared_destination=0x2000)
    assert lib.ferrule_hip_prepare_mxfp4_sfb(C.byref(bad)) == abi.INVALID_ARGUMENT


def test_block_major_preparation_validates_before_any_launch():
    lib = abi.load()
    fn = lib.ferrule_hip_prepare_mxfp4_block_major

    def args(**kw):
        base = dict(n=32, k=256, weight_source=0x10000, scale_source=0x20000, weight_destination=0x30000,
                    scale_destination=0x40000, stream=0)
        base.update(kw)
        return abi.PrepareMxfp4BlockMajorArgs(**base)

    assert C.sizeof(abi.PrepareMxfp4BlockMajorArgs) == 48
    assert fn(None) == abi.INVALID_ARGUMENT
    assert fn(C.byref(args(n=0))) == abi.INVALID_ARGUMENT
    assert fn(C.byref(args(n=24))) == abi.UNSUPPORTED            # whole 16-row tiles only
    assert fn(C.byref(args(k=192))) == abi.UNSUPPORTED           # whole 128-wide K blocks only
    assert fn(C.byref(args(weight_source=0))) == abi.INVALID_ARGUMENT
    assert fn(C.byref(args(scale_destination=0x40004))) == abi.INVALID_ARGUMENT   # alignment
    # 32 x 256 payload is 4096 bytes: a destination inside the source range overlaps
    assert fn(C.byref(args(weight_destination=0x10800))) == abi.INVALID_ARGUMENT
    assert fn(C.byref(args(scale_destination=0x20010))) == abi.INVALID_ARGUMENT


def test_fp8_block_major_preparation_validates_before_any_launch():
    lib = abi.load()
    fn = lib.ferrule_hip_prepare_fp8_block_major

    def args(**kw):
        base = dict(n=32, k=256, weight_source=0x10000, weight_destination=0x30000, stream=0)
        base.update(kw)
        return abi.PrepareFp8BlockMajorArgs(**base)

    assert C.sizeof(abi.PrepareFp8BlockMajorArgs) == 32
    assert fn(None) == abi.INVALID_ARGUMENT
    assert fn(C.byref(args(k=0))) == abi.INVALID_ARGUMENT
    assert fn(C.byref(args(n=8))) == abi.UNSUPPORTED
    assert fn(C.byref(args(k=320))) == abi.UNSUPPORTED
    assert fn(C.byref(args(weight_destination=0))) == abi.INVALID_ARGUMENT
    assert fn(C.byref(args(weight_source=0x10008))) == abi.INVALID_ARGUMENT
    assert fn(C.byref(args(weight_destination=0x11000))) == abi.INVALID_ARGUMENT   # inside the 8 KiB source


def test_moe_decode_validation_codes_without_touching_a_device():
    lib = abi.load()
    ptr_fields = ("active_expert_slots", "expert_route_indptr", "route_token_indices", "route_indices",
                  "route_weights", "gate_ptrs", "gate_scale_ptrs", "up_ptrs", "up_scale_ptrs", "down_ptrs",
                  "down_scale_ptrs", "input_bf16", "route_output", "route_written", "route_error", "workspace")

    def moe(**kw):
        base = dict(active_group_count=4, slot_capacity=4, total_routed_rows=8, num_tokens=4, num_routes=8,
                    routes_per_token=2, input_size=512, intermediate_size=256, hidden_size=256, flags=0,
                    swiglu_limit=0.0, workspace_bytes=1 << 30)
        base.update({name: 0x10000 * (i + 1) for i, name in enumerate(ptr_fields)})
        base.update(kw)
        return C.byref(abi.MoeDecodeArgs(**base))

    ok = lib.ferrule_hip_moe_decode_can_implement
    assert ok(None) == abi.INVALID_ARGUMENT
    assert ok(moe()) == abi.SUCCESS
    assert ok(moe(hidden_size=64)) == abi.SUCCESS          # one partial group of row tiles
    assert ok(moe(hidden_size=192)) == abi.UNSUPPORTED     # a partial group after a whole one
    assert ok(moe(hidden_size=72)) == abi.UNSUPPORTED
    assert ok(moe(input_size=384)) == abi.UNSUPPORTED      # K chunks of four 128-wide blocks
    assert ok(moe(intermediate_size=128)) == abi.UNSUPPORTED
    assert ok(moe(num_routes=7)) == abi.INVALID_ARGUMENT   # tokens x routes_per_token
    assert ok(moe(route_weights=0)) == abi.INVALID_ARGUMENT
    assert ok(moe(workspace=0x10010)) == abi.INVALID_ARGUMENT
    assert ok(moe(workspace_bytes=16)) == abi.INVALID_ARGUMENT
    assert lib.ferrule_hip_moe_decode_workspace_size(moe()) > 0
