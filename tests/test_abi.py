"""CPU-side checks of the C ABI: the library loads without a GPU, exports every
symbol the header declares, the ctypes mirrors have the reference's sizes, and
argument validation (which touches no device) returns the documented codes."""
import ctypes as C
import os
import re

import pytest

from ferrule_amd import abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = open(os.path.join(ROOT, "include", "ferrule_hip_provider.h")).read()


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
