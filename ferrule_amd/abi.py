"""ctypes mirror of ``include/ferrule_hip_provider.h`` and the library loader.

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

KERNEL_FP8_QUERY_A_KV = 1
KERNEL_SHARED_FFN = 4
KERNEL_GROUPED_FP4_MOE = 5
KERNEL_FP8_PROJECTION = 10
KERNEL_QUANT_GEMV = 33
KERNEL_MOE_DECODE = 34
KERNEL_FP8_BLOCK_GEMM = 35

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


# symbol -> (restype, argtypes); every prototype of the header appears here and
# tests/test_abi.py checks the two lists against each other.
PROTOTYPES = {
    "ferrule_hip_provider_manifest": (ProviderManifest, []),
    "ferrule_hip_last_error_code": (C.c_int32, []),
    "ferrule_hip_quant_gemv_can_implement": (C.c_int32, [C.POINTER(QuantGemvArgs)]),
    "ferrule_hip_quant_gemv_launch": (C.c_int32, [C.POINTER(QuantGemvArgs)]),
    "ferrule_hip_dequant_launch": (C.c_int32, [C.POINTER(QuantGemvArgs)]),
    "ferrule_hip_core_linear_launch": (C.c_int32, [C.POINTER(LinearArgs)]),
    "ferrule_hip_core_quantize_launch": (C.c_int32, [C.POINTER(QuantizeArgs)]),
}

_lib = None


class ProviderLibraryMissing(RuntimeError):
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
    for name, (res, args) in PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib
