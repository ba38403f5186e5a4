"""ctypes/numpy front end of the CPU checker (``libferrule_oracle.so``).

TEST INFRASTRUCTURE ONLY.  Importable from ``tests/``, from
``__graft_entry__.smoke()`` and from the CPU-baseline leg of ``bench.py``;
nothing in the ``ferrule_amd`` package may import this module.

Every wrapper keeps the reference citation of the C function it calls (see
``ferrule_oracle.h``).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libferrule_oracle.so")

SCALE_E8M0 = 0
SCALE_F32 = 1


def build(force: bool = False) -> str:
    """Compile the checker with gcc (a few hundred ms)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"])
    return _LIB_PATH


def _load() -> C.CDLL:
    build()
    lib = C.CDLL(_LIB_PATH)
    f32p = C.POINTER(C.c_float)
    u8p = C.POINTER(C.c_uint8)
    sz = C.c_size_t
    sig = {
        "fo_decode_fp4_e2m1_nibble": (C.c_float, [C.c_uint8]),
        "fo_decode_fp4_e2m1_packed_low_first": (None, [u8p, sz, f32p]),
        "fo_decode_e8m0_scale": (C.c_float, [C.c_uint8]),
        "fo_decode_fp8_e4m3fn_byte": (C.c_float, [C.c_uint8]),
        "fo_dequantize_fp4_e2m1_with_e8m0_scales": (C.c_int, [u8p, u8p, sz, sz, sz, f32p]),
        "fo_dequantize_fp8_e4m3fn_with_e8m0_scales": (C.c_int, [u8p, u8p, sz, sz, sz, sz, f32p]),
        "fo_dequantize_fp8_e4m3fn_with_f32_scales": (C.c_int, [u8p, f32p, sz, sz, sz, sz, f32p]),
        "fo_rounded_power_of_two_scale": (C.c_float, [C.c_float, C.c_float]),
        "fo_quantize_fp8_e4m3fn_to_f32": (C.c_float, [C.c_float]),
        "fo_quantize_fp4_e2m1_to_f32": (C.c_float, [C.c_float]),
        "fo_simulate_fp8_act_quant_in_place": (C.c_int, [f32p, sz, sz, sz]),
        "fo_simulate_fp4_act_quant_in_place": (C.c_int, [f32p, sz, sz, sz]),
        "fo_pack_fp8_act": (C.c_int, [f32p, sz, sz, sz, u8p, u8p]),
        "fo_pack_fp4_act": (C.c_int, [f32p, sz, sz, sz, u8p, u8p]),
        "fo_round_to_bf16": (C.c_float, [C.c_float]),
        "fo_bf16_bits": (C.c_uint16, [C.c_float]),
        "fo_matvec_row_major": (None, [f32p, sz, sz, f32p, f32p]),
        "fo_linear_fp4_matvec": (C.c_int, [u8p, u8p, sz, sz, sz, f32p, f32p, C.c_int]),
        "fo_linear_fp8_matvec": (C.c_int, [u8p, C.c_void_p, C.c_int, sz, sz, sz, sz, f32p, f32p, C.c_int]),
        "fo_linear_fp4_matvec_materialized": (C.c_int, [u8p, u8p, sz, sz, sz, f32p, f32p]),
        "fo_linear_fp8_matvec_materialized": (C.c_int, [u8p, C.c_void_p, C.c_int, sz, sz, sz, sz, f32p, f32p]),
        "fo_abs_linear_fp4": (C.c_int, [u8p, u8p, sz, sz, sz, C.POINTER(C.c_double), C.POINTER(C.c_double), C.c_int]),
        "fo_abs_linear_fp8": (C.c_int, [u8p, C.c_void_p, C.c_int, sz, sz, sz, sz, C.POINTER(C.c_double),
                                        C.POINTER(C.c_double), C.c_int]),
        "fo_silu": (C.c_float, [C.c_float]),
        "fo_expert_execute_fp4": (C.c_int, [u8p, u8p, u8p, u8p, u8p, u8p, sz, sz, sz, f32p,
                                            C.c_float, C.c_float, sz, f32p, f32p, C.c_int]),
        "fo_accumulate_routes": (None, [f32p, sz, sz, f32p, f32p]),
        "fo_swiglu_ffn_f32": (None, [f32p, f32p, f32p, sz, sz, f32p, C.c_float, C.c_float, f32p]),
        "fo_reduce_routes_ranked": (None, [f32p, sz, sz, sz, f32p]),
        "fo_expert_table_publish": (None, [C.c_uint32, C.c_uint32, C.c_uint32, C.c_int32, C.POINTER(C.c_uint64),
                                           C.POINTER(C.c_uint64), C.c_uint32] + [C.POINTER(C.c_int32)] * 3),
        "fo_expert_resolve_init": (None, [C.POINTER(C.c_int32), C.c_uint32, C.c_uint32]),
        "fo_expert_resolve": (None, [C.POINTER(C.c_int32)] + [C.c_uint32] * 4 + [C.POINTER(C.c_int32)] * 7),
        "fo_expert_gather_dispatch": (C.c_int32, [C.c_uint32, C.c_uint32, C.c_int32, C.POINTER(C.c_uint64)] +
                                      [C.POINTER(C.c_int32)] * 3 + [f32p, C.POINTER(C.c_int32),
                                                                    C.POINTER(C.c_uint64), f32p,
                                                                    C.POINTER(C.c_int32)]),
        "fo_hc_split_sinkhorn": (C.c_int, [f32p, sz, sz, sz, C.c_float, f32p, f32p, f32p, f32p, f32p]),
        "fo_rms_norm": (C.c_int, [f32p, f32p, sz, C.c_float, f32p]),
        "fo_hc_producer": (C.c_int, [f32p, sz, sz, sz, sz, C.c_float, C.c_float, C.c_float, C.c_int, f32p, f32p, f32p,
                                     f32p, f32p, f32p, f32p, f32p, f32p, f32p, u8p, u8p]),
        "fo_stable_softplus": (C.c_float, [C.c_float]),
        "fo_router_route_sqrt_softplus": (C.c_int, [f32p, sz, f32p, C.POINTER(C.c_int64), sz, sz, C.c_float,
                                                    C.POINTER(C.c_int32), f32p, f32p, f32p]),
        "fo_router_kernel_rows": (None, [C.c_uint32] * 7 + [C.c_float, f32p, f32p, C.POINTER(C.c_int32),
                                                            C.POINTER(C.c_int32), C.c_void_p, f32p]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        _lib = _load()
    return _lib


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.uint8)


def _pf(a: np.ndarray):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _pb(a: np.ndarray):
    return a.ctypes.data_as(C.POINTER(C.c_uint8))


class OracleError(ValueError):
    """The reference would have returned Err(Error::Model{..}) for this shape."""


def _check(rc: int, what: str) -> None:
    if rc != 0:
        raise OracleError(f"{what}: reference rejects this shape (rc={rc})")


# ---- scalars -----------------------------------------------------------------

def decode_fp4_e2m1_nibble(n: int) -> float:
    return lib().fo_decode_fp4_e2m1_nibble(n & 0xFF)


def decode_e8m0_scale(b: int) -> float:
    return lib().fo_decode_e8m0_scale(b & 0xFF)


def decode_fp8_e4m3fn_byte(b: int) -> float:
    return lib().fo_decode_fp8_e4m3fn_byte(b & 0xFF)


def rounded_power_of_two_scale(amax: float, qmax: float) -> float:
    return lib().fo_rounded_power_of_two_scale(amax, qmax)


def quantize_fp8_e4m3fn_to_f32(v: float) -> float:
    return lib().fo_quantize_fp8_e4m3fn_to_f32(v)


def quantize_fp4_e2m1_to_f32(v: float) -> float:
    return lib().fo_quantize_fp4_e2m1_to_f32(v)


def round_to_bf16(v: float) -> float:
    return lib().fo_round_to_bf16(v)


def silu(v: float) -> float:
    return lib().fo_silu(v)


# ---- arrays ------------------------------------------------------------------

def decode_fp4_e2m1_packed_low_first(data) -> np.ndarray:
    data = _u8(data).ravel()
    out = np.empty(data.size * 2, np.float32)
    lib().fo_decode_fp4_e2m1_packed_low_first(_pb(data), data.size, _pf(out))
    return out


def dequantize_fp4(weight, scales, n: int, k: int, block: int = 32) -> np.ndarray:
    weight, scales = _u8(weight).ravel(), _u8(scales).ravel()
    if block == 0 or k % max(block, 1) or k % 2:
        raise OracleError("invalid FP4 shape")
    if weight.size != n * (k // 2) or scales.size != n * (k // block):
        raise OracleError("FP4 length mismatch")
    out = np.empty((n, k), np.float32)
    _check(lib().fo_dequantize_fp4_e2m1_with_e8m0_scales(_pb(weight), _pb(scales), n, k, block, _pf(out)),
           "dequantize_fp4")
    return out


def dequantize_fp8(weight, scales, n: int, k: int, block_m: int = 128, block_k: int = 128) -> np.ndarray:
    """E8M0 scales if ``scales`` is uint8, f32 scales if it is float32."""
    weight = _u8(weight).ravel()
    if block_m == 0 or block_k == 0:
        raise OracleError("invalid FP8 block shape")
    need = -(-n // block_m) * -(-k // block_k)
    if weight.size != n * k or np.asarray(scales).size != need:
        raise OracleError("FP8 length mismatch")
    out = np.empty((n, k), np.float32)
    if np.asarray(scales).dtype == np.float32:
        s = _f32(scales).ravel()
        rc = lib().fo_dequantize_fp8_e4m3fn_with_f32_scales(_pb(weight), _pf(s), n, k, block_m, block_k, _pf(out))
    else:
        s = _u8(scales).ravel()
        rc = lib().fo_dequantize_fp8_e4m3fn_with_e8m0_scales(_pb(weight), _pb(s), n, k, block_m, block_k, _pf(out))
    _check(rc, "dequantize_fp8")
    return out


def simulate_fp8_act_quant(values, row_width: int, block: int = 128) -> np.ndarray:
    v = _f32(values).copy()
    _check(lib().fo_simulate_fp8_act_quant_in_place(_pf(v.reshape(-1)), v.size, row_width, block),
           "simulate_fp8_act_quant")
    return v


def simulate_fp4_act_quant(values, row_width: int, block: int = 32) -> np.ndarray:
    v = _f32(values).copy()
    _check(lib().fo_simulate_fp4_act_quant_in_place(_pf(v.reshape(-1)), v.size, row_width, block),
           "simulate_fp4_act_quant")
    return v


def pack_fp8_act(values, row_width: int, block: int = 128):
    v = _f32(values)
    packed = np.empty(v.size, np.uint8)
    scales = np.empty(v.size // block, np.uint8)
    _check(lib().fo_pack_fp8_act(_pf(v.reshape(-1)), v.size, row_width, block, _pb(packed), _pb(scales)),
           "pack_fp8_act")
    rows = v.size // row_width
    return packed.reshape(rows, row_width), scales.reshape(rows, row_width // block)


def pack_fp4_act(values, row_width: int, block: int = 32):
    v = _f32(values)
    packed = np.empty(v.size // 2, np.uint8)
    scales = np.empty(v.size // block, np.uint8)
    _check(lib().fo_pack_fp4_act(_pf(v.reshape(-1)), v.size, row_width, block, _pb(packed), _pb(scales)),
           "pack_fp4_act")
    rows = v.size // row_width
    return packed.reshape(rows, row_width // 2), scales.reshape(rows, row_width // block)


def round_to_bf16_array(values) -> np.ndarray:
    """Vectorised math.rs:7-14 (same integer arithmetic as fo_round_to_bf16)."""
    bits = _f32(values).view(np.uint32)
    nan = (bits & 0x7FFFFFFF) > 0x7F800000
    bias = np.uint32(0x7FFF) + ((bits >> 16) & 1)
    rounded = (bits + bias) & np.uint32(0xFFFF0000)
    quiet = (((bits >> 16) | 0x0040) & 0xFFFF) << 16
    return np.where(nan, quiet, rounded).astype(np.uint32).view(np.float32)


def bf16_bits_array(values) -> np.ndarray:
    return (round_to_bf16_array(values).view(np.uint32) >> 16).astype(np.uint16)


def matvec_row_major(weights, x) -> np.ndarray:
    w, x = _f32(weights), _f32(x)
    out = np.empty(w.shape[0], np.float32)
    lib().fo_matvec_row_major(_pf(w), w.shape[0], w.shape[1], _pf(x), _pf(out))
    return out


def linear_fp4(weight, scales, n: int, k: int, x, block: int = 32, threads: int = 1,
               materialized: bool = False) -> np.ndarray:
    """LinearWeight::reference_matvec for the FP4 format, one row of x per call row."""
    weight, scales = _u8(weight).ravel(), _u8(scales).ravel()
    x = _f32(x).reshape(-1, k)
    out = np.empty((x.shape[0], n), np.float32)
    for b in range(x.shape[0]):
        if materialized:
            rc = lib().fo_linear_fp4_matvec_materialized(_pb(weight), _pb(scales), n, k, block, _pf(x[b]), _pf(out[b]))
        else:
            rc = lib().fo_linear_fp4_matvec(_pb(weight), _pb(scales), n, k, block, _pf(x[b]), _pf(out[b]), threads)
        _check(rc, "linear_fp4")
    return out


def linear_fp8(weight, scales, n: int, k: int, x, block_m: int = 128, block_k: int = 128,
               threads: int = 1, materialized: bool = False, act_quant_block: int = 0) -> np.ndarray:
    weight = _u8(weight).ravel()
    s = np.asarray(scales)
    if s.dtype == np.float32:
        s = _f32(s).ravel()
        kind = SCALE_F32
    else:
        s = _u8(s).ravel()
        kind = SCALE_E8M0
    x = _f32(x).reshape(-1, k)
    if act_quant_block:
        x = simulate_fp8_act_quant(x, k, act_quant_block)
    out = np.empty((x.shape[0], n), np.float32)
    sp = s.ctypes.data_as(C.c_void_p)
    for b in range(x.shape[0]):
        if materialized:
            rc = lib().fo_linear_fp8_matvec_materialized(_pb(weight), sp, kind, n, k, block_m, block_k,
                                                         _pf(x[b]), _pf(out[b]))
        else:
            rc = lib().fo_linear_fp8_matvec(_pb(weight), sp, kind, n, k, block_m, block_k,
                                            _pf(x[b]), _pf(out[b]), threads)
        _check(rc, "linear_fp8")
    return out


def abs_linear_fp4(weight, scales, n: int, k: int, v, block: int = 32, threads: int = 1) -> np.ndarray:
    """sum_k |dequant(W)[row, k]| * v[k] in float64 (error-bound arithmetic for the tests, not a
    reference function)."""
    weight, scales = _u8(weight).ravel(), _u8(scales).ravel()
    v = np.ascontiguousarray(v, np.float64).ravel()
    if v.size != k or weight.size != n * k // 2 or scales.size != n * (k // block):
        raise OracleError("abs_linear_fp4 shape mismatch")
    out = np.empty(n, np.float64)
    pd = C.POINTER(C.c_double)
    _check(lib().fo_abs_linear_fp4(_pb(weight), _pb(scales), n, k, block, v.ctypes.data_as(pd), out.ctypes.data_as(pd),
                                   threads), "abs_linear_fp4")
    return out


def abs_linear_fp8(weight, scales, n: int, k: int, v, block_m: int = 128, block_k: int = 128,
                   threads: int = 1) -> np.ndarray:
    """sum_k |dequant(W)[row, k]| * v[k] in float64 for the FP8 formats (see abs_linear_fp4)."""
    weight = _u8(weight).ravel()
    s = np.asarray(scales)
    if s.dtype == np.float32:
        s, kind = _f32(s).ravel(), SCALE_F32
    else:
        s, kind = _u8(s).ravel(), SCALE_E8M0
    v = np.ascontiguousarray(v, np.float64).ravel()
    if v.size != k or weight.size != n * k:
        raise OracleError("abs_linear_fp8 shape mismatch")
    out = np.empty(n, np.float64)
    pd = C.POINTER(C.c_double)
    _check(lib().fo_abs_linear_fp8(_pb(weight), s.ctypes.data_as(C.c_void_p), kind, n, k, block_m, block_k,
                                   v.ctypes.data_as(pd), out.ctypes.data_as(pd), threads), "abs_linear_fp8")
    return out


def expert_execute_fp4(gate_w, gate_s, up_w, up_s, down_w, down_s, hidden: int, intermediate: int, x,
                       route_weight: float, swiglu_limit: float = 0.0, block: int = 32,
                       act_quant_block: int = 0, threads: int = 1, return_hidden: bool = False):
    arrs = [_u8(a).ravel() for a in (gate_w, gate_s, up_w, up_s, down_w, down_s)]
    x = _f32(x).ravel()
    if x.size != hidden:
        raise OracleError("expert input length mismatch")
    out = np.empty(hidden, np.float32)
    h = np.empty(intermediate, np.float32)
    rc = lib().fo_expert_execute_fp4(*[_pb(a) for a in arrs], hidden, intermediate, block, _pf(x),
                                     route_weight, swiglu_limit, act_quant_block, _pf(out), _pf(h), threads)
    _check(rc, "expert_execute_fp4")
    return (out, h) if return_hidden else out


def accumulate_routes(route_outputs, shared=None) -> np.ndarray:
    r = _f32(route_outputs)
    out = np.empty(r.shape[1], np.float32)
    sh = _f32(shared) if shared is not None else None
    lib().fo_accumulate_routes(_pf(r), r.shape[0], r.shape[1], _pf(sh) if sh is not None else None, _pf(out))
    return out


def swiglu_ffn_f32(gate, up, down, x, output_scale: float = 1.0, swiglu_limit: float = 0.0) -> np.ndarray:
    g, u, d, x = _f32(gate), _f32(up), _f32(down), _f32(x)
    out = np.empty(d.shape[0], np.float32)
    lib().fo_swiglu_ffn_f32(_pf(g), _pf(u), _pf(d), g.shape[1], g.shape[0], _pf(x), output_scale,
                            swiglu_limit, _pf(out))
    return out


def reduce_routes_ranked(route_output, tokens: int, k: int, hidden: int, prefix=None) -> np.ndarray:
    r = _f32(route_output).reshape(tokens * k, hidden)
    out = np.zeros((tokens, hidden), np.float32) if prefix is None else _f32(prefix).copy().reshape(tokens, hidden)
    lib().fo_reduce_routes_ranked(_pf(r), tokens, k, hidden, _pf(out))
    return out


# ---- router --------------------------------------------------------------------

def stable_softplus(v: float) -> float:
    return lib().fo_stable_softplus(v)


def router_route_sqrt_softplus(logits, top_k: int, route_scale: float, bias=None, hash_experts=None):
    """One token through ``ExpertRouterPolicy::route`` (routing.rs:135-191), sqrt-softplus scores.
    Returns (indices int32 [k], weights, scores, selection scores)."""
    lg = _f32(logits).ravel()
    b = _f32(bias).ravel() if bias is not None else None
    if b is not None and b.size != lg.size:
        raise OracleError("router bias length mismatch")
    hx = np.ascontiguousarray(hash_experts, dtype=np.int64).ravel() if hash_experts is not None else None
    idx = np.empty(top_k, np.int32)
    w, s, sel = (np.empty(top_k, np.float32) for _ in range(3))
    rc = lib().fo_router_route_sqrt_softplus(
        _pf(lg), lg.size, _pf(b) if b is not None else None,
        hx.ctypes.data_as(C.POINTER(C.c_int64)) if hx is not None else None, hx.size if hx is not None else 0,
        top_k, route_scale, idx.ctypes.data_as(C.POINTER(C.c_int32)), _pf(w), _pf(s), _pf(sel))
    _check(rc, "router_route")
    return idx, w, s, sel


def router_kernel_rows(kind: int, logits, k: int, route_scale: float = 1.0, bias=None, token_ids=None,
                       hash_table=None, indices=None, weights=None):
    """The device router restated row by row (portable/entrypoints.cu:770-884).  ``indices`` and
    ``weights`` may be passed in to observe which rows are left untouched."""
    lg = _f32(logits)
    rows, columns = lg.shape
    b = _f32(bias).ravel() if bias is not None else None
    tok = np.ascontiguousarray(token_ids, dtype=np.int32).ravel() if token_ids is not None else None
    tab = np.ascontiguousarray(hash_table, dtype=np.int32) if hash_table is not None else None
    idx_dtype = np.float32 if kind == 3 else np.int32
    idx = np.zeros((rows, k), idx_dtype) if indices is None else np.ascontiguousarray(indices, dtype=idx_dtype).copy()
    w = np.zeros((rows, k), np.float32) if weights is None else _f32(weights).copy()
    i32p = C.POINTER(C.c_int32)
    lib().fo_router_kernel_rows(
        kind, rows, columns, k, tab.shape[0] if tab is not None else 0, tab.shape[1] if tab is not None else 0,
        1 if b is not None else 0, route_scale, _pf(lg), _pf(b) if b is not None else None,
        tok.ctypes.data_as(i32p) if tok is not None else None, tab.ctypes.data_as(i32p) if tab is not None else None,
        idx.ctypes.data_as(C.c_void_p), _pf(w))
    return idx, w


# ---- expert slot table -----------------------------------------------------------

def _pi(a: np.ndarray):
    return a.ctypes.data_as(C.POINTER(C.c_int32))


def _pq(a: np.ndarray):
    return a.ctypes.data_as(C.POINTER(C.c_uint64))


class ExpertTableState:
    """The device arrays of the slot table as the reference kernel leaves them
    (portable/entrypoints.cu:1268-1300): ``table`` is u64 [6, slots] in the order gate weight,
    gate scale, up weight, up scale, down weight, down scale."""

    def __init__(self, expert_capacity: int, slot_capacity: int):
        self.table = np.zeros((6, slot_capacity), np.uint64)
        self.expert_to_slot = np.full(expert_capacity, -1, np.int32)
        self.expert_generations = np.zeros(expert_capacity, np.int32)
        self.slot_generations = np.zeros(slot_capacity, np.int32)

    def publish(self, kind: int, expert: int, slot: int, generation: int, pointers=(0,) * 6) -> None:
        values = np.asarray(pointers, np.uint64)
        lib().fo_expert_table_publish(kind, expert, slot, generation, _pq(values), _pq(self.table),
                                      self.table.shape[1], _pi(self.expert_to_slot), _pi(self.expert_generations),
                                      _pi(self.slot_generations))

    def resolve(self, expert_ids, miss_capacity: int, route_capacity: int | None = None):
        """INITIALIZE_RESOLVE + RESOLVE (entrypoints.cu:1301-1340).  Returns route slots, route
        generations, miss markers and the miss_control array."""
        ids = np.ascontiguousarray(expert_ids, dtype=np.int32)
        n = ids.size
        route_capacity = n if route_capacity is None else route_capacity
        control = np.zeros(2 + miss_capacity + route_capacity, np.int32)
        slots, gens, markers = (np.zeros(n, np.int32) for _ in range(3))
        lib().fo_expert_resolve_init(_pi(control), miss_capacity, route_capacity)
        lib().fo_expert_resolve(_pi(ids), n, self.expert_to_slot.size, self.slot_generations.size, miss_capacity,
                                _pi(self.expert_to_slot), _pi(self.expert_generations), _pi(self.slot_generations),
                                _pi(slots), _pi(gens), _pi(markers), _pi(control))
        return slots, gens, markers, control

    def gather_dispatch(self, route_slots, route_generations, router_weights, active_markers, active_value: int):
        """GATHER_DISPATCH (entrypoints.cu:1341-1379).  Returns pointers u64 [6, routes], route
        weights, the per-route index-or-minus-one array and dispatch_error."""
        rs = np.ascontiguousarray(route_slots, dtype=np.int32)
        rg = np.ascontiguousarray(route_generations, dtype=np.int32)
        rw = _f32(router_weights).ravel()
        am = np.ascontiguousarray(active_markers, dtype=np.int32)
        n = rs.size
        out = np.zeros((6, n), np.uint64)
        w = np.zeros(n, np.float32)
        ids = np.zeros(n, np.int32)
        err = lib().fo_expert_gather_dispatch(n, self.slot_generations.size, active_value, _pq(self.table),
                                              _pi(self.slot_generations), _pi(rs), _pi(rg), _pf(rw), _pi(am), _pq(out),
                                              _pf(w), _pi(ids))
        return out, w, ids, err


# ---- hyper-connection producer ---------------------------------------------------

def hc_split_sinkhorn(mixes, hc: int, sinkhorn_iters: int, eps: float, scale, base):
    """hyper_connection.rs:175-262.  mixes [tokens, (2+hc)*hc] -> pre, post [tokens, hc], comb [tokens, hc, hc]."""
    m = _f32(mixes).reshape(-1, (2 + hc) * hc)
    tokens = m.shape[0]
    pre, post = np.empty((tokens, hc), np.float32), np.empty((tokens, hc), np.float32)
    comb = np.empty((tokens, hc, hc), np.float32)
    sc, bs = _f32(scale).ravel(), _f32(base).ravel()
    if sc.size != 3 or bs.size != (2 + hc) * hc:
        raise OracleError("HC split scale/base mismatch")
    _check(lib().fo_hc_split_sinkhorn(_pf(m), tokens, hc, sinkhorn_iters, eps, _pf(sc), _pf(bs), _pf(pre), _pf(post),
                                      _pf(comb)), "hc_split_sinkhorn")
    return pre, post, comb


def rms_norm(x, weight, eps: float) -> np.ndarray:
    x, w = _f32(x).ravel(), _f32(weight).ravel()
    if x.size != w.size:
        raise OracleError("RMS length mismatch")
    out = np.empty_like(x)
    _check(lib().fo_rms_norm(_pf(x), _pf(w), x.size, eps, _pf(out)), "rms_norm")
    return out


def hc_producer(state, function, scale, base, layer_rms_weight, sinkhorn_iters: int, eps: float, norm_eps: float,
                layer_rms_eps: float, bf16_boundaries: bool = False) -> dict:
    """hc_pre -> rms_norm -> FP8-K128 pack for state [tokens, hc, hidden] (see fo_hc_producer)."""
    st = _f32(state)
    tokens, hc, hidden = st.shape
    mix = (2 + hc) * hc
    fn, sc, bs, rw = _f32(function).reshape(mix, hc * hidden), _f32(scale).ravel(), _f32(base).ravel(), \
        _f32(layer_rms_weight).ravel()
    if sc.size != 3 or bs.size != mix or rw.size != hidden:
        raise OracleError("HC producer parameter shapes")
    out = dict(raw_dots=np.empty((tokens, mix), np.float32), pre=np.empty((tokens, hc), np.float32),
               post=np.empty((tokens, hc), np.float32), comb=np.empty((tokens, hc, hc), np.float32),
               hidden=np.empty((tokens, hidden), np.float32), normalized=np.empty((tokens, hidden), np.float32),
               packed=np.empty((tokens, hidden), np.uint8), scales=np.empty((tokens, hidden // 128), np.uint8))
    rc = lib().fo_hc_producer(_pf(st), tokens, hc, hidden, sinkhorn_iters, eps, norm_eps, layer_rms_eps,
                              1 if bf16_boundaries else 0, _pf(fn), _pf(sc), _pf(bs), _pf(rw), _pf(out["raw_dots"]),
                              _pf(out["pre"]), _pf(out["post"]), _pf(out["comb"]), _pf(out["hidden"]),
                              _pf(out["normalized"]), _pb(out["packed"]), _pb(out["scales"]))
    _check(rc, "hc_producer")
    return out
