"""Host logic: the closed-form quantizers that the device kernels use
(ferrule_amd/csrc/quant_math.h) against the CPU checker's literal restatement of
the reference's candidate search, over dense input sets.  Runs without a GPU."""
import ctypes as C
import os
import subprocess
import tempfile

import numpy as np
import pytest

from oracle import pyoracle as po

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def shim():
    out = os.path.join(tempfile.mkdtemp(prefix="ferrule_shim_"), "libshim.so")
    subprocess.check_call(["g++", "-O2", "-ffp-contract=off", "-shared", "-fPIC", "-o", out,
                           os.path.join(ROOT, "tests", "quant_math_shim.cpp")])
    return C.CDLL(out)


def _ptr(a, t):
    return a.ctypes.data_as(C.POINTER(t))


def _oracle_fp8_bytes(x: np.ndarray, scale: float) -> np.ndarray:
    """Bytes the checker produces for x/scale (block amax forced by a sentinel so the scale is `scale`)."""
    lib = po.lib()
    out = np.empty(x.size, np.uint8)
    dec = {}
    for i, v in enumerate(x):
        q = np.float32(v) / np.float32(scale)
        q = np.float32(min(max(q, np.float32(-448.0)), np.float32(448.0))) if q == q else q
        r = lib.fo_quantize_fp8_e4m3fn_to_f32(float(q))
        key = np.float32(r).view(np.uint32).item()
        if key not in dec:
            dec[key] = _byte_of(np.float32(r))
        out[i] = dec[key]
    return out


def _byte_of(r: np.float32) -> int:
    bits = int(r.view(np.uint32))
    sign = 0x80 if bits >> 31 else 0
    m = abs(float(r))
    if m == 0:
        return sign
    if m != m:
        return sign | 0x7F
    if m < 2.0 ** -6:
        return sign | int(m * 512)
    return sign | ((((bits >> 23) & 0xFF) - 120) << 3) | ((bits >> 20) & 7)


def test_fp8_closed_form_equals_candidate_search_on_dense_grid(shim):
    # every f32 whose low 11 mantissa bits are zero in [2^-12, 2^10): 4096 mantissas x 22 binades,
    # which contains every tie point of the E4M3 grid and of the subnormal grid, plus neighbours
    exps = np.arange(127 - 12, 127 + 10, dtype=np.uint32)
    mant = np.arange(0, 1 << 23, 1 << 11, dtype=np.uint32)
    bits = (exps[:, None] << 23 | mant[None, :]).ravel()
    x = np.concatenate([bits, bits + 1, bits - 1]).astype(np.uint32).view(np.float32)
    x = np.concatenate([x, -x, np.array([0.0, -0.0, np.inf, -np.inf, np.nan], np.float32)])
    got = np.empty(x.size, np.uint8)
    for mode in (0,):
        shim.shim_fp8_bytes(_ptr(x, C.c_float), C.c_size_t(x.size), C.c_float(1.0), C.c_uint32(mode),
                            _ptr(got, C.c_uint8))
        want = _oracle_fp8_bytes(x, 1.0)
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, [(float(x[i]), hex(got[i]), hex(want[i])) for i in bad[:10]]


def test_fp8_closed_form_with_power_of_two_scales(shim):
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(20000) * np.exp(rng.uniform(-8, 8, 20000))).astype(np.float32)
    for scale in (2.0 ** -9, 0.5, 4.0, 2.0 ** 7):
        got = np.empty(x.size, np.uint8)
        shim.shim_fp8_bytes(_ptr(x, C.c_float), C.c_size_t(x.size), C.c_float(scale), C.c_uint32(0),
                            _ptr(got, C.c_uint8))
        assert np.array_equal(got, _oracle_fp8_bytes(x, scale))


def test_fp8_half_even_mode_is_rne_except_where_the_portable_kernel_is_not(shim):
    torch = pytest.importorskip("torch")
    b = np.arange(0x3000, 0x4400, dtype=np.uint32) << 16
    x = b.view(np.float32)
    x = x[x <= 448.0]
    got = np.empty(x.size, np.uint8)
    shim.shim_fp8_bytes(_ptr(x, C.c_float), C.c_size_t(x.size), C.c_float(1.0), C.c_uint32(1), _ptr(got, C.c_uint8))
    rne = torch.from_numpy(x.copy()).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    differ = np.nonzero(got != rne)[0]
    # rintf(7.5) = 8 is clamped to 7 and the 2^-6 candidate does not win the tie
    assert all(float(x[i]) == 7.5 / 512 for i in differ)


def test_fp4_closed_form_equals_checker(shim):
    lib = po.lib()
    rng = np.random.default_rng(2)
    x = np.concatenate([
        np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 0.0, -0.0, 6.0, 7.0, 1e9, -1e9], np.float32),
        (rng.standard_normal(20000) * 3).astype(np.float32),
    ])
    x = np.concatenate([x, -x, np.nextafter(x, np.float32(np.inf)), np.nextafter(x, np.float32(-np.inf))])
    got = np.empty(x.size, np.uint8)
    shim.shim_fp4_nibbles(_ptr(x, C.c_float), C.c_size_t(x.size), C.c_float(1.0), 1, _ptr(got, C.c_uint8))
    mags = {0.0: 0, 0.5: 1, 1.0: 2, 1.5: 3, 2.0: 4, 3.0: 5, 4.0: 6, 6.0: 7}
    for v, g in zip(x, got):
        r = lib.fo_quantize_fp4_e2m1_to_f32(float(np.clip(v, -6.0, 6.0)))
        want = (8 if np.signbit(np.float32(r)) else 0) | mags[abs(r)]
        assert g == want, (float(v), g, want)


def test_scale_byte_matches_libm_form_including_just_above_powers_of_two(shim):
    lib = po.lib()
    # amax values whose quotient lands 0..300 ulps above a power of two, all exponents in use
    cases = []
    for qmax in (448.0, 6.0):
        for e in range(-30, 20):
            base = np.float32(2.0 ** e)
            for ulps in list(range(0, 40)) + [100, 255, 256, 257, 300, 1 << 20]:
                q = (base.view(np.uint32) + np.uint32(ulps)).view(np.float32)
                amax = np.float32(q * np.float32(qmax))
                cases.append((amax, qmax))
    rng = np.random.default_rng(3)
    for v in np.exp(rng.uniform(-12, 12, 4000)).astype(np.float32):
        cases.append((v, 448.0))
        cases.append((v, 6.0))
    for qmax in (448.0, 6.0):
        amax = np.array([c[0] for c in cases if c[1] == qmax], np.float32)
        got = np.empty(amax.size, np.uint8)
        shim.shim_scale_bytes(_ptr(amax, C.c_float), C.c_size_t(amax.size), C.c_float(qmax), _ptr(got, C.c_uint8))
        for a, g in zip(amax, got):
            scale = np.float32(lib.fo_rounded_power_of_two_scale(float(a), qmax))
            want = (int(scale.view(np.uint32)) >> 23) & 0xFF
            assert g == want, (float(a), qmax, g, want)


def test_fp8_branch_free_form_equals_the_branching_form(shim):
    """fp8_e4m3_quantize_byte_pow2 (used by the GEMM epilogues) against fp8_e4m3_quantize_byte:
    every f32 with zero low 11 mantissa bits over 40 binades (all tie points of both grids),
    their neighbours one ulp up and down, both signs, specials; both rounding modes; scales
    2^-20 .. 2^20."""
    exps = np.arange(127 - 24, 127 + 16, dtype=np.uint32)
    mant = np.arange(0, 1 << 23, 1 << 11, dtype=np.uint32)
    bits = (exps[:, None] << 23 | mant[None, :]).ravel()
    x = np.concatenate([bits, bits + 1, bits - 1]).astype(np.uint32).view(np.float32)
    x = np.concatenate([x, -x, np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 3.0e38, -3.0e38, 1e-45], np.float32)])
    rng = np.random.default_rng(7)
    x = np.concatenate([x, (rng.standard_normal(200000) * np.exp(rng.uniform(-12, 12, 200000))).astype(np.float32)])
    want, got = np.empty(x.size, np.uint8), np.empty(x.size, np.uint8)
    for mode in (0, 1):
        for byte in (127 - 20, 127 - 3, 127, 127 + 1, 127 + 9, 127 + 20):
            scale = 2.0 ** (byte - 127)
            shim.shim_fp8_bytes(_ptr(x, C.c_float), C.c_size_t(x.size), C.c_float(scale), C.c_uint32(mode),
                                _ptr(want, C.c_uint8))
            shim.shim_fp8_bytes_pow2(_ptr(x, C.c_float), C.c_size_t(x.size), C.c_uint32(byte), C.c_uint32(mode),
                                     _ptr(got, C.c_uint8))
            bad = np.nonzero(got != want)[0]
            assert bad.size == 0, (mode, byte, [(float(x[i]), hex(got[i]), hex(want[i])) for i in bad[:10]])
