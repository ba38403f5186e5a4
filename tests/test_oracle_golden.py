"""Pins the CPU checker (oracle/) before anything is compared with it.

Three kinds of evidence, none of which re-types the oracle's own formula:
  1. the reference's own known-answer tests, transcribed as values in
     tests/golden/reference_known_answers.json;
  2. independent library routines (torch's float8_e4m3fn decoder, numpy
     float64 matmul, ldexp);
  3. closed forms / brute force on small grids (nearest-grid-point property,
     hand-evaluated tie cases, integer dot products).
"""
import json
import math
import os

import numpy as np
import pytest

from oracle import pyoracle as po

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")))


def bits(x: float) -> int:
    return int(np.float32(x).view(np.uint32))


# ---------------------------------------------------------------- decode tables

def test_fp4_nibble_table_matches_reference_vector():
    want = GOLD["fp4_e2m1_nibble_table"]["values"]
    got = [po.decode_fp4_e2m1_nibble(i) for i in range(16)]
    assert [bits(v) for v in got] == [bits(v) for v in want]  # -0.0 preserved bitwise


def test_fp4_packed_low_nibble_is_even_element():
    out = po.decode_fp4_e2m1_packed_low_first([0x21, 0x87])
    assert [bits(v) for v in out] == [bits(v) for v in (0.5, 1.0, 6.0, -0.0)]


def test_e8m0_reference_cases_and_ldexp_brute_force():
    for byte, want in GOLD["e8m0"]["cases"]:
        assert po.decode_e8m0_scale(byte) == want
    for byte in range(256):
        want = np.float32(math.ldexp(1.0, byte - 127)) if byte < 255 else np.float32(np.inf)
        assert bits(po.decode_e8m0_scale(byte)) == bits(want)
    # the GPU twin of the reference builds the same values from bits
    # (portable/entrypoints.cu:63-66): byte==0 ? 1<<22 : byte<<23
    for byte in range(256):
        twin = np.uint32((1 << 22) if byte == 0 else (byte << 23)).view(np.float32)
        assert bits(po.decode_e8m0_scale(byte)) == bits(twin)


def test_fp8_e4m3fn_reference_cases():
    for byte, want in GOLD["fp8_e4m3fn"]["cases"]:
        assert bits(po.decode_fp8_e4m3fn_byte(byte)) == bits(want)
    for byte in GOLD["fp8_e4m3fn"]["nan"] + [0xFF]:
        assert math.isnan(po.decode_fp8_e4m3fn_byte(byte))


def test_fp8_e4m3fn_all_256_codes_against_torch_decoder():
    torch = pytest.importorskip("torch")
    codes = torch.arange(256, dtype=torch.uint8)
    want = codes.view(torch.float8_e4m3fn).float().numpy()
    got = np.array([po.decode_fp8_e4m3fn_byte(i) for i in range(256)], np.float32)
    nan = np.isnan(want)
    assert list(np.nonzero(nan)[0]) == [0x7F, 0xFF]
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


# ---------------------------------------------------------------- dequant

def test_fp4_dequant_reference_cases():
    for case in GOLD["fp4_dequant_tiny"]["cases"]:
        w = np.zeros(case["n"] * case["k"] // 2, np.uint8)
        w[: len(case["weight_head"])] = case["weight_head"]
        out = po.dequantize_fp4(w, [case["scale"]], case["n"], case["k"], case["block"]).ravel()
        want = case["out_head"]
        assert [bits(v) for v in out[: len(want)]] == [bits(v) for v in want]
        assert not out[len(want) + 2:].any()


def test_fp8_dequant_two_dimensional_scales_reference_case():
    g = GOLD["fp8_dequant_2d"]
    out = po.dequantize_fp8(np.array(g["weight"], np.uint8), np.array(g["scales"], np.uint8),
                            g["n"], g["k"], g["block_m"], g["block_k"])
    assert out.ravel().tolist() == g["out"]


def test_dequant_rejects_the_shapes_the_reference_rejects():
    with pytest.raises(po.OracleError):
        po.dequantize_fp4(np.zeros(16, np.uint8), [127], 1, 32, 0)
    with pytest.raises(po.OracleError):
        po.dequantize_fp4(np.zeros(15, np.uint8), [127], 1, 32, 32)
    with pytest.raises(po.OracleError):
        po.dequantize_fp8(np.zeros(6, np.uint8), np.zeros(3, np.uint8), 2, 3, 1, 2)


def test_fp8_dequant_exhaustive_byte_times_scale_is_exact_product():
    # 256 codes x 256 E8M0 bytes against float64 arithmetic rounded once to f32
    w = np.tile(np.arange(256, dtype=np.uint8), (256, 1))          # row r: all codes
    s = np.arange(256, dtype=np.uint8).reshape(256, 1)             # row r: scale byte r
    with np.errstate(all="ignore"):
        out = po.dequantize_fp8(w, s, 256, 256, 1, 256)
        dec = np.array([po.decode_fp8_e4m3fn_byte(i) for i in range(256)], np.float64)
        scale = np.array([po.decode_e8m0_scale(i) for i in range(256)], np.float64)
        want = (scale[:, None] * dec[None, :]).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(out), nan)
    assert np.array_equal(out[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_fp8_dequant_f32_scales_is_single_rounded_product():
    rng = np.random.default_rng(3)
    w = rng.integers(0, 256, (8, 256), dtype=np.uint8)
    w[(w & 0x7F) == 0x7F] = 0x38
    s = rng.uniform(1e-5, 3e-3, (2, 2)).astype(np.float32)
    out = po.dequantize_fp8(w, s, 8, 256, 4, 128)
    dec = np.array([po.decode_fp8_e4m3fn_byte(i) for i in range(256)], np.float64)
    want = (dec[w] * np.repeat(np.repeat(s.astype(np.float64), 4, 0), 128, 1)).astype(np.float32)
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))


# ---------------------------------------------------------------- activation quantizers

def test_fp8_act_quant_reference_case():
    g = GOLD["fp8_act_quant"]
    v = np.zeros(128, np.float32)
    v[:4] = g["in_head"]
    out = po.simulate_fp8_act_quant(v, g["row_width"], g["block"])
    assert out[:3].tolist() == g["out_head_exact"]
    assert abs(out[3] - g["out3_approx"]) < g["tol"]
    assert not out[4:].any()


def test_fp4_act_quant_reference_case():
    g = GOLD["fp4_act_quant"]
    v = np.zeros(32, np.float32)
    v[:4] = g["in_head"]
    out = po.simulate_fp4_act_quant(v, g["row_width"], g["block"])
    assert out[:4].tolist() == g["out_head"]


def test_fp8_quantizer_hand_evaluated_ties_round_half_away_and_keep_first_minimum():
    for value, want in GOLD["fp8_rounding_worked_examples"]["cases"]:
        assert po.quantize_fp8_e4m3fn_to_f32(value) == want
        assert po.quantize_fp8_e4m3fn_to_f32(-value) == -want


def _e4m3_grid() -> np.ndarray:
    torch = pytest.importorskip("torch")
    vals = torch.arange(0, 0x7F, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    return np.unique(vals.astype(np.float64))


def test_fp8_quantizer_is_a_nearest_grid_point_on_the_whole_bf16_grid():
    # brute force: every positive BF16 value in [2^-12, 512]; result must be on the
    # E4M3 grid and no other grid point may be strictly closer.
    grid = _e4m3_grid()
    b = np.arange(0x3980, 0x4400 + 1, dtype=np.uint32) << 16
    values = b.view(np.float32)
    got = np.array([po.quantize_fp8_e4m3fn_to_f32(float(v)) for v in values], np.float64)
    clipped = np.minimum(values.astype(np.float64), 448.0)
    best = np.abs(grid[None, :] - clipped[:, None]).min(axis=1)
    assert np.isin(got, grid).all()
    assert np.array_equal(np.abs(got - clipped), best)
    # non-tie points agree with hardware-style RNE (torch's converter)
    torch = pytest.importorskip("torch")
    rne = torch.from_numpy(np.minimum(values, np.float32(448.0))).to(torch.float8_e4m3fn).float().numpy()
    ties = np.abs(got - clipped) != np.abs(rne - clipped)
    assert not ties.any()
    differ = got != rne
    # the two roundings differ only where two grid points are equally near
    second = np.sort(np.abs(grid[None, :] - clipped[:, None]), axis=1)[:, 1]
    assert np.array_equal(second[differ], best[differ])
    assert differ.any()


def test_fp8_quantizer_passes_zero_and_non_finite_through():
    assert bits(po.quantize_fp8_e4m3fn_to_f32(-0.0)) == bits(-0.0)
    assert math.isnan(po.quantize_fp8_e4m3fn_to_f32(float("nan")))
    assert po.quantize_fp8_e4m3fn_to_f32(float("inf")) == float("inf")
    assert po.quantize_fp8_e4m3fn_to_f32(1000.0) == 448.0


def test_fp4_quantizer_ties_go_to_the_lower_magnitude():
    # midpoints of the magnitude table
    for mid, want in [(0.25, 0.0), (0.75, 0.5), (1.25, 1.0), (1.75, 1.5), (2.5, 2.0), (3.5, 3.0), (5.0, 4.0)]:
        assert po.quantize_fp4_e2m1_to_f32(mid) == want
        assert po.quantize_fp4_e2m1_to_f32(-mid) == -want
    assert po.quantize_fp4_e2m1_to_f32(100.0) == 6.0


def test_rounded_power_of_two_scale_on_bf16_grid_matches_integer_exponent_form():
    # independent form: smallest power of two >= amax/qmax, from frexp in float64
    b = (np.arange(0x3400, 0x4700, 3, dtype=np.uint32) << 16).view(np.float32)
    for qmax in (448.0, 6.0):
        for amax in b:
            m, e = math.frexp(float(amax) / qmax)          # m in [0.5, 1)
            want = math.ldexp(1.0, e - 1 if m == 0.5 else e)
            assert po.rounded_power_of_two_scale(float(amax), qmax) == want


def test_fp8_pack_bytes_agree_with_simulated_values_and_reference_gpu_grid():
    g = GOLD["fp8_pack_grid"]
    rows, k, block = g["rows"], g["k"], g["block"]
    col = np.arange(k)
    base = ((col % 31).astype(np.float32) - np.float32(15.0)) * np.where(col < block, np.float32(0.25),
                                                                         np.float32(0.00075))
    values = np.stack([(base * np.float32(r + 1)).astype(np.float32) for r in range(rows)])
    packed, scales = po.pack_fp8_act(values, k, block)
    sim = po.simulate_fp8_act_quant(values, k, block)
    dec = np.array([po.decode_fp8_e4m3fn_byte(i) for i in range(256)], np.float32)
    sc = np.array([po.decode_e8m0_scale(int(s)) for s in scales.ravel()], np.float32).reshape(scales.shape)
    assert np.array_equal((dec[packed] * np.repeat(sc, block, 1)).view(np.uint32), sim.view(np.uint32))
    # scale bytes as the reference's GPU-test oracle computes them (fp8_core.rs:85-90)
    for r in range(rows):
        for blk in range(k // block):
            amax = max(1e-4, float(np.abs(values[r, blk * block:(blk + 1) * block]).max()))
            want = min(255, max(0, math.ceil(math.log2(np.float32(amax) / np.float32(448.0))) + 127))
            assert scales[r, blk] == want


def test_fp4_pack_reference_gpu_grid():
    # fp4_core.rs:169-244: expected bytes come from an independent nearest-of-8 scan
    g = GOLD["fp4_pack_grid"]
    rows, cols, block = g["rows"], g["columns"], g["block"]
    idx = np.arange(rows * cols)
    values = (((idx % 17) - 8).astype(np.float32) * np.float32(0.375)
              + np.where(idx % 11 == 0, np.float32(4.25), np.float32(0.0))).astype(np.float32)
    packed, scales = po.pack_fp4_act(values.reshape(rows, cols), cols, block)
    mags = np.array([0, .5, 1, 1.5, 2, 3, 4, 6], np.float32)
    for r in range(rows):
        for blk in range(cols // block):
            seg = values[r * cols + blk * block: r * cols + (blk + 1) * block]
            amax = np.abs(seg).max()
            byte = min(255, max(0, math.ceil(math.log2(amax / np.float32(6.0))) + 127))
            assert scales[r, blk] == byte
            scale = np.float32(math.ldexp(1.0, byte - 127))
            for j in range(0, block, 2):
                nibs = []
                for v in (seg[j], seg[j + 1]):
                    q = np.float32(v) / scale
                    if q == 0:
                        nibs.append(0)
                        continue
                    m = min(abs(float(q)), 6.0)
                    best = int(np.argmin(np.abs(mags - np.float32(m))))   # argmin keeps the first minimum
                    nibs.append((8 if q < 0 else 0) | best)
                assert packed[r, blk * block // 2 + j // 2] == (nibs[0] | (nibs[1] << 4))


# ---------------------------------------------------------------- bf16

def test_bf16_rne_reference_vectors():
    for src, want in GOLD["bf16_rne"]["cases"]:
        v = np.uint32(int(src, 16)).view(np.float32)
        assert bits(po.round_to_bf16(float(v))) == int(want, 16)
    nan = np.uint32(int(GOLD["bf16_rne"]["nan_in"], 16)).view(np.float32)
    r = np.array([nan], np.float32)
    out = po.round_to_bf16_array(r)
    assert np.isnan(out[0]) and (out.view(np.uint32)[0] & 0x00400000)


def test_bf16_rne_matches_torch_on_random_values():
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(0)
    v = rng.standard_normal(100000).astype(np.float32) * np.float32(37.0)
    want = torch.from_numpy(v).to(torch.bfloat16).float().numpy()
    assert np.array_equal(po.round_to_bf16_array(v).view(np.uint32), want.view(np.uint32))
    assert bits(po.round_to_bf16(float(v[0]))) == bits(want[0])


# ---------------------------------------------------------------- matvec

def test_fp8_linear_matvec_reference_case():
    g = GOLD["fp8_matvec"]
    y = po.linear_fp8(np.array(g["weight"], np.uint8), np.array(g["scales"], np.uint8), g["n"], g["k"],
                      g["x"], g["inferred_block"][0], g["inferred_block"][1])
    assert y.ravel().tolist() == g["y"]


def test_fp4_linear_matvec_reference_case():
    g = GOLD["fp4_matvec"]
    w = np.zeros(16, np.uint8)
    w[0] = g["weight_head"][0]
    x = np.zeros(32, np.float32)
    x[:2] = g["x_head"]
    assert po.linear_fp4(w, [g["scale"]], g["n"], g["k"], x, g["block"]).ravel().tolist() == g["y"]
    assert po.linear_fp4(w, [g["scale"]], g["n"], g["k"], x, g["block"], materialized=True).ravel().tolist() == g["y"]


def test_fused_matvec_equals_materialized_reference_order_bitwise():
    rng = np.random.default_rng(5)
    n, k = 24, 256
    w4 = rng.integers(0, 256, (n, k // 2), dtype=np.uint8)
    s4 = rng.integers(118, 126, (n, k // 32), dtype=np.uint8)
    x = po.round_to_bf16_array(rng.standard_normal((3, k)).astype(np.float32))
    a = po.linear_fp4(w4, s4, n, k, x)
    b = po.linear_fp4(w4, s4, n, k, x, materialized=True)
    c = po.linear_fp4(w4, s4, n, k, x, threads=4)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    assert np.array_equal(a.view(np.uint32), c.view(np.uint32))
    # and the materialized path is literally dequant + sequential matvec
    deq = po.dequantize_fp4(w4, s4, n, k)
    assert np.array_equal(po.matvec_row_major(deq, x[1]).view(np.uint32), a[1].view(np.uint32))
    w8 = rng.integers(0, 0x7F, (n, k), dtype=np.uint8)
    for s8 in (rng.integers(118, 126, (2, 2), dtype=np.uint8), rng.uniform(1e-4, 1e-3, (2, 2)).astype(np.float32)):
        a = po.linear_fp8(w8, s8, n, k, x, 16, 128)
        b = po.linear_fp8(w8, s8, n, k, x, 16, 128, materialized=True)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_matvec_closed_form_integer_dot_products_and_float64_bound():
    rng = np.random.default_rng(9)
    n, k = 16, 512
    # nibble 2 (+1.0) / 10 (-1.0), unit scales, small-integer x -> exact integers
    signs = rng.integers(0, 2, (n, k))
    nib = np.where(signs == 1, 10, 2).astype(np.uint8)
    w = (nib[:, 0::2] | (nib[:, 1::2] << 4)).astype(np.uint8)
    s = np.full((n, k // 32), 127, np.uint8)
    x = rng.integers(-8, 9, k).astype(np.float32)
    want = (np.where(signs == 1, -1, 1) * x[None, :]).sum(1)
    assert po.linear_fp4(w, s, n, k, x).ravel().tolist() == want.tolist()
    # E8M0 +1 on one block doubles exactly that block's contribution
    s2 = s.copy()
    s2[:, 3] = 128
    blk = (np.where(signs == 1, -1, 1) * x[None, :])[:, 96:128].sum(1)
    assert po.linear_fp4(w, s2, n, k, x).ravel().tolist() == (want + blk).tolist()
    # random data: |f32 sequential - float64| <= K * 2^-24 * sum|w x|
    w = rng.integers(0, 256, (n, k // 2), dtype=np.uint8)
    s = rng.integers(120, 130, (n, k // 32), dtype=np.uint8)
    x = rng.standard_normal(k).astype(np.float32)
    deq = po.dequantize_fp4(w, s, n, k).astype(np.float64)
    y = po.linear_fp4(w, s, n, k, x).ravel().astype(np.float64)
    assert (np.abs(y - deq @ x) <= k * 2.0 ** -24 * (np.abs(deq) @ np.abs(x))).all()


def test_activation_quant_is_applied_before_the_matvec():
    # weight.rs:567-595: selector weight picks x[0]; 1.1 is not on the FP8 grid
    x = np.zeros(128, np.float32)
    x[0] = 1.1
    q = po.simulate_fp8_act_quant(x, 128, 128)
    assert q[0] != x[0]
    w = np.zeros((1, 128), np.uint8)
    w[0, 0] = 0x38
    y = po.linear_fp8(w, np.array([127], np.uint8), 1, 128, x, 128, 128, act_quant_block=128)
    assert y[0, 0] == q[0]


# ---------------------------------------------------------------- expert / routed / ffn / combine

def _tiny_fp4(nonzero):
    b = np.zeros(32 * 16, np.uint8)
    for row, col, nib in nonzero:
        off = row * 16 + col // 2
        b[off] = (b[off] & 0xF0) | nib if col % 2 == 0 else (b[off] & 0x0F) | (nib << 4)
    return b


def test_expert_swiglu_reference_cases():
    ones = np.full(32, 127, np.uint8)
    for case in GOLD["expert_swiglu"]["cases"]:
        x = np.zeros(32, np.float32)
        x[:2] = case["x_head"]
        out = po.expert_execute_fp4(_tiny_fp4(case["gate"]), ones, _tiny_fp4(case["up"]), ones,
                                    _tiny_fp4(case["down"]), ones, 32, 32, x, case["route_weight"],
                                    case["limit"])
        g, u = np.float32(case["expected_gate"]), np.float32(case["expected_up"])
        want = np.float32(g / (np.float32(1.0) + np.exp(-g, dtype=np.float32))) * u * np.float32(case["route_weight"])
        assert abs(out[0] - want) < case["tol"]
        assert (np.abs(out[1:]) < 1e-6).all()


def test_expert_rejects_wrong_activation_size():
    ones = np.full(32, 127, np.uint8)
    z = _tiny_fp4([])
    with pytest.raises(po.OracleError):
        po.expert_execute_fp4(z, ones, z, ones, z, ones, 32, 32, np.zeros(31, np.float32), 1.0)


def test_expert_with_activation_quantization_quantizes_input_and_hidden():
    rng = np.random.default_rng(11)
    hidden, inter = 256, 128
    mk = lambda n, k: (rng.integers(0, 256, (n, k // 2), dtype=np.uint8), rng.integers(121, 125, (n, k // 32), dtype=np.uint8))
    (gw, gs), (uw, us), (dw, ds) = mk(inter, hidden), mk(inter, hidden), mk(hidden, inter)
    x = rng.standard_normal(hidden).astype(np.float32)
    out, h = po.expert_execute_fp4(gw, gs, uw, us, dw, ds, hidden, inter, x, 0.3, 0.0, act_quant_block=128,
                                   return_hidden=True)
    xq = po.simulate_fp8_act_quant(x, hidden, 128)
    g = po.linear_fp4(gw, gs, inter, hidden, xq).ravel()
    u = po.linear_fp4(uw, us, inter, hidden, xq).ravel()
    hh = np.array([np.float32(np.float32(po.silu(float(a)) * np.float32(b)) * np.float32(0.3)) for a, b in zip(g, u)], np.float32)
    hq = po.simulate_fp8_act_quant(hh, inter, 128)
    assert np.array_equal(h.view(np.uint32), hq.view(np.uint32))
    assert np.array_equal(out.view(np.uint32), po.linear_fp4(dw, ds, hidden, inter, hq).ravel().view(np.uint32))


def test_routed_accumulate_is_route_order_sum_plus_shared():
    rng = np.random.default_rng(2)
    r = rng.standard_normal((8, 64)).astype(np.float32) * np.float32(1e3)
    sh = rng.standard_normal(64).astype(np.float32)
    want = r[0].copy()
    for i in range(1, 8):
        want = want + r[i]
    assert np.array_equal(po.accumulate_routes(r).view(np.uint32), want.view(np.uint32))
    assert np.array_equal(po.accumulate_routes(r, sh).view(np.uint32), (want + sh).view(np.uint32))
    assert not po.accumulate_routes(np.zeros((0, 64), np.float32)).any()


def test_swiglu_ffn_f32_reference_cases():
    c = GOLD["swiglu_ffn_f32"]["case1"]
    out = po.swiglu_ffn_f32(c["gate"], c["up"], c["down"], c["x"], c["output_scale"])
    g, u = np.float32(c["gate0"]), np.float32(c["up0"])
    want = g / (np.float32(1) + np.exp(-g, dtype=np.float32)) * u * np.float32(0.5)
    assert abs(out[0] - want) < c["tol"] and out[1] == 0.0 and out[2] == 0.0
    c = GOLD["swiglu_ffn_f32"]["case2"]
    out = po.swiglu_ffn_f32(c["gate"], c["up"], c["down"], c["x"], 1.0, c["limit"])
    want = np.float32(10.0) / (np.float32(1) + np.exp(np.float32(-10.0))) * np.float32(10.0)
    assert abs(out[0] - want) < c["tol"]


def test_ranked_reducer_reference_case_with_cancellation():
    g = GOLD["ranked_reducer"]
    e, cols, hidden, k = g["experts"], g["batch_cols"], g["hidden"], g["routes_per_col"]
    slots = g["route_slots"]
    route_output = np.zeros((cols * k, hidden), np.float32)
    row = np.arange(hidden)
    for col in range(cols):
        for rank in range(k):
            ex = slots[col * k + rank]
            route_output[col * k + rank] = (16777216.0 if ex == 0 else -16777216.0 if ex == 1 else
                                            1.0 + (row % 13) * 0.0625 + col * 0.125)
    base = (0.25 + (np.arange(cols * hidden) % 11) * 0.03125).astype(np.float32).reshape(cols, hidden)
    want = base.copy()
    for rank in range(k):
        want = (want + route_output.reshape(cols, k, hidden)[:, rank]).astype(np.float32)
    got = po.reduce_routes_ranked(route_output, cols, k, hidden, prefix=base)
    assert np.array_equal(got.view(np.uint32), po.round_to_bf16_array(want).view(np.uint32))
    # column 0 folds +2^24, -2^24, then the small value: the prefix is absorbed by 2^24
    assert got[0, 0] == po.round_to_bf16(float(np.float32(1.0)))
