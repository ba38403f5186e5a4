"""The parity rule and the CPU-side references with their forward-error bounds.

TEST INFRASTRUCTURE ONLY, like everything under ``oracle/``: used by ``tests/``, the smoke
check and ``bench.py``'s parity / CPU-baseline legs, never by the provider.

The rule (decided once for every BF16 output): pass = at most 2 BF16 ulp from
``bf16_rne(oracle_f32)``, OR inside the forward-error bound of the arithmetic the device
really performs, evaluated in float64.  The second clause exists for outputs that cancel
to near zero; the number of elements it decides is counted, limited, and the worst ulp
distance among them is reported.
"""
from __future__ import annotations

import numpy as np

from . import pyoracle as po

# One v_mfma_scale_f32_16x16x128_f8f6f4 aligns its 128 products to the largest and keeps about
# 21 bits below it: measured on gfx950, its result is within 2^-14.6 of the sum of |products|
# of that instruction (the error averages out over K blocks: 2^-17.3 at K = 2048).
MFMA_BLOCK_EPS = 2.0 ** -14.6
# The decode layer splits activations into MX-FP8 terms by truncation (4 significant bits per
# term, every term rescaled to the remainder's block maximum, each scale at most 1/16 of the
# one before):
#   BF16 input, 2 terms: exact for every element that is normal in its first term; what is
#     left of a smaller one is below 2^-9 of the second scale <= 2^-20 of the 32-block maximum;
#   f32 hidden, 4 terms: the remainder of every element is below 16 x the fourth scale
#     <= 2^-15 of the 32-block maximum.
X_SPLIT_TRUNCATION = 2.0 ** -20
H_SPLIT_TRUNCATION = 2.0 ** -15


def ordered(bits16: np.ndarray) -> np.ndarray:
    """BF16 bit patterns -> integers ordered like the values they encode."""
    b = bits16.astype(np.int32)
    return np.where(b & 0x8000, -(b & 0x7FFF), b)


def compare_bf16_bounded(gpu_bits: np.ndarray, oracle_f32: np.ndarray, bound_f64: np.ndarray | None,
                         max_ulp: int = 2, gpu_f32: np.ndarray | None = None,
                         max_decided_fraction: float | None = None):
    """The parity rule with an explicit bound array (same shape as the outputs) on
    |y_gpu - y_oracle| before the final rounding; half a BF16 ulp of the device value is added
    when only its BF16 output is available.  Returns (worst ulp among the elements judged by
    ulp, number decided by the bound, worst ulp among those)."""
    want_bits = po.bf16_bits_array(oracle_f32)
    dist = np.abs(ordered(gpu_bits.astype(np.uint16)) - ordered(want_bits))
    bad = dist > max_ulp
    decided, worst_decided = 0, 0
    if bad.any():
        assert bound_f64 is not None, f"{int(bad.sum())} elements off by more than {max_ulp} ulp (max {int(dist.max())})"
        got = (gpu_bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64) if gpu_f32 is None \
            else gpu_f32.astype(np.float64)
        err = np.abs(got - oracle_f32.astype(np.float64))
        bound = np.asarray(bound_f64, np.float64)
        if gpu_f32 is None:
            bound = bound + np.abs(got) * 2.0 ** -8
        still = bad & ~(err <= bound)        # NaN never passes
        assert not still.any(), f"{int(still.sum())} elements fail both the {max_ulp}-ulp rule and the " \
            f"forward-error bound (worst ulp {int(dist[still].max())})"
        decided, worst_decided = int(bad.sum()), int(dist[bad].max())
        if max_decided_fraction is not None:
            assert decided <= max_decided_fraction * dist.size, \
                f"{decided} of {dist.size} elements needed the error bound (limit {max_decided_fraction:.3%}), " \
                f"worst of them {worst_decided} ulp"
    return (int(dist[~bad].max()) if (~bad).any() else 0), decided, worst_decided


def compare_bf16(gpu_bits: np.ndarray, oracle_f32: np.ndarray, abs_products_f64: np.ndarray | None = None,
                 k: int = 0, max_ulp: int = 2, gpu_f32: np.ndarray | None = None):
    """The rule for a single dot product of length k: bound = k * 2^-24 * sum|w x| (an fp32 sum in
    any order).  Returns (worst ulp among elements judged by ulp, number decided by the bound)."""
    bound = None if abs_products_f64 is None else k * 2.0 ** -24 * np.asarray(abs_products_f64, np.float64)
    worst, decided, _ = compare_bf16_bounded(gpu_bits, oracle_f32, bound, max_ulp, gpu_f32)
    return worst, decided


def _block_max(values: np.ndarray, block: int = 32) -> np.ndarray:
    """max |v| of every `block` consecutive elements, repeated to the input's length."""
    v = np.abs(np.asarray(values, np.float64)).reshape(-1, block)
    return np.repeat(v.max(1), block)


def expert_route_reference(gate, up, down, hidden: int, inter: int, x_row: np.ndarray, route_weight: float,
                           limit: float = 0.0, threads: int = 1, mx_split: bool = True):
    """One route of the decode layer on the CPU: (y, bound) with y = CpuReferenceExpertExecutor's
    output (executor.rs:82-124, no activation quantisation) and bound[n] >= |y_device[n] - y[n]|
    for a device that computes the same chain with fp32 accumulation in any order on the scaled
    MFMA, from MX-split activations when `mx_split`.  gate/up/down = (weight bytes, scale bytes).

    Derivation, every term evaluated in float64:
      dg, du : error of the gate / up dot products = (H 2^-24 + mfma) sum|w x| + sum|w| tx,
               tx = truncation of x by its 2-term split;
      dh     : h = silu(g) u w with |silu'| <= 1.1 and |silu(g)| <= |g| (clamping is 1-Lipschitz):
               w (1.1 |u| dg + |g| du + 1.1 dg du) + 2^-21 |h| (device expf / reciprocal);
      bound  : sum|w2| ((I 2^-24 + mfma) (|h| + dh) + th + dh), th = truncation of the 4-term split.
    """
    (gw, gs), (uw, us), (dw, ds) = gate, up, down
    x_row = np.asarray(x_row, np.float32)
    y, h = po.expert_execute_fp4(gw, gs, uw, us, dw, ds, hidden, inter, x_row, float(route_weight), limit,
                                 threads=threads, return_hidden=True)
    g = po.linear_fp4(gw, gs, inter, hidden, x_row, threads=threads)[0].astype(np.float64)
    u = po.linear_fp4(uw, us, inter, hidden, x_row, threads=threads)[0].astype(np.float64)
    if limit > 0:
        g, u = np.minimum(g, limit), np.clip(u, -limit, limit)
    absx = np.abs(x_row.astype(np.float64))
    eps_in = hidden * 2.0 ** -24 + MFMA_BLOCK_EPS
    vx = eps_in * absx + (X_SPLIT_TRUNCATION * _block_max(absx) if mx_split else 0.0)
    dg = po.abs_linear_fp4(gw, gs, inter, hidden, vx, threads=threads)
    du = po.abs_linear_fp4(uw, us, inter, hidden, vx, threads=threads)
    absh = np.abs(h.astype(np.float64))
    dh = abs(float(route_weight)) * (1.1 * np.abs(u) * dg + np.abs(g) * du + 1.1 * dg * du) + absh * 2.0 ** -21
    eps_mid = inter * 2.0 ** -24 + MFMA_BLOCK_EPS
    vh = eps_mid * (absh + dh) + dh + (H_SPLIT_TRUNCATION * _block_max(absh + dh) if mx_split else 0.0)
    bound = po.abs_linear_fp4(dw, ds, hidden, inter, vh, threads=threads)
    return y, bound


def swiglu_ffn_reference(fmt, gate, up, down, input_size: int, inter: int, output_size: int, x_row: np.ndarray,
                         output_scale: float = 1.0, limit: float = 0.0, threads: int = 1):
    """Dense SwiGLU FFN over quantized linears on the CPU, SwiGluFfn::reference_execute
    (ffn.rs:24-48): (y, bound, hidden) for one activation row.  fmt = "fp4" (MXFP4, E8M0 per 32 k)
    or ("fp8", block_m, block_k) with E8M0-byte or f32 scales; gate/up/down = (weight bytes, scales).
    bound[n] >= |y_device[n] - y[n]| for a device that forms every product exactly and accumulates in
    fp32 in any order (BF16 MFMA; the f32 hidden row enters the down projection as an exact sum of
    three BF16 rows whose three results are added at the end), derived as in expert_route_reference
    without the split and MFMA-alignment terms; the device's silu (hardware exp2 and reciprocal) enters
    with a relative error of (8 + |gate|) * 2^-24."""
    if fmt == "fp4":
        lin = lambda ws, n, k, v: po.linear_fp4(ws[0], ws[1], n, k, v, threads=threads)[0]
        alin = lambda ws, n, k, v: po.abs_linear_fp4(ws[0], ws[1], n, k, v, threads=threads)
    else:
        _, bm, bk = fmt
        lin = lambda ws, n, k, v: po.linear_fp8(ws[0], ws[1], n, k, v, bm, bk, threads=threads)[0]
        alin = lambda ws, n, k, v: po.abs_linear_fp8(ws[0], ws[1], n, k, v, bm, bk, threads=threads)
    x_row = np.asarray(x_row, np.float32)
    g32, u32 = lin(gate, inter, input_size, x_row), lin(up, inter, input_size, x_row)
    if limit > 0:
        g32, u32 = np.minimum(g32, np.float32(limit)), np.clip(u32, np.float32(-limit), np.float32(limit))
    silu = np.array([po.silu(float(v)) for v in g32], np.float32)
    h = (silu * u32 * np.float32(output_scale)).astype(np.float32)      # left to right, every step rounded to f32
    y = lin(down, output_size, inter, h)
    g, u = g32.astype(np.float64), u32.astype(np.float64)
    absx = np.abs(x_row.astype(np.float64))
    dg = alin(gate, inter, input_size, input_size * 2.0 ** -24 * absx)
    du = alin(up, inter, input_size, input_size * 2.0 ** -24 * absx)
    absh = np.abs(h.astype(np.float64))
    # the device's silu uses the hardware exp2 and reciprocal: exp(-g) is formed from the rounded product
    # g * log2(e), so its relative error grows with |g| (about |g| * 2^-24 on top of a few ulp), and with it
    # the error of h; bounded, not ulp-pinned
    silu_term = (8.0 + np.abs(g)) * 2.0 ** -24
    dh = abs(float(output_scale)) * (1.1 * np.abs(u) * dg + np.abs(g) * du + 1.1 * dg * du) + absh * silu_term
    bound = alin(down, output_size, inter, (inter + 3) * 2.0 ** -24 * (absh + dh) + dh)
    return y, bound, h


def moe_layer_reference(host_experts, x: np.ndarray, ids: np.ndarray, weights: np.ndarray, hidden: int, inter: int,
                        limit: float = 0.0, prefix: np.ndarray | None = None, threads: int = 8,
                        mx_split: bool = True):
    """The routed MoE layer on the CPU (routed.rs:85-110 over executor.rs:82-124): per token the
    routes in rank order, first route initialises, optional f32 prefix folded first as the device
    does.  host_experts[e] = [(w, s)] * 3 (gate, up, down; a third tuple element is ignored).
    Returns (out f32 [tokens, hidden], bound f64 like out, routes f32 [tokens, k, hidden],
    route bounds f64)."""
    tokens, k = ids.shape
    out = np.zeros((tokens, hidden), np.float32)
    bound = np.zeros((tokens, hidden), np.float64)
    routes = np.zeros((tokens, k, hidden), np.float32)
    route_bounds = np.zeros((tokens, k, hidden), np.float64)
    for t in range(tokens):
        for j in range(k):
            gate, up, down = (m[:2] for m in host_experts[int(ids[t, j])])
            routes[t, j], route_bounds[t, j] = expert_route_reference(
                gate, up, down, hidden, inter, x[t], float(weights[t, j]), limit, threads, mx_split)
        if prefix is None:
            acc = po.accumulate_routes(routes[t])
            magnitude = np.abs(routes[t].astype(np.float64)).sum(0)
        else:
            acc = prefix[t].astype(np.float32).copy()
            for j in range(k):
                acc = (acc + routes[t, j]).astype(np.float32)
            magnitude = np.abs(routes[t].astype(np.float64)).sum(0) + np.abs(prefix[t].astype(np.float64))
        out[t] = acc
        # the fold itself is the same left fold on both sides; its roundings act on slightly
        # different partial sums: k fp32 roundings of at most the running magnitude
        bound[t] = route_bounds[t].sum(0) + (k + 1) * 2.0 ** -24 * (magnitude + route_bounds[t].sum(0))
    return out, bound, routes, route_bounds


def relative_rms(got: np.ndarray, want: np.ndarray) -> float:
    """rms(got - want) / rms(want) in float64."""
    g, w = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return float(np.sqrt(np.mean((g - w) ** 2)) / max(np.sqrt(np.mean(w ** 2)), 1e-300))


# ---- host-side quantized weights by the reference's recipes (inputs the CPU checker can read)

def mxfp4_weight(rng, n, k, sigma=0.02):
    """W ~ N(0, sigma) quantized by the reference's only FP4 recipe
    (encoding.rs:249-284: block 32, scale 2^ceil(log2(amax/6)), ties to the lower magnitude)."""
    w = (rng.standard_normal((n, k)) * sigma).astype(np.float32)
    return po.pack_fp4_act(w, k, 32)


def fp8_weight_e8m0(rng, n, k, block=128, sigma=0.02):
    """W ~ N(0, sigma) -> per block x block tile E8M0 scale 2^ceil(log2(amax/448)), e4m3 by the
    reference's quantizer."""
    w = (rng.standard_normal((n, k)) * sigma).astype(np.float32)
    rows, cols = -(-n // block), -(-k // block)
    scales = np.empty((rows, cols), np.uint8)
    packed = np.empty((n, k), np.uint8)
    if n % block == 0 and k % block == 0:      # whole tiles: one conversion for the matrix (same values)
        amax = np.maximum(np.abs(w).reshape(rows, block, cols, block).max(axis=(1, 3)), np.float32(1e-4))
        scale = np.array([[po.rounded_power_of_two_scale(float(a), 448.0) for a in row] for row in amax], np.float32)
        scales[:] = (scale.view(np.uint32) >> 23) & 0xFF
        return _to_e4m3(w / np.repeat(np.repeat(scale, block, 0), block, 1)), scales
    for i in range(rows):
        for j in range(cols):
            tile = w[i * block:(i + 1) * block, j * block:(j + 1) * block]
            amax = max(float(np.abs(tile).max()), 1e-4)
            scale = po.rounded_power_of_two_scale(amax, 448.0)
            scales[i, j] = int(np.float32(scale).view(np.uint32) >> 23) & 0xFF
            packed[i * block:(i + 1) * block, j * block:(j + 1) * block] = _to_e4m3(tile / np.float32(scale))
    return packed, scales


def fp8_weight_f32(rng, n, k, block=128, sigma=0.02):
    """W ~ N(0, sigma) -> per tile fp32 scale = amax/448, e4m3 round-to-nearest-even of w/scale."""
    w = (rng.standard_normal((n, k)) * sigma).astype(np.float32)
    rows, cols = -(-n // block), -(-k // block)
    scales = np.empty((rows, cols), np.float32)
    packed = np.empty((n, k), np.uint8)
    if n % block == 0 and k % block == 0:      # whole tiles: one conversion for the matrix (same values)
        amax = np.maximum(np.abs(w).reshape(rows, block, cols, block).max(axis=(1, 3)), np.float32(1e-12))
        scales[:] = amax.astype(np.float32) / np.float32(448.0)
        return _to_e4m3(w / np.repeat(np.repeat(scales, block, 0), block, 1)), scales
    for i in range(rows):
        for j in range(cols):
            tile = w[i * block:(i + 1) * block, j * block:(j + 1) * block]
            s = np.float32(max(float(np.abs(tile).max()), 1e-12)) / np.float32(448.0)
            scales[i, j] = s
            packed[i * block:(i + 1) * block, j * block:(j + 1) * block] = _to_e4m3(tile / s)
    return packed, scales


def _to_e4m3(values: np.ndarray) -> np.ndarray:
    import torch

    t = torch.from_numpy(np.clip(values, -448.0, 448.0).astype(np.float32))
    return t.to(torch.float8_e4m3fn).view(torch.uint8).numpy()


# ---- score router (sqrt-softplus top-k) against the checker, with the tolerance of the device's expf / log1pf

SCORE_ULPS = 8      # |device score - host score| allowed when an id differs (expf + log1pf + sqrtf)
WEIGHT_ULPS = 16    # score / sum * scale: the scores' error enters twice


def f64_scores(logits):
    """sqrt(softplus) in float64 by library routines (the closed form of routing.rs:297-303, 367-372)."""
    x = np.asarray(logits, np.float64)
    return np.sqrt(np.where(x > 20.0, x, np.log1p(np.exp(np.minimum(x, 20.0)))))


def check_score_router(logits, bias, k, scale, idx, w):
    """ids equal the checker's, or differ only where selection values are within SCORE_ULPS ulp."""
    rows = logits.shape[0]
    want_idx, want_w = po.router_kernel_rows(1, logits, k, scale, bias=bias)
    same = (idx == want_idx).all(axis=1)
    assert np.all(np.abs(w[same] - want_w[same]) <= WEIGHT_ULPS * np.spacing(want_w[same]))
    near_ties = 0
    for row in np.flatnonzero(~same):
        near_ties += 1
        sel = f64_scores(logits[row]) + (bias.astype(np.float64) if bias is not None else 0.0)
        tol = SCORE_ULPS * np.spacing(np.float32(np.abs(sel).max()))
        chosen = idx[row]
        assert len(set(chosen.tolist())) == k and chosen.min() >= 0
        assert np.all(np.diff(sel[chosen]) <= tol), f"row {row}: ranks out of order beyond the score tolerance"
        rest = np.setdiff1d(np.arange(logits.shape[1]), chosen)
        assert sel[chosen].min() >= sel[rest].max() - tol, f"row {row}: a better expert was left out"
        sc = f64_scores(logits[row, chosen])
        assert np.all(np.abs(w[row] - sc / sc.sum() * scale) <= WEIGHT_ULPS * np.spacing((sc / sc.sum() * scale).astype(np.float32)))
    assert near_ties <= max(2, rows // 500), f"{near_ties} of {rows} rows differ from the checker"
    return near_ties
