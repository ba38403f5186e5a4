"""Shared test helpers: seeded synthetic inputs and the parity comparison rule."""
from __future__ import annotations

import numpy as np

from ferrule_amd.synthetic import (SEED_BASE, bf16_activations, concentrated_routing, rng_for,  # noqa: F401
                                   uniform_routing, zipf_routing)
from oracle import pyoracle as po
from oracle.parity import (_to_e4m3, check_score_router, compare_bf16, compare_bf16_bounded, expert_route_reference,  # noqa: F401
                           fp8_weight_e8m0, fp8_weight_f32, moe_layer_reference, mxfp4_weight, ordered, relative_rms,
                           swiglu_ffn_reference)


def quantised_chain_check(got_f32, want_f32, code_flip_delta_f64, abs_products_f64, k, min_fraction=0.97,
                          output_rounding=2.0 ** -22):
    """End-to-end check of a chain with a quantiser in the middle (gate/up -> FP8 requantisation ->
    down).  The device's hidden activations differ from the CPU's in the last fp32 bits, so a value on
    a rounding boundary of the quantiser may land on the neighbouring code; `code_flip_delta_f64` is
    the exact effect of those code differences on the output, W (Q(h_gpu) - Q(h_cpu)).  Required:
    every output equals CPU output + that delta within the fp32 / MFMA summation bound (plus
    `output_rounding` relative, 2^-8 when the output was rounded to BF16), and at least
    `min_fraction` of the outputs are within 2 BF16 ulp of the CPU chain outright."""
    got = got_f32.astype(np.float64)
    err = np.abs(got - (want_f32.astype(np.float64) + code_flip_delta_f64))
    bound = 2.0 * (k * 2.0 ** -24 + 2.0 ** -14) * abs_products_f64 + (np.abs(got) + np.abs(want_f32.astype(np.float64))) * output_rounding
    assert (err <= bound + 1e-30).all(), f"{int((err > bound).sum())} outputs not explained by quantiser code flips"
    dist = np.abs(ordered(po.bf16_bits_array(got_f32)) - ordered(po.bf16_bits_array(want_f32)))
    within = float((dist <= 2).mean())
    assert within >= min_fraction, f"only {within:.4f} of the outputs within 2 BF16 ulp of the CPU chain"
    return within


def mx_split_model(x: np.ndarray, terms: int):
    """Numpy model of the decode layer's MX-FP8 activation split.  x: [blocks, 32] holding f32 (or
    BF16) values.  Per term and block: scale byte = clamp(biased f32 exponent of the block's largest
    remainder - 7, 1, 253) (127 for an all-zero block), every element truncated toward zero onto the
    E4M3 grid at that scale (3 mantissa bits for values of at least 2^-6 of the scale, steps of 2^-9
    below), the remainder carried to the next term.  Returns (codes u8 [terms, blocks, 32], scale
    bytes u8 [terms, blocks], |remainder| after the last term)."""
    r = x.astype(np.float64).copy()
    codes = np.empty((terms,) + r.shape, np.uint8)
    scales = np.empty((terms, r.shape[0]), np.uint8)
    for t in range(terms):
        amax = np.abs(r).max(1, keepdims=True).astype(np.float32)
        biased = ((amax.view(np.uint32) >> 23) & 0xFF).astype(np.int64)     # 0 for zero and subnormals
        sbyte = np.clip(biased - 7, 1, 253)
        s = 2.0 ** (sbyte.astype(np.float64) - 127)
        a = np.abs(r) / s
        normal = a >= 2.0 ** -6
        e = np.floor(np.log2(np.where(normal, a, 1.0)))
        mant = np.floor(a / 2.0 ** (e - 3))                                  # 8..15
        kept = np.where(normal, mant * 2.0 ** (e - 3), np.floor(a * 512.0) / 512.0)
        code = np.where(normal, ((e + 7).astype(np.int64) << 3) | (mant.astype(np.int64) - 8), np.floor(a * 512.0).astype(np.int64))
        sign = np.where(np.signbit(r), 0x80, 0)
        codes[t] = (sign | code).astype(np.uint8)
        scales[t] = np.where(amax[:, 0] == 0, 127, sbyte[:, 0]).astype(np.uint8)
        left = np.abs(r) - kept * s
        r = np.where(left == 0, 0.0, np.sign(r) * left)      # an exhausted element continues as +0
    return codes, scales, np.abs(r)
