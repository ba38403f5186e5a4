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
