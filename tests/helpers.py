"""Shared test helpers: seeded synthetic inputs and the parity comparison rule."""
from __future__ import annotations

import numpy as np

from oracle import pyoracle as po

SEED_BASE = 0xF3771E


def rng_for(config_index: int, extra: int = 0) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(SEED_BASE + config_index + 1000 * extra))


def bf16_activations(rng, shape, sigma=1.0) -> np.ndarray:
    """N(0, sigma) in float64 -> f32 -> BF16 RNE, returned as f32 holding BF16 values."""
    return po.round_to_bf16_array((rng.standard_normal(shape) * sigma).astype(np.float32))


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


def ordered(bits16: np.ndarray) -> np.ndarray:
    """BF16 bit patterns -> integers ordered like the values they encode."""
    b = bits16.astype(np.int32)
    return np.where(b & 0x8000, -(b & 0x7FFF), b)


def compare_bf16(gpu_bits: np.ndarray, oracle_f32: np.ndarray, abs_products_f64: np.ndarray | None = None,
                 k: int = 0, max_ulp: int = 2, gpu_f32: np.ndarray | None = None):
    """The parity rule: |ulp distance| <= max_ulp between the GPU's BF16 output and
    bf16_rne(oracle f32); an element that fails it may still pass through the
    forward-error bound of an fp32 sum in any order, |y_gpu - y_oracle| <= K * 2^-24 * sum|w x|
    (plus half a BF16 ulp for the final rounding when only BF16 output is available).
    Returns (worst ulp among elements judged by ulp, number decided by the bound)."""
    want_bits = po.bf16_bits_array(oracle_f32)
    dist = np.abs(ordered(gpu_bits.astype(np.uint16)) - ordered(want_bits))
    bad = dist > max_ulp
    decided = 0
    if bad.any():
        assert abs_products_f64 is not None, f"{int(bad.sum())} elements off by more than {max_ulp} ulp " \
            f"(max {int(dist.max())})"
        got = (gpu_bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64) if gpu_f32 is None \
            else gpu_f32.astype(np.float64)
        err = np.abs(got - oracle_f32.astype(np.float64))
        bound = k * 2.0 ** -24 * abs_products_f64
        if gpu_f32 is None:
            bound = bound + np.abs(got) * 2.0 ** -8
        still = bad & (err > bound)
        assert not still.any(), f"{int(still.sum())} elements fail both the {max_ulp}-ulp rule and the " \
            f"forward-error bound (worst ulp {int(dist[still].max())})"
        decided = int(bad.sum())
    return int(dist[~bad].max()) if (~bad).any() else 0, decided


def zipf_routing(rng, tokens: int, k: int, experts: int, s: float = 1.1):
    """Per token k distinct experts drawn without replacement with probability proportional to
    rank^-s (Efraimidis-Spirakis: the k largest keys u^(1/p)), softmax weights of k N(0,1) logits."""
    p = np.arange(1, experts + 1, dtype=np.float64) ** -s
    keys = rng.random((tokens, experts)) ** (1.0 / p)
    ids = np.argsort(-keys, axis=1)[:, :k].astype(np.int32)
    logits = rng.standard_normal((tokens, k)).astype(np.float32)
    e = np.exp(logits - logits.max(1, keepdims=True))
    return ids, (e / e.sum(1, keepdims=True)).astype(np.float32)


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
