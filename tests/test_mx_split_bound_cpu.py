"""The truncation limits the parity bounds assume for the decode layer's MX-FP8 activation split
(oracle/parity.py: X_SPLIT_TRUNCATION, H_SPLIT_TRUNCATION), checked on a numpy model of the split
(tests/helpers.py: mx_split_model; the device kernel's bytes equal the model's, tests/test_moe_gpu.py):
per term and 32-element block, scale = 2^(exponent of the block's largest remainder - 7), every
element truncated toward zero onto the E4M3 grid at that scale (3 mantissa bits down to 2^-6,
steps of 2^-9 below), remainder carried to the next term."""
import numpy as np

from ferrule_amd.synthetic import round_to_bf16
from oracle import parity
from tests import helpers as H


def _split_remainder(x: np.ndarray, terms: int) -> np.ndarray:
    """|what is left of every element| after `terms` terms; x is [blocks, 32] float64 holding f32 values.
    The model is the one the GPU test compares the device kernel's bytes with."""
    return H.mx_split_model(x, terms)[2]


def _blocks(rng, count, dtype_bits):
    """Blocks with up to 2^40 of dynamic range inside a block, rounded to BF16 or f32."""
    v = rng.standard_normal((count, 32)) * 2.0 ** rng.integers(-20, 21, (count, 32))
    v *= 2.0 ** rng.integers(-30, 31, (count, 1))
    v = v.astype(np.float32)
    return np.asarray(round_to_bf16(v) if dtype_bits == 16 else v, np.float64)


def test_two_terms_of_bf16_cut_less_than_the_assumed_share_of_the_block_maximum():
    rng = H.rng_for(30)
    x = _blocks(rng, 20000, 16)
    left = _split_remainder(x, 2)
    amax = np.abs(x).max(1, keepdims=True)
    assert (left <= parity.X_SPLIT_TRUNCATION * amax).all()
    # and nothing at all is cut from an element that is normal in the first term
    big = np.abs(x) >= amax * 2.0 ** -12
    assert (left[big] == 0).all()
    # ordinary activations (N(0,1)) are reproduced exactly almost everywhere
    plain = np.asarray(H.bf16_activations(rng, (20000, 32)), np.float64)
    assert (_split_remainder(plain, 2) <= parity.X_SPLIT_TRUNCATION * np.abs(plain).max(1, keepdims=True)).all()


def test_four_terms_of_f32_cut_less_than_the_assumed_share_of_the_block_maximum():
    rng = H.rng_for(31)
    x = _blocks(rng, 20000, 32)
    left = _split_remainder(x, 4)
    amax = np.abs(x).max(1, keepdims=True)
    assert (left < parity.H_SPLIT_TRUNCATION * amax).all()
    # the worst case really comes close to it: an element just below the block maximum with all
    # mantissa bits set keeps 16 of its 24 bits
    worst = np.full((1, 32), np.float64(np.float32(np.nextafter(np.float32(2.0), np.float32(0.0)))))
    assert _split_remainder(worst, 4).max() > parity.H_SPLIT_TRUNCATION * worst.max() * 2.0 ** -2
