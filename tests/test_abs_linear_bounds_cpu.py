"""The error-bound arithmetic of the CPU checker, `fo_abs_linear_fp4` / `fo_abs_linear_fp8`
(sum_k |dequant(W)[row, k]| * v[k] in double), pinned against numpy: every forward-error bound of
the parity rule is a multiple of these sums, so a slip in them (a scale taken from the wrong
block, swapped nibbles, a missing absolute value) would loosen every "decided by bound" verdict
without failing anything else.  The dequantised matrix comes from the checker's own dequant
functions, which the reference's known-answer vectors pin; the sum is numpy's float64 matmul."""
import numpy as np
import pytest

from oracle import pyoracle as po
from tests import helpers as H


def _close(got, want, magnitude=None):
    # both are float64 sums of the same terms in different orders; `magnitude` = the sum of the terms' absolute values
    assert got.shape == want.shape
    magnitude = np.abs(want) if magnitude is None else magnitude
    assert np.all(np.abs(got - want) <= 1e-12 * magnitude + 1e-300)


@pytest.mark.parametrize("n,k", [(16, 32), (5, 96), (33, 224), (128, 1024)])
def test_abs_linear_fp4_equals_numpy_on_the_dequantised_matrix(n, k):
    rng = H.rng_for(40, n * 1000 + k)
    w, s = H.mxfp4_weight(rng, n, k, 0.05)
    # scale bytes far apart between neighbouring blocks, so a block mix-up cannot hide
    s = np.asarray(s).copy().reshape(n, k // 32)
    s[:] = rng.integers(100, 140, s.shape, dtype=np.uint8)
    v = rng.standard_normal(k) * 2.0 ** rng.integers(-6, 7, k)      # signed: the bound takes v as given
    deq = po.dequantize_fp4(w, s, n, k).astype(np.float64)
    _close(po.abs_linear_fp4(w, s, n, k, v), np.abs(deq) @ v, np.abs(deq) @ np.abs(v))
    _close(po.abs_linear_fp4(w, s, n, k, np.abs(v), threads=4), np.abs(deq) @ np.abs(v))
    # one-hot v picks single columns: even and odd nibbles, first and last block
    for col in (0, 1, 31, min(32, k - 1), k - 2, k - 1):
        e = np.zeros(k)
        e[col] = 1.0
        assert np.array_equal(po.abs_linear_fp4(w, s, n, k, e), np.abs(deq[:, col]))


@pytest.mark.parametrize("n,k,bm,bk", [(128, 128, 128, 128), (130, 384, 128, 128), (7, 200, 4, 64), (256, 512, 128, 128)])
@pytest.mark.parametrize("kind", ["e8m0", "f32"])
def test_abs_linear_fp8_equals_numpy_on_the_dequantised_matrix(n, k, bm, bk, kind):
    rng = H.rng_for(41, n * 1000 + k + (0 if kind == "e8m0" else 1))
    w = rng.integers(0, 256, (n, k), dtype=np.uint8)
    w[(w & 0x7F) == 0x7F] = 0x3C                       # no NaN codes
    rows, cols = -(-n // bm), -(-k // bk)
    if kind == "e8m0":
        s = rng.integers(110, 135, (rows, cols), dtype=np.uint8)
    else:
        # negative scales too: the bound needs |scale|
        s = (rng.standard_normal((rows, cols)) * 2.0 ** rng.integers(-8, 3, (rows, cols))).astype(np.float32)
    v = np.abs(rng.standard_normal(k))
    deq = po.dequantize_fp8(w, s, n, k, bm, bk).astype(np.float64)
    # the F32-scale dequant rounds the product to f32; the bound multiplies in double
    dec = np.array([po.decode_fp8_e4m3fn_byte(i) for i in range(256)], np.float64)
    scale = np.repeat(np.repeat(np.abs(s.astype(np.float64)) if kind == "f32" else 2.0 ** (s.astype(np.float64) - 127), bm, 0),
                      bk, 1)[:n, :k]
    exact = np.abs(dec[w]) * scale
    _close(po.abs_linear_fp8(w, s, n, k, v, bm, bk), exact @ v)
    _close(po.abs_linear_fp8(w, s, n, k, v, bm, bk, threads=4), exact @ v)
    # and the double-precision magnitudes are the checker's dequantised values up to its f32 rounding
    assert np.all(np.abs(exact - np.abs(deq)) <= 2.0 ** -23 * exact)
    for col in (0, bk - 1, min(bk, k - 1), k - 1):
        e = np.zeros(k)
        e[col] = 1.0
        assert np.array_equal(po.abs_linear_fp8(w, s, n, k, e, bm, bk), exact[:, col])
