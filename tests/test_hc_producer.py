"""Hyper-connection producer: the CPU checker pinned against the reference's expectations and an
independent float64 evaluation (CPU), then the HIP kernel against the checker (GPU).

Tolerances (GPU): sums run in another order than the checker's, so f32 values are compared at
``REL`` of their scale; the FP8 bytes and scale bytes are compared EXACTLY against the CPU
quantiser applied to the device's own normalized values, and against the checker's bytes up to
the few codes that a last-ulp difference of ``normalized`` can move."""
import ctypes as C

import numpy as np
import pytest
import torch

from ferrule_amd import abi
from oracle import pyoracle as po
from tests import helpers as H

REL = 2.0e-5          # f32 sums of 16 384 terms in another order: K * 2^-24 * (|terms| / |sum|) stays below this
EPS = dict(eps=1e-6, norm_eps=1e-6, layer_rms_eps=1e-6)


def _case(rng, rows, hidden, hc=4):
    mix = (2 + hc) * hc
    state = rng.normal(0.0, 1.0, (rows, hc, hidden)).astype(np.float32)
    function = (rng.normal(0.0, 1.0, (mix, hc * hidden)) / np.sqrt(hc * hidden)).astype(np.float32)
    scale = np.array([0.8, 1.3, 0.6], np.float32)
    base = rng.normal(0.0, 0.3, mix).astype(np.float32)
    weight = (1.0 + 0.1 * rng.normal(size=hidden)).astype(np.float32)
    return state, function, scale, base, weight


def _f64_chain(state, function, scale, base, weight, iters, eps, norm_eps, layer_rms_eps):
    """The same formulas in float64 with numpy's vector routines, written from the definition."""
    rows, hc, hidden = state.shape
    x = state.reshape(rows, -1).astype(np.float64)
    rms = 1.0 / np.sqrt((x * x).mean(axis=1) + norm_eps)
    mixes = (x @ function.astype(np.float64).T) * rms[:, None]
    sig = lambda v: 1.0 / (1.0 + np.exp(-v))
    pre = sig(mixes[:, :hc] * scale[0] + base[:hc]) + eps
    post = 2.0 * sig(mixes[:, hc:2 * hc] * scale[1] + base[hc:2 * hc])
    comb = (mixes[:, 2 * hc:] * scale[2] + base[2 * hc:]).reshape(rows, hc, hc)
    comb = np.exp(comb - comb.max(axis=2, keepdims=True))
    comb = comb / comb.sum(axis=2, keepdims=True) + eps
    comb = comb / (comb.sum(axis=1, keepdims=True) + eps)
    for _ in range(1, iters):
        comb = comb / (comb.sum(axis=2, keepdims=True) + eps)
        comb = comb / (comb.sum(axis=1, keepdims=True) + eps)
    hidden_out = np.einsum("rc,rcd->rd", pre, state.astype(np.float64))
    normalized = hidden_out / np.sqrt((hidden_out ** 2).mean(axis=1, keepdims=True) + layer_rms_eps) * weight
    return dict(raw_dots=x @ function.astype(np.float64).T, pre=pre, post=post, comb=comb, hidden=hidden_out,
                normalized=normalized)


# ---- CPU: the checker ---------------------------------------------------------------------------

def test_reference_split_expectations():
    # hyper_connection.rs:433-453: zero mixes, unit scales, hc = 2, three iterations
    pre, post, comb = po.hc_split_sinkhorn(np.zeros((1, 8)), 2, 3, 1e-6, [1.0, 1.0, 1.0], np.zeros(8))
    assert np.array_equal(pre, np.full((1, 2), np.float32(0.5) + np.float32(1e-6)))
    assert np.array_equal(post, np.ones((1, 2), np.float32))
    assert np.all(np.abs(comb[0].sum(axis=0) - 1.0) < 1e-5)


def test_reference_pre_shapes_case():
    # hyper_connection.rs:470-484: zero function, state [1,2,3,4] as [tokens=1, hc=2, dim=2]
    state = np.array([1.0, 2.0, 3.0, 4.0], np.float32).reshape(1, 2, 2)
    out = po.lib()  # noqa: F841  (library loads)
    mixes = np.zeros((1, 8), np.float32)
    pre, _, _ = po.hc_split_sinkhorn(mixes, 2, 3, 1e-6, [1.0, 1.0, 1.0], np.zeros(8))
    hidden = (pre[0, 0] * state[0, 0] + pre[0, 1] * state[0, 1]).astype(np.float32)
    # the value hc_head's test spells out for the same weights: (0.5 + eps) * (1 + 3), (0.5 + eps) * (2 + 4)
    assert np.allclose(hidden, [(0.5 + 1e-6) * 4.0, (0.5 + 1e-6) * 6.0], rtol=1e-6)


@pytest.mark.parametrize("rows,hidden,iters", [(3, 256, 1), (2, 1024, 4), (1, 4096, 20)])
def test_checker_against_float64_and_invariants(rows, hidden, iters):
    rng = H.rng_for(14, hidden + iters)
    state, function, scale, base, weight = _case(rng, rows, hidden)
    got = po.hc_producer(state, function, scale, base, weight, iters, **EPS)
    want = _f64_chain(state, function, scale, base, weight, iters, **EPS)
    for name in ("raw_dots", "pre", "post", "comb", "hidden", "normalized"):
        scale_of = np.abs(want[name]).max()
        assert np.abs(got[name] - want[name]).max() <= 4e-5 * scale_of, name
    # Sinkhorn: the last step normalises columns, so they sum to 1 / (1 + eps); rows converge
    assert np.all(np.abs(got["comb"].sum(axis=1) - 1.0) < 1e-5)
    if iters >= 20:
        assert np.all(np.abs(got["comb"].sum(axis=2) - 1.0) < 1e-4)
    # the packing is the already pinned activation packer on these values
    packed, scales = po.pack_fp8_act(got["normalized"], hidden, 128)
    assert np.array_equal(got["packed"], packed.reshape(rows, hidden)) and np.array_equal(got["scales"], scales.reshape(rows, -1))
    # rms_norm alone: math.rs:22-42
    assert np.allclose(po.rms_norm(got["hidden"][0], weight, 1e-6), got["normalized"][0], rtol=0, atol=0)
    # BF16 boundaries: both intermediates are BF16 values, and close to the unrounded chain
    rounded = po.hc_producer(state, function, scale, base, weight, iters, bf16_boundaries=True, **EPS)
    for name in ("hidden", "normalized"):
        assert not (rounded[name].view(np.uint32) & 0xFFFF).any()
        assert np.abs(rounded[name] - got[name]).max() <= 2.0 ** -7 * np.abs(got[name]).max()


def test_launch_validation_codes_without_touching_a_device():
    lib = abi.load()
    assert lib.ferrule_hip_hc_producer_can_implement(None) == abi.INVALID_ARGUMENT
    good = dict(rows=2, hc=4, hidden=4096, mix=24, sinkhorn_iters=4, hc_eps=1e-6, hc_norm_eps=1e-6, layer_rms_eps=1e-6,
                **{f: 0x1000 * (i + 1) for i, f in enumerate(
                    ("state_f32", "function_row_major_f32", "hc_scale_f32", "hc_base_f32", "layer_rms_weight_f32",
                     "mix_f32", "hidden_f32", "normalized_f32", "packed_e4m3", "scales_ue8m0", "split_pre_f32",
                     "split_post_f32", "split_comb_f32"))})
    assert lib.ferrule_hip_hc_producer_can_implement(C.byref(abi.HcProducerArgs(**good))) == abi.SUCCESS
    for change, code in ((dict(rows=0), abi.INVALID_ARGUMENT), (dict(hc=2), abi.INVALID_ARGUMENT),
                         (dict(mix=8), abi.INVALID_ARGUMENT), (dict(reserved=2), abi.INVALID_ARGUMENT),
                         (dict(sinkhorn_iters=0), abi.INVALID_ARGUMENT), (dict(hc_eps=0.0), abi.INVALID_ARGUMENT),
                         (dict(hc_norm_eps=float("nan")), abi.INVALID_ARGUMENT), (dict(state_f32=0), abi.INVALID_ARGUMENT),
                         (dict(packed_e4m3=0x1008), abi.INVALID_ARGUMENT), (dict(hidden=4000), abi.UNSUPPORTED),
                         (dict(hidden=16384), abi.UNSUPPORTED)):
        args = abi.HcProducerArgs(**{**good, **change})
        assert lib.ferrule_hip_hc_producer_can_implement(C.byref(args)) == code, change
        assert lib.ferrule_hip_hc_producer_launch(C.byref(args)) == code, change
    assert lib.ferrule_hip_provider_manifest().kernel_mask & abi.kernel_bit(abi.KERNEL_HYPER_CONNECTION_PRODUCER)


# ---- GPU ------------------------------------------------------------------------------------------

def _run(ctx, state, function, scale, base, weight, iters, bf16=False, use_workspace=True):
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    out = ctx.hc_pre_rmsnorm_fp8_into(dev(state), dev(function), dev(scale), dev(base), dev(weight), iters, EPS["eps"],
                                      EPS["norm_eps"], EPS["layer_rms_eps"], bf16_boundaries=bf16,
                                      use_workspace=use_workspace)
    ctx.synchronize()
    return {k: v.cpu().numpy() for k, v in out.items() if k != "workspace"}


@pytest.mark.gpu
@pytest.mark.parametrize("rows,hidden,iters,bf16", [(1, 4096, 4, False), (5, 4096, 4, True), (64, 4096, 4, False),
                                                    (3, 7168, 4, False), (2, 1024, 1, False), (1025, 4096, 3, False),
                                                    (1030, 2048, 2, True), (4, 8192, 4, False), (33, 3072, 4, False)])
def test_kernel_matches_the_checker(rows, hidden, iters, bf16):
    from ferrule_amd.provider import HipArtifactOperatorContext

    ctx = HipArtifactOperatorContext(0)
    rng = H.rng_for(15, rows * 13 + hidden)
    state, function, scale, base, weight = _case(rng, rows, hidden)
    got = _run(ctx, state, function, scale, base, weight, iters, bf16)
    if rows <= 64:
        # without a workspace K is not sliced: same results up to the order of the partial sums
        whole = _run(ctx, state, function, scale, base, weight, iters, bf16, use_workspace=False)
        assert np.abs(whole["mix"] - got["mix"]).max() <= REL and np.array_equal(whole["scales"], got["scales"])
        assert (whole["packed"] != got["packed"]).mean() < 0.002
    sample = np.unique(np.concatenate([np.arange(min(rows, 6)), [rows - 1, rows // 2]]))      # rows checked on the CPU
    want = po.hc_producer(state[sample], function, scale, base, weight, iters, bf16_boundaries=bf16, **EPS)
    for name, key in (("mix", "raw_dots"), ("pre", "pre"), ("post", "post"), ("comb", "comb")):
        assert np.abs(got[name][sample] - want[key]).max() <= REL * max(1.0, np.abs(want[key]).max()), name
    slack = 2.0 ** -8 if bf16 else REL          # a BF16 rounding may fall the other way for a value on the edge
    for name in ("hidden", "normalized"):
        err = np.abs(got[name][sample] - want[name])
        assert err.max() <= slack * np.abs(want[name]).max(), name
        if bf16:
            assert not (got[name].view(np.uint32) & 0xFFFF).any()
            assert (err > REL * np.abs(want[name]).max()).mean() < 0.01
    # the quantiser, exactly, on the device's own normalized values - every row
    packed, scales = po.pack_fp8_act(got["normalized"], hidden, 128)
    assert np.array_equal(got["scales"], scales.reshape(rows, -1))
    assert np.array_equal(got["packed"], packed.reshape(rows, hidden))
    # and against the checker's bytes: only codes next to a rounding boundary may differ
    assert (got["packed"][sample] != want["packed"]).mean() < (0.02 if bf16 else 0.002)
    assert np.array_equal(got["scales"][sample], want["scales"]) or (got["scales"][sample] != want["scales"]).sum() <= 1
    # size-independent properties on all rows: columns of comb sum to 1, pre in (0, 1 + eps), post in (0, 2)
    assert np.all(np.abs(got["comb"].sum(axis=1) - 1.0) < 1e-5)
    assert np.all((got["pre"] > 0) & (got["pre"] < 1.0 + 1e-5)) and np.all((got["post"] > 0) & (got["post"] < 2.0))
    # hidden is linear in the state: doubling the state doubles hidden exactly when pre is unchanged - checked
    # through the weighted sum itself on one row
    r = int(sample[-1])
    direct = np.zeros(hidden, np.float32)
    for c in range(4):
        direct = (direct + got["pre"][r, c] * state[r, c]).astype(np.float32)
    if not bf16:
        assert np.array_equal(direct, got["hidden"][r])     # same multiply-then-add order as the CPU loop
