"""Dense FP8 SwiGLU FFN (shared expert) against the CPU reference chain (GPU only):
SwiGluFfn::reference_execute (crates/ferrule-model/src/ffn.rs:24-48) over FP8 linear weights with the
FP8-K128 activation quantisation policy in front of both projections (weight.rs:63-108).  Known answers
follow crates/ferrule-backend/tests/cutlass_provider.rs:3246-3351 (zero weights overwrite with 0, the
accumulate flag keeps the previous contents, M in {1, 2, 4, 8, 17})."""
import numpy as np
import pytest
import torch

from oracle import pyoracle as po
from tests import helpers as H

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from ferrule_amd.provider import HipArtifactOperatorContext

    return HipArtifactOperatorContext(0)


def _upload(ctx, w, s, n, k):
    from ferrule_amd.provider import HipArtifactLinearShape as S

    return ctx.upload_artifact_linear(S.fp8_e4m3_with_e8m0_scale(n, k), w, s)


@pytest.mark.parametrize("rows", [1, 2, 4, 8, 17])
def test_zero_weights_overwrite_and_accumulate_keeps(ctx, rows):
    hidden, inter = 256, 128
    z = lambda n, k: _upload(ctx, np.zeros((n, k), np.uint8), np.full((-(-n // 128), k // 128), 127, np.uint8), n, k)
    gate, up, down = z(inter, hidden), z(inter, hidden), z(hidden, inter)
    x = torch.full((rows, hidden), 0x38, dtype=torch.uint8, device="cuda")
    xs = torch.full((rows, hidden // 128), 127, dtype=torch.uint8, device="cuda")
    out = torch.full((rows, hidden), 3.0, dtype=torch.float32, device="cuda")
    ctx.shared_ffn(x, xs, gate, up, down, out)
    assert (out == 0.0).all()
    out.fill_(3.0)
    ctx.shared_ffn(x, xs, gate, up, down, out, accumulate=True)
    assert (out == 3.0).all()


def test_closed_form_ones(ctx):
    # x = 1 (K = 128), W1 = W3 = 1: gate = up = 128, h = silu(128)*128*scale; with scale 2^-10 h = 16,
    # exact in E4M3 at block scale 2^-4; W2 = 1: every output = 128 * 16 = 2048
    hidden, inter, out_features, rows = 128, 128, 64, 5
    one = lambda n, k: _upload(ctx, np.full((n, k), 0x38, np.uint8), np.full((-(-n // 128), k // 128), 127, np.uint8), n, k)
    x = torch.full((rows, hidden), 0x38, dtype=torch.uint8, device="cuda")
    xs = torch.full((rows, 1), 127, dtype=torch.uint8, device="cuda")
    out = torch.zeros((rows, out_features), dtype=torch.float32, device="cuda")
    h, hq, hs = ctx.shared_ffn(x, xs, one(inter, hidden), one(inter, hidden), one(out_features, inter), out,
                               output_scale=2.0 ** -10)
    assert (h == 16.0).all() and (hs == 123).all() and (out == 2048.0).all()


@pytest.mark.parametrize("rows,hidden,inter,out_features,limit,scale", [
    (9, 256, 128, 256, 0.0, 1.0),
    (150, 512, 384, 208, 0.0, 0.5),     # several row tiles, ragged output features
    (40, 384, 256, 384, 0.05, 1.0),
    (17, 4096, 2048, 4096, 0.0, 1.0),   # DeepSeek-V4's shared expert (4096 -> 2048 -> 4096), a decode batch
    (200, 4096, 2048, 4096, 10.0, 1.0), # the same for a packed batch, with the model's clamp
])
def test_shared_ffn_matches_cpu_chain(ctx, rows, hidden, inter, out_features, limit, scale):
    rng = H.rng_for(4, rows * 13 + inter)
    gw, gs = H.fp8_weight_e8m0(rng, inter, hidden, sigma=0.05)
    uw, us = H.fp8_weight_e8m0(rng, inter, hidden, sigma=0.05)
    dw, ds = H.fp8_weight_e8m0(rng, out_features, inter, sigma=0.05)
    gate, up, down = _upload(ctx, gw, gs, inter, hidden), _upload(ctx, uw, us, inter, hidden), \
        _upload(ctx, dw, ds, out_features, inter)
    x = H.bf16_activations(rng, (rows, hidden)).astype(np.float32)
    xq, xs = ctx.pack_fp8_rows_from_f32(torch.from_numpy(x).cuda())
    prev = rng.standard_normal((rows, out_features)).astype(np.float32)
    out = torch.from_numpy(prev.copy()).cuda()
    h_gpu, hq, hs = ctx.shared_ffn(xq, xs, gate, up, down, out, output_scale=scale, swiglu_limit=limit,
                                   accumulate=True)
    h_gpu, hq, hs, got = h_gpu.cpu().numpy(), hq.cpu().numpy(), hs.cpu().numpy(), out.cpu().numpy()
    xdq = po.simulate_fp8_act_quant(x, hidden, 128)
    g = po.linear_fp8(gw, gs, inter, hidden, xdq, threads=4)
    u = po.linear_fp8(uw, us, inter, hidden, xdq, threads=4)
    if limit > 0:
        g, u = np.minimum(g, np.float32(limit)), np.clip(u, np.float32(-limit), np.float32(limit))
    silu = np.array([[po.silu(float(v)) for v in row] for row in g], np.float32)
    h_ref = (silu * u * np.float32(scale)).astype(np.float32)
    # (1) hidden before quantisation: forward error of the two dot products (see test_grouped_moe_gpu)
    eps = hidden * 2.0 ** -24 + 2.0 ** -14
    ax = np.abs(xdq.astype(np.float64))
    dg = eps * (ax @ np.abs(po.dequantize_fp8(gw, gs, inter, hidden).astype(np.float64)).T)
    du = eps * (ax @ np.abs(po.dequantize_fp8(uw, us, inter, hidden).astype(np.float64)).T)
    bound = abs(scale) * (1.1 * np.abs(u) * dg + np.abs(g) * du + dg * du) + np.abs(h_ref) * 2.0 ** -21
    assert (np.abs(h_gpu - h_ref) <= bound + 1e-30).all()
    # (2) quantiser bit-exact on the device's own hidden values
    want_q, want_s = po.pack_fp8_act(h_gpu, inter, 128)
    assert np.array_equal(hs, want_s) and np.array_equal(hq, want_q)
    # (3) down projection of those bytes, accumulated onto the previous output
    hdq = po.simulate_fp8_act_quant(h_gpu, inter, 128)
    y = po.linear_fp8(dw, ds, out_features, inter, hdq, threads=4)
    absprod = np.abs(hdq.astype(np.float64)) @ np.abs(po.dequantize_fp8(dw, ds, out_features, inter).astype(np.float64)).T
    want = (prev + y).astype(np.float32)
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    assert (err <= (inter * 2.0 ** -24 + 2.0 ** -14) * absprod + np.abs(want) * 2.0 ** -23).all()
    # (4) the whole CPU chain (its own hidden values, quantised by the CPU): equal up to the exactly
    # known effect of quantiser codes that differ because h differs in the last fp32 bits
    hq_cpu = po.simulate_fp8_act_quant(h_ref, inter, 128)
    y_cpu = po.linear_fp8(dw, ds, out_features, inter, hq_cpu, threads=4)
    wd = po.dequantize_fp8(dw, ds, out_features, inter).astype(np.float64)
    delta = (hdq.astype(np.float64) - hq_cpu.astype(np.float64)) @ wd.T
    H.quantised_chain_check(got - prev, y_cpu, delta, absprod + np.abs(prev), inter)
