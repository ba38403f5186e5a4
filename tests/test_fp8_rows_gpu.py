"""The decode-row schedule of the FP8 x FP8 entry points (GPU only).

The reference's FP8 projection and shared FFN are small-M kernels tested at M in {1, 17, 4097} and
M in {1, 2, 4, 8, 17} (crates/ferrule-backend/tests/cutlass_provider.rs:2807-2925, 3246-3351), and its
native providers choose the schedule from the row count (src/cuda/provider.rs:46-49).  Here up to 32
rows stream the weights once with one wave per 16 output features; more rows run MFMA tiles.  What
is checked: a row's bits do not depend on the schedule (every entry point, both scale kinds, every
output mode, ragged shapes, K of every remainder with respect to the load ring), the reference's
known answers at those row counts, and parity with the CPU matvec at the model's shapes."""
import numpy as np
import pytest
import torch

from oracle import pyoracle as po
from tests import helpers as H

pytestmark = pytest.mark.gpu

DEC = np.array([po.decode_fp8_e4m3fn_byte(i) for i in range(256)], np.float64)


@pytest.fixture(scope="module")
def ctx():
    from ferrule_amd.provider import HipArtifactOperatorContext

    return HipArtifactOperatorContext(0)


def _shape():
    from ferrule_amd.provider import HipArtifactLinearShape

    return HipArtifactLinearShape


def _weight(ctx, rng, n, k, scale_kind, sigma=0.02):
    if scale_kind == "e8m0":
        w, s = H.fp8_weight_e8m0(rng, n, k, sigma=sigma)
        shape = _shape().fp8_e4m3_with_e8m0_scale(n, k)
    else:
        w, s = H.fp8_weight_f32(rng, n, k, sigma=sigma)
        shape = _shape().fp8_e4m3_with_f32_scale(n, k)
    return w, s, ctx.upload_artifact_linear(shape, w, s)


def _packed_rows(ctx, rng, rows, k):
    x = H.bf16_activations(rng, (rows, k)).astype(np.float32)
    # block scales that differ from row to row and block to block
    x *= (2.0 ** rng.integers(-3, 4, (rows, k // 128))).repeat(128, 1).astype(np.float32)
    return ctx.pack_fp8_rows_from_f32(torch.from_numpy(x).cuda())


def _bits_of_rounded_f32(out: torch.Tensor) -> np.ndarray:
    raw = out.cpu().numpy().view(np.uint32)
    assert (raw & 0xFFFF == 0).all(), "f32 output must hold BF16-rounded values"
    return (raw >> 16).astype(np.uint16)


@pytest.mark.parametrize("scale_kind", ["e8m0", "f32"])
@pytest.mark.parametrize("n,k", [
    (7168, 7168),   # the model's square projection: 448 waves, 56 K blocks
    (200, 640),     # ragged features (12.5 tiles), 5 K blocks: less than one ring
    (96, 1536),     # 12 K blocks: exactly one ring
    (130, 2176),    # 17 K blocks: one ring and five more
    (1024, 512),    # 4 K blocks: the smallest K the schedule takes
    (17, 512),      # one whole feature tile and one of a single row
    (5, 896),       # less than one feature tile, 7 K blocks
])
def test_a_row_has_the_same_bits_in_both_schedules(ctx, n, k, scale_kind):
    rng = H.rng_for(50, n + k)
    _, _, handle = _weight(ctx, rng, n, k, scale_kind)
    for rows in (1, 2, 3, 8, 15, 16, 17, 31, 32):
        xq, xs = _packed_rows(ctx, rng, rows, k)
        for dtype in (torch.bfloat16, torch.float32):
            streamed = ctx.fp8_block_gemm(xq, xs, handle, out_dtype=dtype)
            tiled = ctx.fp8_block_gemm(xq, xs, handle, out_dtype=dtype, tile_schedule=True)
            assert torch.equal(streamed.view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                               tiled.view(torch.int16 if dtype == torch.bfloat16 else torch.int32)), \
                f"{rows} rows, {dtype}: the decode-row schedule differs from the tiles"
    # and from a packed batch that holds the same rows: 16 (24) rows alone == rows 40..56 (40..64) of 300
    xq, xs = _packed_rows(ctx, rng, 300, k)
    whole = ctx.fp8_block_gemm(xq, xs, handle, out_dtype=torch.float32)
    for end in (56, 64):
        part = ctx.fp8_block_gemm(xq[40:end].clone(), xs[40:end].clone(), handle, out_dtype=torch.float32)
        assert torch.equal(part.view(torch.int32), whole[40:end].view(torch.int32))
    # 100 rows alone are too many for the row stream and too few tiles of 128 x 128 to cover the machine
    # (where the matrix is large): they run on narrower tiles, with the bits of the large batch
    part = ctx.fp8_block_gemm(xq[40:140].clone(), xs[40:140].clone(), handle, out_dtype=torch.float32)
    assert torch.equal(part.view(torch.int32), whole[40:140].view(torch.int32))


@pytest.mark.parametrize("rows", [1, 8, 16, 17, 32])
def test_projection_and_query_a_kv_take_the_row_schedule_with_the_same_bits(ctx, rows):
    """The drop-in entries have no flag word: their results at decode rows are compared with the
    general entry kept on the tile schedule (the same contraction, f32 holding BF16-rounded values)."""
    k, n1, n2 = 4096, 1024, 512
    rng = H.rng_for(51, rows)
    _, _, h1 = _weight(ctx, rng, n1, k, "e8m0")
    _, _, h2 = _weight(ctx, rng, n2, k, "e8m0")
    xq, xs = _packed_rows(ctx, rng, rows, k)
    want1 = ctx.fp8_block_gemm(xq, xs, h1, out_dtype=torch.float32, tile_schedule=True)
    want2 = ctx.fp8_block_gemm(xq, xs, h2, out_dtype=torch.float32, tile_schedule=True)
    o1, o2 = ctx.fp8_query_a_kv(xq, xs, h1.weight.view(n1, k), h1.scale, h2.weight.view(n2, k), h2.scale)
    assert torch.equal(o1.view(torch.int32), want1.view(torch.int32))
    assert torch.equal(o2.view(torch.int32), want2.view(torch.int32))
    single = ctx.fp8_projection(xq, xs, h2.weight.view(n2, k), h2.scale)
    assert torch.equal(single.view(torch.int32), want2.view(torch.int32))


@pytest.mark.parametrize("rows", [1, 16, 17, 33])
def test_projection_all_ones_is_exactly_k_at_a_streamed_k(ctx, rows):
    # the known answer of cutlass_provider.rs:2807-2925 (every byte 1.0, every scale 127) at a K the
    # decode-row schedule takes; 17 rows are the reference's second row count, 33 rows run the tiles
    n, k = 96, 1024
    x = torch.full((rows, k), 0x38, dtype=torch.uint8, device="cuda")
    xs = torch.full((rows, k // 128), 127, dtype=torch.uint8, device="cuda")
    w = torch.full((n, k), 0x38, dtype=torch.uint8, device="cuda")
    ws = torch.full((1, k // 128), 127, dtype=torch.uint8, device="cuda")
    assert (ctx.fp8_projection(x, xs, w, ws) == float(k)).all()


@pytest.mark.parametrize("scale_kind", ["e8m0", "f32"])
@pytest.mark.parametrize("rows", [1, 16, 17])
def test_rows_schedule_matches_the_cpu_matvec_at_the_model_shape(ctx, rows, scale_kind):
    n = k = 7168
    rng = H.rng_for(52, rows)
    w, s, handle = _weight(ctx, rng, n, k, scale_kind)
    xq, xs = _packed_rows(ctx, rng, rows, k)
    out = ctx.fp8_block_gemm(xq, xs, handle)
    xq_h, xs_h = xq.cpu().numpy(), xs.cpu().numpy()
    x = (DEC[xq_h] * np.repeat(2.0 ** (xs_h.astype(np.float64) - 127.0), 128, axis=1)).astype(np.float32)
    sample = np.unique(np.array([0, rows // 2, rows - 1]))
    want = po.linear_fp8(w, s, n, k, x[sample], threads=8)
    absprod = np.stack([po.abs_linear_fp8(w, s, n, k, np.abs(r.astype(np.float64)), threads=8) for r in x[sample]])
    worst, _ = H.compare_bf16(out.view(torch.int16).cpu().numpy().view(np.uint16)[sample], want, absprod, k)
    assert worst <= 2


def _upload_e8m0(ctx, w, s, n, k):
    return ctx.upload_artifact_linear(_shape().fp8_e4m3_with_e8m0_scale(n, k), w, s)


@pytest.mark.parametrize("hidden,inter,out_features,limit,scale", [
    (4096, 2048, 4096, 0.0, 1.0),     # DeepSeek-V4's shared expert
    (4096, 2048, 4096, 10.0, 1.0),    # with the model's clamp
    (512, 640, 80, 0.05, 0.5),        # ragged output features, K of 4 and 5 blocks
])
def test_shared_ffn_rows_schedule_equals_the_tile_schedule(ctx, hidden, inter, out_features, limit, scale):
    """Every buffer the FFN writes - h in f32, its FP8 bytes and scale bytes, the output - has the same
    bits whether the decode-row launches or the tiled kernels produced it, with and without the
    accumulate flag, at the reference's row counts (cutlass_provider.rs:3246-3351: 1, 2, 4, 8, 17) and at 16 and 32."""
    rng = H.rng_for(53, hidden + inter)
    gw, gs = H.fp8_weight_e8m0(rng, inter, hidden, sigma=0.05)
    uw, us = H.fp8_weight_e8m0(rng, inter, hidden, sigma=0.05)
    dw, ds = H.fp8_weight_e8m0(rng, out_features, inter, sigma=0.05)
    gate, up, down = _upload_e8m0(ctx, gw, gs, inter, hidden), _upload_e8m0(ctx, uw, us, inter, hidden), \
        _upload_e8m0(ctx, dw, ds, out_features, inter)
    for rows in (1, 2, 4, 8, 16, 17, 32):
        xq, xs = _packed_rows(ctx, rng, rows, hidden)
        prev = torch.randn((rows, out_features), generator=torch.Generator().manual_seed(rows)).cuda()
        for accumulate in (False, True):
            got_out, want_out = prev.clone(), prev.clone()
            got = ctx.shared_ffn(xq, xs, gate, up, down, got_out, output_scale=scale, swiglu_limit=limit,
                                 accumulate=accumulate)
            want = ctx.shared_ffn(xq, xs, gate, up, down, want_out, output_scale=scale, swiglu_limit=limit,
                                  accumulate=accumulate, tile_schedule=True)
            assert torch.equal(got[0].view(torch.int32), want[0].view(torch.int32)), f"{rows} rows: hidden f32 differs"
            assert torch.equal(got[2], want[2]), f"{rows} rows: hidden scale bytes differ"
            assert torch.equal(got[1], want[1]), f"{rows} rows: hidden FP8 bytes differ"
            assert torch.equal(got_out.view(torch.int32), want_out.view(torch.int32)), f"{rows} rows: output differs"
            assert np.isfinite(got_out.cpu().numpy()).all()


@pytest.mark.parametrize("rows", [1, 8, 16, 24, 40])
def test_prepacked_core_linear_takes_the_gemm_schedules(ctx, rows):
    """ferrule_hip_core_linear_launch kind 5 (packed FP8-K128 activations, the second half of the
    activation-quantisation policy, context.rs:10694-10785) at a shape with whole K blocks: the unrounded
    f32 of the FP8 GEMM schedules, whose BF16 rounding is the general entry's output bit for bit; and
    within the forward-error bound of the CPU matvec."""
    n, k = 1536, 4096
    rng = H.rng_for(54, rows)
    w, s, handle = _weight(ctx, rng, n, k, "e8m0")
    xq, xs = _packed_rows(ctx, rng, rows, k)
    out = torch.empty((rows, n), dtype=torch.float32, device="cuda")
    ctx.gemm_fp8_e4m3fn_e8m0_prepacked(handle, xq, xs, out)
    rounded = ctx.fp8_block_gemm(xq, xs, handle, out_dtype=torch.float32, tile_schedule=True)
    got = out.cpu().numpy()
    assert np.array_equal(po.bf16_bits_array(got), _bits_of_rounded_f32(rounded))
    xq_h, xs_h = xq.cpu().numpy(), xs.cpu().numpy()
    x = (DEC[xq_h] * np.repeat(2.0 ** (xs_h.astype(np.float64) - 127.0), 128, axis=1)).astype(np.float32)
    sample = np.unique(np.array([0, rows // 2, rows - 1]))
    want = po.linear_fp8(w, s, n, k, x[sample], threads=8)
    absprod = np.stack([po.abs_linear_fp8(w, s, n, k, np.abs(r.astype(np.float64)), threads=8) for r in x[sample]])
    err = np.abs(got[sample].astype(np.float64) - want.astype(np.float64))
    assert (err <= (k * 2.0 ** -24 + 2.0 ** -14.6) * absprod + 1e-30).all()
