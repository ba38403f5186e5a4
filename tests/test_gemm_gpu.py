"""FP8 x FP8 block-scaled GEMM on the scaled MFMA against the CPU oracle (GPU only).

The oracle for one output row is LinearWeight::reference_matvec over the dequantized packed
activation row (crates/ferrule-model/src/checkpoint/weight.rs:154-227 with the FP8-K128
activation quantization of weight.rs:63-108), followed by round_to_bf16.  Known answers come
from the reference's own GPU tests (crates/ferrule-backend/tests/fp8_core.rs:151-246,
tests/cutlass_provider.rs:2807-2925)."""
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


def _dequant_rows(xq: np.ndarray, xs: np.ndarray) -> np.ndarray:
    """packed activation rows -> the f32 values the CPU path multiplies with (exact)."""
    scale = 2.0 ** (xs.astype(np.float64) - 127.0)
    return (DEC[xq] * np.repeat(scale, 128, axis=1)).astype(np.float32)


def _check_rows(got_bits, got_f32, rows, xq, xs, w, s, n, k, threads=8):
    x = _dequant_rows(xq[rows], xs[rows])
    want = po.linear_fp8(w, s, n, k, x, threads=threads)
    absprod = np.stack([po.abs_linear_fp8(w, s, n, k, np.abs(row.astype(np.float64)), threads=threads) for row in x])
    return H.compare_bf16(got_bits[rows], want, absprod, k, gpu_f32=None if got_f32 is None else got_f32[rows])


def _bits_of_rounded_f32(out: torch.Tensor) -> np.ndarray:
    raw = out.cpu().numpy().view(np.uint32)
    assert (raw & 0xFFFF == 0).all(), "f32 output must hold BF16-rounded values"
    return (raw >> 16).astype(np.uint16)


@pytest.mark.parametrize("rows", [1, 17, 4097])
def test_projection_all_ones_is_exactly_k(ctx, rows):
    # cutlass_provider.rs:2807-2925: every byte 0x38 (= 1.0), every scale 127, K = 128
    n, k = 96, 128
    x = torch.full((rows, k), 0x38, dtype=torch.uint8, device="cuda")
    xs = torch.full((rows, 1), 127, dtype=torch.uint8, device="cuda")
    w = torch.full((n, k), 0x38, dtype=torch.uint8, device="cuda")
    ws = torch.full((1, 1), 127, dtype=torch.uint8, device="cuda")
    out = ctx.fp8_projection(x, xs, w, ws)
    assert (out == 128.0).all()


def test_query_a_kv_writes_both_outputs(ctx):
    rows, k = 33, 256
    x = torch.full((rows, k), 0x38, dtype=torch.uint8, device="cuda")
    xs = torch.full((rows, 2), 128, dtype=torch.uint8, device="cuda")      # x 2
    w1 = torch.full((48, k), 0x38, dtype=torch.uint8, device="cuda")
    w2 = torch.full((160, k), 0xB8, dtype=torch.uint8, device="cuda")     # -1
    s1 = torch.full((1, 2), 127, dtype=torch.uint8, device="cuda")
    s2 = torch.full((2, 2), 126, dtype=torch.uint8, device="cuda")        # x 0.5
    o1, o2 = ctx.fp8_query_a_kv(x, xs, w1, s1, w2, s2)
    assert (o1 == 512.0).all() and (o2 == -256.0).all()


@pytest.mark.parametrize("rows", [8, 300])
def test_query_a_kv_at_the_model_shape(ctx, rows):
    """DeepSeek-V4's QueryA + KV pair (hidden 4096 -> q_lora 1024 and KV 512, E8M0 block scales): both
    outputs of the one launch against the CPU matvec over the dequantised packed rows."""
    k, n1, n2 = 4096, 1024, 512
    rng = H.rng_for(4, 4096 + rows)
    w1, s1 = H.fp8_weight_e8m0(rng, n1, k)
    w2, s2 = H.fp8_weight_e8m0(rng, n2, k)
    x = H.bf16_activations(rng, (rows, k)).astype(np.float32)
    xq, xs = ctx.pack_fp8_rows_from_f32(torch.from_numpy(x).cuda())
    o1, o2 = ctx.fp8_query_a_kv(xq, xs, torch.from_numpy(w1).cuda(), torch.from_numpy(s1).cuda(),
                                torch.from_numpy(w2).cuda(), torch.from_numpy(s2).cuda())
    sample = np.unique(np.array([0, 1, rows // 2, rows - 1]))
    for out, w, s, n in ((o1, w1, s1, n1), (o2, w2, s2, n2)):
        worst, _ = _check_rows(_bits_of_rounded_f32(out), None, sample, xq.cpu().numpy(), xs.cpu().numpy(), w, s, n, k)
        assert worst <= 2


@pytest.mark.parametrize("rows,n1,n2", [(300, 1024, 512), (8192, 1024, 512), (1000, 200, 72), (8192, 1536, 1024)])
def test_query_a_kv_equals_two_single_projections(ctx, rows, n1, n2):
    """The pair runs as ONE launch whose grid holds the feature tiles of both matrices (both tile
    shapes: 8192 rows take the 256 x 256 one; the last case is 320 such tiles, a short last round that
    is cut into half tiles across both matrices): the same bits as two projection launches."""
    k = 4096
    rng = H.rng_for(4, rows + n1)
    w1, s1 = H.fp8_weight_e8m0(rng, n1, k)
    w2, s2 = H.fp8_weight_e8m0(rng, n2, k)
    x = torch.randn((rows, k), generator=torch.Generator().manual_seed(rows)).cuda()
    xq, xs = ctx.pack_fp8_rows_from_f32(x)
    dev = [torch.from_numpy(a).cuda() for a in (w1, s1, w2, s2)]
    o1, o2 = ctx.fp8_query_a_kv(xq, xs, *dev)
    assert torch.equal(o1, ctx.fp8_projection(xq, xs, dev[0], dev[1]))
    assert torch.equal(o2, ctx.fp8_projection(xq, xs, dev[2], dev[3]))


def test_projection_reference_tile(ctx):
    # fp8_core.rs:151-246: weight [16,128], activation [8,128], palette codes, scales 126 / 125+row%4
    M, N, K = 16, 8, 128
    codes = [0x20, 0x28, 0x30, 0x38, 0x3C, 0x40, 0x44]
    weight = np.zeros((M, K), np.uint8)
    x = np.zeros((N, K), np.uint8)
    for row in range(M):
        for col in range(K):
            weight[row, col] = codes[(row + col * 5) % 7] | (0x80 if (row * 7 + col * 3) % 11 == 0 else 0)
    for row in range(N):
        for col in range(K):
            x[row, col] = codes[(row * 3 + col * 2) % 7] | (0x80 if (row * 5 + col) % 13 == 0 else 0)
    ws = np.array([[126]], np.uint8)
    xs = np.array([[125 + (r % 4)] for r in range(N)], np.uint8)
    out = ctx.fp8_projection(torch.from_numpy(x).cuda(), torch.from_numpy(xs).cuda(),
                             torch.from_numpy(weight).cuda(), torch.from_numpy(ws).cuda())
    want = (DEC[x] * 2.0 ** (xs.astype(np.float64) - 127)) @ (DEC[weight] * 0.5).T
    # the reference's tolerance max(2e-3, 2e-4|y|) is for the unrounded f32 of the core kind-5 linear;
    # this entry rounds to BF16 like fp8_projection.cuh:398-414, and the sum is exactly representable
    assert np.array_equal(_bits_of_rounded_f32(out), po.bf16_bits_array(want.astype(np.float32)))


@pytest.mark.parametrize("rows,n,k,scale_kind", [
    (200, 320, 1024, "e8m0"),
    (1, 128, 128, "e8m0"),
    (130, 200, 384, "e8m0"),      # ragged rows and features
    (200, 320, 1024, "f32"),
    (77, 130, 256, "f32"),
])
def test_block_gemm_matches_the_cpu_reference(ctx, rows, n, k, scale_kind):
    rng = H.rng_for(4, rows * 7 + n)
    if scale_kind == "e8m0":
        w, s = H.fp8_weight_e8m0(rng, n, k)
        shape = _shape().fp8_e4m3_with_e8m0_scale(n, k)
    else:
        w, s = H.fp8_weight_f32(rng, n, k)
        shape = _shape().fp8_e4m3_with_f32_scale(n, k)
    h = ctx.upload_artifact_linear(shape, w, s)
    x = H.bf16_activations(rng, (rows, k)).astype(np.float32)
    xq, xs = ctx.pack_fp8_rows_from_f32(torch.from_numpy(x).cuda())
    xq_h, xs_h = xq.cpu().numpy(), xs.cpu().numpy()
    want_q, want_s = po.pack_fp8_act(x, k, 128)
    assert np.array_equal(xq_h, want_q.reshape(rows, k)) and np.array_equal(xs_h, want_s.reshape(rows, -1))
    out_bf16 = ctx.fp8_block_gemm(xq, xs, h)
    out_f32 = ctx.fp8_block_gemm(xq, xs, h, out_dtype=torch.float32)
    bits = out_bf16.view(torch.int16).cpu().numpy().view(np.uint16)
    assert np.array_equal(bits, _bits_of_rounded_f32(out_f32))
    worst, decided = _check_rows(bits, None, np.arange(rows), xq_h, xs_h, w, s, n, k)
    assert worst <= 2
    if scale_kind == "e8m0":
        # the drop-in entry is the same contraction
        again = ctx.fp8_projection(xq, xs, h.weight.view(n, k), h.scale)
        assert np.array_equal(_bits_of_rounded_f32(again), bits)


def test_block_gemm_large_tile_path(ctx):
    # 4096 x 4096 selects the 256 x 256 workgroup tile; compare everything with a float64 product
    rows, n, k = 4096, 4096, 512
    rng = H.rng_for(4, 99)
    w, s = H.fp8_weight_e8m0(rng, n, k)
    h = ctx.upload_artifact_linear(_shape().fp8_e4m3_with_e8m0_scale(n, k), w, s)
    x = H.bf16_activations(rng, (rows, k)).astype(np.float32)
    xq, xs = ctx.pack_fp8_rows_from_f32(torch.from_numpy(x).cuda())
    out = ctx.fp8_block_gemm(xq, xs, h, out_dtype=torch.float32)
    xd = _dequant_rows(xq.cpu().numpy(), xs.cpu().numpy()).astype(np.float64)
    wd = po.dequantize_fp8(w, s, n, k).astype(np.float64)
    want = xd @ wd.T
    bound = k * 2.0 ** -24 * (np.abs(xd) @ np.abs(wd).T) + np.abs(want) * 2.0 ** -8
    assert (np.abs(out.cpu().numpy().astype(np.float64) - want) <= bound).all()
    sample = np.array([0, 255, 256, 1777, 4095])
    bits = _bits_of_rounded_f32(out)
    worst, _ = _check_rows(bits, None, sample, xq.cpu().numpy(), xs.cpu().numpy(), w, s, n, k)
    assert worst <= 2
    # rows are independent of the tiling: the same rows as a small problem give the same bits
    small = ctx.fp8_block_gemm(xq[256:300].contiguous(), xs[256:300].contiguous(), h, out_dtype=torch.float32)
    assert torch.equal(small, out[256:300])


@pytest.mark.parametrize("rows,n,scale_kind", [
    (2104, 7424, "f32"),     # 9 x 29 = 261 large tiles: 5 tiles in quarters (side by side), one of them 56 rows
    (2304, 7424, "e8m0"),    # the same grid with a full last token tile
    (4096, 4608, "f32"),     # 288 large tiles: 32 tiles in quarters, the pieces of a tile on one XCD
    (2304, 9728, "f32"),     # 342 large tiles: 86 tiles in halves
    (2104, 9728, "e8m0"),    # the same with a last token tile that ends inside its first half
    (2304, 9600, "f32"),     # N not a multiple of 256: 37.5 feature tiles -> 342 tiles, the last feature tile half empty
    (2304, 7360, "e8m0"),    # 261 tiles in quarters, the last feature tile's second half of 64 features
])
def test_block_gemm_short_last_round_is_cut_into_pieces(ctx, rows, n, scale_kind):
    """When the last round of 256 x 256 tiles would fill at most half (a quarter) of the CUs its tiles
    are cut in two along the tokens (in four 128 x 128 ones).  Every output against a float64
    product; the rows of the cut tiles (and the rest) bit for bit against the 128 x 128 path on
    slices of the same rows."""
    k = 512
    rng = H.rng_for(4, rows + n)
    if scale_kind == "f32":
        w, s = H.fp8_weight_f32(rng, n, k)
        shape = _shape().fp8_e4m3_with_f32_scale(n, k)
    else:
        w, s = H.fp8_weight_e8m0(rng, n, k)
        shape = _shape().fp8_e4m3_with_e8m0_scale(n, k)
    h = ctx.upload_artifact_linear(shape, w, s)
    x = H.bf16_activations(rng, (rows, k)).astype(np.float32)
    xq, xs = ctx.pack_fp8_rows_from_f32(torch.from_numpy(x).cuda())
    out = ctx.fp8_block_gemm(xq, xs, h, out_dtype=torch.float32)
    dec = torch.from_numpy(DEC).cuda()
    xd = dec[xq.long()] * torch.repeat_interleave(torch.exp2(xs.double() - 127.0), 128, dim=1)
    wd = torch.from_numpy(po.dequantize_fp8(w, s, n, k)).cuda().double()
    want = xd @ wd.T
    bound = (k * 2.0 ** -24 + 2.0 ** -14.6) * (xd.abs() @ wd.abs().T) + want.abs() * 2.0 ** -8
    assert bool(((out.double() - want).abs() <= bound).all())
    # 100 rows at a time take the 128 x 128 tiles
    for first in range(0, rows, 100):
        last = min(first + 100, rows)
        small = ctx.fp8_block_gemm(xq[first:last].contiguous(), xs[first:last].contiguous(), h, out_dtype=torch.float32)
        assert torch.equal(small, out[first:last]), first


_CONFIG4_WEIGHTS = {}


def _config4_weight(ctx, n, k, scale_kind):
    """W [n, k] ~ N(0, 0.02) of configs[3], quantised on the host by the recipe of its scale kind; one
    copy per (n, kind) for the module."""
    key = (n, k, scale_kind)
    if key not in _CONFIG4_WEIGHTS:
        rng = H.rng_for(4, n)
        if scale_kind == "f32":
            w, s = H.fp8_weight_f32(rng, n, k)
            shape = _shape().fp8_e4m3_with_f32_scale(n, k)
        else:
            w, s = H.fp8_weight_e8m0(rng, n, k)
            shape = _shape().fp8_e4m3_with_e8m0_scale(n, k)
        _CONFIG4_WEIGHTS[key] = (w, s, ctx.upload_artifact_linear(shape, w, s))
    return _CONFIG4_WEIGHTS[key]


@pytest.mark.parametrize("rows,n,scale_kind", [
    (512, 7168, "f32"),        # configs[3], the metric's M = 512: 128 x 128 tiles
    (2048, 7168, "f32"),       # 256 x 256 tiles
    (4096, 18432, "f32"),      # the largest shape of configs[3]
    (512, 18432, "f32"),       # the remaining M x N combinations of configs[3]
    (2048, 18432, "f32"),
    (4096, 7168, "f32"),
    (4096, 18432, "e8m0"),     # the same with the checkpoint's E8M0 block scales
    (4001, 18432, "f32"),      # ragged last token tile
])
def test_config4_prefill_gemm(ctx, rows, n, scale_kind):
    """configs[3]: M BF16 rows ~N(0,1) -> FP8-K128 activation quantisation, W [N, 7168] FP8 with 128x128
    block scales, BF16 output.  Sampled rows against the CPU matvec (<= 2 BF16 ulp), every element
    against a float64 product on the device inside the fp32-sum bound."""
    k = 7168
    w, s, h = _config4_weight(ctx, n, k, scale_kind)
    rng = H.rng_for(4, rows)
    x = H.bf16_activations(rng, (rows, k)).astype(np.float32)
    xq, xs = ctx.pack_fp8_rows_from_f32(torch.from_numpy(x).cuda())
    out = ctx.fp8_block_gemm(xq, xs, h)
    bits = out.view(torch.int16).cpu().numpy().view(np.uint16)
    sample = np.unique(np.array([0, 15, 16, 127, 128, 255, 256, rows // 2 + 3, rows - 130, rows - 2, rows - 1]))
    worst, decided = _check_rows(bits, None, sample, xq.cpu().numpy(), xs.cpu().numpy(), w, s, n, k)
    assert worst <= 2
    # every element against a float64 product on the device (bound: fp32 sum in any order + the MFMA's
    # own alignment of one K block + BF16 rounding)
    dec = torch.from_numpy(DEC).cuda()
    xd = dec[xq.long()] * torch.repeat_interleave(torch.exp2(xs.double() - 127.0), 128, dim=1)
    wd = torch.from_numpy(po.dequantize_fp8(w, s, n, k)).cuda().double()
    want = xd @ wd.T
    bound = (k * 2.0 ** -24 + 2.0 ** -14.6) * (xd.abs() @ wd.abs().T) + want.abs() * 2.0 ** -8
    err = (out.double() - want).abs()
    assert bool((err <= bound).all())
    rms = float((err.pow(2).mean() / want.pow(2).mean()).sqrt())
    assert rms <= 2.0 ** -8, rms           # BF16 rounding alone is 2^-9.8 rms
    print(f"config4 M={rows} N={n} {scale_kind}: worst {worst} ulp over {sample.size} rows ({decided} decided by the "
          f"bound), relative rms of all {rows * n} outputs vs float64 {rms:.2e}")


def test_config4_all_ones_is_exactly_k_on_the_large_tiles(ctx):
    """cutlass_provider.rs:2807-2925 re-sized to configs[3]'s largest shape: every byte 0x38 (= 1.0),
    every scale 1 -> every output exactly K = 7168 (a BF16 value), on every tile of the 256 x 256 path."""
    rows, n, k = 4096, 18432, 7168
    x = torch.full((rows, k), 0x38, dtype=torch.uint8, device="cuda")
    xs = torch.full((rows, k // 128), 127, dtype=torch.uint8, device="cuda")
    for kind, scale in (("f32", torch.ones((n // 128, k // 128), dtype=torch.float32)),
                        ("e8m0", torch.full((n // 128, k // 128), 127, dtype=torch.uint8))):
        shape = _shape().fp8_e4m3_with_f32_scale(n, k) if kind == "f32" else _shape().fp8_e4m3_with_e8m0_scale(n, k)
        h = ctx.upload_artifact_linear(shape, torch.full((n, k), 0x38, dtype=torch.uint8), scale)
        out = ctx.fp8_block_gemm(x, xs, h)
        assert bool((out == float(k)).all()), kind
