"""GPU parity: dequantisation (bit-exact) and the decode GEMV (<= 2 BF16 ulp, with
the fp32 forward-error bound deciding only for outputs that cancel) against the
CPU checker, through the C ABI."""
import numpy as np
import pytest

from oracle import pyoracle as po
from tests import helpers as H

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def ctx():
    from ferrule_amd.provider import HipArtifactOperatorContext

    return HipArtifactOperatorContext(0)


def _shape():
    from ferrule_amd.provider import HipArtifactLinearShape

    return HipArtifactLinearShape


def _bf16_dev(x_f32: np.ndarray):
    return torch.from_numpy(x_f32).to(torch.bfloat16).cuda()


def _bits(t) -> np.ndarray:
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def _assert_bitwise(got: np.ndarray, want: np.ndarray):
    nan = np.isnan(want)
    nan_mismatch = int((np.isnan(got) != nan).sum())
    assert nan_mismatch == 0, f"{nan_mismatch} NaN positions differ"
    diff = int((got[~nan].view(np.uint32) != want[~nan].view(np.uint32)).sum())
    assert diff == 0, f"{diff} elements differ bitwise"


def _assert_non_finite_like(got: np.ndarray, want: np.ndarray):
    """E8M0 byte 255: the reference's f32 scale overflows to +inf (so products are +-inf, or NaN
    for a zero code); the gfx950 converters read byte 255 as the MX NaN scale.  Both are
    non-finite garbage no checkpoint holds; only non-finiteness is compared."""
    assert not np.isfinite(want).any()
    assert not np.isfinite(got).any()


# ------------------------------------------------------------------ dequant

def test_dequant_mxfp4_every_byte_times_every_scale_is_bit_exact(ctx):
    n, k = 256, 512
    w = np.tile(np.arange(256, dtype=np.uint8), (n, 1))
    s = np.repeat(np.arange(256, dtype=np.uint8)[:, None], k // 32, 1)
    h = ctx.upload_artifact_linear(_shape().fp4_e2m1_packed_with_e8m0_scale(n, k), w, s)
    got = ctx.artifact_linear_dequantize(h).cpu().numpy()
    with np.errstate(all="ignore"):
        want = po.dequantize_fp4(w, s, n, k)
    # scale byte 255 (+inf in the reference) times a zero nibble is NaN there; rows 1..254
    # are the range checkpoints can hold and must match exactly, 0 and 255 are checked too
    _assert_bitwise(got[1:255], want[1:255])
    _assert_bitwise(got[0], want[0])
    _assert_non_finite_like(got[255], want[255])


def test_dequant_fp8_e8m0_every_byte_times_every_scale_is_bit_exact(ctx):
    n, k = 256, 256
    w = np.tile(np.arange(256, dtype=np.uint8), (n, 1))
    s = np.arange(256, dtype=np.uint8).reshape(n, 1)
    h = ctx.upload_artifact_linear(_shape().fp8_e4m3_with_e8m0_scale(n, k, 1, 256), w, s)
    got = ctx.artifact_linear_dequantize(h).cpu().numpy()
    with np.errstate(all="ignore"):
        want = po.dequantize_fp8(w, s, n, k, 1, 256)
    _assert_bitwise(got[3:255], want[3:255])
    # scale bytes 0..2 (2^-127..2^-125) times E4M3 subnormals fall below the smallest BF16
    # subnormal step (2^-133); the converters feed BF16 MFMA operands, so those 96 products
    # are the BF16 rounding of the exact value.  No checkpoint scale is anywhere near.
    representable = po.round_to_bf16_array(want[:3]).view(np.uint32) == want[:3].view(np.uint32)
    representable |= np.isnan(want[:3])
    assert int((~representable).sum()) == 96
    _assert_bitwise(np.where(representable, got[:3], 0), np.where(representable, want[:3], 0))
    err = np.abs(got[:3].astype(np.float64) - want[:3].astype(np.float64))
    assert (err[~representable] <= 2.0 ** -134).all()
    _assert_non_finite_like(got[255], want[255])


def test_dequant_fp8_f32_scales_is_bit_exact(ctx):
    rng = H.rng_for(1, 7)
    n, k = 256, 512
    w, s = H.fp8_weight_f32(rng, n, k)
    h = ctx.upload_artifact_linear(_shape().fp8_e4m3_with_f32_scale(n, k), w, torch.from_numpy(s))
    got = ctx.artifact_linear_dequantize(h).cpu().numpy()
    _assert_bitwise(got, po.dequantize_fp8(w, s, n, k))


# ------------------------------------------------------------------ GEMV parity

def _check_gemv(ctx, shape, w, s, x_f32, deq=None, label=""):
    h = ctx.upload_artifact_linear(shape, w, torch.from_numpy(s) if s.dtype == np.float32 else s)
    y = ctx.artifact_linear_gemv_bf16(h, _bf16_dev(x_f32))
    yf = ctx.artifact_linear_gemv_bf16(h, _bf16_dev(x_f32), out_dtype=torch.float32)
    ctx.synchronize()
    n, k = shape.out_features, shape.in_features
    if shape.weight_format == 2:
        want = po.linear_fp4(w, s, n, k, x_f32, threads=8)
        if deq is None:
            deq = po.dequantize_fp4(w, s, n, k)
    else:
        want = po.linear_fp8(w, s, n, k, x_f32, shape.block_m, shape.block_k, threads=8)
        if deq is None:
            deq = po.dequantize_fp8(w, s, n, k, shape.block_m, shape.block_k)
    absprod = np.abs(x_f32.astype(np.float64)) @ np.abs(deq.astype(np.float64)).T
    worst, decided = H.compare_bf16(_bits(y), want, absprod, k)
    # the f32 output is the same accumulator before rounding
    assert np.array_equal(_bits(y), po.bf16_bits_array(yf.cpu().numpy()))
    err = np.abs(yf.cpu().numpy().astype(np.float64) - want.astype(np.float64))
    assert (err <= k * 2.0 ** -24 * absprod + 1e-30).all()
    print(f"{label}: worst ulp {worst}, decided by bound {decided}/{want.size}")
    return y


def test_config1_fp8_gemv_4096x4096_f32_block_scales(ctx):
    rng = H.rng_for(1)
    n = k = 4096
    x = H.bf16_activations(rng, (1, k))
    w, s = H.fp8_weight_f32(rng, n, k)
    _check_gemv(ctx, _shape().fp8_e4m3_with_f32_scale(n, k), w, s, x, label="C1 f32 scales")


def test_config1_fp8_gemv_4096x4096_e8m0_block_scales(ctx):
    rng = H.rng_for(1, 1)
    n = k = 4096
    x = H.bf16_activations(rng, (1, k))
    w, s = H.fp8_weight_e8m0(rng, n, k)
    _check_gemv(ctx, _shape().fp8_e4m3_with_e8m0_scale(n, k), w, s, x, label="C1 e8m0 scales")


@pytest.mark.parametrize("batch", [1, 4, 8])
def test_config2_mxfp4_gemv_4096x7168(ctx, batch):
    rng = H.rng_for(2)
    n, k = 4096, 7168
    w, s = H.mxfp4_weight(rng, n, k)
    x = H.bf16_activations(rng, (batch, k))
    _check_gemv(ctx, _shape().fp4_e2m1_packed_with_e8m0_scale(n, k), w, s, x, label=f"C2 B={batch}")


@pytest.mark.parametrize("n,k,batch", [(16, 128, 1), (48, 384, 3), (4096, 7168, 1), (4096, 7168, 8), (7168, 2048, 17)])
def test_mxfp4_gemv_on_block_major_weights_gives_the_same_bits(ctx, n, k, batch):
    """The prepared (block-major) order changes which bytes a wave load brings, not which
    products enter which accumulator in which order."""
    rng = H.rng_for(2, n * 3 + k + batch)
    w, s = H.mxfp4_weight(rng, n, k)
    x = _bf16_dev(H.bf16_activations(rng, (batch, k)))
    handle = ctx.upload_artifact_linear(_shape().fp4_e2m1_packed_with_e8m0_scale(n, k), w, s)
    prepared = ctx.prepare_mxfp4_block_major(handle)
    want = ctx.artifact_linear_gemv_bf16(handle, x)
    got = ctx.artifact_linear_gemv_bf16(prepared, x)
    ctx.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("n,k,batch,f32", [(16, 128, 1, True), (48, 384, 3, False), (4096, 4096, 1, True),
                                           (4096, 4096, 8, False), (7168, 2048, 5, True)])
def test_fp8_gemv_on_block_major_weights_gives_the_same_bits(ctx, n, k, batch, f32):
    rng = H.rng_for(1, n * 3 + k + batch)
    x = _bf16_dev(H.bf16_activations(rng, (batch, k)))
    if f32:
        w, s = H.fp8_weight_f32(rng, n, k)
        handle = ctx.upload_artifact_linear(_shape().fp8_e4m3_with_f32_scale(n, k), w, torch.from_numpy(s))
    else:
        w, s = H.fp8_weight_e8m0(rng, n, k)
        handle = ctx.upload_artifact_linear(_shape().fp8_e4m3_with_e8m0_scale(n, k), w, s)
    prepared = ctx.prepare_fp8_block_major(handle)
    # the documented permutation: [tile][row][cell][64 B] -> [tile][cell][row][64 B]
    want_w = np.ascontiguousarray(w.reshape(n // 16, 16, k // 64, 64).transpose(0, 2, 1, 3)).reshape(-1)
    assert np.array_equal(prepared.weight.cpu().numpy().reshape(-1), want_w)
    want = ctx.artifact_linear_gemv_bf16(handle, x)
    got = ctx.artifact_linear_gemv_bf16(prepared, x)
    ctx.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    with pytest.raises(ValueError):
        ctx.fp8_block_gemm(torch.zeros((1, k), dtype=torch.uint8, device="cuda"),
                           torch.zeros((1, k // 128), dtype=torch.uint8, device="cuda"), prepared)


def test_block_major_gemv_needs_whole_tiles(ctx):
    from ferrule_amd.provider import HipArtifactLinearHandle, ProviderError

    rng = H.rng_for(2, 5)
    w, s = H.mxfp4_weight(rng, 24, 160)
    h = ctx.upload_artifact_linear(_shape().fp4_e2m1_packed_with_e8m0_scale(24, 160), w, s)
    with pytest.raises(ProviderError):
        ctx.prepare_mxfp4_block_major(h)                      # 24 rows, K = 160: no whole tiles
    fake = HipArtifactLinearHandle(h.shape, h.weight, h.scale, block_major=True)
    with pytest.raises(ProviderError):
        ctx.artifact_linear_gemv_bf16(fake, _bf16_dev(np.ones((1, 160), np.float32)))


def test_batch_rows_equal_single_row_results_bit_for_bit(ctx):
    # the invariant the reference asserts for its own kernels (fp8_core.rs:412-425)
    rng = H.rng_for(2, 3)
    n, k = 512, 1024
    w, s = H.mxfp4_weight(rng, n, k)
    x = H.bf16_activations(rng, (5, k))
    h = ctx.upload_artifact_linear(_shape().fp4_e2m1_packed_with_e8m0_scale(n, k), w, s)
    full = ctx.artifact_linear_gemv_bf16(h, _bf16_dev(x), out_dtype=torch.float32).cpu().numpy()
    for b in range(5):
        one = ctx.artifact_linear_gemv_bf16(h, _bf16_dev(x[b:b + 1]), out_dtype=torch.float32).cpu().numpy()
        assert np.array_equal(one[0].view(np.uint32), full[b].view(np.uint32))


@pytest.mark.parametrize("fmt,block_major", [("fp4", False), ("fp4", True), ("fp8_f32", False), ("fp8_e8m0", True)])
def test_several_matrices_in_one_launch_equal_the_single_launches(ctx, fmt, block_major):
    """ferrule_hip_quant_gemv_multi_launch: matrices of different shapes, batches and inputs in one
    launch give the bits of one launch each (the single launches are checked against the CPU above)."""
    from ferrule_amd import abi
    from ferrule_amd.provider import ProviderError

    rng = H.rng_for(2, 77 + len(fmt))
    shapes = [(4096, 7168, 1), (1024, 4096, 3), (512, 4096, 1), (48, 384, 8), (7168, 2048, 9)]
    handles, xs = [], []
    for n, k, batch in shapes:
        if fmt == "fp4":
            w, s = H.mxfp4_weight(rng, n, k)
            h = ctx.upload_artifact_linear(_shape().fp4_e2m1_packed_with_e8m0_scale(n, k), w, s)
            h = ctx.prepare_mxfp4_block_major(h) if block_major else h
        elif fmt == "fp8_f32":
            w, s = H.fp8_weight_f32(rng, n, k)
            h = ctx.upload_artifact_linear(_shape().fp8_e4m3_with_f32_scale(n, k), w, torch.from_numpy(s))
        else:
            w, s = H.fp8_weight_e8m0(rng, n, k)
            h = ctx.upload_artifact_linear(_shape().fp8_e4m3_with_e8m0_scale(n, k), w, s)
            h = ctx.prepare_fp8_block_major(h) if block_major else h
        handles.append(h)
        xs.append(_bf16_dev(H.bf16_activations(rng, (batch, k))))
    want = [ctx.artifact_linear_gemv_bf16(h, x) for h, x in zip(handles, xs)]
    outs = [torch.full_like(w_, float("nan")) for w_ in want]
    before = ctx.kernel_launches
    ctx.artifact_linears_gemv_bf16_into(handles, xs, outs)
    ctx.synchronize()
    assert ctx.kernel_launches == before + 1
    for got, ref in zip(outs, want):
        assert torch.equal(got.view(torch.int16), ref.view(torch.int16))
    # f32 and bf16 outputs may be mixed; one matrix alone is the plain launch
    f32 = torch.empty((xs[1].shape[0], shapes[1][0]), dtype=torch.float32, device="cuda")
    ctx.artifact_linears_gemv_bf16_into(handles[1:2], xs[1:2], [f32])
    assert np.array_equal(po.bf16_bits_array(f32.cpu().numpy()), _bits(want[1]))
    # mixed weight orders or formats are refused, and more than the limit too
    if fmt == "fp4" and block_major:
        w, s = H.mxfp4_weight(rng, 16, 128)
        row_major = ctx.upload_artifact_linear(_shape().fp4_e2m1_packed_with_e8m0_scale(16, 128), w, s)
        x16 = _bf16_dev(H.bf16_activations(rng, (1, 128)))
        o16 = torch.empty((1, 16), dtype=torch.bfloat16, device="cuda")
        with pytest.raises(ProviderError):
            ctx.artifact_linears_gemv_bf16_into([handles[3], row_major], [xs[3], x16], [outs[3], o16])
        with pytest.raises(ValueError):
            ctx.artifact_linears_gemv_bf16_into([row_major] * (abi.GEMV_MULTI_MAX + 1), [x16] * (abi.GEMV_MULTI_MAX + 1),
                                                [o16] * (abi.GEMV_MULTI_MAX + 1))


@pytest.mark.parametrize("fmt", ["fp4", "fp8_f32"])
def test_the_largest_multi_matrix_launch_equals_the_single_launches(ctx, fmt):
    """FERRULE_HIP_GEMV_MULTI_MAX (32) matrices of assorted shapes and batches in one launch: the bits
    of 32 single launches (a grouped linear takes a descriptor array, abi/core_provider.h:478-480)."""
    from ferrule_amd import abi

    rng = H.rng_for(2, 3200 + len(fmt))
    pool = [(256, 1024, 1), (512, 4096, 2), (48, 384, 1), (1024, 2048, 3), (4096, 7168, 1), (128, 512, 8), (7168, 2048, 1)]
    handles, xs = [], []
    for i in range(abi.GEMV_MULTI_MAX):
        n, k, batch = pool[i % len(pool)]
        if fmt == "fp4":
            w, s = H.mxfp4_weight(rng, n, k)
            h = ctx.prepare_mxfp4_block_major(ctx.upload_artifact_linear(_shape().fp4_e2m1_packed_with_e8m0_scale(n, k), w, s))
        else:
            w, s = H.fp8_weight_f32(rng, n, k)
            h = ctx.upload_artifact_linear(_shape().fp8_e4m3_with_f32_scale(n, k), w, torch.from_numpy(s))
        handles.append(h)
        xs.append(_bf16_dev(H.bf16_activations(rng, (batch, k))))
    want = [ctx.artifact_linear_gemv_bf16(h, x) for h, x in zip(handles, xs)]
    outs = [torch.full_like(w_, float("nan")) for w_ in want]
    before = ctx.kernel_launches
    ctx.artifact_linears_gemv_bf16_into(handles, xs, outs)
    ctx.synchronize()
    assert ctx.kernel_launches == before + 1
    for i, (got, ref) in enumerate(zip(outs, want)):
        assert torch.equal(got.view(torch.int16), ref.view(torch.int16)), f"matrix {i} differs from its single launch"


@pytest.mark.parametrize("fmt", ["fp4", "fp8_e8m0"])
def test_tall_matrix_runs_small_workgroups_with_the_same_bits(ctx, fmt):
    """More than 1024 row tiles: four small workgroups per CU, each wave walking several K slices.
    Against the CPU matvec, and the first 4096 rows bit for bit against a launch of those rows alone
    (256 tiles: one wave per K slice)."""
    rng = H.rng_for(2, 1025 + len(fmt))
    n, k, batch = 16400, 4096, 2
    x = H.bf16_activations(rng, (batch, k))
    if fmt == "fp4":
        w, s = H.mxfp4_weight(rng, n, k)
        shape, head = _shape().fp4_e2m1_packed_with_e8m0_scale(n, k), _shape().fp4_e2m1_packed_with_e8m0_scale(4096, k)
        s_head = s[:4096]
    else:
        w, s = H.fp8_weight_e8m0(rng, n, k)
        shape, head = _shape().fp8_e4m3_with_e8m0_scale(n, k), _shape().fp8_e4m3_with_e8m0_scale(4096, k)
        s_head = s[:4096 // 128]
    _check_gemv(ctx, shape, w, s, x, label=f"tall {fmt}")
    full = ctx.artifact_linear_gemv_bf16(ctx.upload_artifact_linear(shape, w, s), _bf16_dev(x))
    part = ctx.artifact_linear_gemv_bf16(ctx.upload_artifact_linear(head, w[:4096], s_head), _bf16_dev(x))
    assert torch.equal(full[:, :4096].view(torch.int16), part.view(torch.int16))


def test_closed_forms_unit_weights_and_scale_doubling(ctx):
    n, k = 48, 256
    # nibble 2 = +1.0 everywhere, unit scales, x = small integers -> exact integer sums
    w = np.full((n, k // 2), 0x22, np.uint8)
    s = np.full((n, k // 32), 127, np.uint8)
    x = (np.arange(k) % 7 - 3).astype(np.float32)[None, :]
    h = ctx.upload_artifact_linear(_shape().fp4_e2m1_packed_with_e8m0_scale(n, k), w, s)
    y = ctx.artifact_linear_gemv_bf16(h, _bf16_dev(x), out_dtype=torch.float32).cpu().numpy()
    assert (y == x.sum()).all()
    # E8M0 byte +1 on block 2 doubles exactly that block's contribution
    s2 = s.copy()
    s2[:, 2] = 128
    h2 = ctx.upload_artifact_linear(_shape().fp4_e2m1_packed_with_e8m0_scale(n, k), w, s2)
    y2 = ctx.artifact_linear_gemv_bf16(h2, _bf16_dev(x), out_dtype=torch.float32).cpu().numpy()
    assert (y2 == x.sum() + x[0, 64:96].sum()).all()
    # FP8: all 0x38 (=1.0), scale 127, K=128, x=1 -> every output exactly 128
    # (the reference's own closed form, cutlass_provider.rs:2807-2865)
    w8 = np.full((32, 128), 0x38, np.uint8)
    h8 = ctx.upload_artifact_linear(_shape().fp8_e4m3_with_e8m0_scale(32, 128), w8, np.array([[127]], np.uint8))
    y8 = ctx.artifact_linear_gemv_bf16(h8, _bf16_dev(np.ones((3, 128), np.float32))).float().cpu().numpy()
    assert (y8 == 128.0).all()


@pytest.mark.parametrize("n,k,batch", [(100, 160, 3), (16, 32, 1), (33, 4096, 17), (1, 7168, 2)])
def test_mxfp4_ragged_shapes(ctx, n, k, batch):
    rng = H.rng_for(2, n + k)
    w, s = H.mxfp4_weight(rng, n, k)
    x = H.bf16_activations(rng, (batch, k))
    _check_gemv(ctx, _shape().fp4_e2m1_packed_with_e8m0_scale(n, k), w, s, x, label=f"fp4 {n}x{k} B={batch}")


@pytest.mark.parametrize("n,k,bm,bk,batch,f32", [
    (100, 48, 128, 128, 2, False),     # K tail below one block
    (130, 384, 128, 128, 1, True),     # partial last scale row
    (64, 256, 16, 128, 9, True),       # small block_m
    (40, 192, 1, 64, 2, False),        # per-row scales, 64-wide K blocks (per-lane scale path)
    (24, 100, 5, 24, 3, False),        # odd everything -> generic kernel
    (24, 100, 5, 24, 3, True),
])
def test_fp8_ragged_shapes_and_generic_blocks(ctx, n, k, bm, bk, batch, f32):
    rng = H.rng_for(1, n * k + bm)
    wq = rng.integers(0, 256, (n, k), dtype=np.uint8)
    wq[(wq & 0x7F) == 0x7F] = 0x30
    rows, cols = -(-n // bm), -(-k // bk)
    s = rng.uniform(2e-4, 2e-3, (rows, cols)).astype(np.float32) if f32 else \
        rng.integers(115, 123, (rows, cols), dtype=np.uint8)
    x = H.bf16_activations(rng, (batch, k))
    mk = _shape().fp8_e4m3_with_f32_scale if f32 else _shape().fp8_e4m3_with_e8m0_scale
    _check_gemv(ctx, mk(n, k, bm, bk), wq, s, x, label=f"fp8 {n}x{k} bm{bm} bk{bk}")


def test_gemv_rejects_bad_activations(ctx):
    from ferrule_amd.provider import ProviderError

    w = np.zeros((16, 16), np.uint8)
    s = np.full((16, 1), 127, np.uint8)
    h = ctx.upload_artifact_linear(_shape().fp4_e2m1_packed_with_e8m0_scale(16, 32), w, s)
    with pytest.raises(ValueError):
        ctx.artifact_linear_gemv_bf16(h, torch.zeros((1, 32), device="cuda"))          # f32, not bf16
    with pytest.raises(ValueError):
        ctx.artifact_linear_gemv_bf16(h, torch.zeros((1, 64), dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(ProviderError):
        ctx.artifact_linear_gemv_bf16(h, torch.zeros((0, 32), dtype=torch.bfloat16, device="cuda"))


# ------------------------------------------------------------------ quantizers (kinds 4, 5)

def test_fp8_pack_matches_cpu_reference_bitwise(ctx):
    rng = H.rng_for(4, 1)
    rows, k = 64, 1024
    vals = np.concatenate([
        H.bf16_activations(rng, (rows // 2, k)),                                   # BF16-valued
        (rng.standard_normal((rows // 2, k)) * np.exp(rng.uniform(-6, 6, (rows // 2, 1)))).astype(np.float32),
    ])
    vals[3, 128:256] = 0.0                      # an all-zero block (amax floor)
    vals[5, 7] = np.float32(1e9)                # clamp
    vals[6, 0:128] = np.float32(2.0 ** -20)     # below the 1e-4 floor
    packed, scales = ctx.pack_fp8_rows_from_f32(torch.from_numpy(vals).cuda())
    want_p, want_s = po.pack_fp8_act(vals, k, 128)
    assert np.array_equal(scales.cpu().numpy(), want_s)
    assert np.array_equal(packed.cpu().numpy(), want_p)


def test_fp8_pack_of_a_large_matrix_matches_cpu_reference_bitwise(ctx):
    """8 M values and more take the quantiser's sixteen-values-per-thread form: the same bytes and
    scales, special blocks included (zeros, below the amax floor, clamped, non-finite, every tie of
    the grid under the CPU's half-away rule and under half-even)."""
    from ferrule_amd import abi, synthetic

    rng = H.rng_for(4, 2)
    rows, k = 1184, 7168                         # 8.49 M values
    vals = (rng.standard_normal((rows, k)) * np.exp(rng.uniform(-6, 6, (rows, 1)))).astype(np.float32)
    vals[:rows // 2] = synthetic.round_to_bf16(vals[:rows // 2])
    vals[3, 128:256] = 0.0
    vals[5, 7] = np.float32(1e9)
    vals[6, 0:128] = np.float32(2.0 ** -20)
    vals[7, 300] = np.float32(np.inf)            # non-finite block maximum
    vals[8, 900] = np.float32(np.nan)
    # ties: with amax 448 the scale is 1 and the block holds values halfway between grid points
    ties = np.array([448.0, 17.0, 18.0, 19.0, 0.001953125 * 1.5, 0.001953125 * 2.5, 1.0625, 1.1875, 27.0, 29.0,
                     -17.0, -19.0, 2.0 ** -10, 3 * 2.0 ** -10], np.float32)
    vals[9, 0:ties.size] = ties
    vals[9, ties.size:128] = 0.0
    dev = torch.from_numpy(vals).cuda()
    for mode in (abi.FP8_ROUND_CPU_REFERENCE, abi.FP8_ROUND_HALF_EVEN):
        packed, scales = ctx.pack_fp8_rows_from_f32(dev, rounding=mode)
        # the same launch cut into pieces below the size that selects the wide form
        small_p, small_s = [], []
        for r0 in range(0, rows, 400):
            p, s = ctx.pack_fp8_rows_from_f32(dev[r0:r0 + 400].contiguous(), rounding=mode)
            small_p.append(p)
            small_s.append(s)
        assert torch.equal(packed, torch.cat(small_p)) and torch.equal(scales, torch.cat(small_s))
        if mode == abi.FP8_ROUND_CPU_REFERENCE:
            with np.errstate(all="ignore"):
                want_p, want_s = po.pack_fp8_act(vals, k, 128)
            finite = np.isfinite(vals).reshape(rows, k // 128, 128).all(2)
            got_s, got_p = scales.cpu().numpy(), packed.cpu().numpy()
            assert np.array_equal(got_s[finite], want_s.reshape(rows, -1)[finite])
            assert np.array_equal(got_p.reshape(rows, -1, 128)[finite], want_p.reshape(rows, -1, 128)[finite])


def test_fp8_pack_reference_gpu_grid(ctx):
    # fp8_core.rs:111-122
    col = np.arange(256)
    base = ((col % 31).astype(np.float32) - np.float32(15.0)) * np.where(col < 128, np.float32(0.25), np.float32(0.00075))
    vals = np.stack([base, base * np.float32(2.0)]).astype(np.float32)
    packed, scales = ctx.pack_fp8_rows_from_f32(torch.from_numpy(vals).cuda())
    want_p, want_s = po.pack_fp8_act(vals, 256, 128)
    assert np.array_equal(scales.cpu().numpy(), want_s) and np.array_equal(packed.cpu().numpy(), want_p)


def test_fp8_pack_every_bf16_value_against_cpu_reference(ctx):
    # all finite BF16 bit patterns as one long row set; each 128-block holds one binade mix
    b = np.arange(0x0080, 0x7F80, dtype=np.uint32)
    b = np.concatenate([b, b | 0x8000])
    vals = (b << 16).view(np.float32)
    pad = (-vals.size) % 128
    vals = np.concatenate([vals, np.zeros(pad, np.float32)]).reshape(-1, 128)
    packed, scales = ctx.pack_fp8_rows_from_f32(torch.from_numpy(vals).cuda())
    want_p, want_s = po.pack_fp8_act(vals, 128, 128)
    assert np.array_equal(scales.cpu().numpy(), want_s)
    assert np.array_equal(packed.cpu().numpy(), want_p)


def test_hardware_fp8_converter_equals_the_cpu_rule_off_the_ties(ctx):
    """The GEMM epilogues take E4M3 bytes from the hardware converter (round to nearest even) and fall back to
    the exact routine - the CPU quantiser's rule, encoding.rs:207-242, pinned by the tests above - when a
    value has the low 19 bits of its f32 pattern clear.  Every finite f32 pattern through both: off those
    patterns they never differ; on them they do differ somewhere (else the fallback would be dead code)."""
    counts = torch.zeros(3, dtype=torch.int64, device="cuda")
    status = ctx.lib.ferrule_hip_fp8_converter_selftest_launch(counts.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert status == 0
    torch.cuda.synchronize()
    wrong, example, ties = (int(v) for v in counts.cpu())
    assert wrong == 0, f"{wrong} patterns off the ties differ, e.g. 0x{example - 1:08x}"
    assert ties > 0


def test_fp4_pack_matches_cpu_reference_bitwise(ctx):
    rng = H.rng_for(2, 9)
    vals = (rng.standard_normal((128, 512)) * 0.02).astype(np.float32)
    vals[0, :32] = 0.0
    idx = np.arange(128)                        # fp4_core.rs:187-192 grid in rows 1..2
    vals[1, :128] = ((idx % 17) - 8).astype(np.float32) * np.float32(0.375) + np.where(idx % 11 == 0, 4.25, 0.0).astype(np.float32)
    packed, scales = ctx.pack_fp4_rows_from_f32(torch.from_numpy(vals).cuda())
    want_p, want_s = po.pack_fp4_act(vals, 512, 32)
    assert np.array_equal(scales.cpu().numpy(), want_s)
    assert np.array_equal(packed.cpu().numpy(), want_p)


def test_pack_with_odd_block_size_uses_the_scalar_kernel(ctx):
    rng = H.rng_for(4, 3)
    vals = rng.standard_normal((6, 144)).astype(np.float32)
    packed, scales = ctx.pack_fp8_rows_from_f32(torch.from_numpy(vals).cuda(), block_size=48)
    want_p, want_s = po.pack_fp8_act(vals, 144, 48)
    assert np.array_equal(scales.cpu().numpy(), want_s) and np.array_equal(packed.cpu().numpy(), want_p)


# ------------------------------------------------------------------ core linear drop-in (kinds 4, 5, 8)

def _f32_close(got, want, absprod, k):
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    assert (err <= k * 2.0 ** -24 * absprod + 1e-30).all(), float(err.max())


def test_core_linear_kind4_and_kind8(ctx):
    rng = H.rng_for(1, 21)
    n, k, batch = 96, 384, 3
    w, s = H.fp8_weight_e8m0(rng, n, k)
    h = ctx.upload_artifact_linear(_shape().fp8_e4m3_with_e8m0_scale(n, k), w, s)
    x = rng.standard_normal((batch, k)).astype(np.float32)
    deq = po.dequantize_fp8(w, s, n, k).astype(np.float64)
    out = torch.empty((batch, n), dtype=torch.float32, device="cuda")
    ctx.artifact_linear_matvec_into(h, torch.from_numpy(x).cuda(), out)
    _f32_close(out.cpu().numpy(), po.linear_fp8(w, s, n, k, x), np.abs(x.astype(np.float64)) @ np.abs(deq).T, k)
    ctx.artifact_linear_matvec_into(h, torch.from_numpy(x).cuda(), out, quantize_input=True)
    xq = po.simulate_fp8_act_quant(x, k, 128)
    _f32_close(out.cpu().numpy(), po.linear_fp8(w, s, n, k, x, act_quant_block=128),
               np.abs(xq.astype(np.float64)) @ np.abs(deq).T, k)


def test_core_linear_kind5_prepacked_reference_tile(ctx):
    # fp8_core.rs:151-246: 16x8x128 tile, codes from a small palette, scales 126 / 125+row%4
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
    h = ctx.upload_artifact_linear(_shape().fp8_e4m3_with_e8m0_scale(M, K), weight, ws)
    out = torch.empty((N, M), dtype=torch.float32, device="cuda")
    ctx.gemm_fp8_e4m3fn_e8m0_prepacked(h, torch.from_numpy(x).cuda(), torch.from_numpy(xs).cuda(), out)
    dec = np.array([po.decode_fp8_e4m3fn_byte(i) for i in range(256)], np.float64)
    want = (dec[x] * 2.0 ** (xs.astype(np.float64) - 127)) @ (dec[weight] * 0.5).T
    got = out.cpu().numpy()
    tol = np.maximum(2e-3, np.abs(want) * 2e-4)                     # the reference's own tolerance
    assert (np.abs(got - want) <= tol).all()
    assert (np.abs(got - want) <= 1e-4 * np.abs(want) + 1e-6).all()  # and a much tighter one
