"""Dense SwiGLU FFN for decode batches in GEMV form (ferrule_hip_dense_ffn_decode_launch) against the CPU
chain SwiGluFfn::reference_execute (crates/ferrule-model/src/ffn.rs:24-48) over quantized LinearWeights
(checkpoint/weight.rs:154-173), through the C ABI.  Known answers follow the reference's own FFN tests
(ffn.rs:80-137: f32 linears, output scale, clamp) re-expressed with exactly representable quantized
weights, and its shared-FFN batch sizes M in {1, 2, 4, 8, 17} (cutlass_provider.rs:3246-3351)."""
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


def _S():
    from ferrule_amd.provider import HipArtifactLinearShape

    return HipArtifactLinearShape


def _linears(ctx, rng, fmt, input_size, inter, output_size, sigma, block_major):
    """(gate, up, down) as host (weight, scales) pairs and device handles."""
    host, dev = [], []
    for n, k in ((inter, input_size), (inter, input_size), (output_size, inter)):
        if fmt == "fp4":
            w, s = H.mxfp4_weight(rng, n, k, sigma)
            h = ctx.upload_artifact_linear(_S().fp4_e2m1_packed_with_e8m0_scale(n, k), w, s)
            h = ctx.prepare_mxfp4_block_major(h) if block_major else h
        elif fmt == "fp8_f32":
            w, s = H.fp8_weight_f32(rng, n, k, sigma=sigma)
            h = ctx.upload_artifact_linear(_S().fp8_e4m3_with_f32_scale(n, k), w, torch.from_numpy(s))
            h = ctx.prepare_fp8_block_major(h) if block_major else h
        else:
            w, s = H.fp8_weight_e8m0(rng, n, k, sigma=sigma)
            h = ctx.upload_artifact_linear(_S().fp8_e4m3_with_e8m0_scale(n, k), w, s)
            h = ctx.prepare_fp8_block_major(h) if block_major else h
        host.append((w, s))
        dev.append(h)
    return host, dev


@pytest.mark.parametrize("fmt,batch,input_size,inter,output_size,limit,scale,block_major", [
    ("fp4", 1, 512, 256, 384, 0.0, 1.0, False),
    ("fp4", 3, 1024, 512, 1024, 0.05, 0.5, True),
    ("fp4", 17, 512, 384, 256, 0.0, 1.0, True),          # five passes of the down projection (4 rows each)
    ("fp8_e8m0", 2, 512, 256, 512, 0.0, 1.0, False),
    ("fp8_e8m0", 8, 768, 384, 256, 0.05, 2.0, True),
    ("fp8_f32", 4, 512, 256, 512, 0.0, 1.0, False),
    ("fp8_f32", 5, 1024, 128, 768, 0.0, 1.0, True),
    ("fp8_e8m0", 1, 4096, 2048, 4096, 10.0, 1.0, True),   # DeepSeek-V4's shared expert, one token
    ("fp8_e8m0", 8, 4096, 2048, 4096, 10.0, 1.0, False),  # and a batch of eight, checkpoint order
    ("fp4", 4, 7168, 2048, 7168, 0.0, 1.0, True),         # an MXFP4 expert of the baseline's shape run densely
])
def test_dense_ffn_decode_matches_the_cpu_chain(ctx, fmt, batch, input_size, inter, output_size, limit, scale,
                                                block_major):
    rng = H.rng_for(12, batch * 31 + inter + len(fmt))
    host, dev = _linears(ctx, rng, fmt, input_size, inter, output_size, 0.05 if input_size <= 1024 else 0.02, block_major)
    x = H.bf16_activations(rng, (batch, input_size))
    xd = torch.from_numpy(x).to(torch.bfloat16).cuda()
    out, sums = ctx.dense_ffn_decode(dev[0], dev[1], dev[2], xd, output_scale=scale, swiglu_limit=limit)
    out32, sums32 = ctx.dense_ffn_decode(dev[0], dev[1], dev[2], xd, output_scale=scale, swiglu_limit=limit,
                                         out_dtype=torch.float32)
    ctx.synchronize()
    bits = out.view(torch.int16).cpu().numpy().view(np.uint16)
    assert np.array_equal(bits, po.bf16_bits_array(out32.cpu().numpy()))       # one rounding of the same sums
    assert torch.equal(sums, sums32)
    # the gate and up sums are those of two plain GEMV launches, bit for bit
    for j in range(2):
        alone = ctx.artifact_linear_gemv_bf16(dev[j], xd, out_dtype=torch.float32)
        assert torch.equal(alone, sums[j])
    hidden = _hidden_from_sums(sums.cpu().numpy(), scale, limit)
    kind = "fp4" if fmt == "fp4" else ("fp8", 128, 128)
    rows = range(batch) if input_size <= 1024 else sorted({0, batch // 2, batch - 1})
    worst_h = 0.0
    for b in rows:
        want, bound, h = H.swiglu_ffn_reference(kind, host[0], host[1], host[2], input_size, inter, output_size, x[b],
                                                scale, limit, threads=8)
        # the hidden row (f32, before the down projection): a few ulp of the CPU's, dot products reordered
        h_gpu = hidden[b]
        worst_h = max(worst_h, float(np.abs(h_gpu - h).max() / max(np.abs(h).max(), 1e-30)))
        err = np.abs(out32[b].cpu().numpy().astype(np.float64) - want)
        assert (err <= bound + 1e-30).all(), f"row {b}: {int((err > bound).sum())} outputs outside the forward-error bound"
        worst, decided, _ = H.compare_bf16_bounded(bits[b], want, bound, max_decided_fraction=0.005)
        assert worst <= 2
    assert worst_h <= 2e-5, worst_h
    # rows do not depend on the batch they travel in (the reference's own invariant for its linears,
    # fp8_core.rs:412-425)
    alone, _ = ctx.dense_ffn_decode(dev[0], dev[1], dev[2], xd[batch - 1:batch].contiguous(), output_scale=scale,
                                    swiglu_limit=limit, out_dtype=torch.float32)
    assert torch.equal(alone[0], out32[batch - 1])


def _hidden_from_sums(sums, scale, limit):
    """silu(gate) * up * scale in f32, left to right, clamped first (ffn.rs:33-47): what the down launch
    forms from the two rows of sums on its way in."""
    gate, up = sums[0].astype(np.float32), sums[1].astype(np.float32)
    if limit > 0:
        gate, up = np.minimum(gate, np.float32(limit)), np.clip(up, np.float32(-limit), np.float32(limit))
    silu = (gate / (np.float32(1) + np.exp(-gate, dtype=np.float32))).astype(np.float32)
    return ((silu * up).astype(np.float32) * np.float32(scale)).astype(np.float32)


def test_dense_ffn_closed_form_and_clamp(ctx):
    """ffn.rs:80-137 in quantized form: x = 1 (K = 128), W1 = W3 = +1 everywhere (nibble 2, unit scales):
    gate = up = 128, hidden = silu(128) * 128 * 2^-10 = 16; W2 = +1: every output 128 * 16 = 2048.  With the
    clamp at 4: gate = up = 4, hidden = silu(4) * 4 * 2^-10, output 128 * hidden."""
    n_in = inter = 128
    n_out = 64
    ones = lambda n, k: ctx.upload_artifact_linear(_S().fp4_e2m1_packed_with_e8m0_scale(n, k),
                                                   np.full((n, k // 2), 0x22, np.uint8), np.full((n, k // 32), 127, np.uint8))
    gate, up, down = ones(inter, n_in), ones(inter, n_in), ones(n_out, inter)
    x = torch.ones((2, n_in), dtype=torch.bfloat16, device="cuda")
    out, sums = ctx.dense_ffn_decode(gate, up, down, x, output_scale=2.0 ** -10, out_dtype=torch.float32)
    assert bool((sums == 128.0).all()) and bool((out == 2048.0).all())
    out, sums = ctx.dense_ffn_decode(gate, up, down, x, output_scale=2.0 ** -10, swiglu_limit=4.0,
                                     out_dtype=torch.float32)
    assert bool((sums == 128.0).all())      # the clamp acts where the hidden value is formed
    h = np.float32(np.float32(np.float32(po.silu(4.0)) * np.float32(4.0)) * np.float32(2.0 ** -10))
    # 128 equal terms: the exact sum 128 h' is an f32 value, and the device forms it without any rounding
    # (each of the three BF16 parts of h' sums exactly), so every output is the same number, a multiple
    # of 128; h' is the device's hidden value, within 4 ulp of the CPU's (hardware exp2 and reciprocal
    # in its silu); the CPU's sequential f32 sum is within 128 * 2^-24 of 128 h
    values = out.cpu().numpy()
    assert (values == values.flat[0]).all()
    assert abs(float(values.flat[0]) / 128.0 - float(h)) <= 4 * 2.0 ** -24 * float(h)
    want = po.linear_fp4(np.full((n_out, inter // 2), 0x22, np.uint8), np.full((n_out, inter // 32), 127, np.uint8),
                         n_out, inter, np.full(inter, h, np.float32))[0]
    assert (np.abs(want.astype(np.float64) - 128.0 * float(h)) <= 128 * 2.0 ** -24 * 128.0 * float(h)).all()


def test_dense_ffn_refuses_mismatched_linears(ctx):
    rng = H.rng_for(12, 5)
    host, dev = _linears(ctx, rng, "fp4", 512, 256, 512, 0.05, False)
    other = ctx.prepare_mxfp4_block_major(dev[2])
    x = torch.zeros((1, 512), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):
        ctx.dense_ffn_decode(dev[0], dev[1], other, x)            # mixed weight orders
    with pytest.raises(ValueError):
        ctx.dense_ffn_decode(dev[0], dev[2], dev[1], x)           # shapes do not chain
