"""Seeded synthetic inputs of the benchmark configurations: activations, routings and
quantized weights, the latter drawn and quantized ON THE DEVICE by the provider's own
packers.  Used by ``bench.py``, the smoke check and the tests; imports nothing from the
CPU checker.

Seeds: PCG64(0xF3771E + config index) on the host, ``torch.Generator`` with the same
number on the device.
"""
from __future__ import annotations

import numpy as np

SEED_BASE = 0xF3771E


def rng_for(config_index: int, extra: int = 0) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(SEED_BASE + config_index + 1000 * extra))


def round_to_bf16(values: np.ndarray) -> np.ndarray:
    """f32 -> f32 holding BF16 values: round to nearest even on bit 16, NaN quieted, like
    ``round_to_bf16`` (crates/ferrule-model/src/models/common/math.rs:7-14)."""
    bits = np.ascontiguousarray(values, np.float32).view(np.uint32)
    nan = (bits & 0x7FFFFFFF) > 0x7F800000
    rounded = (bits + (0x7FFF + ((bits >> 16) & 1))) & 0xFFFF0000
    rounded = np.where(nan, (bits | 0x00400000) & 0xFFFF0000, rounded).astype(np.uint32)
    return rounded.view(np.float32).reshape(np.shape(values))


def bf16_activations(rng, shape, sigma: float = 1.0) -> np.ndarray:
    """N(0, sigma) in float64 -> f32 -> BF16 RNE, returned as f32 holding BF16 values."""
    return round_to_bf16((rng.standard_normal(shape) * sigma).astype(np.float32))


def uniform_routing(rng, tokens: int, k: int, experts: int):
    """Per token k distinct experts drawn uniformly without replacement, softmax weights of
    k N(0,1) logits (f32)."""
    ids = np.stack([rng.permutation(experts)[:k] for _ in range(tokens)]).astype(np.int32)
    logits = rng.standard_normal((tokens, k)).astype(np.float32)
    e = np.exp(logits - logits.max(1, keepdims=True))
    return ids, (e / e.sum(1, keepdims=True)).astype(np.float32)


def zipf_routing(rng, tokens: int, k: int, experts: int, s: float = 1.1):
    """Per token k distinct experts drawn without replacement with probability proportional to
    rank^-s (Efraimidis-Spirakis: the k largest keys u^(1/p)), softmax weights of k N(0,1) logits."""
    p = np.arange(1, experts + 1, dtype=np.float64) ** -s
    keys = rng.random((tokens, experts)) ** (1.0 / p)
    ids = np.argsort(-keys, axis=1)[:, :k].astype(np.int32)
    logits = rng.standard_normal((tokens, k)).astype(np.float32)
    e = np.exp(logits - logits.max(1, keepdims=True))
    return ids, (e / e.sum(1, keepdims=True)).astype(np.float32)


def concentrated_routing(rng, tokens: int, k: int, experts: int, hot: int):
    """Every token routes to k distinct experts out of the first ``hot`` ones only: the
    worst case for a decode layer that sizes its work by the slot capacity."""
    if hot < k or hot > experts:
        raise ValueError("need k <= hot <= experts")
    ids = np.stack([rng.permutation(hot)[:k] for _ in range(tokens)]).astype(np.int32)
    logits = rng.standard_normal((tokens, k)).astype(np.float32)
    e = np.exp(logits - logits.max(1, keepdims=True))
    return ids, (e / e.sum(1, keepdims=True)).astype(np.float32)


def device_mxfp4_linear(ctx, gen, n: int, k: int, sigma: float = 0.02):
    """W ~ N(0, sigma) drawn on the device and quantized to MXFP4 by the provider's FP4
    packer (the reference's only FP4 recipe, encoding.rs:249-284); row-major handle."""
    import torch

    from .provider import HipArtifactLinearHandle
    from .provider import HipArtifactLinearShape as S

    w = torch.randn((n, k), generator=gen, device="cuda", dtype=torch.float32) * sigma
    packed, scales = ctx.pack_fp4_rows_from_f32(w)
    return HipArtifactLinearHandle(S.fp4_e2m1_packed_with_e8m0_scale(n, k), packed.reshape(-1), scales.reshape(-1))


def device_fp8_linear(ctx, gen, n: int, k: int, scale_kind: str = "f32", sigma: float = 0.02):
    """W ~ N(0, sigma) drawn on the device, e4m3 per 128x128 tile with an fp32 scale amax/448
    (``f32``) or the power of two 2^ceil(log2(amax/448)) as an E8M0 byte (``e8m0``)."""
    import torch

    from .provider import HipArtifactLinearHandle
    from .provider import HipArtifactLinearShape as S

    if n % 128 or k % 128:
        raise ValueError("device_fp8_linear draws whole 128x128 tiles")
    w = torch.randn((n, k), generator=gen, device="cuda", dtype=torch.float32) * sigma
    tiles = w.reshape(n // 128, 128, k // 128, 128)
    amax = tiles.abs().amax(dim=(1, 3)).clamp_min(1e-12)
    if scale_kind == "f32":
        scales = (amax / 448.0).contiguous()
        shape = S.fp8_e4m3_with_f32_scale(n, k)
        stored = scales
    else:
        exponent = torch.ceil(torch.log2(amax.clamp_min(1e-4) / 448.0))
        scales = torch.exp2(exponent)
        stored = (exponent + 127.0).clamp(0, 254).to(torch.uint8).contiguous()
        shape = S.fp8_e4m3_with_e8m0_scale(n, k)
    q = (tiles / scales[:, None, :, None]).clamp(-448, 448).reshape(n, k)
    packed = q.to(torch.float8_e4m3fn).view(torch.uint8)
    return HipArtifactLinearHandle(shape, packed.reshape(-1), stored.reshape(-1))


def build_device_experts(ctx, experts: int, hidden: int, inter: int, seed: int, sigma: float = 0.02):
    """``experts`` routed MXFP4 experts (gate, up [inter, hidden]; down [hidden, inter]) drawn and
    quantized on the device, installed row-major in a fresh slot table.  Returns (table, handles)."""
    import torch

    from .provider import HipRoutedExpertTable

    gen = torch.Generator(device="cuda").manual_seed(seed)
    table = HipRoutedExpertTable(experts, ctx.device)
    handles = []
    for e in range(experts):
        trio = [device_mxfp4_linear(ctx, gen, n, k, sigma) for n, k in ((inter, hidden), (inter, hidden), (hidden, inter))]
        table.install(e, *trio)
        handles.append(trio)
    table.commit()
    return table, handles


def block_major_table(ctx, handles):
    """The same experts in the block-major order (the one-off preparation an expert gets when it
    is installed in a slot), as a second table."""
    from .provider import HipRoutedExpertTable

    table = HipRoutedExpertTable(len(handles), ctx.device)
    for e, trio in enumerate(handles):
        table.install(e, *(ctx.prepare_mxfp4_block_major(h) for h in trio))
    table.commit()
    return table


def host_expert(trio):
    """Device handles of one expert -> [(weight [n, k/2] u8, scales [n, k/32] u8)] * 3 on the host."""
    return [(h.weight.cpu().numpy().reshape(h.shape.out_features, -1),
             h.scale.cpu().numpy().reshape(h.shape.out_features, -1)) for h in trio]
