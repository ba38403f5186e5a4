"""Device router (ferrule_hip_core_router_launch) against the CPU checker, through the C ABI.

Bar: ids bit-exact wherever the arithmetic is exact (plain top-k, hash routing, ties); for the
sqrt-softplus score router the device's expf/log1pf may differ from the host's in the last ulps,
so ids must be the checker's unless the two selection values involved are closer than
``SCORE_ULPS`` ulp, and weights must be within ``WEIGHT_ULPS`` ulp of the checker's."""
import numpy as np
import pytest
import torch

from oracle import pyoracle as po
from tests import helpers as H
from tests.test_router_oracle import (HASH_EXPECTED, HASH_LOGITS, HASH_TABLE, HASH_TOKENS, TOPK_BIAS, TOPK_LOGITS,
                                      f64_scores)

pytestmark = pytest.mark.gpu

from oracle.parity import SCORE_ULPS, WEIGHT_ULPS  # noqa: E402


@pytest.fixture(scope="module")
def ctx():
    from ferrule_amd.provider import HipArtifactOperatorContext

    return HipArtifactOperatorContext(0)


def _dev(a, dtype):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dtype).cuda()


def _topk(ctx, logits, k, scale, bias=None, fill=None):
    rows, experts = logits.shape
    idx = torch.full((rows, k), -7 if fill is None else fill, dtype=torch.int32, device="cuda")
    w = torch.full((rows, k), -7.0, dtype=torch.float32, device="cuda")
    ctx.dsv4_router_topk_sqrt_softplus_rows_from_device_into(
        _dev(logits, torch.float32), None if bias is None else _dev(bias, torch.float32), rows, experts, k, scale, idx, w)
    ctx.synchronize()
    return idx.cpu().numpy(), w.cpu().numpy()


def _raw(ctx, kind, logits, k, **kw):
    """Straight through the C ABI, for shapes the host wrappers refuse."""
    from ferrule_amd import abi

    rows, columns = logits.shape
    lg = _dev(logits, torch.float32)
    idx = torch.full((rows, k), 9, dtype=torch.float32 if kind == abi.VOCAB_TOPK_F32_INDEX else torch.int32,
                     device="cuda")
    w = torch.full((rows, k), 9.0, dtype=torch.float32, device="cuda")
    a = abi.RouterArgs(kind=kind, rows=rows, columns=columns, k=k, route_scale=kw.get("scale", 1.0),
                       logits=lg.data_ptr(), indices=idx.data_ptr(), weights=w.data_ptr())
    ctx._core("router", ctx.lib.ferrule_hip_core_router_launch, a)
    ctx.synchronize()
    return idx.cpu().numpy(), w.cpu().numpy()


def test_reference_topk_case(ctx):
    # dsv4_decode_topk_boundary.rs:629-690
    idx, w = _topk(ctx, TOPK_LOGITS, 3, 1.25, TOPK_BIAS)
    want_idx, want_w = po.router_kernel_rows(1, TOPK_LOGITS, 3, 1.25, bias=TOPK_BIAS)
    assert idx.tolist() == want_idx.tolist() == [[4, 2, 1], [3, 0, 4]]
    assert np.all(np.abs(w - want_w) <= 1.0e-4)          # the reference's tolerance
    assert np.all(np.abs(w - want_w) <= WEIGHT_ULPS * np.spacing(want_w))


def test_reference_hash_case_and_token_id_update(ctx):
    # dsv4_decode_topk_boundary.rs:732-855
    table = ctx.upload_dsv4_router_hash_table(HASH_TABLE.ravel().tolist(), 5, 3, 4, 2)
    tokens = ctx.dsv4_router_token_ids(HASH_TOKENS, 5)
    idx = torch.zeros((3, 2), dtype=torch.int32, device="cuda")
    w = torch.zeros((3, 2), dtype=torch.float32, device="cuda")
    launches = ctx.kernel_launches
    ctx.dsv4_router_hash_sqrt_softplus_rows_from_device_into(_dev(HASH_LOGITS, torch.float32), tokens, table, 3, 4, 2,
                                                             1.5, idx, w)
    assert ctx.kernel_launches == launches + 1
    ctx.synchronize()
    assert idx.cpu().numpy().tolist() == HASH_EXPECTED
    for row in range(3):
        sc = f64_scores(HASH_LOGITS[row, HASH_EXPECTED[row]])
        assert np.all(np.abs(w[row].cpu().numpy() - sc / sc.sum() * 1.5) <= 1.0e-4)
    # other token ids, same buffers
    tokens.copy_(ctx.dsv4_router_token_ids([3, 0, 4], 5))
    ctx.dsv4_router_hash_sqrt_softplus_rows_from_device_into(_dev(HASH_LOGITS, torch.float32), tokens, table, 3, 4, 2,
                                                             1.5, idx, w)
    ctx.synchronize()
    want_idx, want_w = po.router_kernel_rows(2, HASH_LOGITS, 2, 1.5, token_ids=[3, 0, 4], hash_table=HASH_TABLE)
    assert idx.cpu().numpy().tolist() == want_idx.tolist()
    assert np.all(np.abs(w.cpu().numpy() - want_w) <= WEIGHT_ULPS * np.spacing(want_w))


@pytest.mark.parametrize("rows,columns,k", [(5, 3, 1), (9, 64, 8), (7, 65, 40), (33, 150, 40), (64, 256, 8),
                                            (16, 512, 64), (6, 513, 8), (3, 1000, 40), (2, 129280, 4)])
def test_plain_topk_is_bit_exact_with_heavy_ties(ctx, rows, columns, k):
    from ferrule_amd import abi

    rng = H.rng_for(6, rows * 1000 + columns)
    logits = rng.integers(-6, 7, (rows, columns)).astype(np.float32) * 0.5
    logits[0, columns // 2] = -0.0
    logits[0, 0] = 0.0
    logits[rows - 1, :] = 1.25                           # a row of equal values: ids 0..k-1
    if k <= columns and k <= 40:
        idx = torch.zeros((rows, k), dtype=torch.int32, device="cuda")
        val = torch.zeros((rows, k), dtype=torch.float32, device="cuda")
        ctx.topk_vocab_rows_from_device_into(_dev(logits, torch.float32), rows, columns, k, idx, val)
        ctx.synchronize()
        idx, val = idx.cpu().numpy(), val.cpu().numpy()
    else:
        idx, val = _raw(ctx, abi.VOCAB_TOPK_I32_INDEX, logits, k)
    want_idx, want_val = po.router_kernel_rows(4, logits, k)
    assert np.array_equal(idx, want_idx)
    assert np.array_equal(val.view(np.uint32), want_val.view(np.uint32))
    idx_f, val_f = _raw(ctx, abi.VOCAB_TOPK_F32_INDEX, logits, k)
    assert np.array_equal(idx_f, want_idx.astype(np.float32)) and np.array_equal(val_f, want_val)


def test_more_slots_than_columns_and_non_finite_values(ctx):
    from ferrule_amd import abi

    logits = np.array([[0.0, 1.0, -1.0], [np.inf, -np.inf, 2.0]], np.float32)
    idx, val = _raw(ctx, abi.VOCAB_TOPK_I32_INDEX, logits, 5)
    want_idx, want_val = po.router_kernel_rows(4, logits, 5)
    assert idx.tolist() == want_idx.tolist() == [[1, 0, 2, -1, -1], [0, 2, 1, -1, -1]]
    assert np.array_equal(val, want_val)
    idx, w = _raw(ctx, abi.ROUTER_TOPK, logits[:1], 5)
    want_idx, want_w = po.router_kernel_rows(1, logits[:1], 5)
    assert idx.tolist() == want_idx.tolist() and np.all(np.abs(w - want_w) <= WEIGHT_ULPS * np.spacing(want_w))
    assert w[0, 3] == 0.0 and w[0, 4] == 0.0
    # an infinite score makes the sum infinite: every weight is 0, ids still ranked
    idx, w = _raw(ctx, abi.ROUTER_TOPK, logits[1:], 2)
    assert idx.tolist() == [[0, 2]] and w.tolist() == [[0.0, 0.0]]
    # k outside 1..64 is a successful no-op
    idx, w = _raw(ctx, abi.VOCAB_TOPK_I32_INDEX, logits, 65)
    assert (idx == 9).all() and (w == 9.0).all()


_check_score_router = H.check_score_router


@pytest.mark.parametrize("rows,experts,k,with_bias", [(64, 256, 8, True), (64, 256, 8, False), (8192, 256, 8, True),
                                                      (1, 256, 6, True), (301, 64, 6, False), (130, 384, 64, True),
                                                      (50, 512, 8, True), (19, 100, 3, True)])
def test_score_router_matches_the_checker(ctx, rows, experts, k, with_bias):
    rng = H.rng_for(7, rows * 7 + experts)
    logits = rng.normal(0.0, 2.5, (rows, experts)).astype(np.float32)
    logits[0, : experts // 2] = logits[0, 0]                       # exact ties: lower id first
    if rows > 2:
        logits[1, :k] = 21.0 + np.arange(k)                        # identity branch of softplus
        logits[2, k:] = -25.0 - (np.arange(experts - k) % 60)      # exp branch, scores near 1e-6
    bias = rng.normal(0.0, 0.25, experts).astype(np.float32) if with_bias else None
    idx, w = _topk(ctx, logits, k, 2.5, bias)
    _check_score_router(logits, bias, k, 2.5, idx, w)
    if not with_bias:
        assert idx[0].tolist()[:1] == [int(np.argmax(logits[0]))] or logits[0].max() == logits[0, 0]


def test_hash_router_rows_and_untouched_rows(ctx):
    from ferrule_amd import abi

    rng = H.rng_for(8)
    rows, experts, k, hash_rows, hash_cols = 4096, 256, 6, 1000, 8
    logits = rng.normal(0.0, 2.5, (rows, experts)).astype(np.float32)
    table = np.stack([rng.permutation(experts)[:hash_cols] for _ in range(hash_rows)]).astype(np.int32)
    token_ids = rng.integers(0, hash_rows, rows).astype(np.int32)
    dtab = ctx.upload_dsv4_router_hash_table(table.ravel().tolist(), hash_rows, hash_cols, experts, k)
    idx = torch.full((rows, k), 77, dtype=torch.int32, device="cuda")
    w = torch.full((rows, k), 0.5, dtype=torch.float32, device="cuda")
    ctx.dsv4_router_hash_sqrt_softplus_rows_from_device_into(
        _dev(logits, torch.float32), ctx.dsv4_router_token_ids(token_ids.tolist(), hash_rows), dtab, rows, experts, k,
        1.5, idx, w)
    ctx.synchronize()
    want_idx, want_w = po.router_kernel_rows(2, logits, k, 1.5, token_ids=token_ids, hash_table=table)
    assert np.array_equal(idx.cpu().numpy(), want_idx)
    assert np.all(np.abs(w.cpu().numpy() - want_w) <= WEIGHT_ULPS * np.spacing(want_w))
    # what host validation would have refused: the kernel leaves such rows as they were
    bad_tokens = token_ids.copy()
    bad_tokens[5] = hash_rows
    bad_tokens[6] = -1
    bad_table = table.copy()
    bad_table[bad_tokens[9], k - 1] = experts
    idx.fill_(77)
    w.fill_(0.5)
    a = abi.RouterArgs(kind=abi.ROUTER_HASH, rows=rows, columns=experts, k=k, hash_rows=hash_rows,
                       hash_columns=hash_cols, route_scale=1.5, logits=_dev(logits, torch.float32).data_ptr(),
                       token_ids=_dev(bad_tokens, torch.int32).data_ptr(),
                       hash_table=_dev(bad_table, torch.int32).data_ptr(), indices=idx.data_ptr(), weights=w.data_ptr())
    keep = (_dev(logits, torch.float32), _dev(bad_tokens, torch.int32), _dev(bad_table, torch.int32))
    a.logits, a.token_ids, a.hash_table = (t.data_ptr() for t in keep)
    ctx._core("hash router", ctx.lib.ferrule_hip_core_router_launch, a)
    ctx.synchronize()
    want_idx, want_w = po.router_kernel_rows(2, logits, k, 1.5, token_ids=bad_tokens, hash_table=bad_table,
                                             indices=np.full((rows, k), 77, np.int32),
                                             weights=np.full((rows, k), 0.5, np.float32))
    got_idx = idx.cpu().numpy()
    assert np.array_equal(got_idx, want_idx)
    untouched = np.flatnonzero((got_idx == 77).all(axis=1))
    assert {5, 6, 9} <= set(untouched.tolist())
    assert np.all(np.abs(w.cpu().numpy() - want_w) <= WEIGHT_ULPS * np.spacing(want_w))


def test_host_wrappers_refuse_what_the_reference_refuses(ctx):
    lg = torch.zeros((2, 600), dtype=torch.float32, device="cuda")
    idx = torch.zeros((2, 8), dtype=torch.int32, device="cuda")
    w = torch.zeros((2, 8), dtype=torch.float32, device="cuda")
    with pytest.raises(ValueError, match="at most 512 experts"):
        ctx.dsv4_router_topk_sqrt_softplus_rows_from_device_into(lg, None, 2, 600, 8, 1.0, idx, w)
    with pytest.raises(ValueError, match="top_k"):
        ctx.dsv4_router_topk_sqrt_softplus_rows_from_device_into(lg[:, :4].contiguous(), None, 2, 4, 8, 1.0, idx, w)
    with pytest.raises(ValueError, match="output mismatch"):
        ctx.dsv4_router_topk_sqrt_softplus_rows_from_device_into(lg[:, :16].contiguous(), None, 2, 16, 4, 1.0, idx, w)
    with pytest.raises(ValueError, match="bias length"):
        ctx.dsv4_router_topk_sqrt_softplus_rows_from_device_into(lg[:, :16].contiguous(), lg[0, :8].contiguous(), 2, 16,
                                                                 8, 1.0, idx, w)
    with pytest.raises(ValueError, match="k in 1"):
        ctx.topk_vocab_rows_from_device_into(lg, 2, 600, 41, idx, w)


def test_router_feeds_the_decode_layer_without_leaving_the_device(ctx):
    """logits -> router -> fused decode plan -> MoE decode layer, every hand-over a device buffer;
    the result equals the layer run on the checker's routes."""
    from tests.test_moe_gpu import _make_experts, _oracle_moe

    tokens, k, experts, hidden, inter = 6, 2, 8, 512, 256
    rng = H.rng_for(9)
    table, host = _make_experts(ctx, rng, experts, hidden, inter, sigma=0.05)
    x = H.bf16_activations(rng, (tokens, hidden))
    logits = rng.normal(0.0, 2.0, (tokens, experts)).astype(np.float32)
    bias = rng.normal(0.0, 0.2, experts).astype(np.float32)

    idx = torch.zeros((tokens, k), dtype=torch.int32, device="cuda")
    w = torch.zeros((tokens, k), dtype=torch.float32, device="cuda")
    ctx.dsv4_router_topk_sqrt_softplus_rows_from_device_into(_dev(logits, torch.float32), _dev(bias, torch.float32),
                                                             tokens, experts, k, 1.5, idx, w)
    plan = ctx.expert_group_route_plan(table.slot_capacity, tokens * k, tokens, hidden, inter, hidden)
    generations = torch.ones(tokens * k, dtype=torch.int32, device="cuda")
    ctx.prepare_decode_route_plan(plan, table, idx.view(-1), generations, w.view(-1), k)
    out = torch.empty((tokens, hidden), dtype=torch.bfloat16, device="cuda")
    ctx.moe_decode_from_prepared_plan(plan, table, torch.from_numpy(x).to(torch.bfloat16).cuda(), out, None, 0.0)
    ctx.synchronize()

    want_idx, want_w = po.router_kernel_rows(1, logits, k, 1.5, bias=bias)
    assert np.array_equal(idx.cpu().numpy(), want_idx)
    got_w = w.cpu().numpy()
    assert np.all(np.abs(got_w - want_w) <= WEIGHT_ULPS * np.spacing(want_w))
    # the layer is linear in a route's weight: run the checker on the device's weights
    want, bound, _, _ = _oracle_moe(host, x, want_idx, got_w, hidden, inter)
    worst, _, _ = H.compare_bf16_bounded(out.view(torch.int16).cpu().numpy().view(np.uint16), want, bound,
                                         max_decided_fraction=0.005)
    assert worst <= 2
    assert plan.route_error.item() == 0
