"""Grouped MXFP4 MoE over packed FP8 rows (prefill / verification) against the CPU executor with
FP8-K128 activation quantisation (crates/ferrule-model/src/moe/executor.rs:82-124; GPU only).

Parity is checked stage by stage so that the discontinuous quantiser cannot hide or amplify
anything: (1) the unquantised hidden activations against the executor's, (2) the quantised
bytes and scales bit-exactly against the CPU quantiser applied to the device's own hidden
values, (3) route outputs against the CPU down projection of those bytes, (4) the combined
BF16 output against the whole CPU chain."""
import numpy as np
import pytest
import torch

from oracle import pyoracle as po
from tests import helpers as H
from ferrule_amd.synthetic import build_device_experts
from tests.test_moe_gpu import _f32, _i32, _make_experts, _routing

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from ferrule_amd.provider import HipArtifactOperatorContext

    return HipArtifactOperatorContext(0)


def _plan_and_run(ctx, table, x, ids, weights, hidden, inter, limit=0.0, debug=False, clear_output=True):
    tokens, k = ids.shape
    plan = ctx.expert_group_route_plan(table.slot_capacity, tokens * k, tokens, hidden, inter, hidden)
    if not clear_output:
        plan.route_output.fill_(float("nan"))
    ctx.begin_expert_group_route_invocation(plan, tokens * k, clear_output=clear_output)
    ctx.prepare_expert_group_route_plan(plan, table, _i32(ids.ravel()), _i32(np.ones(tokens * k)),
                                        _f32(weights.ravel()), k)
    xq, xs = ctx.pack_fp8_rows_from_f32(torch.from_numpy(np.ascontiguousarray(x, np.float32)).cuda())
    meta = plan.host_metadata()
    dbg = torch.zeros((meta["total_routed_rows"], inter), dtype=torch.float32, device="cuda") if debug else None
    ctx.grouped_fp4_moe_from_prepared_plan(plan, table, xq, xs, limit, meta=meta, debug_hidden=dbg)
    return plan, meta, dbg


def _combine(ctx, plan, tokens, k, hidden):
    out = torch.zeros((tokens, hidden), dtype=torch.float32, device="cuda")
    ctx.reduce_moe_route_outputs_ranked(plan.route_output, tokens, k, hidden, out, plan.route_written,
                                        plan.route_error)
    return out.cpu().numpy()


def test_closed_form_groups_gather_scatter_and_reduce(ctx):
    # the shape of moe_grouped_smoke.rs:116-333: x = 1, W1 = W3 = +1 (nibbles 0x22), W2 = +1 or +2,
    # all scales 127, H = I = 128, 64 outputs, weight 1/1024: gate = up = 128, h = 128*128/1024 = 16
    # (exact in E4M3 with the block scale 2^-4), route value 128*16*{1,2} = {2048, 4096}
    from ferrule_amd.provider import HipArtifactLinearShape as S
    from ferrule_amd.provider import HipRoutedExpertTable

    hidden_in, inter, out_features, experts, tokens, k = 128, 128, 64, 4, 6, 2
    table = HipRoutedExpertTable(experts, ctx.device)
    for e in range(experts):
        w13 = np.full((inter, hidden_in // 2), 0x22, np.uint8)
        w2 = np.full((out_features, inter // 2), 0x22 if e % 2 == 0 else 0x44, np.uint8)
        s13 = np.full((inter, hidden_in // 32), 127, np.uint8)
        s2 = np.full((out_features, inter // 32), 127, np.uint8)
        up = lambda n, kk, w, s: ctx.upload_artifact_linear(S.fp4_e2m1_packed_with_e8m0_scale(n, kk), w, s)
        table.install(e, up(inter, hidden_in, w13, s13), up(inter, hidden_in, w13, s13),
                      up(out_features, inter, w2, s2), generation=1)
    table.commit()
    ids = np.array([[0, 1], [1, 2], [3, 0], [2, 2 ^ 1], [0, 2], [1, 3]], np.int32)
    weights = np.full((tokens, k), 1.0 / 1024.0, np.float32)
    plan = ctx.expert_group_route_plan(experts, tokens * k, tokens, hidden_in, inter, out_features)
    ctx.begin_expert_group_route_invocation(plan, tokens * k)
    ctx.prepare_expert_group_route_plan(plan, table, _i32(ids.ravel()), _i32(np.ones(tokens * k)),
                                        _f32(weights.ravel()), k)
    xq = torch.full((tokens, hidden_in), 0x38, dtype=torch.uint8, device="cuda")
    xs = torch.full((tokens, 1), 127, dtype=torch.uint8, device="cuda")
    ctx.grouped_fp4_moe_from_prepared_plan(plan, table, xq, xs)
    routes = plan.route_output.cpu().numpy()[:tokens * k]
    want = np.where(ids.ravel() % 2 == 0, 2048.0, 4096.0)
    assert (routes == want[:, None]).all()
    assert (plan.route_written.cpu().numpy()[:tokens * k] == 1).all() and int(plan.route_error.item()) == 0
    out = torch.full((tokens, out_features), 1.5, dtype=torch.float32, device="cuda")     # prefix
    ctx.reduce_moe_route_outputs_ranked(plan.route_output, tokens, k, out_features, out, plan.route_written,
                                        plan.route_error)
    per_token = want.reshape(tokens, k).sum(1) + 1.5
    assert np.array_equal(out.cpu().numpy(), np.repeat(po.round_to_bf16_array(per_token.astype(np.float32))[:, None],
                                                       out_features, 1))


@pytest.mark.parametrize("tokens,k,experts,hidden,inter,limit", [
    (7, 2, 4, 256, 128, 0.0),
    (150, 2, 3, 512, 256, 0.0),      # groups larger than one 128-row tile
    (33, 3, 5, 384, 640, 0.05),      # clamp; feature tiles that end inside a workgroup tile
    # K extents of six and more 128-blocks: the persistent kernels with chained K loops
    (150, 2, 3, 1024, 1024, 0.0),    # both GEMMs; several items per workgroup only with more tiles (below)
    (33, 3, 5, 768, 640, 0.05),      # gate/up persistent with a partial feature tile, down one item per workgroup
    (40, 2, 4, 768, 1024, 0.0),      # down persistent with a partial feature tile (hidden 768 = 512 + 256)
])
def test_grouped_moe_matches_cpu_executor_stage_by_stage(ctx, tokens, k, experts, hidden, inter, limit):
    rng = H.rng_for(5, tokens * 31 + inter)
    table, host = _make_experts(ctx, rng, experts, hidden, inter, sigma=0.05)
    x = H.bf16_activations(rng, (tokens, hidden)).astype(np.float32)
    ids, weights = _routing(rng, tokens, k, experts)
    _check_stage_by_stage(ctx, table, host, x, ids, weights, hidden, inter, limit)


@pytest.mark.parametrize("hidden,inter", [(256, 128), (768, 1024)])
def test_ragged_tiles_with_every_count_of_live_token_fragments(ctx, hidden, inter):
    """A 128-row tile is eight 16-row fragments; the kernels skip the dead ones of an expert's last
    tile, with a K loop of its own per live count and wave.  One expert per row count: 1..8 live
    fragments, counts on both sides of every fragment edge, and experts of more than one tile.  The
    second shape runs the persistent kernels, where a workgroup's consecutive items differ in it."""
    counts = [1, 15, 16, 17, 32, 33, 47, 48, 49, 64, 65, 80, 81, 97, 112, 113, 127, 128, 129, 145, 300]
    if hidden > 256:
        counts = [1, 16, 17, 33, 48, 65, 81, 112, 113, 129]      # every live count once (CPU time of the larger shape)
    k = 1
    rng = H.rng_for(5, 4242 + hidden)
    table, host = _make_experts(ctx, rng, len(counts), hidden, inter, sigma=0.05)
    ids = rng.permutation(np.repeat(np.arange(len(counts), dtype=np.int32), counts))[:, None]
    tokens = ids.shape[0]
    x = H.bf16_activations(rng, (tokens, hidden)).astype(np.float32)
    weights = rng.uniform(0.05, 1.0, (tokens, k)).astype(np.float32)
    _check_stage_by_stage(ctx, table, host, x, ids, weights, hidden, inter, 0.0)


def test_persistent_workgroups_take_several_items_each(ctx):
    """More items than the 256 persistent workgroups in both GEMMs (100 experts of a few rows each: 100 token
    tiles x 4 and x 3 feature tiles), so that a workgroup chains K loops of different experts, row counts and
    feature tiles; every stage against the CPU executor."""
    experts, hidden, inter, k = 100, 1536, 1024, 1
    rng = H.rng_for(5, 777)
    table, host = _make_experts(ctx, rng, experts, hidden, inter, sigma=0.05)
    counts = rng.integers(1, 4, experts)
    ids = rng.permutation(np.repeat(np.arange(experts, dtype=np.int32), counts))[:, None]
    tokens = ids.shape[0]
    x = H.bf16_activations(rng, (tokens, hidden)).astype(np.float32)
    weights = rng.uniform(0.05, 1.0, (tokens, k)).astype(np.float32)
    _check_stage_by_stage(ctx, table, host, x, ids, weights, hidden, inter, 0.0)


def _check_stage_by_stage(ctx, table, host, x, ids, weights, hidden, inter, limit):
    tokens, k = ids.shape
    plan, meta, dbg = _plan_and_run(ctx, table, x, ids, weights, hidden, inter, limit, debug=True)
    assert int(plan.route_error.item()) == 0
    rows = meta["total_routed_rows"]
    assert rows == tokens * k
    h_gpu = dbg.cpu().numpy()
    route_of_row = plan.route_indices.cpu().numpy()[:rows]
    token_of_row = plan.route_token_indices.cpu().numpy()[:rows]
    hq, hs = (t.cpu().numpy() for t in ctx.grouped_workspace_views(plan, meta))
    routes_gpu = plan.route_output.cpu().numpy()
    xq = po.simulate_fp8_act_quant(x, hidden, 128)          # what the packed rows decode to
    # (2) quantiser: bit-exact on the device's own hidden values
    want_q, want_s = po.pack_fp8_act(h_gpu, inter, 128)
    assert np.array_equal(hs, want_s.reshape(rows, -1))
    assert np.array_equal(hq, want_q.reshape(rows, inter))
    hq_values = po.simulate_fp8_act_quant(h_gpu, inter, 128)
    worst_h, worst_y = 0.0, 0.0
    for row in range(rows):
        route, token = int(route_of_row[row]), int(token_of_row[row])
        assert route // k == token
        e = int(ids.ravel()[route])
        (gw, gs, _), (uw, us, _), (dw, ds, _) = host[e]
        # (1) hidden activations before quantisation: the executor on the dequantised input, no act-quant
        _, h_ref = po.expert_execute_fp4(gw, gs, uw, us, dw, ds, hidden, inter, xq[token],
                                         float(weights.ravel()[route]), limit, return_hidden=True)
        # forward error of h = silu(g) * u * w for errors dg, du of the two dot products (|silu'| <= 1.1,
        # |silu(g)| <= |g|), each within (K 2^-24 + 2^-14) of its sum of |products| (see (3) below)
        xr = xq[token].astype(np.float64)
        gate = po.linear_fp4(gw, gs, inter, hidden, xq[token])[0].astype(np.float64)
        up = po.linear_fp4(uw, us, inter, hidden, xq[token])[0].astype(np.float64)
        eps = hidden * 2.0 ** -24 + 2.0 ** -14
        dg = eps * (np.abs(po.dequantize_fp4(gw, gs, inter, hidden).astype(np.float64)) @ np.abs(xr))
        du = eps * (np.abs(po.dequantize_fp4(uw, us, inter, hidden).astype(np.float64)) @ np.abs(xr))
        if limit > 0:
            gate, up = np.minimum(gate, limit), np.clip(up, -limit, limit)
        bound_h = float(weights.ravel()[route]) * (1.1 * np.abs(up) * dg + np.abs(gate) * du + dg * du) \
            + np.abs(h_ref) * 2.0 ** -21
        worst_h = max(worst_h, float((np.abs(h_gpu[row] - h_ref) / (bound_h + 1e-30)).max()))
        # (3) down projection of the device's own quantised hidden row
        y_ref = po.linear_fp4(dw, ds, hidden, inter, hq_values[row])[0]
        absprod = np.abs(po.dequantize_fp4(dw, ds, hidden, inter).astype(np.float64)) @ np.abs(
            hq_values[row].astype(np.float64))
        err = np.abs(routes_gpu[route].astype(np.float64) - y_ref)
        # fp32 summation in any order, plus the scaled MFMA's own 128-term reduction: the instruction
        # aligns the products of one K block to the largest and keeps about 21 bits below it; measured,
        # one instruction is within 2^-14.6 of the sum of |products| (the error averages out over the K
        # blocks: 2^-17.3 at K = 2048).  The oracle's sequential fp32 sum is inside the first term.
        assert (err <= (inter * 2.0 ** -24 + 2.0 ** -14) * absprod + 1e-30).all()
        worst_y = max(worst_y, float((err / (absprod + 1e-30)).max()))
    assert worst_h <= 1.0, worst_h
    # (4) whole chain through the ranked combine: equal to the CPU chain up to the exactly known effect
    # of quantiser codes that differ because h differs in the last fp32 bits
    got = _combine(ctx, plan, tokens, k, hidden)
    row_of_route = np.empty(rows, np.int64)
    row_of_route[route_of_row] = np.arange(rows)
    want = np.zeros((tokens, hidden), np.float32)
    delta = np.zeros((tokens, hidden), np.float64)
    absdown = np.zeros((tokens, hidden), np.float64)
    for t in range(tokens):
        ys = []
        for j in range(k):
            (gw, gs, _), (uw, us, _), (dw, ds, _) = host[ids[t, j]]
            y, h = po.expert_execute_fp4(gw, gs, uw, us, dw, ds, hidden, inter, x[t], float(weights[t, j]), limit,
                                         act_quant_block=128, return_hidden=True)
            ys.append(y)
            wd = po.dequantize_fp4(dw, ds, hidden, inter).astype(np.float64)
            hq_gpu = hq_values[row_of_route[t * k + j]].astype(np.float64)
            delta[t] += wd @ (hq_gpu - h.astype(np.float64))
            absdown[t] += np.abs(wd) @ np.abs(hq_gpu)
        want[t] = po.accumulate_routes(np.stack(ys))
    # the combine rounds to BF16
    H.quantised_chain_check(got, po.round_to_bf16_array(want), delta, absdown, inter, min_fraction=0.97,
                            output_rounding=2.0 ** -8)


@pytest.mark.parametrize("tokens,k,experts,hidden,inter,limit", [
    (7, 2, 4, 256, 128, 0.0),
    (150, 2, 3, 512, 256, 0.0),
    (33, 3, 5, 384, 640, 0.05),
    (300, 4, 6, 1024, 512, 0.0),
    (96, 6, 8, 4096, 2048, 10.0),    # DeepSeek-V4 Flash: hidden 4096, routed intermediate 2048, top-6
])
def test_one_prepared_copy_serves_prefill_and_decode(ctx, tokens, k, experts, hidden, inter, limit):
    """The grouped GEMM reads the block-major copy the decode layer prefers: same products in the same
    order as from the checkpoint order (checked stage by stage against the CPU above), so not one bit of
    route_output, of the quantised hidden rows or of the combined output may differ."""
    from ferrule_amd import synthetic

    rng = H.rng_for(5, tokens * 17 + inter)
    table, host = _make_experts(ctx, rng, experts, hidden, inter, sigma=0.05)
    prepared = synthetic.block_major_table(ctx, [[m[2] for m in mats] for mats in host])
    assert prepared.block_major and not table.block_major
    x = H.bf16_activations(rng, (tokens, hidden)).astype(np.float32)
    ids, weights = _routing(rng, tokens, k, experts)
    plan, meta, _ = _plan_and_run(ctx, table, x, ids, weights, hidden, inter, limit)
    plan_bm, meta_bm, _ = _plan_and_run(ctx, prepared, x, ids, weights, hidden, inter, limit)
    assert meta == meta_bm and int(plan_bm.route_error.item()) == 0
    rows = meta["total_routed_rows"]
    assert torch.equal(plan.route_output[:tokens * k].view(torch.int32), plan_bm.route_output[:tokens * k].view(torch.int32))
    for a, b in zip(ctx.grouped_workspace_views(plan, meta), ctx.grouped_workspace_views(plan_bm, meta_bm)):
        assert torch.equal(a[:rows], b[:rows])
    assert np.array_equal(_combine(ctx, plan, tokens, k, hidden).view(np.uint32),
                          _combine(ctx, plan_bm, tokens, k, hidden).view(np.uint32))
    # and the very same table runs the decode layer
    out = torch.empty((tokens, hidden), dtype=torch.bfloat16, device="cuda")
    if tokens * k <= 2048:
        dplan = ctx.expert_group_route_plan(experts, tokens * k, tokens, hidden, inter, hidden)
        ctx.prepare_decode_route_plan(dplan, prepared, _i32(ids.ravel()), _i32(np.ones(tokens * k)), _f32(weights.ravel()), k)
        if hidden % 512 == 0 and inter % 256 == 0:
            ctx.moe_decode_from_prepared_plan(dplan, prepared, torch.from_numpy(x).to(torch.bfloat16).cuda(), out, None, limit)
            ctx.synchronize()
            assert int(dplan.route_error.item()) == 0 and bool(torch.isfinite(out.float()).all())


def test_unresolved_and_empty_groups(ctx):
    rng = H.rng_for(5, 77)
    tokens, k, experts, hidden, inter = 9, 2, 6, 256, 128
    table, host = _make_experts(ctx, rng, experts, hidden, inter, sigma=0.05)
    table.evict(4)
    table.commit()
    x = H.bf16_activations(rng, (tokens, hidden)).astype(np.float32)
    ids, weights = _routing(rng, tokens, k, experts)
    ids[0, 0] = 4                      # evicted expert: that route stays unwritten
    plan, meta, _ = _plan_and_run(ctx, table, x, ids, weights, hidden, inter)
    out = _combine(ctx, plan, tokens, k, hidden)
    assert np.isnan(out[0]).all()
    touched = (ids == 4).any(1)
    assert np.isfinite(out[~touched]).all()


def test_flags_only_invocation_reset_is_enough_for_the_grouped_chain(ctx):
    """With route_output left dirty (NaN everywhere) the combined result is the same: the down GEMM
    writes every live row in full and the checked reducer never reads an unwritten one."""
    rng = H.rng_for(5, 78)
    tokens, k, experts, hidden, inter = 150, 3, 6, 256, 128
    table, host = _make_experts(ctx, rng, experts, hidden, inter, sigma=0.05)
    table.evict(2)
    table.commit()
    x = H.bf16_activations(rng, (tokens, hidden)).astype(np.float32)
    ids, weights = _routing(rng, tokens, k, experts)
    plan, _, _ = _plan_and_run(ctx, table, x, ids, weights, hidden, inter)
    want = _combine(ctx, plan, tokens, k, hidden)
    plan2, _, _ = _plan_and_run(ctx, table, x, ids, weights, hidden, inter, clear_output=False)
    got = _combine(ctx, plan2, tokens, k, hidden)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.isnan(got[(ids == 2).any(1)]).all() and np.isfinite(got[~(ids == 2).any(1)]).all()


def test_config5_moe_prefill_8192_tokens_256_experts_zipf(ctx):
    # configs[4]: 8192 tokens, 256 MXFP4 experts (gate/up [2048,7168] x2, down [7168,2048]), top-8 with
    # Zipf(1.1) expert popularity.  A stratified sample of tokens (all their routes: the hottest expert and
    # rare ones among them) against the CPU executor STAGE BY STAGE as in the small shapes above, plus
    # properties at full size: every route is written exactly once and doubling the route weights doubles
    # every route output bit for bit (powers of two commute with both quantisers).
    tokens, k, experts, hidden, inter = 8192, 8, 256, 7168, 2048
    rng = H.rng_for(5)
    table, handles = build_device_experts(ctx, experts, hidden, inter, H.SEED_BASE + 5)
    ids, weights = H.zipf_routing(rng, tokens, k, experts)
    counts = np.bincount(ids.ravel(), minlength=experts)
    assert counts.max() > 20 * np.median(counts)          # the skew the config asks for
    gen = torch.Generator(device="cuda").manual_seed(H.SEED_BASE + 5)
    x = torch.randn((tokens, hidden), generator=gen, device="cuda").to(torch.bfloat16).float()
    xq, xs = ctx.pack_fp8_rows_from_f32(x)
    plan = ctx.expert_group_route_plan(experts, tokens * k, tokens, hidden, inter, hidden)
    h_all = torch.zeros((tokens * k, inter), dtype=torch.float32, device="cuda")

    def run(w, debug=None):
        ctx.begin_expert_group_route_invocation(plan, tokens * k)
        ctx.prepare_expert_group_route_plan(plan, table, _i32(ids.ravel()), _i32(np.ones(tokens * k)),
                                            _f32(w.ravel()), k)
        meta = plan.host_metadata()
        ctx.grouped_fp4_moe_from_prepared_plan(plan, table, xq, xs, meta=meta, debug_hidden=debug)
        return meta

    meta = run(weights, h_all)
    assert meta["total_routed_rows"] == tokens * k and meta["active_group_count"] == int((counts > 0).sum())
    assert meta["max_group_rows"] == int(counts.max())
    assert int(plan.route_error.item()) == 0
    assert bool((plan.route_written == 1).all())
    out = torch.zeros((tokens, hidden), dtype=torch.float32, device="cuda")
    ctx.reduce_moe_route_outputs_ranked(plan.route_output, tokens, k, hidden, out, plan.route_written,
                                        plan.route_error)
    hq, hs = ctx.grouped_workspace_views(plan, meta)
    row_of_route = torch.empty(tokens * k, dtype=torch.long, device="cuda")
    row_of_route[plan.route_indices[:tokens * k].long()] = torch.arange(tokens * k, device="cuda")
    rare = int(np.argmin(np.where(counts > 0, counts, 1 << 30)))
    sample = sorted({0, 4097, 8191, int(np.nonzero((ids == rare).any(1))[0][0]),
                     *(int(t) for t in rng.integers(0, tokens, 12))})
    want = np.zeros((len(sample), hidden), np.float32)
    delta = np.zeros((len(sample), hidden), np.float64)
    absdown = np.zeros((len(sample), hidden), np.float64)
    worst_h = worst_y = 0.0
    eps_in = hidden * 2.0 ** -24 + 2.0 ** -14
    for n, t in enumerate(sample):
        xt = x[t].cpu().numpy()
        xdq = po.simulate_fp8_act_quant(xt, hidden, 128)     # what the packed row decodes to
        ax = np.abs(xdq.astype(np.float64))
        ys = []
        for j in range(k):
            (gw, gs), (uw, us), (dw, ds) = [(h.weight.cpu().numpy().reshape(h.shape.out_features, -1),
                                             h.scale.cpu().numpy().reshape(h.shape.out_features, -1))
                                            for h in handles[int(ids[t, j])]]
            y, h = po.expert_execute_fp4(gw, gs, uw, us, dw, ds, hidden, inter, xt, float(weights[t, j]),
                                         act_quant_block=128, threads=8, return_hidden=True)
            ys.append(y)
            row = int(row_of_route[t * k + j].item())
            # (1) gate/up stage at K = 7168: the device's hidden row before quantisation against the
            # executor's on the dequantised input, inside the forward-error bound of the two dot products
            _, h_ref = po.expert_execute_fp4(gw, gs, uw, us, dw, ds, hidden, inter, xdq, float(weights[t, j]),
                                             threads=8, return_hidden=True)
            gate = po.linear_fp4(gw, gs, inter, hidden, xdq, threads=8)[0].astype(np.float64)
            up = po.linear_fp4(uw, us, inter, hidden, xdq, threads=8)[0].astype(np.float64)
            dg = po.abs_linear_fp4(gw, gs, inter, hidden, eps_in * ax, threads=8)
            du = po.abs_linear_fp4(uw, us, inter, hidden, eps_in * ax, threads=8)
            bound_h = float(weights[t, j]) * (1.1 * np.abs(up) * dg + np.abs(gate) * du + dg * du) + np.abs(h_ref) * 2.0 ** -21
            h_row = h_all[row].cpu().numpy()
            worst_h = max(worst_h, float((np.abs(h_row - h_ref) / (bound_h + 1e-30)).max()))
            # (2) the quantiser, bit-exact on the device's own hidden row
            want_q, want_s = po.pack_fp8_act(h_row, inter, 128)
            hq_row, hs_row = hq[row].cpu().numpy(), hs[row].cpu().numpy()
            assert np.array_equal(hs_row, want_s.reshape(-1)) and np.array_equal(hq_row, want_q.reshape(-1)), (t, j)
            # (3) down projection of those bytes
            h_gpu = po.simulate_fp8_act_quant(h_row, inter, 128)
            y_ref = po.linear_fp4(dw, ds, hidden, inter, h_gpu, threads=8)[0]
            absprod = po.abs_linear_fp4(dw, ds, hidden, inter, np.abs(h_gpu.astype(np.float64)), threads=8)
            err = np.abs(plan.route_output[t * k + j].cpu().numpy().astype(np.float64) - y_ref)
            assert (err <= (inter * 2.0 ** -24 + 2.0 ** -14) * absprod + 1e-30).all(), (t, j)
            worst_y = max(worst_y, float((err / (absprod + 1e-30)).max()))
            # (4) accounting for the end-to-end comparison below
            wd = po.dequantize_fp4(dw, ds, hidden, inter).astype(np.float64)
            delta[n] += wd @ (h_gpu.astype(np.float64) - h.astype(np.float64))
            absdown[n] += absprod
        want[n] = po.accumulate_routes(np.stack(ys))
    assert worst_h <= 1.0, worst_h
    within = H.quantised_chain_check(out[sample].cpu().numpy(), po.round_to_bf16_array(want), delta, absdown, inter,
                                     min_fraction=0.99, output_rounding=2.0 ** -8)
    print(f"config5: {len(sample)} tokens x {k} routes stage by stage: hidden rows use at most {worst_h:.3f} of their "
          f"bound, route outputs at most 2^{np.log2(worst_y + 1e-300):.1f} of sum|w h|, {within:.4f} of the combined "
          f"outputs within 2 BF16 ulp of the CPU chain")
    first = plan.route_output[:4096].clone()
    run(weights * np.float32(2.0))
    assert torch.equal(plan.route_output[:4096], first * 2.0)
    # the block-major copy of the same experts (the decode layer's) gives the same bits at full size
    run(weights)
    want_routes = plan.route_output[:tokens * k].clone()
    from ferrule_amd import synthetic

    prepared = synthetic.block_major_table(ctx, handles)
    plan_bm = ctx.expert_group_route_plan(experts, tokens * k, tokens, hidden, inter, hidden)
    ctx.begin_expert_group_route_invocation(plan_bm, tokens * k)
    ctx.prepare_expert_group_route_plan(plan_bm, prepared, _i32(ids.ravel()), _i32(np.ones(tokens * k)),
                                        _f32(weights.ravel()), k)
    ctx.grouped_fp4_moe_from_prepared_plan(plan_bm, prepared, xq, xs, meta=plan_bm.host_metadata())
    assert int(plan_bm.route_error.item()) == 0
    assert torch.equal(plan_bm.route_output[:tokens * k].view(torch.int32), want_routes.view(torch.int32))
