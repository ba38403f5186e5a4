"""Device slot table (ferrule_hip_core_expert_table_launch) through the C ABI: the reference's own
test case, random tables against the CPU checker (bit-exact; the miss list as a set, its order being
unspecified in the reference too), and the whole device chain logits -> router -> resolve -> route
plan -> MoE decode layer."""
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


def _i32(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.int32)).cuda()


def test_reference_stable_slot_table_case(ctx):
    # expert_group_route_plan.rs:29-107
    from ferrule_amd.provider import HipExpertSlotPointers

    pointers = HipExpertSlotPointers(16, 32, 48, 64, 80, 96)
    table = ctx.expert_slot_table(4, 1)
    launches = ctx.kernel_launches
    first = ctx.install_expert_slot(table, 2, pointers)
    assert ctx.kernel_launches == launches + 1
    workspace = ctx.expert_route_resolve_workspace(4, 2)
    ctx.resolve_expert_routes(table, _i32([2, 1, -1, 4]), 4, workspace)
    resolved = ctx.download_expert_route_resolve(workspace, 4)
    assert resolved.route_slots == [first.slot, -1, -1, -1]
    assert resolved.route_generations == [first.generation, 0, 0, 0]
    assert resolved.miss_markers == [0, 1, 1, 1]
    assert len(resolved.miss_ids) == 2 and all(i in (1, -1, 4) for i in resolved.miss_ids)
    assert resolved.miss_ids[0] != resolved.miss_ids[1] and resolved.miss_overflow

    assert ctx.evict_expert_slot(table, 2)
    second = ctx.install_expert_slot(table, 1, pointers)
    assert second.slot == first.slot and second.generation != first.generation
    assert not table.host.is_current(first) and table.host.is_current(second)
    ctx.resolve_expert_routes(table, _i32([2, 1]), 2, workspace)
    resolved = ctx.download_expert_route_resolve(workspace, 2)
    assert resolved.route_slots == [-1, second.slot] and resolved.route_generations == [0, second.generation]
    assert resolved.miss_ids == [2] and not resolved.miss_overflow
    # the device arrays are the host mirror
    assert table.slot_generations.cpu().tolist() == table.host.slot_generation
    assert table.expert_to_slot.cpu().tolist() == table.host.expert_to_slot
    assert table.gate_ptrs.cpu().tolist() == [16] and table.down_scale_ptrs.cpu().tolist() == [96]


@pytest.mark.parametrize("experts,slots,routes,miss_capacity,seed", [(256, 64, 512, 32, 0), (256, 256, 65536, 16, 1),
                                                                      (16, 4, 7, 3, 2), (384, 100, 4099, 5000, 3)])
def test_random_tables_resolve_and_gather_like_the_checker(ctx, experts, slots, routes, miss_capacity, seed):
    from ferrule_amd.provider import HipExpertSlotPointers

    rng = H.rng_for(10, seed)
    table = ctx.expert_slot_table(experts, slots)
    state = po.ExpertTableState(experts, slots)

    def install(e):
        ptrs = HipExpertSlotPointers(*[int(v) for v in rng.integers(1, 1 << 40, 6) * 16])
        b = ctx.install_expert_slot(table, e, ptrs)
        state.publish(1, e, b.slot, b.generation, ptrs.as_tuple())

    def evict(e):
        b = table.host.binding(e)
        assert ctx.evict_expert_slot(table, e)
        state.publish(2, e, b.slot, table.host.slot_generation[b.slot])

    order = rng.permutation(experts)
    for e in order[:slots]:
        install(int(e))
    for e in order[:slots // 3]:                     # churn: evict a third and install other experts there
        evict(int(e))
    for e in order[slots:slots + slots // 4]:
        install(int(e))
    for name, dev in (("gate", table.gate_ptrs), ("gate_scale", table.gate_scale_ptrs), ("up", table.up_ptrs),
                      ("up_scale", table.up_scale_ptrs), ("down", table.down_ptrs), ("down_scale", table.down_scale_ptrs)):
        row = ("gate", "gate_scale", "up", "up_scale", "down", "down_scale").index(name)
        assert np.array_equal(dev.cpu().numpy().view(np.uint64), state.table[row]), name
    assert np.array_equal(table.expert_to_slot.cpu().numpy(), state.expert_to_slot)
    assert np.array_equal(table.expert_generations.cpu().numpy(), state.expert_generations)
    assert np.array_equal(table.slot_generations.cpu().numpy(), state.slot_generations)

    ids = rng.integers(-2, experts + 2, routes).astype(np.int32)
    workspace = ctx.expert_route_resolve_workspace(routes + 5, miss_capacity)
    ctx.resolve_expert_routes(table, _i32(ids), routes, workspace)
    ctx.synchronize()
    want_slots, want_gens, want_markers, want_control = state.resolve(ids, miss_capacity, routes + 5)
    assert np.array_equal(workspace.route_slots.cpu().numpy()[:routes], want_slots)
    assert np.array_equal(workspace.route_generations.cpu().numpy()[:routes], want_gens)
    assert np.array_equal(workspace.miss_markers.cpu().numpy()[:routes], want_markers)
    control = workspace.miss_control.cpu().numpy()
    assert control[0] == want_control[0] and control[1] == want_control[1]
    assert np.array_equal(control[2 + miss_capacity:], want_control[2 + miss_capacity:])
    missing = ids[want_markers == 1]
    listed = control[2:2 + min(miss_capacity, int(control[0]))]
    if control[0] <= miss_capacity:
        assert sorted(listed.tolist()) == sorted(missing.tolist())
        assert (control[2 + int(control[0]):2 + miss_capacity] == -1).all()
    else:
        # an overflowing list holds miss_capacity of the missing ids, each no more often than it is missing
        have = {v: c for v, c in zip(*np.unique(missing, return_counts=True))}
        for v, c in zip(*np.unique(listed, return_counts=True)):
            assert have.get(v, 0) >= c

    weights = rng.random(routes).astype(np.float32)
    markers = rng.integers(0, 3, routes).astype(np.int32)
    gens = want_gens.copy()
    gens[rng.integers(0, routes, max(1, routes // 50))] += 1          # stale generations among the routes
    for active_value, use_gens in ((1, gens), (2, want_gens)):
        out = ctx.gather_stable_moe_dispatch(table, workspace.route_slots, _i32(use_gens), torch.from_numpy(weights).cuda(),
                                             _i32(markers), active_value, routes)
        ctx.synchronize()
        want_out, want_w, want_ids, want_err = state.gather_dispatch(want_slots, use_gens, weights, markers, active_value)
        for row, name in enumerate(("gate", "gate_scale", "up", "up_scale", "down", "down_scale")):
            assert np.array_equal(out[name].cpu().numpy().view(np.uint64), want_out[row]), name
        assert np.array_equal(out["route_weights"].cpu().numpy(), want_w)
        assert np.array_equal(out["route_slots"].cpu().numpy(), want_ids)
        assert out["dispatch_error"].item() == want_err


def test_logits_to_decode_layer_on_the_device(ctx):
    """logits -> router ids -> resolved slots and generations -> fused decode plan -> MoE decode layer.
    Experts live in slots that differ from their ids, one routed expert is not resident: its tokens come
    out as NaN (the layer's rule for an unresolved route), every other token equals the CPU executor."""
    from ferrule_amd.provider import HipArtifactLinearShape as S
    from ferrule_amd.provider import HipExpertSlotPointers
    from tests.test_moe_gpu import _oracle_moe

    tokens, k, experts, slots, hidden, inter = 6, 2, 8, 8, 512, 256
    rng = H.rng_for(11)
    table = ctx.expert_slot_table(experts, slots)
    absent = 5
    order = [int(e) for e in rng.permutation(experts)]  # install order decides the slot: slot != expert id
    host = [None] * experts
    for e in order:
        mats = []
        for n, kk in ((inter, hidden), (inter, hidden), (hidden, inter)):
            w, s = H.mxfp4_weight(rng, n, kk, 0.05)
            mats.append((w, s, ctx.upload_artifact_linear(S.fp4_e2m1_packed_with_e8m0_scale(n, kk), w, s)))
        host[e] = mats
        if e != absent:
            ctx.install_expert_slot(table, e, HipExpertSlotPointers.from_handles(mats[0][2], mats[1][2], mats[2][2]),
                                    keepalive=tuple(m[2] for m in mats), block_major=False)
    assert any(table.host.binding(e).slot != e for e in range(experts) if e != absent)

    x = H.bf16_activations(rng, (tokens, hidden))
    logits = rng.normal(0.0, 2.0, (tokens, experts)).astype(np.float32)
    logits[0, absent] = 9.0                             # token 0 certainly routes to the absent expert
    logits[1:, absent] = -9.0                           # nobody else does
    idx = torch.zeros((tokens, k), dtype=torch.int32, device="cuda")
    w = torch.zeros((tokens, k), dtype=torch.float32, device="cuda")
    ctx.dsv4_router_topk_sqrt_softplus_rows_from_device_into(torch.from_numpy(logits).cuda(), None, tokens, experts, k,
                                                             1.5, idx, w)
    workspace = ctx.expert_route_resolve_workspace(tokens * k, 4)
    ctx.resolve_expert_routes(table, idx.view(-1), tokens * k, workspace)
    plan = ctx.expert_group_route_plan(table.slot_capacity, tokens * k, tokens, hidden, inter, hidden)
    ctx.prepare_decode_route_plan(plan, table, workspace.route_slots, workspace.route_generations, w.view(-1), k)
    out = torch.empty((tokens, hidden), dtype=torch.bfloat16, device="cuda")
    ctx.moe_decode_from_prepared_plan(plan, table, torch.from_numpy(x).to(torch.bfloat16).cuda(), out, None, 0.0)
    resolved = ctx.download_expert_route_resolve(workspace, tokens * k)

    want_idx, _ = po.router_kernel_rows(1, logits, k, 1.5)
    assert np.array_equal(idx.cpu().numpy(), want_idx)
    assert resolved.miss_ids == [absent] and not resolved.miss_overflow
    got_w = w.cpu().numpy()
    got = out.float().cpu().numpy()
    assert np.isnan(got[0]).all()
    want, bound, _, _ = _oracle_moe(host, x[1:], want_idx[1:], got_w[1:], hidden, inter)
    worst, _, _ = H.compare_bf16_bounded(out[1:].contiguous().view(torch.int16).cpu().numpy().view(np.uint16), want,
                                         bound, max_decided_fraction=0.005)
    assert worst <= 2
