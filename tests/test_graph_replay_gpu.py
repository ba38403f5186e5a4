"""The steps around the MoE layer inside a captured HIP graph: HC producer -> router -> slot resolve
-> fused decode plan -> MoE decode layer.  The graph is replayed several times with new inputs
written into the captured buffers between replays (and eager work in between); every replay must
reproduce the eager results bit for bit - nothing in the chain may depend on state a previous
replay left behind, and nothing may allocate or synchronise."""
import numpy as np
import pytest
import torch

from tests import helpers as H

pytestmark = pytest.mark.gpu


def test_captured_chain_replays_like_eager_runs():
    from ferrule_amd.provider import HipArtifactOperatorContext, HipExpertSlotPointers
    from tests.test_moe_gpu import _make_experts

    tokens, k, experts, hidden, inter, hc_hidden = 6, 2, 8, 1024, 256, 1024
    rng = H.rng_for(16)
    side = torch.cuda.Stream()
    ctx = HipArtifactOperatorContext(0, stream=side)
    with torch.cuda.stream(side):
        routed, host = _make_experts(ctx, rng, experts, hidden, inter, sigma=0.05)
        table = ctx.expert_slot_table(experts, experts)
        for e in reversed(range(experts)):
            gate, up, down = (m[2] for m in host[e])
            ctx.install_expert_slot(table, e, HipExpertSlotPointers.from_handles(gate, up, down),
                                    keepalive=(gate, up, down), block_major=False)

        # captured buffers
        state = torch.zeros((tokens, 4, hc_hidden), dtype=torch.float32, device="cuda")
        function = torch.from_numpy((rng.normal(size=(24, 4 * hc_hidden)) / 64).astype(np.float32)).cuda()
        hc_scale = torch.tensor([0.8, 1.3, 0.6], device="cuda")
        hc_base = torch.from_numpy(rng.normal(0, 0.3, 24).astype(np.float32)).cuda()
        rms_weight = torch.ones(hc_hidden, device="cuda")
        logits = torch.zeros((tokens, experts), dtype=torch.float32, device="cuda")
        idx = torch.zeros((tokens, k), dtype=torch.int32, device="cuda")
        w = torch.zeros((tokens, k), dtype=torch.float32, device="cuda")
        workspace = ctx.expert_route_resolve_workspace(tokens * k, 4)
        plan = ctx.expert_group_route_plan(table.slot_capacity, tokens * k, tokens, hidden, inter, hidden)
        x = torch.zeros((tokens, hidden), dtype=torch.bfloat16, device="cuda")
        out = torch.zeros((tokens, hidden), dtype=torch.bfloat16, device="cuda")
        hc_out = None

        def chain():
            nonlocal hc_out
            hc_out = ctx.hc_pre_rmsnorm_fp8_into(state, function, hc_scale, hc_base, rms_weight, 4, 1e-6, 1e-6, 1e-6,
                                                 out=hc_out)
            ctx.dsv4_router_topk_sqrt_softplus_rows_from_device_into(logits, None, tokens, experts, k, 1.5, idx, w)
            ctx.resolve_expert_routes(table, idx.view(-1), tokens * k, workspace)
            ctx.prepare_decode_route_plan(plan, table, workspace.route_slots, workspace.route_generations, w.view(-1), k)
            ctx.moe_decode_from_prepared_plan(plan, table, x, out, None, 0.0)

        def new_inputs(seed):
            g = np.random.default_rng(seed)
            state.copy_(torch.from_numpy(g.normal(size=tuple(state.shape)).astype(np.float32)))
            logits.copy_(torch.from_numpy(g.normal(0, 2, tuple(logits.shape)).astype(np.float32)))
            x.copy_(torch.from_numpy(g.normal(size=tuple(x.shape)).astype(np.float32)).to(torch.bfloat16))

        def snapshot():
            side.synchronize()
            return [t.clone() for t in (hc_out["packed"], hc_out["scales"], hc_out["normalized"], hc_out["comb"], idx, w,
                                        workspace.route_slots, workspace.miss_control, plan.expert_route_indptr,
                                        out.view(torch.int16))]

        new_inputs(0)
        chain()                      # allocates hc_out's buffers once, outside the capture
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            chain()
        for seed in (1, 2, 3, 1):
            new_inputs(seed)
            chain()
            want = snapshot()
            for t in (idx, w, out, hc_out["packed"], workspace.route_slots):     # eager work between the replays
                t.zero_()
            graph.replay()
            got = snapshot()
            for a, b in zip(got, want):
                assert torch.equal(a, b), f"replay with seed {seed} differs from the eager run"
