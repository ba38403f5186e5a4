"""The MoE decode entry point that allocates nothing
(``ferrule_hip_moe_decode_launch_static_workspace``): same block, same kernels, workspace in a
fixed array of the library's device image.  Its outputs must equal those of
``ferrule_hip_moe_decode_launch`` bit for bit, also on a second, smaller call that finds the
first call's contents in the array, and sizes beyond the array are refused."""
import ctypes as C

import numpy as np
import pytest

from tests import helpers as H

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _i32(a):
    return torch.tensor(np.asarray(a, np.int32)).cuda()


def _f32(a):
    return torch.tensor(np.asarray(a, np.float32)).cuda()


def _experts(ctx, rng, experts, hidden, inter):
    from ferrule_amd.provider import HipArtifactLinearShape as S
    from ferrule_amd.provider import HipRoutedExpertTable

    table = HipRoutedExpertTable(experts, ctx.device)
    for e in range(experts):
        trio = []
        for n, k in ((inter, hidden), (inter, hidden), (hidden, inter)):
            w, s = H.mxfp4_weight(rng, n, k, 0.05)
            trio.append(ctx.prepare_mxfp4_block_major(
                ctx.upload_artifact_linear(S.fp4_e2m1_packed_with_e8m0_scale(n, k), w, s)))
        table.install(e, *trio, generation=1)
    table.commit()
    return table


def _layer(ctx, table, x, ids, weights, hidden, inter, static):
    tokens, k = ids.shape
    plan = ctx.expert_group_route_plan(table.slot_capacity, tokens * k, tokens, hidden, inter, hidden)
    ctx.prepare_decode_route_plan(plan, table, _i32(ids.ravel()), _i32(np.ones(tokens * k)), _f32(weights.ravel()), k)
    out = torch.empty((tokens, hidden), dtype=torch.bfloat16, device="cuda")
    xd = torch.from_numpy(x).to(torch.bfloat16).cuda()
    ctx.synchronize()
    if static and not _layer.set_up:
        # the first call on a device is the entry point's set-up (the array's address is looked up and its
        # completion event created): made here once, before anything is measured
        ctx.moe_decode_from_prepared_plan(plan, table, xd, out, static_workspace=True)
        ctx.synchronize()
        _layer.set_up = True
    allocated = torch.cuda.memory_allocated()
    free_before, _ = torch.cuda.mem_get_info()
    ctx.moe_decode_from_prepared_plan(plan, table, xd, out, static_workspace=static)
    ctx.synchronize()
    if static:
        # the host wrapper took nothing from torch's allocator, and the device's free memory is what it
        # was: the library did not allocate behind torch's back either (hipMalloc would show here)
        assert torch.cuda.memory_allocated() == allocated and plan.workspace is None
        assert torch.cuda.mem_get_info()[0] == free_before
    assert plan.route_error.item() == 0
    routes = plan.route_output.cpu().numpy()[:tokens * k].copy()
    return out.view(torch.int16).cpu().numpy().view(np.uint16), routes


_layer.set_up = False


def _routing(rng, tokens, k, experts):
    ids = np.stack([rng.permutation(experts)[:k] for _ in range(tokens)]).astype(np.int32)
    w = rng.random((tokens, k)).astype(np.float32)
    return ids, w / w.sum(1, keepdims=True)


def test_static_workspace_entry_equals_the_caller_workspace_entry_twice_in_a_row():
    from ferrule_amd.provider import HipArtifactOperatorContext

    ctx = HipArtifactOperatorContext(0)
    rng = H.rng_for(3, 7001)
    hidden, inter, experts, k = 1024, 512, 12, 4
    table = _experts(ctx, rng, experts, hidden, inter)
    # first call: 24 tokens (several experts with more than 8 rows: packed and general tiles);
    # second call: 3 tokens, which finds the first call's terms and hidden rows in the array
    for tokens in (24, 3):
        x = H.bf16_activations(rng, (tokens, hidden))
        ids, weights = _routing(rng, tokens, k, experts)
        got, got_routes = _layer(ctx, table, x, ids, weights, hidden, inter, static=True)
        want, want_routes = _layer(ctx, table, x, ids, weights, hidden, inter, static=False)
        assert np.array_equal(got_routes.view(np.uint32), want_routes.view(np.uint32)), f"{tokens} tokens: routes differ"
        assert np.array_equal(got, want), f"{tokens} tokens: outputs differ"
        assert np.isfinite(got_routes).all()


def test_static_workspace_entry_refuses_what_does_not_fit_and_a_caller_workspace():
    from ferrule_amd import abi
    from ferrule_amd.provider import HipArtifactOperatorContext, ProviderError

    ctx = HipArtifactOperatorContext(0)
    lib = abi.load()
    # scalar fields only: the size check comes before any pointer is looked at
    big = abi.MoeDecodeArgs(active_group_count=256, slot_capacity=256, total_routed_rows=2048, num_tokens=256,
                            num_routes=2048, routes_per_token=8, input_size=7168, intermediate_size=2048,
                            hidden_size=7168)
    assert lib.ferrule_hip_moe_decode_workspace_size(C.byref(big)) > abi.MOE_DECODE_STATIC_WORKSPACE_BYTES
    assert lib.ferrule_hip_moe_decode_launch_static_workspace(C.byref(big)) == abi.UNSUPPORTED
    fits = abi.MoeDecodeArgs(active_group_count=256, slot_capacity=256, total_routed_rows=512, num_tokens=64,
                             num_routes=512, routes_per_token=8, input_size=7168, intermediate_size=2048,
                             hidden_size=7168)
    assert lib.ferrule_hip_moe_decode_workspace_size(C.byref(fits)) <= abi.MOE_DECODE_STATIC_WORKSPACE_BYTES
    # it fits, so the block is validated like the other entry point's: null pointers are refused
    assert lib.ferrule_hip_moe_decode_launch_static_workspace(C.byref(fits)) == abi.INVALID_ARGUMENT
    fits.workspace, fits.workspace_bytes = 256, 1 << 30
    assert lib.ferrule_hip_moe_decode_launch_static_workspace(C.byref(fits)) == abi.INVALID_ARGUMENT
    assert lib.ferrule_hip_moe_decode_launch_static_workspace(None) == abi.INVALID_ARGUMENT
    # the host wrapper names the limit
    plan = ctx.expert_group_route_plan(256, 2048, 256, 7168, 2048, 7168)
    plan.invocation_routes, plan.routes_per_token = 2048, 8
    x = torch.zeros((256, 7168), dtype=torch.bfloat16, device="cuda")
    from ferrule_amd.provider import HipRoutedExpertTable

    with pytest.raises(ProviderError, match="static workspace holds"):
        ctx.moe_decode_from_prepared_plan(plan, HipRoutedExpertTable(256, ctx.device), x, static_workspace=True)


def test_static_workspace_entry_refuses_a_call_that_would_overlap_on_another_stream():
    """The array is one per GPU: while a call on one stream has not completed, a call on another stream is
    refused (UNSUPPORTED, nothing launched); once the first stream has drained it is accepted, and calls
    queued on ONE stream are always accepted."""
    from ferrule_amd import abi
    from ferrule_amd.provider import HipArtifactOperatorContext, ProviderError

    ctx = HipArtifactOperatorContext(0)
    rng = H.rng_for(3, 7002)
    hidden, inter, experts, k, tokens = 1024, 512, 12, 4, 16
    table = _experts(ctx, rng, experts, hidden, inter)
    x = torch.from_numpy(H.bf16_activations(rng, (tokens, hidden))).to(torch.bfloat16).cuda()
    ids, weights = _routing(rng, tokens, k, experts)
    plan = ctx.expert_group_route_plan(table.slot_capacity, tokens * k, tokens, hidden, inter, hidden)
    ctx.prepare_decode_route_plan(plan, table, _i32(ids.ravel()), _i32(np.ones(tokens * k)), _f32(weights.ravel()), k)
    out = torch.empty((tokens, hidden), dtype=torch.bfloat16, device="cuda")
    ctx.moe_decode_from_prepared_plan(plan, table, x, out, static_workspace=True)
    ctx.synchronize()
    want = out.clone()
    first, second = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    busy = torch.randn((8192, 8192), device="cuda")
    torch.cuda.synchronize()
    with torch.cuda.stream(first):
        for _ in range(4):        # tens of milliseconds of other work in front of the layer on this stream
            busy = busy @ busy
            busy = busy / busy.abs().max()
        for _ in range(3):        # calls queued on one stream: every one accepted
            ctx.moe_decode_from_prepared_plan(plan, table, x, out, static_workspace=True)
    with torch.cuda.stream(second):
        with pytest.raises(ProviderError) as refused:
            ctx.moe_decode_from_prepared_plan(plan, table, x, out, static_workspace=True)
        assert refused.value.status == abi.UNSUPPORTED
    first.synchronize()
    with torch.cuda.stream(second):
        ctx.moe_decode_from_prepared_plan(plan, table, x, out, static_workspace=True)
    second.synchronize()
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))
