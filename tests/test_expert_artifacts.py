"""Routed-expert artifacts: safetensors shards -> index -> six-tensor bundles (CPU), and -> arena ->
slot table -> decode layer (GPU).  Shards are written with the ``safetensors`` library, so the
reader is checked against an independent writer of the format."""
import json
import os
import struct

import numpy as np
import pytest
import torch

from ferrule_amd import expert_artifacts as EA
from tests import helpers as H


def _write_checkpoint(directory, rng, layer, experts, hidden, inter, shards=2, sigma=0.05, with_index=True):
    """experts' w1/w3/w2 weight (I8) + scale (F8_E8M0) spread over `shards` files, plus decoys."""
    from safetensors.torch import save_file

    host, per_shard, weight_map = {}, [dict() for _ in range(shards)], {}
    for e in experts:
        mats = []
        for name, (n, k) in (("w1", (inter, hidden)), ("w3", (inter, hidden)), ("w2", (hidden, inter))):
            w, s = H.mxfp4_weight(rng, n, k, sigma)
            mats.append((w, s))
            shard = (e + len(name) + n) % shards
            base = f"layers.{layer}.ffn.experts.{e}.{name}"
            per_shard[shard][base + ".weight"] = torch.from_numpy(w.reshape(n, k // 2).view(np.int8).copy())
            per_shard[(shard + 1) % shards][base + ".scale"] = \
                torch.from_numpy(s.reshape(n, k // 32).copy()).view(torch.float8_e8m0fnu)
        host[e] = mats
    per_shard[0]["embed.weight"] = torch.zeros((2, 3), dtype=torch.bfloat16)
    per_shard[0][f"layers.{layer}.ffn.shared_experts.w1.weight"] = torch.zeros((4, 4), dtype=torch.int8)
    for i, tensors in enumerate(per_shard):
        name = f"model-{i + 1:05d}-of-{shards:05d}.safetensors"
        save_file(tensors, os.path.join(directory, name))
        for t in tensors:
            weight_map[t] = name
    if with_index:
        json.dump({"metadata": {}, "weight_map": weight_map}, open(os.path.join(directory, "model.safetensors.index.json"), "w"))
    return host


def test_tensor_name_rule():
    # families/deepseek_v4.rs:111-140; the name of checkpoint/inventory.rs:603
    ref = EA.parse_hf_routed_expert_tensor("layers.0.ffn.experts.3.w1.weight")
    assert ref == EA.RoutedExpertTensorRef(0, 3, "gate", "weight")
    assert EA.parse_hf_routed_expert_tensor("layers.12.ffn.experts.255.w3.scale") == \
        EA.RoutedExpertTensorRef(12, 255, "up", "scale")
    assert EA.parse_hf_routed_expert_tensor("layers.1.ffn.experts.0.w2.bias").part == "bias"
    for other in ("layers.0.ffn.shared_experts.w1.weight", "layers.0.ffn.experts.3.w4.weight",
                  "layers.x.ffn.experts.3.w1.weight", "layers.0.ffn.experts.3.w1", "mtp.0.ffn.experts.3.w1.weight",
                  "layers.0.ffn.experts.-3.w1.weight", "model.layers.0.ffn.experts.3.w1.weight"):
        assert EA.parse_hf_routed_expert_tensor(other) is None, other


def test_index_finds_every_expert_and_reads_the_written_bytes(tmp_path):
    rng = H.rng_for(12)
    host = _write_checkpoint(str(tmp_path), rng, 3, [0, 2, 5], 128, 64)
    index = EA.RoutedExpertArtifactIndex.open(str(tmp_path))
    assert index.experts(3) == [0, 2, 5] and index.experts(0) == []
    for e in (0, 2, 5):
        bundle = index.bundle(3, e)
        assert bundle.gate.format == EA.ExpertLinearFormat(True, 64, 128, 32)
        assert bundle.down.format == EA.ExpertLinearFormat(True, 128, 64, 32)
        assert bundle.payload_bytes() == 3 * (64 * 128 // 2 + 64 * 128 // 32)
        for linear, (w, s) in zip(bundle.linears(), host[e]):
            for sl, want in ((linear.weight, w), (linear.scale, s)):
                with open(sl.path, "rb") as f:
                    f.seek(sl.offset)
                    assert f.read(sl.bytes) == np.ascontiguousarray(want).tobytes()
            assert linear.weight.dtype == "I8" and linear.scale.dtype == "F8_E8M0"
    # without the index file every *.safetensors of the directory is scanned
    os.remove(tmp_path / "model.safetensors.index.json")
    assert EA.RoutedExpertArtifactIndex.open(str(tmp_path)).experts(3) == [0, 2, 5]


def _raw_shard(path, header, data=b""):
    text = json.dumps(header).encode()
    text += b" " * (-(8 + len(text)) % 8)
    open(path, "wb").write(struct.pack("<Q", len(text)) + text + data)


def test_header_and_bundle_errors(tmp_path):
    p = str(tmp_path / "a.safetensors")
    ok = {"dtype": "I8", "shape": [2, 16], "data_offsets": [0, 32]}
    for bad, message in (({"dtype": "I8", "shape": [2, 16]}, "missing data_offsets"),
                         ({"dtype": "I8", "shape": [2, 16], "data_offsets": [0]}, "invalid data_offsets"),
                         ({"dtype": "I8", "shape": [2, 16], "data_offsets": [8, 0]}, "reversed data_offsets"),
                         ({"shape": [2, 16], "data_offsets": [0, 32]}, "missing dtype"),
                         ({"dtype": "I8", "data_offsets": [0, 32]}, "missing shape"),
                         ({"dtype": "I8", "shape": [2, 1.5], "data_offsets": [0, 32]}, "non-integer shape")):
        _raw_shard(p, {"layers.0.ffn.experts.0.w1.weight": bad})
        with pytest.raises(EA.ArtifactError, match=message):
            EA.read_safetensors_shard_header(p)
    _raw_shard(p, {"layers.0.ffn.experts.0.w1.weight": ok}, b"\0" * 16)
    with pytest.raises(EA.ArtifactError, match="past the end"):
        EA.RoutedExpertArtifactIndex.open(str(tmp_path))
    open(p, "wb").write(struct.pack("<Q", 1 << 40))
    with pytest.raises(EA.ArtifactError, match="header too large"):
        EA.read_safetensors_shard_header(p)

    # bundles: streaming.rs:2178-2236
    header = {"__metadata__": {"format": "pt"}}
    cursor = 0
    for m, (n, k) in (("w1", (4, 64)), ("w3", (4, 64))):
        header[f"layers.0.ffn.experts.1.{m}.weight"] = {"dtype": "I8", "shape": [n, k // 2], "data_offsets": [cursor, cursor + n * k // 2]}
        cursor += n * k // 2
        header[f"layers.0.ffn.experts.1.{m}.scale"] = {"dtype": "F8_E8M0", "shape": [n, k // 32], "data_offsets": [cursor, cursor + n * k // 32]}
        cursor += n * k // 32
    _raw_shard(p, header, b"\0" * cursor)
    index = EA.RoutedExpertArtifactIndex.open(str(tmp_path))
    with pytest.raises(EA.ArtifactError, match="missing down matrix"):
        index.bundle(0, 1)
    header["layers.0.ffn.experts.1.w2.scale"] = {"dtype": "F8_E8M0", "shape": [64, 1], "data_offsets": [0, 64]}
    _raw_shard(p, header, b"\0" * cursor)
    with pytest.raises(EA.ArtifactError, match="missing down weight"):
        EA.RoutedExpertArtifactIndex.open(str(tmp_path)).bundle(0, 1)
    header["layers.0.ffn.experts.1.w2.weight"] = {"dtype": "I8", "shape": [64, 2], "data_offsets": [0, 128]}
    header["layers.0.ffn.experts.1.w2.scale"] = {"dtype": "F8_E8M0", "shape": [64, 2], "data_offsets": [0, 128]}
    _raw_shard(p, header, b"\0" * cursor)
    with pytest.raises(EA.ArtifactError, match="scale shape mismatch"):
        EA.RoutedExpertArtifactIndex.open(str(tmp_path)).bundle(0, 1)
    header["layers.0.ffn.experts.1.w2.scale"] = {"dtype": "F8_E8M0", "shape": [64, 0], "data_offsets": [0, 0]}
    header["layers.0.ffn.experts.1.w2.bias"] = {"dtype": "F32", "shape": [1], "data_offsets": [0, 4]}
    _raw_shard(p, header, b"\0" * cursor)
    with pytest.raises(EA.ArtifactError, match="unsupported down component 'bias'"):
        EA.RoutedExpertArtifactIndex.open(str(tmp_path)).bundle(0, 1)
    # a weight without a scale is an opaque linear, not an error (streaming.rs:2254-2256)
    del header["layers.0.ffn.experts.1.w2.bias"], header["layers.0.ffn.experts.1.w2.scale"]
    _raw_shard(p, header, b"\0" * cursor)
    assert not EA.RoutedExpertArtifactIndex.open(str(tmp_path)).bundle(0, 1).down.format.fp4


def test_arena_layout_is_sixteen_byte_aligned_views():
    shape = EA.HipRoutedExpertShape(input=96, intermediate=32, output=5)      # the down scale is 5 bytes
    assert shape.tensor_lengths() == [1536, 96, 1536, 96, 80, 5]
    assert shape.frame_bytes() == 1536 + 96 + 1536 + 96 + 80 + 16
    with pytest.raises(EA.ArtifactError):
        EA.HipRoutedExpertShape(100, 40, 96).tensor_lengths()


@pytest.mark.gpu
def test_experts_from_shards_to_slots_run_the_decode_layer(tmp_path):
    from ferrule_amd.provider import HipArtifactOperatorContext, HipExpertSlotPointers
    from oracle import pyoracle as po
    from tests.test_moe_gpu import _oracle_moe, _routing

    ctx = HipArtifactOperatorContext(0)
    layer, experts, hidden, inter, tokens, k = 7, 6, 512, 256, 5, 2
    rng = H.rng_for(13)
    host = _write_checkpoint(str(tmp_path), rng, layer, range(experts), hidden, inter, shards=3)
    index = EA.RoutedExpertArtifactIndex.open(str(tmp_path))
    assert index.experts(layer) == list(range(experts))

    shape = EA.HipRoutedExpertShape(hidden, inter, hidden)
    arena = EA.HipRoutedExpertArena(ctx, shape, experts, block_major=True)
    table = ctx.expert_slot_table(experts, experts)
    for e in reversed(range(experts)):                      # slot != expert id
        frame = arena.allocate_frame()
        raw, prepared = EA.materialize_routed_expert(ctx, arena, frame, index.bundle(layer, e))
        for handle, (w, s) in zip(raw, host[e]):            # the device holds the file's bytes
            assert handle.weight.cpu().numpy().tobytes() == np.ascontiguousarray(w).tobytes()
            assert handle.scale.cpu().numpy().tobytes() == np.ascontiguousarray(s).tobytes()
            assert handle.weight.data_ptr() % 16 == 0 and handle.scale.data_ptr() % 16 == 0
        ctx.install_expert_slot(table, e, HipExpertSlotPointers.from_handles(*prepared), keepalive=(arena,),
                                block_major=True)
    with pytest.raises(EA.ArtifactError, match="arena is full"):
        arena.allocate_frame()

    x = H.bf16_activations(rng, (tokens, hidden))
    ids, weights = _routing(rng, tokens, k, experts)
    workspace = ctx.expert_route_resolve_workspace(tokens * k, 4)
    ctx.resolve_expert_routes(table, torch.from_numpy(ids.ravel()).cuda(), tokens * k, workspace)
    plan = ctx.expert_group_route_plan(table.slot_capacity, tokens * k, tokens, hidden, inter, hidden)
    ctx.prepare_decode_route_plan(plan, table, workspace.route_slots, workspace.route_generations,
                                  torch.from_numpy(weights.ravel()).cuda(), k)
    out = torch.empty((tokens, hidden), dtype=torch.bfloat16, device="cuda")
    ctx.moe_decode_from_prepared_plan(plan, table, torch.from_numpy(x).to(torch.bfloat16).cuda(), out, None, 0.0)
    ctx.synchronize()
    host_list = [[(w, s, None) for (w, s) in host[e]] for e in range(experts)]
    want, bound, _, _ = _oracle_moe(host_list, x, ids, weights, hidden, inter)
    worst, _, _ = H.compare_bf16_bounded(out.view(torch.int16).cpu().numpy().view(np.uint16), want, bound,
                                         max_decided_fraction=0.005)
    assert worst <= 2 and plan.route_error.item() == 0

    # a bundle of another shape is refused before anything is copied
    small = EA.HipRoutedExpertArena(ctx, EA.HipRoutedExpertShape(hidden, inter // 2, hidden), 1, block_major=False)
    with pytest.raises(EA.ArtifactError, match="is not the arena's MXFP4"):
        EA.materialize_routed_expert(ctx, small, small.allocate_frame(), index.bundle(layer, 0))
