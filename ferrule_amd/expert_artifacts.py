"""Routed-expert weights from safetensors shards to device slots: the data format on the input
side of the MoE kernels.

Mirrors, for this one path, what Ferrule does between a checkpoint directory and a resident
expert:
  * shard header parsing (crates/ferrule-model/src/checkpoint/inventory.rs:433-573),
  * the HF tensor-name rule ``layers.<L>.ffn.experts.<E>.{w1,w3,w2}.{weight,scale}``
    (crates/ferrule-model/src/families/deepseek_v4.rs:111-140; w1 = gate, w3 = up, w2 = down),
  * the six-tensor expert bundle and its MXFP4 format inference
    (crates/ferrule-model/src/moe/streaming.rs:1138-1200, 2178-2292),
  * the device arena of 16-byte aligned views and the materialisation of one expert from
    pinned host memory: six host-to-device copies, then the provider's one-off layout
    preparation (crates/ferrule-backend/src/cuda/context.rs:702-745, 5048-5105, 5136-5287) -
    here ``ferrule_hip_prepare_mxfp4_block_major`` where the reference runs ``prepare_mxfp4_sfb``.

Nothing here computes on the CPU: bytes go from the file (memory-mapped) through pinned memory
to the device unchanged, and the tests compare them there.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass, field

MAX_SAFETENSORS_HEADER_BYTES = 512 * 1024 * 1024   # inventory.rs:18
ARENA_ALIGNMENT = 16                               # context.rs:703
MATRICES = ("gate", "up", "down")
_MATRIX_OF_NAME = {"w1": "gate", "w3": "up", "w2": "down"}


class ArtifactError(ValueError):
    """Where the reference returns ``Error::Model`` / ``Error::Internal`` for this path."""


@dataclass(frozen=True)
class RoutedExpertTensorRef:
    """crates/ferrule-model/src/semantic.rs:23-29."""
    layer: int
    expert: int
    matrix: str      # "gate" | "up" | "down"
    part: str        # "weight" | "scale" | anything else = unsupported component


def parse_hf_routed_expert_tensor(name: str) -> RoutedExpertTensorRef | None:
    """families/deepseek_v4.rs:111-140: exactly seven dot-separated parts, decimal layer and
    expert, matrix in {w1, w3, w2}; any other part name is kept (and refused later)."""
    parts = name.split(".")
    if len(parts) != 7 or parts[0] != "layers" or parts[2] != "ffn" or parts[3] != "experts":
        return None
    layer, expert, matrix, part = parts[1], parts[4], parts[5], parts[6]
    if not (layer.isascii() and layer.isdigit() and expert.isascii() and expert.isdigit()):
        return None
    if matrix not in _MATRIX_OF_NAME:
        return None
    return RoutedExpertTensorRef(int(layer), int(expert), _MATRIX_OF_NAME[matrix], part)


@dataclass(frozen=True)
class ShardHeaderTensor:
    name: str
    dtype: str
    shape: tuple
    data_offset: int   # relative to the shard's data section
    byte_size: int


def parse_safetensors_header_json(header: object, path: str) -> list[ShardHeaderTensor]:
    """inventory.rs:468-573."""
    if not isinstance(header, dict):
        raise ArtifactError(f"safetensors shard header '{path}' is not a JSON object")
    tensors = []
    for name, info in header.items():
        if name == "__metadata__":
            continue
        info = info if isinstance(info, dict) else {}
        dtype, shape, offsets = info.get("dtype"), info.get("shape"), info.get("data_offsets")
        if not isinstance(dtype, str):
            raise ArtifactError(f"safetensors tensor '{name}' in '{path}' missing dtype")
        if not isinstance(shape, list):
            raise ArtifactError(f"safetensors tensor '{name}' in '{path}' missing shape")
        if any(not isinstance(d, int) or isinstance(d, bool) or d < 0 for d in shape):
            raise ArtifactError(f"safetensors tensor '{name}' in '{path}' has non-integer shape dim")
        if not isinstance(offsets, list):
            raise ArtifactError(f"safetensors tensor '{name}' in '{path}' missing data_offsets")
        if len(offsets) != 2 or any(not isinstance(o, int) or isinstance(o, bool) or o < 0 for o in offsets):
            raise ArtifactError(f"safetensors tensor '{name}' in '{path}' has invalid data_offsets")
        if offsets[1] < offsets[0]:
            raise ArtifactError(f"safetensors tensor '{name}' in '{path}' has reversed data_offsets")
        tensors.append(ShardHeaderTensor(name, dtype, tuple(shape), offsets[0], offsets[1] - offsets[0]))
    tensors.sort(key=lambda t: t.name)
    return tensors


def read_safetensors_shard_header(path: str) -> tuple[int, list[ShardHeaderTensor]]:
    """(data_start, tensors) of one shard (inventory.rs:433-466): u64 little-endian header
    length, JSON header, data section from the next multiple of 8."""
    try:
        with open(path, "rb") as f:
            raw = f.read(8)
            if len(raw) != 8:
                raise ArtifactError(f"safetensors shard header length '{path}': file too short")
            header_len = struct.unpack("<Q", raw)[0]
            if header_len > MAX_SAFETENSORS_HEADER_BYTES:
                raise ArtifactError(f"safetensors shard header too large in '{path}': {header_len} bytes")
            text = f.read(header_len)
    except OSError as e:
        raise ArtifactError(f"safetensors shard open '{path}': {e}") from e
    if len(text) != header_len:
        raise ArtifactError(f"safetensors shard header read '{path}': file too short")
    try:
        header = json.loads(text.decode("utf-8"))
    except UnicodeDecodeError as e:
        raise ArtifactError(f"safetensors shard header utf8 '{path}': {e}") from e
    except json.JSONDecodeError as e:
        raise ArtifactError(f"safetensors shard header json '{path}': {e}") from e
    return (8 + header_len + 7) & ~7, parse_safetensors_header_json(header, path)


@dataclass(frozen=True)
class ExpertTensorSlice:
    """streaming.rs:145-160: where one tensor of one expert lies on disk."""
    layer: int
    expert: int
    matrix: str
    component: str
    path: str
    offset: int      # absolute file offset
    bytes: int
    dtype: str
    shape: tuple

    def end_offset(self) -> int:
        return self.offset + self.bytes


@dataclass(frozen=True)
class ExpertLinearFormat:
    """streaming.rs:1151-1162; ``Opaque`` is ``fp4 = False``."""
    fp4: bool
    out_features: int = 0
    in_features: int = 0
    block_size: int = 0


def infer_expert_linear_format(weight: ExpertTensorSlice, weight_len: int,
                               scale: tuple[ExpertTensorSlice, int] | None) -> ExpertLinearFormat:
    """streaming.rs:2249-2292: I8 [out, in/2] + F8_E8M0 [out, in/32] is packed MXFP4."""
    if scale is None:
        return ExpertLinearFormat(False)
    scale_slice, scale_len = scale
    if weight.dtype == "I8" and scale_slice.dtype == "F8_E8M0":
        if len(weight.shape) != 2 or len(scale_slice.shape) != 2:
            raise ArtifactError(f"FP4 expert tensor expects 2D weight/scale shapes, got {list(weight.shape)} and "
                                f"{list(scale_slice.shape)}")
        out, packed_in = weight.shape
        logical_in = packed_in * 2
        expected_cols = logical_in // 32
        if scale_slice.shape[0] != out or scale_slice.shape[1] != expected_cols:
            raise ArtifactError(f"FP4 expert scale shape mismatch: weight {list(weight.shape)} implies scale "
                                f"[{out}, {expected_cols}], got {list(scale_slice.shape)}")
        if weight_len != weight.bytes or scale_len != scale_slice.bytes:
            raise ArtifactError("expert payload byte length does not match tensor slice metadata")
        return ExpertLinearFormat(True, out, logical_in, 32)
    return ExpertLinearFormat(False)


@dataclass
class ExpertLinearSlices:
    matrix: str
    weight: ExpertTensorSlice
    scale: ExpertTensorSlice | None
    format: ExpertLinearFormat


@dataclass
class ExpertBundleSlices:
    """streaming.rs:1171-1200 ``ExpertComputeBundle``, as file slices instead of bytes."""
    layer: int
    expert: int
    gate: ExpertLinearSlices
    up: ExpertLinearSlices
    down: ExpertLinearSlices

    def linears(self):
        return self.gate, self.up, self.down

    def payload_bytes(self) -> int:
        return sum(l.weight.bytes + (l.scale.bytes if l.scale else 0) for l in self.linears())


def _build_linear(layer: int, expert: int, matrix: str, tensors: list[ExpertTensorSlice] | None) -> ExpertLinearSlices:
    """streaming.rs:2178-2236."""
    if not tensors:
        raise ArtifactError(f"expert artifact bundle missing {matrix} matrix for layer {layer} expert {expert}")
    weight = scale = None
    for t in tensors:
        if t.component == "weight":
            if weight is not None:
                raise ArtifactError(f"expert artifact bundle has duplicate {matrix} weight for layer {layer} "
                                    f"expert {expert}")
            weight = t
        elif t.component == "scale":
            if scale is not None:
                raise ArtifactError(f"expert artifact bundle has duplicate {matrix} scale for layer {layer} "
                                    f"expert {expert}")
            scale = t
        else:
            raise ArtifactError(f"expert artifact bundle has unsupported {matrix} component '{t.component}' for "
                                f"layer {layer} expert {expert}")
    if weight is None:
        raise ArtifactError(f"expert artifact bundle missing {matrix} weight for layer {layer} expert {expert}")
    fmt = infer_expert_linear_format(weight, weight.bytes, (scale, scale.bytes) if scale else None)
    return ExpertLinearSlices(matrix, weight, scale, fmt)


@dataclass
class RoutedExpertArtifactIndex:
    """Every routed-expert tensor of a checkpoint directory, by (layer, expert)."""
    slices: dict = field(default_factory=dict)     # (layer, expert) -> [ExpertTensorSlice]

    @staticmethod
    def open(model_dir: str) -> "RoutedExpertArtifactIndex":
        """Shards named by ``model.safetensors.index.json``'s weight_map when present
        (inventory.rs:144-200), else every ``*.safetensors`` file of the directory."""
        index_path = os.path.join(model_dir, "model.safetensors.index.json")
        if os.path.exists(index_path):
            try:
                weight_map = json.load(open(index_path))["weight_map"]
            except (KeyError, json.JSONDecodeError, TypeError) as e:
                raise ArtifactError(f"safetensors index '{index_path}': {e}") from e
            shards = sorted(set(weight_map.values()))
        else:
            weight_map = None
            shards = sorted(f for f in os.listdir(model_dir) if f.endswith(".safetensors"))
        index = RoutedExpertArtifactIndex()
        for shard in shards:
            path = os.path.join(model_dir, shard)
            data_start, tensors = read_safetensors_shard_header(path)
            size = os.path.getsize(path)
            for t in tensors:
                if weight_map is not None and weight_map.get(t.name) != shard:
                    continue
                ref = parse_hf_routed_expert_tensor(t.name)
                if ref is None:
                    continue
                offset = data_start + t.data_offset
                if offset + t.byte_size > size:
                    raise ArtifactError(f"safetensors tensor '{t.name}' in '{path}' extends past the end of the file")
                index.slices.setdefault((ref.layer, ref.expert), []).append(ExpertTensorSlice(
                    ref.layer, ref.expert, ref.matrix, ref.part, path, offset, t.byte_size, t.dtype, t.shape))
        return index

    def experts(self, layer: int) -> list[int]:
        return sorted(e for (l, e) in self.slices if l == layer)

    def bundle(self, layer: int, expert: int) -> ExpertBundleSlices:
        """streaming.rs:1179-1200 ``from_artifact_payload``."""
        grouped: dict = {}
        for t in self.slices.get((layer, expert), []):
            grouped.setdefault(t.matrix, []).append(t)
        return ExpertBundleSlices(layer, expert, *[_build_linear(layer, expert, m, grouped.get(m)) for m in MATRICES])


# ---- device side ------------------------------------------------------------------------------

@dataclass(frozen=True)
class HipRoutedExpertShape:
    """context.rs ``CudaRoutedExpertShape``: gate and up are [intermediate, input], down is
    [output, intermediate], all MXFP4 with one E8M0 scale per 32 k."""
    input: int
    intermediate: int
    output: int

    def linear_dims(self):
        return ((self.intermediate, self.input), (self.intermediate, self.input), (self.output, self.intermediate))

    def tensor_lengths(self) -> list[int]:
        """weight, scale bytes of gate, up, down - the order of the six copies (context.rs:5208-5240)."""
        out = []
        for n, k in self.linear_dims():
            if n == 0 or k == 0 or k % 32:
                raise ArtifactError(f"invalid HIP routed-expert shape: {self}")
            out += [n * (k // 2), n * (k // 32)]
        return out

    def frame_bytes(self) -> int:
        return sum((b + ARENA_ALIGNMENT - 1) // ARENA_ALIGNMENT * ARENA_ALIGNMENT for b in self.tensor_lengths())


class HipRoutedExpertArena:
    """Device storage for ``frame_capacity`` experts of one shape: per frame six raw views
    (checkpoint bytes) and, when asked for, six block-major views, all 16-byte aligned
    (context.rs:702-745, 5048-5105).  Allocated once; frames are handed out in order and reused
    by the caller's residency policy."""

    def __init__(self, ctx, shape: HipRoutedExpertShape, frame_capacity: int, block_major: bool = True):
        import torch

        if frame_capacity == 0:
            raise ArtifactError("HIP routed-expert arena requires positive frame capacity")
        self.ctx, self.shape, self.frame_capacity, self.block_major = ctx, shape, frame_capacity, block_major
        self.lengths = shape.tensor_lengths()
        self.frame_bytes = shape.frame_bytes()
        self.raw = torch.empty(self.frame_bytes * frame_capacity, dtype=torch.uint8, device=ctx.device)
        self.prepared = torch.empty_like(self.raw) if block_major else None
        # pinned staging frames, allocated (not registered); the second one on first batch use
        self.staging = torch.empty(self.frame_bytes, dtype=torch.uint8, pin_memory=True)
        self._staging2 = None
        self.allocated_frames = 0
        self._maps: dict = {}     # shard path -> read-only memory map, opened once

    def shard_bytes(self, path: str):
        """The shard as a read-only uint8 array over a memory map (opened on first use)."""
        import numpy as np

        if path not in self._maps:
            with open(path, "rb") as f:
                self._maps[path] = np.frombuffer(mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ), dtype=np.uint8)
        return self._maps[path]

    def staging_frames(self) -> list:
        import torch

        if self._staging2 is None:
            self._staging2 = torch.empty(self.frame_bytes, dtype=torch.uint8, pin_memory=True)
        return [self.staging, self._staging2]

    def view_offsets(self) -> list[int]:
        offsets, cursor = [], 0
        for b in self.lengths:
            cursor = (cursor + ARENA_ALIGNMENT - 1) & ~(ARENA_ALIGNMENT - 1)
            offsets.append(cursor)
            cursor += b
        return offsets

    def allocate_frame(self) -> int:
        if self.allocated_frames >= self.frame_capacity:
            raise ArtifactError("HIP routed-expert arena is full")
        self.allocated_frames += 1
        return self.allocated_frames - 1

    def views(self, storage, frame: int):
        base = frame * self.frame_bytes
        return [storage[base + o: base + o + b] for o, b in zip(self.view_offsets(), self.lengths)]


def materialize_routed_experts(ctx, arena: HipRoutedExpertArena, frames, bundles) -> list:
    """Several experts from their shard(s) into the given frames.  Per expert the six byte ranges
    are copied from the memory-mapped file into a pinned staging frame, ONE host-to-device copy
    moves the frame (the reference issues six, one per tensor, context.rs:5208-5240; the staging
    frame already has the arena's layout), then the three matrices are reordered block-major on
    the device.  Two staging frames alternate: while one is in flight to the device (copy and
    reorder are asynchronous on the context's stream), the host fills the other; an event per
    staging frame says when it may be overwritten.  Returns a list of (raw handles, prepared
    handles or None), each a (gate, up, down) triple of ``HipArtifactLinearHandle``; everything
    has completed when the call returns."""
    import torch

    from .provider import HipArtifactLinearHandle
    from .provider import HipArtifactLinearShape as S

    frames, bundles = list(frames), list(bundles)
    if len(frames) != len(bundles):
        raise ArtifactError("one frame per expert bundle")
    dims = arena.shape.linear_dims()
    for frame, bundle in zip(frames, bundles):    # everything is checked before anything is copied
        if not 0 <= frame < arena.allocated_frames:
            raise ArtifactError("HIP routed-expert frame was not allocated from this arena")
        for linear, (n, k) in zip(bundle.linears(), dims):
            f = linear.format
            if not f.fp4 or (f.out_features, f.in_features, f.block_size) != (n, k, 32):
                raise ArtifactError(f"expert layer {bundle.layer} expert {bundle.expert} {linear.matrix} is not the "
                                    f"arena's MXFP4 [{n}, {k}] matrix: {f}")
            if linear.weight.bytes != n * (k // 2) or linear.scale.bytes != n * (k // 32):
                raise ArtifactError("expert payload byte length does not match tensor slice metadata")
    offsets = arena.view_offsets()
    staging = arena.staging_frames()
    free_again = [None] * len(staging)
    results = []
    for index, (frame, bundle) in enumerate(zip(frames, bundles)):
        which = index % len(staging)
        if free_again[which] is not None:
            free_again[which].synchronize()
        host = staging[which].numpy()
        slices = [s for linear in bundle.linears() for s in (linear.weight, linear.scale)]
        for s, o, b in zip(slices, offsets, arena.lengths):
            host[o:o + b] = arena.shard_bytes(s.path)[s.offset:s.offset + b]
        base = frame * arena.frame_bytes
        with torch.cuda.stream(ctx.stream):
            arena.raw[base:base + arena.frame_bytes].copy_(staging[which], non_blocking=True)
            free_again[which] = torch.cuda.Event()
            free_again[which].record(ctx.stream)
        raw_views = arena.views(arena.raw, frame)
        raw = tuple(HipArtifactLinearHandle(S.fp4_e2m1_packed_with_e8m0_scale(n, k), raw_views[2 * i],
                                            raw_views[2 * i + 1]) for i, (n, k) in enumerate(dims))
        prepared = None
        if arena.block_major:
            prepared_views = arena.views(arena.prepared, frame)
            prepared = tuple(ctx.prepare_mxfp4_block_major_into(raw[i], prepared_views[2 * i], prepared_views[2 * i + 1])
                             for i in range(3))
        results.append((raw, prepared))
    ctx.synchronize()
    return results


def materialize_routed_expert(ctx, arena: HipRoutedExpertArena, frame: int, bundle: ExpertBundleSlices):
    """One expert into ``frame``: ``materialize_routed_experts`` for a single bundle."""
    return materialize_routed_experts(ctx, arena, [frame], [bundle])[0]
