"""Host side of the provider: the Python stand-in for the part of Ferrule's
``CudaArtifactOperatorContext`` (crates/ferrule-backend/src/cuda/context.rs) that
drives the quantized-weight matmul path.

It owns nothing the C ABI needs to know about: torch is used only to hold device
memory and to lend a ``hipStream_t``.  Every operation fills a POD argument block
(``ferrule_amd.abi``), calls ``*_can_implement`` and then ``*_launch`` exactly as
the reference does (crates/ferrule-backend/src/cuda/cutlass.rs:1780-1812), and maps
a non-zero status to an exception the way
crates/ferrule-backend/src/cuda/cutlass.rs:2938-2963 maps it to ``Error::Internal``.

There is no CPU path here: without a GPU, or without the built library, every
operation raises.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import torch

from . import abi


class ProviderError(RuntimeError):
    """A native entry point returned a non-zero status."""

    def __init__(self, what: str, status: int):
        names = {abi.INVALID_ARGUMENT: "invalid argument", abi.LAUNCH_FAILED: "launch failed",
                 abi.UNSUPPORTED: "unsupported"}
        detail = ""
        if status == abi.LAUNCH_FAILED:
            detail = f", hipError_t {abi.load().ferrule_hip_last_error_code()}"
        super().__init__(f"HIP provider {what} failed: {names.get(status, 'error')} ({status}{detail})")
        self.status = status


@dataclass(frozen=True)
class HipArtifactLinearShape:
    """Counterpart of ``CudaArtifactLinearShape`` (context.rs:386-405) for the two
    quantized layouts, plus the F32-scale variant this provider adds for FP8."""

    weight_format: int            # abi.WEIGHT_FP8_E4M3 | abi.WEIGHT_MXFP4_E2M1
    out_features: int
    in_features: int
    block_m: int = 1
    block_k: int = 32
    scale_kind: int = abi.SCALE_E8M0

    @staticmethod
    def fp8_e4m3_with_e8m0_scale(out_features, in_features, block_m=128, block_k=128):
        return HipArtifactLinearShape(abi.WEIGHT_FP8_E4M3, out_features, in_features, block_m, block_k,
                                      abi.SCALE_E8M0)

    @staticmethod
    def fp8_e4m3_with_f32_scale(out_features, in_features, block_m=128, block_k=128):
        return HipArtifactLinearShape(abi.WEIGHT_FP8_E4M3, out_features, in_features, block_m, block_k,
                                      abi.SCALE_F32)

    @staticmethod
    def fp4_e2m1_packed_with_e8m0_scale(out_features, in_features):
        return HipArtifactLinearShape(abi.WEIGHT_MXFP4_E2M1, out_features, in_features, 1, 32,
                                      abi.SCALE_E8M0)

    @property
    def scale_rows(self) -> int:
        return -(-self.out_features // self.block_m)

    @property
    def scale_cols(self) -> int:
        return -(-self.in_features // self.block_k)

    def storage_lengths(self) -> tuple[int, int]:
        """(weight bytes, scale bytes) - context.rs:433-527."""
        if self.in_features == 0 or self.out_features == 0 or self.block_m == 0 or self.block_k == 0:
            raise ValueError(f"invalid HIP artifact linear shape: {self}")
        if self.weight_format == abi.WEIGHT_MXFP4_E2M1:
            if self.in_features % 32 or self.in_features % 2:
                raise ValueError(f"invalid HIP FP4 artifact linear shape: out={self.out_features} "
                                 f"in={self.in_features}")
            return self.out_features * (self.in_features // 2), self.out_features * (self.in_features // 32)
        scale_elems = self.scale_rows * self.scale_cols
        return self.out_features * self.in_features, scale_elems * (4 if self.scale_kind == abi.SCALE_F32 else 1)


@dataclass
class HipArtifactLinearHandle:
    """Device-resident weight + scale bytes (context.rs ``CudaArtifactLinearHandle``)."""

    shape: HipArtifactLinearShape
    weight: torch.Tensor   # uint8
    scale: torch.Tensor    # uint8 (E8M0) or float32
    # True once ``prepare_mxfp4_block_major`` has reordered the bytes: only the decode MoE
    # layer reads that order
    block_major: bool = False


def _ptr(t: torch.Tensor | None) -> int:
    return 0 if t is None else t.data_ptr()


def validate_dsv4_router_token_ids(token_ids, hash_rows: int) -> list[int]:
    """context.rs:1861-1891: every id must address a row of the hash table."""
    token_ids = [int(t) for t in token_ids]
    if not token_ids or hash_rows == 0:
        raise ValueError(f"HIP DSV4 hash router requires non-empty token ids and hash rows, got "
                         f"tokens={len(token_ids)} rows={hash_rows}")
    for row, token_id in enumerate(token_ids):
        if token_id < 0 or token_id >= hash_rows:
            raise ValueError(f"HIP DSV4 hash router token id {token_id} at batch row {row} exceeds hash rows "
                             f"{hash_rows}")
        if token_id > 0x7fffffff:
            raise ValueError(f"HIP DSV4 hash router token id {token_id} at batch row {row} does not fit i32")
    return token_ids


def validate_dsv4_router_hash_table(table, rows: int, cols: int, experts: int, top_k: int) -> list[int]:
    """context.rs:1893-1950: shape, top_k range, and for every row the first top_k ids in range
    and distinct."""
    table = [int(v) for v in table]
    if rows == 0 or cols == 0 or len(table) != rows * cols:
        raise ValueError(f"HIP DSV4 hash router table shape mismatch: values={len(table)} rows={rows} cols={cols}")
    if top_k == 0 or top_k > cols or top_k > experts or top_k > abi.ROUTER_MAX_TOP_K:
        raise ValueError(f"HIP DSV4 hash router requires top_k in 1..={min(cols, experts, abi.ROUTER_MAX_TOP_K)}, "
                         f"got {top_k}")
    for row in range(rows):
        selected = table[row * cols:row * cols + top_k]
        for slot, expert in enumerate(selected):
            if expert < 0 or expert >= experts:
                raise ValueError(f"HIP DSV4 hash router expert id {expert} at table row {row} slot {slot} exceeds "
                                 f"expert count {experts}")
            if expert in selected[:slot]:
                raise ValueError(f"HIP DSV4 hash router duplicate expert id {expert} at table row {row} within "
                                 f"top_k {top_k}")
    for index, expert in enumerate(table):
        if expert > 0x7fffffff:
            raise ValueError(f"HIP DSV4 hash router table value {expert} at flat index {index} does not fit i32")
    return table


@dataclass
class HipDsv4RouterHashTable:
    """context.rs ``CudaDsv4RouterHashTable``: validated int32 [rows, cols] on the device."""
    buffer: torch.Tensor
    rows: int
    cols: int


I32_MAX = 0x7fffffff


@dataclass(frozen=True)
class HipExpertSlotPointers:
    """context.rs:1952-1970: the six device addresses of one resident expert."""
    gate_weight: int = 0
    gate_scale: int = 0
    up_weight: int = 0
    up_scale: int = 0
    down_weight: int = 0
    down_scale: int = 0

    def is_complete(self) -> bool:
        return all(self.as_tuple())

    def as_tuple(self) -> tuple[int, ...]:
        return (self.gate_weight, self.gate_scale, self.up_weight, self.up_scale, self.down_weight, self.down_scale)

    @staticmethod
    def from_handles(gate: "HipArtifactLinearHandle", up: "HipArtifactLinearHandle",
                     down: "HipArtifactLinearHandle") -> "HipExpertSlotPointers":
        return HipExpertSlotPointers(gate.weight.data_ptr(), gate.scale.data_ptr(), up.weight.data_ptr(),
                                     up.scale.data_ptr(), down.weight.data_ptr(), down.scale.data_ptr())


@dataclass(frozen=True)
class HipExpertSlotBinding:
    """context.rs:1972-1976."""
    slot: int
    generation: int


class HipExpertSlotTableHost:
    """Host mirror of one layer's stable expert slot table, ``CudaExpertSlotTableHost``
    (context.rs:1978-2293): which expert sits in which slot at which generation.  A slot's
    generation advances on every eviction, so a (slot, generation) pair handed out earlier can
    be recognised as stale.  Every method either applies completely or raises and changes
    nothing."""

    _FIELDS = ("gate_weight", "gate_scale", "up_weight", "up_scale", "down_weight", "down_scale")

    def __init__(self, expert_capacity: int, slot_capacity: int):
        if expert_capacity == 0 or slot_capacity == 0:
            raise ValueError(f"HIP expert slot table requires positive capacities: experts={expert_capacity} "
                             f"slots={slot_capacity}")
        self.pointers = [HipExpertSlotPointers() for _ in range(slot_capacity)]
        self.expert_to_slot = [-1] * expert_capacity
        self.expert_generation = [0] * expert_capacity
        self.slot_generation = [0] * slot_capacity

    def clone(self) -> "HipExpertSlotTableHost":
        other = HipExpertSlotTableHost(len(self.expert_to_slot), len(self.slot_generation))
        other.pointers, other.expert_to_slot = list(self.pointers), list(self.expert_to_slot)
        other.expert_generation, other.slot_generation = list(self.expert_generation), list(self.slot_generation)
        return other

    def __eq__(self, other) -> bool:
        return isinstance(other, HipExpertSlotTableHost) and \
            (self.pointers, self.expert_to_slot, self.expert_generation, self.slot_generation) == \
            (other.pointers, other.expert_to_slot, other.expert_generation, other.slot_generation)

    def expert_capacity(self) -> int:
        return len(self.expert_to_slot)

    def slot_capacity(self) -> int:
        return len(self.slot_generation)

    def binding(self, expert: int) -> HipExpertSlotBinding | None:
        if not 0 <= expert < self.expert_capacity():
            return None
        slot = self.expert_to_slot[expert]
        if slot < 0 or slot >= self.slot_capacity():
            return None
        generation = self.expert_generation[expert]
        if generation > 0 and generation == self.slot_generation[slot]:
            return HipExpertSlotBinding(slot, generation)
        return None

    def is_current(self, binding: HipExpertSlotBinding) -> bool:
        return 0 <= binding.slot < self.slot_capacity() and self.slot_generation[binding.slot] == binding.generation

    def pointers_at(self, slot: int) -> HipExpertSlotPointers:
        return self.pointers[slot]

    def _exact_coordinates(self, expert: int, slot: int, generation: int) -> None:
        if not 0 <= expert < self.expert_capacity():
            raise ValueError(f"HIP expert id {expert} exceeds slot table capacity {self.expert_capacity()}")
        if not 0 <= slot < self.slot_capacity():
            raise ValueError(f"HIP expert slot {slot} exceeds slot table capacity {self.slot_capacity()}")
        if not 0 < generation <= I32_MAX:
            raise ValueError(f"HIP expert slot generation must be positive and fit i32, got {generation}")

    def install_at(self, expert: int, slot: int, generation: int,
                   pointers: HipExpertSlotPointers) -> HipExpertSlotBinding:
        """context.rs:2089-2166: install at coordinates chosen elsewhere (a prepared replacement)."""
        self._exact_coordinates(expert, slot, generation)
        if not pointers.is_complete():
            raise ValueError("HIP expert slot table requires a complete non-null weight/scale pointer tuple")
        if self.expert_to_slot[expert] >= 0:
            current = self.binding(expert)
            if current is None:
                raise ValueError(f"HIP expert {expert} has an inconsistent existing slot binding")
            if current.slot == slot and current.generation == generation:
                if self.pointers[slot] != pointers:
                    raise ValueError(f"HIP expert {expert} slot {slot} generation {generation} is already installed "
                                     "with a different pointer tuple")
                return current
            raise ValueError(f"HIP expert {expert} is already bound to slot {current.slot} generation "
                             f"{current.generation}, not slot {slot} generation {generation}")
        if slot in self.expert_to_slot:
            raise ValueError(f"HIP expert slot {slot} is already bound to expert {self.expert_to_slot.index(slot)}")
        held = self.slot_generation[slot]
        if held == I32_MAX:
            raise ValueError("HIP expert slot generation exhausted")
        expected = 1 if held == 0 else held
        if generation != expected:
            raise ValueError(f"HIP expert slot {slot} expected generation {expected}, got {generation}")
        self.slot_generation[slot] = generation
        self.expert_to_slot[expert] = slot
        self.expert_generation[expert] = generation
        self.pointers[slot] = pointers
        return HipExpertSlotBinding(slot, generation)

    def evict_binding(self, expert: int, slot: int, generation: int) -> None:
        """context.rs:2168-2201: evict exactly this binding; the slot's generation advances."""
        self._exact_coordinates(expert, slot, generation)
        current = self.binding(expert)
        if current is None or current.slot != slot or current.generation != generation:
            raise ValueError(f"HIP expert slot eviction rejected stale binding: expert {expert} slot {slot} "
                             f"generation {generation}")
        if generation + 1 > I32_MAX:
            raise ValueError("HIP expert slot generation exhausted")
        self.expert_to_slot[expert] = -1
        self.expert_generation[expert] = 0
        self.pointers[slot] = HipExpertSlotPointers()
        self.slot_generation[slot] = generation + 1

    def install(self, expert: int, pointers: HipExpertSlotPointers) -> HipExpertSlotBinding:
        """context.rs:2203-2262: first free slot whose generation can still advance."""
        current = self.binding(expert)
        if current is not None:
            return current
        if not 0 <= expert < self.expert_capacity():
            raise ValueError(f"HIP expert id {expert} exceeds slot table capacity {self.expert_capacity()}")
        used = [False] * self.slot_capacity()
        for slot in self.expert_to_slot:
            if 0 <= slot < len(used):
                used[slot] = True
        free = [slot for slot, taken in enumerate(used) if not taken]
        usable = [slot for slot in free if self.slot_generation[slot] < I32_MAX - 1]
        if not usable:
            raise ValueError("HIP expert slot generation exhausted" if free else "HIP expert slot table is full")
        slot = usable[0]
        generation = self.slot_generation[slot] + 1
        self.slot_generation[slot] = generation
        self.expert_to_slot[expert] = slot
        self.expert_generation[expert] = generation
        self.pointers[slot] = pointers
        return HipExpertSlotBinding(slot, generation)

    def evict(self, expert: int) -> bool:
        """context.rs:2264-2284."""
        current = self.binding(expert)
        if current is None:
            return False
        if self.slot_generation[current.slot] + 1 > I32_MAX:
            raise ValueError("HIP expert slot generation exhausted")
        self.expert_to_slot[expert] = -1
        self.expert_generation[expert] = 0
        self.pointers[current.slot] = HipExpertSlotPointers()
        self.slot_generation[current.slot] += 1
        return True


class HipExpertSlotTable:
    """``CudaExpertSlotTable`` (context.rs:2449-2545 reduced to the synchronous path): the stable
    device arrays plus their authoritative host mirror.  The array attributes carry the names
    the MoE entry points of this module read from a table, so a slot table can stand where a
    ``HipRoutedExpertTable`` does."""

    def __init__(self, expert_capacity: int, slot_capacity: int, device):
        self.host = HipExpertSlotTableHost(expert_capacity, slot_capacity)
        self.slot_capacity, self.expert_capacity, self.device = slot_capacity, expert_capacity, device
        z = lambda: torch.zeros(slot_capacity, dtype=torch.int64, device=device)
        self.gate_ptrs, self.gate_scale_ptrs = z(), z()
        self.up_ptrs, self.up_scale_ptrs = z(), z()
        self.down_ptrs, self.down_scale_ptrs = z(), z()
        self.expert_to_slot = torch.full((expert_capacity,), -1, dtype=torch.int32, device=device)
        self.expert_generations = torch.zeros(expert_capacity, dtype=torch.int32, device=device)
        self.slot_generations = torch.zeros(slot_capacity, dtype=torch.int32, device=device)
        self.block_major: bool | None = None
        self.keepalive: dict[int, tuple] = {}


@dataclass
class HipExpertRouteResolveWorkspace:
    """context.rs:3015-3045: outputs of a resolve, allocated once."""
    route_slots: torch.Tensor
    route_generations: torch.Tensor
    miss_markers: torch.Tensor
    miss_control: torch.Tensor
    miss_capacity: int
    route_capacity: int


@dataclass
class HipExpertRouteResolveResult:
    """context.rs ``CudaExpertRouteResolveResult``."""
    route_slots: list
    route_generations: list
    miss_markers: list
    miss_ids: list
    miss_overflow: bool


class HipRoutedExpertTable:
    """Device-resident expert slot table: six pointer arrays indexed by slot plus the slot
    generations, the layout the reference's grouped MoE consumes
    (abi/cutlass_provider.h:355-364; host side context.rs:1952-2296, reduced here to
    install/evict because residency policy is outside this provider)."""

    def __init__(self, slot_capacity: int, device):
        self.slot_capacity = slot_capacity
        self.device = device
        z = lambda: torch.zeros(slot_capacity, dtype=torch.int64, device=device)
        self.gate_ptrs, self.gate_scale_ptrs = z(), z()
        self.up_ptrs, self.up_scale_ptrs = z(), z()
        self.down_ptrs, self.down_scale_ptrs = z(), z()
        self.slot_generations = torch.zeros(slot_capacity, dtype=torch.int32, device=device)
        self._keepalive: dict[int, tuple] = {}
        self._host = {name: [0] * slot_capacity for name in
                      ("gate", "gate_scale", "up", "up_scale", "down", "down_scale", "generation")}
        # storage order of every installed expert (None while the table is empty): the kernels
        # take one order for the whole table
        self.block_major: bool | None = None

    def install(self, slot: int, gate: HipArtifactLinearHandle, up: HipArtifactLinearHandle,
                down: HipArtifactLinearHandle, generation: int = 1) -> None:
        if not 0 <= slot < self.slot_capacity or generation <= 0:
            raise ValueError("invalid expert slot or generation")
        for h in (gate, up, down):
            if h.shape.weight_format != abi.WEIGHT_MXFP4_E2M1:
                raise ValueError("routed experts are MXFP4 artifacts")
        order = gate.block_major
        if up.block_major != order or down.block_major != order or \
                (self._keepalive and self.block_major is not None and self.block_major != order):
            raise ValueError("all experts of a table share one weight order (row-major or block-major)")
        self.block_major = order
        self._keepalive[slot] = (gate, up, down)
        hst = self._host
        hst["gate"][slot], hst["gate_scale"][slot] = gate.weight.data_ptr(), gate.scale.data_ptr()
        hst["up"][slot], hst["up_scale"][slot] = up.weight.data_ptr(), up.scale.data_ptr()
        hst["down"][slot], hst["down_scale"][slot] = down.weight.data_ptr(), down.scale.data_ptr()
        hst["generation"][slot] = generation

    def evict(self, slot: int) -> None:
        self._keepalive.pop(slot, None)
        for name in self._host:
            self._host[name][slot] = 0

    def commit(self) -> None:
        """Upload the host copy of the table (one small H2D per array)."""
        pairs = (("gate", self.gate_ptrs), ("gate_scale", self.gate_scale_ptrs), ("up", self.up_ptrs),
                 ("up_scale", self.up_scale_ptrs), ("down", self.down_ptrs),
                 ("down_scale", self.down_scale_ptrs))
        for name, dev in pairs:
            dev.copy_(torch.tensor(self._host[name], dtype=torch.int64))
        self.slot_generations.copy_(torch.tensor(self._host["generation"], dtype=torch.int32))


class HipExpertGroupRoutePlan:
    """Buffers of ``CudaExpertGroupRoutePlan`` (context.rs:1651-1681) that this provider's
    kernels read or write; allocated once, reused for every invocation."""

    def __init__(self, ctx: "HipArtifactOperatorContext", max_experts: int, route_capacity: int,
                 tokens: int, input_size: int, intermediate_size: int, hidden_size: int):
        # context.rs:8956-8994
        if max_experts == 0 or max_experts > 512:
            raise ValueError(f"HIP expert group route plan expects 1..=512 slots, got {max_experts}")
        if route_capacity == 0 or tokens == 0:
            raise ValueError("HIP expert group route capacity and token count must be positive")
        if input_size == 0 or intermediate_size == 0 or hidden_size == 0:
            raise ValueError("HIP expert group route plan invalid shape")
        if input_size % 64 or intermediate_size % 64 or hidden_size % 4:
            raise ValueError("grouped FP4 MoE expects input/intermediate multiples of 64 and hidden a "
                             "multiple of 4")
        dev = ctx.device
        i32 = lambda n: torch.zeros(n, dtype=torch.int32, device=dev)
        self.max_experts, self.route_capacity, self.tokens = max_experts, route_capacity, tokens
        self.input_size, self.intermediate_size, self.hidden_size = input_size, intermediate_size, hidden_size
        self.slot_counts, self.slot_route_offsets, self.slot_cursors = i32(max_experts), i32(max_experts), i32(max_experts)
        self.active_expert_slots, self.active_group_generations = i32(max_experts), i32(max_experts)
        self.expert_route_indptr, self.expert_route_counts = i32(max_experts + 1), i32(max_experts)
        self.route_token_indices, self.route_indices = i32(route_capacity), i32(route_capacity)
        self.route_weights = torch.zeros(route_capacity, dtype=torch.float32, device=dev)
        self.host_scalars = i32(4)
        self.route_written, self.route_error = i32(route_capacity), i32(1)
        self.route_output = torch.zeros((route_capacity, hidden_size), dtype=torch.float32, device=dev)
        self.invocation_routes: int | None = None
        self.routes_per_token = 0
        self.host_active_groups = None   # set by prepare_decode_route_plan from the host's slot ids
        self.workspace: torch.Tensor | None = None
        self.grouped_workspace: torch.Tensor | None = None

    def host_metadata(self) -> dict:
        """The 16-byte scalar readback of context.rs:9401-9410 (synchronises; optional here)."""
        g, s, m, t = self.host_scalars.cpu().tolist()
        return {"active_group_count": g, "small_group_count": s, "max_group_rows": m, "total_routed_rows": t}


class HipArtifactOperatorContext:
    """One owner thread, one device, borrowed stream - as the reference's context
    (context.rs:2546-2589).  ``stream`` defaults to torch's current stream."""

    def __init__(self, device: int | str | torch.device = 0, stream: torch.cuda.Stream | None = None):
        if not torch.cuda.is_available():
            raise RuntimeError("HipArtifactOperatorContext needs a GPU (no CPU path exists)")
        self.lib = abi.load()
        self.device = torch.device("cuda", device) if isinstance(device, int) else torch.device(device)
        self._stream = stream
        self.manifest = self.lib.ferrule_hip_provider_manifest().kernel_mask
        self.kernel_launches = 0      # counterpart of CudaOpCounters.kernel_launches

    # -- plumbing ---------------------------------------------------------
    @property
    def stream(self) -> torch.cuda.Stream:
        return self._stream if self._stream is not None else torch.cuda.current_stream(self.device)

    def stream_handle(self) -> int:
        """``stream.cu_stream() as usize as u64`` (kernels.rs:547-553)."""
        return int(self.stream.cuda_stream)

    def supports(self, kernel_id: int) -> bool:
        return bool(self.manifest & abi.kernel_bit(kernel_id))

    def _two_phase(self, what: str, can_implement, launch, args) -> None:
        """``can_implement`` then ``launch`` (cutlass.rs:2851-2861)."""
        args.stream = self.stream_handle()
        status = can_implement(C.byref(args))
        if status != abi.SUCCESS:
            raise ProviderError(f"validate {what}", status)
        status = launch(C.byref(args))
        if status != abi.SUCCESS:
            raise ProviderError(f"launch {what}", status)
        self.kernel_launches += 1

    # -- uploads ----------------------------------------------------------
    def upload_artifact_linear(self, shape: HipArtifactLinearShape, weight, scale) -> HipArtifactLinearHandle:
        """Copy host bytes to the device after the same length checks as
        context.rs:5049-5135."""
        wb, sb = shape.storage_lengths()
        w = torch.as_tensor(weight).contiguous().view(torch.uint8).reshape(-1)
        s = torch.as_tensor(scale).contiguous()
        s_bytes = s.numel() * s.element_size()
        if w.numel() != wb or s_bytes != sb:
            raise ValueError(f"artifact linear payload length mismatch: weight {w.numel()} vs {wb}, "
                             f"scale {s_bytes} vs {sb}")
        if shape.scale_kind == abi.SCALE_F32 and s.dtype != torch.float32:
            raise ValueError("F32 scale kind needs a float32 scale tensor")
        return HipArtifactLinearHandle(shape, w.to(self.device), s.reshape(-1).to(self.device))

    @staticmethod
    def _require_row_major(handle: HipArtifactLinearHandle) -> None:
        if handle.block_major:
            raise ValueError("this operator reads the row-major artifact order, the handle is block-major")

    # -- decode GEMV ------------------------------------------------------
    def _gemv_args(self, handle: HipArtifactLinearHandle, x: torch.Tensor | None,
                   out: torch.Tensor, flags: int = 0) -> abi.QuantGemvArgs:
        sh = handle.shape
        if handle.block_major:
            if x is None:
                self._require_row_major(handle)      # the dequantiser reads the artifact order
            flags |= abi.GEMV_BLOCK_MAJOR_WEIGHTS
        a = abi.QuantGemvArgs()
        a.weight_format, a.scale_kind = sh.weight_format, sh.scale_kind
        a.batch = 0 if x is None else x.shape[0]
        a.n, a.k = sh.out_features, sh.in_features
        a.block_m, a.block_k, a.scale_cols = sh.block_m, sh.block_k, sh.scale_cols
        a.flags = flags
        a.x, a.weight, a.weight_scales, a.output = _ptr(x), _ptr(handle.weight), _ptr(handle.scale), _ptr(out)
        a.stream = self.stream_handle()
        return a

    def artifact_linear_gemv_bf16_into(self, handle: HipArtifactLinearHandle, x: torch.Tensor,
                                       out: torch.Tensor) -> torch.Tensor:
        """y[b,:] = bf16(W_dequant @ x[b,:]) for BF16 activations.  The decode
        counterpart of ``artifact_linear_matvec_into`` (context.rs:5726-5759), which
        the reference only has for f32 activations and not at all for FP4
        (context.rs:10909-10911)."""
        sh = handle.shape
        if x.dtype != torch.bfloat16 or x.dim() != 2 or x.shape[1] != sh.in_features or not x.is_contiguous():
            raise ValueError(f"linear input must be contiguous bf16 [batch, {sh.in_features}], got "
                             f"{x.dtype} {tuple(x.shape)}")
        flags = 0
        if out.dtype == torch.float32:
            flags |= abi.GEMV_OUTPUT_F32
        elif out.dtype != torch.bfloat16:
            raise ValueError("linear output must be bf16 or f32")
        if tuple(out.shape) != (x.shape[0], sh.out_features) or not out.is_contiguous():
            raise ValueError(f"linear output length mismatch: expected {(x.shape[0], sh.out_features)}, "
                             f"got {tuple(out.shape)}")
        args = self._gemv_args(handle, x, out, flags)
        self._two_phase("quantized GEMV", self.lib.ferrule_hip_quant_gemv_can_implement,
                        self.lib.ferrule_hip_quant_gemv_launch, args)
        return out

    def artifact_linears_gemv_bf16_into(self, handles, xs, outs) -> None:
        """Several independent decode linears in ONE launch (the role of the reference's
        ``dual_linear`` / ``grouped_linear`` entries, kernels.rs:578-640): ``handles[i]`` applied to
        ``xs[i]`` into ``outs[i]``.  All weights share format, scale kind and storage order; results
        equal the single launches bit for bit."""
        if not (len(handles) == len(xs) == len(outs)) or not 1 <= len(handles) <= abi.GEMV_MULTI_MAX:
            raise ValueError(f"1..{abi.GEMV_MULTI_MAX} matrices with one input and one output each")
        blocks = (abi.QuantGemvArgs * len(handles))()
        for i, (handle, x, out) in enumerate(zip(handles, xs, outs)):
            sh = handle.shape
            if x.dtype != torch.bfloat16 or x.dim() != 2 or x.shape[1] != sh.in_features or not x.is_contiguous():
                raise ValueError(f"linear input {i} must be contiguous bf16 [batch, {sh.in_features}]")
            if out.dtype not in (torch.float32, torch.bfloat16) or tuple(out.shape) != (x.shape[0], sh.out_features) \
                    or not out.is_contiguous():
                raise ValueError(f"linear output {i} must be contiguous bf16 or f32 {(x.shape[0], sh.out_features)}")
            args = self._gemv_args(handle, x, out, abi.GEMV_OUTPUT_F32 if out.dtype == torch.float32 else 0)
            args.stream = self.stream_handle()
            blocks[i] = args
        multi = abi.QuantGemvMultiArgs(count=len(handles), matrices=C.addressof(blocks))
        status = self.lib.ferrule_hip_quant_gemv_multi_can_implement(C.byref(multi))
        if status != abi.SUCCESS:
            raise ProviderError("validate quantized multi-GEMV", status)
        status = self.lib.ferrule_hip_quant_gemv_multi_launch(C.byref(multi))
        if status != abi.SUCCESS:
            raise ProviderError("launch quantized multi-GEMV", status)
        self.kernel_launches += 1

    def dense_ffn_decode(self, gate: HipArtifactLinearHandle, up: HipArtifactLinearHandle,
                         down: HipArtifactLinearHandle, x: torch.Tensor, out: torch.Tensor | None = None,
                         output_scale: float = 1.0, swiglu_limit: float = 0.0, out_dtype=torch.bfloat16,
                         hidden: torch.Tensor | None = None):
        """Dense SwiGLU FFN for a decode batch (``SwiGluFfn::reference_execute``, ffn.rs:24-48) in two
        HBM-bound launches: gate and up as two matrices of one GEMV launch, then down, which forms
        silu(gate) * up * scale from the two sums on the way in.  Returns (output, sums) with
        sums f32 [2, batch, intermediate]: the gate sums and the up sums."""
        sg, su, sd = gate.shape, up.shape, down.shape
        if (sg.out_features, sg.in_features) != (su.out_features, su.in_features) or sd.in_features != sg.out_features:
            raise ValueError("SwiGLU gate/up/down shapes do not chain")
        for h in (up, down):
            if (h.shape.weight_format, h.shape.scale_kind, h.shape.block_m, h.shape.block_k, h.block_major) != \
                    (sg.weight_format, sg.scale_kind, sg.block_m, sg.block_k, gate.block_major):
                raise ValueError("the three linears of a dense FFN share format, scale kind, blocks and weight order")
        if x.dtype != torch.bfloat16 or x.dim() != 2 or x.shape[1] != sg.in_features or not x.is_contiguous():
            raise ValueError(f"FFN input must be contiguous bf16 [batch, {sg.in_features}]")
        batch = x.shape[0]
        if out is None:
            out = torch.empty((batch, sd.out_features), dtype=out_dtype, device=self.device)
        if out.dtype not in (torch.bfloat16, torch.float32) or tuple(out.shape) != (batch, sd.out_features):
            raise ValueError("FFN output must be bf16 or f32 [batch, output]")
        if hidden is None:
            hidden = torch.empty((2, batch, sg.out_features), dtype=torch.float32, device=self.device)
        if hidden.dtype != torch.float32 or hidden.numel() != 2 * batch * sg.out_features or not hidden.is_contiguous():
            raise ValueError("FFN scratch must be contiguous f32 [2, batch, intermediate]")
        flags = (abi.GEMV_OUTPUT_F32 if out.dtype == torch.float32 else 0) | \
            (abi.GEMV_BLOCK_MAJOR_WEIGHTS if gate.block_major else 0)
        a = abi.DenseFfnDecodeArgs(
            weight_format=sg.weight_format, scale_kind=sg.scale_kind, batch=batch, input_size=sg.in_features,
            intermediate_size=sg.out_features, output_size=sd.out_features, block_m=sg.block_m, block_k=sg.block_k,
            flags=flags, swiglu_limit=swiglu_limit, output_scale=output_scale, x=_ptr(x),
            gate_weight=_ptr(gate.weight), gate_scales=_ptr(gate.scale), up_weight=_ptr(up.weight),
            up_scales=_ptr(up.scale), down_weight=_ptr(down.weight), down_scales=_ptr(down.scale),
            hidden_f32=_ptr(hidden), output=_ptr(out))
        self._two_phase("dense FFN decode", self.lib.ferrule_hip_dense_ffn_decode_can_implement,
                        self.lib.ferrule_hip_dense_ffn_decode_launch, a)
        self.kernel_launches += 2
        return out, hidden

    def artifact_linear_gemv_bf16(self, handle: HipArtifactLinearHandle, x: torch.Tensor,
                                  out_dtype=torch.bfloat16) -> torch.Tensor:
        out = torch.empty((x.shape[0], handle.shape.out_features), dtype=out_dtype, device=self.device)
        return self.artifact_linear_gemv_bf16_into(handle, x, out)

    def artifact_linear_dequantize(self, handle: HipArtifactLinearHandle) -> torch.Tensor:
        """f32 [n,k] through the device converters (diagnostic / parity entry)."""
        sh = handle.shape
        out = torch.empty((sh.out_features, sh.in_features), dtype=torch.float32, device=self.device)
        args = self._gemv_args(handle, None, out)
        status = self.lib.ferrule_hip_dequant_launch(C.byref(args))
        if status != abi.SUCCESS:
            raise ProviderError("launch dequantize", status)
        self.kernel_launches += 1
        return out

    # -- drop-ins for the reference's core linear / quantize ops --------------
    def _core(self, what: str, fn, args) -> None:
        """``invoke!`` of kernels.rs:555-576: write the stream, call, map a non-zero
        hipError_t to an exception."""
        args.stream = self.stream_handle()
        status = fn(C.byref(args))
        if status != 0:
            raise ProviderError(f"core {what}", status)
        self.kernel_launches += 1

    def pack_fp8_rows_from_f32(self, values: torch.Tensor, block_size: int = 128,
                               rounding: int = abi.FP8_ROUND_CPU_REFERENCE):
        """f32 [rows, width] -> (e4m3 [rows, width], e8m0 [rows, width/block]).
        Counterpart of ``pack_fp8_rows_from_f32_preallocated`` (context.rs:10694-10741)."""
        if values.dtype != torch.float32 or values.dim() != 2 or not values.is_contiguous():
            raise ValueError("pack_fp8_rows_from_f32 expects contiguous f32 [rows, width]")
        rows, width = values.shape
        if width % block_size:
            raise ValueError(f"row width {width} is not a multiple of block {block_size}")
        packed = torch.empty((rows, width), dtype=torch.uint8, device=self.device)
        scales = torch.empty((rows, width // block_size), dtype=torch.uint8, device=self.device)
        a = abi.QuantizeArgs(kind=abi.QUANTIZE_FP8_PACKED, value_offset=0, value_len=rows * width,
                             row_width=width, block_size=block_size, rope_dim=0, reserved=rounding,
                             values=_ptr(values), packed=_ptr(packed), scales=_ptr(scales))
        self._core("FP8 pack", self.lib.ferrule_hip_core_quantize_launch, a)
        return packed, scales

    def pack_fp4_rows_from_f32(self, values: torch.Tensor, block_size: int = 32,
                               rounding: int = abi.FP8_ROUND_CPU_REFERENCE):
        """f32 [rows, width] -> (e2m1 [rows, width/2], e8m0 [rows, width/block]); the
        reference's ``fp4_e2m1_e8m0_quantize_f32_packed`` (kernels.rs, kind 4)."""
        if values.dtype != torch.float32 or values.dim() != 2 or not values.is_contiguous():
            raise ValueError("pack_fp4_rows_from_f32 expects contiguous f32 [rows, width]")
        rows, width = values.shape
        if width % block_size or block_size % 2:
            raise ValueError(f"row width {width} is not a multiple of block {block_size}")
        packed = torch.empty((rows, width // 2), dtype=torch.uint8, device=self.device)
        scales = torch.empty((rows, width // block_size), dtype=torch.uint8, device=self.device)
        a = abi.QuantizeArgs(kind=abi.QUANTIZE_FP4_PACKED, value_offset=0, value_len=rows * width,
                             row_width=width, block_size=block_size, rope_dim=0, reserved=rounding,
                             values=_ptr(values), packed=_ptr(packed), scales=_ptr(scales))
        self._core("FP4 pack", self.lib.ferrule_hip_core_quantize_launch, a)
        return packed, scales

    def artifact_linear_matvec_into(self, handle: HipArtifactLinearHandle, x: torch.Tensor,
                                    out: torch.Tensor, quantize_input: bool = False) -> torch.Tensor:
        """f32 activations -> f32 outputs for an FP8/E8M0 artifact (context.rs:5726-5759:
        kind 8 when the caller wants the K-block activation quantization, else kind 4)."""
        sh = handle.shape
        self._require_row_major(handle)
        if sh.weight_format != abi.WEIGHT_FP8_E4M3 or sh.scale_kind != abi.SCALE_E8M0:
            raise ProviderError("artifact_linear_matvec_into (FP8/E8M0 artifacts only)", abi.UNSUPPORTED)
        if x.dtype != torch.float32 or x.dim() != 2 or x.shape[1] != sh.in_features or not x.is_contiguous():
            raise ValueError("linear input must be contiguous f32 [batch, in_features]")
        if out.dtype != torch.float32 or tuple(out.shape) != (x.shape[0], sh.out_features):
            raise ValueError("linear output must be f32 [batch, out_features]")
        kind = abi.LINEAR_FP8_E4M3_E8M0_FROM_F32 if quantize_input else abi.LINEAR_FP8_E4M3_E8M0
        a = abi.LinearArgs(kind=kind, batch=x.shape[0], n=sh.out_features, k=sh.in_features,
                           scale_cols=sh.scale_cols, block_m=sh.block_m, block_k=sh.block_k,
                           x=_ptr(x), x_scales=0, weight=_ptr(handle.weight),
                           weight_scales=_ptr(handle.scale), output=_ptr(out))
        self._core("linear", self.lib.ferrule_hip_core_linear_launch, a)
        return out

    def gemm_fp8_e4m3fn_e8m0_prepacked(self, handle: HipArtifactLinearHandle, x_packed: torch.Tensor,
                                       x_scales: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        """e4m3 activations + per-K128 e8m0 scales -> f32 (kind 5; the reference's
        ``gemm_fp8_e4m3fn_e8m0_prepacked``, context.rs:10766-10785)."""
        sh = handle.shape
        self._require_row_major(handle)
        a = abi.LinearArgs(kind=abi.LINEAR_FP8_E4M3_E8M0_PACKED, batch=x_packed.shape[0], n=sh.out_features,
                           k=sh.in_features, scale_cols=sh.in_features // 128, block_m=128, block_k=128,
                           x=_ptr(x_packed), x_scales=_ptr(x_scales), weight=_ptr(handle.weight),
                           weight_scales=_ptr(handle.scale), output=_ptr(out))
        self._core("prepacked linear", self.lib.ferrule_hip_core_linear_launch, a)
        return out

    # -- packed verification / prefill GEMM on the scaled MFMA -----------------
    def fp8_projection(self, x_packed: torch.Tensor, x_scales: torch.Tensor, weight: torch.Tensor,
                       weight_scales: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        """E4M3 rows + UE8M0 K128 scales times an E4M3 weight with UE8M0 128x128 block scales ->
        f32 [rows, n] holding BF16-rounded values (``launch_fp8_projection``, cutlass.rs;
        ferrule_cutlass_fp8_projection_launch)."""
        rows, k = x_packed.shape
        n = weight.shape[0]
        if out is None:
            out = torch.empty((rows, n), dtype=torch.float32, device=self.device)
        a = abi.Fp8QueryAKvArgs(rows=rows, n1=n, n2=0, k=k, scale_cols=k // 128, activation_fp8=_ptr(x_packed),
                                activation_ue8m0=_ptr(x_scales), query_a_weight_fp8=_ptr(weight),
                                query_a_weight_ue8m0=_ptr(weight_scales), query_a_output_f32=_ptr(out))
        self._two_phase("fp8 projection", self.lib.ferrule_hip_fp8_projection_can_implement,
                        self.lib.ferrule_hip_fp8_projection_launch, a)
        return out

    def fp8_query_a_kv(self, x_packed, x_scales, w1, w1_scales, w2, w2_scales):
        """Both projections of one packed activation (ferrule_cutlass_fp8_query_a_kv_launch)."""
        rows, k = x_packed.shape
        out1 = torch.empty((rows, w1.shape[0]), dtype=torch.float32, device=self.device)
        out2 = torch.empty((rows, w2.shape[0]), dtype=torch.float32, device=self.device)
        a = abi.Fp8QueryAKvArgs(rows=rows, n1=w1.shape[0], n2=w2.shape[0], k=k, scale_cols=k // 128,
                                activation_fp8=_ptr(x_packed), activation_ue8m0=_ptr(x_scales),
                                query_a_weight_fp8=_ptr(w1), query_a_weight_ue8m0=_ptr(w1_scales),
                                kv_weight_fp8=_ptr(w2), kv_weight_ue8m0=_ptr(w2_scales),
                                query_a_output_f32=_ptr(out1), kv_output_f32=_ptr(out2))
        self._two_phase("fp8 query_a+kv", self.lib.ferrule_hip_fp8_query_a_kv_can_implement,
                        self.lib.ferrule_hip_fp8_query_a_kv_launch, a)
        return out1, out2

    def fp8_block_gemm(self, x_packed: torch.Tensor, x_scales: torch.Tensor, handle: HipArtifactLinearHandle,
                       out: torch.Tensor | None = None, out_dtype=torch.bfloat16,
                       tile_schedule: bool = False) -> torch.Tensor:
        """Packed rows times an FP8 artifact weight with E8M0 or F32 128x128 block scales.  The
        library chooses its schedule from the row count (up to 32 rows stream the weights, more run
        MFMA tiles; same bits); ``tile_schedule`` keeps the tiles, for comparisons."""
        sh = handle.shape
        self._require_row_major(handle)
        rows = x_packed.shape[0]
        if out is None:
            out = torch.empty((rows, sh.out_features), dtype=out_dtype, device=self.device)
        a = abi.Fp8BlockGemmArgs(rows=rows, n=sh.out_features, k=sh.in_features, scale_cols=sh.in_features // 128,
                                 weight_scale_kind=sh.scale_kind,
                                 flags=(abi.GEMM_OUTPUT_BF16 if out.dtype == torch.bfloat16 else 0) |
                                 (abi.GEMM_TILE_SCHEDULE if tile_schedule else 0),
                                 activation_fp8=_ptr(x_packed), activation_ue8m0=_ptr(x_scales),
                                 weight_fp8=_ptr(handle.weight), weight_scales=_ptr(handle.scale), output=_ptr(out))
        self._two_phase("fp8 block gemm", self.lib.ferrule_hip_fp8_block_gemm_can_implement,
                        self.lib.ferrule_hip_fp8_block_gemm_launch, a)
        return out

    def shared_ffn(self, x_packed: torch.Tensor, x_scales: torch.Tensor, gate: HipArtifactLinearHandle,
                   up: HipArtifactLinearHandle, down: HipArtifactLinearHandle, output: torch.Tensor,
                   output_scale: float = 1.0, swiglu_limit: float = 0.0, accumulate: bool = False,
                   tile_schedule: bool = False):
        """Dense FP8 SwiGLU FFN over packed rows into f32 ``output`` (``launch_shared_ffn``, cutlass.rs;
        ferrule_cutlass_shared_ffn_launch). Returns (hidden_f32, hidden_fp8, hidden_ue8m0), the compact
        intermediate storage the reference's caller also supplies.  Up to 32 rows take the decode-row
        schedule (three streaming launches) unless ``tile_schedule`` is set; the bits are the same."""
        for handle in (gate, up, down):
            self._require_row_major(handle)
        rows, k = x_packed.shape
        inter, out_features = gate.shape.out_features, down.shape.out_features
        hidden_f32 = torch.empty((rows, inter), dtype=torch.float32, device=self.device)
        hidden_fp8 = torch.empty((rows, inter), dtype=torch.uint8, device=self.device)
        hidden_s = torch.empty((rows, inter // 128), dtype=torch.uint8, device=self.device)
        a = abi.SharedFfnArgs(
            input_fp8=_ptr(x_packed), input_ue8m0=_ptr(x_scales), gate_weight_fp8=_ptr(gate.weight),
            gate_weight_ue8m0=_ptr(gate.scale), up_weight_fp8=_ptr(up.weight), up_weight_ue8m0=_ptr(up.scale),
            down_weight_fp8=_ptr(down.weight), down_weight_ue8m0=_ptr(down.scale), hidden_f32=_ptr(hidden_f32),
            hidden_fp8=_ptr(hidden_fp8), hidden_ue8m0=_ptr(hidden_s), output_f32=_ptr(output), rows=rows,
            input_size=k, intermediate_size=inter, output_size=out_features, gate_block_m=gate.shape.block_m,
            gate_block_k=gate.shape.block_k, up_block_m=up.shape.block_m, up_block_k=up.shape.block_k,
            down_block_m=down.shape.block_m, down_block_k=down.shape.block_k, output_scale=output_scale,
            swiglu_limit=swiglu_limit, flags=(abi.SHARED_FFN_ACCUMULATE if accumulate else 0) |
            (abi.SHARED_FFN_TILE_SCHEDULE if tile_schedule else 0))
        self._two_phase("shared FFN", self.lib.ferrule_hip_shared_ffn_can_implement,
                        self.lib.ferrule_hip_shared_ffn_launch, a)
        self.kernel_launches += 1
        return hidden_f32, hidden_fp8, hidden_s

    # -- expert slot table: router ids -> resident slots, on the device ---------------------
    def expert_slot_table(self, expert_capacity: int, slot_capacity: int) -> HipExpertSlotTable:
        """context.rs:2600-2640."""
        return HipExpertSlotTable(expert_capacity, slot_capacity, self.device)

    def _table_args(self, table: HipExpertSlotTable, kind: int, **kw) -> abi.ExpertTableArgs:
        return abi.ExpertTableArgs(
            kind=kind, expert_capacity=table.expert_capacity, slot_capacity=table.slot_capacity,
            gate_weights=_ptr(table.gate_ptrs), gate_scales=_ptr(table.gate_scale_ptrs),
            up_weights=_ptr(table.up_ptrs), up_scales=_ptr(table.up_scale_ptrs), down_weights=_ptr(table.down_ptrs),
            down_scales=_ptr(table.down_scale_ptrs), expert_to_slot=_ptr(table.expert_to_slot),
            expert_generations=_ptr(table.expert_generations), slot_generations=_ptr(table.slot_generations), **kw)

    def install_expert_slot(self, table: HipExpertSlotTable, expert: int, pointers: HipExpertSlotPointers,
                            keepalive: tuple = (), block_major: bool | None = None) -> HipExpertSlotBinding:
        """Bind ``expert`` to a free slot: the host mirror decides, ONE one-thread launch publishes
        it, no host-to-device copy (context.rs:2942-2985).  ``keepalive`` holds whatever owns the
        six addresses for as long as the binding lives."""
        current = table.host.binding(expert)
        if current is not None:
            return current
        if block_major is not None and table.keepalive and table.block_major not in (None, block_major):
            raise ValueError("all experts of a table share one weight order (row-major or block-major)")
        nxt = table.host.clone()
        binding = nxt.install(expert, pointers)
        g, gs, u, us, d, ds = pointers.as_tuple()
        a = self._table_args(table, abi.EXPERT_INSTALL, expert=expert, slot=binding.slot, generation=binding.generation,
                             gate_weight_value=g, gate_scale_value=gs, up_weight_value=u, up_scale_value=us,
                             down_weight_value=d, down_scale_value=ds)
        self._core("expert slot binding publication", self.lib.ferrule_hip_core_expert_table_launch, a)
        table.host = nxt
        table.keepalive[binding.slot] = keepalive
        if block_major is not None:
            table.block_major = block_major
        return binding

    def evict_expert_slot(self, table: HipExpertSlotTable, expert: int) -> bool:
        """context.rs:2987-3002 (through ``evict_expert_slot_binding``, :2904-2940)."""
        current = table.host.binding(expert)
        if current is None:
            return False
        nxt = table.host.clone()
        nxt.evict_binding(expert, current.slot, current.generation)
        a = self._table_args(table, abi.EXPERT_EVICT, expert=expert, slot=current.slot,
                             generation=nxt.slot_generation[current.slot])
        self._core("expert slot eviction", self.lib.ferrule_hip_core_expert_table_launch, a)
        table.host = nxt
        table.keepalive.pop(current.slot, None)
        return True

    def expert_route_resolve_workspace(self, route_capacity: int, miss_capacity: int) -> HipExpertRouteResolveWorkspace:
        """context.rs:3015-3045."""
        if route_capacity == 0 or miss_capacity == 0:
            raise ValueError(f"HIP expert route resolve requires positive capacities: routes={route_capacity} "
                             f"misses={miss_capacity}")
        z = lambda n: torch.zeros(n, dtype=torch.int32, device=self.device)
        return HipExpertRouteResolveWorkspace(z(route_capacity), z(route_capacity), z(route_capacity),
                                              z(2 + miss_capacity + route_capacity), miss_capacity, route_capacity)

    def resolve_expert_routes(self, table: HipExpertSlotTable, expert_ids: torch.Tensor, route_count: int,
                              workspace: HipExpertRouteResolveWorkspace) -> None:
        """Router expert ids -> (slot, generation) per route plus the bounded miss list, two
        launches, nothing leaves the device (context.rs:3047-3125)."""
        if route_count > expert_ids.numel() or route_count > workspace.route_capacity or \
                expert_ids.dtype != torch.int32:
            raise ValueError(f"HIP expert route resolve exceeds capacity: routes={route_count} "
                             f"ids={expert_ids.numel()} slots={workspace.route_capacity}")
        common = dict(route_count=route_count, miss_capacity=workspace.miss_capacity,
                      route_capacity=workspace.route_capacity, expert_ids=_ptr(expert_ids),
                      route_slots=_ptr(workspace.route_slots), route_generations=_ptr(workspace.route_generations),
                      miss_markers=_ptr(workspace.miss_markers), miss_control=_ptr(workspace.miss_control))
        fn = self.lib.ferrule_hip_core_expert_table_launch
        self._core("expert resolve init", fn, self._table_args(table, abi.EXPERT_INITIALIZE_RESOLVE, **common))
        self._core("expert resolve", fn, self._table_args(table, abi.EXPERT_RESOLVE, **common))

    def download_expert_route_resolve(self, workspace: HipExpertRouteResolveWorkspace,
                                      route_count: int) -> HipExpertRouteResolveResult:
        """context.rs:3127-3200: the control words and the per-route arrays, copied to the host."""
        if route_count > workspace.route_capacity:
            raise ValueError("HIP expert route resolve download exceeds route capacity")
        self.synchronize()
        control = workspace.miss_control.cpu().tolist()
        count, overflow = max(control[0], 0), control[1] != 0
        take = min(count, workspace.miss_capacity)
        return HipExpertRouteResolveResult(
            workspace.route_slots.cpu().tolist()[:route_count],
            workspace.route_generations.cpu().tolist()[:route_count],
            workspace.miss_markers.cpu().tolist()[:route_count], control[2:2 + take],
            overflow or count > workspace.miss_capacity)

    def gather_stable_moe_dispatch(self, table: HipExpertSlotTable, resolved_slots: torch.Tensor,
                                   resolved_generations: torch.Tensor, router_weights: torch.Tensor,
                                   active_markers: torch.Tensor, active_value: int, route_count: int) -> dict:
        """Per-route pointers, weights and indices for the routes whose marker equals
        ``active_value`` (kernels.rs:2718-2771; kernel kind 5)."""
        u64 = lambda: torch.zeros(route_count, dtype=torch.int64, device=self.device)
        out = dict(gate=u64(), gate_scale=u64(), up=u64(), up_scale=u64(), down=u64(), down_scale=u64(),
                   route_weights=torch.zeros(route_count, dtype=torch.float32, device=self.device),
                   route_slots=torch.zeros(route_count, dtype=torch.int32, device=self.device),
                   dispatch_error=torch.ones(1, dtype=torch.int32, device=self.device))
        a = self._table_args(table, abi.EXPERT_GATHER_DISPATCH, route_count=route_count, active_value=active_value,
                             expert_ids=_ptr(out["route_slots"]), route_slots=_ptr(resolved_slots),
                             route_generations=_ptr(resolved_generations), router_weights=_ptr(router_weights),
                             active_markers=_ptr(active_markers), output_gate_weights=_ptr(out["gate"]),
                             output_gate_scales=_ptr(out["gate_scale"]), output_up_weights=_ptr(out["up"]),
                             output_up_scales=_ptr(out["up_scale"]), output_down_weights=_ptr(out["down"]),
                             output_down_scales=_ptr(out["down_scale"]), output_route_weights=_ptr(out["route_weights"]),
                             dispatch_error=_ptr(out["dispatch_error"]))
        self._core("stable MoE dispatch gather", self.lib.ferrule_hip_core_expert_table_launch, a)
        return out

    # -- router: logits -> expert ids and route weights, on the device ----------------
    def upload_dsv4_router_hash_table(self, table, rows: int, cols: int, experts: int,
                                      top_k: int) -> HipDsv4RouterHashTable:
        """context.rs:7103-7127: validate on the host once, then keep the table on the device."""
        values = validate_dsv4_router_hash_table(table, rows, cols, experts, top_k)
        return HipDsv4RouterHashTable(torch.tensor(values, dtype=torch.int32, device=self.device).view(rows, cols),
                                      rows, cols)

    def dsv4_router_token_ids(self, token_ids, hash_rows: int) -> torch.Tensor:
        """Validated token ids as device int32 (context.rs ``dsv4_router_token_ids``)."""
        return torch.tensor(validate_dsv4_router_token_ids(token_ids, hash_rows), dtype=torch.int32,
                            device=self.device)

    def dsv4_router_topk_sqrt_softplus_rows_from_device_into(self, logits: torch.Tensor, bias: torch.Tensor | None,
                                                             tokens: int, experts: int, top_k: int,
                                                             route_scale: float, indices: torch.Tensor,
                                                             weights: torch.Tensor) -> None:
        """Score top-k routing of ``tokens`` rows in one launch, everything device resident
        (context.rs:7129-7214; kernel kind 1)."""
        if tokens == 0 or experts == 0 or top_k == 0:
            raise ValueError(f"HIP DSV4 router topk requires non-empty shape: tokens={tokens} experts={experts} "
                             f"top_k={top_k}")
        if experts > abi.ROUTER_TOPK_MAX_EXPERTS:
            raise ValueError(f"HIP DSV4 router topk supports at most 512 experts, got {experts}")
        if top_k > abi.ROUTER_MAX_TOP_K or top_k > experts:
            raise ValueError(f"HIP DSV4 router topk requires top_k in 1..={min(experts, 64)} and <=64, got {top_k}")
        if logits.dtype != torch.float32 or logits.numel() != tokens * experts:
            raise ValueError(f"HIP DSV4 router topk logits length mismatch: got {logits.numel()} expected "
                             f"{tokens}x{experts}")
        if bias is not None and (bias.dtype != torch.float32 or bias.numel() != experts):
            raise ValueError(f"HIP DSV4 router topk bias length mismatch: got {bias.numel()} expected {experts}")
        self._check_router_outputs("router topk", tokens * top_k, indices, weights)
        a = abi.RouterArgs(kind=abi.ROUTER_TOPK, rows=tokens, columns=experts, k=top_k,
                           flags=1 if bias is not None else 0, route_scale=route_scale, logits=_ptr(logits),
                           bias=_ptr(bias if bias is not None else logits), indices=_ptr(indices),
                           weights=_ptr(weights))
        self._core("router topk", self.lib.ferrule_hip_core_router_launch, a)

    def dsv4_router_hash_sqrt_softplus_rows_from_device_into(self, logits: torch.Tensor, token_ids: torch.Tensor,
                                                             hash_table: HipDsv4RouterHashTable, tokens: int,
                                                             experts: int, top_k: int, route_scale: float,
                                                             indices: torch.Tensor, weights: torch.Tensor) -> None:
        """Hash-table routing of ``tokens`` rows (context.rs:7216-7296; kernel kind 2)."""
        if tokens == 0 or experts == 0 or top_k == 0:
            raise ValueError(f"HIP DSV4 hash router requires non-empty shape: tokens={tokens} experts={experts} "
                             f"top_k={top_k}")
        if top_k > abi.ROUTER_MAX_TOP_K or top_k > experts or top_k > hash_table.cols:
            raise ValueError(f"HIP DSV4 hash router top_k {top_k} exceeds experts={experts}, "
                             f"hash_cols={hash_table.cols}, or kernel limit 64")
        if route_scale != route_scale or route_scale in (float("inf"), float("-inf")):
            raise ValueError(f"HIP DSV4 hash router route_scale must be finite, got {route_scale}")
        if logits.dtype != torch.float32 or logits.numel() != tokens * experts or token_ids.numel() != tokens \
                or token_ids.dtype != torch.int32:
            raise ValueError(f"HIP DSV4 hash router input mismatch: logits={logits.numel()} expected="
                             f"{tokens * experts}, token_ids={token_ids.numel()} expected={tokens}")
        self._check_router_outputs("hash router", tokens * top_k, indices, weights)
        a = abi.RouterArgs(kind=abi.ROUTER_HASH, rows=tokens, columns=experts, k=top_k, hash_rows=hash_table.rows,
                           hash_columns=hash_table.cols, route_scale=route_scale, logits=_ptr(logits),
                           token_ids=_ptr(token_ids), hash_table=_ptr(hash_table.buffer), indices=_ptr(indices),
                           weights=_ptr(weights))
        self._core("hash router", self.lib.ferrule_hip_core_router_launch, a)

    def topk_vocab_rows_from_device_into(self, logits: torch.Tensor, rows: int, vocab: int, top_k: int,
                                         indices: torch.Tensor, values: torch.Tensor) -> None:
        """Plain top-k of every row with int32 ids (context.rs:7298-7360; kernel kind 4)."""
        if rows == 0 or vocab == 0 or vocab > 0x7fffffff or top_k == 0 or top_k > vocab or \
                top_k > abi.VOCAB_TOPK_MAX_K:
            raise ValueError(f"HIP vocab rows top-k requires rows>0, vocab<=i32::MAX, and k in 1..={min(vocab, 40)}, "
                             f"got rows={rows} vocab={vocab} k={top_k}")
        if logits.dtype != torch.float32 or logits.numel() != rows * vocab:
            raise ValueError("HIP vocab rows top-k logits length mismatch")
        self._check_router_outputs("vocab rows top-k", rows * top_k, indices, values)
        a = abi.RouterArgs(kind=abi.VOCAB_TOPK_I32_INDEX, rows=rows, columns=vocab, k=top_k, logits=_ptr(logits),
                           indices=_ptr(indices), weights=_ptr(values))
        self._core("vocab rows top-k", self.lib.ferrule_hip_core_router_launch, a)

    @staticmethod
    def _check_router_outputs(what: str, expected: int, indices: torch.Tensor, weights: torch.Tensor) -> None:
        if indices.numel() != expected or weights.numel() != expected or indices.dtype != torch.int32 or \
                weights.dtype != torch.float32:
            raise ValueError(f"HIP DSV4 {what} output mismatch: expected {expected}, indices={indices.numel()}, "
                             f"weights={weights.numel()}")

    # -- hyper-connection producer: HC state -> hidden, normalized, packed FP8 ------------
    def hc_pre_rmsnorm_fp8_into(self, state: torch.Tensor, function: torch.Tensor, hc_scale: torch.Tensor,
                                hc_base: torch.Tensor, layer_rms_weight: torch.Tensor, sinkhorn_iters: int,
                                hc_eps: float, hc_norm_eps: float, layer_rms_eps: float,
                                bf16_boundaries: bool = False, out: dict | None = None,
                                use_workspace: bool = True) -> dict:
        """Two launches per batch of rows (dot products, then everything else): HC mix and split,
        weighted copy sum, layer RMSNorm and FP8-K128 packing (the reference's semantic HC producer, cutlass_provider.h:76-106;
        context.rs:6131-6182).  ``state`` is f32 [rows, 4, hidden]; returns the output buffers
        (``out`` lets a caller reuse them)."""
        rows, hc, hidden = state.shape
        mix = (2 + hc) * hc
        for name, t, n in (("state", state, rows * hc * hidden), ("function", function, mix * hc * hidden),
                           ("hc_scale", hc_scale, 3), ("hc_base", hc_base, mix), ("layer_rms_weight", layer_rms_weight, hidden)):
            if t.dtype != torch.float32 or t.numel() != n or not t.is_contiguous():
                raise ValueError(f"HIP HC producer {name} must be contiguous f32 with {n} elements")
        if out is None:
            f = lambda *shape: torch.empty(shape, dtype=torch.float32, device=self.device)
            out = dict(mix=f(rows, mix), hidden=f(rows, hidden), normalized=f(rows, hidden),
                       packed=torch.empty((rows, hidden), dtype=torch.uint8, device=self.device),
                       scales=torch.empty((rows, hidden // 128), dtype=torch.uint8, device=self.device),
                       pre=f(rows, hc), post=f(rows, hc), comb=f(rows, hc, hc),
                       # the reference's workspace rule, hyper_connection.cuh:480-483
                       workspace=torch.empty(rows * mix * 64 * 4 + 16, dtype=torch.uint8, device=self.device))
        a = abi.HcProducerArgs(
            rows=rows, hc=hc, hidden=hidden, mix=mix, sinkhorn_iters=sinkhorn_iters, hc_eps=hc_eps,
            hc_norm_eps=hc_norm_eps, layer_rms_eps=layer_rms_eps,
            reserved=abi.HC_PRODUCER_BF16_BOUNDARIES if bf16_boundaries else 0, state_f32=_ptr(state),
            function_row_major_f32=_ptr(function), hc_scale_f32=_ptr(hc_scale), hc_base_f32=_ptr(hc_base),
            layer_rms_weight_f32=_ptr(layer_rms_weight), mix_f32=_ptr(out["mix"]),
            workspace=_ptr(out["workspace"]) if use_workspace else 0,
            workspace_bytes=out["workspace"].numel() if use_workspace else 0, hidden_f32=_ptr(out["hidden"]),
            normalized_f32=_ptr(out["normalized"]), packed_e4m3=_ptr(out["packed"]), scales_ue8m0=_ptr(out["scales"]),
            split_pre_f32=_ptr(out["pre"]), split_post_f32=_ptr(out["post"]), split_comb_f32=_ptr(out["comb"]))
        self._two_phase("HC producer", self.lib.ferrule_hip_hc_producer_can_implement,
                        self.lib.ferrule_hip_hc_producer_launch, a)
        return out

    # -- routed MoE ---------------------------------------------------------------
    def expert_group_route_plan(self, max_experts: int, route_capacity: int, tokens: int, input_size: int,
                                intermediate_size: int, hidden_size: int) -> HipExpertGroupRoutePlan:
        """context.rs:8947-9095."""
        return HipExpertGroupRoutePlan(self, max_experts, route_capacity, tokens, input_size,
                                       intermediate_size, hidden_size)

    def _plan_args(self, plan: HipExpertGroupRoutePlan, kind: int, **kw) -> abi.ExpertGroupRoutePlanArgs:
        a = abi.ExpertGroupRoutePlanArgs(
            kind=kind, route_count=kw.get("route_count", 0), routes_per_token=kw.get("routes_per_token", 0),
            slot_capacity=plan.max_experts, route_capacity=plan.route_capacity,
            output_elements=kw.get("output_elements", 0), small_group_row_limit=abi.SMALL_GROUP_ROW_LIMIT,
            route_slots=_ptr(kw.get("route_slots")), route_generations=_ptr(kw.get("route_generations")),
            router_weights=_ptr(kw.get("router_weights")), slot_generations=_ptr(kw.get("slot_generations")),
            slot_counts=_ptr(plan.slot_counts), slot_route_offsets=_ptr(plan.slot_route_offsets),
            slot_cursors=_ptr(plan.slot_cursors), active_expert_slots=_ptr(plan.active_expert_slots),
            active_group_generations=_ptr(plan.active_group_generations),
            expert_route_indptr=_ptr(plan.expert_route_indptr), expert_route_counts=_ptr(plan.expert_route_counts),
            route_token_indices=_ptr(plan.route_token_indices), route_indices=_ptr(plan.route_indices),
            route_weights=_ptr(plan.route_weights), host_scalars=_ptr(plan.host_scalars),
            route_output=_ptr(plan.route_output), route_written=_ptr(plan.route_written),
            route_error=_ptr(plan.route_error))
        return a

    def begin_expert_group_route_invocation(self, plan: HipExpertGroupRoutePlan, route_count: int,
                                            clear_output: bool = True) -> None:
        """Zero route_output / route_written / route_error (context.rs:9206-9262).
        ``clear_output=False`` passes ``output_elements = 0``: only the flags are reset.  The
        expert kernels of this provider write every row they mark as written in full and the
        checked reducer (kind 8) never reads an unmarked row, so the 4*hidden bytes per route
        (1.9 GB at 65 536 routes) need not be written first."""
        if route_count == 0 or route_count > plan.route_capacity:
            raise ValueError("route count exceeds the plan's capacity")
        a = self._plan_args(plan, abi.ROUTE_INIT_INVOCATION, route_count=route_count,
                            output_elements=route_count * plan.hidden_size if clear_output else 0)
        self._core("route invocation init", self.lib.ferrule_hip_core_expert_group_route_plan_launch, a)
        plan.invocation_routes = route_count

    def prepare_expert_group_route_plan(self, plan: HipExpertGroupRoutePlan, table: HipRoutedExpertTable,
                                        route_slots: torch.Tensor, route_generations: torch.Tensor,
                                        router_weights: torch.Tensor, routes_per_token: int) -> None:
        """init, count, compact, scatter (context.rs:9273-9445) - four launches, no host wait."""
        n = route_slots.numel()
        if plan.invocation_routes != n:
            raise ValueError("begin_expert_group_route_invocation must precede the plan with the same route count")
        if route_generations.numel() != n or router_weights.numel() != n or n % routes_per_token:
            raise ValueError("route arrays disagree in length")
        if route_slots.dtype != torch.int32 or route_generations.dtype != torch.int32 or \
                router_weights.dtype != torch.float32:
            raise ValueError("route slots/generations are int32 and router weights f32")
        common = dict(route_count=n, routes_per_token=routes_per_token, route_slots=route_slots,
                      route_generations=route_generations, router_weights=router_weights,
                      slot_generations=table.slot_generations)
        fn = self.lib.ferrule_hip_core_expert_group_route_plan_launch
        for kind in (abi.ROUTE_INIT_PLAN, abi.ROUTE_COUNT, abi.ROUTE_COMPACT, abi.ROUTE_SCATTER):
            self._core(f"route plan kind {kind}", fn, self._plan_args(plan, kind, **common))
        plan.routes_per_token = routes_per_token
        plan.host_active_groups = None

    def prepare_decode_route_plan(self, plan: HipExpertGroupRoutePlan, table: HipRoutedExpertTable,
                                  route_slots: torch.Tensor, route_generations: torch.Tensor,
                                  router_weights: torch.Tensor, routes_per_token: int,
                                  host_route_slots=None) -> None:
        """``begin_expert_group_route_invocation`` + ``prepare_expert_group_route_plan`` for a
        decode batch (at most 2048 routes) in ONE launch.  The plan buffers end up exactly as
        after the five launches; ``route_output`` is not cleared, which only
        ``moe_decode_from_prepared_plan`` tolerates (it never reads a route it has not written).

        ``host_route_slots``: the same slot ids as the host holds them, when it does (a scheduler
        that resolved the routes itself), or the number of distinct ones.  The number of distinct valid ones bounds the plan's
        active expert groups, and ``moe_decode_from_prepared_plan`` then chooses its regime from
        that count instead of the plan's capacity, with no readback."""
        n = route_slots.numel()
        plan.host_active_groups = None
        if isinstance(host_route_slots, int):     # the count itself, from a caller that keeps it
            plan.host_active_groups = max(1, min(plan.max_experts, host_route_slots))
        elif host_route_slots is not None:
            if len(host_route_slots) != n:
                raise ValueError("host_route_slots must hold one slot per route")
            ids = {int(v) for v in host_route_slots}
            plan.host_active_groups = max(1, min(plan.max_experts, sum(1 for v in ids if 0 <= v < table.slot_capacity)))
        if n == 0 or n > plan.route_written.numel() or n > abi.FUSED_PLAN_MAX_ROUTES:
            raise ValueError("the fused decode plan takes 1..=2048 routes within the plan's capacity")
        if route_generations.numel() != n or router_weights.numel() != n or n % routes_per_token:
            raise ValueError("route arrays disagree in length")
        if route_slots.dtype != torch.int32 or route_generations.dtype != torch.int32 or \
                router_weights.dtype != torch.float32:
            raise ValueError("route slots/generations are int32 and router weights f32")
        a = self._plan_args(plan, abi.ROUTE_FUSED_DECODE_PLAN, route_count=n, routes_per_token=routes_per_token,
                            route_slots=route_slots, route_generations=route_generations,
                            router_weights=router_weights, slot_generations=table.slot_generations)
        self._core("fused decode route plan", self.lib.ferrule_hip_core_expert_group_route_plan_launch, a)
        plan.invocation_routes = n
        plan.routes_per_token = routes_per_token

    def _moe_decode_args(self, plan, table, x, output, prefix, swiglu_limit, combine, stages=0,
                         workspace=True, active_groups=None) -> abi.MoeDecodeArgs:
        flags = (abi.MOE_DECODE_COMBINE if combine else 0) | (abi.MOE_DECODE_PREFIX_F32 if prefix is not None else 0)
        flags |= stages
        if table.block_major:
            flags |= abi.MOE_DECODE_BLOCK_MAJOR_WEIGHTS
        n = plan.invocation_routes or 0
        a = abi.MoeDecodeArgs(
            active_group_count=plan.max_experts if active_groups is None else active_groups,
            slot_capacity=table.slot_capacity,
            total_routed_rows=plan.route_capacity, num_tokens=plan.tokens if x is None else x.shape[0], num_routes=n,
            routes_per_token=plan.routes_per_token, input_size=plan.input_size,
            intermediate_size=plan.intermediate_size, hidden_size=plan.hidden_size, flags=flags,
            swiglu_limit=swiglu_limit,
            active_expert_slots=_ptr(plan.active_expert_slots), expert_route_indptr=_ptr(plan.expert_route_indptr),
            route_token_indices=_ptr(plan.route_token_indices), route_indices=_ptr(plan.route_indices),
            route_weights=_ptr(plan.route_weights), host_scalars=_ptr(plan.host_scalars),
            gate_ptrs=_ptr(table.gate_ptrs), gate_scale_ptrs=_ptr(table.gate_scale_ptrs),
            up_ptrs=_ptr(table.up_ptrs), up_scale_ptrs=_ptr(table.up_scale_ptrs),
            down_ptrs=_ptr(table.down_ptrs), down_scale_ptrs=_ptr(table.down_scale_ptrs),
            input_bf16=_ptr(x), route_output=_ptr(plan.route_output), route_written=_ptr(plan.route_written),
            route_error=_ptr(plan.route_error), prefix_f32=_ptr(prefix), output=_ptr(output),
            workspace=_ptr(plan.workspace) if workspace else 0,
            workspace_bytes=0 if plan.workspace is None or not workspace else plan.workspace.numel(),
            stream=self.stream_handle())
        return a

    def moe_decode_from_prepared_plan(self, plan: HipExpertGroupRoutePlan, table: HipRoutedExpertTable,
                                      x: torch.Tensor, output: torch.Tensor | None = None,
                                      prefix: torch.Tensor | None = None, swiglu_limit: float = 0.0,
                                      stages: int = 0, static_workspace: bool = False,
                                      active_groups: int | None = None) -> None:
        """Routed experts for BF16 activations, the decode counterpart of
        ``grouped_fp4_moe_from_prepared_plan`` (context.rs:9478-9589); with ``output`` the
        rank-ordered combine and the single BF16 writeback run in the same call.

        ``active_groups`` is an upper bound of the plan's active expert groups that the host knows
        (``plan.host_metadata()``, or a scheduler that knows its routing); without it the count that
        ``prepare_decode_route_plan`` derived from ``host_route_slots`` is used, and without that the
        plan's capacity.  The layer sizes its grids by it and chooses its regime from it:
        at most four routes per group on average run in the packed kernels only, more also launch
        the general kernels, which take an expert's rows 16 at a time instead of 8.

        ``static_workspace`` takes the entry point that allocates nothing: the workspace is a
        fixed 16 MiB array inside the library (one per GPU, shared by every such call on that
        GPU, so calls must not overlap in time) and this method touches no allocator."""
        if x.dtype != torch.bfloat16 or x.dim() != 2 or x.shape[1] != plan.input_size or not x.is_contiguous():
            raise ValueError(f"MoE input must be contiguous bf16 [tokens, {plan.input_size}]")
        if plan.invocation_routes != x.shape[0] * plan.routes_per_token:
            raise ValueError("the prepared plan does not belong to this batch")
        if output is not None and (output.dtype != torch.bfloat16 or tuple(output.shape) != (x.shape[0], plan.hidden_size)):
            raise ValueError("MoE output must be bf16 [tokens, hidden]")
        if prefix is not None and (prefix.dtype != torch.float32 or tuple(prefix.shape) != (x.shape[0], plan.hidden_size)):
            raise ValueError("MoE prefix must be f32 [tokens, hidden]")
        if active_groups is None:
            active_groups = plan.host_active_groups
        if active_groups is not None and not 1 <= active_groups <= plan.max_experts:
            raise ValueError("active_groups must lie in 1..=plan.max_experts")
        if static_workspace:
            probe = self._moe_decode_args(plan, table, None, None, None, swiglu_limit, False, workspace=False,
                                          active_groups=active_groups)
            size = self.lib.ferrule_hip_moe_decode_workspace_size(C.byref(probe))
            if size == 0 or size > abi.MOE_DECODE_STATIC_WORKSPACE_BYTES:
                raise ProviderError(
                    f"MoE decode needs {size} workspace bytes, the library's static workspace holds "
                    f"{abi.MOE_DECODE_STATIC_WORKSPACE_BYTES}", abi.UNSUPPORTED)
            args = self._moe_decode_args(plan, table, x, output, prefix, swiglu_limit, output is not None, stages,
                                         workspace=False, active_groups=active_groups)
            args.stream = self.stream_handle()
            status = self.lib.ferrule_hip_moe_decode_launch_static_workspace(C.byref(args))
            if status != abi.SUCCESS:
                raise ProviderError("launch MoE decode (static workspace)", status)
            self.kernel_launches += 2 if output is not None else 1
            return
        if plan.workspace is None:
            # workspace query with null pointers (cutlass_provider.h:446-449), allocated once
            probe = self._moe_decode_args(plan, table, None, None, None, swiglu_limit, False)
            size = self.lib.ferrule_hip_moe_decode_workspace_size(C.byref(probe))
            if size == 0:
                raise ProviderError("MoE decode workspace query", abi.UNSUPPORTED)
            plan.workspace = torch.empty(size, dtype=torch.uint8, device=self.device)
        args = self._moe_decode_args(plan, table, x, output, prefix, swiglu_limit, output is not None, stages,
                                     active_groups=active_groups)
        self._two_phase("MoE decode", self.lib.ferrule_hip_moe_decode_can_implement,
                        self.lib.ferrule_hip_moe_decode_launch, args)
        self.kernel_launches += 2 if output is not None else 1

    def prepare_mxfp4_block_major(self, handle: HipArtifactLinearHandle) -> HipArtifactLinearHandle:
        """Row-major MXFP4 artifact -> the block-major order the decode MoE layer streams at
        full width (16 rows x 64 B of one K block contiguous).  Done once when an expert is
        materialised in a slot, like the scale preparation of the reference
        (context.rs:5185-5204); the returned handle owns new storage of the same size."""
        return self.prepare_mxfp4_block_major_into(handle, torch.empty_like(handle.weight),
                                                   torch.empty_like(handle.scale))

    def prepare_mxfp4_block_major_into(self, handle: HipArtifactLinearHandle, weight: torch.Tensor,
                                       scale: torch.Tensor) -> HipArtifactLinearHandle:
        """``prepare_mxfp4_block_major`` into storage the caller owns (an arena frame)."""
        sh = handle.shape
        if sh.weight_format != abi.WEIGHT_MXFP4_E2M1 or handle.block_major:
            raise ValueError("block-major preparation takes a row-major MXFP4 artifact")
        if weight.numel() != handle.weight.numel() or scale.numel() != handle.scale.numel() or \
                weight.dtype != torch.uint8 or scale.dtype != torch.uint8:
            raise ValueError("block-major destination must have the source's byte sizes")
        a = abi.PrepareMxfp4BlockMajorArgs(n=sh.out_features, k=sh.in_features, weight_source=_ptr(handle.weight),
                                           scale_source=_ptr(handle.scale), weight_destination=_ptr(weight),
                                           scale_destination=_ptr(scale), stream=self.stream_handle())
        status = self.lib.ferrule_hip_prepare_mxfp4_block_major(C.byref(a))
        if status != abi.SUCCESS:
            raise ProviderError("prepare MXFP4 block-major weights", status)
        self.kernel_launches += 1
        return HipArtifactLinearHandle(sh, weight, scale, block_major=True)

    def prepare_fp8_block_major(self, handle: HipArtifactLinearHandle) -> HipArtifactLinearHandle:
        """Row-major FP8 artifact -> block-major payload for the decode GEMV (the block scales
        are shared with the source handle, they are not reordered)."""
        sh = handle.shape
        if sh.weight_format != abi.WEIGHT_FP8_E4M3 or handle.block_major:
            raise ValueError("block-major preparation takes a row-major FP8 artifact")
        weight = torch.empty_like(handle.weight)
        a = abi.PrepareFp8BlockMajorArgs(n=sh.out_features, k=sh.in_features, weight_source=_ptr(handle.weight),
                                         weight_destination=_ptr(weight), stream=self.stream_handle())
        status = self.lib.ferrule_hip_prepare_fp8_block_major(C.byref(a))
        if status != abi.SUCCESS:
            raise ProviderError("prepare FP8 block-major weights", status)
        self.kernel_launches += 1
        return HipArtifactLinearHandle(sh, weight, handle.scale, block_major=True)

    def prepare_mxfp4_sfb(self, linear_scales: torch.Tensor, n: int, k: int) -> torch.Tensor:
        """Linear UE8M0 [n, k/32] -> this provider's prepared scale storage
        (``materialize_routed_expert_from_pinned_async`` does this per expert matrix,
        context.rs:5185-5204)."""
        size = self.lib.ferrule_hip_mxfp4_sfb_storage_bytes(n, k)
        if size == 0:
            raise ProviderError("MXFP4 scale storage query", abi.UNSUPPORTED)
        out = torch.empty(size, dtype=torch.uint8, device=self.device)
        a = abi.PrepareMxfp4SfbArgs(n=n, k=k, reserved0=0, linear_source=_ptr(linear_scales),
                                    prepared_destination=_ptr(out), stream=self.stream_handle())
        status = self.lib.ferrule_hip_prepare_mxfp4_sfb(C.byref(a))
        if status != abi.SUCCESS:
            raise ProviderError("prepare MXFP4 scales", status)
        self.kernel_launches += 1
        return out

    def _grouped_args(self, plan, table, meta, x_packed, x_scales, swiglu_limit) -> abi.GroupedFp4MoeArgs:
        return abi.GroupedFp4MoeArgs(
            active_group_count=meta["active_group_count"], small_group_count=meta["small_group_count"],
            slot_capacity=table.slot_capacity, max_group_rows=meta["max_group_rows"],
            total_routed_rows=meta["total_routed_rows"], num_tokens=plan.tokens,
            num_routes=plan.invocation_routes or 0, input_size=plan.input_size,
            intermediate_size=plan.intermediate_size, hidden_size=plan.hidden_size, swiglu_limit=swiglu_limit,
            active_expert_slots=_ptr(plan.active_expert_slots),
            active_group_generations=_ptr(plan.active_group_generations),
            expert_route_indptr=_ptr(plan.expert_route_indptr), expert_route_counts=_ptr(plan.expert_route_counts),
            route_token_indices=_ptr(plan.route_token_indices), route_indices=_ptr(plan.route_indices),
            route_weights=_ptr(plan.route_weights), slot_generations=_ptr(table.slot_generations),
            gate_ptrs=_ptr(table.gate_ptrs), gate_scale_ptrs=_ptr(table.gate_scale_ptrs),
            up_ptrs=_ptr(table.up_ptrs), up_scale_ptrs=_ptr(table.up_scale_ptrs),
            down_ptrs=_ptr(table.down_ptrs), down_scale_ptrs=_ptr(table.down_scale_ptrs),
            input_fp8=_ptr(x_packed), input_ue8m0=_ptr(x_scales), route_output=_ptr(plan.route_output),
            route_written=_ptr(plan.route_written), route_error=_ptr(plan.route_error),
            workspace=_ptr(plan.grouped_workspace),
            workspace_bytes=0 if plan.grouped_workspace is None else plan.grouped_workspace.numel(),
            stream=self.stream_handle())

    def grouped_fp4_moe_from_prepared_plan(self, plan: HipExpertGroupRoutePlan, table: HipRoutedExpertTable,
                                           x_packed: torch.Tensor, x_scales: torch.Tensor,
                                           swiglu_limit: float = 0.0, meta: dict | None = None,
                                           debug_hidden: torch.Tensor | None = None) -> None:
        """Routed MXFP4 experts over packed FP8 rows into ``plan.route_output``
        (``grouped_fp4_moe_from_prepared_plan``, context.rs:9478-9589).  ``meta`` is the 16-byte
        scalar readback of the plan (context.rs:9401-9410); it is read here when not given.  The
        table may hold the checkpoint (row-major) order or the block-major order the decode layer
        prefers: the results are the same bits."""
        if table.block_major and debug_hidden is not None:
            raise ValueError("the debug launch of the grouped MoE GEMM reads row-major expert weights")
        if x_packed.dtype != torch.uint8 or tuple(x_packed.shape) != (plan.tokens, plan.input_size):
            raise ValueError(f"grouped MoE input must be e4m3 bytes [{plan.tokens}, {plan.input_size}]")
        if tuple(x_scales.shape) != (plan.tokens, plan.input_size // 128):
            raise ValueError("grouped MoE input scales must be ue8m0 [tokens, input/128]")
        meta = meta or plan.host_metadata()
        if meta["active_group_count"] == 0:
            return
        probe = self._grouped_args(plan, table, meta, None, None, swiglu_limit)
        size = self.lib.ferrule_hip_grouped_fp4_moe_workspace_size(C.byref(probe))
        if size == 0:
            raise ProviderError("grouped MoE workspace query", abi.UNSUPPORTED)
        if plan.grouped_workspace is None or plan.grouped_workspace.numel() < size:
            plan.grouped_workspace = torch.empty(size, dtype=torch.uint8, device=self.device)
        args = self._grouped_args(plan, table, meta, x_packed, x_scales, swiglu_limit)
        if debug_hidden is None:
            # one prepared copy per expert: a block-major table (the decode layer's) is read in place
            launch = self.lib.ferrule_hip_grouped_fp4_moe_block_major_launch if table.block_major \
                else self.lib.ferrule_hip_grouped_fp4_moe_launch
            self._two_phase("grouped FP4 MoE", self.lib.ferrule_hip_grouped_fp4_moe_can_implement, launch, args)
        else:
            status = self.lib.ferrule_hip_grouped_fp4_moe_debug_launch(C.byref(args), _ptr(debug_hidden))
            if status != abi.SUCCESS:
                raise ProviderError("launch grouped FP4 MoE (debug)", status)
        self.kernel_launches += 2

    def grouped_workspace_views(self, plan: HipExpertGroupRoutePlan, meta: dict):
        """(hq [rows, I] e4m3, hs [rows, I/128] ue8m0) inside the grouped workspace, for tests: the
        layout is tile map | quantised hidden rows | their scales, each 256-byte aligned."""
        rows, groups, inter = meta["total_routed_rows"], meta["active_group_count"], plan.intermediate_size
        align = lambda v: (v + 255) & ~255
        max_tiles = rows // 128 + groups
        hq_off = align(64 + 80 * max_tiles)      # a 64-byte head and one 80-byte record per tile
        hs_off = align(hq_off + rows * inter)
        ws = plan.grouped_workspace
        return (ws[hq_off:hq_off + rows * inter].view(rows, inter),
                ws[hs_off:hs_off + rows * (inter // 128)].view(rows, inter // 128))

    def reduce_moe_route_outputs_ranked(self, route_output: torch.Tensor, tokens: int, routes_per_token: int,
                                        hidden: int, output: torch.Tensor, route_written=None,
                                        route_error=None) -> None:
        """out[t,h] = bf16(out[t,h] + sum_rank route_output[t*k+rank,h]) in f32 storage
        (context.rs ``reduce_moe_route_outputs_ranked``; kind 8 when the completeness
        arrays are given, kind 7 otherwise)."""
        if output.dtype != torch.float32 or output.numel() != tokens * hidden:
            raise ValueError("ranked reduction output must be f32 [tokens, hidden]")
        if route_output.numel() < tokens * routes_per_token * hidden:
            raise ValueError("route output is shorter than tokens * routes * hidden")
        checked = route_written is not None
        a = abi.MoeArgs(kind=abi.MOE_REDUCE_EXPERT_GROUP_ROUTES if checked else abi.MOE_REDUCE_ROUTES,
                        tokens=tokens, routes_per_token=routes_per_token, hidden=hidden,
                        route_output=_ptr(route_output), route_written=_ptr(route_written),
                        route_error=_ptr(route_error), output=_ptr(output))
        self._core("ranked route reduction", self.lib.ferrule_hip_core_moe_launch, a)

    def moe_weighted_swiglu_f32(self, gate: torch.Tensor, up: torch.Tensor, hidden: torch.Tensor,
                                route_weight: float = 1.0, route_weights: torch.Tensor | None = None,
                                swiglu_limit: float = 0.0) -> None:
        """kind 2: hidden = silu(gate) * up * weight on f32 [routes, n] (entrypoints.cu:1518-1537)."""
        routes, n = gate.shape
        a = abi.MoeArgs(kind=abi.MOE_WEIGHTED_SWIGLU_F32, n=n, batch_columns=routes, experts=1,
                        route_weight=route_weight, swiglu_limit=swiglu_limit, gate=_ptr(gate), up=_ptr(up),
                        route_weights=_ptr(route_weights), hidden_values=_ptr(hidden))
        self._core("weighted SwiGLU", self.lib.ferrule_hip_core_moe_launch, a)

    def synchronize(self) -> None:
        self.stream.synchronize()
