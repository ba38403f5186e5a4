"""Pins the CPU checker's slot-table functions and the host mirror of the table against the literal
expectations of Ferrule's own tests; no GPU."""
import ctypes as C

import numpy as np
import pytest

from ferrule_amd import abi
from ferrule_amd.provider import (I32_MAX, HipExpertSlotBinding, HipExpertSlotPointers, HipExpertSlotTableHost)
from oracle import pyoracle as po

POINTERS = HipExpertSlotPointers(1, 2, 3, 4, 5, 6)      # context.rs:2300-2307


def test_host_exact_install_evict_and_reuse_follow_external_generations():
    # context.rs:2309-2352
    table = HipExpertSlotTableHost(3, 2)
    first = table.install_at(2, 1, 1, POINTERS)
    assert first == HipExpertSlotBinding(1, 1) and table.binding(2) == first and table.pointers_at(1) == POINTERS
    table.evict_binding(2, 1, 1)
    assert table.binding(2) is None and not table.is_current(first) and table.slot_generation[1] == 2
    assert table.pointers_at(1) == HipExpertSlotPointers()
    second = table.install_at(1, 1, 2, POINTERS)
    assert second == HipExpertSlotBinding(1, 2) and table.binding(1) == second


def test_host_exact_binding_mismatches_are_failure_atomic():
    # context.rs:2354-2383
    table = HipExpertSlotTableHost(3, 2)
    table.install_at(0, 0, 1, POINTERS)
    installed = table.clone()
    for call in (lambda: table.install_at(1, 0, 2, POINTERS), lambda: table.install_at(0, 1, 1, POINTERS),
                 lambda: table.evict_binding(0, 0, 2), lambda: table.evict_binding(0, 1, 1),
                 lambda: table.evict_binding(1, 0, 1)):
        with pytest.raises(ValueError):
            call()
        assert table == installed
    table.evict_binding(0, 0, 1)
    evicted = table.clone()
    with pytest.raises(ValueError):
        table.install_at(1, 0, 3, POINTERS)
    assert table == evicted


def test_host_exact_install_validates_coordinates_generation_and_full_pointer_tuple():
    # context.rs:2385-2424
    table = HipExpertSlotTableHost(2, 1)
    empty = table.clone()
    for args in ((2, 0, 1), (0, 1, 1), (0, 0, 0), (0, 0, I32_MAX + 1)):
        with pytest.raises(ValueError):
            table.install_at(*args, POINTERS)
    for missing in range(6):
        values = list(POINTERS.as_tuple())
        values[missing] = 0
        with pytest.raises(ValueError):
            table.install_at(0, 0, 1, HipExpertSlotPointers(*values))
    assert table == empty


def test_host_terminal_generation_is_free_but_exhausted():
    # context.rs:2426-2441
    table = HipExpertSlotTableHost(2, 1)
    table.slot_generation[0] = I32_MAX - 2
    resident = table.install(0, POINTERS)
    assert resident.generation == I32_MAX - 1
    assert table.evict(0) and table.slot_generation[0] == I32_MAX and table.binding(0) is None
    with pytest.raises(ValueError, match="generation exhausted"):
        table.install(1, POINTERS)
    assert table.binding(1) is None


def test_host_install_picks_the_first_free_slot_and_reports_a_full_table():
    table = HipExpertSlotTableHost(4, 2)
    assert table.install(3, POINTERS) == HipExpertSlotBinding(0, 1)
    assert table.install(3, POINTERS) == HipExpertSlotBinding(0, 1)      # idempotent
    assert table.install(1, POINTERS) == HipExpertSlotBinding(1, 1)
    with pytest.raises(ValueError, match="table is full"):
        table.install(0, POINTERS)
    assert table.evict(3) and not table.evict(3)
    assert table.install(0, POINTERS) == HipExpertSlotBinding(0, 3)      # 1 -> evicted 2 -> reinstalled 3


def test_checker_reference_resolve_case():
    # expert_group_route_plan.rs:29-107 with the table driven as the host mirror drives the device
    host = HipExpertSlotTableHost(4, 1)
    state = po.ExpertTableState(4, 1)
    pointers = HipExpertSlotPointers(16, 32, 48, 64, 80, 96)
    first = host.install(2, pointers)
    state.publish(1, 2, first.slot, first.generation, pointers.as_tuple())
    slots, gens, markers, control = state.resolve([2, 1, -1, 4], miss_capacity=2, route_capacity=4)
    assert slots.tolist() == [first.slot, -1, -1, -1] and gens.tolist() == [first.generation, 0, 0, 0]
    assert markers.tolist() == [0, 1, 1, 1]
    miss_ids = control[2:4].tolist()
    assert control[0] == 3 and control[1] == 1                       # three misses, list of two overflowed
    assert set(miss_ids) <= {1, -1, 4} and miss_ids[0] != miss_ids[1]
    assert control[4:8].tolist() == [2, 1, -1, 4]                    # every route's expert id
    assert host.evict(2)
    state.publish(2, 2, first.slot, host.slot_generation[first.slot])
    second = host.install(1, pointers)
    state.publish(1, 1, second.slot, second.generation, pointers.as_tuple())
    assert second.slot == first.slot and second.generation != first.generation
    assert not host.is_current(first) and host.is_current(second)
    slots, gens, markers, control = state.resolve([2, 1], miss_capacity=2, route_capacity=4)
    assert slots.tolist() == [-1, second.slot] and gens.tolist() == [0, second.generation]
    assert control[0] == 1 and control[1] == 0 and control[2] == 2
    assert state.table[:, 0].tolist() == list(pointers.as_tuple())


def test_checker_gather_dispatch_semantics():
    state = po.ExpertTableState(8, 3)
    state.publish(1, 5, 0, 1, (10, 11, 12, 13, 14, 15))
    state.publish(1, 6, 2, 4, (20, 21, 22, 23, 24, 0))               # incomplete tuple
    slots = [0, 2, 1, 0, -1, 0]
    gens = [1, 4, 1, 2, 0, 1]                                          # route 3 carries a stale generation
    weights = np.arange(1, 7, dtype=np.float32) / 8
    markers = [7, 7, 0, 7, 0, 0]
    out, w, ids, err = state.gather_dispatch(slots, gens, weights, markers, 7)
    assert out[:, 0].tolist() == [10, 11, 12, 13, 14, 15] and out[:, 1].tolist() == [20, 21, 22, 23, 24, 0]
    assert not out[:, 2].any() and not out[:, 3].any() and not out[:, 4].any()
    assert out[:, 5].tolist() == [10, 11, 12, 13, 14, 15]            # inactive but current: pointers still gathered
    assert w.tolist() == [0.125, 0, 0, 0, 0, 0] and ids.tolist() == [0, -1, -1, -1, -1, -1]
    assert err == 1                                                    # routes 1 and 3 are active and not dispatchable
    _, _, _, err = state.gather_dispatch(slots[:1] + slots[4:], gens[:1] + gens[4:], weights[:3], [7, 0, 0], 7)
    assert err == 0


def test_expert_table_launch_validation_codes_without_touching_a_device():
    lib = abi.load()
    fn = lib.ferrule_hip_core_expert_table_launch
    assert fn(None) == 1
    table = dict(gate_weights=8, gate_scales=8, up_weights=8, up_scales=8, down_weights=8, down_scales=8,
                 slot_generations=8, expert_to_slot=8, expert_generations=8, expert_capacity=4, slot_capacity=2)
    for change in (dict(kind=0), dict(kind=6), dict(kind=abi.EXPERT_INSTALL, slot=2), dict(kind=abi.EXPERT_EVICT, expert=4),
                   dict(kind=abi.EXPERT_INSTALL, gate_scales=0), dict(kind=abi.EXPERT_INITIALIZE_RESOLVE),
                   dict(kind=abi.EXPERT_RESOLVE, route_count=1), dict(kind=abi.EXPERT_GATHER_DISPATCH, route_count=1)):
        args = abi.ExpertTableArgs(**{**table, **change})
        assert fn(C.byref(args)) == 1, change
