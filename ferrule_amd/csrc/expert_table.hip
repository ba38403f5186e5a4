// Drop-in for ferrule_core_expert_table_launch (abi/core_provider.h:490; kernel
// portable/entrypoints.cu:1268-1380, launch :2006-2027): the device side of the stable
// expert slot table that sits between the router's expert ids and the route plan's slots.
//   1  INSTALL             publish one (expert -> slot, generation, six pointers) binding
//   2  EVICT               retire it: expert unbound, pointers zeroed, slot generation advanced
//   3  INITIALIZE_RESOLVE  miss_control = {count 0, overflow 0, -1 ...}
//   4  RESOLVE             route expert id -> (slot, generation) if the binding is current, else
//                          (-1, 0) and a miss: marker, id appended to the bounded miss list
//   5  GATHER_DISPATCH     per route: the slot's six pointers (0 when stale), the router weight
//                          (0 when not dispatchable), the route's own index or -1; a route that
//                          is active but not dispatchable raises dispatch_error
// All of it is 4- and 8-byte integer metadata, a few KB per layer; the work is in keeping the
// launch count and the number of atomics low:
//   * RESOLVE appends misses with ONE atomic per wave (ballot + prefix rank inside the wave)
//     instead of one per missing route.  The order of the miss list is as unspecified as the
//     reference's (its order is the order in which threads reach atomicAdd);
//   * GATHER_DISPATCH clears dispatch_error with a one-thread kernel ahead of the gather (the
//     reference uses cudaMemsetAsync, entrypoints.cu:2011-2017; a memset node is avoided so
//     that the pair can be captured into a graph), and raises it with one atomic per wave.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <initializer_list>

#include "../../include/ferrule_hip_provider.h"
#include "numeric.cuh"

namespace ferrule_hip {
namespace {

template <typename T>
__device__ __forceinline__ T *ptr(uint64_t address) {
  return global_ptr<T>(address);
}

// entrypoints.cu:1270-1300, one thread
__global__ void expert_binding_kernel(FerruleHipExpertTableArgs a) {
  if (blockIdx.x != 0 || threadIdx.x != 0) return;
  uint64_t *gate = ptr<uint64_t>(a.gate_weights), *gate_scale = ptr<uint64_t>(a.gate_scales);
  uint64_t *up = ptr<uint64_t>(a.up_weights), *up_scale = ptr<uint64_t>(a.up_scales);
  uint64_t *down = ptr<uint64_t>(a.down_weights), *down_scale = ptr<uint64_t>(a.down_scales);
  if (a.kind == FERRULE_HIP_EXPERT_INSTALL) {
    gate[a.slot] = a.gate_weight_value;
    gate_scale[a.slot] = a.gate_scale_value;
    up[a.slot] = a.up_weight_value;
    up_scale[a.slot] = a.up_scale_value;
    down[a.slot] = a.down_weight_value;
    down_scale[a.slot] = a.down_scale_value;
    ptr<int32_t>(a.slot_generations)[a.slot] = a.generation;
    ptr<int32_t>(a.expert_to_slot)[a.expert] = static_cast<int32_t>(a.slot);
    ptr<int32_t>(a.expert_generations)[a.expert] = a.generation;
  } else {
    ptr<int32_t>(a.expert_to_slot)[a.expert] = -1;
    ptr<int32_t>(a.expert_generations)[a.expert] = 0;
    gate[a.slot] = gate_scale[a.slot] = up[a.slot] = up_scale[a.slot] = 0;
    down[a.slot] = down_scale[a.slot] = 0;
    ptr<int32_t>(a.slot_generations)[a.slot] = a.generation;
  }
}

// entrypoints.cu:1301-1307
__global__ __launch_bounds__(256) void resolve_init_kernel(FerruleHipExpertTableArgs a) {
  const uint64_t index = static_cast<uint64_t>(blockIdx.x) * 256u + threadIdx.x;
  const uint64_t count = static_cast<uint64_t>(a.miss_capacity) + a.route_capacity + 2u;
  if (index < count) ptr<int32_t>(a.miss_control)[index] = index < 2u ? 0 : -1;
}

// number of set bits of `mask` below this lane
__device__ __forceinline__ uint32_t rank_in_wave(uint64_t mask) {
  return __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(mask >> 32),
                                   __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0u));
}

// entrypoints.cu:1311-1340
__global__ __launch_bounds__(256) void resolve_kernel(FerruleHipExpertTableArgs a) {
  const uint32_t route = blockIdx.x * 256u + threadIdx.x;
  const bool live = route < a.route_count;
  int32_t expert = -1, slot = -1, generation = 0;
  if (live) {
    expert = ptr<const int32_t>(a.expert_ids)[route];
    if (expert >= 0 && static_cast<uint32_t>(expert) < a.expert_capacity) {
      const int32_t mapped = ptr<const int32_t>(a.expert_to_slot)[expert];
      const int32_t expert_generation = ptr<const int32_t>(a.expert_generations)[expert];
      if (mapped >= 0 && static_cast<uint32_t>(mapped) < a.slot_capacity && expert_generation > 0 &&
          ptr<const int32_t>(a.slot_generations)[mapped] == expert_generation) {
        slot = mapped;
        generation = expert_generation;
      }
    }
    ptr<int32_t>(a.route_slots)[route] = slot;
    ptr<int32_t>(a.route_generations)[route] = generation;
    ptr<int32_t>(a.miss_markers)[route] = slot < 0 ? 1 : 0;
    ptr<int32_t>(a.miss_control)[2u + a.miss_capacity + route] = expert;
  }
  const bool miss = live && slot < 0;
  const uint64_t missing = __ballot(miss);
  if (missing == 0ull) return;  // wave-uniform
  int32_t *control = ptr<int32_t>(a.miss_control);
  const uint32_t leader = static_cast<uint32_t>(__ffsll(static_cast<unsigned long long>(missing))) - 1u;
  int32_t base = 0;
  if ((threadIdx.x & 63u) == leader) base = atomicAdd(control, static_cast<int32_t>(__popcll(missing)));
  base = __shfl(base, static_cast<int>(leader), 64);
  if (miss) {
    const int64_t position = static_cast<int64_t>(base) + rank_in_wave(missing);
    if (position >= 0 && position < static_cast<int64_t>(a.miss_capacity)) {
      control[2 + position] = expert;
    } else {
      atomicOr(control + 1, 1);
    }
  }
}

__global__ void clear_flag_kernel(int32_t *flag) {
  if (blockIdx.x == 0 && threadIdx.x == 0) *flag = 0;
}

// entrypoints.cu:1341-1379
__global__ __launch_bounds__(256) void gather_dispatch_kernel(FerruleHipExpertTableArgs a) {
  const uint32_t route = blockIdx.x * 256u + threadIdx.x;
  bool bad = false;
  if (route < a.route_count) {
    const int32_t slot = ptr<const int32_t>(a.route_slots)[route];
    const int32_t generation = ptr<const int32_t>(a.route_generations)[route];
    const bool active = ptr<const int32_t>(a.active_markers)[route] == a.active_value;
    const bool current = slot >= 0 && static_cast<uint32_t>(slot) < a.slot_capacity && generation > 0 &&
                         ptr<const int32_t>(a.slot_generations)[slot] == generation;
    const uint64_t gate = current ? ptr<const uint64_t>(a.gate_weights)[slot] : 0;
    const uint64_t gate_scale = current ? ptr<const uint64_t>(a.gate_scales)[slot] : 0;
    const uint64_t up = current ? ptr<const uint64_t>(a.up_weights)[slot] : 0;
    const uint64_t up_scale = current ? ptr<const uint64_t>(a.up_scales)[slot] : 0;
    const uint64_t down = current ? ptr<const uint64_t>(a.down_weights)[slot] : 0;
    const uint64_t down_scale = current ? ptr<const uint64_t>(a.down_scales)[slot] : 0;
    const bool good = active && current && gate != 0 && gate_scale != 0 && up != 0 && up_scale != 0 && down != 0 &&
                      down_scale != 0;
    bad = active && !good;
    ptr<uint64_t>(a.output_gate_weights)[route] = gate;
    ptr<uint64_t>(a.output_gate_scales)[route] = gate_scale;
    ptr<uint64_t>(a.output_up_weights)[route] = up;
    ptr<uint64_t>(a.output_up_scales)[route] = up_scale;
    ptr<uint64_t>(a.output_down_weights)[route] = down;
    ptr<uint64_t>(a.output_down_scales)[route] = down_scale;
    ptr<float>(a.output_route_weights)[route] = good ? ptr<const float>(a.router_weights)[route] : 0.0f;
    ptr<int32_t>(a.expert_ids)[route] = good ? static_cast<int32_t>(route) : -1;
  }
  const uint64_t failing = __ballot(bad);
  if (failing != 0ull && (threadIdx.x & 63u) == static_cast<uint32_t>(__ffsll(static_cast<unsigned long long>(failing))) - 1u) {
    atomicOr(ptr<int32_t>(a.dispatch_error), 1);
  }
}

bool any_null(std::initializer_list<uint64_t> pointers) {
  for (uint64_t p : pointers) {
    if (p == 0) return true;
  }
  return false;
}

}  // namespace
}  // namespace ferrule_hip

extern "C" int32_t ferrule_hip_core_expert_table_launch(const FerruleHipExpertTableArgs *args) {
  using namespace ferrule_hip;
  if (args == nullptr) return 1;  // hipErrorInvalidValue, as entrypoints.cu:2008-2010
  const FerruleHipExpertTableArgs &a = *args;
  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(a.stream));
  const bool table_null = any_null({a.gate_weights, a.gate_scales, a.up_weights, a.up_scales, a.down_weights,
                                    a.down_scales, a.slot_generations});
  clear_launch_error();
  switch (a.kind) {
    case FERRULE_HIP_EXPERT_INSTALL:
    case FERRULE_HIP_EXPERT_EVICT:
      // the kernel indexes with these unchecked (the host mirror validated them,
      // context.rs:2059-2092); a bound violation here would be a stray device write
      if (table_null || any_null({a.expert_to_slot, a.expert_generations}) || a.slot >= a.slot_capacity ||
          a.expert >= a.expert_capacity) {
        return 1;
      }
      expert_binding_kernel<<<1, 64, 0, stream>>>(a);
      break;
    case FERRULE_HIP_EXPERT_INITIALIZE_RESOLVE: {
      if (a.miss_control == 0) return 1;
      const uint64_t count = static_cast<uint64_t>(a.miss_capacity) + a.route_capacity + 2u;
      resolve_init_kernel<<<static_cast<uint32_t>((count + 255u) / 256u), 256, 0, stream>>>(a);
      break;
    }
    case FERRULE_HIP_EXPERT_RESOLVE:
      if (any_null({a.expert_ids, a.expert_to_slot, a.expert_generations, a.slot_generations, a.route_slots,
                    a.route_generations, a.miss_markers, a.miss_control})) {
        return 1;
      }
      if (a.route_count == 0) return 0;
      resolve_kernel<<<(a.route_count + 255u) / 256u, 256, 0, stream>>>(a);
      break;
    case FERRULE_HIP_EXPERT_GATHER_DISPATCH:
      if (table_null || any_null({a.expert_ids, a.route_slots, a.route_generations, a.router_weights,
                                  a.active_markers, a.output_gate_weights, a.output_gate_scales,
                                  a.output_up_weights, a.output_up_scales, a.output_down_weights,
                                  a.output_down_scales, a.output_route_weights, a.dispatch_error})) {
        return 1;
      }
      clear_flag_kernel<<<1, 64, 0, stream>>>(reinterpret_cast<int32_t *>(static_cast<uintptr_t>(a.dispatch_error)));
      if (a.route_count != 0) gather_dispatch_kernel<<<(a.route_count + 255u) / 256u, 256, 0, stream>>>(a);
      break;
    default:
      return 1;
  }
  return static_cast<int32_t>(take_launch_error());
}
