// Expert-major route plan: from per-(token, rank) expert slots to compact groups
// with contiguous rows.  Drop-in for ferrule_core_expert_group_route_plan_launch
// (abi/core_provider.h:490; kernel portable/entrypoints.cu:1382-1513), same five
// kinds and the same outputs:
//   1 INIT_INVOCATION  zero route_output / route_written / route_error
//   2 INIT_PLAN        reset counts, offsets(-1), cursors, groups, indptr, rows(-1), scalars
//   3 COUNT            slot_counts[slot] += 1 for every route whose (slot, generation) is live
//   4 COMPACT          groups = live slots, small groups (count < limit) first, then large,
//                      each in ascending slot order; indptr / counts / offsets; 4 scalars
//   5 SCATTER          (token, route, weight) of every live route into its group's rows
// All of it is int32 metadata, a few KB: the work is latency, not bandwidth.  The
// reference compacts with ONE thread looping twice over the slots and scatters with an
// atomic cursor; here COMPACT is one workgroup doing block-wide prefix sums and SCATTER
// gives each slot a workgroup that ranks its routes with ballot prefix sums, so rows
// inside a group come out in ascending route order on every run.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ferrule_hip_provider.h"
#include "numeric.cuh"

namespace ferrule_hip {
namespace {

template <typename T>
__device__ __forceinline__ T *ptr(uint64_t address) {
  return global_ptr<T>(address);
}

__global__ __launch_bounds__(256) void route_init_invocation_kernel(FerruleHipExpertGroupRoutePlanArgs a) {
  const uint32_t index = blockIdx.x * 256u + threadIdx.x;
  if (index < a.output_elements) ptr<float>(a.route_output)[index] = 0.0f;
  if (index < a.route_count) ptr<int32_t>(a.route_written)[index] = 0;
  if (index == 0) ptr<int32_t>(a.route_error)[0] = 0;
}

__global__ __launch_bounds__(256) void route_init_plan_kernel(FerruleHipExpertGroupRoutePlanArgs a) {
  const uint32_t index = blockIdx.x * 256u + threadIdx.x;
  if (index < a.slot_capacity) {
    ptr<int32_t>(a.slot_counts)[index] = 0;
    ptr<int32_t>(a.slot_route_offsets)[index] = -1;
    ptr<int32_t>(a.slot_cursors)[index] = 0;
    ptr<int32_t>(a.active_expert_slots)[index] = -1;
    ptr<int32_t>(a.active_group_generations)[index] = 0;
    ptr<int32_t>(a.expert_route_counts)[index] = 0;
  }
  if (index <= a.slot_capacity) ptr<int32_t>(a.expert_route_indptr)[index] = 0;
  if (index < a.route_capacity) {
    ptr<int32_t>(a.route_token_indices)[index] = -1;
    ptr<int32_t>(a.route_indices)[index] = -1;
    ptr<float>(a.route_weights)[index] = 0.0f;
  }
  if (index < 4) ptr<int32_t>(a.host_scalars)[index] = 0;
}

__device__ __forceinline__ bool route_is_live(const FerruleHipExpertGroupRoutePlanArgs &a, uint32_t route,
                                              int32_t &slot) {
  slot = ptr<const int32_t>(a.route_slots)[route];
  const int32_t generation = ptr<const int32_t>(a.route_generations)[route];
  return slot >= 0 && static_cast<uint32_t>(slot) < a.slot_capacity && generation > 0 &&
         ptr<const int32_t>(a.slot_generations)[slot] == generation;
}

// Each workgroup counts kCountRoutesPerGroup routes into an LDS histogram and adds its non-empty
// bins to the global counters: with 65 536 routes on 256 slots, one global atomic per route
// spends 119 us queueing on 256 addresses.  A thread's four routes are fetched together (clamped
// indices, no load inside a branch): a route costs two dependent load latencies, and a workgroup
// pays them once.
constexpr uint32_t kCountRoutesPerGroup = 1024;
__global__ __launch_bounds__(256) void route_count_kernel(FerruleHipExpertGroupRoutePlanArgs a) {
  __shared__ int32_t bins[1024];
  const bool privatised = a.slot_capacity <= 1024u;
  if (privatised) {
    for (uint32_t i = threadIdx.x; i < 1024u; i += 256u) bins[i] = 0;
    __syncthreads();
  }
  constexpr uint32_t kPerThread = kCountRoutesPerGroup / 256u;
  const uint32_t begin = blockIdx.x * kCountRoutesPerGroup + threadIdx.x;
  const uint32_t last_route = a.route_count - 1u;  // route_count >= 1 (checked by the launcher)
  int32_t slot[kPerThread], generation[kPerThread], current[kPerThread];
#pragma unroll
  for (uint32_t u = 0; u < kPerThread; ++u) {
    const uint32_t route = begin + u * 256u;
    const uint32_t at = min(route, last_route);
    const int32_t s = ptr<const int32_t>(a.route_slots)[at];
    generation[u] = ptr<const int32_t>(a.route_generations)[at];
    const bool candidate = route <= last_route && s >= 0 && static_cast<uint32_t>(s) < a.slot_capacity && generation[u] > 0;
    slot[u] = candidate ? s : -1;
  }
#pragma unroll
  for (uint32_t u = 0; u < kPerThread; ++u) current[u] = ptr<const int32_t>(a.slot_generations)[slot[u] >= 0 ? slot[u] : 0];
#pragma unroll
  for (uint32_t u = 0; u < kPerThread; ++u) {
    if (slot[u] >= 0 && current[u] == generation[u]) {
      if (privatised) {
        atomicAdd(&bins[slot[u]], 1);
      } else {
        atomicAdd(ptr<int32_t>(a.slot_counts) + slot[u], 1);
      }
    }
  }
  if (privatised) {
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < a.slot_capacity; i += 256u) {
      if (bins[i] != 0) atomicAdd(ptr<int32_t>(a.slot_counts) + i, bins[i]);
    }
  }
}

// Block-wide exclusive prefix sum of one value per thread (1024 threads).
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t value, uint32_t *wave_totals,
                                                         uint32_t &block_total) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = threadIdx.x >> 6;
  uint32_t inclusive = value;
#pragma unroll
  for (int offset = 1; offset < 64; offset <<= 1) {
    const uint32_t other = __shfl_up(inclusive, offset, 64);
    if (lane >= static_cast<uint32_t>(offset)) inclusive += other;
  }
  if (lane == 63u) wave_totals[wave] = inclusive;
  __syncthreads();
  uint32_t before = 0;
  uint32_t total = 0;
  const uint32_t waves = blockDim.x >> 6;
  for (uint32_t w = 0; w < waves; ++w) {
    const uint32_t t = wave_totals[w];
    if (w < wave) before += t;
    total += t;
  }
  __syncthreads();
  block_total = total;
  return before + inclusive - value;
}

// One workgroup of 1024 threads, thread s owns slot s.
__global__ __launch_bounds__(1024) void route_compact_kernel(FerruleHipExpertGroupRoutePlanArgs a) {
  __shared__ uint32_t wave_totals[16];
  const uint32_t slot = threadIdx.x;
  const bool in_range = slot < a.slot_capacity;
  const int32_t raw = in_range ? ptr<const int32_t>(a.slot_counts)[slot] : 0;
  const uint32_t count = raw > 0 ? static_cast<uint32_t>(raw) : 0u;
  const bool is_small = count != 0u && count < a.small_group_row_limit;
  const bool is_large = count != 0u && !is_small;

  uint32_t small_groups, large_groups, small_rows, large_rows;
  const uint32_t small_rank = block_exclusive_scan(is_small ? 1u : 0u, wave_totals, small_groups);
  const uint32_t large_rank = block_exclusive_scan(is_large ? 1u : 0u, wave_totals, large_groups);
  const uint32_t small_before = block_exclusive_scan(is_small ? count : 0u, wave_totals, small_rows);
  const uint32_t large_before = block_exclusive_scan(is_large ? count : 0u, wave_totals, large_rows);
  uint32_t max_rows = count;
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) max_rows = max(max_rows, __shfl_xor(max_rows, offset, 64));
  if ((threadIdx.x & 63u) == 0u) wave_totals[threadIdx.x >> 6] = max_rows;
  __syncthreads();
  max_rows = 0;
  for (uint32_t w = 0; w < (blockDim.x >> 6); ++w) max_rows = max(max_rows, wave_totals[w]);

  const uint32_t groups = small_groups + large_groups;
  const uint32_t total_rows = small_rows + large_rows;
  if (total_rows > a.route_capacity) {
    // the reference stops at the first group that does not fit and raises the flag
    if (threadIdx.x == 0) ptr<int32_t>(a.route_error)[0] = 1;
    return;
  }
  if (count != 0u) {
    const uint32_t group = is_small ? small_rank : small_groups + large_rank;
    const uint32_t offset = is_small ? small_before : small_rows + large_before;
    ptr<int32_t>(a.active_expert_slots)[group] = static_cast<int32_t>(slot);
    ptr<int32_t>(a.active_group_generations)[group] = ptr<const int32_t>(a.slot_generations)[slot];
    ptr<int32_t>(a.expert_route_indptr)[group] = static_cast<int32_t>(offset);
    ptr<int32_t>(a.expert_route_counts)[group] = static_cast<int32_t>(count);
    ptr<int32_t>(a.slot_route_offsets)[slot] = static_cast<int32_t>(offset);
  }
  if (threadIdx.x == 0) {
    ptr<int32_t>(a.expert_route_indptr)[groups] = static_cast<int32_t>(total_rows);
    int32_t *scalars = ptr<int32_t>(a.host_scalars);
    scalars[0] = static_cast<int32_t>(groups);
    scalars[1] = static_cast<int32_t>(small_groups);
    scalars[2] = static_cast<int32_t>(max_rows);
    scalars[3] = static_cast<int32_t>(total_rows);
  }
}

// One workgroup of 16 waves per slot.  Wave w owns the w-th contiguous segment of the route
// list: a first pass counts the slot's live routes per segment, a prefix over the 16 counts gives
// every wave its first row, a second pass writes.  Rows of a group are in ascending route order.
// No barrier inside the passes (one per 256 routes made 65 536 routes take 199 us).
__global__ __launch_bounds__(1024) void route_scatter_kernel(FerruleHipExpertGroupRoutePlanArgs a) {
  __shared__ uint32_t wave_counts[16];
  const uint32_t slot = blockIdx.x;
  const int32_t offset = ptr<const int32_t>(a.slot_route_offsets)[slot];
  if (offset < 0) return;  // no live route points at this slot
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = threadIdx.x >> 6;
  const uint32_t per_wave = ((a.route_count + 15u) / 16u + 63u) & ~63u;
  const uint32_t begin = min(wave * per_wave, a.route_count);
  const uint32_t end = min(begin + per_wave, a.route_count);
  auto hit_at = [&](uint32_t route) {
    int32_t s;
    return route < end && route_is_live(a, route, s) && static_cast<uint32_t>(s) == slot;
  };
  uint32_t count = 0;
  for (uint32_t base = begin; base < end; base += 64u) count += __popcll(__ballot(hit_at(base + lane)));
  if (lane == 0u) wave_counts[wave] = count;
  __syncthreads();
  uint32_t before = 0, total = 0;
#pragma unroll
  for (uint32_t w = 0; w < 16u; ++w) {
    const uint32_t c = wave_counts[w];
    if (w < wave) before += c;
    total += c;
  }
  uint32_t running = static_cast<uint32_t>(offset) + before;
  for (uint32_t base = begin; base < end; base += 64u) {
    const uint32_t route = base + lane;
    const bool hit = hit_at(route);
    const uint64_t ballot = __ballot(hit);
    if (hit) {
      const uint32_t position = running + __popcll(ballot & ((1ull << lane) - 1ull));
      if (position >= a.route_capacity) {
        atomicOr(ptr<int32_t>(a.route_error), 1);
      } else {
        ptr<int32_t>(a.route_token_indices)[position] = static_cast<int32_t>(route / a.routes_per_token);
        ptr<int32_t>(a.route_indices)[position] = static_cast<int32_t>(route);
        ptr<float>(a.route_weights)[position] = ptr<const float>(a.router_weights)[route];
      }
    }
    running += __popcll(ballot);
  }
  if (threadIdx.x == 0) ptr<int32_t>(a.slot_cursors)[slot] = static_cast<int32_t>(total);
}

// The same scatter for long route lists and at most 1024 slots: one workgroup per chunk of 1024
// routes instead of one per slot.  With one workgroup per slot every workgroup reads the whole
// route list twice (256 slots x 65 536 routes: 101 us); here workgroup c reads the routes before
// its chunk once to count them per slot (LDS bins) and ranks its own 1024 routes:
//   row = slot_route_offsets[slot] + live routes of the slot in earlier chunks
//         + ... in earlier waves of the chunk + ... in earlier lanes of the wave
// i.e. ascending route order inside a group, exactly what route_scatter_kernel writes.
constexpr uint32_t kScatterChunk = 1024;
__global__ __launch_bounds__(1024) void route_scatter_chunks_kernel(FerruleHipExpertGroupRoutePlanArgs a) {
  __shared__ uint32_t before[1024];         // live routes per slot in the chunks before this one
  __shared__ uint8_t in_wave[16][1024];     // live routes per slot in each wave of this chunk (<= 64)
  __shared__ int32_t current[1024];         // the slots' generations: a route's liveness costs one global load round
  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & 63u;
  const uint32_t wave = tid >> 6;
  const uint32_t chunk_begin = blockIdx.x * kScatterChunk;
  const uint32_t last_route = a.route_count - 1u;  // route_count >= 1 (checked by the launcher)
  before[tid] = 0;
  current[tid] = tid < a.slot_capacity ? ptr<const int32_t>(a.slot_generations)[tid] : 0;
#pragma unroll
  for (uint32_t w = 0; w < 16u; ++w) in_wave[w][tid] = 0;
  __syncthreads();
  // live slot of a route (-1: none), loads unconditional (clamped index) so that all are in flight together
  constexpr uint32_t kPerPass = 16;
  auto live_slots = [&](uint32_t first, int32_t (&out)[kPerPass]) {
    int32_t gen[kPerPass];
#pragma unroll
    for (uint32_t u = 0; u < kPerPass; ++u) {
      const uint32_t at = min(first + u * 1024u, last_route);
      out[u] = ptr<const int32_t>(a.route_slots)[at];
      gen[u] = ptr<const int32_t>(a.route_generations)[at];
    }
#pragma unroll
    for (uint32_t u = 0; u < kPerPass; ++u) {
      const int32_t s = out[u];
      const bool candidate = first + u * 1024u <= last_route && s >= 0 && static_cast<uint32_t>(s) < a.slot_capacity && gen[u] > 0;
      out[u] = candidate && current[s] == gen[u] ? s : -1;
    }
  };
  // routes before the chunk, sixteen per thread and pass
  for (uint32_t base = 0; base < chunk_begin; base += kPerPass * 1024u) {
    int32_t s[kPerPass];
    live_slots(base + tid, s);
#pragma unroll
    for (uint32_t u = 0; u < kPerPass; ++u) {
      if (s[u] >= 0 && base + tid + u * 1024u < chunk_begin) atomicAdd(&before[s[u]], 1u);
    }
  }
  // this thread's own route
  const uint32_t route = chunk_begin + tid;
  int32_t mine;
  {
    const uint32_t at = min(route, last_route);
    const int32_t s = ptr<const int32_t>(a.route_slots)[at];
    const int32_t gen = ptr<const int32_t>(a.route_generations)[at];
    const bool candidate = route <= last_route && s >= 0 && static_cast<uint32_t>(s) < a.slot_capacity && gen > 0;
    mine = candidate && current[s] == gen ? s : -1;
  }
  // rank among the wave's lanes with the same slot, and how many there are
  uint32_t rank = 0, same = 0;
  for (uint32_t j = 0; j < 64u; ++j) {
    const int32_t other = __builtin_amdgcn_readlane(mine, static_cast<int>(j));
    const bool equal = other == mine;
    rank += (equal && j < lane) ? 1u : 0u;
    same += equal ? 1u : 0u;
  }
  if (mine >= 0 && rank + 1u == same) in_wave[wave][mine] = static_cast<uint8_t>(same);  // the slot's last lane
  __syncthreads();
  if (mine >= 0) {
    uint32_t earlier_waves = 0;
    for (uint32_t w = 0; w < wave; ++w) earlier_waves += in_wave[w][mine];
    const int32_t offset = ptr<const int32_t>(a.slot_route_offsets)[mine];
    if (offset >= 0) {
      const uint32_t position = static_cast<uint32_t>(offset) + before[mine] + earlier_waves + rank;
      if (position >= a.route_capacity) {
        atomicOr(ptr<int32_t>(a.route_error), 1);
      } else {
        ptr<int32_t>(a.route_token_indices)[position] = static_cast<int32_t>(route / a.routes_per_token);
        ptr<int32_t>(a.route_indices)[position] = static_cast<int32_t>(route);
        ptr<float>(a.route_weights)[position] = ptr<const float>(a.router_weights)[route];
      }
    }
  }
  // the last chunk knows every slot's total
  if (blockIdx.x + 1u == gridDim.x && tid < a.slot_capacity) {
    uint32_t total = before[tid];
#pragma unroll
    for (uint32_t w = 0; w < 16u; ++w) total += in_wave[w][tid];
    if (ptr<const int32_t>(a.slot_route_offsets)[tid] >= 0) ptr<int32_t>(a.slot_cursors)[tid] = static_cast<int32_t>(total);
  }
}

// Kinds 2..5 and the flag reset of kind 1 in one launch for decode batches (a few hundred
// routes).  One workgroup per slot and no communication between workgroups: each one rebuilds
// the slot histogram of the whole (small) route list in LDS, scans it, and from that knows its
// own group index and row offset; it then scatters the routes of its slot in ascending order
// (the ballot scheme of route_scatter_kernel) and writes the entries of the plan that belong to
// its slot, to the group index equal to its workgroup index when that group does not exist,
// and its share of the untouched tail of the row arrays.  Redundant work per workgroup is a
// few microseconds on otherwise idle CUs; the alternative is five dependent launches.
__global__ __launch_bounds__(256) void route_fused_decode_plan_kernel(FerruleHipExpertGroupRoutePlanArgs a) {
  constexpr uint32_t kPerThread = FERRULE_HIP_FUSED_PLAN_MAX_ROUTES / 256u;  // routes kept per thread
  __shared__ int32_t counts[1024];
  __shared__ uint64_t wave_sums[4];
  __shared__ uint32_t wave_max[4];
  __shared__ uint32_t mine[3];  // results of the owner of this workgroup's slot
  __shared__ uint32_t wave_counts[kPerThread][4];
  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & 63u;
  const uint32_t wave = tid >> 6;
  const uint32_t slot = blockIdx.x;
  // live slot of route tid + 256 i (or -1), read once and kept for the scatter below.  Every
  // load is unconditional (index clamped, result selected afterwards): the loads of a thread are
  // then all in flight together instead of one branch and one round trip each.
  int32_t rslot[kPerThread];
#pragma unroll
  for (uint32_t i = 0; i < 4u; ++i) counts[tid * 4u + i] = 0;
#pragma unroll
  for (uint32_t i = 0; i < kPerThread; ++i) rslot[i] = -1;
  if (a.route_count != 0u) {  // uniform
    const uint32_t last_route = a.route_count - 1u;
    int32_t rgen[kPerThread], current[kPerThread];
#pragma unroll
    for (uint32_t i = 0; i < kPerThread; ++i) {
      const uint32_t route = tid + 256u * i;
      const uint32_t at = min(route, last_route);
      const int32_t s = ptr<const int32_t>(a.route_slots)[at];
      rgen[i] = ptr<const int32_t>(a.route_generations)[at];
      const bool candidate =
          route <= last_route && s >= 0 && static_cast<uint32_t>(s) < a.slot_capacity && rgen[i] > 0;
      rslot[i] = candidate ? s : -1;
    }
#pragma unroll
    for (uint32_t i = 0; i < kPerThread; ++i) {
      current[i] = ptr<const int32_t>(a.slot_generations)[rslot[i] >= 0 ? rslot[i] : 0];
    }
#pragma unroll
    for (uint32_t i = 0; i < kPerThread; ++i) rslot[i] = current[i] == rgen[i] ? rslot[i] : -1;
  }
  __syncthreads();
#pragma unroll
  for (uint32_t i = 0; i < kPerThread; ++i) {
    if (rslot[i] >= 0) atomicAdd(&counts[rslot[i]], 1);
  }
  __syncthreads();
  // thread t scans slots 4t .. 4t+3: small/large group ranks and row offsets (kind 4).  The four
  // sums ride in one 64-bit word (groups <= 1024 and rows <= 2048 fit 16 bits each).
  uint32_t cnt[4], max_rows = 0;
  uint64_t packed = 0;
#pragma unroll
  for (uint32_t i = 0; i < 4u; ++i) {
    const uint32_t s = tid * 4u + i;
    cnt[i] = s < a.slot_capacity ? static_cast<uint32_t>(counts[s]) : 0u;
    const bool small = cnt[i] != 0u && cnt[i] < a.small_group_row_limit;
    if (cnt[i] != 0u) {
      packed += small ? (1ull | (static_cast<uint64_t>(cnt[i]) << 32))
                      : ((1ull << 16) | (static_cast<uint64_t>(cnt[i]) << 48));
    }
    max_rows = max(max_rows, cnt[i]);
  }
  uint64_t inclusive = packed;
#pragma unroll
  for (int offset = 1; offset < 64; offset <<= 1) {
    const uint64_t other = __shfl_up(inclusive, offset, 64);
    if (lane >= static_cast<uint32_t>(offset)) inclusive += other;
  }
#pragma unroll
  for (int offset = 32; offset > 0; offset >>= 1) max_rows = max(max_rows, __shfl_xor(max_rows, offset, 64));
  if (lane == 63u) wave_sums[wave] = inclusive;
  if (lane == 0u) wave_max[wave] = max_rows;
  __syncthreads();
  uint64_t before_waves = 0, total = 0;
#pragma unroll
  for (uint32_t w = 0; w < 4u; ++w) {
    const uint64_t t = wave_sums[w];
    if (w < wave) before_waves += t;
    total += t;
  }
  max_rows = max(max(wave_max[0], wave_max[1]), max(wave_max[2], wave_max[3]));
  const uint64_t exclusive = before_waves + inclusive - packed;
  uint32_t small_rank = static_cast<uint32_t>(exclusive & 0xffffu);
  uint32_t large_rank = static_cast<uint32_t>((exclusive >> 16) & 0xffffu);
  uint32_t small_before = static_cast<uint32_t>((exclusive >> 32) & 0xffffu);
  uint32_t large_before = static_cast<uint32_t>(exclusive >> 48);
  const uint32_t small_groups = static_cast<uint32_t>(total & 0xffffu);
  const uint32_t large_groups = static_cast<uint32_t>((total >> 16) & 0xffffu);
  const uint32_t small_rows = static_cast<uint32_t>((total >> 32) & 0xffffu);
  const uint32_t large_rows = static_cast<uint32_t>(total >> 48);
  const uint32_t groups = small_groups + large_groups;
  const uint32_t total_rows = small_rows + large_rows;
  const bool overflow = total_rows > a.route_capacity;
  if (tid == slot / 4u) {
#pragma unroll
    for (uint32_t i = 0; i < 4u; ++i) {
      const bool small = cnt[i] != 0u && cnt[i] < a.small_group_row_limit;
      if (i == (slot & 3u)) {
        mine[0] = cnt[i];
        mine[1] = small ? small_rank : small_groups + large_rank;         // group index
        mine[2] = small ? small_before : small_rows + large_before;       // first row
      }
      if (small) {
        ++small_rank;
        small_before += cnt[i];
      } else if (cnt[i] != 0u) {
        ++large_rank;
        large_before += cnt[i];
      }
    }
  }
  // kind 5 for this slot, first half: where this wave's hits of every 256-route chunk start
  bool hit[kPerThread];
  uint32_t before_in_wave[kPerThread];
#pragma unroll
  for (uint32_t i = 0; i < kPerThread; ++i) {
    hit[i] = rslot[i] == static_cast<int32_t>(slot);
    const uint64_t ballot = __ballot(hit[i]);
    before_in_wave[i] = __popcll(ballot & ((1ull << lane) - 1ull));
    if (lane == 0u) wave_counts[i][wave] = __popcll(ballot);
  }
  __syncthreads();
  const uint32_t count = mine[0], group = mine[1], offset = mine[2];
  const bool placed = count != 0u && !overflow;  // kind 4 stops before writing anything on overflow

  // entries of this slot, and of the group index = this workgroup's index when no group has it
  if (tid == 0u) {
    ptr<int32_t>(a.slot_counts)[slot] = static_cast<int32_t>(count);
    ptr<int32_t>(a.slot_route_offsets)[slot] = placed ? static_cast<int32_t>(offset) : -1;
    if (placed) {
      ptr<int32_t>(a.active_expert_slots)[group] = static_cast<int32_t>(slot);
      ptr<int32_t>(a.active_group_generations)[group] = ptr<const int32_t>(a.slot_generations)[slot];
      ptr<int32_t>(a.expert_route_indptr)[group] = static_cast<int32_t>(offset);
      ptr<int32_t>(a.expert_route_counts)[group] = static_cast<int32_t>(count);
    }
    const uint32_t live_groups = overflow ? 0u : groups;
    if (slot >= live_groups) {
      ptr<int32_t>(a.active_expert_slots)[slot] = -1;
      ptr<int32_t>(a.active_group_generations)[slot] = 0;
      ptr<int32_t>(a.expert_route_counts)[slot] = 0;
      if (slot > live_groups) ptr<int32_t>(a.expert_route_indptr)[slot] = 0;
    }
    if (slot == 0u) {
      int32_t *indptr = ptr<int32_t>(a.expert_route_indptr);
      indptr[live_groups] = overflow ? 0 : static_cast<int32_t>(total_rows);
      if (a.slot_capacity > live_groups) indptr[a.slot_capacity] = 0;
      if (live_groups == a.slot_capacity) indptr[a.slot_capacity] = static_cast<int32_t>(total_rows);
      int32_t *scalars = ptr<int32_t>(a.host_scalars);
      scalars[0] = overflow ? 0 : static_cast<int32_t>(groups);
      scalars[1] = overflow ? 0 : static_cast<int32_t>(small_groups);
      scalars[2] = overflow ? 0 : static_cast<int32_t>(max_rows);
      scalars[3] = overflow ? 0 : static_cast<int32_t>(total_rows);
      ptr<int32_t>(a.route_error)[0] = overflow ? 1 : 0;
    }
  }
  // flags of kind 1 and the rows no live route lands on (kind 2's fill), spread over the grid
  const uint32_t first_free = overflow ? 0u : total_rows;
  for (uint32_t i = slot * 256u + tid; i < a.route_capacity; i += gridDim.x * 256u) {
    if (i < a.route_count) ptr<int32_t>(a.route_written)[i] = 0;
    if (i >= first_free) {
      ptr<int32_t>(a.route_token_indices)[i] = -1;
      ptr<int32_t>(a.route_indices)[i] = -1;
      ptr<float>(a.route_weights)[i] = 0.0f;
    }
  }
  for (uint32_t i = a.route_capacity + slot * 256u + tid; i < a.route_count; i += gridDim.x * 256u) {
    ptr<int32_t>(a.route_written)[i] = 0;
  }

  // kind 5, second half: ascending route order = chunk after chunk, wave after wave, lane after lane
  uint32_t running = 0;
#pragma unroll
  for (uint32_t i = 0; i < kPerThread; ++i) {
    uint32_t before = 0, chunk_total = 0;
#pragma unroll
    for (uint32_t w = 0; w < 4u; ++w) {
      const uint32_t c = wave_counts[i][w];
      if (w < wave) before += c;
      chunk_total += c;
    }
    if (placed && hit[i]) {
      const uint32_t route = tid + 256u * i;
      const uint32_t position = offset + running + before + before_in_wave[i];
      ptr<int32_t>(a.route_token_indices)[position] = static_cast<int32_t>(route / a.routes_per_token);
      ptr<int32_t>(a.route_indices)[position] = static_cast<int32_t>(route);
      ptr<float>(a.route_weights)[position] = ptr<const float>(a.router_weights)[route];
    }
    running += chunk_total;
  }
  if (tid == 0u) ptr<int32_t>(a.slot_cursors)[slot] = placed ? static_cast<int32_t>(running) : 0;
}

}  // namespace
}  // namespace ferrule_hip

extern "C" int32_t ferrule_hip_core_expert_group_route_plan_launch(
    const FerruleHipExpertGroupRoutePlanArgs *args) {
  using namespace ferrule_hip;
  // invalid => hipErrorInvalidValue (1), as portable/entrypoints.cu:2029-2044
  if (args == nullptr) return 1;
  const FerruleHipExpertGroupRoutePlanArgs &a = *args;
  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(a.stream));
  auto blocks = [](uint64_t count) { return static_cast<uint32_t>((count + 255u) / 256u); };
  clear_launch_error();
  switch (a.kind) {
  case FERRULE_HIP_EXPERT_GROUP_ROUTE_INIT_INVOCATION: {
    if (a.route_output == 0 || a.route_written == 0 || a.route_error == 0) return 1;
    const uint64_t count = a.output_elements > a.route_count ? a.output_elements : a.route_count;
    route_init_invocation_kernel<<<blocks(count > 0 ? count : 1), 256, 0, stream>>>(a);
    break;
  }
  case FERRULE_HIP_EXPERT_GROUP_ROUTE_INIT_PLAN: {
    if (a.slot_counts == 0 || a.slot_route_offsets == 0 || a.slot_cursors == 0 ||
        a.active_expert_slots == 0 || a.active_group_generations == 0 || a.expert_route_indptr == 0 ||
        a.expert_route_counts == 0 || a.route_token_indices == 0 || a.route_indices == 0 ||
        a.route_weights == 0 || a.host_scalars == 0)
      return 1;
    uint64_t count = static_cast<uint64_t>(a.slot_capacity) + 1u;
    if (a.route_capacity > count) count = a.route_capacity;
    if (count < 4) count = 4;
    route_init_plan_kernel<<<blocks(count), 256, 0, stream>>>(a);
    break;
  }
  case FERRULE_HIP_EXPERT_GROUP_ROUTE_COUNT:
    if (a.route_slots == 0 || a.route_generations == 0 || a.slot_generations == 0 || a.slot_counts == 0)
      return 1;
    if (a.route_count == 0 || a.slot_capacity == 0) return 0;  // nothing can be live
    route_count_kernel<<<(a.route_count + kCountRoutesPerGroup - 1u) / kCountRoutesPerGroup, 256, 0, stream>>>(a);
    break;
  case FERRULE_HIP_EXPERT_GROUP_ROUTE_COMPACT:
    if (a.slot_capacity == 0 || a.slot_capacity > 1024u) return 1;
    if (a.slot_counts == 0 || a.slot_generations == 0 || a.host_scalars == 0 || a.route_error == 0) return 1;
    route_compact_kernel<<<1, 1024, 0, stream>>>(a);
    break;
  case FERRULE_HIP_EXPERT_GROUP_ROUTE_SCATTER:
    if (a.routes_per_token == 0 || a.slot_capacity == 0) return 1;
    if (a.route_slots == 0 || a.route_generations == 0 || a.slot_generations == 0 || a.router_weights == 0 ||
        a.slot_route_offsets == 0 || a.slot_cursors == 0 || a.route_token_indices == 0 || a.route_indices == 0 ||
        a.route_weights == 0 || a.route_error == 0)
      return 1;
    if (a.route_count == 0) return 0;
    if (a.slot_capacity <= 1024u && a.route_count > 4u * kScatterChunk) {
      route_scatter_chunks_kernel<<<(a.route_count + kScatterChunk - 1u) / kScatterChunk, 1024, 0, stream>>>(a);
    } else {
      route_scatter_kernel<<<a.slot_capacity, 1024, 0, stream>>>(a);
    }
    break;
  case FERRULE_HIP_EXPERT_GROUP_ROUTE_FUSED_DECODE_PLAN:
    if (a.slot_capacity == 0 || a.slot_capacity > 1024u || a.route_count > FERRULE_HIP_FUSED_PLAN_MAX_ROUTES ||
        a.routes_per_token == 0)
      return 1;
    if (a.route_slots == 0 || a.route_generations == 0 || a.router_weights == 0 || a.slot_generations == 0 ||
        a.slot_counts == 0 || a.slot_route_offsets == 0 || a.slot_cursors == 0 || a.active_expert_slots == 0 ||
        a.active_group_generations == 0 || a.expert_route_indptr == 0 || a.expert_route_counts == 0 ||
        a.route_token_indices == 0 || a.route_indices == 0 || a.route_weights == 0 || a.host_scalars == 0 ||
        a.route_written == 0 || a.route_error == 0)
      return 1;
    route_fused_decode_plan_kernel<<<a.slot_capacity, 256, 0, stream>>>(a);
    break;
  default:
    return 1;
  }
  return static_cast<int32_t>(take_launch_error());
}
