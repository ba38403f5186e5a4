// Grouped MXFP4 MoE for packed prefill / verification rows: drop-in for
// ferrule_cutlass_grouped_fp4_moe_{workspace_size,can_implement,launch}
// (abi/cutlass_provider.h:337-376, 446-453; kernels sm103/grouped_fp4_moe.cuh:578-1222).
//
//   tile map   one workgroup turns expert_route_indptr into a list of (group, first row)
//              token tiles, so the GEMM grids need no host knowledge of the group sizes
//   gate/up    grouped GEMM on v_mfma_scale_f32_16x16x128_f8f6f4: FP8 token rows (gathered
//              through route_token_indices by the loads themselves, nothing is copied) times
//              the expert's MXFP4 W1 and W3, which share every token fragment.  Epilogue in
//              registers: SwiGLU x route weight, then the FP8-K128 activation quantiser -
//              a wave owns exactly one 128-wide block of the intermediate dimension, so the
//              block maximum is 32 values per lane and two cross-lane steps
//   down       grouped GEMM of the quantised hidden rows times MXFP4 W2, fp32 route_output
//
// Arithmetic is that of CpuReferenceExpertExecutor with FP8-K128 activation quantisation
// (crates/ferrule-model/src/moe/executor.rs:82-124): exact products, fp32 accumulation in
// another order, the CPU quantiser's tie rule.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ferrule_hip_diagnostics.h"
#include "../../include/ferrule_hip_provider.h"
#include "mx_gemm.cuh"
#include "quant_math.h"
#include "swiglu_quant.cuh"

namespace ferrule_hip {
namespace {

constexpr uint32_t kTileRows = 128;  // token rows per workgroup tile, both GEMMs

// Eight waves per workgroup (two per SIMD, 128 accumulator registers each): while one wave of a
// SIMD sits in the per-K-step wait and barrier the other one issues MFMAs.  Four waves with 256
// accumulator registers each ran the layer 13 % slower.
// Smaller tiles with two workgroups per CU (down 256 x 128, gate/up 2 x 128 x 128, four waves and two
// stages each) ran the layer 15 % and 35 % slower.
// A wave's 16-row token fragments are every fourth / every second one of the tile (SPREAD_T): the
// last tile of an expert is ragged, its dead fragments are skipped (gemm_mainloop_ragged), and spread
// like this the work that remains is even over the waves.
// gate/up: 2 matrices x 256 features x 128 tokens per workgroup; a wave = 128 features x 32 tokens
template <int NSTAGE>
using GateUpShape = GemmShape<kMfmaFmtFp4, 2, 8, 2, 2, 4, NSTAGE, true>;
// down: 512 features x 128 tokens; a wave = 128 features x 64 tokens
template <int NSTAGE>
using DownShape = GemmShape<kMfmaFmtFp4, 1, 8, 4, 4, 2, NSTAGE, true>;
static_assert(GateUpShape<3>::TM == kTileRows && DownShape<3>::TM == kTileRows, "tile map granularity");

struct GroupedParams {
  const int32_t *active_expert_slots;
  const uint32_t *expert_route_indptr;
  const int32_t *route_token_indices;
  const int32_t *route_indices;
  const float *route_weights;
  const uint64_t *gate_ptrs, *gate_scale_ptrs, *up_ptrs, *up_scale_ptrs, *down_ptrs, *down_scale_ptrs;
  const uint8_t *input_fp8;
  const uint8_t *input_ue8m0;
  float *route_output;
  int32_t *route_written;
  int32_t *route_error;
  // workspace
  int32_t *tile_map;  // [0] = tile count (a 64-byte head), then one TileEntry per tile
  uint8_t *hq;        // [rows][I] E4M3
  uint8_t *hs;        // [rows][I/128] UE8M0
  float *hidden_f32;  // optional debug copy of h
  uint32_t groups, slot_capacity, rows, num_tokens, num_routes, input_size, intermediate_size, hidden_size;
  uint32_t max_tiles;
  float swiglu_limit;
  uint32_t block_major;  // expert weights and scales in the order of ferrule_hip_prepare_mxfp4_block_major
};

__host__ __device__ inline uint64_t align256(uint64_t v) { return (v + 255u) & ~static_cast<uint64_t>(255u); }

// All a workgroup has to know about a 128-row token tile, in one record: its look-up is ONE load
// whose address depends on the item number only (group -> slot -> pointer tables would be a chain
// of three).  Tiles of one panel (kPanelTiles below) belong to one group and differ in row0 only.
struct TileEntry {
  int32_t group, row0, panel_first, panel_tiles;  // row0: first routed row; the panel's first tile and tile count
  int32_t row_end, slot, reserved0, reserved1;    // end of the group's rows; its expert slot
  uint64_t gate_w, gate_s, up_w, up_s, down_w, down_s;
};
static_assert(sizeof(TileEntry) == 80, "twenty dwords");
constexpr uint64_t kTileMapHead = 64;  // [0] = tile count

struct WorkspaceLayout {
  uint64_t tile_map, hq, hs, total;
  uint32_t max_tiles;
};

WorkspaceLayout workspace_layout(uint32_t groups, uint32_t rows, uint32_t intermediate) {
  WorkspaceLayout l;
  l.max_tiles = rows / kTileRows + groups;  // sum over groups of ceil(m/128) is at most this
  uint64_t cursor = 0;
  l.tile_map = cursor;
  cursor = align256(cursor + kTileMapHead + static_cast<uint64_t>(l.max_tiles) * sizeof(TileEntry));
  l.hq = cursor;
  cursor = align256(cursor + static_cast<uint64_t>(rows) * intermediate);
  l.hs = cursor;
  cursor = align256(cursor + static_cast<uint64_t>(rows) * (intermediate / 128u));
  l.total = cursor;
  return l;
}

// Token tiles of one expert are cut into panels of at most kPanelTiles.  Work items run panel after
// panel; inside a panel the feature tile is the slow index and the token tile the fast one.  What
// is in flight at any time (a few hundred consecutive items) is then one weight tile per run of
// token tiles, and a panel's token rows (at most kPanelTiles x 128 rows of K bytes) come back once
// per feature tile after a few tens of MB of other traffic, i.e. from the 256 MB memory-side cache
// rather than from HBM.  With the feature tile as the slow index of the WHOLE problem every token
// row was fetched from HBM once per feature tile (8 and 14 times).
constexpr uint32_t kPanelTiles = 32;

// (group, first row, first tile of its panel, tiles of its panel) of every 128-row token tile, in
// group order.  One workgroup; groups are handled 256 at a time with an LDS prefix sum.  Groups
// with an invalid slot get no tiles and raise route_error (their routes stay unwritten, so the
// reducer yields NaN for them).
__device__ __forceinline__ TileEntry *tile_entries(const GroupedParams &p) {
  return reinterpret_cast<TileEntry *>(reinterpret_cast<uint8_t *>(p.tile_map) + kTileMapHead);
}

__global__ __launch_bounds__(256) void tile_map_kernel(GroupedParams p) {
  __shared__ uint32_t scan[256];
  __shared__ uint32_t base;
  if (threadIdx.x == 0) base = 0;
  __syncthreads();
  for (uint32_t g0 = 0; g0 < p.groups; g0 += 256u) {
    const uint32_t g = g0 + threadIdx.x;
    uint32_t begin = 0, tiles = 0;
    if (g < p.groups) {
      begin = p.expert_route_indptr[g];
      const uint32_t end = p.expert_route_indptr[g + 1];
      const int32_t slot = p.active_expert_slots[g];
      const bool ok = slot >= 0 && static_cast<uint32_t>(slot) < p.slot_capacity && begin <= end && end <= p.rows;
      if (ok) {
        tiles = (end - begin + kTileRows - 1u) / kTileRows;
      } else {
        atomicOr(p.route_error, 1);
      }
    }
    scan[threadIdx.x] = tiles;
    __syncthreads();
    for (uint32_t d = 1; d < 256u; d <<= 1) {
      const uint32_t add = threadIdx.x >= d ? scan[threadIdx.x - d] : 0u;
      __syncthreads();
      scan[threadIdx.x] += add;
      __syncthreads();
    }
    const uint32_t first = base + scan[threadIdx.x] - tiles;
    if (tiles != 0u) {
      const int32_t slot = p.active_expert_slots[g];
      TileEntry e;
      e.group = static_cast<int32_t>(g);
      e.row_end = static_cast<int32_t>(p.expert_route_indptr[g + 1]);
      e.slot = slot;
      e.reserved0 = e.reserved1 = 0;
      e.gate_w = p.gate_ptrs[slot];
      e.gate_s = p.gate_scale_ptrs[slot];
      e.up_w = p.up_ptrs[slot];
      e.up_s = p.up_scale_ptrs[slot];
      e.down_w = p.down_ptrs[slot];
      e.down_s = p.down_scale_ptrs[slot];
      for (uint32_t j = 0; j < tiles && first + j < p.max_tiles; ++j) {
        const uint32_t panel_first = j - j % kPanelTiles;
        e.row0 = static_cast<int32_t>(begin + j * kTileRows);
        e.panel_first = static_cast<int32_t>(first + panel_first);
        e.panel_tiles = static_cast<int32_t>(min(kPanelTiles, tiles - panel_first));
        tile_entries(p)[first + j] = e;
      }
    }
    __syncthreads();
    if (threadIdx.x == 255) base += scan[255];
    __syncthreads();
  }
  if (threadIdx.x == 0) p.tile_map[0] = static_cast<int32_t>(min(base, p.max_tiles));
}

// Work item of a workgroup.  Items are numbered panel after panel (see kPanelTiles); a panel of n
// token tiles starting at tile a owns items [a * feature_tiles, (a + n) * feature_tiles).
// Workgroups are dealt round-robin to the 8 XCDs (each with its own L2): runs of kXcdRun
// consecutive items go to one XCD, so that what shares a weight tile or a token tile shares an L2,
// and the runs go round the XCDs, so that every XCD gets the same mix of full and ragged tiles.
struct GroupedItem {
  uint32_t tile, ftile, row0, m;   // token tile, feature tile, first routed row, rows (1..128)
  const TileEntry *entry;          // of a tile of the same panel: group, slot and pointers are the item's
  bool live;
};
constexpr uint32_t kXcdRun = 32;
// Item number `id` in the order above.
__device__ __forceinline__ GroupedItem grouped_item_at(const GroupedParams &p, uint32_t feature_tiles, uint32_t id) {
  GroupedItem item;
  const uint32_t coarse = id / feature_tiles;  // a tile of the item's panel
  item.live = coarse < static_cast<uint32_t>(p.tile_map[0]);
  item.tile = item.ftile = item.row0 = 0;
  item.m = 1;
  item.entry = tile_entries(p);
  if (!item.live) return item;
  // one entry says it all: the item's tile lies in the same panel (same group) as `coarse`
  const TileEntry *entry = tile_entries(p) + coarse;
  const uint32_t panel_first = static_cast<uint32_t>(entry->panel_first);
  const uint32_t panel_tiles = static_cast<uint32_t>(entry->panel_tiles);
  const uint32_t local = id - panel_first * feature_tiles;
  item.ftile = local / panel_tiles;
  item.tile = panel_first + local % panel_tiles;
  item.row0 = static_cast<uint32_t>(entry->row0) + (item.tile - coarse) * kTileRows;  // wraps for earlier tiles
  item.m = min(kTileRows, static_cast<uint32_t>(entry->row_end) - item.row0);
  item.entry = entry;
  return item;
}
__device__ __forceinline__ const uint8_t *entry_ptr(uint64_t bits) {
  return reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(bits));
}
// One workgroup per item: the item of this workgroup.
__device__ __forceinline__ GroupedItem grouped_item(const GroupedParams &p, uint32_t feature_tiles) {
  uint32_t id = blockIdx.x;
  const uint32_t whole = gridDim.x - gridDim.x % (8u * kXcdRun);
  if (id < whole) {
    const uint32_t xcd = id & 7u, j = id >> 3;
    id = ((j / kXcdRun) * 8u + xcd) * kXcdRun + j % kXcdRun;
  }
  return grouped_item_at(p, feature_tiles, id);
}
// Persistent workgroups, kXcdRun per XCD (a grid of 8 * kXcdRun): workgroup (xcd, j) takes item j
// of every run of its XCD, so the workgroups of an XCD work on one run at a time, as above.
__device__ __forceinline__ GroupedItem grouped_item_of_round(const GroupedParams &p, uint32_t feature_tiles,
                                                             uint32_t round) {
  const uint32_t xcd = blockIdx.x & 7u, j = blockIdx.x >> 3;
  return grouped_item_at(p, feature_tiles, (round * 8u + xcd) * kXcdRun + j);
}

template <typename T>
__device__ __forceinline__ const T *slot_ptr(const uint64_t *table, int32_t slot) {
  return reinterpret_cast<const T *>(static_cast<uintptr_t>(table[slot]));
}

template <typename S>
__host__ __device__ constexpr uint32_t grouped_lds_bytes(uint32_t cols) {
  return S::NSTAGE * S::kStageBytes + ((S::TM * scale_row_pitch(cols) + 15u) & ~15u);
}

// Scale bytes of the tile's S::TM rows -> LDS, `cols` per row; row_base(r) = the row's first
// byte in global memory.  A row belongs to kThreads / TM adjacent threads that copy its dwords
// in turn: whatever row_base has to look up is looked up once per thread, and the copies of a
// thread do not depend on each other.  (One byte per thread and pass, each behind its own index
// lookup, kept a workgroup busy for tens of microseconds before its first K step.)
template <typename S, typename RowBase>
__device__ __forceinline__ void stage_row_scales(uint8_t *xsc, uint32_t cols, RowBase row_base) {
  constexpr uint32_t kPerRow = S::kThreads / S::TM;
  static_assert(S::kThreads % S::TM == 0 && kPerRow >= 1, "whole threads per row");
  const uint32_t row = threadIdx.x / kPerRow, first = threadIdx.x % kPerRow;
  const uint8_t *src = row_base(row);
  uint8_t *dst = xsc + row * scale_row_pitch(cols);
  if (((cols | static_cast<uint32_t>(reinterpret_cast<uintptr_t>(src))) & 3u) == 0u) {
#pragma unroll 4
    for (uint32_t j = first; j < cols / 4u; j += kPerRow) {
      reinterpret_cast<uint32_t *>(dst)[j] = reinterpret_cast<const uint32_t *>(src)[j];
    }
  } else {
#pragma unroll 4
    for (uint32_t j = first; j < cols; j += kPerRow) dst[j] = src[j];
  }
}

// Byte offset of row `row`'s first K block inside an MXFP4 matrix [n, k/2] and inside its scales
// [n, k/32].  Checkpoint order: rows follow each other.  Block-major order (16-row tiles of
// [K block][row][64 B] and [K block][row][4 B]): the row's cell of K block 0 of its tile; the next
// K block lies 1024 (payload) or 64 (scales) bytes further.
__device__ __forceinline__ size_t weight_row_offset(uint32_t row, uint32_t k, uint32_t block_major) {
  return block_major ? static_cast<size_t>(row >> 4) * (static_cast<size_t>(k) * 8u) + (row & 15u) * 64u
                     : static_cast<size_t>(row) * (k >> 1);
}
__device__ __forceinline__ size_t scale_row_offset(uint32_t row, uint32_t k, uint32_t block_major) {
  return block_major ? static_cast<size_t>(row >> 4) * (k >> 1) + (row & 15u) * 4u : static_cast<size_t>(row) * (k >> 5);
}

template <typename S>
__global__ __launch_bounds__(S::kThreads) void grouped_gate_up_kernel(GroupedParams p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const GroupedItem item = grouped_item(p, (p.intermediate_size + S::FN - 1u) / S::FN);
  if (!item.live) return;
  const uint32_t ftile = item.ftile, row0 = item.row0, m = item.m;
  const uint32_t f0 = ftile * S::FN;
  const uint32_t cols = p.input_size >> 7;

  uint8_t *stages = lds;
  uint8_t *xsc = lds + S::NSTAGE * S::kStageBytes;
  auto token_of = [&](uint32_t r) {
    const int32_t token = p.route_token_indices[row0 + min(r, m - 1u)];
    return (token >= 0 && static_cast<uint32_t>(token) < p.num_tokens) ? static_cast<uint32_t>(token) : 0u;
  };
  GemmOperands<2> op;
  op.x = p.input_fp8;
  op.w[0] = entry_ptr(item.entry->gate_w);
  op.w[1] = entry_ptr(item.entry->up_w);
  op.wscale[0] = entry_ptr(item.entry->gate_s);
  op.wscale[1] = entry_ptr(item.entry->up_s);
  op.k = p.input_size;
  GemmCursors<S> cur;
  gemm_init_cursors<S>(
      cur, op, wave, lane, [&](uint32_t r) { return token_of(r) * p.input_size; },  // < 4 GiB: checked at launch
      [&](uint32_t, uint32_t r) { return weight_row_offset(min(f0 + r, p.intermediate_size - 1u), p.input_size, p.block_major); },
      [&](uint32_t, uint32_t r) { return scale_row_offset(min(f0 + r, p.intermediate_size - 1u), p.input_size, p.block_major); });
  if (p.block_major) {
    cur.w_step = 1024u;
    cur.s_step = 64u;
  }
  // first stages in flight, then the token scales under their latency
  gemm_prologue<S>(cur, stages, p.input_size >> 7, wave);
  stage_row_scales<S>(xsc, cols, [&](uint32_t r) { return p.input_ue8m0 + static_cast<size_t>(token_of(r)) * cols; });
  __syncthreads();

  f32x4_t acc[2][S::NF][S::NT];
#pragma unroll
  for (int mat = 0; mat < 2; ++mat) {
#pragma unroll
    for (int f = 0; f < S::NF; ++f) {
#pragma unroll
      for (int t = 0; t < S::NT; ++t) acc[mat][f][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
  }
  const uint32_t i = lane & 15u;
  const uint32_t wt = wave / S::WAVES_F;
  const uint32_t pitch = scale_row_pitch(cols);
  // route weights of this lane's token rows, fetched before the K loop instead of behind it
  float row_weight[S::NT];
#pragma unroll
  for (int t = 0; t < S::NT; ++t) {
    const uint32_t r = S::token_row(wt, t) + i;
    row_weight[t] = r < m ? p.route_weights[row0 + r] : 0.0f;
  }
  gemm_mainloop_ragged<S, WScaleMode::PerRow32, true>(
      acc, cur, stages, p.input_size >> 7, wave, lane, S::live_fragments(wt, m),
      [&](int t, uint32_t kb) { return static_cast<uint32_t>(xsc[(S::token_row(wt, t) + i) * pitch + kb]); },
      [&](int, uint32_t) { return 0u; });

  // Epilogue: this wave holds features [fbase, fbase+128) of S::NT token tiles
  swiglu_quantize_store<S>(
      acc, lane, wave, f0, p.intermediate_size, p.swiglu_limit, p.hq, p.hs, p.hidden_f32, p.route_error,
      [&](int t, uint32_t r, bool &live, size_t &row, float &weight) {
        live = r < m;
        row = row0 + r;
        weight = row_weight[t];
      });
}

// LDS of the persistent form: the stages, the token scales, the token indices of the next item.
template <typename S>
__host__ __device__ constexpr uint32_t grouped_chained_lds_bytes(uint32_t cols) {
  return grouped_lds_bytes<S>(cols) + S::TM * 4u;
}

// The same GEMM with persistent workgroups (8 * kXcdRun of them) whose K loops form one chain
// (GemmChain): while an item is multiplied, the next one is looked up, its token indices are
// fetched into LDS, its cursors are set up, and the item's last K steps fetch the next item's
// first stages.  One workgroup per item spends about 10 us of a 100 us item between the last
// MFMA of one item and the first of the next (result stores, dispatch, three dependent look-ups,
// the first stages' latency); here the token scales of the next item and the epilogue are all
// that is left there.  Needs input_size / 128 >= 6 K steps.
template <typename S>
__global__ __launch_bounds__(S::kThreads) void grouped_gate_up_chained_kernel(GroupedParams p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const uint32_t lane0 = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t feature_tiles = (p.intermediate_size + S::FN - 1u) / S::FN;
  const uint32_t cols = p.input_size >> 7;
  const uint32_t pitch = scale_row_pitch(cols);
  uint8_t *stages = lds;
  uint8_t *xsc = lds + S::NSTAGE * S::kStageBytes;
  int32_t *next_tokens = reinterpret_cast<int32_t *>(lds + grouped_lds_bytes<S>(cols));  // [TM]
  const uint32_t wt = wave / S::WAVES_F;

  struct View {
    uint32_t row0, m, f0;
    GemmOperands<2> op;
  };
  auto view_of = [&](const GroupedItem &item) {
    View v;
    v.row0 = item.row0;
    v.m = item.m;
    v.f0 = item.ftile * S::FN;
    v.op.x = p.input_fp8;
    v.op.w[0] = entry_ptr(item.entry->gate_w);
    v.op.w[1] = entry_ptr(item.entry->up_w);
    v.op.wscale[0] = entry_ptr(item.entry->gate_s);
    v.op.wscale[1] = entry_ptr(item.entry->up_s);
    v.op.k = p.input_size;
    return v;
  };
  auto checked = [&](int32_t token) {
    return (token >= 0 && static_cast<uint32_t>(token) < p.num_tokens) ? static_cast<uint32_t>(token) : 0u;
  };
  // token(r) -> token of the view's row r (clamped to its rows)
  auto set_cursors = [&](GemmCursors<S> &c, const View &v, uint32_t lane, auto token) {
    gemm_init_cursors<S>(
        c, v.op, wave, lane, [&](uint32_t r) { return token(r) * p.input_size; },  // < 4 GiB: checked at launch
        [&](uint32_t, uint32_t r) { return weight_row_offset(min(v.f0 + r, p.intermediate_size - 1u), p.input_size, p.block_major); },
        [&](uint32_t, uint32_t r) { return scale_row_offset(min(v.f0 + r, p.intermediate_size - 1u), p.input_size, p.block_major); });
    if (p.block_major) {
      c.w_step = 1024u;
      c.s_step = 64u;
    }
  };

  GroupedItem item = grouped_item_of_round(p, feature_tiles, 0u);
  if (!item.live) return;
  View cur_v = view_of(item);
  GemmCursors<S> cur, nxt;
  {
    auto token = [&](uint32_t r) { return checked(p.route_token_indices[cur_v.row0 + min(r, cur_v.m - 1u)]); };
    set_cursors(cur, cur_v, lane0, token);
    gemm_prologue<S>(cur, stages, cols, wave);
    stage_row_scales<S>(xsc, cols, [&](uint32_t r) { return p.input_ue8m0 + static_cast<size_t>(token(r)) * cols; });
  }
  // The direct-to-LDS loads are inline assembly, which the compiler's wait counts do not cover:
  // the barrier alone would not wait for them.  The chained loop skips its waits in the first
  // NSTAGE-1 steps, so this wave's share of the first stages is waited for here, once.
  wait_vmcnt(0);
  __syncthreads();
  GemmChain<S> chain;
  chain.buf = 0;
  chain.fill = S::NSTAGE - 1;
  chain.next = &nxt;

  // Items are looked up (chains of scalar loads) a whole item before they are needed.
  GroupedItem next_item = grouped_item_of_round(p, feature_tiles, 1u);
  View nxt_v = next_item.live ? view_of(next_item) : cur_v;
  for (uint32_t round = 0;; ++round) {
    const GroupedItem after_item = grouped_item_of_round(p, feature_tiles, round + 2u);
    const View after_v = after_item.live ? view_of(after_item) : nxt_v;
    if (next_item.live) {
      // token indices of the next item's rows -> LDS; the first K step that waits finds them landed
      if (wave * 64u < S::TM) {
        lds_dma4(p.route_token_indices + nxt_v.row0, min(wave * 64u + lane0, nxt_v.m - 1u) * 4u, next_tokens + wave * 64u);
      }
    } else {
      // nothing follows: the last steps fetch this item's first K blocks once more
      nxt = cur;
      gemm_rewind<S>(nxt);
    }
    f32x4_t acc[2][S::NF][S::NT];
#pragma unroll
    for (int mat = 0; mat < 2; ++mat) {
#pragma unroll
      for (int f = 0; f < S::NF; ++f) {
#pragma unroll
        for (int t = 0; t < S::NT; ++t) acc[mat][f][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      }
    }
    // The lane index is taken afresh for every item: what the K loop derives from it (fragment
    // addresses and the like) would otherwise be kept in registers through the epilogue of every
    // item, which has none to spare.
    uint32_t lane = lane0;
    asm volatile("" : "+v"(lane));
    const uint32_t i = lane & 15u;
    // route weights of this lane's token rows, fetched before the K loop instead of behind it
    float row_weight[S::NT];
#pragma unroll
    for (int t = 0; t < S::NT; ++t) {
      const uint32_t r = S::token_row(wt, t) + i;
      row_weight[t] = r < cur_v.m ? p.route_weights[cur_v.row0 + r] : 0.0f;
    }
    auto next_token = [&](uint32_t r) { return checked(next_tokens[min(r, nxt_v.m - 1u)]); };
    gemm_mainloop_ragged<S, WScaleMode::PerRow32, true, true>(
        acc, cur, stages, cols, wave, lane, S::live_fragments(wt, cur_v.m),
        [&](int t, uint32_t kb) { return static_cast<uint32_t>(xsc[(S::token_row(wt, t) + i) * pitch + kb]); },
        [&](int, uint32_t) { return 0u; }, &chain,
        [&](uint32_t step) {
          if (step == static_cast<uint32_t>(S::NSTAGE - 1) && next_item.live) set_cursors(nxt, nxt_v, lane, next_token);
        });
    lds_barrier();  // every wave has read its last token scale
    if (next_item.live) {
      stage_row_scales<S>(xsc, cols, [&](uint32_t r) { return p.input_ue8m0 + static_cast<size_t>(next_token(r)) * cols; });
    }
    swiglu_quantize_store<S>(
        acc, lane, wave, cur_v.f0, p.intermediate_size, p.swiglu_limit, p.hq, p.hs, p.hidden_f32, p.route_error,
        [&](int t, uint32_t r, bool &live, size_t &row, float &weight) {
          live = r < cur_v.m;
          row = cur_v.row0 + r;
          weight = row_weight[t];
        });
    if (!next_item.live) break;
    cur = nxt;
    cur_v = nxt_v;
    next_item = after_item;
    nxt_v = after_v;
    lds_barrier();  // the scales are in place; next_tokens may be overwritten
  }
}

template <typename S>
__global__ __launch_bounds__(S::kThreads) void grouped_down_kernel(GroupedParams p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const GroupedItem item = grouped_item(p, (p.hidden_size + S::FN - 1u) / S::FN);
  if (!item.live) return;
  const uint32_t ftile = item.ftile, row0 = item.row0, m = item.m;
  const uint32_t f0 = ftile * S::FN;
  const uint32_t cols = p.intermediate_size >> 7;

  uint8_t *stages = lds;
  uint8_t *xsc = lds + S::NSTAGE * S::kStageBytes;
  GemmOperands<1> op;
  op.x = p.hq + static_cast<size_t>(row0) * p.intermediate_size;  // the tile's first row: 32-bit lane offsets
  op.w[0] = entry_ptr(item.entry->down_w);
  op.wscale[0] = entry_ptr(item.entry->down_s);
  op.k = p.intermediate_size;
  GemmCursors<S> cur;
  gemm_init_cursors<S>(
      cur, op, wave, lane,
      [&](uint32_t r) { return min(r, m - 1u) * p.intermediate_size; },
      [&](uint32_t, uint32_t r) { return weight_row_offset(min(f0 + r, p.hidden_size - 1u), p.intermediate_size, p.block_major); },
      [&](uint32_t, uint32_t r) { return scale_row_offset(min(f0 + r, p.hidden_size - 1u), p.intermediate_size, p.block_major); });
  if (p.block_major) {
    cur.w_step = 1024u;
    cur.s_step = 64u;
  }
  gemm_prologue<S>(cur, stages, p.intermediate_size >> 7, wave);
  stage_row_scales<S>(xsc, cols, [&](uint32_t r) { return p.hs + static_cast<size_t>(row0 + min(r, m - 1u)) * cols; });
  __syncthreads();

  f32x4_t acc[1][S::NF][S::NT];
#pragma unroll
  for (int f = 0; f < S::NF; ++f) {
#pragma unroll
    for (int t = 0; t < S::NT; ++t) acc[0][f][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
  const uint32_t i = lane & 15u, g = lane >> 4;
  const uint32_t wf = wave % S::WAVES_F, wt = wave / S::WAVES_F;
  const uint32_t pitch = scale_row_pitch(cols);
  // destination routes of this lane's token rows, fetched before the K loop instead of behind it
  int32_t row_route[S::NT];
#pragma unroll
  for (int t = 0; t < S::NT; ++t) {
    const uint32_t r = S::token_row(wt, t) + i;
    row_route[t] = r < m ? p.route_indices[row0 + r] : -1;
  }
  gemm_mainloop_ragged<S, WScaleMode::PerRow32, true>(
      acc, cur, stages, p.intermediate_size >> 7, wave, lane, S::live_fragments(wt, m),
      [&](int t, uint32_t kb) { return static_cast<uint32_t>(xsc[(S::token_row(wt, t) + i) * pitch + kb]); },
      [&](int, uint32_t) { return 0u; });

#pragma unroll
  for (int t = 0; t < S::NT; ++t) {
    const int32_t route = row_route[t];  // -1 beyond the tile's rows
    if (route < 0 || static_cast<uint32_t>(route) >= p.num_routes) continue;
    float *out = p.route_output + static_cast<size_t>(route) * p.hidden_size;
#pragma unroll
    for (int f = 0; f < S::NF; ++f) {
      const uint32_t feat = f0 + (wf * S::NF + f) * 16u + g * 4u;
      if (feat < p.hidden_size) {  // hidden_size is a multiple of 16: whole quads
        const f32x4_t a = acc[0][f][t];
        *reinterpret_cast<float4 *>(out + feat) = make_float4(a[0], a[1], a[2], a[3]);
      }
    }
    if (ftile == 0u && wf == 0u && g == 0u) p.route_written[route] = 1;
  }
}

// LDS of the persistent down GEMM: the stages and TWO tables of token scales (they are small here:
// intermediate_size / 128 bytes per row), the next item's filled while the current one is read.
template <typename S>
__host__ __device__ constexpr uint32_t grouped_down_chained_lds_bytes(uint32_t cols) {
  return S::NSTAGE * S::kStageBytes + 2u * ((S::TM * scale_row_pitch(cols) + 15u) & ~15u);
}

// The down GEMM with persistent workgroups and chained K loops (see grouped_gate_up_chained_kernel).
// Rows and scale rows of an item are consecutive, so nothing has to be looked up through LDS: the
// next item's cursors are set before the K loop and its scale rows are fetched by direct-to-LDS
// loads behind the first barrier of the loop; between two items there is only the result store.
// Needs intermediate_size / 128 >= 6 K steps and intermediate_size % 512 == 0 (whole
// dwords of scale bytes per row).
template <typename S>
__global__ __launch_bounds__(S::kThreads) void grouped_down_chained_kernel(GroupedParams p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t feature_tiles = (p.hidden_size + S::FN - 1u) / S::FN;
  const uint32_t cols = p.intermediate_size >> 7;
  const uint32_t pitch = scale_row_pitch(cols);
  const uint32_t table_bytes = (S::TM * pitch + 15u) & ~15u;
  uint8_t *stages = lds;
  uint8_t *tables = lds + S::NSTAGE * S::kStageBytes;
  const uint32_t i = lane & 15u, g = lane >> 4;
  const uint32_t wf = wave % S::WAVES_F, wt = wave / S::WAVES_F;

  struct View {
    uint32_t row0, m, f0, ftile;
    const uint8_t *w, *s;
  };
  auto view_of = [&](const GroupedItem &item) {
    View v;
    v.row0 = item.row0;
    v.m = item.m;
    v.ftile = item.ftile;
    v.f0 = item.ftile * S::FN;
    v.w = entry_ptr(item.entry->down_w);
    v.s = entry_ptr(item.entry->down_s);
    return v;
  };
  auto set_cursors = [&](GemmCursors<S> &c, const View &v) {
    GemmOperands<1> op;
    op.x = p.hq + static_cast<size_t>(v.row0) * p.intermediate_size;  // the tile's first row: 32-bit lane offsets
    op.w[0] = v.w;
    op.wscale[0] = v.s;
    op.k = p.intermediate_size;
    gemm_init_cursors<S>(
        c, op, wave, lane, [&](uint32_t r) { return min(r, v.m - 1u) * p.intermediate_size; },
        [&](uint32_t, uint32_t r) { return weight_row_offset(min(v.f0 + r, p.hidden_size - 1u), p.intermediate_size, p.block_major); },
        [&](uint32_t, uint32_t r) { return scale_row_offset(min(v.f0 + r, p.hidden_size - 1u), p.intermediate_size, p.block_major); });
    if (p.block_major) {
      c.w_step = 1024u;
      c.s_step = 64u;
    }
  };
  // Scale rows of the view's token rows -> table, one dword per lane: lane q of the table's dwords is
  // (row q / (pitch / 4), dword q % (pitch / 4)); dwords beyond a row's cols (the padding of the
  // pitch) and rows beyond the view's fetch something valid that nobody reads.
  auto fetch_scales = [&](uint8_t *table, const View &v) {
    const uint32_t dwords_per_row = pitch >> 2, data_dwords = cols >> 2;
    const uint32_t total = S::TM * dwords_per_row;
    for (uint32_t first = wave * 64u; first < total; first += S::kWaves * 64u) {
      const uint32_t q = min(first + lane, total - 1u);
      const uint32_t row = min(q / dwords_per_row, v.m - 1u), dword = min(q % dwords_per_row, data_dwords - 1u);
      lds_dma4(p.hs + static_cast<size_t>(v.row0) * cols, row * cols + dword * 4u, table + first * 4u);
    }
  };

  GroupedItem item = grouped_item_of_round(p, feature_tiles, 0u);
  if (!item.live) return;
  View cur_v = view_of(item);
  GemmCursors<S> cur, nxt;
  set_cursors(cur, cur_v);
  gemm_prologue<S>(cur, stages, cols, wave);
  fetch_scales(tables, cur_v);
  // The direct-to-LDS loads (stages and scale table) are inline assembly, which the compiler's
  // wait counts do not cover: each wave waits for its own here, the barrier then publishes all of
  // them.  The chained loop skips its waits in the first NSTAGE-1 steps and reads the scale table
  // before its first barrier.
  wait_vmcnt(0);
  __syncthreads();
  GemmChain<S> chain;
  chain.buf = 0;
  chain.fill = S::NSTAGE - 1;
  chain.next = &nxt;

  // Items are looked up (chains of scalar loads) a whole item before they are needed.
  GroupedItem next_item = grouped_item_of_round(p, feature_tiles, 1u);
  View nxt_v = next_item.live ? view_of(next_item) : cur_v;
  for (uint32_t round = 0;; ++round) {
    const uint8_t *xsc = tables + (round & 1u) * table_bytes;
    uint8_t *next_xsc = tables + ((round + 1u) & 1u) * table_bytes;
    const GroupedItem after_item = grouped_item_of_round(p, feature_tiles, round + 2u);
    const View after_v = after_item.live ? view_of(after_item) : nxt_v;
    if (next_item.live) {
      set_cursors(nxt, nxt_v);
    } else {
      // nothing follows: the last steps fetch this item's first K blocks once more
      nxt = cur;
      gemm_rewind<S>(nxt);
    }
    f32x4_t acc[1][S::NF][S::NT];
#pragma unroll
    for (int f = 0; f < S::NF; ++f) {
#pragma unroll
      for (int t = 0; t < S::NT; ++t) acc[0][f][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
    // destination routes of this lane's token rows, fetched before the K loop instead of behind it
    int32_t row_route[S::NT];
#pragma unroll
    for (int t = 0; t < S::NT; ++t) {
      const uint32_t r = S::token_row(wt, t) + i;
      row_route[t] = r < cur_v.m ? p.route_indices[cur_v.row0 + r] : -1;
    }
    gemm_mainloop_ragged<S, WScaleMode::PerRow32, true, true>(
        acc, cur, stages, cols, wave, lane, S::live_fragments(wt, cur_v.m),
        [&](int t, uint32_t kb) { return static_cast<uint32_t>(xsc[(S::token_row(wt, t) + i) * pitch + kb]); },
        [&](int, uint32_t) { return 0u; }, &chain,
        [&](uint32_t step) {
          // behind the first barrier every wave has left the previous item, whose table this is
          if (step == 0u && next_item.live) fetch_scales(next_xsc, nxt_v);
        });
#pragma unroll
    for (int t = 0; t < S::NT; ++t) {
      const int32_t route = row_route[t];  // -1 beyond the tile's rows
      if (route < 0 || static_cast<uint32_t>(route) >= p.num_routes) continue;
      float *out = p.route_output + static_cast<size_t>(route) * p.hidden_size;
#pragma unroll
      for (int f = 0; f < S::NF; ++f) {
        const uint32_t feat = cur_v.f0 + (wf * S::NF + f) * 16u + g * 4u;
        if (feat < p.hidden_size) {  // hidden_size is a multiple of 16: whole quads
          const f32x4_t a = acc[0][f][t];
          *reinterpret_cast<float4 *>(out + feat) = make_float4(a[0], a[1], a[2], a[3]);
        }
      }
      if (cur_v.ftile == 0u && wf == 0u && g == 0u) p.route_written[route] = 1;
    }
    if (!next_item.live) break;
    cur = nxt;
    cur_v = nxt_v;
    next_item = after_item;
    nxt_v = after_v;
  }
}

__global__ __launch_bounds__(256) void copy_bytes_kernel(const uint8_t *src, uint8_t *dst, uint64_t bytes) {
  const uint64_t idx = (static_cast<uint64_t>(blockIdx.x) * 256u + threadIdx.x) * 16u;
  if (idx + 16u <= bytes) {
    *reinterpret_cast<uint4 *>(dst + idx) = *reinterpret_cast<const uint4 *>(src + idx);
  } else {
    for (uint64_t j = idx; j < bytes; ++j) dst[j] = src[j];
  }
}

constexpr uint32_t kMaxLds = 160u * 1024u;

bool aligned(uint64_t address, uint64_t to) { return address != 0 && (address % to) == 0; }

// sm103/grouped_fp4_moe.cuh:206-229 (scalars), :231-260 (pointers)
int32_t validate_scalars(const FerruleHipGroupedFp4MoeArgs &a) {
  const bool ok = a.active_group_count != 0 && a.active_group_count <= 0x3fffffffu &&
                  a.small_group_count <= a.active_group_count && a.slot_capacity != 0 && a.max_group_rows != 0 &&
                  a.total_routed_rows != 0 && a.total_routed_rows <= a.num_routes &&
                  a.total_routed_rows >= a.active_group_count &&
                  static_cast<uint64_t>(a.total_routed_rows) <=
                      static_cast<uint64_t>(a.active_group_count) * a.max_group_rows &&
                  a.num_tokens != 0 && a.num_routes != 0 && a.input_size != 0 && a.intermediate_size != 0 &&
                  a.hidden_size != 0 && (a.input_size % 128u) == 0 && (a.intermediate_size % 128u) == 0 &&
                  (a.hidden_size % 64u) == 0 && a.swiglu_limit == a.swiglu_limit &&
                  fabsf(a.swiglu_limit) <= 3.4028234e38f;
  if (!ok) return FERRULE_HIP_INVALID_ARGUMENT;
  if (grouped_lds_bytes<GateUpShape<2>>(a.input_size >> 7) > kMaxLds ||
      grouped_lds_bytes<DownShape<2>>(a.intermediate_size >> 7) > kMaxLds) {
    return FERRULE_HIP_UNSUPPORTED;
  }
  return FERRULE_HIP_SUCCESS;
}

template <typename S, typename Kernel>
hipError_t launch_grouped(Kernel kernel, const GroupedParams &p, uint32_t feature_tiles, uint32_t cols,
                          hipStream_t stream) {
  const uint32_t lds = grouped_lds_bytes<S>(cols);
  hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
  if (err != hipSuccess) return err;
  kernel<<<p.max_tiles * feature_tiles, S::kThreads, lds, stream>>>(p);
  return hipSuccess;
}

int32_t launch(const FerruleHipGroupedFp4MoeArgs *args, uint64_t hidden_f32, bool block_major) {
  const int32_t status = ferrule_hip_grouped_fp4_moe_can_implement(args);
  if (status != FERRULE_HIP_SUCCESS) return status;
  const FerruleHipGroupedFp4MoeArgs &a = *args;
  const WorkspaceLayout l = workspace_layout(a.active_group_count, a.total_routed_rows, a.intermediate_size);
  GroupedParams p;
  auto ptr = [](uint64_t v) { return reinterpret_cast<void *>(static_cast<uintptr_t>(v)); };
  p.active_expert_slots = static_cast<const int32_t *>(ptr(a.active_expert_slots));
  p.expert_route_indptr = static_cast<const uint32_t *>(ptr(a.expert_route_indptr));
  p.route_token_indices = static_cast<const int32_t *>(ptr(a.route_token_indices));
  p.route_indices = static_cast<const int32_t *>(ptr(a.route_indices));
  p.route_weights = static_cast<const float *>(ptr(a.route_weights));
  p.gate_ptrs = static_cast<const uint64_t *>(ptr(a.gate_ptrs));
  p.gate_scale_ptrs = static_cast<const uint64_t *>(ptr(a.gate_scale_ptrs));
  p.up_ptrs = static_cast<const uint64_t *>(ptr(a.up_ptrs));
  p.up_scale_ptrs = static_cast<const uint64_t *>(ptr(a.up_scale_ptrs));
  p.down_ptrs = static_cast<const uint64_t *>(ptr(a.down_ptrs));
  p.down_scale_ptrs = static_cast<const uint64_t *>(ptr(a.down_scale_ptrs));
  p.input_fp8 = static_cast<const uint8_t *>(ptr(a.input_fp8));
  p.input_ue8m0 = static_cast<const uint8_t *>(ptr(a.input_ue8m0));
  p.route_output = static_cast<float *>(ptr(a.route_output));
  p.route_written = static_cast<int32_t *>(ptr(a.route_written));
  p.route_error = static_cast<int32_t *>(ptr(a.route_error));
  uint8_t *ws = static_cast<uint8_t *>(ptr(a.workspace));
  p.tile_map = reinterpret_cast<int32_t *>(ws + l.tile_map);
  p.hq = ws + l.hq;
  p.hs = ws + l.hs;
  p.hidden_f32 = static_cast<float *>(ptr(hidden_f32));
  p.groups = a.active_group_count;
  p.slot_capacity = a.slot_capacity;
  p.rows = a.total_routed_rows;
  p.num_tokens = a.num_tokens;
  p.num_routes = a.num_routes;
  p.input_size = a.input_size;
  p.intermediate_size = a.intermediate_size;
  p.hidden_size = a.hidden_size;
  p.max_tiles = l.max_tiles;
  p.swiglu_limit = a.swiglu_limit;
  p.block_major = block_major ? 1u : 0u;

  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(a.stream));
  clear_launch_error();
  tile_map_kernel<<<1, 256, 0, stream>>>(p);
  const uint32_t in_cols = a.input_size >> 7, mid_cols = a.intermediate_size >> 7;
  hipError_t err;
  const uint32_t gate_tiles = (a.intermediate_size + GateUpShape<3>::FN - 1) / GateUpShape<3>::FN;
  if (grouped_chained_lds_bytes<GateUpShape<3>>(in_cols) <= kMaxLds && in_cols >= 6u) {
    auto kernel = grouped_gate_up_chained_kernel<GateUpShape<3>>;
    const uint32_t lds = grouped_chained_lds_bytes<GateUpShape<3>>(in_cols);
    err = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                              static_cast<int>(lds));
    if (err == hipSuccess) kernel<<<8u * kXcdRun, GateUpShape<3>::kThreads, lds, stream>>>(p);
  } else if (grouped_lds_bytes<GateUpShape<3>>(in_cols) <= kMaxLds) {
    err = launch_grouped<GateUpShape<3>>(grouped_gate_up_kernel<GateUpShape<3>>, p, gate_tiles, in_cols, stream);
  } else {
    err = launch_grouped<GateUpShape<2>>(grouped_gate_up_kernel<GateUpShape<2>>, p, gate_tiles, in_cols, stream);
  }
  if (err == hipSuccess) {
    const uint32_t down_tiles = (a.hidden_size + DownShape<3>::FN - 1) / DownShape<3>::FN;
    if (grouped_down_chained_lds_bytes<DownShape<3>>(mid_cols) <= kMaxLds && mid_cols >= 6u && mid_cols % 4u == 0u) {
      auto kernel = grouped_down_chained_kernel<DownShape<3>>;
      const uint32_t lds = grouped_down_chained_lds_bytes<DownShape<3>>(mid_cols);
      err = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(lds));
      if (err == hipSuccess) kernel<<<8u * kXcdRun, DownShape<3>::kThreads, lds, stream>>>(p);
    } else if (grouped_lds_bytes<DownShape<3>>(mid_cols) <= kMaxLds) {
      err = launch_grouped<DownShape<3>>(grouped_down_kernel<DownShape<3>>, p, down_tiles, mid_cols, stream);
    } else {
      err = launch_grouped<DownShape<2>>(grouped_down_kernel<DownShape<2>>, p, down_tiles, mid_cols, stream);
    }
  }
  if (err != hipSuccess) {
    g_last_hip_error = static_cast<int32_t>(err);
    return FERRULE_HIP_LAUNCH_FAILED;
  }
  return take_launch_error() == 0 ? FERRULE_HIP_SUCCESS : FERRULE_HIP_LAUNCH_FAILED;
}

}  // namespace
}  // namespace ferrule_hip

using namespace ferrule_hip;

extern "C" uint64_t ferrule_hip_grouped_fp4_moe_workspace_size(const FerruleHipGroupedFp4MoeArgs *args) {
  if (args == nullptr || validate_scalars(*args) != FERRULE_HIP_SUCCESS) return 0;
  return workspace_layout(args->active_group_count, args->total_routed_rows, args->intermediate_size).total;
}

extern "C" int32_t ferrule_hip_grouped_fp4_moe_can_implement(const FerruleHipGroupedFp4MoeArgs *args) {
  if (args == nullptr) return FERRULE_HIP_INVALID_ARGUMENT;
  const int32_t scalars = validate_scalars(*args);
  if (scalars != FERRULE_HIP_SUCCESS) return scalars;
  const FerruleHipGroupedFp4MoeArgs &a = *args;
  const bool pointers = aligned(a.active_expert_slots, 4) && aligned(a.expert_route_indptr, 4) &&
                        aligned(a.route_token_indices, 4) && aligned(a.route_indices, 4) &&
                        aligned(a.route_weights, 4) && aligned(a.gate_ptrs, 8) && aligned(a.gate_scale_ptrs, 8) &&
                        aligned(a.up_ptrs, 8) && aligned(a.up_scale_ptrs, 8) && aligned(a.down_ptrs, 8) &&
                        aligned(a.down_scale_ptrs, 8) && aligned(a.input_fp8, 16) && aligned(a.input_ue8m0, 1) &&
                        aligned(a.route_output, 16) && aligned(a.route_written, 4) && aligned(a.route_error, 4) &&
                        aligned(a.workspace, 256);
  if (!pointers) return FERRULE_HIP_INVALID_ARGUMENT;
  // the stage loads address a token row of the input and a weight row of one expert with 32-bit
  // offsets from the operand's base
  const uint64_t kOffsetLimit = 1ull << 32;
  if (static_cast<uint64_t>(a.num_tokens) * a.input_size >= kOffsetLimit ||
      static_cast<uint64_t>(a.intermediate_size) * (a.input_size / 2u) >= kOffsetLimit ||
      static_cast<uint64_t>(a.hidden_size) * (a.intermediate_size / 2u) >= kOffsetLimit)
    return FERRULE_HIP_UNSUPPORTED;
  const uint64_t need = workspace_layout(a.active_group_count, a.total_routed_rows, a.intermediate_size).total;
  if (a.workspace_bytes < need) return FERRULE_HIP_INVALID_ARGUMENT;
  return FERRULE_HIP_SUCCESS;
}

extern "C" int32_t ferrule_hip_grouped_fp4_moe_launch(const FerruleHipGroupedFp4MoeArgs *args) {
  return launch(args, 0, false);
}

extern "C" int32_t ferrule_hip_grouped_fp4_moe_block_major_launch(const FerruleHipGroupedFp4MoeArgs *args) {
  // whole 16-row tiles and 128-wide K blocks: intermediate_size % 128 == 0 and input_size % 128 == 0 are
  // validated for every launch, hidden_size % 64 == 0 too
  return launch(args, 0, true);
}

extern "C" int32_t ferrule_hip_grouped_fp4_moe_debug_launch(const FerruleHipGroupedFp4MoeArgs *args,
                                                            uint64_t hidden_f32) {
  if (hidden_f32 == 0 || (hidden_f32 & 15u) != 0) return FERRULE_HIP_INVALID_ARGUMENT;
  return launch(args, hidden_f32, false);
}

extern "C" uint64_t ferrule_hip_mxfp4_sfb_storage_bytes(uint32_t n, uint32_t k) {
  if (n == 0 || k == 0 || n > 0x7fffffffu || k > 0x7fffffffu || (k % 32u) != 0) return 0;
  return static_cast<uint64_t>(n) * (k / 32u);
}

extern "C" int32_t ferrule_hip_prepare_mxfp4_sfb(const FerruleHipPrepareMxfp4SfbArgs *args) {
  if (args == nullptr || args->reserved0 != 0u) return FERRULE_HIP_INVALID_ARGUMENT;
  const uint64_t bytes = ferrule_hip_mxfp4_sfb_storage_bytes(args->n, args->k);
  if (bytes == 0 || args->linear_source == 0 || args->prepared_destination == 0 ||
      ((args->linear_source | args->prepared_destination) & 15u) != 0) {
    return FERRULE_HIP_INVALID_ARGUMENT;
  }
  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(args->stream));
  clear_launch_error();
  const uint64_t threads = (bytes + 15u) / 16u;
  copy_bytes_kernel<<<static_cast<uint32_t>((threads + 255u) / 256u), 256, 0, stream>>>(
      reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(args->linear_source)),
      reinterpret_cast<uint8_t *>(static_cast<uintptr_t>(args->prepared_destination)), bytes);
  return take_launch_error() == 0 ? FERRULE_HIP_SUCCESS : FERRULE_HIP_LAUNCH_FAILED;
}
