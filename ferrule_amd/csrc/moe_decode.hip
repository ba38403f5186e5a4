// Decode MoE layer over MXFP4 experts with BF16 activations (no activation quantisation).
//
// Semantics, per route (token t, rank j, expert e, router weight w):
//   gate = W1_e x_t, up = W3_e x_t          fp32 accumulation
//   clamp when swiglu_limit > 0:  gate = min(gate, L), up = clamp(up, -L, L)
//   h    = silu(gate) * up * w              (left to right, fp32)
//   y    = W2_e h                           fp32 accumulation
// which is CpuReferenceExpertExecutor::execute with its default construction
// (crates/ferrule-model/src/moe/executor.rs:82-124); then per token the routes are summed
// in rank order (crates/ferrule-model/src/moe/routed.rs:85-110) on top of an optional f32
// prefix, and rounded once to BF16 (crates/ferrule-model/src/models/common/math.rs:7-14).
//
// The MXFP4 weights go to the scaled MFMA (v_mfma_scale_f32_16x16x128_f8f6f4) as they lie in
// memory, nibbles and E8M0 scales; its other operand must be FP8, so x and h are first split
// into a short sum of MX-FP8 terms by truncation (mx_split_kernel, mx_core.cuh: 2 terms for the
// BF16 input, 4 for the f32 hidden values, cutting less than 2^-20 resp. 2^-15 of an element's
// 32-block maximum) and every term is multiplied separately.  Launches of one layer:
//   mx_split (x) -> gate_up -> mx_split (h) -> down -> combine
//   gate_up : grid (I/128, groups); a workgroup = 4 consumer waves + 1 producer wave.  A
//             consumer owns 16-row tiles of W1 and the same tiles of W3, walks ALL of K for
//             each (no cross-wave reduction) and applies SwiGLU * weight from the accumulators;
//             the producer moves the expert's token rows global->LDS (mx_rowstream).
//   down    : grid (H/512, groups); the same scheme, a consumer's two matrices being two row
//             tiles of W2.
//   combine : rank-ordered fp32 fold + single BF16 writeback.
// gate_up and down each exist in a packed and a general form (BColumn); which of them are
// launched depends on how dense the routes are (token_tile_rows).
// Data movement: every weight byte is read once with 16-byte loads (nontemporal on block-major
// weights), a ring of DEPTH K blocks ahead per wave that runs on across row tiles.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <atomic>
#include <mutex>
#include <type_traits>

#include "../../include/ferrule_hip_diagnostics.h"
#include "../../include/ferrule_hip_provider.h"
#include "numeric.cuh"
#include "skinny_core.cuh"
#include "mx_core.cuh"

namespace ferrule_hip {
namespace {

constexpr uint32_t kTokenTile = 16;
constexpr uint32_t kWaves = 4;
// MX-FP8 terms per activation (4 significant bits each, see mx_core.cuh):
//   input  (BF16, 8 significant bits): 2 terms are exact for every element within 2^-13 of
//          its 32-block maximum; smaller elements keep an absolute error below 2^-20 of that
//          maximum, which is below the fp32 resolution of the dot product they enter;
//   hidden (f32): 4 terms = 16 significant bits of the block maximum (every element is cut by
//          less than 2^-15 of its 32-block maximum).
constexpr int kTermsX = 2;
constexpr int kTermsH = 4;

struct MoeParams {
  const int32_t *active_expert_slots;
  const int32_t *expert_route_indptr;
  const int32_t *route_token_indices;
  const int32_t *route_indices;
  const float *route_weights;
  const int32_t *host_scalars;
  const uint64_t *gate_ptrs, *gate_scale_ptrs, *up_ptrs, *up_scale_ptrs, *down_ptrs, *down_scale_ptrs;
  const uint16_t *input;
  float *route_output;
  int32_t *route_written;
  int32_t *route_error;
  const float *prefix;
  uint16_t *output;
  // workspace
  uint8_t *xq;      // [kTermsX][num_tokens][H]     E4M3 terms of the input
  uint8_t *xs;      // [kTermsX][num_tokens][H/32]  their E8M0 scales
  float *hidden;    // [rows][I]                    h = silu(gate)*up*w in f32
  uint8_t *hq;      // [kTermsH][rows][I]
  uint8_t *hs;      // [kTermsH][rows][I/32]
  uint32_t active_group_count, slot_capacity, num_tokens, num_routes, routes_per_token, row_capacity;
  uint32_t input_size, intermediate_size, hidden_size, flags;
  uint32_t packed_only;  // the packed kernels own every token tile (see token_tile_rows)
  // row tiles per wave of the packed kernels' work items (full-length items, items of the tail),
  // chosen on the host from the number of active expert groups: see PackedItems
  uint32_t gate_tpw, gate_tpw_tail, down_tpw, down_tpw_tail;
  float swiglu_limit;
};


// Activation stages of one workgroup.  LDS is not what bounds residency: a workgroup of five waves
// takes two wave slots on EVERY SIMD (the dispatcher reserves the rounded-up share, whichever
// SIMD gets the fifth wave), so at 128 registers (four slots per SIMD) a CU holds two workgroups -
// measured with per-wave time stamps and hardware ids: never more than ten waves on a CU.
constexpr uint32_t kLdsPool = 36u * 1024u;

// ---------------------------------------------------------------------------------------
// Activation stages in LDS, filled by direct global->LDS loads (no VGPR staging).
// A stage holds one K chunk (CKB K blocks) of the m token rows of the current tile:
//   q[term][row][CKB*128 bytes]   the 16-byte piece p of row n sits at slot p ^ n, so the 16
//                                 lanes of one ds_read_b128 hit 16 different bank groups
//   s[term][row][CKB*4 bytes]     scale bytes
// A direct-to-LDS load writes lane i's bytes at base + i*size: one wave instruction fills 64
// consecutive slots (= 64/(CKB*8) rows of one term) or up to 64 scale dwords of one term.
// The number of stages is chosen per token tile so that they fill the pool.  With few tokens
// (the decode case) the whole K extent fits: the activations are loaded once and stay
// resident while the waves walk over several weight row tiles.
// ---------------------------------------------------------------------------------------
template <int TERMS, int CKB>
struct XStages {
  static constexpr uint32_t kRowBytes = CKB * 128u;
  static constexpr uint32_t kSlotsPerRow = CKB * 8u;
  static constexpr uint32_t kRowsPerDma = 64u / kSlotsPerRow;
  uint32_t groups;       // DMA row groups per term
  uint32_t q_term;       // bytes of one term's rows
  uint32_t s_term;       // bytes of one term's scales
  uint32_t stage_bytes;
  uint32_t stages;
  uint32_t loads_per_chunk;
  bool resident;         // stages == chunks of K: every chunk is loaded exactly once

  __device__ XStages(uint32_t m, uint32_t nchunks) {
    groups = (m + kRowsPerDma - 1u) / kRowsPerDma;
    q_term = groups * kRowsPerDma * kRowBytes;
    s_term = (m * CKB * 4u + 63u) & ~63u;
    stage_bytes = TERMS * (q_term + s_term);
    loads_per_chunk = TERMS * (groups + 1u);
    stages = kLdsPool / stage_bytes;
    resident = stages >= nchunks;
    if (resident) {
      stages = nchunks;
    } else {
      stages = stages > 8u ? 8u : stages;
      while (stages > 2u && (stages - 2u) * loads_per_chunk > 48u) --stages;  // vmcnt is 6 bits
    }
  }
  __device__ uint8_t *q(uint8_t *lds, uint32_t stage, uint32_t term) const {
    return lds + stage * stage_bytes + term * q_term;
  }
  __device__ uint8_t *s(uint8_t *lds, uint32_t stage, uint32_t term) const {
    return lds + stage * stage_bytes + TERMS * q_term + term * s_term;
  }
};

// Per-lane source rows of the producer wave, resolved once per token tile (no load may sit
// between two direct-to-LDS loads: the vmcnt it needs would drain them all).
template <int TERMS, int CKB>
struct XSources {
  static constexpr int kMaxGroups = static_cast<int>(kTokenTile / XStages<TERMS, CKB>::kRowsPerDma);
  uint32_t q_row[kMaxGroups];  // row index (token or routed row) this lane copies in group grp
  uint32_t s_row;              // row index whose scale dword this lane copies
};

// Issue the loads that bring chunk `chunk` of the m rows into `stage` (producer wave).
template <int TERMS, int CKB>
__device__ __forceinline__ void xstage_issue(const XStages<TERMS, CKB> &geo, const XSources<TERMS, CKB> &src,
                                             const uint8_t *q_base, const uint8_t *s_base, size_t plane_q,
                                             size_t plane_s, uint8_t *lds, uint32_t stage, uint32_t chunk,
                                             uint32_t m, uint32_t k, uint32_t lane, bool packed) {
  using T = XStages<TERMS, CKB>;
  // swizzle key of row n of a term: the MFMA column that reads it (see mx_consume)
  const uint32_t key_step = packed ? 16u / TERMS : 0u;
  const uint32_t sub = lane / T::kSlotsPerRow;
  const uint32_t slot = lane % T::kSlotsPerRow;
#pragma unroll
  for (uint32_t term = 0; term < static_cast<uint32_t>(TERMS); ++term) {
#pragma unroll
    for (int grp = 0; grp < XSources<TERMS, CKB>::kMaxGroups; ++grp) {
      if (static_cast<uint32_t>(grp) < geo.groups) {
        const uint32_t n = grp * T::kRowsPerDma + sub;
        const uint32_t piece = slot ^ ((n + term * key_step) & (T::kSlotsPerRow - 1u));
        const uint32_t k0 = chunk * T::kRowBytes + piece * 16u;  // FP8: one byte per k
        if (n < m && k0 < k) {
          const uint8_t *from = q_base + term * plane_q + static_cast<size_t>(src.q_row[grp]) * k + k0;
          uint8_t *dst = geo.q(lds, stage, term) + grp * T::kRowsPerDma * T::kRowBytes;
          __builtin_amdgcn_global_load_lds((global_u8_ptr)(from), (lds_void_t *)(dst), 16, 0, 0);
        }
      }
    }
    const uint32_t sn = lane / CKB;
    const uint32_t sk = chunk * CKB * 4u + (lane % CKB) * 4u;  // scale byte index = k / 32
    if (sn < m && sn < kTokenTile && sk * 32u < k) {
      const uint8_t *from = s_base + term * plane_s + static_cast<size_t>(src.s_row) * (k >> 5) + sk;
      __builtin_amdgcn_global_load_lds((global_u8_ptr)(from), (lds_void_t *)(geo.s(lds, stage, term)), 4, 0, 0);
    }
  }
}

// The activation operand of one MFMA: the lane's two 16-byte halves of a K block and its scale.
struct BSlot {
  u32x4_t lo, hi;
  uint32_t sb;
};

// Which activation row and term an MFMA column (lane % 16) multiplies in MFMA slot t of a K
// block.  FORM names the arrangement:
//   0 (general)  column i = activation row i; slot t = term t (TERMS MFMAs per K block)
//   P >= 1 (packed, m * TERMS <= 16 P)  column i = (term i / NPACK, row t * NPACK + i % NPACK)
//                with NPACK = 16 / TERMS: slot t = pass t over NPACK rows with all their terms
//                (P MFMAs per K block), and the columns of a row are added afterwards
template <int FORM, int TERMS>
struct BColumn {
  static constexpr uint32_t kPack = 16u / TERMS;
  static constexpr int kSlots = FORM ? FORM : TERMS;
  uint32_t row, term, last;
  __device__ BColumn(uint32_t lane, uint32_t m) {
    const uint32_t i = lane & 15u;
    term = FORM ? i / kPack : 0u;
    row = FORM ? i % kPack : i;
    last = m - 1u;
  }
};

template <int FORM, int TERMS, int CKB>
__device__ __forceinline__ void read_b(BSlot &f, const XStages<TERMS, CKB> &geo, const uint8_t *lds, uint32_t stage,
                                       uint32_t kk, uint32_t slot, const BColumn<FORM, TERMS> &col, uint32_t g) {
  using T = XStages<TERMS, CKB>;
  using Col = BColumn<FORM, TERMS>;
  const uint32_t term = FORM ? col.term : slot;
  // packed columns beyond m repeat the last row (a broadcast read)
  const uint32_t n = FORM ? min(col.row + slot * Col::kPack, col.last) : col.row;
  // the producer's swizzle key of (row n, term)
  const uint32_t swz = (FORM ? term * Col::kPack + n : n) & (T::kSlotsPerRow - 1u);
  const uint8_t *row = geo.q(const_cast<uint8_t *>(lds), stage, term) + n * T::kRowBytes;
  // 8-bit operand layout: lane g supplies k [16g,16g+16) and [64+16g,64+16g+16)
  f.lo = *reinterpret_cast<const u32x4_t *>(row + ((kk * 8u + g) ^ swz) * 16u);
  f.hi = *reinterpret_cast<const u32x4_t *>(row + ((kk * 8u + 4u + g) ^ swz) * 16u);
  f.sb = geo.s(const_cast<uint8_t *>(lds), stage, term)[n * CKB * 4u + kk * 4u + g];
}

template <int NMAT>
struct MxWFrag {
  u32x4_t w[NMAT];
};

// Weight operands of one wave.  Two storage orders of a [N, K] MXFP4 matrix are walked with
// the same code, both seen as 16-row tiles of K/128 blocks of 64 bytes per row:
//   row-major   [tile][row 0..15][K block][64 B]   the checkpoint order; one wave load of a K
//                                                  block touches 16 rows K/2 bytes apart
//   block-major [tile][K block][row 0..15][64 B]   prepared order; the same load is 1 KB of
//                                                  consecutive bytes, and so is the next one
// and likewise for the scales with 4 bytes (the 4 E8M0 of one K block) in place of 64.  A tile
// has the same size in both, so only the lane's base offset and the K block stride differ.
template <int NMAT>
struct MxOperands {
  const uint8_t *wlane[NMAT];  // this lane's 16 weight bytes of K block 0 in the wave's FIRST row tile
  const uint8_t *slane[NMAT];  // scale dword of this lane's row, K block 0, same tile
  uint32_t k;                  // multiple of 128
  uint32_t tiles;              // row tiles this wave walks over (>= 1)
  uint32_t tile_stride_rows;   // rows between two consecutive tiles of this wave
  uint32_t w_kb_stride;        // bytes from one K block to the next: 64 row-major, 1024 block-major
  uint32_t s_kb_stride;        // same for the scale dwords: 4 or 64
};

// Fills the lane pointers and strides of matrix `m` for the row tile `tile` (clamped by the
// caller to an existing tile).
template <int NMAT>
__device__ __forceinline__ void mx_set_operand(MxOperands<NMAT> &op, int m, const uint8_t *w, const uint8_t *s,
                                               uint32_t tile, uint32_t k, bool block_major, uint32_t lane) {
  const uint32_t r = lane & 15u;
  const uint32_t g = lane >> 4;
  const size_t tile_w = static_cast<size_t>(tile) * 16u * (k >> 1);
  const size_t tile_s = static_cast<size_t>(tile) * 16u * (k >> 5);
  if (block_major) {
    op.wlane[m] = w + tile_w + r * 64u + g * 16u;
    op.slane[m] = s + tile_s + r * 4u;
  } else {
    op.wlane[m] = w + tile_w + static_cast<size_t>(r) * (k >> 1) + g * 16u;
    op.slane[m] = s + tile_s + static_cast<size_t>(r) * (k >> 5);
  }
  op.w_kb_stride = block_major ? 1024u : 64u;
  op.s_kb_stride = block_major ? 64u : 4u;
}

// STREAM: nontemporal loads.  Measured on 4 GiB read once: consecutive 1 KiB wave loads (the
// block-major order) run at 7.0-7.1 TB/s nontemporal against 6.2 TB/s plain, while the 16-row
// pattern of the row-major order is the other way round (4.0 against 5.5 TB/s).
template <bool STREAM, int NMAT>
__device__ __forceinline__ void mx_load_w(MxWFrag<NMAT> &f, const MxOperands<NMAT> &op, uint32_t tile,
                                          uint32_t kb) {
  const size_t off = static_cast<size_t>(tile) * op.tile_stride_rows * (op.k >> 1) + kb * op.w_kb_stride;
#pragma unroll
  for (int m = 0; m < NMAT; ++m) {
    f.w[m] = STREAM ? load_stream16(op.wlane[m] + off) : load16(op.wlane[m] + off);
  }
}

// Weight scales of FOUR consecutive stream positions in one wave load: lane (r, g) fetches the
// scale dword (the 4 E8M0 bytes of one K block) of row r at the g-th of the four positions.
// A K block's MFMA needs, in lane (r, g'), byte g' of the dword held by lane (r, position):
// one ds_bpermute (a cross-lane move, no LDS memory) and a shift.  Loading the dword in every
// lane instead costs four times the load instructions and, because each touches 16 rows,
// twice the L2->L1 line traffic of the weights themselves - measured, that halves the
// achieved bandwidth.
template <int NMAT>
__device__ __forceinline__ void mx_load_scales(uint32_t (&sc)[NMAT], const MxOperands<NMAT> &op, uint32_t tile,
                                               uint32_t kb) {
  const size_t off = static_cast<size_t>(tile) * op.tile_stride_rows * (op.k >> 5) + kb * op.s_kb_stride;
#pragma unroll
  for (int m = 0; m < NMAT; ++m) {
    sc[m] = load4(op.slane[m] + off);
  }
}

// Consumer waves of mx_rowstream.  Every ring refill is unconditional (the stream position is
// clamped instead), so a ring slot is always the plain destination of a load: a conditional
// refill turns the slot into a select between the old and the new value, and the wave then
// waits for the load it has just issued.
// Every term accumulates in its own accumulator (general) or its own MFMA column (packed) over
// the whole K extent and the terms are added at the end in the same tree order, so a row's
// result does not depend on how many rows share its expert.
template <int FORM, bool STREAM, int NMAT, int TERMS, int DEPTH, int CKB, typename Epilogue>
__device__ __forceinline__ void mx_consume(const MxOperands<NMAT> &op, const uint8_t *lds,
                                           const XStages<TERMS, CKB> &geo, uint32_t m, uint32_t lane,
                                           Epilogue epilogue) {
  static_assert(TERMS == 2 || TERMS == 4, "the term sum is a two-level tree");
  using Col = BColumn<FORM, TERMS>;
  constexpr int kSlots = Col::kSlots;
  constexpr int kChunksPerRound = DEPTH / CKB;
  const uint32_t kblocks = op.k >> 7;
  const uint32_t nchunks = kblocks / CKB;
  const uint32_t total_chunks = nchunks * op.tiles;
  const Col col(lane, m);
  const uint32_t g = lane >> 4;
  const uint32_t shift = 8u * g;
  static_assert(DEPTH == 4, "one scale dword group per ring round");
  MxWFrag<NMAT> ring[DEPTH];
  uint32_t sc_cur[NMAT], sc_next[NMAT];
  const uint32_t bperm_base = (lane & 15u) * 4u;  // byte address of lane (r, 0) for ds_bpermute
  // stream position of the next refill
  uint32_t pf_tile = 0, pf_kb = 0;
  // this lane's own position in the scale stream: entry g of the ring round being loaded
  uint32_t sc_tile = 0, sc_kb = g;
  auto clamp_scale_pos = [&]() {
    while (sc_kb >= kblocks) {
      sc_kb -= kblocks;
      ++sc_tile;
    }
    if (sc_tile >= op.tiles) {
      sc_tile = op.tiles - 1u;
      sc_kb = kblocks - 1u;
    }
  };
  clamp_scale_pos();
  mx_load_scales(sc_cur, op, sc_tile, sc_kb);
  sc_kb += DEPTH;
  clamp_scale_pos();
  auto advance = [&]() {
    if (pf_kb + 1u < kblocks) {
      ++pf_kb;
    } else if (pf_tile + 1u < op.tiles) {
      pf_kb = 0;
      ++pf_tile;
    }  // else: stay on the last block (harmless reload)
  };
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) {
    mx_load_w<STREAM>(ring[d], op, pf_tile, pf_kb);
    advance();
    // the loads must leave in ring order here as in the loop below: the wait counts of the loop
    // are fixed at compile time from the worse of the two orders
    __builtin_amdgcn_sched_barrier(0);
  }
  uint32_t stage = 0;
  uint32_t tile = 0, kb = 0;
  f32x4_t acc[NMAT][kSlots];
#pragma unroll
  for (int mm = 0; mm < NMAT; ++mm) {
#pragma unroll
    for (int t = 0; t < kSlots; ++t) acc[mm][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
  for (uint32_t c0 = 0; c0 < total_chunks; c0 += kChunksPerRound) {
    // scales of the NEXT ring round, a full round ahead like the weights themselves
    mx_load_scales(sc_next, op, sc_tile, sc_kb);
    sc_kb += DEPTH;
    clamp_scale_pos();
#pragma unroll
    for (int cc = 0; cc < kChunksPerRound; ++cc) {
      if (c0 + cc < total_chunks) {
        if (!geo.resident || c0 + cc < nchunks) lds_barrier();  // this chunk has landed
        // The MFMAs of a chunk form a list of items (K block, term slot); the B operand of an
        // item is read from LDS kAhead items before its MFMA into a small rotating buffer, so
        // the LDS latency hides behind the matrix work in between.
        constexpr int kItems = CKB * kSlots;
        constexpr int kAhead = FORM == 0 ? 2 : (FORM == 1 ? 1 : 0);
        constexpr int kBuf = kAhead + 1;
        BSlot buf[kBuf];
#pragma unroll
        for (int j = 0; j < kAhead && j < kItems; ++j) {
          read_b<FORM, TERMS, CKB>(buf[j % kBuf], geo, lds, stage, static_cast<uint32_t>(j / kSlots),
                                   static_cast<uint32_t>(j % kSlots), col, g);
        }
        i32x8_t a[NMAT];
        uint32_t sa[NMAT];
#pragma unroll
        for (int j = 0; j < kItems; ++j) {
          const int kk = j / kSlots, t = j % kSlots;
          if (j + kAhead < kItems) {
            read_b<FORM, TERMS, CKB>(buf[(j + kAhead) % kBuf], geo, lds, stage,
                                     static_cast<uint32_t>((j + kAhead) / kSlots),
                                     static_cast<uint32_t>((j + kAhead) % kSlots), col, g);
          }
          if (t == 0) {
#pragma unroll
            for (int mm = 0; mm < NMAT; ++mm) {
              a[mm] = make_a_fp4(ring[cc * CKB + kk].w[mm]);
              sa[mm] = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(
                           static_cast<int>(bperm_base + (cc * CKB + kk) * 64u), static_cast<int>(sc_cur[mm]))) >>
                       shift;
            }
          }
          const i32x8_t b = make_b_fp8(buf[j % kBuf].lo, buf[j % kBuf].hi);
#pragma unroll
          for (int mm = 0; mm < NMAT; ++mm) {
            acc[mm][t] = mfma_fp4_fp8(a[mm], b, acc[mm][t], sa[mm], buf[j % kBuf].sb);
          }
          if (t == kSlots - 1) {
            mx_load_w<STREAM>(ring[cc * CKB + kk], op, pf_tile, pf_kb);
            advance();
            __builtin_amdgcn_sched_barrier(0);  // refills stay in ring order (see the prologue)
          }
        }
        stage = stage + 1u == geo.stages ? 0u : stage + 1u;
        kb += CKB;
        if (kb == kblocks) {
          f32x4_t sum[NMAT];
#pragma unroll
          for (int mm = 0; mm < NMAT; ++mm) {
            if (FORM) {
              // columns (term, row) of one row sit Col::kPack lanes apart: xor-butterfly over the
              // term bits = (t0 + t1) + (t2 + t3), the order of the general path.  Afterwards
              // every column of a row holds the row's sum, so lane r (the epilogue's row r) finds
              // it in its own lane, in the pass that carried row r.
#pragma unroll
              for (int t = 0; t < kSlots; ++t) {
                f32x4_t v = acc[mm][t];
#pragma unroll
                for (uint32_t step = Col::kPack; step < 16u; step <<= 1) {
#pragma unroll
                  for (int e = 0; e < 4; ++e) v[e] += __shfl_xor(v[e], static_cast<int>(step), 64);
                }
                if (t == 0 || (lane & 15u) / Col::kPack == static_cast<uint32_t>(t)) sum[mm] = v;
              }
            } else if (TERMS == 2) {
              sum[mm] = acc[mm][0] + acc[mm][kSlots - 1];
            } else {
              sum[mm] = (acc[mm][0] + acc[mm][1 % kSlots]) + (acc[mm][2 % kSlots] + acc[mm][3 % kSlots]);
            }
          }
          epilogue(tile, sum);
#pragma unroll
          for (int mm = 0; mm < NMAT; ++mm) {
#pragma unroll
            for (int t = 0; t < kSlots; ++t) acc[mm][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
          }
          kb = 0;
          ++tile;
        }
      }
    }
#pragma unroll
    for (int mm = 0; mm < NMAT; ++mm) sc_cur[mm] = sc_next[mm];
  }
  lds_barrier();  // end
}

// acc[m] = W_m[16 rows, K] * X[K, <=16 tokens] for each of the wave's row tiles, X given as
// TERMS MX-FP8 terms; `epilogue(tile, acc)` is called once per tile.
// The workgroup has kWaves consumer waves and ONE producer wave that only moves activation
// chunks into LDS, several chunks ahead: before the barrier that opens a chunk it waits
// (in-order vmcnt) until that chunk's loads have landed, and right after the barrier it
// refills the stage the consumers have just left.  Consumers never wait on those loads, and
// their weight stream (tile after tile, K block after K block) is one uninterrupted prefetch
// ring.  Requires k % (CKB*128) == 0 so that chunks do not straddle tiles.
// The role is a template parameter and the kernels branch on it ONCE, outside their token
// tile loop: when both roles share a loop, the compiler's wait-count bookkeeping carries the
// producer's outstanding direct-to-LDS loads around the back edge into the consumer code and
// the consumers then drain all their own weight loads (vmcnt(0)) at every ring round.
template <bool PRODUCER, int FORM, bool STREAM, int NMAT, int TERMS, int DEPTH, int CKB, typename Epilogue>
__device__ __forceinline__ void mx_rowstream(const MxOperands<NMAT> &op, uint8_t *lds, uint32_t m,
                                             uint32_t lane,
                                             const XSources<TERMS, CKB> &src, const uint8_t *q_base,
                                             const uint8_t *s_base, size_t plane_q, size_t plane_s,
                                             Epilogue epilogue) {
  static_assert(DEPTH % CKB == 0, "the ring is addressed with the unrolled block index");
  using T = XStages<TERMS, CKB>;
  const uint32_t kblocks = op.k >> 7;
  const uint32_t nchunks = kblocks / CKB;
  const T geo(m, nchunks);
  const uint32_t total_chunks = nchunks * op.tiles;
  constexpr bool packed = FORM != 0;

  if constexpr (PRODUCER) {
    const uint32_t to_load = geo.resident ? nchunks : total_chunks;
    const uint32_t ahead = geo.resident ? nchunks : geo.stages - 1u;
    uint32_t fill = 0;      // stage that receives the next chunk
    uint32_t chunk_k = 0;   // K chunk (0..nchunks-1) of the next load
    uint32_t issued = 0;
    for (; issued < ahead && issued < to_load; ++issued) {
      xstage_issue<TERMS, CKB>(geo, src, q_base, s_base, plane_q, plane_s, lds, fill, chunk_k, m, op.k, lane, packed);
      fill = fill + 1u == geo.stages ? 0u : fill + 1u;
      chunk_k = chunk_k + 1u == nchunks ? 0u : chunk_k + 1u;
    }
    // resident activations: only the first pass over K synchronises (the chunks are arriving);
    // afterwards the stages are read-only
    const uint32_t sync_chunks = geo.resident ? nchunks : total_chunks;
    for (uint32_t c = 0; c < sync_chunks; ++c) {
      // loads younger than chunk c's may stay in flight
      const uint32_t younger = issued > c + 1u ? issued - c - 1u : 0u;
      wait_vmcnt(younger * geo.loads_per_chunk);
      // bare barrier: a fence here would make this wave wait for ALL its direct-to-LDS loads
      // (vmcnt(0)) and the chunks ahead could never stay in flight
      stage_barrier();  // chunk c is visible; the consumers have left chunk c-1
      if (issued < to_load) {
        xstage_issue<TERMS, CKB>(geo, src, q_base, s_base, plane_q, plane_s, lds, fill, chunk_k, m, op.k, lane, packed);
        fill = fill + 1u == geo.stages ? 0u : fill + 1u;
        chunk_k = chunk_k + 1u == nchunks ? 0u : chunk_k + 1u;
        ++issued;
      }
    }
    stage_barrier();  // end: nobody reads the stages any more
  } else {
    mx_consume<FORM, STREAM, NMAT, TERMS, DEPTH, CKB>(op, lds, geo, m, lane, epilogue);
  }
}

__device__ __forceinline__ uint32_t live_groups(const MoeParams &p) {
  uint32_t groups = p.active_group_count;
  if (p.host_scalars != nullptr) {
    const int32_t planned = p.host_scalars[0];
    groups = planned < 0 ? 0u : min(groups, static_cast<uint32_t>(planned));
  }
  return groups;
}

constexpr uint32_t kThreads = (kWaves + 1u) * 64u;  // four consumer waves + the producer

// A token tile whose rows x terms fit PASSES x 16 MFMA columns runs in a packed form (BColumn),
// in as many passes as it needs; longer ones run in the general form.  Packed and general live
// in separate kernels (each keeps its own register budget), both launched over the same grid; a
// workgroup leaves at once when its expert has no tile of its form.  PASSES is 1 or 2 and set
// per projection (kGatePasses, kDownPasses).
template <int TERMS>
__device__ __forceinline__ uint32_t tile_passes(uint32_t m) {
  return (m * TERMS + 15u) / 16u;
}
template <int TERMS, int PASSES>
__device__ __forceinline__ bool tile_is_packed(uint32_t m) {
  return tile_passes<TERMS>(m) <= static_cast<uint32_t>(PASSES);
}
template <int TERMS, int PASSES, bool PACKED>
__device__ __forceinline__ bool expert_has_tiles(uint32_t rows) {
  if (rows == 0u) return false;
  const uint32_t last = rows % kTokenTile == 0u ? kTokenTile : rows % kTokenTile;
  const bool full = rows > kTokenTile;  // whole tiles of kTokenTile rows before the last one
  return PACKED ? (tile_is_packed<TERMS, PASSES>(last) || (full && tile_is_packed<TERMS, PASSES>(kTokenTile)))
                : (!tile_is_packed<TERMS, PASSES>(last) || (full && !tile_is_packed<TERMS, PASSES>(kTokenTile)));
}
// Calls run(integral_constant<int, FORM>) with the form of a token tile of m rows that this
// kernel kind (packed or general) owns.
template <int TERMS, int PASSES, bool PACKED, typename Run>
__device__ __forceinline__ void with_tile_form(uint32_t m, Run run) {
  static_assert(PASSES == 1 || PASSES == 2, "forms 1 and 2 are instantiated");
  if constexpr (!PACKED) {
    run(std::integral_constant<int, 0>{});
  } else if constexpr (PASSES == 1) {
    run(std::integral_constant<int, 1>{});
  } else {
    if (tile_passes<TERMS>(m) == 1u) {
      run(std::integral_constant<int, 1>{});
    } else {
      run(std::integral_constant<int, 2>{});
    }
  }
}
// Rows of one token tile.  Normally kTokenTile, and a tile goes to the kernel of its form.  When
// the routes are sparse (few rows per expert on average) nearly every launch of the general
// kernels would find nothing to do, so they are not launched at all: the packed kernels then cut
// the rows of an expert into tiles that fit their passes, and the rare long expert streams its
// weights once more per extra tile.  A row's bits are the same either way.
template <int TERMS, int PASSES, bool PACKED>
__device__ __forceinline__ uint32_t token_tile_rows(const MoeParams &p) {
  constexpr uint32_t kPackedRows = 16u * PASSES / TERMS;
  static_assert(kPackedRows >= 1u && kPackedRows <= kTokenTile, "a packed tile is a part of a token tile");
  return (PACKED && p.packed_only) ? kPackedRows : kTokenTile;
}
// Passes of the packed kernels.  gate/up stays at one: with two, the kernel needs 15-20 spilled
// registers at the 128-register occupancy cap and ran 100 us slower although the spills sit
// outside the K loop.  Its 9..16-row tiles go to the general kernel (or, for sparse routes, are
// cut into 8-row tiles).
constexpr int kGatePasses = 1;
constexpr int kDownPasses = 2;

// Work item of a workgroup: (expert group, chunk of row tiles, row tiles per wave).  The item lengths
// are chosen on the host per launch (packed_items); the template parameter TPW is the longest one.
//   general kernels: grid (chunks, groups), every item of the full length.
//   packed kernels:  a 1-D grid in dispatch order.  The first three quarters of the live groups
//     run full-length items; the last quarter runs items of half the length, twice as many workgroups,
//     so that the machine drains over a shorter tail (all workgroups of a stage are otherwise
//     equally long, 80-150 us, and the last ones run on a nearly empty machine).
struct WorkItem {
  uint32_t group, chunk, tpw;
  bool live;
};
template <int TPW, bool PACKED>
__device__ __forceinline__ WorkItem work_item(const MoeParams &p, uint32_t total_tiles, uint32_t tpw_full,
                                              uint32_t tpw_tail) {
  WorkItem w;
  const uint32_t groups = live_groups(p);
  if constexpr (!PACKED) {
    w.group = blockIdx.y;
    w.chunk = blockIdx.x;
    w.tpw = tpw_full;   // the general kernels' grid is (chunks of this length, groups)
    w.live = w.group < groups;
  } else {
    const uint32_t chunks_full = (total_tiles + kWaves * tpw_full - 1u) / (kWaves * tpw_full);
    const uint32_t chunks_half = (total_tiles + kWaves * tpw_tail - 1u) / (kWaves * tpw_tail);
    const uint32_t full = groups - groups / 4u;
    const uint32_t id = blockIdx.x;
    if (id < full * chunks_full) {
      w.group = id / chunks_full;
      w.chunk = id - w.group * chunks_full;
      w.tpw = tpw_full;
      w.live = true;
    } else {
      const uint32_t rest = id - full * chunks_full;
      w.group = full + rest / chunks_half;
      w.chunk = rest % chunks_half;
      w.tpw = tpw_tail;
      w.live = w.group < groups;
    }
  }
  return w;
}
// Item lengths of a packed launch.  With the layer's usual few hundred active expert groups an item
// is `most` row tiles per wave (about 1 MB of weights per workgroup), the tail half of that.  A small
// decode batch activates few experts (one token: top-k of them), and items of that length would
// leave most of the machine idle: 8 experts are 128 gate/up and 56 down workgroups on 256 CUs.
// The length is halved until the launch has about `kItemsWanted` workgroups or reaches `least`
// (gate/up: one tile per wave; down walks its tiles in pairs).  Which tiles share a workgroup does
// not touch any row's arithmetic.  Measured per step with the experts of successive steps rotating
// (64 tokens per step are 0.81 ms): one token 82 -> 58 us, two 101 -> 86 us, four 146 -> 141 us, six
// and more unchanged; asking for 512 or 1024 workgroups made four and eight tokens 5-9 % slower.
struct PackedItems {
  uint32_t full, tail, grid;
};
inline PackedItems packed_items(uint32_t groups, uint32_t total_tiles, uint32_t most, uint32_t least) {
  constexpr uint32_t kItemsWanted = 384u;
  auto chunks = [&](uint32_t tpw) { return (total_tiles + kWaves * tpw - 1u) / (kWaves * tpw); };
  PackedItems it;
  it.full = most;
  while (it.full > least && static_cast<uint64_t>(groups) * chunks(it.full) < kItemsWanted) it.full /= 2u;
  it.tail = it.full / 2u >= least ? it.full / 2u : it.full;
  const uint32_t full_groups = groups - groups / 4u;
  // fewer live groups than `groups` move the boundary down: all of them live is the worst case
  it.grid = full_groups * chunks(it.full) + (groups - full_groups) * chunks(it.tail);
  if (it.grid == 0u) it.grid = 1u;
  return it;
}

// Row tiles of one workgroup: kWaves * TPW consecutive tiles; wave w owns tiles w, w+4, ...
// so that at every step the four waves read adjacent rows.
template <int DEPTH, int TPW, bool BLOCK_MAJOR, bool PACKED>
__global__ __launch_bounds__(kThreads, PACKED ? 4 : 3) void moe_gate_up_kernel(MoeParams p) {
  constexpr int CKB = 4;
  __shared__ __attribute__((aligned(1024))) uint8_t lds[kLdsPool];
  const uint32_t total_tiles = p.intermediate_size >> 4;
  const WorkItem item = work_item<TPW, PACKED>(p, total_tiles, p.gate_tpw, p.gate_tpw_tail);
  if (!item.live) return;
  const uint32_t group = item.group;
  const int32_t slot = p.active_expert_slots[group];
  if (slot < 0 || static_cast<uint32_t>(slot) >= p.slot_capacity) {
    if (threadIdx.x == 0 && item.chunk == 0u) atomicOr(p.route_error, 1);
    return;
  }
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const bool producer = wave == kWaves;
  const uint32_t r = lane & 15u;
  const uint32_t g = lane >> 4;
  const uint32_t chunk_tile = item.chunk * (kWaves * item.tpw);  // first row tile of the workgroup
  const uint32_t first_tile = chunk_tile + (producer ? 0u : wave);
  const uint32_t row_begin = static_cast<uint32_t>(p.expert_route_indptr[group]);
  const uint32_t row_end = static_cast<uint32_t>(p.expert_route_indptr[group + 1]);
  const uint32_t tile_rows = token_tile_rows<kTermsX, kGatePasses, PACKED>(p);
  if (PACKED && p.packed_only) {
    if (row_end <= row_begin) return;
  } else if (!expert_has_tiles<kTermsX, kGatePasses, PACKED>(row_end > row_begin ? row_end - row_begin : 0u)) {
    return;
  }

  MxOperands<2> op;
  constexpr bool block_major = BLOCK_MAJOR;
  const uint32_t base_tile = min(first_tile, total_tiles - 1u);
  mx_set_operand(op, 0, reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(p.gate_ptrs[slot])),
                 reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(p.gate_scale_ptrs[slot])), base_tile,
                 p.input_size, block_major, lane);
  mx_set_operand(op, 1, reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(p.up_ptrs[slot])),
                 reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(p.up_scale_ptrs[slot])), base_tile,
                 p.input_size, block_major, lane);
  op.k = p.input_size;
  op.tile_stride_rows = kWaves * 16u;
  // tiles of this wave that exist (the grid covers total_tiles exactly when it divides)
  uint32_t tiles = 0;
  for (uint32_t j = 0; j < item.tpw; ++j) {
    if (first_tile + j * kWaves < total_tiles) ++tiles;
  }
  // every wave must run the same number of chunks: use the workgroup's maximum (wave 0's)
  uint32_t wg_tiles = 0;
  for (uint32_t j = 0; j < item.tpw; ++j) {
    if (chunk_tile + j * kWaves < total_tiles) ++wg_tiles;
  }
  op.tiles = wg_tiles;

  const size_t plane_q = static_cast<size_t>(p.num_tokens) * p.input_size;
  const size_t plane_s = static_cast<size_t>(p.num_tokens) * (p.input_size >> 5);
  if (producer) {
    for (uint32_t t0 = row_begin; t0 < row_end; t0 += tile_rows) {
      const uint32_t m = min(tile_rows, row_end - t0);
      if (tile_is_packed<kTermsX, kGatePasses>(m) != PACKED) continue;
      XSources<kTermsX, CKB> src;
      using T = XStages<kTermsX, CKB>;
      auto token_of = [&](uint32_t nrow) {
        if (nrow >= m) return 0u;
        const int32_t token = p.route_token_indices[t0 + nrow];
        return (token >= 0 && static_cast<uint32_t>(token) < p.num_tokens) ? static_cast<uint32_t>(token) : 0u;
      };
#pragma unroll
      for (int grp = 0; grp < XSources<kTermsX, CKB>::kMaxGroups; ++grp) {
        src.q_row[grp] = token_of(grp * T::kRowsPerDma + lane / T::kSlotsPerRow);
      }
      src.s_row = token_of(lane / CKB);
      mx_rowstream<true, PACKED ? 1 : 0, BLOCK_MAJOR, 2, kTermsX, DEPTH, CKB>(op, lds, m, lane, src, p.xq, p.xs, plane_q, plane_s,
                                                 [](uint32_t, f32x4_t (&)[2]) {});
    }
    return;
  }
  for (uint32_t t0 = row_begin; t0 < row_end; t0 += tile_rows) {
    const uint32_t m = min(tile_rows, row_end - t0);
    if (tile_is_packed<kTermsX, kGatePasses>(m) != PACKED) continue;
    const XSources<kTermsX, CKB> src{};
    const float weight = r < m ? p.route_weights[t0 + r] : 0.0f;
    auto epilogue = [&](uint32_t tile_j, f32x4_t (&acc)[2]) {
      const uint32_t tile = first_tile + tile_j * kWaves;
      if (tile_j < tiles && tile < total_tiles && r < m) {
        float h[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          float gate = acc[0][v];
          float up = acc[1][v];
          if (p.swiglu_limit > 0.0f) {
            gate = fminf(gate, p.swiglu_limit);
            up = fminf(p.swiglu_limit, fmaxf(-p.swiglu_limit, up));
          }
          h[v] = silu_ref(gate) * up * weight;
        }
        float *out = p.hidden + static_cast<size_t>(t0 + r) * p.intermediate_size + tile * 16u + g * 4u;
        *reinterpret_cast<float4 *>(out) = make_float4(h[0], h[1], h[2], h[3]);
      }
    };
    with_tile_form<kTermsX, kGatePasses, PACKED>(m, [&](auto form) {
      mx_rowstream<false, decltype(form)::value, BLOCK_MAJOR, 2, kTermsX, DEPTH, CKB>(op, lds, m, lane, src, p.xq, p.xs,
                                                                                     plane_q, plane_s, epilogue);
    });
  }
}

template <int DEPTH, int TPW, bool BLOCK_MAJOR, bool PACKED>
__global__ __launch_bounds__(kThreads, PACKED ? 4 : 3) void moe_down_kernel(MoeParams p) {
  constexpr int CKB = 2;
  __shared__ __attribute__((aligned(1024))) uint8_t lds[kLdsPool];
  const uint32_t total_tiles = p.hidden_size >> 4;
  const WorkItem item = work_item<TPW, PACKED>(p, total_tiles, p.down_tpw, p.down_tpw_tail);
  if (!item.live) return;
  const uint32_t group = item.group;
  const int32_t slot = p.active_expert_slots[group];
  if (slot < 0 || static_cast<uint32_t>(slot) >= p.slot_capacity) return;  // flagged by gate_up
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const bool producer = wave == kWaves;
  const uint32_t r = lane & 15u;
  const uint32_t g = lane >> 4;
  const uint32_t chunk_tile = item.chunk * (kWaves * item.tpw);
  const uint32_t first_tile = chunk_tile + (producer ? 0u : wave);
  const uint32_t row_begin = static_cast<uint32_t>(p.expert_route_indptr[group]);
  const uint32_t row_end = static_cast<uint32_t>(p.expert_route_indptr[group + 1]);
  const uint32_t tile_rows = token_tile_rows<kTermsH, kDownPasses, PACKED>(p);
  if (PACKED && p.packed_only) {
    if (row_end <= row_begin) return;
  } else if (!expert_has_tiles<kTermsH, kDownPasses, PACKED>(row_end > row_begin ? row_end - row_begin : 0u)) {
    return;
  }

  // Two row tiles at a time (tile and tile + kWaves) share every activation fragment read
  // from LDS: the "two matrices" of the stream are two row tiles of the same W2.
  static_assert(TPW % 2 == 0 && (!PACKED || TPW % 4 == 0), "down walks its row tiles in pairs");
  MxOperands<2> op;
  const uint8_t *down_w = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(p.down_ptrs[slot]));
  const uint8_t *down_s = reinterpret_cast<const uint8_t *>(static_cast<uintptr_t>(p.down_scale_ptrs[slot]));
  constexpr bool block_major = BLOCK_MAJOR;
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    mx_set_operand(op, half, down_w, down_s, min(first_tile + half * kWaves, total_tiles - 1u),
                   p.intermediate_size, block_major, lane);
  }
  op.k = p.intermediate_size;
  op.tile_stride_rows = 2u * kWaves * 16u;
  uint32_t wg_pairs = 0;
  for (uint32_t j = 0; j < item.tpw / 2u; ++j) {
    if (chunk_tile + j * 2u * kWaves < total_tiles) ++wg_pairs;
  }
  op.tiles = wg_pairs;

  const size_t plane_q = static_cast<size_t>(p.row_capacity) * p.intermediate_size;
  const size_t plane_s = static_cast<size_t>(p.row_capacity) * (p.intermediate_size >> 5);
  if (producer) {
    for (uint32_t t0 = row_begin; t0 < row_end; t0 += tile_rows) {
      const uint32_t m = min(tile_rows, row_end - t0);
      if (tile_is_packed<kTermsH, kDownPasses>(m) != PACKED) continue;
      XSources<kTermsH, CKB> src;
      using T = XStages<kTermsH, CKB>;
#pragma unroll
      for (int grp = 0; grp < XSources<kTermsH, CKB>::kMaxGroups; ++grp) {
        src.q_row[grp] = t0 + min(grp * T::kRowsPerDma + lane / T::kSlotsPerRow, m - 1u);
      }
      src.s_row = t0 + min(lane / CKB, m - 1u);
      mx_rowstream<true, PACKED ? 1 : 0, BLOCK_MAJOR, 2, kTermsH, DEPTH, CKB>(op, lds, m, lane, src, p.hq, p.hs, plane_q, plane_s,
                                                 [](uint32_t, f32x4_t (&)[2]) {});
    }
    return;
  }
  for (uint32_t t0 = row_begin; t0 < row_end; t0 += tile_rows) {
    const uint32_t m = min(tile_rows, row_end - t0);
    if (tile_is_packed<kTermsH, kDownPasses>(m) != PACKED) continue;
    const XSources<kTermsH, CKB> src{};
    const int32_t route = r < m ? p.route_indices[t0 + r] : -1;
    auto epilogue = [&](uint32_t pair_j, f32x4_t (&acc)[2]) {
      if (route < 0 || static_cast<uint32_t>(route) >= p.num_routes) return;
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const uint32_t tile = first_tile + (pair_j * 2u + half) * kWaves;
        if (tile < total_tiles) {
          float *out = p.route_output + static_cast<size_t>(route) * p.hidden_size + tile * 16u + g * 4u;
          *reinterpret_cast<float4 *>(out) =
              make_float4(acc[half][0], acc[half][1], acc[half][2], acc[half][3]);
          if (tile == 0u && g == 0u) p.route_written[route] = 1;
        }
      }
    };
    with_tile_form<kTermsH, kDownPasses, PACKED>(m, [&](auto form) {
      mx_rowstream<false, decltype(form)::value, BLOCK_MAJOR, 2, kTermsH, DEPTH, CKB>(op, lds, m, lane, src, p.hq, p.hs,
                                                                                     plane_q, plane_s, epilogue);
    });
  }
}

// output[t,h] = bf16(prefix[t,h] + sum over ranks in order); NaN when a route of the token
// was not produced or the error flag is up (portable/entrypoints.cu:1591-1603).
__global__ __launch_bounds__(256) void moe_combine_kernel(MoeParams p) {
  const uint32_t per_row = p.hidden_size >> 2;
  const uint64_t index = static_cast<uint64_t>(blockIdx.x) * 256u + threadIdx.x;
  if (index >= static_cast<uint64_t>(p.num_tokens) * per_row) return;
  const uint32_t token = static_cast<uint32_t>(index / per_row);
  const uint32_t h0 = static_cast<uint32_t>(index % per_row) * 4u;
  // The route rows are requested before the flags are known (a row that was not written is
  // allocated memory all the same): one memory round trip instead of three in a kernel that is
  // nothing but latency.  Eight rows in flight, added in rank order.
  typedef float f32x4v __attribute__((ext_vector_type(4)));
  const f32x4v *rows = reinterpret_cast<const f32x4v *>(
      p.route_output + static_cast<size_t>(token) * p.routes_per_token * p.hidden_size + h0);
  const size_t stride = p.hidden_size >> 2;
  f32x4v acc = {0.f, 0.f, 0.f, 0.f};
  if (p.prefix != nullptr) {
    acc = *reinterpret_cast<const f32x4v *>(p.prefix + static_cast<size_t>(token) * p.hidden_size + h0);
  }
  bool complete = true;
  for (uint32_t rank0 = 0; rank0 < p.routes_per_token; rank0 += 8u) {
    f32x4v v[8];
    int32_t written[8];
#pragma unroll
    for (uint32_t j = 0; j < 8u; ++j) {
      const bool in = rank0 + j < p.routes_per_token;
      v[j] = in ? __builtin_nontemporal_load(rows + (rank0 + j) * stride) : f32x4v{0.f, 0.f, 0.f, 0.f};
      written[j] = in ? p.route_written[token * p.routes_per_token + rank0 + j] : 1;
    }
#pragma unroll
    for (uint32_t j = 0; j < 8u; ++j) {
      complete &= written[j] != 0;
      if (rank0 + j < p.routes_per_token) {
        // routed.rs:183-201: without a prefix the first route initialises the accumulator
        acc = (rank0 + j == 0u && p.prefix == nullptr) ? v[j] : acc + v[j];
      }
    }
  }
  complete &= p.route_error[0] == 0;
  uint16_t *out = p.output + static_cast<size_t>(token) * p.hidden_size + h0;
  if (!complete) {
    *reinterpret_cast<uint2 *>(out) = make_uint2(0x7fc07fc0u, 0x7fc07fc0u);
    return;
  }
  const uint32_t b0 = bf16_rne_bits(acc[0]), b1 = bf16_rne_bits(acc[1]);
  const uint32_t b2 = bf16_rne_bits(acc[2]), b3 = bf16_rne_bits(acc[3]);
  *reinterpret_cast<uint2 *>(out) = make_uint2(b0 | (b1 << 16), b2 | (b3 << 16));
}

// Row-major -> block-major reorder of one [n, k] MXFP4 matrix (see MxOperands): within every
// 16-row tile the (row, K block) grid of 64-byte payload cells and of 4-byte scale cells is
// transposed.  One thread moves one 16-byte payload piece; the first n*k/128 threads also move
// one scale dword.  Reads come in 64-byte runs, writes are consecutive.
__global__ __launch_bounds__(256) void mxfp4_block_major_kernel(const uint8_t *__restrict__ w_src,
                                                                const uint8_t *__restrict__ s_src,
                                                                uint8_t *__restrict__ w_dst,
                                                                uint8_t *__restrict__ s_dst, uint32_t n,
                                                                uint32_t kblocks) {
  const uint64_t cells = static_cast<uint64_t>(n) * kblocks;
  const uint64_t at = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (at >= cells * 4u) return;
  const uint32_t piece = static_cast<uint32_t>(at & 3u);
  const uint64_t cell = at >> 2;  // destination cell: [tile][kblock][row]
  const uint32_t row = static_cast<uint32_t>(cell & 15u);
  const uint64_t tk = cell >> 4;
  const uint32_t kb = static_cast<uint32_t>(tk % kblocks);
  const uint64_t tile = tk / kblocks;
  const uint64_t src_cell = (tile * 16u + row) * kblocks + kb;
  *reinterpret_cast<uint4 *>(w_dst + cell * 64u + piece * 16u) =
      *reinterpret_cast<const uint4 *>(w_src + src_cell * 64u + piece * 16u);
  if (piece == 0u && s_src != nullptr) {
    *reinterpret_cast<uint32_t *>(s_dst + cell * 4u) = *reinterpret_cast<const uint32_t *>(s_src + src_cell * 4u);
  }
}

inline uint64_t align256(uint64_t v) { return (v + 255u) & ~static_cast<uint64_t>(255u); }

struct WorkspaceLayout {
  uint64_t xq, xs, hidden, hq, hs, total;
};

// Regions (each 256-byte aligned): the MX terms of the input, h in f32, the MX terms of h.
inline WorkspaceLayout workspace_layout(const FerruleHipMoeDecodeArgs &a) {
  WorkspaceLayout w;
  uint64_t at = 0;
  w.xq = at; at += align256(static_cast<uint64_t>(kTermsX) * a.num_tokens * a.input_size);
  w.xs = at; at += align256(static_cast<uint64_t>(kTermsX) * a.num_tokens * (a.input_size / 32u));
  w.hidden = at; at += align256(static_cast<uint64_t>(a.total_routed_rows) * a.intermediate_size * 4u);
  w.hq = at; at += align256(static_cast<uint64_t>(kTermsH) * a.total_routed_rows * a.intermediate_size);
  w.hs = at; at += align256(static_cast<uint64_t>(kTermsH) * a.total_routed_rows * (a.intermediate_size / 32u));
  w.total = at;
  return w;
}

int32_t validate(const FerruleHipMoeDecodeArgs *a) {
  if (a == nullptr) return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->active_group_count == 0 || a->slot_capacity == 0 || a->active_group_count > a->slot_capacity)
    return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->total_routed_rows == 0 || a->num_tokens == 0 || a->num_routes == 0 || a->routes_per_token == 0)
    return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->num_routes != a->num_tokens * a->routes_per_token) return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->input_size == 0 || a->intermediate_size == 0 || a->hidden_size == 0)
    return FERRULE_HIP_INVALID_ARGUMENT;
  // K extents are walked in chunks of 4 (gate/up) and 2 (down) 128-wide blocks
  if (a->input_size % 512u != 0 || a->intermediate_size % 256u != 0 || a->hidden_size % 16u != 0)
    return FERRULE_HIP_UNSUPPORTED;
  // down walks its output rows in groups of 8 tiles (4 waves x a pair); only the first group of a
  // workgroup is clamped to the matrix, so a partial group is accepted only when it is the only one
  if (a->hidden_size % 128u != 0 && a->hidden_size > 128u) return FERRULE_HIP_UNSUPPORTED;
  if (a->active_group_count > 65535u) return FERRULE_HIP_UNSUPPORTED;  // grid.y of the general kernels
  // the packed kernels' 1-D grids: at most one workgroup per group and four row tiles
  const uint64_t most_tiles = (a->intermediate_size > a->hidden_size ? a->intermediate_size : a->hidden_size) / 16u;
  if (static_cast<uint64_t>(a->active_group_count) * ((most_tiles + 3u) / 4u) > 0x7fffffffull) return FERRULE_HIP_UNSUPPORTED;
  const uint64_t ptrs[] = {a->active_expert_slots, a->expert_route_indptr, a->route_token_indices,
                           a->route_indices, a->route_weights, a->gate_ptrs, a->gate_scale_ptrs,
                           a->up_ptrs, a->up_scale_ptrs, a->down_ptrs, a->down_scale_ptrs,
                           a->input_bf16, a->route_output, a->route_written, a->route_error, a->workspace};
  for (uint64_t v : ptrs) {
    if (v == 0) return FERRULE_HIP_INVALID_ARGUMENT;
  }
  if ((a->input_bf16 & 15u) || (a->route_output & 15u) || (a->workspace & 255u))
    return FERRULE_HIP_INVALID_ARGUMENT;
  if (a->flags & FERRULE_HIP_MOE_DECODE_COMBINE) {
    if (a->output == 0 || (a->output & 7u)) return FERRULE_HIP_INVALID_ARGUMENT;
    if ((a->flags & FERRULE_HIP_MOE_DECODE_PREFIX_F32) && (a->prefix_f32 == 0 || (a->prefix_f32 & 15u)))
      return FERRULE_HIP_INVALID_ARGUMENT;
  }
  if (a->workspace_bytes < workspace_layout(*a).total) return FERRULE_HIP_INVALID_ARGUMENT;
  return FERRULE_HIP_SUCCESS;
}

template <typename T>
T *as_ptr(uint64_t v) {
  return reinterpret_cast<T *>(static_cast<uintptr_t>(v));
}

}  // namespace
}  // namespace ferrule_hip

using namespace ferrule_hip;

extern "C" int32_t ferrule_hip_prepare_mxfp4_block_major(const FerruleHipPrepareMxfp4BlockMajorArgs *args) {
  if (args == nullptr || args->n == 0 || args->k == 0) return FERRULE_HIP_INVALID_ARGUMENT;
  if (args->n % 16u != 0 || args->k % 128u != 0) return FERRULE_HIP_UNSUPPORTED;
  const uint64_t ptrs[] = {args->weight_source, args->scale_source, args->weight_destination,
                           args->scale_destination};
  for (uint64_t v : ptrs) {
    if (v == 0 || (v & 15u)) return FERRULE_HIP_INVALID_ARGUMENT;
  }
  const uint64_t w_bytes = static_cast<uint64_t>(args->n) * (args->k / 2u);
  const uint64_t s_bytes = static_cast<uint64_t>(args->n) * (args->k / 32u);
  auto overlap = [](uint64_t a, uint64_t b, uint64_t bytes) { return a < b + bytes && b < a + bytes; };
  if (overlap(args->weight_source, args->weight_destination, w_bytes) ||
      overlap(args->scale_source, args->scale_destination, s_bytes))
    return FERRULE_HIP_INVALID_ARGUMENT;
  const uint64_t threads = w_bytes / 16u;
  if ((threads + 255u) / 256u > 0x7fffffffull) return FERRULE_HIP_UNSUPPORTED;
  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(args->stream));
  clear_launch_error();
  mxfp4_block_major_kernel<<<dim3(static_cast<uint32_t>((threads + 255u) / 256u)), dim3(256), 0, stream>>>(
      as_ptr<const uint8_t>(args->weight_source), as_ptr<const uint8_t>(args->scale_source),
      as_ptr<uint8_t>(args->weight_destination), as_ptr<uint8_t>(args->scale_destination), args->n,
      args->k / 128u);
  return take_launch_error() == hipSuccess ? FERRULE_HIP_SUCCESS : FERRULE_HIP_LAUNCH_FAILED;
}

extern "C" int32_t ferrule_hip_prepare_fp8_block_major(const FerruleHipPrepareFp8BlockMajorArgs *args) {
  if (args == nullptr || args->n == 0 || args->k == 0) return FERRULE_HIP_INVALID_ARGUMENT;
  if (args->n % 16u != 0 || args->k % 128u != 0) return FERRULE_HIP_UNSUPPORTED;
  if (args->weight_source == 0 || args->weight_destination == 0 || (args->weight_source & 15u) ||
      (args->weight_destination & 15u))
    return FERRULE_HIP_INVALID_ARGUMENT;
  const uint64_t bytes = static_cast<uint64_t>(args->n) * args->k;
  if (args->weight_source < args->weight_destination + bytes && args->weight_destination < args->weight_source + bytes)
    return FERRULE_HIP_INVALID_ARGUMENT;
  const uint64_t threads = bytes / 16u;
  if ((threads + 255u) / 256u > 0x7fffffffull) return FERRULE_HIP_UNSUPPORTED;
  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(args->stream));
  clear_launch_error();
  // the same 64-byte-cell transposition as for MXFP4, with k/64 cells per row and no scale cells
  mxfp4_block_major_kernel<<<dim3(static_cast<uint32_t>((threads + 255u) / 256u)), dim3(256), 0, stream>>>(
      as_ptr<const uint8_t>(args->weight_source), nullptr, as_ptr<uint8_t>(args->weight_destination), nullptr,
      args->n, args->k / 64u);
  return take_launch_error() == hipSuccess ? FERRULE_HIP_SUCCESS : FERRULE_HIP_LAUNCH_FAILED;
}

extern "C" uint64_t ferrule_hip_moe_decode_workspace_size(const FerruleHipMoeDecodeArgs *args) {
  if (args == nullptr || args->total_routed_rows == 0 || args->intermediate_size == 0 ||
      args->num_tokens == 0 || args->input_size == 0)
    return 0;
  return workspace_layout(*args).total;
}

extern "C" int32_t ferrule_hip_moe_decode_can_implement(const FerruleHipMoeDecodeArgs *args) {
  return validate(args);
}

namespace ferrule_hip {
namespace {

// Scratch of ferrule_hip_moe_decode_launch_static_workspace: the layer's workspace regions
// (MX terms of the input, h in f32, MX terms of h) for callers that cannot bring device
// memory of their own.  Every GPU the library runs on holds its own copy at its own address
// until the process ends.  In host code the array's NAME is only a handle for
// hipGetSymbolAddress, never a device address.
static __device__ __align__(256) unsigned char scratch[FERRULE_HIP_MOE_DECODE_STATIC_WORKSPACE_BYTES];

constexpr int kMaxDevices = 64;
std::atomic<unsigned char *> g_scratch_address[kMaxDevices];

// Device address of `scratch` on the CURRENT device, looked up once per device.
unsigned char *scratch_address() {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return nullptr;
  unsigned char *address = g_scratch_address[device].load(std::memory_order_acquire);
  if (address == nullptr) {
    void *symbol = nullptr;
    const hipError_t e = hipGetSymbolAddress(&symbol, HIP_SYMBOL(scratch));
    if (e != hipSuccess || symbol == nullptr) {
      g_last_hip_error = static_cast<int32_t>(e);
      return nullptr;
    }
    address = static_cast<unsigned char *>(symbol);
    // concurrent first calls on one device resolve the same address: a plain store is enough
    g_scratch_address[device].store(address, std::memory_order_release);
  }
  return address;
}

int32_t launch_validated(const FerruleHipMoeDecodeArgs &a);

// Who used the array last on each device: calls on ONE stream are ordered by the stream, calls on
// different streams are not, and the second would overwrite what the first still reads.  After every
// launch an event is recorded behind it; a call on another stream while that event has not completed is
// refused.  The event is created with the array's address, once per device; recording and querying it
// allocate nothing.  A capturing stream is left alone (an event query is not allowed there, and the
// order of a captured graph is its owner's business).
struct ScratchUse {
  std::mutex lock;
  hipEvent_t done = nullptr;
  uint64_t stream = 0;
  bool recorded = false;
};
ScratchUse g_scratch_use[kMaxDevices];

}  // namespace
}  // namespace ferrule_hip

extern "C" int32_t ferrule_hip_moe_decode_launch(const FerruleHipMoeDecodeArgs *args) {
  const int32_t status = validate(args);
  if (status != FERRULE_HIP_SUCCESS) return status;
  return launch_validated(*args);
}

extern "C" int32_t ferrule_hip_moe_decode_launch_static_workspace(const FerruleHipMoeDecodeArgs *args) {
  if (args == nullptr) return FERRULE_HIP_INVALID_ARGUMENT;
  // the caller's workspace fields are not used: they must be zero, so that a block meant
  // for the other entry point is not run on shared scratch by mistake
  if (args->workspace != 0 || args->workspace_bytes != 0) return FERRULE_HIP_INVALID_ARGUMENT;
  if (args->total_routed_rows == 0 || args->intermediate_size == 0 || args->num_tokens == 0 || args->input_size == 0)
    return FERRULE_HIP_INVALID_ARGUMENT;
  // sizes beyond the static array: FERRULE_HIP_UNSUPPORTED, before anything is looked up or launched
  if (workspace_layout(*args).total > FERRULE_HIP_MOE_DECODE_STATIC_WORKSPACE_BYTES) return FERRULE_HIP_UNSUPPORTED;
  unsigned char *address = scratch_address();
  if (address == nullptr) return FERRULE_HIP_LAUNCH_FAILED;
  FerruleHipMoeDecodeArgs with_scratch = *args;
  with_scratch.workspace = static_cast<uint64_t>(reinterpret_cast<uintptr_t>(address));
  with_scratch.workspace_bytes = FERRULE_HIP_MOE_DECODE_STATIC_WORKSPACE_BYTES;
  const int32_t status = validate(&with_scratch);
  if (status != FERRULE_HIP_SUCCESS) return status;
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return FERRULE_HIP_LAUNCH_FAILED;
  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(args->stream));
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capture) != hipSuccess) {
    (void)hipGetLastError();
    capture = hipStreamCaptureStatusNone;
  }
  if (capture != hipStreamCaptureStatusNone) return launch_validated(with_scratch);
  ScratchUse &use = g_scratch_use[device];
  std::lock_guard<std::mutex> guard(use.lock);
  if (use.done == nullptr && hipEventCreateWithFlags(&use.done, hipEventDisableTiming) != hipSuccess) {
    (void)hipGetLastError();
    use.done = nullptr;
    return FERRULE_HIP_LAUNCH_FAILED;
  }
  if (use.recorded && use.stream != args->stream) {
    const hipError_t state = hipEventQuery(use.done);
    if (state == hipErrorNotReady) {
      (void)hipGetLastError();
      return FERRULE_HIP_UNSUPPORTED;   // the array is still in use by a call on another stream
    }
  }
  const int32_t launched = launch_validated(with_scratch);
  if (launched == FERRULE_HIP_SUCCESS) {
    if (hipEventRecord(use.done, stream) == hipSuccess) {
      use.stream = args->stream;
      use.recorded = true;
    } else {
      (void)hipGetLastError();
    }
  }
  return launched;
}

namespace ferrule_hip {
namespace {

int32_t launch_validated(const FerruleHipMoeDecodeArgs &a) {
  MoeParams p;
  p.active_expert_slots = as_ptr<const int32_t>(a.active_expert_slots);
  p.expert_route_indptr = as_ptr<const int32_t>(a.expert_route_indptr);
  p.route_token_indices = as_ptr<const int32_t>(a.route_token_indices);
  p.route_indices = as_ptr<const int32_t>(a.route_indices);
  p.route_weights = as_ptr<const float>(a.route_weights);
  p.host_scalars = as_ptr<const int32_t>(a.host_scalars);
  p.gate_ptrs = as_ptr<const uint64_t>(a.gate_ptrs);
  p.gate_scale_ptrs = as_ptr<const uint64_t>(a.gate_scale_ptrs);
  p.up_ptrs = as_ptr<const uint64_t>(a.up_ptrs);
  p.up_scale_ptrs = as_ptr<const uint64_t>(a.up_scale_ptrs);
  p.down_ptrs = as_ptr<const uint64_t>(a.down_ptrs);
  p.down_scale_ptrs = as_ptr<const uint64_t>(a.down_scale_ptrs);
  p.input = as_ptr<const uint16_t>(a.input_bf16);
  p.route_output = as_ptr<float>(a.route_output);
  p.route_written = as_ptr<int32_t>(a.route_written);
  p.route_error = as_ptr<int32_t>(a.route_error);
  p.prefix = (a.flags & FERRULE_HIP_MOE_DECODE_PREFIX_F32) ? as_ptr<const float>(a.prefix_f32) : nullptr;
  p.output = as_ptr<uint16_t>(a.output);
  const WorkspaceLayout ws = workspace_layout(a);
  p.xq = as_ptr<uint8_t>(a.workspace + ws.xq);
  p.xs = as_ptr<uint8_t>(a.workspace + ws.xs);
  p.hidden = as_ptr<float>(a.workspace + ws.hidden);
  p.hq = as_ptr<uint8_t>(a.workspace + ws.hq);
  p.hs = as_ptr<uint8_t>(a.workspace + ws.hs);
  p.row_capacity = a.total_routed_rows;
  p.active_group_count = a.active_group_count;
  p.slot_capacity = a.slot_capacity;
  p.num_tokens = a.num_tokens;
  p.num_routes = a.num_routes;
  p.routes_per_token = a.routes_per_token;
  p.input_size = a.input_size;
  p.intermediate_size = a.intermediate_size;
  p.hidden_size = a.hidden_size;
  p.flags = a.flags;
  p.swiglu_limit = a.swiglu_limit;
  // sparse routes: at most kSparseRowsPerGroup rows per expert group on average.  Measured with uniform
  // routes over 256 experts (packed kernels only / packed + general): 128 tokens (4.1 rows per group) 0.935 /
  // 1.005 ms, 160 tokens (5.0) 1.013 / 1.034 ms, 192 tokens (6.0) 1.160 / 1.141 ms, 256 tokens (8.0) 1.391 / 1.296 ms.
  constexpr uint64_t kSparseRowsPerGroup = 5;
  p.packed_only = static_cast<uint64_t>(a.num_routes) <= kSparseRowsPerGroup * a.active_group_count ? 1u : 0u;

  constexpr int kGateTilesPerWave = 2;
  constexpr int kDownTilesPerWave = 16;
  const PackedItems gate_items = packed_items(a.active_group_count, a.intermediate_size / 16u, kGateTilesPerWave, 1u);
  const PackedItems down_items = packed_items(a.active_group_count, a.hidden_size / 16u, kDownTilesPerWave, 2u);
  p.gate_tpw = gate_items.full;
  p.gate_tpw_tail = gate_items.tail;
  p.down_tpw = down_items.full;
  p.down_tpw_tail = down_items.tail;

  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(a.stream));
  clear_launch_error();
  if (!(a.flags & FERRULE_HIP_MOE_DECODE_SKIP_GATE_UP)) {
    // input -> MX terms (tokens * H/32 blocks), then the gate/up stream
    const uint64_t blocks = static_cast<uint64_t>(a.num_tokens) * (a.input_size / 32u);
    mx_split_kernel<uint16_t, kTermsX><<<static_cast<uint32_t>((blocks * 4u + 255u) / 256u), 256, 0, stream>>>(
        p.input, p.xq, p.xs, a.num_tokens, a.num_tokens, a.input_size);
    // the general kernel is launched for dense routes only, where most experts have work for it
    constexpr int kGateGeneralTilesPerWave = kGateTilesPerWave;
    const uint32_t per_general_wg = kWaves * gate_items.full;
    const uint32_t gate_packed_grid = gate_items.grid;
    const dim3 gate_general_grid((a.intermediate_size / 16u + per_general_wg - 1u) / per_general_wg,
                                 a.active_group_count);
    // general token tiles first (the long ones), then the packed ones; see tile_is_packed
    constexpr bool kGateHasGeneral = kTermsX * kTokenTile > 16u * kGatePasses;
    if (a.flags & FERRULE_HIP_MOE_DECODE_BLOCK_MAJOR_WEIGHTS) {
      if (kGateHasGeneral && !p.packed_only) {
        moe_gate_up_kernel<4, kGateGeneralTilesPerWave, true, false><<<gate_general_grid, kThreads, 0, stream>>>(p);
      }
      moe_gate_up_kernel<4, kGateTilesPerWave, true, true><<<gate_packed_grid, kThreads, 0, stream>>>(p);
    } else {
      if (kGateHasGeneral && !p.packed_only) {
        moe_gate_up_kernel<4, kGateGeneralTilesPerWave, false, false><<<gate_general_grid, kThreads, 0, stream>>>(p);
      }
      moe_gate_up_kernel<4, kGateTilesPerWave, false, true><<<gate_packed_grid, kThreads, 0, stream>>>(p);
    }
  }
  if (!(a.flags & FERRULE_HIP_MOE_DECODE_SKIP_DOWN)) {
    // h -> MX terms over the rows this batch can have routed (one per route; rows beyond the
    // plan's last group, if some routes were dropped, hold stale values that nobody reads back)
    const uint32_t split_rows = a.num_routes < a.total_routed_rows ? a.num_routes : a.total_routed_rows;
    const uint64_t blocks = static_cast<uint64_t>(split_rows) * (a.intermediate_size / 32u);
    mx_split_kernel<float, kTermsH><<<static_cast<uint32_t>((blocks * 4u + 255u) / 256u), 256, 0, stream>>>(
        p.hidden, p.hq, p.hs, split_rows, a.total_routed_rows, a.intermediate_size);
    constexpr int kDownGeneralTilesPerWave = kDownTilesPerWave;
    const uint32_t per_general_wg = kWaves * down_items.full;
    const dim3 down_general_grid((a.hidden_size / 16u + per_general_wg - 1u) / per_general_wg, a.active_group_count);
    const uint32_t down_packed_grid = down_items.grid;
    if (a.flags & FERRULE_HIP_MOE_DECODE_BLOCK_MAJOR_WEIGHTS) {
      if (!p.packed_only) {
        moe_down_kernel<4, kDownGeneralTilesPerWave, true, false><<<down_general_grid, kThreads, 0, stream>>>(p);
      }
      moe_down_kernel<4, kDownTilesPerWave, true, true><<<down_packed_grid, kThreads, 0, stream>>>(p);
    } else {
      if (!p.packed_only) {
        moe_down_kernel<4, kDownGeneralTilesPerWave, false, false><<<down_general_grid, kThreads, 0, stream>>>(p);
      }
      moe_down_kernel<4, kDownTilesPerWave, false, true><<<down_packed_grid, kThreads, 0, stream>>>(p);
    }
  }
  if (a.flags & FERRULE_HIP_MOE_DECODE_COMBINE) {
    const uint64_t total = static_cast<uint64_t>(a.num_tokens) * (a.hidden_size / 4u);
    moe_combine_kernel<<<static_cast<uint32_t>((total + 255u) / 256u), 256, 0, stream>>>(p);
  }
  return take_launch_error() == hipSuccess ? FERRULE_HIP_SUCCESS : FERRULE_HIP_LAUNCH_FAILED;
}

}  // namespace
}  // namespace ferrule_hip

// Diagnostic: the layer's activation split on its own (ferrule_hip_diagnostics.h).
extern "C" int32_t ferrule_hip_mx_split_launch(const FerruleHipMxSplitArgs *args) {
  using namespace ferrule_hip;
  if (args == nullptr || args->rows == 0 || args->k == 0 || (args->k % 32u) != 0 || args->input_kind > 1u ||
      args->reserved != 0 || args->input == 0 || args->q == 0 || args->s == 0 || (args->input % 16u) != 0 ||
      (args->q % 8u) != 0) {
    return FERRULE_HIP_INVALID_ARGUMENT;
  }
  hipStream_t stream = reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(args->stream));
  const uint64_t blocks = static_cast<uint64_t>(args->rows) * (args->k / 32u);
  const uint32_t grid = static_cast<uint32_t>((blocks * 4u + 255u) / 256u);
  clear_launch_error();
  if (args->input_kind == 0u) {
    mx_split_kernel<uint16_t, kTermsX><<<grid, 256, 0, stream>>>(as_ptr<const uint16_t>(args->input), as_ptr<uint8_t>(args->q),
                                                                 as_ptr<uint8_t>(args->s), args->rows, args->rows, args->k);
  } else {
    mx_split_kernel<float, kTermsH><<<grid, 256, 0, stream>>>(as_ptr<const float>(args->input), as_ptr<uint8_t>(args->q),
                                                              as_ptr<uint8_t>(args->s), args->rows, args->rows, args->k);
  }
  return take_launch_error() == hipSuccess ? FERRULE_HIP_SUCCESS : FERRULE_HIP_LAUNCH_FAILED;
}
