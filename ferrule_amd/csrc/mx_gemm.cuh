// Tiled GEMM core on the gfx950 scaled MFMA (v_mfma_scale_f32_16x16x128_f8f6f4):
//     Y[token, feature] = sum_k X[token, k] * W[feature, k]
// X is MX-FP8 (E4M3 bytes, one E8M0 scale per row and 128-wide K block), W is FP8 (E4M3, one
// scale per 128x128 block) or MXFP4 (E2M1 nibbles, one E8M0 scale per row and 32 k).  Both
// operands are K-major, so a weight row fragment is the MFMA's A operand and a token row
// fragment its B operand; accumulator register v of lane (i, g) is (feature 4g+v, token i),
// i.e. each lane ends up with four consecutive features of one token.
//
// One workgroup owns FN features x TM tokens (per weight matrix; up to NMAT matrices share
// the token fragments, e.g. gate and up).  Its waves form a WAVES_F x WAVES_T grid, each wave
// holds NF x NT accumulator tiles.  K advances 128 per step through an NSTAGE-deep ring of
// LDS stages that are filled with direct global->LDS loads (no VGPR staging): every wave
// issues the same number of loads per stage, so "stage s has landed" is an in-order vmcnt
// wait of the wave followed by one workgroup barrier, and the barrier also proves that the
// stage about to be refilled has been left by everybody.
//
// LDS layout of a stage: X rows of 128 bytes, then weight rows of 128 (FP8) or 64 (FP4)
// bytes, then for FP4 the rows' four scale bytes.  LDS has 32 banks of 4 bytes, a ds_read_b128
// is served 8 lanes (128 bytes) per clock, and the 8 lanes of a phase read the same 16-byte
// piece of 8 consecutive rows - which all start at bank 0.  16-byte pieces are therefore
// XOR-swizzled with the row index so that those 8 lanes hit 8 different bank groups:
//   128-byte rows: piece p of row r sits at slot p ^ (r & 7)
//    64-byte rows: piece p of row r sits at slot p ^ ((r >> 1) & 3)   (two rows per 128 bytes)
// (with the pairs-of-rows swizzle of a 64-bank layout the reads ran at half rate: measured,
// the K step was bound by LDS at ~64 B/clk)
// The swizzle costs nothing: a direct-to-LDS load writes lane l at base + 16*l, so it is
// applied to the lane's SOURCE address instead.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mx_core.cuh"
#include "numeric.cuh"
#include "skinny_core.cuh"

namespace ferrule_hip {

template <int WFMT_, int NMAT_, int NF_, int NT_, int WAVES_F_, int WAVES_T_, int NSTAGE_, bool SPREAD_T_ = false>
struct GemmShape {
  static constexpr int WFMT = WFMT_, NMAT = NMAT_, NF = NF_, NT = NT_;
  static constexpr int WAVES_F = WAVES_F_, WAVES_T = WAVES_T_, NSTAGE = NSTAGE_;
  // Which 16-row token fragments of the tile a wave of token-wave index wt owns: NT consecutive
  // ones, or (SPREAD_T) every WAVES_T-th one.  A ragged tile (grouped GEMMs: the last tile of an
  // expert) has its dead rows at the end; spread over the waves, every wave - and every SIMD -
  // loses about the same number of fragments, and the K step gets shorter for all of them.
  static constexpr bool SPREAD_T = SPREAD_T_;
  __host__ __device__ static constexpr uint32_t token_row(uint32_t wt, int t) {
    return SPREAD_T ? (static_cast<uint32_t>(t) * WAVES_T + wt) * 16u : (wt * NT + static_cast<uint32_t>(t)) * 16u;
  }
  // fragments of wave wt that hold at least one of the tile's m rows (they are its first ones)
  __host__ __device__ static constexpr uint32_t live_fragments(uint32_t wt, uint32_t m) {
    uint32_t n = 0;
    for (int t = 0; t < NT; ++t) n += token_row(wt, t) < m ? 1u : 0u;
    return n;
  }
  static constexpr bool kFp4W = WFMT == kMfmaFmtFp4;
  static constexpr int kWaves = WAVES_F * WAVES_T;
  static constexpr int kThreads = kWaves * 64;
  static constexpr int FN = WAVES_F * NF * 16;  // features per workgroup and matrix
  static constexpr int TM = WAVES_T * NT * 16;  // tokens per workgroup
  static constexpr int kWRow = kFp4W ? 64 : 128;  // bytes of a weight row per K step
  static constexpr int kWPieces = kWRow / 16;
  static constexpr int kXBytes = TM * 128;
  static constexpr int kWBytes = NMAT * FN * kWRow;
  static constexpr int kSBytes = kFp4W ? NMAT * FN * 4 : 0;
  static constexpr int kStageBytes = kXBytes + kWBytes + kSBytes;
  // wave-wide load instructions per stage, by region
  static constexpr int kXInstr = kXBytes / 1024;
  static constexpr int kWInstr = kWBytes / 1024;
  static constexpr int kSInstr = kSBytes / 256;
  static_assert(kXInstr % kWaves == 0 && kWInstr % kWaves == 0 && kSInstr % kWaves == 0,
                "every wave issues the same loads per stage");
  static constexpr int kXSlots = kXInstr / kWaves;
  static constexpr int kWSlots = kWInstr / kWaves;
  static constexpr int kSSlots = kSInstr / kWaves;
  static constexpr int kSlots = kXSlots + kWSlots + kSSlots;  // loads per wave and stage
  static_assert((NSTAGE - 1) * kSlots <= 48, "vmcnt is a 6-bit counter");
  static_assert(NF * 16 <= 128, "a wave's features stay inside one 128-row scale block");
};

// What the core needs to know about the operands.  Row resolvers return the byte offset of a
// row from the operand's base, already clamped to a valid row.
template <int NMAT>
struct GemmOperands {
  const uint8_t *x;            // E4M3 rows
  const uint8_t *w[NMAT];      // weight rows
  const uint8_t *wscale[NMAT]; // FP4: [n, k/32] row scales; FP8: unused by the core
  uint32_t k;                  // multiple of 128
};

// Sources of the wave's loads for one stage.  A load's address is a wave-uniform base (scalar
// registers; one per operand region, moved on by a constant per K step on the scalar unit) plus
// this lane's 32-bit offset, which stays what it is for the whole K loop: the K loop spends no
// vector instruction and no 64-bit vector register on addresses.
template <typename S>
struct GemmCursors {
  uint32_t off[S::kSlots];       // lane offsets from the slot's region base
  const uint8_t *x;              // region bases after `steps` K steps: token rows,
  const uint8_t *w[S::NMAT];     //   weight rows per matrix,
  const uint8_t *s[S::NMAT];     //   MXFP4 scale bytes per matrix
  uint32_t steps;
  // bytes from one K step to the next of a weight row's payload and of its scale bytes: the row
  // pitch pieces of the checkpoint order (kWRow, 4), or 1024 and 64 for MXFP4 weights in the
  // block-major order, where the 16 rows of a tile lie side by side inside every K block
  uint32_t w_step, s_step;
};

// Matrix of the wave's load number i of the weight (or scale) region: a wave instruction covers
// 64 / kWPieces weight rows (64 scale rows), which never straddle two matrices.
template <typename S>
__device__ __forceinline__ uint32_t gemm_slot_matrix(uint32_t wave, int i, bool scale_region) {
  static_assert(S::FN % (64 / S::kWPieces) == 0 && S::FN % 64 == 0, "one matrix per wave load");
  const uint32_t first_row = (i * S::kWaves + wave) * 64u / (scale_region ? 1u : S::kWPieces);
  return S::NMAT == 1 ? 0u : first_row / S::FN;
}

// xrow(r) / wrow(mat, r): byte offset of workgroup-local row r's first k from op.x / op.w[mat]
// (clamped rows for r beyond the problem); srow(mat, r): offset of its scale bytes from
// op.wscale[mat].  Offsets are 32-bit: a caller whose operand is larger than 4 GiB points the
// operand at its tile's first row and returns offsets from there.
template <typename S, typename XRow, typename WRow, typename SRow>
__device__ __forceinline__ void gemm_init_cursors(GemmCursors<S> &c, const GemmOperands<S::NMAT> &op,
                                                  uint32_t wave, uint32_t lane, XRow xrow, WRow wrow,
                                                  SRow srow) {
#pragma unroll
  for (int i = 0; i < S::kXSlots; ++i) {
    const uint32_t q = (i * S::kWaves + wave) * 64u + lane;  // 16-byte slot of the X region
    const uint32_t row = q >> 3, slot = q & 7u;
    const uint32_t piece = slot ^ (row & 7u);
    c.off[i] = static_cast<uint32_t>(xrow(row)) + piece * 16u;
  }
#pragma unroll
  for (int i = 0; i < S::kWSlots; ++i) {
    const uint32_t q = (i * S::kWaves + wave) * 64u + lane;
    const uint32_t row = q / S::kWPieces, slot = q % S::kWPieces;
    const uint32_t piece = S::kFp4W ? slot ^ ((row >> 1) & 3u) : slot ^ (row & 7u);
    c.off[S::kXSlots + i] = static_cast<uint32_t>(wrow(gemm_slot_matrix<S>(wave, i, false), row % S::FN)) + piece * 16u;
  }
#pragma unroll
  for (int i = 0; i < S::kSSlots; ++i) {
    const uint32_t row = (i * S::kWaves + wave) * 64u + lane;
    c.off[S::kXSlots + S::kWSlots + i] = static_cast<uint32_t>(srow(gemm_slot_matrix<S>(wave, i, true), row % S::FN));
  }
  c.x = op.x;
#pragma unroll
  for (int m = 0; m < S::NMAT; ++m) {
    c.w[m] = op.w[m];
    c.s[m] = op.wscale[m];
  }
  c.steps = 0;
  c.w_step = S::kWRow;
  c.s_step = 4u;
}

// Load number i (0 .. kSlots-1) of this wave for one stage; i is a compile-time constant at every
// call site (unrolled loops), so the region tests fold away.  `live` = false where there is
// nothing (left) to prefetch - the last NSTAGE-1 K steps, or prologue stages beyond a short K:
// the load is issued all the same, from the region's first K block into a stage nobody reads.  A
// branch around it would cut the K step into basic blocks, and the hand-placed order of reads,
// MFMAs and loads (sched_barrier works inside a block) would be lost: the compiler then hoists
// every read and load of the step to its top.  It also makes the wait count of a step a constant.
template <typename S>
__device__ __forceinline__ void gemm_issue_slot(const GemmCursors<S> &c, uint8_t *stage, uint32_t wave, int i,
                                                bool live) {
  if (i < S::kXSlots) {
    const uint8_t *from = live ? c.x : c.x - static_cast<size_t>(c.steps) * 128u;
    lds_dma16(from, c.off[i], stage + (i * S::kWaves + wave) * 1024u);
  } else if (i < S::kXSlots + S::kWSlots) {
    const int j = i - S::kXSlots;
    const uint8_t *base = c.w[0];
#pragma unroll
    for (int m = 1; m < S::NMAT; ++m) base = gemm_slot_matrix<S>(wave, j, false) == static_cast<uint32_t>(m) ? c.w[m] : base;
    const uint8_t *from = live ? base : base - static_cast<size_t>(c.steps) * c.w_step;
    lds_dma16(from, c.off[i], stage + S::kXBytes + (j * S::kWaves + wave) * 1024u);
  } else {
    const int j = i - S::kXSlots - S::kWSlots;
    const uint8_t *base = c.s[0];
#pragma unroll
    for (int m = 1; m < S::NMAT; ++m) base = gemm_slot_matrix<S>(wave, j, true) == static_cast<uint32_t>(m) ? c.s[m] : base;
    const uint8_t *from = live ? base : base - static_cast<size_t>(c.steps) * c.s_step;
    lds_dma4(from, c.off[i], stage + S::kXBytes + S::kWBytes + (j * S::kWaves + wave) * 256u);
  }
}

// The bases move on by one K step: after a stage's live loads have all been issued.
template <typename S>
__device__ __forceinline__ void gemm_advance(GemmCursors<S> &c) {
  c.x += 128;
#pragma unroll
  for (int m = 0; m < S::NMAT; ++m) {
    c.w[m] += c.w_step;
    if (S::kFp4W) c.s[m] += c.s_step;
  }
  ++c.steps;
}

// Back to the first K block.
template <typename S>
__device__ __forceinline__ void gemm_rewind(GemmCursors<S> &c) {
  c.x -= static_cast<size_t>(c.steps) * 128u;
#pragma unroll
  for (int m = 0; m < S::NMAT; ++m) {
    c.w[m] -= static_cast<size_t>(c.steps) * c.w_step;
    if (S::kFp4W) c.s[m] -= static_cast<size_t>(c.steps) * c.s_step;
  }
  c.steps = 0;
}

template <typename S>
__device__ __forceinline__ void gemm_issue_stage(GemmCursors<S> &c, uint8_t *stage, uint32_t wave, bool live) {
#pragma unroll
  for (int i = 0; i < S::kSlots; ++i) gemm_issue_slot<S>(c, stage, wave, i, live);
  if (live) gemm_advance<S>(c);
}

// One weight scale per (wave, K block) for FP8 weights: `Byte` = an E8M0 byte folded into the
// MFMA, `Float` = an f32 factor applied to the K block's partial sums on the VALU.
enum class WScaleMode { PerRow32 /* FP4 */, Byte, Float };

// The first NSTAGE-1 stages of the ring.  gemm_mainloop issues them itself unless told that the
// caller already has (PROLOGUE_ISSUED): a kernel with set-up work of its own between the cursor
// initialisation and the K loop issues them first and does that work under their latency.
template <typename S>
__device__ __forceinline__ void gemm_prologue(GemmCursors<S> &cur, uint8_t *stages, uint32_t nk, uint32_t wave) {
#pragma unroll
  for (int s = 0; s < S::NSTAGE - 1; ++s) {
    gemm_issue_stage<S>(cur, stages + s * S::kStageBytes, wave, static_cast<uint32_t>(s) < nk);
  }
}

// K loops of a persistent workgroup run as ONE sequence of steps over its items: the stage ring
// keeps turning, and the last NSTAGE-1 steps of an item, which have nothing of their own left to
// fetch, fetch the first NSTAGE-1 stages of the next item instead.  When the loop returns, these
// have landed (this wave's share: it has waited for them); the next loop starts without a
// prologue and without waiting in its first NSTAGE-1 steps, so that what the caller stores in
// between (an item's results) drains under them.  nk >= NSTAGE-1 for every item.
template <typename S>
struct GemmChain {
  uint32_t buf, fill;     // ring position: the stage of the next K step and the stage of the next refill
  GemmCursors<S> *next;   // sources of the next item's first stages; with no next item, any cursors
                          // whose loads are harmless (their data lands in stages nobody reads)
};

struct GemmNoHook {
  __device__ __forceinline__ void operator()(uint32_t) const {}
};

// Accumulate all K steps.  x_scale(t, kb) -> scale byte of this lane's token in token tile t;
// w_block_scale(mat, kb) -> uint32_t byte (Byte) or float bits (Float) for this wave.
// NT_LIVE < S::NT: only the wave's first NT_LIVE token fragments are read and multiplied (the rest
// lie beyond a ragged tile's rows; their accumulators stay as they are).  The loads, waits and
// barriers of a K step are the same for every NT_LIVE, so waves of one workgroup may differ.
// CHAINED: see GemmChain.  at_step(s) runs at the top of K step s, behind its barrier (wave-uniform
// work of the caller that must not cut a K step in two).
// STAGGER (three stages or more, not chained): 0 = every wave of the workgroup runs the same K step
// at the same time.  1 / 2 = the loop of the first / second half of the waves (waves w and
// w + kWaves/2 share a SIMD): a second barrier sits in the middle of every K step and the second
// half runs half a step behind the first, so that while one wave of a SIMD stands at the top of a
// step (barrier, first fragment reads) the other is in the middle of its MFMAs.  A stage is then
// left by everybody half a step later; the first group issues its refill loads in the second half
// of its steps and the second group in the first half of its own (the same half step for both), and
// the refill still has more than a K step to land.  Every wave waits for its loads before each
// barrier; both halves pass the same number of barriers (one more before the second half's loop,
// one more behind the first half's).  The caller branches on the wave once and calls one of the two.
template <typename S, WScaleMode MODE, bool PROLOGUE_ISSUED = false, int NT_LIVE = S::NT, bool CHAINED = false,
          int STAGGER = 0, typename XScale, typename WBlockScale, typename AtStep = GemmNoHook>
__device__ __forceinline__ void gemm_mainloop(f32x4_t (&acc)[S::NMAT][S::NF][S::NT], GemmCursors<S> &cur,
                                              uint8_t *stages, uint32_t nk, uint32_t wave, uint32_t lane,
                                              XScale x_scale, WBlockScale w_block_scale,
                                              GemmChain<S> *chain = nullptr, AtStep at_step = AtStep{}) {
  static_assert(!CHAINED || PROLOGUE_ISSUED, "a chained loop finds its first stages in place");
  static_assert(STAGGER == 0 || (S::NSTAGE >= 3 && !CHAINED && STAGGER <= 2), "a staggered loop needs three stages");
  const uint32_t i = lane & 15u, g = lane >> 4;
  const uint32_t wf = wave % S::WAVES_F, wt = wave / S::WAVES_F;
  // This lane's fragment addresses inside a stage: one lane-dependent offset per region plus
  // compile-time constants (16-row steps keep the swizzle term of a row what it is), so they cost
  // three or four registers and the reads carry the constants as immediate offsets.
  const uint32_t x_row = S::token_row(wt, 0) + i;
  const uint32_t x_lo0 = x_row * 128u + ((g ^ (x_row & 7u)) << 4);
  const uint32_t x_hi0 = x_row * 128u + (((4u + g) ^ (x_row & 7u)) << 4);
  const uint32_t w_row = wf * S::NF * 16u + i;
  const uint32_t w_lo0 = S::kFp4W ? S::kXBytes + w_row * 64u + ((g ^ ((w_row >> 1) & 3u)) << 4)
                                  : S::kXBytes + w_row * 128u + ((g ^ (w_row & 7u)) << 4);
  const uint32_t w_hi0 = S::kXBytes + w_row * 128u + (((4u + g) ^ (w_row & 7u)) << 4);   // FP8 only
  const uint32_t w_sc0 = S::kXBytes + S::kWBytes + w_row * 4u + g;                       // FP4 only
  auto x_const = [](int t) { return (S::token_row(0, t) - S::token_row(0, 0)) * 128u; };
  auto w_const = [](int m, int f) { return static_cast<uint32_t>(m * S::FN + f * 16) * (S::kFp4W ? 64u : 128u); };
  auto s_const = [](int m, int f) { return static_cast<uint32_t>(m * S::FN + f * 16) * 4u; };

  // prologue: NSTAGE-1 stages in flight
  if constexpr (!PROLOGUE_ISSUED) gemm_prologue<S>(cur, stages, nk, wave);
  uint32_t buf = 0, fill = S::NSTAGE - 1;
  if constexpr (CHAINED) {
    buf = chain->buf;
    fill = chain->fill;
  }
  static_assert(NT_LIVE >= 1 && NT_LIVE <= S::NT, "at least one live fragment (else gemm_mainloop_idle)");
  if constexpr (STAGGER == 2) {   // half a K step behind the first group from here on
    wait_vmcnt((S::NSTAGE - 2) * S::kSlots);  // this wave's share of the first stage, which the first group reads now
    stage_barrier();
  }
  uint32_t sx_ahead[NT_LIVE];
#pragma unroll
  for (int t = 0; t < NT_LIVE; ++t) sx_ahead[t] = x_scale(t, 0u);
  // the first weight block scale of a K step is fetched a step ahead as well: the step's first MFMA
  // takes it as an operand (Byte), and a read at the top of the step would put its latency there
  uint32_t ws_ahead = 0;
  if constexpr (MODE != WScaleMode::PerRow32) ws_ahead = w_block_scale(0, 0u);
  // pending partial sums of the Float mode (see `fold` below)
  constexpr int kFoldLag = 2;
  f32x4_t part[kFoldLag];
  uint32_t part_scale[kFoldLag];
#pragma unroll
  for (int j = 0; j < kFoldLag; ++j) {
    part[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    part_scale[j] = 0u;
  }
  // One K step; its refill loads come from `from` (`refill` false: from where nobody reads them).
  auto k_step = [&](const uint32_t s, GemmCursors<S> &from, const bool refill) {
    // every K step issues its kSlots loads (see gemm_issue_slot): NSTAGE-2 younger steps' worth
    // may stay in flight.  The first stages of a chained loop landed before it began; the count
    // may also hold stores of the previous item, which a wait would sit out.
    if (!CHAINED || s >= static_cast<uint32_t>(S::NSTAGE - 1)) wait_vmcnt((S::NSTAGE - 2) * S::kSlots);
    stage_barrier();
    at_step(s);
    // The refill of the stage that everybody has just left is not issued here in one burst: a
    // wave cannot issue anything else while its loads queue up in the memory pipeline, and the
    // matrix pipe would idle for the length of the burst.  The loads are spread evenly over the K
    // step's MFMAs instead.
    uint8_t *const fill_stage = stages + fill * S::kStageBytes;
    fill = fill + 1u == S::NSTAGE ? 0u : fill + 1u;
    const uint8_t *st = stages + buf * S::kStageBytes;
    buf = buf + 1u == S::NSTAGE ? 0u : buf + 1u;

    // Fragment reads are software-pipelined by hand in the first feature row: the first MFMA
    // needs one weight and one token fragment only, and each following one its own token
    // fragment, read kLookahead MFMAs earlier.  Left to itself the scheduler hoists all reads
    // of the K step to its top and waits for the last of them, which idles the matrix pipe
    // for the whole burst (all waves of the workgroup read at the same time after the barrier).
    constexpr int kLookahead = 3;
    i32x8_t xb[NT_LIVE];
    uint32_t sx[NT_LIVE];
    auto read_x = [&](int t) {
      xb[t] = make_b_fp8(*reinterpret_cast<const u32x4_t *>(st + x_lo0 + x_const(t)),
                         *reinterpret_cast<const u32x4_t *>(st + x_hi0 + x_const(t)));
    };
    auto read_w = [&](int m, int f, i32x8_t &wa, uint32_t &sw, uint32_t wsc) {
      if constexpr (S::kFp4W) {
        wa = make_a_fp4(*reinterpret_cast<const u32x4_t *>(st + w_lo0 + w_const(m, f)));
        sw = (st + w_sc0)[s_const(m, f)];
      } else {
        wa = make_b_fp8(*reinterpret_cast<const u32x4_t *>(st + w_lo0 + w_const(m, f)),
                        *reinterpret_cast<const u32x4_t *>(st + w_hi0 + w_const(m, f)));
        sw = MODE == WScaleMode::Byte ? wsc : 127u;
      }
    };
    // Float scales: the K block's partial sums of MFMA j land in slot j % kFoldLag of `part` (C = 0)
    // and are folded into the running sums, one v_fma each, when the slot is needed again kFoldLag
    // MFMAs later (for the last ones that is in the next K step; the slots start as zeros).  A fold
    // right behind its own MFMA makes the wave sit out the instruction's whole latency before every
    // fold, and the matrix pipe with it.
    auto fold = [&](int j) {   // MFMA number j of a K step (row j / NT_LIVE, token fragment j % NT_LIVE)
      const int r = j / NT_LIVE, t = j % NT_LIVE;
      const float ws = __uint_as_float(part_scale[j % kFoldLag]);
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        acc[r / S::NF][r % S::NF][t][v] = fmaf(part[j % kFoldLag][v], ws, acc[r / S::NF][r % S::NF][t][v]);
      }
    };
    auto mma = [&](int m, int f, int t, const i32x8_t &wa, uint32_t sw, uint32_t wsc) {
      if constexpr (MODE == WScaleMode::Float) {
        constexpr int kStepMmas = S::NMAT * S::NF * NT_LIVE;
        static_assert(kStepMmas % kFoldLag == 0, "a slot's tenants are kFoldLag MFMAs apart across K steps too");
        const int j = (m * S::NF + f) * NT_LIVE + t;
        const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
        const f32x4_t fresh = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
            wa, xb[t], zero, S::WFMT, kMfmaFmtFp8, 0, static_cast<int>(sw), 0, static_cast<int>(sx[t]));
        __builtin_amdgcn_sched_barrier(0);   // the fold stays behind the MFMA just issued
        fold((j + kStepMmas - kFoldLag) % kStepMmas);
        part[j % kFoldLag] = fresh;
        part_scale[j % kFoldLag] = wsc;
      } else {
        acc[m][f][t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
            wa, xb[t], acc[m][f][t], S::WFMT, kMfmaFmtFp8, 0, static_cast<int>(sw), 0, static_cast<int>(sx[t]));
      }
    };
    // token scales do not live in the stage: those of the next K step are fetched now
    uint32_t sx_next[NT_LIVE];
    const uint32_t s_next = s + 1u < nk ? s + 1u : s;
#pragma unroll
    for (int t = 0; t < NT_LIVE; ++t) sx[t] = sx_ahead[t];
    constexpr int kRows = S::NMAT * S::NF;
    constexpr int kMmas = kRows * NT_LIVE;
    i32x8_t wa[2];
    uint32_t sw[2], wsc[2] = {0u, 0u};
    if constexpr (MODE != WScaleMode::PerRow32) wsc[0] = ws_ahead;
    read_w(0, 0, wa[0], sw[0], wsc[0]);
#pragma unroll
    for (int t = 0; t < kLookahead && t < NT_LIVE; ++t) read_x(t);
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      const int m = r / S::NF, f = r % S::NF;
#pragma unroll
      for (int t = 0; t < NT_LIVE; ++t) {
        __builtin_amdgcn_sched_barrier(0);
        if (r == 0 && t + kLookahead < NT_LIVE) read_x(t + kLookahead);
        if (t == (NT_LIVE > 2 ? NT_LIVE / 2 - 1 : 0) && r + 1 < kRows) {  // next row's weights, half a row ahead
          const int m1 = (r + 1) / S::NF, f1 = (r + 1) % S::NF;
          if constexpr (MODE != WScaleMode::PerRow32) wsc[(r + 1) & 1] = f1 == 0 ? w_block_scale(m1, s) : wsc[r & 1];
          read_w(m1, f1, wa[(r + 1) & 1], sw[(r + 1) & 1], wsc[(r + 1) & 1]);
        }
        mma(m, f, t, wa[r & 1], sw[r & 1], wsc[r & 1]);
        // refill load `slot` follows MFMA slot * kSpan / kSlots; in a staggered loop all of them lie in the
        // half of the step in which the stage they fill has been left by both groups.  With two stages a
        // load has only what is left of its own K step to land, so the loads go out in the first half of
        // the step: spread over the whole step the last of them were waited for at the top of the next
        // one (256 x 256 tile, M=4096 N=18432: 474 -> 445 us with f32 scales, 470 -> 457 us with E8M0;
        // M=8192: 968 -> 902 us; a quarter of the step: 460 us).  With three stages the position does not
        // matter (grouped kernels: 2.98-3.00 ms for every span).
        const int j = r * NT_LIVE + t;
        constexpr int kSpan = (STAGGER != 0 || S::NSTAGE == 2) ? kMmas / 2 : kMmas;
        constexpr int kFirst = STAGGER == 1 ? kMmas / 2 : 0;
#pragma unroll
        for (int slot = 0; slot < S::kSlots; ++slot) {
          if (kFirst + slot * kSpan / S::kSlots == j) gemm_issue_slot<S>(from, fill_stage, wave, slot, refill);
        }
        if constexpr (STAGGER != 0) {
          if (j == kMmas / 2 - 1) {   // the other group's K step begins or ends here
            wait_vmcnt((S::NSTAGE - 2) * S::kSlots);
            stage_barrier();
          }
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (refill) gemm_advance<S>(from);
#pragma unroll
    for (int t = 0; t < NT_LIVE; ++t) sx_next[t] = x_scale(t, s_next);
    if constexpr (MODE != WScaleMode::PerRow32) ws_ahead = w_block_scale(0, s_next);
#pragma unroll
    for (int t = 0; t < NT_LIVE; ++t) sx_ahead[t] = sx_next[t];
  };
  // the last steps have nothing of this item left to fetch
  const uint32_t tail = min(nk, static_cast<uint32_t>(S::NSTAGE - 1));
  uint32_t s = 0;
  for (; s + tail < nk; ++s) k_step(s, cur, true);
  if constexpr (CHAINED) {
    for (; s < nk; ++s) k_step(s, *chain->next, true);
  } else {
    for (; s < nk; ++s) k_step(s, cur, false);
  }
  if constexpr (MODE == WScaleMode::Float) {   // the last K step's last partial sums
    constexpr int kStepMmas = S::NMAT * S::NF * NT_LIVE;
#pragma unroll
    for (int j = kStepMmas - kFoldLag; j < kStepMmas; ++j) {
      const int r = j / NT_LIVE, t = j % NT_LIVE;
      const float ws = __uint_as_float(part_scale[j % kFoldLag]);
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        acc[r / S::NF][r % S::NF][t][v] = fmaf(part[j % kFoldLag][v], ws, acc[r / S::NF][r % S::NF][t][v]);
      }
    }
  }
  if constexpr (CHAINED) {
    chain->buf = buf;
    chain->fill = fill;
    wait_vmcnt(0);  // this wave's share of the next item's first stages (the next barrier publishes them)
  } else {
    if constexpr (STAGGER == 1) stage_barrier();  // the second group's last half step
    lds_barrier();  // nobody reads the stages any more (the caller may reuse the LDS)
  }
}

// The K loop of a wave none of whose token fragments is live: its share of the stage loads, the
// waits and the barriers of gemm_mainloop, nothing else (the matrix pipe of its SIMD is left to
// the other wave).
template <typename S, bool PROLOGUE_ISSUED = false, bool CHAINED = false, typename AtStep = GemmNoHook>
__device__ __forceinline__ void gemm_mainloop_idle(GemmCursors<S> &cur, uint8_t *stages, uint32_t nk, uint32_t wave,
                                                   GemmChain<S> *chain = nullptr, AtStep at_step = AtStep{}) {
  static_assert(!CHAINED || PROLOGUE_ISSUED, "a chained loop finds its first stages in place");
  if constexpr (!PROLOGUE_ISSUED) gemm_prologue<S>(cur, stages, nk, wave);
  uint32_t fill = S::NSTAGE - 1;
  if constexpr (CHAINED) fill = chain->fill;
  const uint32_t tail = min(nk, static_cast<uint32_t>(S::NSTAGE - 1));
  for (uint32_t s = 0; s < nk; ++s) {
    if (!CHAINED || s >= static_cast<uint32_t>(S::NSTAGE - 1)) wait_vmcnt((S::NSTAGE - 2) * S::kSlots);
    stage_barrier();
    at_step(s);
    const bool own = s + tail < nk;
    uint8_t *const fill_stage = stages + fill * S::kStageBytes;
    fill = fill + 1u == S::NSTAGE ? 0u : fill + 1u;
    if constexpr (CHAINED) {
      if (own) gemm_issue_stage<S>(cur, fill_stage, wave, true);
      else gemm_issue_stage<S>(*chain->next, fill_stage, wave, true);
    } else {
      gemm_issue_stage<S>(cur, fill_stage, wave, own);
    }
  }
  if constexpr (CHAINED) {
    chain->buf = (chain->buf + nk) % S::NSTAGE;
    chain->fill = fill;
    wait_vmcnt(0);
  } else {
    lds_barrier();
  }
}

// gemm_mainloop for a wave with `live` (0 .. S::NT, wave-uniform) live token fragments.
template <typename S, WScaleMode MODE, bool PROLOGUE_ISSUED = false, bool CHAINED = false, typename XScale,
          typename WBlockScale, typename AtStep = GemmNoHook>
__device__ __forceinline__ void gemm_mainloop_ragged(f32x4_t (&acc)[S::NMAT][S::NF][S::NT], GemmCursors<S> &cur,
                                                     uint8_t *stages, uint32_t nk, uint32_t wave, uint32_t lane,
                                                     uint32_t live, XScale x_scale, WBlockScale w_block_scale,
                                                     GemmChain<S> *chain = nullptr, AtStep at_step = AtStep{}) {
  static_assert(S::NT == 1 || S::NT == 2 || S::NT == 4, "instantiated fragment counts");
  if (live == 0u) {
    gemm_mainloop_idle<S, PROLOGUE_ISSUED, CHAINED>(cur, stages, nk, wave, chain, at_step);
  } else if (live >= static_cast<uint32_t>(S::NT)) {
    gemm_mainloop<S, MODE, PROLOGUE_ISSUED, S::NT, CHAINED>(acc, cur, stages, nk, wave, lane, x_scale, w_block_scale,
                                                           chain, at_step);
  } else if constexpr (S::NT >= 2) {
    if (live == 1u) {
      gemm_mainloop<S, MODE, PROLOGUE_ISSUED, 1, CHAINED>(acc, cur, stages, nk, wave, lane, x_scale, w_block_scale,
                                                          chain, at_step);
    } else if constexpr (S::NT == 4) {
      if (live == 2u) {
        gemm_mainloop<S, MODE, PROLOGUE_ISSUED, 2, CHAINED>(acc, cur, stages, nk, wave, lane, x_scale, w_block_scale,
                                                            chain, at_step);
      } else {
        gemm_mainloop<S, MODE, PROLOGUE_ISSUED, 3, CHAINED>(acc, cur, stages, nk, wave, lane, x_scale, w_block_scale,
                                                            chain, at_step);
      }
    }
  }
}

// Row pitch of a [rows][cols] table of scale bytes in LDS that 16 lanes read one row each at the
// same column: the pitch in dwords must not be a multiple of 4, or lanes i and i + 8 share a bank.
__host__ __device__ constexpr uint32_t scale_row_pitch(uint32_t cols) {
  const uint32_t pitch = (cols + 3u) & ~3u;
  return (pitch >> 2) % 4u == 0u ? pitch + 4u : pitch;
}

}  // namespace ferrule_hip
