// Bidirectional chunked GLA forward on MFMA tiles (gfx950), Dk in {32, 64}, Dv = 64, bf16 in and out.
//
// One persistent workgroup of 8 waves per CU walks (batch, head) slabs of up to 256
// tokens.  A slab is cut into 4 chunks of ceil(L/4) <= 64 tokens; wave (chunk c,
// direction d) handles one chunk in one direction, so the two directions of a chunk run
// side by side on the same SIMD and read the same q/k/v lines.  A wave
//   1. forms the chunk-local cumulative log-gates G with a triangular-ones MFMA
//      (bf16 gates are exact MFMA inputs, the sums accumulate in fp32),
//   2. builds operands anchored at half the chunk total, q~ = q*exp(G - G_end/2) and
//      k~ = k*exp(G_end/2 - G): both stay within exp(|G_end|/2) of the inputs,
//   3. computes the masked intra-chunk scores P^T = k~ q~^T on fp16 operands (11-bit
//      significands, one MFMA term) and P V on bf16 with P split hi + lo (V is exact bf16),
//   4. accumulates the chunk's state contribution U = k~^T V  [Dk x Dv] in fp32 (k~ as bf16).
// The U's of a direction meet once in LDS, where the four waves of the direction run the
// chunk-to-chunk state recurrence S <- sqrt(D) (sqrt(D) S + U), D = exp(G_end), in parallel over
// disjoint state slices and leave, for every chunk, sqrt(D) S_in as ready bf16 MFMA
// fragments; each wave adds q~ (sqrt(D) S_in) to its outputs.  The two waves of a
// chunk then swap half of their fp32 output tiles through LDS, add, scale and store
// bf16 once.  Loads for the next slab are issued before the swap.
//
// fp16 score operands need |G_end|/2 * log2(e) <= 6 in every channel of every chunk (ViG's
// logsigmoid(.)/16 gates reach about 2.5) and rows of q, k, V with sums of squares below 2^15; every wave checks both for
// its chunk.  A workgroup that meets a segment outside that range redoes it, and does all its later
// segments, with bf16 hi + lo operands and three score terms per k-step (same algebra,
// any gate total up to ~80 per chunk and channel).
//
// Chunk algebra follows flash-linear-attention/fla/ops/gla/chunk_util.py:9-78 and
// chunk_fuse.py:76-97,245-254 (here with 64-token chunks, a mid-range anchor so that both
// operands stay small, and matrix-core intra-chunk scores); both directions are served by
// one launch as in recurrent_fuse.py:19-148.
//
// Register layouts (lane l: r = l & 31, h = l >> 5), v_mfma_f32_32x32x16_{bf16,f16}:
//   A/B operand: lane supplies index r and contraction slots e = 0..7 (4 VGPRs);
//   C/D: lane holds column r, register c = 4*g + m holds row 8*g + 4*h + m.
// "Transposed" fragments (tokens in the contraction slots) are read as one dword =
// two adjacent channels per token and de-interleaved with v_perm_b32; lane-row rho
// reads channel pair cpair(rho), chosen so that every accumulator ends up holding
// 32 contiguous channels (32*h + 8*g + 2*m + p) of one token.
#include "common.h"
#include "launch.h"
#include "mfma_tiles.h"
#include <stdlib.h>

namespace vig {

namespace {

// Scheduling fence: keeps the machine scheduler from hoisting the next phase's loads over this one's math.
#define VIG_PHASE() __builtin_amdgcn_sched_barrier(0)


// fp16 score operands are used while |G_end|/2 * log2(e) <= this for every channel of the chunk: the scaled
// operands then stay within 2^6 of the inputs' magnitudes (fp16 holds |x| < 65504 and full precision above 6e-5).
constexpr float kFastHalfRange = 6.0f;
// bf16 / fp16 elements per row of a wave's k~ scratch.  Dk = 64: 128-byte rows padded to 144 (conflict-free 16-byte
// writes), 9 KB, i.e. reaching into unit 8 of the region.  Dk = 32: 64-byte rows padded to 80 (eight lanes' writes
// still cover all 32 banks once), 5 KB: inside the lower half, as the Dk = 32 slabs without barrier D need it (their
// unit 8 carries an output half that the partner may still be reading when the next slab's scratch is written).
template <int NG>
constexpr int kFwdKtStride = NG == 4 ? kKtStride : 40;
constexpr int kRegionBytes = 16 * 1024;      // per wave: k~ scratch, then published U / state fragments / output half
constexpr int kLdsDvec = 8 * kRegionBytes;   // per wave: 64 chunk decays exp(G_end)
constexpr int kLdsGend = kLdsDvec + 8 * 64 * 4;  // per wave: 64 anchors G_end * log2(e), laid out [h][p][16]
constexpr int kLdsVeto = kLdsGend + 8 * 64 * 4;  // one word: some chunk refused the fp16 variant
constexpr int kLdsGateW = kLdsVeto + 16;          // fused locality gate: the 64 x 9 stencil weights of the slab's head
constexpr int kLdsHalf16 = kLdsGateW + 64 * 9 * 4;  // per wave: 64 half decays exp(G_end/2) as fp16, channel order
constexpr int kLdsTotal = kLdsHalf16 + 8 * 64 * 2;

// The fp16 variant rounds q~ = q 2^x and k~ = k 2^-x (|x| <= kFastHalfRange = 6), the scores P = q~ . k~ and V to fp16.
// With every row's sum of squares below 2^15 (the guard sums the rows of two tokens of q, k and V, which only makes it
// stricter), elements stay below 182, the scaled operands below 182 * 64, and |P| <= |q_i| |k_j| below 2^15: all
// inside fp16 range.  Inf or huge inputs fail the guard; NaN inputs give NaN outputs on every path.
constexpr float kFastMaxSquares = 32768.0f;
__device__ __forceinline__ bool gram_too_large(const f32x4acc_t& acc) {
  const float m = fmaxf(fmaxf(fabsf(acc[0]), fabsf(acc[1])), fmaxf(fabsf(acc[2]), fabsf(acc[3])));
  return __builtin_amdgcn_ballot_w64(!(m < kFastMaxSquares)) != 0;
}

// q~ and k~ of one 32-token tile for the fp16 score path: one exponent per element serves both (the factors are
// reciprocal), each product is rounded once to fp16 (11-bit significand): k~ serves the scores and, through LDS, the
// state update (against V converted to fp16, which holds every bf16 value of ordinary magnitude exactly); q~ is
// rounded a second time to bf16 for the inter-chunk product with the bf16 state fragments, or (KEEP16: whole slabs)
// kept as it is for the products with the earlier chunks' fp16 contributions.
template <bool WITH_Q, int NG, bool KEEP16 = false>
__device__ __forceinline__ void make_pair16(const u32x4_t (&rawq)[NG], const u32x4_t (&rawk)[NG],
                                            const f32x16_t (&G)[2], const float* gend2, u32x4_t (&q16)[NG],
                                            u32x4_t (&k16)[NG], u32x4_t (&qb)[NG]) {
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    const f32x4_t a0 = *reinterpret_cast<const f32x4_t*>(gend2 + 4 * g);
    const f32x4_t a1 = *reinterpret_cast<const f32x4_t*>(gend2 + 16 + 4 * g);
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int c = 4 * g + m;
      const float x0 = __builtin_fmaf(G[0][c], kLog2e, -a0[m]);
      const float x1 = __builtin_fmaf(G[1][c], kLog2e, -a1[m]);
      const uint32_t wk = rawk[g][m];
      const float k0 = bf16lo_to_f32(wk) * exp2_fast(-x0);
      const float k1 = bf16hi_to_f32(wk) * exp2_fast(-x1);
      k16[g][m] = pack_f16x2(k0, k1);
      if (WITH_Q) {
        const uint32_t wq = rawq[g][m];
        const float q0 = bf16lo_to_f32(wq) * exp2_fast(x0);
        const float q1 = bf16hi_to_f32(wq) * exp2_fast(x1);
        q16[g][m] = pack_f16x2(q0, q1);
        if (KEEP16) {
          qb[g][m] = q16[g][m];
        } else {
          qb[g][m] = pack_bf16x2(q0, q1);
          asm volatile("" : "+v"(qb[g][m]));  // packed here: the two floats must not stay alive until the pair is used
        }
      }
    }
  }
}

// O^T[p] += V^T (k-steps 2*jt, 2*jt+1 of vfrag) x P^T tile, with P split into bf16 hi + lo against bf16 V, or (F16)
// P as one fp16 operand against fp16 V.
// MASK: 0 none, 1 keep j <= i (forward diagonal tile), 2 keep j >= i (reverse diagonal tile).
template <int MASK, bool F16 = false>
__device__ __forceinline__ void apply_scores(f32x16_t P, int jt, int r, int h, const u32x4_t (&vfrag)[4][2],
                                             f32x16_t& O0, f32x16_t& O1) {
  if (MASK != 0) {
#pragma unroll
    for (int c = 0; c < 16; ++c) {
      const int j = 8 * (c >> 2) + 4 * h + (c & 3);
      const bool keep = MASK == 1 ? (j <= r) : (j >= r);
      P[c] = keep ? P[c] : 0.f;
    }
  }
  if (F16) {  // P rounded once to fp16 (11-bit significand) against fp16 V: one term
#pragma unroll
    for (int tl = 0; tl < 2; ++tl) {
      u32x4_t ph;
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int c = 4 * (2 * tl + (x >> 1)) + 2 * (x & 1);
        ph[x] = pack_f16x2(P[c], P[c + 1]);
      }
      const int t = 2 * jt + tl;
      O0 = mfma_f16(vfrag[t][0], ph, O0);
      O1 = mfma_f16(vfrag[t][1], ph, O1);
    }
    return;
  }
#pragma unroll
  for (int tl = 0; tl < 2; ++tl) {
    u32x4_t ph, pl;
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const int c = 4 * (2 * tl + (x >> 1)) + 2 * (x & 1);
      const uint32_t hi = pack_bf16x2(P[c], P[c + 1]);
      ph[x] = hi;
      pl[x] = pack_bf16x2(P[c] - bf16lo_to_f32(hi), P[c + 1] - bf16hi_to_f32(hi));
    }
    const int t = 2 * jt + tl;
    O0 = mfma(vfrag[t][0], ph, O0);
    O0 = mfma(vfrag[t][0], pl, O0);
    O1 = mfma(vfrag[t][1], ph, O1);
    O1 = mfma(vfrag[t][1], pl, O1);
  }
}

// What a wave carries from the end of one slab to the start of the next: the loads of its first phase.
template <int NG>
struct Prefetch {
  uint32_t gD[4][8];           // gate dwords, all four k-steps of the chunk
  uint32_t vD[2][8];           // V dwords of the tile walked first
  u32x4_t rawk[NG], rawq[NG];  // raw rows of the tile walked first
};

// The four tensors of one chunk: gate rows are contiguous (32*NG bytes); q, k and v rows lie a pitch apart, which is
// the row itself for plain [B, H, L, D] tensors and more when a head's channels sit inside wider token rows.
struct ChunkSrc {
  rsrc_t q, k, v, g;
  unsigned q_pitch, k_pitch, v_pitch;  // bytes
};

template <int NG>
__device__ __forceinline__ void issue_gates(const ChunkSrc& src, int r, int h, Prefetch<NG>& pf) {
  issue_tdwords<0, 4, NG>(src.g, r, h, pf.gD);
}
// (PITCHED: q, k, v rows lie the descriptors' pitches apart; else they are contiguous and every token offset is an
// instruction immediate)
template <bool FWD, bool WITH_Q, int NG, bool PITCHED = false>
__device__ __forceinline__ void issue_rows(const ChunkSrc& src, int r, int h, Prefetch<NG>& pf) {
  constexpr int TA = FWD ? 0 : 1;
  if (PITCHED) {
    issue_raw_tile_pitched<NG>(src.k, TA, r, h, src.k_pitch, pf.rawk);
    if (WITH_Q) issue_raw_tile_pitched<NG>(src.q, TA, r, h, src.q_pitch, pf.rawq);
    issue_tdwords_pitched<2 * TA, 2, 4>(src.v, r, h, src.v_pitch, pf.vD);
  } else {
    issue_raw_tile<NG>(src.k, TA, r, h, pf.rawk);
    if (WITH_Q) issue_raw_tile<NG>(src.q, TA, r, h, pf.rawq);
    issue_tdwords<2 * TA, 2, 4>(src.v, r, h, pf.vD);
  }
}
template <bool FWD, bool WITH_Q, int NG, bool PITCHED = false>
__device__ __forceinline__ void issue_first_phase(const ChunkSrc& src, int r, int h, Prefetch<NG>& pf) {
  issue_gates<NG>(src, r, h, pf);
  issue_rows<FWD, WITH_Q, NG, PITCHED>(src, r, h, pf);
}

// Segment modes of the kernel.  A sequence longer than 256 tokens is cut into segments of <= 256 tokens that are
// processed like slabs, chained through per-segment states in a caller workspace:
//   kModeSlab   whole sequence in one segment, no state in or out;
//   kModeState  pass 1 of a long sequence: only k~, V and the gates are touched; the segment's end-anchored state
//               contribution and total decay are written to the workspace (no outputs);
//   kModeChain  pass 2 of a long sequence: the state entering the segment (from the left for the forward direction,
//               from the right for the reverse one) is read from the workspace and outputs are produced.
//   kModeStateDual  two state passes in one launch, for the backward of a long sequence: items below
//               Geometry::dual_first are kModeState items; the others build the per-segment gradient states: the
//               same pass fed the q tensor for k and the output gradient (the o argument) for v, with the other
//               direction's gates and the cumulative gates taken exclusive of a token's own gate (so that the weight
//               of a token reaches back to and includes it).
//   kModeSlabPitched  kModeSlab on q, k, v whose token rows lie a pitch apart (column blocks of a wider matrix read in
//               place): the same arithmetic, token offsets in scalar registers instead of instruction immediates.
constexpr int kModeSlab = 0, kModeState = 1, kModeChain = 2, kModeStateDual = 3, kModeSlabPitched = 4;
constexpr bool is_state_mode(int mode) { return mode == kModeState || mode == kModeStateDual; }
constexpr bool is_slab(int mode) { return mode == kModeSlab || mode == kModeSlabPitched; }
constexpr bool is_pitched(int mode) { return mode == kModeSlabPitched; }
constexpr int kStateFloats = kGlaStateFloats;  // per (sequence, segment, direction): state in unit order, then 64 decays

// Intra-chunk part of one wave: scores of the three tile pairs of its chunk, applied to V; k~ (bf16) goes to the
// wave's LDS scratch for the state update, q~ (bf16) is kept for the inter-chunk product.  The second tile's rows
// and V fragments are fetched while the first is worked on.
//   F16: score operands are single fp16 roundings (valid while the chunk's gate totals keep them inside fp16 range);
//   otherwise bf16 hi + lo pairs and three MFMA terms per k-step.
// Returns (F16 only, wave-uniform) whether some raw q or k value of the chunk is too large for fp16 operands.
template <bool FWD, int MODE, int NG, bool F16>
__device__ __forceinline__ bool tile_phase(const ChunkSrc& cur, const Prefetch<NG>& pf, const f32x16_t (&G)[2][2],
                                           const float* gend2, uint16_t* kt, int r, int h, f32x16_t (&O)[2][2],
                                           u32x4_t (&qkeep)[2][NG], u32x4_t (&vfrag)[4][2]) {
  constexpr bool OUT = !is_state_mode(MODE);
  constexpr int TA = FWD ? 0 : 1;  // tile walked first
  constexpr int TB = FWD ? 1 : 0;
  constexpr int MASK = FWD ? 1 : 2;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) O[i][j] = f32x16_t{0.f};
  u32x4_t rawk[NG], rawq[NG];
  uint32_t vDb[2][8];
  f32x4acc_t gram = {0.f, 0.f, 0.f, 0.f};  // (fp16 variant) magnitude guard over the chunk's q, k and V
  // a reverse wave only runs beside the forward wave of the same chunk, which sees the same q, k and V rows
  constexpr bool GUARD = F16 && FWD;
  auto set_vfrag = [&](const uint32_t (&D)[2][8], int t0) {
    u32x4_t vf[2][2];
    finish_tfrags<2>(D, vf);
#pragma unroll
    for (int tl = 0; tl < 2; ++tl)
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        if (F16) {  // bf16 pairs -> fp16 pairs (exact for magnitudes the variant admits: the guard sees them first)
          if (GUARD) gram_acc(vf[tl][p], gram);
#pragma unroll
          for (int x = 0; x < 4; ++x) vf[tl][p][x] = pack_f16x2(bf16lo_to_f32(vf[tl][p][x]), bf16hi_to_f32(vf[tl][p][x]));
        }
        vfrag[t0 + tl][p] = vf[tl][p];
      }
  };
  auto fetch_second = [&]() {
    if (is_pitched(MODE)) {
      if (OUT) issue_raw_tile_pitched<NG>(cur.q, TB, r, h, cur.q_pitch, rawq);
      issue_raw_tile_pitched<NG>(cur.k, TB, r, h, cur.k_pitch, rawk);
      issue_tdwords_pitched<2 * TB, 2, 4>(cur.v, r, h, cur.v_pitch, vDb);
    } else {
      if (OUT) issue_raw_tile<NG>(cur.q, TB, r, h, rawq);
      issue_raw_tile<NG>(cur.k, TB, r, h, rawk);
      issue_tdwords<2 * TB, 2, 4>(cur.v, r, h, vDb);
    }
  };
  bool too_large = false;
  if (F16) {
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      if (GUARD) gram_acc(pf.rawk[g], gram);
      if (GUARD && OUT) gram_acc(pf.rawq[g], gram);
    }
    u32x4_t ka[NG], qb[NG];
    // the second tile's loads go out before the first tile's operands are built where registers allow it (measured:
    // earlier is better for whole slabs, later for the chained segments of long sequences)
    constexpr bool EARLY = is_slab(MODE);
    if (EARLY) fetch_second();
    VIG_PHASE();
    {
      u32x4_t qa[NG];
      make_pair16<OUT, NG, is_slab(MODE)>(pf.rawq, pf.rawk, G[TA], gend2, qa, ka, qkeep[TA]);
      store_kt<NG, kFwdKtStride<NG>>(kt, 32 * TA + r, h, ka);
      VIG_PHASE();
      if (!EARLY) fetch_second();
      set_vfrag(pf.vD, 2 * TA);
      if (OUT) apply_scores<MASK, true>(score_tile16<NG>(ka, qa), TA, r, h, vfrag, O[0][TA], O[1][TA]);
    }
    VIG_PHASE();
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      if (GUARD) gram_acc(rawk[g], gram);
      if (GUARD && OUT) gram_acc(rawq[g], gram);
    }
    u32x4_t kb[NG];
    make_pair16<OUT, NG, is_slab(MODE)>(rawq, rawk, G[TB], gend2, qb, kb, qkeep[TB]);
    store_kt<NG, kFwdKtStride<NG>>(kt, 32 * TB + r, h, kb);
    if (OUT) apply_scores<0, true>(score_tile16<NG>(ka, qb), TA, r, h, vfrag, O[0][TB], O[1][TB]);
    VIG_PHASE();
    set_vfrag(vDb, 2 * TB);
    if (OUT) apply_scores<MASK, true>(score_tile16<NG>(kb, qb), TB, r, h, vfrag, O[0][TB], O[1][TB]);
    too_large = GUARD && gram_too_large(gram);
  } else {
    HalfOps<NG> ka, qb;
    {
      HalfOps<NG> qa;
      make_half<false, NG>(pf.rawk, G[TA], gend2, ka);
      if (OUT) make_half<true, NG>(pf.rawq, G[TA], gend2, qa);
      VIG_PHASE();
      fetch_second();
      set_vfrag(pf.vD, 2 * TA);
      if (OUT) apply_scores<MASK>(score_tile(ka, qa), TA, r, h, vfrag, O[0][TA], O[1][TA]);
      store_kt<NG, kFwdKtStride<NG>>(kt, 32 * TA + r, h, ka.h);
      if (OUT) {
#pragma unroll
        for (int ks = 0; ks < NG; ++ks) qkeep[TA][ks] = qa.h[ks];
      }
    }
    VIG_PHASE();
    if (OUT) {
      make_half<true, NG>(rawq, G[TB], gend2, qb);
      apply_scores<0>(score_tile(ka, qb), TA, r, h, vfrag, O[0][TB], O[1][TB]);
    }
    VIG_PHASE();
    {
      HalfOps<NG> kb;
      make_half<false, NG>(rawk, G[TB], gend2, kb);
      set_vfrag(vDb, 2 * TB);
      if (OUT) apply_scores<MASK>(score_tile(kb, qb), TB, r, h, vfrag, O[0][TB], O[1][TB]);
      store_kt<NG, kFwdKtStride<NG>>(kt, 32 * TB + r, h, kb.h);
    }
    if (OUT) {
#pragma unroll
      for (int ks = 0; ks < NG; ++ks) qkeep[TB][ks] = qb.h[ks];
    }
  }
  return too_large;
}


// Locality gate fused into the output of a whole-sequence slab:  y = o * sigmoid(conv3x3(o)), the depthwise 3x3
// stencil taken over the gw x gh token grid of the slab (zero padding), per channel, on the bf16-rounded o.
struct GateCtx {
  const float* w;  // [64][9] stencil weights of this slab's head
  int gw, gh;      // token grid: gw columns, gh rows, gw * gh = L
  int t0, nvalid;  // first token of this wave's chunk in the slab and its number of rows
};
// The rounded outputs of the slab are staged as a zero-padded (gh+2) x (gw+2) grid of 128-byte cells in one half of
// every LDS region (the half that is dead by then: the lower one, behind the fp16 variant's contributions, the upper
// one otherwise).  A padded row never straddles two regions: each half takes rph = 64 / (gw+2) whole rows, so the
// three taps of a stencil row are at constant offsets from the first.
constexpr int kGateCellsPerRegion = 64;
struct GateLayout {
  int pw, rph, half;  // half: byte offset of the staging half inside a region
  float inv_rph;
  __device__ __forceinline__ GateLayout(int gw, int half_offset)
      : pw(gw + 2), rph(kGateCellsPerRegion / (gw + 2)), half(half_offset) {
    inv_rph = 1.0f / (float)rph;
  }
  // byte offset in LDS of padded cell (py, 0); exact for py < 2^20
  __device__ __forceinline__ int row(int py) const {
    const int reg = (int)(((float)py + 0.5f) * inv_rph);
    return reg * kRegionBytes + half + __mul24(py - __mul24(reg, rph), pw * 128);  // (24-bit: full rate)
  }
};

// Everything one wave does for one segment: chunk c (the valid rows its descriptors cover) in
// direction FWD / reverse.  Every wave of the workgroup passes the same three barriers here (plus the caller's).
// F16 selects fp16 score operands; that variant returns false (for every wave of the workgroup alike, and without
// having stored anything) when some chunk of the segment has gates too strong for it.
template <bool FWD, int MODE, int NG, bool F16, bool GATE>
__device__ __forceinline__ bool direction_wave(const ChunkSrc& cur, const ChunkSrc& nxt, rsrc_t o, int c, int lane,
                                               char* lds, float oscale, bool bidir, float* state, Prefetch<NG>& pf,
                                               const GateCtx& gate, bool strict = false) {
  constexpr bool OUT = !is_state_mode(MODE);  // produces outputs (needs q)
  int r = lane & 31, h = lane >> 5;
  const int wi = (FWD ? 0 : 4) + c;
  constexpr int TA = FWD ? 0 : 1;  // tile walked first
  constexpr int TB = FWD ? 1 : 0;
  char* region = lds + wi * kRegionBytes;
  uint16_t* kt = reinterpret_cast<uint16_t*>(region);
  float* dvec_all = reinterpret_cast<float*>(lds + kLdsDvec);
  if (!FWD) issue_rows<FWD, OUT, NG, is_pitched(MODE)>(cur, r, h, pf);
  // fused gate: the first 144 threads fetch the head's stencil weights now and park them in LDS before barrier A
  f32x4_t gate_w4 = {0.f, 0.f, 0.f, 0.f};
  const bool gate_w_mine = GATE && wi * 64 + lane < 64 * 9 / 4;
  if (GATE && gate_w_mine) gate_w4 = reinterpret_cast<const f32x4_t*>(gate.w)[wi * 64 + lane];

  // ---- cumulative log-gates G[it][p] via triangular-ones MFMA on transposed gate fragments ----
  f32x16_t G[2][2];
  f32x16_t Gend[2];
  {
    u32x4_t gfrag[4][2];
    finish_tfrags<4>(pf.gD, gfrag);
    const u32x4_t ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
    u32x4_t tri0 = tri_frag<FWD>(0, 0, r, h), tri1 = tri_frag<FWD>(1, 0, r, h);
    if (MODE == kModeStateDual && strict) tri0 = tri_frag<FWD, true>(0, 0, r, h), tri1 = tri_frag<FWD, true>(1, 0, r, h);
    // k-steps of the tile walked first / second (the triangular operand depends on (k-step, tile) only through
    // their offset, so two fragments serve both tiles)
    constexpr int A0 = FWD ? 0 : 2, B0 = FWD ? 2 : 0;
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      // total of the tile walked first, in every column: the second tile's sums start from it
      f32x16_t carry = {0.f};
      carry = mfma(gfrag[A0][p], ones, carry);
      carry = mfma(gfrag[A0 + 1][p], ones, carry);
      f32x16_t ga = {0.f};
      ga = mfma(gfrag[A0][p], tri0, ga);
      ga = mfma(gfrag[A0 + 1][p], tri1, ga);
      f32x16_t gb = mfma(gfrag[B0][p], tri0, carry);
      gb = mfma(gfrag[B0 + 1][p], tri1, gb);
      // the chunk total (= G at the anchor token) for every column at once: no cross-lane broadcast needed
      f32x16_t ge = mfma(gfrag[B0][p], ones, carry);
      ge = mfma(gfrag[B0 + 1][p], ones, ge);
      Gend[p] = ge;
      G[FWD ? 0 : 1][p] = ga;
      G[FWD ? 1 : 0][p] = gb;
    }
  }
  // ---- anchor: half of the chunk total G_end (G at the last token forward / first token reverse), per channel, so
  // that q~ = q*exp(G - G_end/2) and k~ = k*exp(G_end/2 - G) share the exponent range [-|G_end|/2, |G_end|/2].
  // The anchors (x log2 e) and the half decays exp(G_end/2) go to LDS: the operand builders re-read the former per
  // tile, the state recurrence reads the latter after barrier A, and no register holds them across phases. ----
  float* gend2 = reinterpret_cast<float*>(lds + kLdsGend) + wi * 64 + 32 * h;
  constexpr int HC = 8 * NG;  // channels per lane half
  bool fast = true;
  {
    // every lane of a half holds the same 32 chunk totals, one per register: one lane writes them out, then each
    // lane of the wave turns one of the 64 values into its anchor and half decay (one exponential per wave
    // instead of one per value)
    if (r == 0) {
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        const f32x4_t x0 = {Gend[0][4 * gq], Gend[0][4 * gq + 1], Gend[0][4 * gq + 2], Gend[0][4 * gq + 3]};
        const f32x4_t x1 = {Gend[1][4 * gq], Gend[1][4 * gq + 1], Gend[1][4 * gq + 2], Gend[1][4 * gq + 3]};
        *reinterpret_cast<f32x4_t*>(gend2 + 4 * gq) = x0;
        *reinterpret_cast<f32x4_t*>(gend2 + 16 + 4 * gq) = x1;
      }
    }
    wave_lds_sync();
    float* mine = reinterpret_cast<float*>(lds + kLdsGend) + wi * 64 + lane;  // value (h, p, 4*g + m), lane = 32h+16p+4g+m
    const float an = *mine * (0.5f * kLog2e);
    // wave-uniform: fp16 score operands while every channel's exponent range stays within +-kFastHalfRange
    if (F16) fast = __builtin_amdgcn_ballot_w64(fabsf(an) > kFastHalfRange) == 0;
    *mine = an;
    const int p = (lane >> 4) & 1, g = (lane >> 2) & 3, m = lane & 3;
    // half decay of channel 8*g + 2*m + p of this lane half (register quads >= NG carry no channel)
    if (g < NG) {
      if (is_slab(MODE) && F16)
        reinterpret_cast<_Float16*>(lds + kLdsHalf16)[wi * 64 + HC * h + 8 * g + 2 * m + p] = (_Float16)exp2_fast(an);
      else
        dvec_all[wi * 64 + HC * h + 8 * g + 2 * m + p] = exp2_fast(an);
    }
  }
  wave_lds_sync();
  // ---- intra-chunk scores, tile by tile ----
  f32x16_t O[2][2];
  u32x4_t qkeep[2][NG];
  u32x4_t vfrag[4][2];
  if (tile_phase<FWD, MODE, NG, F16>(cur, pf, G, gend2, kt, r, h, O, qkeep, vfrag)) fast = false;
  wave_lds_sync();  // k~ rows of this wave visible to its other lanes
  // ---- chunk state contribution U[pk][pv] = k~^T V; publish it (register-native fp32) ----
  {
    f32x16_t U[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) U[i][j] = f32x16_t{0.f};
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      u32x4_t ktf[2];
      load_tfrag_lds<NG, kFwdKtStride<NG>>(kt, t, r, h, ktf);
#pragma unroll
      for (int pk = 0; pk < 2; ++pk)
#pragma unroll
        for (int pv = 0; pv < 2; ++pv)
          U[pk][pv] = F16 ? mfma_f16(ktf[pk], vfrag[t][pv], U[pk][pv]) : mfma(ktf[pk], vfrag[t][pv], U[pk][pv]);
    }
    constexpr bool DIRECT = is_slab(MODE) && F16;
    if (DIRECT) {
      // whole slab on fp16 operands: the later chunks of the direction take this contribution as it is (fp16, as
      // ready fragments: dword m of unit pv*4 + cq holds rows (pk = 0, 1) of register 4*cq + m) instead of a state
      // chained through it; its entries have to fit fp16
      float umax = 0.f;
#pragma unroll
      for (int pk = 0; pk < 2; ++pk)
#pragma unroll
        for (int pv = 0; pv < 2; ++pv)
#pragma unroll
          for (int i = 0; i < 16; ++i) umax = fmaxf(umax, fabsf(U[pk][pv][i]));
      if (__builtin_amdgcn_ballot_w64(!(umax < 60000.0f)) != 0) fast = false;
      if (FWD ? (c < 3) : (c > 0)) {
#pragma unroll
        for (int pv = 0; pv < 2; ++pv)
#pragma unroll
          for (int cq = 0; cq < NG; ++cq) {
            u32x4_t fr;
#pragma unroll
            for (int m = 0; m < 4; ++m) fr[m] = pack_f16x2(U[0][pv][4 * cq + m], U[1][pv][4 * cq + m]);
            *reinterpret_cast<u32x4_t*>(unit_ptr(region, pv * 4 + cq, lane)) = fr;
          }
      }
    } else
    // the chunk walked last is consumed by nobody inside the segment, unless the segment's own total is wanted
    if (is_state_mode(MODE) || (FWD ? (c < 3) : (c > 0))) {
#pragma unroll
      for (int pk = 0; pk < 2; ++pk)
#pragma unroll
        for (int pv = 0; pv < 2; ++pv)
#pragma unroll
          for (int cq = 0; cq < NG; ++cq) {  // rows of register quads >= NG carry no channel
            const f32x4_t x = {U[pk][pv][4 * cq], U[pk][pv][4 * cq + 1], U[pk][pv][4 * cq + 2], U[pk][pv][4 * cq + 3]};
            *reinterpret_cast<f32x4_t*>(unit_ptr(region, (pk * 2 + pv) * 4 + cq, lane)) = x;
          }
    }
  }
  // ---- forward waves fetch the whole first phase of the NEXT segment here; reverse waves fetch only its gate
  // dwords (needed first) here and the rows at the top of the segment: a wave stalls while the memory pipe accepts
  // its loads, and this way the other wave of the SIMD has math to do.  (Always issued: after the last segment the
  // descriptors are empty, which keeps branches off the loads.) ----
  if (FWD) issue_first_phase<FWD, OUT, NG, is_pitched(MODE)>(nxt, r, h, pf);
  else issue_gates<NG>(nxt, r, h, pf);
  // lane-derived addresses of the exchange phases are rebuilt here instead of being carried (and spilled) across
  // the register-heavy tile phase
  asm volatile("" : "+v"(lane));
  r = lane & 31;
  h = lane >> 5;
  int* veto = reinterpret_cast<int*>(lds + kLdsVeto);
  if (F16 && !fast && lane == 0) *veto = 1;
  if (GATE && gate_w_mine) reinterpret_cast<f32x4_t*>(lds + kLdsGateW)[wi * 64 + lane] = gate_w4;
  lds_barrier();  // (A) published U's and decays visible
  // same answer in every wave: the word is only written before this barrier and the variant is left once it is set
  const bool ok = !F16 || __builtin_amdgcn_readfirstlane(*veto) == 0;
  if (F16 && !ok) return false;  // every wave alike: the segment is walked again, barriers B and C are skipped by all
  constexpr bool DIRECT = is_slab(MODE) && F16;
  if (DIRECT) {
    // ---- whole slab on fp16 operands: O^T += (E (.) U_j)^T q~ for every chunk j walked earlier in this direction,
    // E = h_c h_j prod(h_i^2, i between) per k channel with h = exp(G_end/2) <= 1 (the decay from the end of chunk j
    // to the tokens of this chunk, given the half anchors inside q~ and U_j); fp16 x fp16 -> fp16, no factor exceeds
    // one, tiny products may flush to zero.  No state, no serial chain: a wave with d earlier chunks does d products.
    const int npairs = FWD ? c : 3 - c;
    const _Float16* hdir = reinterpret_cast<const _Float16*>(lds + kLdsHalf16) + (FWD ? 0 : 4) * 64 + HC * h;
    u32x4_t base16[NG];  // h_c times the squares of the chunks passed so far
#pragma unroll
    for (int g = 0; g < NG; ++g) base16[g] = *reinterpret_cast<const u32x4_t*>(hdir + 64 * c + 8 * g);
#pragma unroll 1
    for (int d = 1; d <= npairs; ++d) {
      const int j = FWD ? c - d : c + d;
      u32x4_t e16[NG];
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const u32x4_t hj = *reinterpret_cast<const u32x4_t*>(hdir + 64 * j + 8 * g);
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          const uint32_t x = hj[m];
          e16[g][m] = mul_f16x2(base16[g][m], x);
          base16[g][m] = mul_f16x2(e16[g][m], x);
        }
      }
      char* ureg = lds + ((FWD ? 0 : 4) + j) * kRegionBytes;
      // (E goes onto the contribution's fragments, whose dwords hold the same k-channel pairs as q~'s: one scaling
      // serves both query tiles)
#pragma unroll
      for (int pv = 0; pv < 2; ++pv) {
        u32x4_t uf[NG];
#pragma unroll
        for (int ks = 0; ks < NG; ++ks) {
          uf[ks] = *reinterpret_cast<const u32x4_t*>(unit_ptr(ureg, pv * 4 + ks, lane));
#pragma unroll
          for (int m = 0; m < 4; ++m) uf[ks][m] = mul_f16x2(uf[ks][m], e16[ks][m]);
        }
#pragma unroll
        for (int ks = 0; ks < NG; ++ks)
#pragma unroll
          for (int it = 0; it < 2; ++it) O[pv][it] = mfma_f16(uf[ks], qkeep[it][ks], O[pv][it]);
      }
    }
  } else {
    // ---- state recurrence over the chunks of this direction, one slice (pv, NG/2 register quads) per wave ----
    constexpr int NQ = NG / 2;
    const int pv = c & 1, cqa = NQ * (c >> 1);
    char* dirbase = lds + (FWD ? 0 : 4) * kRegionBytes;
    const float* ddir = dvec_all + (FWD ? 0 : 4) * 64;
    constexpr int W0 = FWD ? 0 : 3, STEP = FWD ? 1 : -1;
    f32x4_t S[2][NQ];
#pragma unroll
    for (int pk = 0; pk < 2; ++pk)
#pragma unroll
      for (int j = 0; j < NQ; ++j) {
        const int u = (pk * 2 + pv) * 4 + cqa + j;
        if (MODE == kModeChain) {  // state entering the segment, written by the segment scan in the same unit order
          S[pk][j] = *reinterpret_cast<const f32x4_t*>(state + (u * 64 + lane) * 4);
        } else {  // state after the first chunk: its half-anchored contribution times its half decay
          S[pk][j] = *reinterpret_cast<const f32x4_t*>(unit_ptr(dirbase + W0 * kRegionBytes, u, lane));
          const float* dw = ddir + W0 * 64 + HC * h + 8 * (cqa + j);
#pragma unroll
          for (int m = 0; m < 4; ++m) S[pk][j][m] *= dw[2 * m + pk];
        }
      }
    // every decay vector and contribution a slice needs is fetched before its serial chain starts: one LDS round
    // trip per slice instead of one per chunk (3 % on the Dk = 32 slab shape, neutral on the others)
    constexpr int I0 = MODE == kModeChain ? 0 : 1;
#pragma unroll
    for (int j = 0; j < NQ; ++j) {
      const int cq = cqa + j;
      f32x4_t d0[4], d1[4], u0[4], u1[4];
#pragma unroll
      for (int i = I0; i < 4; ++i) {
        const int wc = W0 + STEP * i;  // consumer chunk: needs exp(G_end(wc)/2) * S as fragments
        char* creg = dirbase + wc * kRegionBytes;
        d0[i] = *reinterpret_cast<const f32x4_t*>(ddir + wc * 64 + HC * h + 8 * cq);
        d1[i] = *reinterpret_cast<const f32x4_t*>(ddir + wc * 64 + HC * h + 8 * cq + 4);
        u0[i] = u1[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        if (is_state_mode(MODE) || i < 3) {
          u0[i] = *reinterpret_cast<const f32x4_t*>(unit_ptr(creg, (0 * 2 + pv) * 4 + cq, lane));
          u1[i] = *reinterpret_cast<const f32x4_t*>(unit_ptr(creg, (1 * 2 + pv) * 4 + cq, lane));
        }
      }
#pragma unroll
      for (int i = I0; i < 4; ++i) {
        const int wc = W0 + STEP * i;
        char* creg = dirbase + wc * kRegionBytes;
        // half decay of row (m, pk): element 2*m + pk of the eight
        const float dk0[4] = {d0[i][0], d0[i][2], d1[i][0], d1[i][2]};
        const float dk1[4] = {d0[i][1], d0[i][3], d1[i][1], d1[i][3]};
        u32x4_t fr;
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          // with the half anchor: fragment = sqrt(D) * S_in,  S_out = sqrt(D) * (sqrt(D) * S_in + U)
          const float t0 = S[0][j][m] * dk0[m];
          const float t1 = S[1][j][m] * dk1[m];
          fr[m] = pack_bf16x2(t0, t1);
          S[0][j][m] = (t0 + u0[i][m]) * dk0[m];
          S[1][j][m] = (t1 + u1[i][m]) * dk1[m];
        }
        if (OUT) *reinterpret_cast<u32x4_t*>(unit_ptr(creg, pv * 4 + cq, lane)) = fr;
      }
    }
    if (is_state_mode(MODE) && ok) {
      // the segment's end-anchored contribution (unit order) and its total decay per channel
#pragma unroll
      for (int pk = 0; pk < 2; ++pk)
#pragma unroll
        for (int j = 0; j < NQ; ++j)
          *reinterpret_cast<f32x4_t*>(state + (((pk * 2 + pv) * 4 + cqa + j) * 64 + lane) * 4) = S[pk][j];
      if (c == 0 && lane < 16 * NG) {
        const float hd = ddir[lane] * ddir[64 + lane] * ddir[128 + lane] * ddir[192 + lane];
        state[64 * 64 + lane] = hd * hd;
      }
    }
  }
  // (whole slabs on fp16 operands send their output halves through the upper halves of the regions, which nothing
  // else uses there: the published contributions stay readable and barrier B is not needed)
  constexpr int kSendUnit = DIRECT ? 8 : 0;
  if (!DIRECT) lds_barrier();  // (B) incoming-state fragments of every chunk visible
  if (OUT) {
    // ---- O^T += (exp(G_end) * S_in) q~hi  for every chunk that has an incoming state ----
    if (!DIRECT && (MODE == kModeChain || (FWD ? (c > 0) : (c < 3)))) {
#pragma unroll
      for (int pv = 0; pv < 2; ++pv)
#pragma unroll
        for (int ks = 0; ks < NG; ++ks) {
          const u32x4_t sf = *reinterpret_cast<const u32x4_t*>(unit_ptr(region, pv * 4 + ks, lane));
#pragma unroll
          for (int it = 0; it < 2; ++it) O[pv][it] = mfma(sf, qkeep[it][ks], O[pv][it]);
        }
    }
    // ---- the output swap: each wave of a chunk keeps one 32-token tile ----
    constexpr int KEEP = FWD ? 0 : 1;
    constexpr int SEND = 1 - KEEP;
    if (bidir) {
#pragma unroll
      for (int pv = 0; pv < 2; ++pv)
#pragma unroll
        for (int cq = 0; cq < 4; ++cq) {
          const f32x4_t x = {O[pv][SEND][4 * cq], O[pv][SEND][4 * cq + 1], O[pv][SEND][4 * cq + 2],
                             O[pv][SEND][4 * cq + 3]};
          *reinterpret_cast<f32x4_t*>(unit_ptr(region, kSendUnit + pv * 4 + cq, lane)) = x;
        }
    }
    lds_barrier();  // (C) swapped output halves visible
    if (bidir) {
      char* partner = lds + ((FWD ? 4 : 0) + c) * kRegionBytes;
#pragma unroll
      for (int pv = 0; pv < 2; ++pv)
#pragma unroll
        for (int cq = 0; cq < 4; ++cq) {
          const f32x4_t x = *reinterpret_cast<const f32x4_t*>(unit_ptr(partner, kSendUnit + pv * 4 + cq, lane));
#pragma unroll
          for (int m = 0; m < 4; ++m) O[pv][KEEP][4 * cq + m] += x[m];
        }
    }
    if (GATE) {
      // (needs both directions: every wave owns the 32-row tile KEEP of its chunk)
      // (fp16 variant: the output halves travelled through the upper region halves, the cells go to the lower ones,
      // where the contributions are dead after barrier C; otherwise the other way round)
      const GateLayout lay(gate.gw, DIRECT ? 0 : kRegionBytes / 2);
      const float inv_w = 1.0f / (float)gate.gw;
      {
        const int row = 32 * KEEP + r;
        if (row < gate.nvalid) {
          const int T = gate.t0 + row;
          const int y = (int)(((float)T + 0.5f) * inv_w), x = T - __mul24(y, gate.gw);
          char* cell = lds + lay.row(y + 1) + (x + 1) * 128 + 64 * h;
#pragma unroll
          for (int gq = 0; gq < 4; ++gq) {
            u32x4_t w;
#pragma unroll
            for (int m = 0; m < 4; ++m)
              w[m] = pack_bf16x2(O[0][KEEP][4 * gq + m] * oscale, O[1][KEEP][4 * gq + m] * oscale);
            *reinterpret_cast<u32x4_t*>(cell + 16 * gq) = w;
          }
        }
      }
      const int oct = lane & 7, tl = lane >> 3;
      {  // the border cells, by the whole workgroup: top row, bottom row, then the two ends of every other row
        const int nborder = 2 * lay.pw + 2 * gate.gh;
        const u32x4_t zero = {0u, 0u, 0u, 0u};
        for (int bc = wi * 8 + tl; bc < nborder; bc += 64) {
          int py, px;
          if (bc < 2 * lay.pw) {
            py = bc < lay.pw ? 0 : gate.gh + 1;
            px = bc < lay.pw ? bc : bc - lay.pw;
          } else {
            const int j = bc - 2 * lay.pw;
            py = 1 + (j >> 1);
            px = (j & 1) ? lay.pw - 1 : 0;
          }
          *reinterpret_cast<u32x4_t*>(lds + lay.row(py) + px * 128 + 16 * oct) = zero;
        }
      }
      float wreg[8][9];
      {
        const f32x4_t* wp = reinterpret_cast<const f32x4_t*>(lds + kLdsGateW + oct * 72 * 4);
#pragma unroll
        for (int i = 0; i < 18; ++i) {
          const f32x4_t x = wp[i];
#pragma unroll
          for (int m = 0; m < 4; ++m) wreg[(4 * i + m) / 9][(4 * i + m) % 9] = x[m];
        }
      }
      lds_barrier();  // (C') the slab's outputs and the zero border are staged
#pragma unroll 1
      for (int i = 0; i < 4; ++i) {
        const int row = 32 * KEEP + tl + 8 * i;
        if (row < gate.nvalid) {
          const int T = gate.t0 + row;
          const int y = (int)(((float)T + 0.5f) * inv_w), x = T - __mul24(y, gate.gw);
          float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, ctr[8];
#pragma unroll
          for (int di = 0; di < 3; ++di) {
            const char* tap = lds + lay.row(y + di) + x * 128 + 16 * oct;  // padded cell of tap (di - 1, -1)
#pragma unroll
            for (int dj = 0; dj < 3; ++dj) {
              const u32x4_t w = *reinterpret_cast<const u32x4_t*>(tap + dj * 128);
#pragma unroll
              for (int m = 0; m < 4; ++m) {
                const float lo = bf16lo_to_f32(w[m]), hi = bf16hi_to_f32(w[m]);
                acc[2 * m] = __builtin_fmaf(lo, wreg[2 * m][di * 3 + dj], acc[2 * m]);
                acc[2 * m + 1] = __builtin_fmaf(hi, wreg[2 * m + 1][di * 3 + dj], acc[2 * m + 1]);
                if (di == 1 && dj == 1) ctr[2 * m] = lo, ctr[2 * m + 1] = hi;
              }
            }
          }
          u32x4_t out;
#pragma unroll
          for (int m = 0; m < 4; ++m)
            out[m] = pack_bf16x2(ctr[2 * m] * sigmoidf_(acc[2 * m]), ctr[2 * m + 1] * sigmoidf_(acc[2 * m + 1]));
          __builtin_amdgcn_raw_buffer_store_b128(out, o, (unsigned)row * 128u + 16u * oct, 0, 0);
        }
      }
    } else
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      if (bidir && it != KEEP) continue;
      const unsigned row = 32u * it + r;  // rows beyond the chunk fall outside the descriptor and are dropped
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        u32x4_t x;
#pragma unroll
        for (int m = 0; m < 4; ++m) x[m] = pack_bf16x2(O[0][it][4 * gq + m] * oscale, O[1][it][4 * gq + m] * oscale);
        __builtin_amdgcn_raw_buffer_store_b128(x, o, row * 128u + 64u * h + 16u * gq, 0, 0);
      }
    }
  } else {
    lds_barrier();  // (C) keeps the barrier count of the output modes
  }
  return ok;
}

// where sequence (b, h) of a tensor starts and how far its token rows lie apart, in elements
struct Strides {
  long long batch, head;
  int token;
};
// Geometry of the work items: item = sequence * nseg + segment; a segment holds seg_len tokens (the last one of a
// sequence possibly fewer) cut into 4 chunks of cw tokens.
struct Geometry {
  int L, nseg, seg_len, cw, nitems;
  int H;               // heads per batch element: sequence = b * H + h
  Strides sq, sk, sv;  // q, k, v (gates and outputs are contiguous [B, H, L, D])
  int gw, gh, heads;  // fused locality gate only: token grid and heads per batch element
  int wide_gates;     // nonzero: skip the fp16 score variant from the start
  int dual_first;     // kModeStateDual: first item of the gradient-state set (= items of the plain set)
};

template <bool FWD, int MODE, int NG, bool F16, bool GATE>
__device__ __forceinline__ int wave_loop(const uint16_t* q, const uint16_t* k, const uint16_t* v, const uint16_t* g,
                                         const uint16_t* g_other, uint16_t* o, const Geometry& geo, int item, int c,
                                         int lane, char* lds, float oscale, bool bidir, float* state_ws,
                                         const float* gate_w) {
  constexpr bool OUT = !is_state_mode(MODE);
  constexpr int DK = 16 * NG;
  // descriptors of this wave's chunk of an item; past the last item (or for a chunk with no tokens) they are empty
  auto locate = [&](int it, ChunkSrc& src, rsrc_t& dst) {
    int nvalid = 0;
    size_t off = 0, tok = 0;
    int b = 0, hd = 0;
    const uint16_t *kk = k, *vv = v, *gg = g;
    if (it < geo.nitems) {
      int it2 = it;
      if (MODE == kModeStateDual && it >= geo.dual_first) it2 = it - geo.dual_first, kk = q, vv = o, gg = g_other;
      const int seq = it2 / geo.nseg, seg = it2 - seq * geo.nseg;
      const int seg_tokens = min(geo.seg_len, geo.L - seg * geo.seg_len);
      nvalid = min(max(seg_tokens - c * geo.cw, 0), geo.cw);
      tok = (size_t)seg * geo.seg_len + (size_t)(nvalid > 0 ? c * geo.cw : 0);
      off = (size_t)seq * geo.L + tok;  // in tokens
      b = seq / geo.H, hd = seq - b * geo.H;
    }
    if (is_pitched(MODE)) {
      src.q_pitch = 2u * geo.sq.token, src.k_pitch = 2u * geo.sk.token, src.v_pitch = 2u * geo.sv.token;
      src.q = chunk_rsrc(q + b * geo.sq.batch + hd * geo.sq.head + tok * geo.sq.token, nvalid, src.q_pitch);
      src.k = chunk_rsrc(kk + b * geo.sk.batch + hd * geo.sk.head + tok * geo.sk.token, nvalid, src.k_pitch);
      src.v = chunk_rsrc(vv + b * geo.sv.batch + hd * geo.sv.head + tok * geo.sv.token, nvalid, src.v_pitch);
    } else {
      src.q_pitch = src.k_pitch = 2 * DK, src.v_pitch = 128;
      src.q = chunk_rsrc(q + off * DK, nvalid, 2 * DK);
      src.k = chunk_rsrc(kk + off * DK, nvalid, 2 * DK);
      src.v = chunk_rsrc(vv + off * 64, nvalid, 128);
    }
    src.g = chunk_rsrc(gg + off * DK, nvalid, 2 * DK);
    dst = chunk_rsrc(o + off * 64, nvalid, 128);
  };
  Prefetch<NG> pf;
  ChunkSrc cur;
  rsrc_t dst;
  locate(item, cur, dst);
  if (item < geo.nitems) {
    if (FWD) issue_first_phase<FWD, OUT, NG, is_pitched(MODE)>(cur, lane & 31, lane >> 5, pf);
    else issue_gates<NG>(cur, lane & 31, lane >> 5, pf);
  }
  for (; item < geo.nitems; item += gridDim.x) {
    ChunkSrc nxt;
    rsrc_t dst_next;
    locate(item + gridDim.x, nxt, dst_next);
    float* state = state_ws ? state_ws + ((size_t)item * 2 + (FWD ? 0 : 1)) * kStateFloats : nullptr;
    asm volatile("" : "+v"(lane));  // per-lane constants are rebuilt per item instead of living across the loop
    GateCtx gate{};
    if (GATE) {  // slab mode: item = sequence = batch element * heads + head
      const int nvalid = min(max(geo.L - c * geo.cw, 0), geo.cw);
      gate = GateCtx{gate_w + (size_t)(item % geo.heads) * (64 * 9), geo.gw, geo.gh, c * geo.cw, nvalid};
    }
    const bool strict = MODE == kModeStateDual && item >= geo.dual_first;
    const bool ok =
        direction_wave<FWD, MODE, NG, F16, GATE>(cur, nxt, dst, c, lane, lds, oscale, bidir, state, pf, gate, strict);
    // (D) the next item reuses the LDS regions.  Not needed after an fp16 slab without the fused gate: what a wave
    // writes before the next barrier A is its own (k~ scratch, anchors, contribution fragments: read by others only
    // between A and C of the same slab), and the output half it sends after the next A was read by its partner
    // before that wave could reach the next A.  (Measured: -2.0 us on the Dk = 32 slab shape, +0.7 us at Dk = 64,
    // where the waves that run ahead take issue slots from the late ones' stores: dropped for Dk = 32 only.)
    if (!(is_slab(MODE) && F16 && !GATE && NG == 2 && ok)) lds_barrier();
    if (F16 && !ok) break;  // this item again, and all that follow, with split-bf16 scores
    cur = nxt;
    dst = dst_next;
  }
  return item;
}

// The items of one wave: fp16 score operands until a segment refuses them, split bf16 from there on.
template <bool FWD, int MODE, int NG, bool GATE>
__device__ __forceinline__ void wave_items(const uint16_t* q, const uint16_t* k, const uint16_t* v, const uint16_t* g,
                                           const uint16_t* g_other, uint16_t* o, const Geometry& geo, int c, int lane,
                                           char* lds, float oscale, bool bidir, float* state_ws, const float* gate_w) {
  int item = (int)blockIdx.x;
  // (a caller that knows its gates to be strong starts with the split-bf16 variant: no segment is walked in vain)
  if (!geo.wide_gates)
    item = wave_loop<FWD, MODE, NG, true, GATE>(q, k, v, g, g_other, o, geo, item, c, lane, lds, oscale, bidir,
                                                state_ws, gate_w);
  wave_loop<FWD, MODE, NG, false, GATE>(q, k, v, g, g_other, o, geo, item, c, lane, lds, oscale, bidir, state_ws,
                                        gate_w);
}

}  // namespace

template <int MODE, int NG, bool GATE = false>
__global__ __launch_bounds__(512) void gla_mfma_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ k,
                                                       const uint16_t* __restrict__ v, const uint16_t* __restrict__ gf,
                                                       const uint16_t* __restrict__ gb, uint16_t* __restrict__ o,
                                                       Geometry geo, float oscale, float* state_ws,
                                                       const float* __restrict__ gate_w) {
  extern __shared__ __align__(16) char lds[];
  const int tid = threadIdx.x;
  const int wi = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: region / chunk addressing stays scalar
  const int lane = tid & 63;
  const int c = wi & 3;
  const bool bidir = gb != nullptr;
  if (tid == 0) *reinterpret_cast<int*>(lds + kLdsVeto) = 0;
  lds_barrier();
  if (wi < 4) {
    wave_items<true, MODE, NG, GATE>(q, k, v, gf, gb, o, geo, c, lane, lds, oscale, bidir, state_ws, gate_w);
  } else if (bidir) {
    wave_items<false, MODE, NG, GATE>(q, k, v, gb, gf, o, geo, c, lane, lds, oscale, bidir, state_ws, gate_w);
  } else {
    // idle half of a one-direction launch: keeps the barrier count of the working waves, including the segment
    // that is walked twice when the fp16 variant is refused
    const int* veto = reinterpret_cast<const int*>(lds + kLdsVeto);
    int item = blockIdx.x;
    if (!geo.wide_gates)
    for (; item < geo.nitems; item += gridDim.x) {
      lds_barrier();  // (A)
      const bool refused = __builtin_amdgcn_readfirstlane(*veto) != 0;
      if (!refused) {  // a refused segment leaves after barrier A
        if (!is_slab(MODE)) lds_barrier();  // (B: not in the fp16 variant of whole slabs)
        lds_barrier();
      }
      if (!is_slab(MODE) || NG != 2 || refused) lds_barrier();  // (D: only behind a refused segment for Dk = 32 fp16 slabs)
      if (refused) break;
    }
    for (; item < geo.nitems; item += gridDim.x) {
      lds_barrier();
      lds_barrier();
      lds_barrier();
      lds_barrier();
    }
  }
}

// Chains the segments of every sequence: in place, the workspace slot of segment s (its own contribution U_s and
// decay D_s) is replaced by the state entering it,  S_in(s') = D_s * S_in(s) + U_s  with s' the next segment in the
// direction's walk order.  One thread per state element; all accesses are coalesced (unit order is kept).  The
// contributions and decays of eight segments are fetched together, so that the serial part is arithmetic only.
// The causal op may start from a caller's state and hand the last one back (init / final: fp32 [nseq, Dk, Dv] row-major,
// null: zero / not wanted; one direction only): the thread of state element e is also the one that knows its row
// (k channel) and column (v channel).
// maxima (null: not wanted): [nseq][2 directions][kGlaScanMaxima], the largest |state entering a segment| each block saw.
__global__ __launch_bounds__(256) void gla_segment_scan_kernel(float* state_ws, int nseq, int nseg, int ndir, int ng,
                                                               const float* __restrict__ init, float* __restrict__ final,
                                                               float* __restrict__ maxima) {
  static_assert(64 * 64 / 256 == kGlaScanMaxima, "one partial maximum per block of the scan");
  __shared__ float wave_top[4];
  const int e = blockIdx.x * 256 + threadIdx.x;  // element in unit order: ((u*64 + lane)*4 + m)
  const int seq = blockIdx.y / ndir, dir = blockIdx.y % ndir;
  if (seq >= nseq) return;
  const int m = e & 3, lane = (e >> 2) & 63, u = e >> 8;
  const int pk = u >> 3, cq = u & 3, h = lane >> 5;
  if (cq >= ng) {  // register quads beyond Dk/16 carry no channel (a whole block at a time: u is block-uniform)
    if (maxima && threadIdx.x == 0) maxima[((size_t)seq * 2 + dir) * kGlaScanMaxima + blockIdx.x] = 0.f;
    return;
  }
  const int ch = 8 * ng * h + 8 * cq + 2 * m + pk;
  constexpr int kBatch = 24;  // (a 4096-token sequence: 16 to 19 segments, fetched in one round)
  float S = 0.f, top = 0.f;
  // column of the state held by (lane, unit): the v channel the accumulator column r of output tile pv belongs to
  const int vch = 2 * cpair<4>(lane & 31) + ((u >> 2) & 1);
  const size_t rc = ((size_t)seq * (16 * ng) + ch) * 64 + vch;
  if (init) S = init[rc];
  for (int i0 = 0; i0 < nseg; i0 += kBatch) {
    float us[kBatch], ds[kBatch];
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      const int i = min(i0 + j, nseg - 1);
      const int seg = dir == 0 ? i : nseg - 1 - i;
      const float* slot = state_ws + (((size_t)seq * nseg + seg) * 2 + dir) * kStateFloats;
      us[j] = slot[e];
      ds[j] = slot[64 * 64 + ch];
    }
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      const int i = i0 + j;
      if (i < nseg) {
        const int seg = dir == 0 ? i : nseg - 1 - i;
        state_ws[(((size_t)seq * nseg + seg) * 2 + dir) * kStateFloats + e] = S;
        top = fmaxf(top, fabsf(S));
        S = __builtin_fmaf(ds[j], S, us[j]);
      }
    }
  }
  if (final) final[rc] = S;
  if (maxima) {  // (uniform: every thread of the block is still here)
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) top = fmaxf(top, __shfl_xor(top, s, 64));
    if ((threadIdx.x & 63) == 0) wave_top[threadIdx.x >> 6] = top;
    __syncthreads();
    if (threadIdx.x == 0)
      maxima[((size_t)seq * 2 + dir) * kGlaScanMaxima + blockIdx.x] =
          fmaxf(fmaxf(wave_top[0], wave_top[1]), fmaxf(wave_top[2], wave_top[3]));
  }
}

// tiles: the segments of the tile-pair output pass (whole 32-token tiles) instead of this kernel's own
static Geometry make_geometry(int nseq, int L, bool tiles = false) {
  Geometry g{};
  g.L = L;
  g.nseg = tiles ? gla_tile_segments(L) : gla_segments(L);
  g.seg_len = tiles ? 32 * gla_tile_segment_tiles(L) : gla_segment_len(L);
  g.cw = (g.seg_len + 3) / 4;
  g.nitems = nseq * g.nseg;
  return g;
}
// plain [B, H, L, D] layout of a tensor, or the caller's strides (batch, head, token; channels contiguous)
static Strides make_strides(const long long* given, int H, int L, int D) {
  if (given && given[2] != 0) return Strides{given[0], given[1], (int)given[2]};
  return Strides{(long long)H * L * D, (long long)L * D, D};
}

// the padded grid must fit the staging cells: whole padded rows per region half, eight halves
bool gla_mfma_gate_grid_ok(int rows, int cols) {
  if (rows <= 0 || cols <= 0 || cols + 2 > kGateCellsPerRegion) return false;
  return rows + 2 <= 8 * (kGateCellsPerRegion / (cols + 2));
}

bool gla_mfma_supported(const GlaArgs& a) {
  return a.io_dtype == 1 && a.gate_dtype == 1 && (a.Dk == 64 || a.Dk == 32) && a.Dv == 64;
}

// (sized for either segmentation: the tile-pair output pass cuts finer, and wants the scan's maxima behind the slots)
size_t gla_mfma_workspace(int B, int H, int L, int Dk, int Dv) {
  if ((Dk != 64 && Dk != 32) || Dv != 64 || L <= 256) return 0;
  const Geometry g = make_geometry(B * H, L), gt = make_geometry(B * H, L, true);
  const size_t items = g.nitems > gt.nitems ? g.nitems : gt.nitems;
  return (items * 2 * kStateFloats + (size_t)B * H * 2 * kGlaScanMaxima) * sizeof(float);
}

// with an initial or final state every sequence goes through the segment passes, also a single-segment one
size_t gla_mfma_state_workspace(int B, int H, int L, int Dk, int Dv) {
  if ((Dk != 64 && Dk != 32) || Dv != 64) return 0;
  const Geometry g = make_geometry(B * H, L);
  return (size_t)g.nitems * 2 * kStateFloats * sizeof(float);
}

constexpr int kMaxDevices = 64;

template <int NG>
static int launch_gla_mfma_t(const GlaArgs& a, int num_cu, int dev) {
  // the attribute is per device; concurrent first calls only repeat an idempotent setting
  static bool attr_done_dev[kMaxDevices] = {};
  bool& attr_done = attr_done_dev[dev];
  if (!attr_done) {
    const void* kernels[6] = {reinterpret_cast<const void*>(gla_mfma_kernel<kModeSlab, NG>),
                              reinterpret_cast<const void*>(gla_mfma_kernel<kModeSlabPitched, NG>),
                              reinterpret_cast<const void*>(gla_mfma_kernel<kModeState, NG>),
                              reinterpret_cast<const void*>(gla_mfma_kernel<kModeChain, NG>),
                              reinterpret_cast<const void*>(gla_mfma_kernel<kModeSlab, NG, true>),
                              reinterpret_cast<const void*>(gla_mfma_kernel<kModeStateDual, NG>)};
    for (const void* kf : kernels)
      if (hipFuncSetAttribute(kf, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsTotal) != hipSuccess) return -5;
    attr_done = true;
  }
  // long sequences whose output pass the tile-pair kernel can do are cut its way
  static const bool chunked_only = [] {
    const char* e = getenv("VIG_GLA_CHUNKED_SLABS");
    return e && e[0] == '1';
  }();
  const bool tile_chain = !chunked_only && !a.state_pass && gla_tiles_chain_supported(a);
  Geometry geo = make_geometry(a.B * a.H, a.L, tile_chain);
  geo.wide_gates = a.wide_gates;
  geo.H = a.H;
  geo.sq = make_strides(a.q_strides, a.H, a.L, a.Dk);
  geo.sk = make_strides(a.k_strides, a.H, a.L, a.Dk);
  geo.sv = make_strides(a.v_strides, a.H, a.L, a.Dv);
  // q, k, v read in place from wider rows: whole-sequence slabs only; rows 16-byte aligned, pitches within the
  // descriptors' 32-bit extents
  const bool pitched = a.q_strides || a.k_strides || a.v_strides;
  if (pitched) {
    if (geo.nseg != 1 || a.state_pass || a.init_state || a.final_state) return -95;
    for (const Strides* st : {&geo.sq, &geo.sk, &geo.sv})
      if (st->token <= 0 || st->token % 8 != 0 || st->batch % 8 != 0 || st->head % 8 != 0 || st->token > (1 << 20))
        return -22;
  }
  int grid = geo.nitems < num_cu ? geo.nitems : num_cu;
  const uint16_t* q = (const uint16_t*)a.q;
  const uint16_t* k = (const uint16_t*)a.k;
  const uint16_t* v = (const uint16_t*)a.v;
  const uint16_t* gf = (const uint16_t*)a.g_fwd;
  const uint16_t* gb = (const uint16_t*)a.g_bwd;
  uint16_t* o = (uint16_t*)a.o;
  const float oscale = a.scale * a.out_scale;
  const float* no_gate = nullptr;
  if (a.state_pass) {
    // one state pass alone: contributions and decays of every (sequence, segment, direction), no scan, no outputs
    if (a.state_pass == 2) {
      // plain set on (k, v, gates) and gradient-state set on (q for k, o for v, gates exchanged) in one launch
      if (!gb) return -22;
      geo.dual_first = geo.nitems;
      geo.nitems *= 2;
      grid = geo.nitems < num_cu ? geo.nitems : num_cu;
      hipLaunchKernelGGL((gla_mfma_kernel<kModeStateDual, NG>), dim3(grid), dim3(512), kLdsTotal, a.stream, q, k, v,
                         gf, gb, o, geo, oscale, (float*)a.workspace, no_gate);
    } else
      hipLaunchKernelGGL((gla_mfma_kernel<kModeState, NG>), dim3(grid), dim3(512), kLdsTotal, a.stream, q, k, v, gf, gb,
                         o, geo, oscale, (float*)a.workspace, no_gate);
  } else if (a.gate_w) {
    // fused locality gate: whole-sequence slabs, both directions, the padded token grid must fit the staging cells
    if (geo.nseg != 1 || !gb || a.gate_cols <= 0 || a.gate_rows <= 0 || a.gate_cols * a.gate_rows != a.L ||
        !gla_mfma_gate_grid_ok(a.gate_rows, a.gate_cols))
      return -95;
    geo.gw = a.gate_cols;
    geo.gh = a.gate_rows;
    geo.heads = a.H;
    if (pitched) return -95;
    hipLaunchKernelGGL((gla_mfma_kernel<kModeSlab, NG, true>), dim3(grid), dim3(512), kLdsTotal, a.stream, q, k, v, gf,
                       gb, o, geo, oscale, (float*)nullptr, a.gate_w);
  } else if (geo.nseg == 1 && !a.init_state && !a.final_state) {
    if (pitched)
      hipLaunchKernelGGL((gla_mfma_kernel<kModeSlabPitched, NG>), dim3(grid), dim3(512), kLdsTotal, a.stream, q, k, v,
                         gf, gb, o, geo, oscale, (float*)nullptr, no_gate);
    else
      hipLaunchKernelGGL((gla_mfma_kernel<kModeSlab, NG>), dim3(grid), dim3(512), kLdsTotal, a.stream, q, k, v, gf, gb,
                         o, geo, oscale, (float*)nullptr, no_gate);
  } else {
    if ((a.init_state || a.final_state) && gb) return -22;  // a state in or out belongs to the causal op
    float* ws = (float*)a.workspace;
    hipLaunchKernelGGL((gla_mfma_kernel<kModeState, NG>), dim3(grid), dim3(512), kLdsTotal, a.stream, q, k, v, gf, gb, o,
                       geo, oscale, ws, no_gate);
    const int ndir = gb ? 2 : 1;
    float* maxima = tile_chain ? ws + (size_t)geo.nitems * 2 * kStateFloats : nullptr;
    hipLaunchKernelGGL(gla_segment_scan_kernel, dim3(64 * 64 / 256, a.B * a.H * ndir), dim3(256), 0, a.stream, ws,
                       a.B * a.H, geo.nseg, ndir, NG, a.init_state, a.final_state, maxima);
    if (tile_chain) {
      if (hipGetLastError() != hipSuccess) return -5;
      return launch_gla_tiles_chain(a, ws, maxima);
    }
    hipLaunchKernelGGL((gla_mfma_kernel<kModeChain, NG>), dim3(grid), dim3(512), kLdsTotal, a.stream, q, k, v, gf, gb, o,
                       geo, oscale, ws, no_gate);
  }
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

int launch_gla_mfma(const GlaArgs& a) {
  // whole-sequence slabs go to the tile-pair kernel (VIG_GLA_CHUNKED_SLABS=1 keeps them here: comparisons only)
  static const bool chunked_slabs = [] {
    const char* e = getenv("VIG_GLA_CHUNKED_SLABS");
    return e && e[0] == '1';
  }();
  if (!chunked_slabs && gla_tiles_supported(a)) return launch_gla_tiles(a);
  static int num_cu_dev[kMaxDevices] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return -5;
  int& num_cu = num_cu_dev[dev];
  if (num_cu == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return -5;
    num_cu = n > 0 ? n : 256;
  }
  return a.Dk == 64 ? launch_gla_mfma_t<4>(a, num_cu, dev) : launch_gla_mfma_t<2>(a, num_cu, dev);
}


}  // namespace vig
