// Backward of the bidirectional GLA op on MFMA tiles (gfx950): bf16 tensors and gates, Dk in {32, 64}, Dv = 64.
// L <= 256 is one slab per (batch, head); a longer sequence is cut into the forward's segments (<= 256 tokens), each
// handled like a slab plus three products with the states that link it to the other segments (see SEG below).
//
// Per direction the whole (batch, head) slab is one quadratic form (no chunk states): with G the inclusive
// cumulative log-gate along the direction and the anchor a = G_total / 2,
//   q~_i = q_i e^{G_i - a},  k~_j = k_j e^{a - G_j}   (both within e^{|G_total|/2} of the inputs),
//   P_ij = q~_i . k~_j,  A_ij = do_i . v_j            for the pairs the direction keeps (j <= i forward, j >= i reverse),
//   dv_j = s sum_i P_ij do_i,   dq_i = s e^{G_i - a} (.) sum_j A_ij k~_j,   dk_j = s e^{a - G_j} (.) sum_i A_ij q~_i,
//   dg_t = sum over the tokens i the gate of t acts on (i >= t forward, i <= t reverse) of q_i (.) dq_i - k_i (.) dk_i,
// s = scale * out_scale.  This is the natural-order form of flash-linear-attention/fla/ops/gla/chunk_fuse.py:413-518
// with one chunk per sequence; the flip-concat glue of classification/models/vig.py:407-426 never materialises.
//
// One persistent workgroup of 8 waves per CU walks slabs; wave w owns the 32-token tile w.  Per direction the
// workgroup stages q~, k~ (and once v, do) as bf16 rows in LDS; then wave w accumulates dq of its tile over the key
// tiles the direction keeps, and dk, dv of its tile over the query tiles: score tiles P, A come out of the matrix
// cores in the register layout that feeds the next product directly (mfma_tiles.h), operands with tokens in the
// contraction slots are read from the LDS rows as dwords.  The two directions take turns in LDS; a tile that is heavy
// in one direction is light in the other, so over both every wave does the same amount of work.  dg needs a running
// sum over tokens: inside the tile the lanes (= tokens) add up q dq - k dk by lane shifts, the tile totals are
// exchanged through LDS.  Loads of the next direction (or slab) are issued before that exchange, when the accumulators
// are dead (its gates a phase earlier), and its cumulative gates and their tile totals are prepared there as well.
// Two barriers per direction: staged q~ / k~, and the totals of q dq - k dk together with the next direction's gate
// totals; the second also tells that nobody reads this direction's staged rows any more.
//
// Slabs whose gate totals exceed the anchor's range (|G_total| / 2 * log2(e) > 60 in some channel) are not computed
// here: the workgroup raises the slab's flag and the token-recurrent kernel, launched afterwards with that flag
// array, computes exactly those.
#include "common.h"
#include "launch.h"
#include "mfma_tiles.h"

namespace vig {

namespace {

constexpr int kBwdTiles = 8;                                // 32-token tiles per slab
constexpr int kBwdMatBytes = kBwdTiles * 32 * kKtStride * 2;  // one staged 256 x 64 bf16 matrix, 144-byte rows
constexpr int kBwdLdsQ = 0;
constexpr int kBwdLdsK = kBwdMatBytes;
constexpr int kBwdLdsV = 2 * kBwdMatBytes;
constexpr int kBwdLdsDo = 3 * kBwdMatBytes;
constexpr int kBwdLdsTot = 4 * kBwdMatBytes;           // [8][64] f32: gate totals of the tiles
constexpr int kBwdLdsOff = kBwdLdsTot + 8 * 64 * 4;    // [8][64] f32: per wave, (prefix - anchor) of its tile
constexpr int kBwdLdsDgTot = kBwdLdsOff + 8 * 64 * 4;  // [8][64] f32: totals of q dq - k dk of the tiles
constexpr int kBwdLdsTotal = kBwdLdsDgTot + 8 * 64 * 4;
constexpr float kBwdHalfRange = 60.0f;


// fragment of 8 consecutive channels (k-step ks, lane half h) of a staged row: contraction over channels
__device__ __forceinline__ u32x4_t row_frag(const uint16_t* mat, int row, int ks, int h) {
  return *reinterpret_cast<const u32x4_t*>(mat + row * kKtStride + 16 * ks + 8 * h);
}

// accumulator tile (rows 8g+4h+m in registers, column = lane) -> operand fragments with its rows in the contraction
// slots, k-steps t = 0, 1
__device__ __forceinline__ void tile_frags(const f32x16_t& T, u32x4_t (&f)[2]) {
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int x = 0; x < 4; ++x) f[t][x] = pack_bf16x2(T[8 * t + 2 * x], T[8 * t + 2 * x + 1]);
}

// keeps the entries of a diagonal tile (diag) the direction uses, and all of any other tile; ROWS_ARE_QUERIES: rows
// i, column j (else rows j, column i).  Selects, not a branch around them: a branch between the matrix instructions
// and the first vector read of their result left that read without its wait states in one build of this kernel.
template <bool FWD, bool ROWS_ARE_QUERIES>
__device__ __forceinline__ void mask_diag(f32x16_t& T, int r, int h, bool diag) {
#pragma unroll
  for (int c = 0; c < 16; ++c) {
    const int row = 8 * (c >> 2) + 4 * h + (c & 3);
    const int i = ROWS_ARE_QUERIES ? row : r, j = ROWS_ARE_QUERIES ? r : row;
    const bool keep = !diag || (FWD ? (j <= i) : (j >= i));
    T[c] = keep ? T[c] : 0.f;
  }
}

// Inclusive running sums over the 32 tokens of a lane half (lanes 32h .. 32h + 31, in lane order) for N values at
// once: four shifted adds inside the rows of 16 lanes (lanes shifted in from outside a row read zero), then lane 15 of
// the lower row added to every lane of the upper one.  Step by step over all values, so that consecutive lane-shift
// instructions never wait for each other's results.
template <int CTRL>
__device__ __forceinline__ float row_shifted(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
template <int CTRL, int N>
__device__ __forceinline__ void add_row_shifted(float (&x)[N]) {
#pragma unroll
  for (int i = 0; i < N; ++i) x[i] += row_shifted<CTRL>(x[i]);
  __builtin_amdgcn_sched_barrier(0);
}
template <int N>
__device__ __forceinline__ void half_prefix_sums(float (&x)[N]) {
  __builtin_amdgcn_sched_barrier(0);
  add_row_shifted<0x111>(x);  // row_shr:1
  add_row_shifted<0x112>(x);  // row_shr:2
  add_row_shifted<0x114>(x);  // row_shr:4
  add_row_shifted<0x118>(x);  // row_shr:8
#pragma unroll
  for (int i = 0; i < N; ++i)  // row_bcast:15 into rows 1 and 3 (row mask 0b1010); rows 0 and 2 keep the zero
    x[i] += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x[i]), 0x142, 0xa, 0xf, false));
}

struct BwdSlab {
  const uint16_t *q, *k, *v, *gf, *gb, *d_o;
  uint16_t *dq, *dk, *dv, *dgf, *dgb;
  // segments of a long sequence only (direction 1 follows direction 0 in each array):
  const uint16_t *sp, *rp, *rpt;  // sqrt(D) S_in as [k channel][v], sqrt(D) R_out as [k channel][v] and as [v][k channel]
  const float* carry;             // [2 directions][2 partial sums][64]: q dq - k dk summed over the segments walked later
  int L;                          // tokens of this slab / segment
};
constexpr int kBwdStateElems = 64 * 64;

// What a wave loads for one direction of one slab (its own 32-token tile), issued one phase ahead.
template <int NG>
struct BwdLoads {
  uint32_t gD[2][8];             // gate dwords (tokens in the contraction slots)
  u32x4_t rawq[NG], rawk[NG];    // q and k rows
  u32x4_t rawv[4], rawd[4];      // v and do rows (first direction of a slab only)
};
struct BwdNext {  // the direction whose loads are issued while this one finishes
  BwdSlab sl;
  const uint16_t* g;
  int L;  // 0: nothing follows (empty descriptors, no memory traffic)
};
template <int NG>
__device__ __forceinline__ void issue_bwd_gate_loads(const BwdNext& n, int w, int r, int h, BwdLoads<NG>& ld) {
  constexpr int DK = 16 * NG;
  const int rows = __builtin_amdgcn_readfirstlane(min(max(n.L - 32 * w, 0), 32));  // (scalar: descriptors stay in SGPRs)
  issue_tdwords<0, 2, NG>(chunk_rsrc(n.g + (size_t)32 * w * DK, rows, 2 * DK), r, h, ld.gD);
}
template <bool WITH_VDO, int NG>
__device__ __forceinline__ void issue_bwd_row_loads(const BwdNext& n, int w, int r, int h, BwdLoads<NG>& ld) {
  constexpr int DK = 16 * NG;
  const int rows = __builtin_amdgcn_readfirstlane(min(max(n.L - 32 * w, 0), 32));
  const size_t tk = (size_t)32 * w * DK, tv = (size_t)32 * w * 64;
  issue_raw_tile<NG>(chunk_rsrc(n.sl.q + tk, rows, 2 * DK), 0, r, h, ld.rawq);
  issue_raw_tile<NG>(chunk_rsrc(n.sl.k + tk, rows, 2 * DK), 0, r, h, ld.rawk);
  if (WITH_VDO) {
    issue_raw_tile<4>(chunk_rsrc(n.sl.v + tv, rows, 128), 0, r, h, ld.rawv);
    issue_raw_tile<4>(chunk_rsrc(n.sl.d_o + tv, rows, 128), 0, r, h, ld.rawd);
  }
}

// Tile-local cumulative gates of the direction whose gate dwords have arrived: G^T = g^T T, lane = token, registers =
// channels HC*h + 8g + 2m + p; the tile total (at the tile's last token in walking order) goes to `tot`.
template <bool FWD, int NG>
__device__ __forceinline__ void bwd_cumulate_gates(const BwdLoads<NG>& ld, int w, int lane, char* lds, f32x16_t (&G)[2]) {
  constexpr int HC = 8 * NG;
  const int r = lane & 31, h = lane >> 5;
  float* tot = reinterpret_cast<float*>(lds + kBwdLdsTot);
  u32x4_t gfrag[2][2];
  finish_tfrags<2>(ld.gD, gfrag);  // (rows that carry no channel, NG = 2, hold zeros)
  const u32x4_t tri0 = tri_frag<FWD>(0, 0, r, h), tri1 = tri_frag<FWD>(1, 0, r, h);
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    f32x16_t z = {0.f};
    z = mfma(gfrag[0][p], tri0, z);
    G[p] = mfma(gfrag[1][p], tri1, z);
  }
  if (r == (FWD ? 31 : 0)) {
#pragma unroll
    for (int c = 0; c < 4 * NG; ++c) {
      const int ch = HC * h + 8 * (c >> 2) + 2 * (c & 3);
      tot[w * 64 + ch] = G[0][c];
      tot[w * 64 + ch + 1] = G[1][c];
    }
  }
}

// One direction of one slab, for wave w (tile w).  dv accumulates over both directions (raw, unscaled).  The first
// direction (FIRST, not LAST) stages v and do and parks its dq and dk, rounded to bf16, in the output tensors; the
// second (LAST, not FIRST) adds its own to them and stores dq, dk, dv.  A one-direction (causal) launch runs a single
// direction that is both.  Returns false, for every wave alike and before it has stored anything,
// when the gates are out of range.
// SEG: the slab is a segment of a longer sequence.  With S_in the state entering it along the direction, R_out the
// gradient of the state leaving it, a = half the segment's gate total and ' = times e^a per k channel:
//   dq^_i += S_in' do_i,   dk^_j += R_out' v_j,   dv_j += R_out'^T k~_j
// (the e^{G_i - a}, e^{a - G_j} factors applied to dq^, dk^ at the end turn e^a into e^{G_i}, e^{T - G_j}), and the
// running sum of the gate gradient starts from the total of q dq - k dk over the segments walked later.
template <bool FWD, bool FIRST, bool LAST, int NG, bool SEG>
__device__ __forceinline__ bool bwd_direction(const BwdSlab& sl, int L, int ntiles, int w, int lane, char* lds,
                                              float s, f32x16_t (&dv)[2], u32x4_t (&keepq)[NG], u32x4_t (&keepk)[NG],
                                              BwdLoads<NG>& ld, const BwdNext& nxt, f32x16_t (&G)[2]) {
  // where the first direction's dq, dk (bf16) wait for the second: in registers when the kernel has them to spare
  // (Dk = 32), else parked in the output tensors
  constexpr bool kKeepInRegs = NG == 2;
  constexpr bool stage_vdo = FIRST;
  constexpr int DK = 16 * NG;   // channels of q, k and the gates
  constexpr int HC = 8 * NG;    // channels per lane half
  asm volatile("" : "+v"(lane));  // per-lane constants are rebuilt per direction instead of living across the slab loop
  const int r = lane & 31, h = lane >> 5;
  uint16_t* Q = reinterpret_cast<uint16_t*>(lds + kBwdLdsQ);
  uint16_t* K = reinterpret_cast<uint16_t*>(lds + kBwdLdsK);
  uint16_t* V = reinterpret_cast<uint16_t*>(lds + kBwdLdsV);
  uint16_t* DO = reinterpret_cast<uint16_t*>(lds + kBwdLdsDo);
  float* tot = reinterpret_cast<float*>(lds + kBwdLdsTot);
  float* offs = reinterpret_cast<float*>(lds + kBwdLdsOff) + w * 64;
  float* dgtot = reinterpret_cast<float*>(lds + kBwdLdsDgTot);
  const int rows = __builtin_amdgcn_readfirstlane(min(max(L - 32 * w, 0), 32));  // valid tokens of this wave's tile
  const size_t tk = (size_t)32 * w * DK, tv = (size_t)32 * w * 64;

  // ---- this tile's loads were issued a phase ago; v and do rows go to LDS once per slab (nobody reads the previous
  // slab's any more; the next barrier makes them visible) ----
  if (stage_vdo) {
    store_kt<4>(V, 32 * w + r, h, ld.rawv);
    store_kt<4>(DO, 32 * w + r, h, ld.rawd);
  }
  u32x4_t rawq[NG], rawk[NG];
#pragma unroll
  for (int i = 0; i < NG; ++i) rawq[i] = ld.rawq[i], rawk[i] = ld.rawk[i];

  // ---- the cumulative gates G of this tile and every tile's total were left by the previous direction's tail (or
  // the kernel's head), one barrier ago ----
  // lane = channel: gates before this tile in walking order, minus the anchor (half the slab total)
  bool out_of_range;
  {
    float pre = 0.f, all = 0.f;
#pragma unroll
    for (int t = 0; t < kBwdTiles; ++t) {
      const float x = lane < DK ? tot[t * 64 + lane] : 0.f;
      all += x;
      pre += (FWD ? (t < w) : (t > w)) ? x : 0.f;
    }
    offs[lane] = pre - 0.5f * all;
    out_of_range = __builtin_amdgcn_ballot_w64(fabsf(all) * (0.5f * kLog2e) > kBwdHalfRange) != 0;
  }
  if (out_of_range) return false;  // same totals in every wave: the whole workgroup leaves together
  wave_lds_sync();
  // x = (G - a) * log2(e) per (token, channel): q~ = q 2^x, k~ = k 2^-x
  f32x16_t x[2] = {{0.f}, {0.f}};
#pragma unroll
  for (int gq = 0; gq < NG; ++gq) {
    const f32x4_t o0 = *reinterpret_cast<const f32x4_t*>(offs + HC * h + 8 * gq);
    const f32x4_t o1 = *reinterpret_cast<const f32x4_t*>(offs + HC * h + 8 * gq + 4);
    const float o8[8] = {o0[0], o0[1], o0[2], o0[3], o1[0], o1[1], o1[2], o1[3]};
#pragma unroll
    for (int m = 0; m < 4; ++m)
#pragma unroll
      for (int p = 0; p < 2; ++p) x[p][4 * gq + m] = (G[p][4 * gq + m] + o8[2 * m + p]) * kLog2e;
  }
  {
    u32x4_t qt[NG], kt[NG];
#pragma unroll
    for (int gq = 0; gq < NG; ++gq)
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const int c = 4 * gq + m;
        const float e0 = exp2_fast(x[0][c]), e1 = exp2_fast(x[1][c]);
        const uint32_t wq = rawq[gq][m], wk = rawk[gq][m];
        qt[gq][m] = pack_bf16x2(bf16lo_to_f32(wq) * e0, bf16hi_to_f32(wq) * e1);
        kt[gq][m] = pack_bf16x2(bf16lo_to_f32(wk) * exp2_fast(-x[0][c]), bf16hi_to_f32(wk) * exp2_fast(-x[1][c]));
      }
    store_kt<NG>(Q, 32 * w + r, h, qt);
    store_kt<NG>(K, 32 * w + r, h, kt);
  }
  lds_barrier();  // (2) q~, k~ of every tile visible

  // ---- dq of tile w: over the key tiles J the direction keeps ----
  f32x16_t dqh[2] = {{0.f}, {0.f}};
  if (w < ntiles) {
    u32x4_t doB[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) doB[ks] = row_frag(DO, 32 * w + r, ks, h);
    const int j0 = FWD ? 0 : w, j1 = FWD ? w : ntiles - 1;
    // Two steps in flight: the score tile of the next key tile is on the matrix cores while this one is masked,
    // packed and multiplied on (after the last tile the next one is that tile again, computed and dropped).
    f32x16_t T = {0.f};  // A^T tile: rows j in J, columns i in tile w
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) T = mfma(row_frag(V, 32 * j0 + r, ks, h), doB[ks], T);
#pragma unroll 1
    for (int J = j0; J <= j1; ++J) {
      const int Jn = min(J + 1, j1);
      u32x4_t kf[2][2];
#pragma unroll
      for (int t = 0; t < 2; ++t) load_tfrag_lds<NG>(K + 32 * J * kKtStride, t, r, h, kf[t]);
      f32x16_t Tn = {0.f};
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) Tn = mfma(row_frag(V, 32 * Jn + r, ks, h), doB[ks], Tn);
      mask_diag<FWD, false>(T, r, h, J == w);
      u32x4_t f[2];
      tile_frags(T, f);
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        dqh[0] = mfma(kf[t][0], f[t], dqh[0]);
        dqh[1] = mfma(kf[t][1], f[t], dqh[1]);
      }
      T = Tn;
    }
    if (SEG) {  // the state entering the segment: rows = the k channels of this lane's accumulator rows, over v
      const uint16_t* sp = sl.sp + (FWD ? 0 : kBwdStateElems);
      const bool row_ok = row_has_channel<NG>(r);
      const int row0 = row_ok ? 2 * cpair<NG>(r) : 0;
#pragma unroll
      for (int p = 0; p < 2; ++p)
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          u32x4_t a = *reinterpret_cast<const u32x4_t*>(sp + (row0 + p) * 64 + 16 * ks + 8 * h);
          if (NG != 4 && !row_ok) a = u32x4_t{0u, 0u, 0u, 0u};
          dqh[p] = mfma(a, doB[ks], dqh[p]);
        }
    }
  }
  // dq^ waits as bf16 pairs while the other accumulators are at work
  uint32_t dqp[16];
#pragma unroll
  for (int c = 0; c < 16; ++c) dqp[c] = pack_bf16x2(dqh[0][c], dqh[1][c]);
  // the first direction parked its dq and dk (rounded to bf16) in the output tensors; fetch them under the loops
  const rsrc_t oq = chunk_rsrc(sl.dq + tk, rows, 2 * DK), okk = chunk_rsrc(sl.dk + tk, rows, 2 * DK);
  u32x4_t prevq[NG], prevk[NG];
  if (!FIRST && kKeepInRegs) {
#pragma unroll
    for (int gq = 0; gq < NG; ++gq) prevq[gq] = keepq[gq], prevk[gq] = keepk[gq];
  }
  if (!FIRST && !kKeepInRegs) {
#pragma unroll
    for (int gq = 0; gq < NG; ++gq) {
      const unsigned off = (unsigned)r * (2u * DK) + (2u * HC) * h + 16u * gq;
      prevq[gq] = __builtin_amdgcn_raw_buffer_load_b128(oq, off, 0, 0);
      prevk[gq] = __builtin_amdgcn_raw_buffer_load_b128(okk, off, 0, 0);
    }
  }
  // ---- dv and dk of tile w: over the query tiles I the direction keeps.  Dk = 32 has the registers to do both in
  // one loop: the two score tiles of a step are independent, so one's masks and packs run under the other's matrix
  // instructions.  Dk = 64: two loops (fewer live registers). ----
  f32x16_t dkh[2] = {{0.f}, {0.f}};
  if (w < ntiles) {
    const int i0 = FWD ? w : 0, i1 = FWD ? ntiles - 1 : w;
    if constexpr (NG == 2) {
#pragma unroll 1
      for (int I = i0; I <= i1; ++I) {
        f32x16_t P = {0.f}, A = {0.f};  // rows i in I, columns j in tile w
#pragma unroll
        for (int ks = 0; ks < NG; ++ks) P = mfma(row_frag(Q, 32 * I + r, ks, h), row_frag(K, 32 * w + r, ks, h), P);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) A = mfma(row_frag(DO, 32 * I + r, ks, h), row_frag(V, 32 * w + r, ks, h), A);
        mask_diag<FWD, true>(P, r, h, I == w);
        u32x4_t pf[2];
        tile_frags(P, pf);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          u32x4_t df[2];
          load_tfrag_lds<4>(DO + 32 * I * kKtStride, t, r, h, df);
          dv[0] = mfma(df[0], pf[t], dv[0]);
          dv[1] = mfma(df[1], pf[t], dv[1]);
        }
        mask_diag<FWD, true>(A, r, h, I == w);
        u32x4_t af[2];
        tile_frags(A, af);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          u32x4_t qf[2];
          load_tfrag_lds<NG>(Q + 32 * I * kKtStride, t, r, h, qf);
          dkh[0] = mfma(qf[0], af[t], dkh[0]);
          dkh[1] = mfma(qf[1], af[t], dkh[1]);
        }
      }
    } else {
#pragma unroll 1
      for (int I = i0; I <= i1; ++I) {
        f32x16_t P = {0.f};  // rows i in I, columns j in tile w
#pragma unroll
        for (int ks = 0; ks < NG; ++ks) P = mfma(row_frag(Q, 32 * I + r, ks, h), row_frag(K, 32 * w + r, ks, h), P);
        mask_diag<FWD, true>(P, r, h, I == w);
        u32x4_t pf[2];
        tile_frags(P, pf);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          u32x4_t df[2];
          load_tfrag_lds<4>(DO + 32 * I * kKtStride, t, r, h, df);
          dv[0] = mfma(df[0], pf[t], dv[0]);
          dv[1] = mfma(df[1], pf[t], dv[1]);
        }
      }
#pragma unroll 1
      for (int I = i0; I <= i1; ++I) {
        f32x16_t A = {0.f};
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) A = mfma(row_frag(DO, 32 * I + r, ks, h), row_frag(V, 32 * w + r, ks, h), A);
        mask_diag<FWD, true>(A, r, h, I == w);
        u32x4_t af[2];
        tile_frags(A, af);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          u32x4_t qf[2];
          load_tfrag_lds<NG>(Q + 32 * I * kKtStride, t, r, h, qf);
          dkh[0] = mfma(qf[0], af[t], dkh[0]);
          dkh[1] = mfma(qf[1], af[t], dkh[1]);
        }
      }
    }
    if (SEG) {  // the gradient of the state leaving the segment, against this tile's k~ rows (dv) and v rows (dk)
      const uint16_t* rpt = sl.rpt + (FWD ? 0 : kBwdStateElems);
      const int vrow = 2 * cpair<4>(r);
#pragma unroll
      for (int p = 0; p < 2; ++p)
#pragma unroll
        for (int ks = 0; ks < NG; ++ks) {
          const u32x4_t a = *reinterpret_cast<const u32x4_t*>(rpt + (vrow + p) * 64 + 16 * ks + 8 * h);
          dv[p] = mfma(a, row_frag(K, 32 * w + r, ks, h), dv[p]);
        }
      const uint16_t* rp = sl.rp + (FWD ? 0 : kBwdStateElems);
      const bool row_ok = row_has_channel<NG>(r);
      const int row0 = row_ok ? 2 * cpair<NG>(r) : 0;
#pragma unroll
      for (int p = 0; p < 2; ++p)
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          u32x4_t a = *reinterpret_cast<const u32x4_t*>(rp + (row0 + p) * 64 + 16 * ks + 8 * h);
          if (NG != 4 && !row_ok) a = u32x4_t{0u, 0u, 0u, 0u};
          dkh[p] = mfma(a, row_frag(V, 32 * w + r, ks, h), dkh[p]);
        }
    }
  }
  issue_bwd_gate_loads<NG>(nxt, w, r, h, ld);  // the next direction's gates travel under the rest of this one
  // ---- scale back; X = q dq - k dk = s (q~ dq^ - k~ dk^): the exponentials cancel, and the staged rows serve ----
  f32x16_t X[2];
  {
    const rsrc_t ov = chunk_rsrc(sl.dv + tv, rows, 128);
    if (LAST) {
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        u32x4_t xv;
#pragma unroll
        for (int m = 0; m < 4; ++m) xv[m] = pack_bf16x2(dv[0][4 * gq + m] * s, dv[1][4 * gq + m] * s);
        __builtin_amdgcn_raw_buffer_store_b128(xv, ov, (unsigned)r * 128u + 64u * h + 16u * gq, 0, 0);
      }
    }
#pragma unroll
    for (int gq = 0; gq < NG; ++gq) {
      const u32x4_t qrow = *reinterpret_cast<const u32x4_t*>(Q + (32 * w + r) * kKtStride + HC * h + 8 * gq);
      const u32x4_t krow = *reinterpret_cast<const u32x4_t*>(K + (32 * w + r) * kKtStride + HC * h + 8 * gq);
      u32x4_t xq, xk;
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const int c = 4 * gq + m;
        float a[2], b[2];
#pragma unroll
        for (int p = 0; p < 2; ++p) {
          const float dqc = p ? bf16hi_to_f32(dqp[c]) : bf16lo_to_f32(dqp[c]);
          const float dkc = dkh[p][c];
          const float qt = p ? bf16hi_to_f32(qrow[m]) : bf16lo_to_f32(qrow[m]);
          const float kt = p ? bf16hi_to_f32(krow[m]) : bf16lo_to_f32(krow[m]);
          X[p][c] = s * (qt * dqc - kt * dkc);
          a[p] = s * exp2_fast(x[p][c]) * dqc;
          b[p] = s * exp2_fast(-x[p][c]) * dkc;
          if (!FIRST) {
            a[p] += p ? bf16hi_to_f32(prevq[gq][m]) : bf16lo_to_f32(prevq[gq][m]);
            b[p] += p ? bf16hi_to_f32(prevk[gq][m]) : bf16lo_to_f32(prevk[gq][m]);
          }
        }
        xq[m] = pack_bf16x2(a[0], a[1]);
        xk[m] = pack_bf16x2(b[0], b[1]);
      }
      const unsigned off = (unsigned)r * (2u * DK) + (2u * HC) * h + 16u * gq;
      if (!LAST && kKeepInRegs) {
        keepq[gq] = xq;
        keepk[gq] = xk;
      } else {
        __builtin_amdgcn_raw_buffer_store_b128(xq, oq, off, 0, 0);
        __builtin_amdgcn_raw_buffer_store_b128(xk, okk, off, 0, 0);
      }
    }
  }
  // ---- dg: the running sum of X over the tokens the gate acts on.  Inside the tile by lane shifts (lane = token),
  // across tiles through the tile totals in LDS: walking forward a token takes everything from itself to the end,
  // i.e. the totals of this and the later tiles minus what lies before it in the tile. ----
  {
    float pfx[8 * NG];  // [p][c]
#pragma unroll
    for (int p = 0; p < 2; ++p)
#pragma unroll
      for (int c = 0; c < 4 * NG; ++c) pfx[4 * NG * p + c] = X[p][c];
    half_prefix_sums(pfx);
    if (r == 31) {
#pragma unroll
      for (int c = 0; c < 4 * NG; ++c) {
        const int ch = HC * h + 8 * (c >> 2) + 2 * (c & 3);
        dgtot[w * 64 + ch] = pfx[c];
        dgtot[w * 64 + ch + 1] = pfx[4 * NG + c];
      }
    }
    // the next direction's rows travel while this one finishes; its cumulative gates and tile totals are prepared
    // here, so that one barrier serves both exchanges
    issue_bwd_row_loads<LAST, NG>(nxt, w, r, h, ld);
    bwd_cumulate_gates<LAST, NG>(ld, w, lane, lds, G);
    lds_barrier();  // (4) tile totals of X and of the next gates visible; nobody reads q~, k~, v, do of this direction
    {
      const int cl = lane < DK ? lane : 0;
      float run = 0.f;
#pragma unroll
      for (int t = 0; t < kBwdTiles; ++t) {
        const float y = dgtot[t * 64 + cl];
        run += (FWD ? (t >= w) : (t < w)) ? y : 0.f;
      }
      if (SEG) {
        const float* cy = sl.carry + (FWD ? 0 : 128) + cl;
        run += s * (cy[0] + cy[64]);
      }
      offs[lane] = run;
    }
    wave_lds_sync();
    uint16_t* dg = FWD ? sl.dgf : sl.dgb;
    const rsrc_t rdg = chunk_rsrc(dg + tk, rows, 2 * DK);
#pragma unroll
    for (int gq = 0; gq < NG; ++gq) {
      const f32x4_t o0 = *reinterpret_cast<const f32x4_t*>(offs + HC * h + 8 * gq);
      const f32x4_t o1 = *reinterpret_cast<const f32x4_t*>(offs + HC * h + 8 * gq + 4);
      const float o8[8] = {o0[0], o0[1], o0[2], o0[3], o1[0], o1[1], o1[2], o1[3]};
      u32x4_t out;
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const int c = 4 * gq + m;
        float d[2];
#pragma unroll
        for (int p = 0; p < 2; ++p)
          d[p] = FWD ? o8[2 * m + p] - (pfx[4 * NG * p + c] - X[p][c]) : o8[2 * m + p] + pfx[4 * NG * p + c];
        out[m] = pack_bf16x2(d[0], d[1]);
      }
      __builtin_amdgcn_raw_buffer_store_b128(out, rdg, (unsigned)r * (2u * DK) + (2u * HC) * h + 16u * gq, 0, 0);
    }
  }
  return true;
}

}  // namespace

// What the segments of long sequences read besides the tensors (see bwd_direction, SEG): per (sequence, segment) the
// two directions' matrices, written by gla_backward_segment_scan_kernel.
struct BwdSegments {
  const uint16_t *sp, *rp, *rpt;
  const float* carry;
  int nseg, seg_len;
};

template <int NG, bool BIDIR, bool SEG>
__global__ __launch_bounds__(512) void gla_backward_mfma_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k, const uint16_t* __restrict__ v,
    const uint16_t* __restrict__ gf, const uint16_t* __restrict__ gb, const uint16_t* __restrict__ d_o,
    uint16_t* __restrict__ dq, uint16_t* __restrict__ dk, uint16_t* __restrict__ dv, uint16_t* __restrict__ dgf,
    uint16_t* __restrict__ dgb, int* __restrict__ flags, int nslabs, int L, float s, BwdSegments sg) {
  extern __shared__ __align__(16) char lds[];
  const int tid = threadIdx.x;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  // slab i: a whole sequence, or (SEG) segment i % nseg of sequence i / nseg
  auto slab_of = [&](int i) {
    size_t t0 = (size_t)i * L;
    int len = L;
    BwdSlab sl{};
    if (SEG) {
      const int seq = i / sg.nseg, seg = i - seq * sg.nseg;
      t0 = (size_t)seq * L + (size_t)seg * sg.seg_len;
      len = min(sg.seg_len, L - seg * sg.seg_len);
      sl.sp = sg.sp + (size_t)i * 2 * kBwdStateElems;
      sl.rp = sg.rp + (size_t)i * 2 * kBwdStateElems;
      sl.rpt = sg.rpt + (size_t)i * 2 * kBwdStateElems;
      sl.carry = sg.carry + (size_t)i * 256;
    }
    const size_t bk = t0 * (16 * NG), bv = t0 * 64;
    sl.q = q + bk, sl.k = k + bk, sl.v = v + bv, sl.gf = gf + bk, sl.gb = BIDIR ? gb + bk : nullptr, sl.d_o = d_o + bv;
    sl.dq = dq + bk, sl.dk = dk + bk, sl.dv = dv + bv, sl.dgf = dgf + bk, sl.dgb = BIDIR ? dgb + bk : nullptr;
    sl.L = len;
    return sl;
  };
  const int r = lane & 31, h = lane >> 5;
  BwdLoads<NG> ld;
  f32x16_t G[2];  // cumulative gates of the direction about to run, prepared one barrier ahead of it
  if ((int)blockIdx.x < nslabs) {
    const BwdSlab s0 = slab_of(blockIdx.x);
    const BwdNext first{s0, s0.gf, s0.L};
    issue_bwd_gate_loads<NG>(first, w, r, h, ld);
    issue_bwd_row_loads<true, NG>(first, w, r, h, ld);
    bwd_cumulate_gates<true, NG>(ld, w, lane, lds, G);
    lds_barrier();
  }
  for (int slab = blockIdx.x; slab < nslabs; slab += gridDim.x) {
    const BwdSlab sl = slab_of(slab);
    const int ntiles = (sl.L + 31) / 32;
    const int following = slab + (int)gridDim.x;
    const BwdSlab sn = slab_of(following < nslabs ? following : slab);
    const BwdNext second{sl, sl.gb, sl.L}, next_first{sn, sn.gf, following < nslabs ? sn.L : 0};
    f32x16_t dvacc[2] = {{0.f}, {0.f}};
    u32x4_t keepq[NG], keepk[NG];
    bool ok;
    if constexpr (BIDIR) {
      ok = bwd_direction<true, true, false, NG, SEG>(sl, sl.L, ntiles, w, lane, lds, s, dvacc, keepq, keepk, ld, second, G);
      if (ok) {
        ok = bwd_direction<false, false, true, NG, SEG>(sl, sl.L, ntiles, w, lane, lds, s, dvacc, keepq, keepk, ld,
                                                        next_first, G);
      }
    } else {  // the causal op: the forward direction alone, first and last at once
      ok = bwd_direction<true, true, true, NG, SEG>(sl, sl.L, ntiles, w, lane, lds, s, dvacc, keepq, keepk, ld,
                                                    next_first, G);
    }
    // a direction that left early has neither issued the loads of the slab that follows nor prepared its gates
    if (!ok) {
      lds_barrier();  // a wave that has left must not touch the gate totals the others still read
      issue_bwd_gate_loads<NG>(next_first, w, r, h, ld);
      issue_bwd_row_loads<true, NG>(next_first, w, r, h, ld);
      bwd_cumulate_gates<true, NG>(ld, w, lane, lds, G);
      lds_barrier();
    }
    if (SEG) {  // one flag per sequence, cleared by the segment scan: any segment out of range gives the sequence away
      if (tid == 0 && !ok) flags[slab / sg.nseg] = 1;
    } else if (tid == 0) {
      flags[slab] = ok ? 0 : 1;
    }
  }
}

// Links the segments of every (sequence, direction) for the backward.  Per segment s (walked in the direction's order)
// it reads the forward's state pass (contribution U_s, decay D_s) and the gradient state pass (Q_s = sum over the
// segment's tokens of (q e^{G})^T do, unscaled), and leaves
//   sp   = sqrt(D_s) S_in(s),     S_in(s') = D_s S_in(s) + U_s   for the segment s' walked next,
//   rp   = sqrt(D_s) R_out(s),    R_out(s) = Q_{s'} + D_{s'} R_out(s'),  zero for the segment walked last,
//   rpt  = rp transposed,
//   carry(s) = sum over the segments walked after s of rowsum_v(S_in Q - R_out U): what q dq - k dk adds up to there
// (bf16 matrices in plain row-major order; carry in the first of two slots per channel, the second zero).
// A thread holds the four state elements (k channels c, c+1) x (v columns x, x+1) of the passes' register order
// (units pk = 0, 1 and pv = 0, 1 of one register quad cq, lane, register m), so that its bf16 results leave as
// 4-byte words: whole 128-byte rows of sp and rp per 32 lanes, 16-byte pieces of rpt per four threads.  `term` holds
// S_in Q between the two sweeps.  Both sweeps fetch eight segments at a time: the serial part is arithmetic only.
__global__ __launch_bounds__(256) void gla_backward_segment_scan_kernel(
    const float* __restrict__ ws_fwd, const float* __restrict__ ws_grad, float* __restrict__ term, uint16_t* __restrict__ sp,
    uint16_t* __restrict__ rp, uint16_t* __restrict__ rpt, float* __restrict__ carry, int* __restrict__ flags, int nseq,
    int nseg, int ndir, int ng) {
  constexpr int kBatch = 8;
  __shared__ float red[kBatch][2][256];
  const int tid = threadIdx.x;
  const int cq = blockIdx.x;  // register quad: 4 blocks per (sequence, direction)
  const int seq = blockIdx.y / ndir, dir = blockIdx.y % ndir;
  if (cq == 0 && tid == 0 && dir == 0) flags[seq] = 0;
  if (cq >= ng) return;  // register quads beyond Dk/16 carry no channel (whole blocks)
  const int m = tid & 3, lane = tid >> 2, h = lane >> 5;
  const int ch0 = 8 * ng * h + 8 * cq + 2 * m;  // k channels ch0 (pk = 0), ch0 + 1 (pk = 1)
  const int v0 = 2 * cpair<4>(lane & 31);         // v columns v0 (pv = 0), v0 + 1 (pv = 1)
  // element (pk, pv) of this thread in register order: unit u = (pk*2 + pv)*4 + cq
  int e[2][2];
#pragma unroll
  for (int pk = 0; pk < 2; ++pk)
#pragma unroll
    for (int pv = 0; pv < 2; ++pv) e[pk][pv] = ((((pk * 2 + pv) * 4 + cq) * 64 + lane) << 2) + m;
  auto slot = [&](int seg, int d) { return (((size_t)seq * nseg + seg) * 2 + d); };
  // the gradient state pass ran with the directions' roles exchanged (see launch_gla_backward_mfma)
  const int gdir = 1 - dir;
  float S[2][2] = {{0.f, 0.f}, {0.f, 0.f}};
  for (int i0 = 0; i0 < nseg; i0 += kBatch) {
    float U[kBatch][2][2], Q[kBatch][2][2], D[kBatch][2];
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      const int i = min(i0 + j, nseg - 1);
      const int seg = dir == 0 ? i : nseg - 1 - i;
      const float* f = ws_fwd + slot(seg, dir) * kGlaStateFloats;
      const float* g = ws_grad + slot(seg, gdir) * kGlaStateFloats;
#pragma unroll
      for (int pk = 0; pk < 2; ++pk) {
        D[j][pk] = f[64 * 64 + ch0 + pk];
#pragma unroll
        for (int pv = 0; pv < 2; ++pv) U[j][pk][pv] = f[e[pk][pv]], Q[j][pk][pv] = g[e[pk][pv]];
      }
    }
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      const int i = i0 + j;
      if (i < nseg) {
        const int seg = dir == 0 ? i : nseg - 1 - i;
        uint16_t* spm = sp + slot(seg, dir) * kBwdStateElems;
        float* tm = term + slot(seg, dir) * kBwdStateElems;
#pragma unroll
        for (int pk = 0; pk < 2; ++pk) {
          const float rd = __builtin_sqrtf(D[j][pk]);
          *reinterpret_cast<uint32_t*>(spm + (ch0 + pk) * 64 + v0) = pack_bf16x2(rd * S[pk][0], rd * S[pk][1]);
#pragma unroll
          for (int pv = 0; pv < 2; ++pv) {
            tm[e[pk][pv]] = S[pk][pv] * Q[j][pk][pv];
            S[pk][pv] = __builtin_fmaf(D[j][pk], S[pk][pv], U[j][pk][pv]);
          }
        }
      }
    }
  }
  float R[2][2] = {{0.f, 0.f}, {0.f, 0.f}}, later[2] = {0.f, 0.f};
  for (int i0 = nseg - 1; i0 >= 0; i0 -= kBatch) {  // segments i0, i0 - 1, ... in this batch
    float U[kBatch][2][2], Q[kBatch][2][2], T1[kBatch][2][2], D[kBatch][2];
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      const int i = max(i0 - j, 0);
      const int seg = dir == 0 ? i : nseg - 1 - i;
      const float* f = ws_fwd + slot(seg, dir) * kGlaStateFloats;
      const float* g = ws_grad + slot(seg, gdir) * kGlaStateFloats;
      const float* tm = term + slot(seg, dir) * kBwdStateElems;
#pragma unroll
      for (int pk = 0; pk < 2; ++pk) {
        D[j][pk] = f[64 * 64 + ch0 + pk];
#pragma unroll
        for (int pv = 0; pv < 2; ++pv)
          U[j][pk][pv] = f[e[pk][pv]], Q[j][pk][pv] = g[e[pk][pv]], T1[j][pk][pv] = tm[e[pk][pv]];
      }
    }
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      const int i = i0 - j;
      red[j][0][tid] = later[0];
      red[j][1][tid] = later[1];
      if (i >= 0) {
        const int seg = dir == 0 ? i : nseg - 1 - i;
        uint16_t* rpm = rp + slot(seg, dir) * kBwdStateElems;
        uint16_t* rtm = rpt + slot(seg, dir) * kBwdStateElems;
        float x[2][2];
#pragma unroll
        for (int pk = 0; pk < 2; ++pk) {
          const float rd = __builtin_sqrtf(D[j][pk]);
          x[pk][0] = rd * R[pk][0], x[pk][1] = rd * R[pk][1];
          *reinterpret_cast<uint32_t*>(rpm + (ch0 + pk) * 64 + v0) = pack_bf16x2(x[pk][0], x[pk][1]);
        }
#pragma unroll
        for (int pv = 0; pv < 2; ++pv)
          *reinterpret_cast<uint32_t*>(rtm + (v0 + pv) * 64 + ch0) = pack_bf16x2(x[0][pv], x[1][pv]);
#pragma unroll
        for (int pk = 0; pk < 2; ++pk)
#pragma unroll
          for (int pv = 0; pv < 2; ++pv) {
            later[pk] += T1[j][pk][pv] - R[pk][pv] * U[j][pk][pv];
            R[pk][pv] = __builtin_fmaf(D[j][pk], R[pk][pv], Q[j][pk][pv]);
          }
      }
    }
    // the block holds 16 channels (lane half h, register m, pk) x all 64 v columns: summed in a fixed order
    __syncthreads();
    if (tid < 16 * kBatch) {
      const int j = tid >> 4, hh = (tid >> 3) & 1, mm = (tid >> 1) & 3, pk = tid & 1;
      const int i = i0 - j;
      if (i >= 0) {
        const int seg = dir == 0 ? i : nseg - 1 - i;
        float acc = 0.f;
        for (int x = 0; x < 32; ++x) acc += red[j][pk][(32 * hh + x) * 4 + mm];
        const int ch = 8 * ng * hh + 8 * cq + 2 * mm + pk;
        carry[slot(seg, dir) * 128 + ch] = acc;
        carry[slot(seg, dir) * 128 + 64 + ch] = 0.f;
      }
    }
    __syncthreads();
  }
}

static bool seg_grid_ok(int B, int H, bool bidir) { return (long long)B * H * (bidir ? 2 : 1) <= 65535; }

bool gla_backward_mfma_supported(int B, int H, int L, int Dk, int Dv, int io_dtype, int gate_dtype, bool bidir) {
  if (!(io_dtype == 1 && gate_dtype == 1 && (Dk == 64 || Dk == 32) && Dv == 64)) return false;
  return L <= 32 * kBwdTiles || seg_grid_ok(B, H, true);
}

// Long sequences: two state passes (kGlaStateFloats floats per sequence, segment and direction each), the S_in Q terms
// and the carries (fp32), then the three bf16 matrices the segments read.
static size_t seg_slots(int B, int H, int L) { return (size_t)B * H * gla_segments(L) * 2; }
size_t gla_backward_mfma_workspace(int B, int H, int L, int Dk, int Dv) {
  if (L <= 32 * kBwdTiles || !(Dk == 64 || Dk == 32) || Dv != 64) return 0;
  const size_t n = seg_slots(B, H, L);
  return n * ((2 * (size_t)kGlaStateFloats + kBwdStateElems + 128) * sizeof(float) + 3 * (size_t)kBwdStateElems * 2);
}

// flags: one int per (batch, head) sequence, written by every launch: 1 = not computed here (gates out of range)
int launch_gla_backward_mfma(const void* q, const void* k, const void* v, const void* gf, const void* gb,
                             const void* d_o, void* dq, void* dk, void* dv, void* dgf, void* dgb, int* flags,
                             void* seg_workspace, int B, int H, int L, int Dk, float s, hipStream_t stream) {
  constexpr int kMaxDevices = 64;
  static bool attr_done_dev[kMaxDevices] = {};
  static int num_cu_dev[kMaxDevices] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return -5;
  if (!attr_done_dev[dev]) {
    const void* kernels[8] = {reinterpret_cast<const void*>(gla_backward_mfma_kernel<4, true, false>),
                              reinterpret_cast<const void*>(gla_backward_mfma_kernel<2, true, false>),
                              reinterpret_cast<const void*>(gla_backward_mfma_kernel<4, false, false>),
                              reinterpret_cast<const void*>(gla_backward_mfma_kernel<2, false, false>),
                              reinterpret_cast<const void*>(gla_backward_mfma_kernel<4, true, true>),
                              reinterpret_cast<const void*>(gla_backward_mfma_kernel<2, true, true>),
                              reinterpret_cast<const void*>(gla_backward_mfma_kernel<4, false, true>),
                              reinterpret_cast<const void*>(gla_backward_mfma_kernel<2, false, true>)};
    for (const void* kf : kernels)
      if (hipFuncSetAttribute(kf, hipFuncAttributeMaxDynamicSharedMemorySize, kBwdLdsTotal) != hipSuccess) return -5;
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return -5;
    num_cu_dev[dev] = n > 0 ? n : 256;
    attr_done_dev[dev] = true;
  }
  const bool seg = L > 32 * kBwdTiles;
  BwdSegments sg{};
  int nslabs = B * H;
  if (seg) {
    if (!seg_workspace || !seg_grid_ok(B, H, gb != nullptr)) return -22;
    const size_t n = seg_slots(B, H, L);
    float* ws_fwd = (float*)seg_workspace;
    float* ws_grad = ws_fwd + n * kGlaStateFloats;
    float* term = ws_grad + n * kGlaStateFloats;
    float* carry = term + n * kBwdStateElems;
    uint16_t* sp = (uint16_t*)(carry + n * 128);
    uint16_t* rp = sp + n * kBwdStateElems;
    uint16_t* rpt = rp + n * kBwdStateElems;
    // One launch for both state passes.  The forward's: contributions k~^T v and decays of every segment, both
    // directions.  The gradient states: the same pass on (q for k, do for v) with each token's own gate included in
    // its weight.  A state pass anchors a token at the END of its walk (the weight of token j is the decay from j to
    // the last token walked); the gradient state needs the decay from the FIRST token walked to i, i.e. the walk of
    // the other direction over the same gates: the forward gates go to the reverse waves and the reverse gates to the
    // forward waves, and slot d of that pass belongs to direction 1 - d.  (The causal op runs both directions on its
    // one gate tensor and uses the forward slot of the first pass and the reverse slot of the second.)
    GlaArgs a{};
    a.q = q, a.k = k, a.v = v, a.g_fwd = gf, a.g_bwd = gb ? gb : gf, a.o = const_cast<void*>(d_o), a.workspace = ws_fwd;
    a.B = B, a.H = H, a.L = L, a.Dk = Dk, a.Dv = 64, a.scale = 1.f, a.out_scale = 1.f, a.io_dtype = 1, a.gate_dtype = 1;
    a.stream = stream, a.state_pass = 2;
    const int rc = launch_gla_mfma(a);
    if (rc != 0) return rc;
    const int ndir = gb ? 2 : 1;
    hipLaunchKernelGGL(gla_backward_segment_scan_kernel, dim3(4, B * H * ndir), dim3(256), 0, stream, ws_fwd,
                       ws_grad, term, sp, rp, rpt, carry, flags, B * H, gla_segments(L), ndir, Dk / 16);
    sg = BwdSegments{sp, rp, rpt, carry, gla_segments(L), gla_segment_len(L)};
    nslabs = B * H * sg.nseg;
  }
  const int grid = nslabs < num_cu_dev[dev] ? nslabs : num_cu_dev[dev];
#define VIG_BWD_LAUNCH(NG, BIDIR, SEG)                                                                          \
  hipLaunchKernelGGL((gla_backward_mfma_kernel<NG, BIDIR, SEG>), dim3(grid), dim3(512), kBwdLdsTotal, stream,    \
                     (const uint16_t*)q, (const uint16_t*)k, (const uint16_t*)v, (const uint16_t*)gf,            \
                     (const uint16_t*)gb, (const uint16_t*)d_o, (uint16_t*)dq, (uint16_t*)dk, (uint16_t*)dv,     \
                     (uint16_t*)dgf, (uint16_t*)dgb, flags, nslabs, L, s, sg)
#define VIG_BWD_LAUNCH_SEG(NG, BIDIR) \
  do {                                \
    if (seg) VIG_BWD_LAUNCH(NG, BIDIR, true); \
    else VIG_BWD_LAUNCH(NG, BIDIR, false);    \
  } while (0)
  if (gb) {
    if (Dk == 64) VIG_BWD_LAUNCH_SEG(4, true);
    else VIG_BWD_LAUNCH_SEG(2, true);
  } else {
    if (Dk == 64) VIG_BWD_LAUNCH_SEG(4, false);
    else VIG_BWD_LAUNCH_SEG(2, false);
  }
#undef VIG_BWD_LAUNCH_SEG
#undef VIG_BWD_LAUNCH
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

}  // namespace vig
