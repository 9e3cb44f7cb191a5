// Bidirectional GLA forward on MFMA tiles (gfx950), Dk in {32, 64}, Dv = 64, bf16 in and out: one workgroup per
// (batch, head) slab of up to 256 tokens, one wave per 32-token query tile, both directions in the same wave.  A longer
// sequence is cut into segments of at most seven tiles, each handled like a slab plus the products with the states
// that enter it from either side (apply_state; the states come from a state pass and a scan, gla_mfma.hip).
//
// Wave i owns the queries of tile i.  Along the forward direction they see the keys of tiles j <= i, along the
// reverse direction those of tiles j >= i, so every wave multiplies against NT + 1 key tiles whatever its position, the
// two directions add up in the wave's own accumulators (no exchange of outputs), and the only thing waves hand each
// other is what a key tile contributes: its decayed keys, its values and its total decay, published once in LDS.
// A wave
//   1. loads its 32 rows of q, k, v and of both gate tensors,
//   2. forms the tile-local cumulative log-gates G with a triangular-ones MFMA (bf16 gates are exact MFMA inputs,
//      the sums accumulate in fp32); the tile total T is G at the tile's last token walked,
//   3. builds q^ = q exp(G) (decay from the tile's first token walked: what an earlier tile's keys still see),
//      k^ = k exp(T - G) (decay up to the end of the tile: what a later tile's queries see) and, for its own diagonal
//      tile only, k' = k exp(-G); all as fp16 (11-bit significands, one MFMA term per k-step),
//   4. publishes k^ (both directions), V as fp16 transposed fragments and D = exp(T) per channel,
//   5. computes its diagonal tile from registers: P = mask_fwd(k'_f q^_f) + mask_rev(k'_r q^_r), O = V^T P,
//   6. after the one workgroup barrier walks outwards over the other tiles, P = k^_j (q^ (.) decays of the tiles in
//      between), O += V_j^T P, and stores its 32 output rows once.
// Every published factor is at most one in magnitude relative to its input, so distant tiles underflow gracefully; only
// k' grows (by exp(|T|)), which is why the fp16 form asks for |T| log2(e) <= 10 per 32-token tile and channel (ViG's
// logsigmoid(.)/16 gates reach about 2.5) and for rows of q, k, v of ordinary magnitude (sums of squares checked
// through a Gram-matrix MFMA).  A slab outside that range is redone by the same workgroup in the general form: inputs
// rescaled by slab-wide powers of two, the diagonal tile on half-anchored bf16 hi + lo operands with three MFMA terms
// per k-step (any tile total down to about -160, i.e. gates of -5 per token).
//
// Chunk algebra follows flash-linear-attention/fla/ops/gla/chunk_util.py:9-78 and chunk_fuse.py:76-97,245-254 (there
// with 16-token chunks and a carried state; here 32-token tiles and direct tile-pair products, which for L <= 256 cost
// fewer matrix instructions than carrying the Dk x Dv state); both directions in one launch as in
// recurrent_fuse.py:19-148.
//
// Register layouts as in mfma_tiles.h.  LDS: k^ tiles of the forward direction (tiles 0..NT-2) and of the reverse
// direction (tiles 1..NT-1) as ready A-operand units, V tiles as ready A-operand units, decays as fp16 in channel
// order; a wave's V region doubles as its private scratch until the values are published.
#include "common.h"
#include "launch.h"
#include "mfma_tiles.h"
#include <stddef.h>
#include <stdlib.h>

namespace vig {

namespace {

#define VIG_PHASE() __builtin_amdgcn_sched_barrier(0)

constexpr float kTileRange = 10.0f;     // fp16 form: |tile total| * log2(e) per channel
constexpr float kMaxSquaresQ = 32768.0f;  // rows of q: |q| < 182
constexpr float kMaxSquaresK = 1024.0f;   // rows of k: |k| < 32, so k' = k 2^10 stays inside fp16, and |P| <= |q||k| < 5800
constexpr float kMaxSquaresV = 1.0e8f;    // |v| < 10^4
constexpr float kExpFloor = -240.0f;      // general form: exponents are clamped here (what lies beyond is zero)

struct TileGeo {
  int L, NT, H;             // tokens per sequence, 32-token tiles per sequence, heads per batch element
  long long sq[3], sk[3], sv[3];  // (batch, head, token) strides in elements of q, k, v
  int wide;                 // nonzero: go straight to the general form
  int gw, gh, heads;        // fused locality gate: token grid (gw columns, gh rows, gw * gh = L), heads per batch element
  // output pass of a long sequence: grid (sequence, segment), NT tiles per segment; the states entering
  // the segments and their maxima as the segment scan leaves them
  int nseg;
  const float* states;
  const float* maxima;
};

// byte offsets of the workgroup's LDS areas
template <int NG>
struct TileLds {
  static constexpr int KB = NG * 1024;  // one k^ tile: NG units
  static constexpr int VB = 4096;       // one V tile: 4 units
  int kf, kb, v, d, scratch, guard, total;
  // gate_bytes: what the fused locality gate stages in the tile regions once they are dead (0: no gate)
  __host__ __device__ explicit TileLds(int NT, int gate_bytes = 0) {
    kf = 0;
    kb = (NT - 1) * KB;
    v = 2 * (NT - 1) * KB;
    d = v + NT * VB;
    if (d < gate_bytes) d = gate_bytes;
    scratch = d + 2 * NT * 128;  // per wave: 64 floats (tile totals on their way from one lane pair to a lane per channel)
    guard = scratch + NT * 256;
    total = guard + NT * 16;
  }
};

// Fused locality gate: the slab's rounded outputs as a zero-padded (gh + 2) x (gw + 2) grid of cells (64 channels as
// fp16: 128 bytes, 144 bytes apart, so that eight lanes on neighbouring tokens cover every LDS bank once), then the
// 64 x 9 stencil weights of the slab's head.
constexpr int kGateWeightBytes = 64 * 9 * 4;
constexpr int kGateCell = 144;
__host__ __device__ inline int gate_stage_bytes(int gw, int gh) { return (gw + 2) * (gh + 2) * kGateCell + kGateWeightBytes; }

struct TileCtx {
  const float* gate_w;  // fused locality gate: [64][9] stencil weights of this slab's head
  int gw, gh;
  rsrc_t q, k, v, gf, gb, o;
  unsigned q_pitch, k_pitch, v_pitch;
  char* lds;
  int ti, NT, lane;
  float oscale;
  const float* state_in;  // long sequences: this segment's slots (forward, then reverse direction)
  const float* state_top;  // ... and the sequence's maxima (kGlaScanMaxima floats per direction)
};

__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
  for (int s = 32; s >= 1; s >>= 1) x = fmaxf(x, __shfl_xor(x, s, 64));
  return x;
}
// power of two e such that m * 4^-e <= 2^target (m >= 0; inf or nan: the largest exponent)
__device__ __forceinline__ int scale_exponent(float m, int target) {
  const int ex = (int)((__float_as_uint(m) >> 23) & 0xffu) - 127;  // m < 2^(ex+1)
  const int e = (ex + 1 - target + 1) >> 1;
  return e > 0 ? e : 0;
}

// Which of the tile's tokens a direction keeps for column token r (j <= r forward, j >= r reverse), as a bit per token,
// shifted so that both lane halves read their tokens (4h + ...) at the same bit positions.
template <bool FWD>
__device__ __forceinline__ uint32_t keep_bits(int r, int h) {
  const uint32_t K = FWD ? (2u << r) - 1u : 0xFFFFFFFFu << r;
  return K >> (4 * h);
}
// 0xFFFF for each of the two token slots of dword X of k-step T (tokens jmap(T, h, 2X) and the next one) that is kept
template <int T, int X>
__device__ __forceinline__ uint32_t keep_mask(uint32_t kh) {
  constexpr unsigned j0 = 16 * T + 8 * (X >> 1) + 2 * (X & 1);
  const uint32_t lo = (uint32_t)__builtin_amdgcn_sbfe((int)kh, j0, 1), hi = (uint32_t)__builtin_amdgcn_sbfe((int)kh, j0 + 1, 1);
  return __builtin_amdgcn_perm(hi, lo, 0x07060100u);
}
template <int T>
__device__ __forceinline__ u32x4_t keep_masks(uint32_t kh) {
  return u32x4_t{keep_mask<T, 0>(kh), keep_mask<T, 1>(kh), keep_mask<T, 2>(kh), keep_mask<T, 3>(kh)};
}

// tile-local cumulative gates of one direction: G[p][4g+m] = channel 8*NG*h + 8g + 2m + p of token r
template <bool FWD>
__device__ __forceinline__ void cumulative_gates(const uint32_t (&gD)[2][8], int r, int h, f32x16_t (&G)[2]) {
  u32x4_t gfrag[2][2];
  finish_tfrags<2>(gD, gfrag);
  // B operand: bf16 ones where token slot j is on the kept side of column token r
  const uint32_t kh = keep_bits<FWD>(r, h);
  const u32x4_t tri0 = keep_masks<0>(kh) & 0x3F803F80u, tri1 = keep_masks<1>(kh) & 0x3F803F80u;
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    f32x16_t g = {0.f};
    g = mfma(gfrag[0][p], tri0, g);
    g = mfma(gfrag[1][p], tri1, g);
    G[p] = g;
  }
}

// the tile totals (G at the last token walked) travel from the one lane pair that holds them to a lane per channel:
// sc[32h + 16p + 4g + m] = total of channel 8*NG*h + 8g + 2m + p
template <bool FWD>
__device__ __forceinline__ void park_totals(f32x16_t (&G)[2], float* sc, int r, int h) {
  // (G comes straight out of the matrix cores and the store below sits behind a branch: the compiler's wait states
  // cover the path it expects to be taken; these cover the other one as well, where a register of G may be reused
  // before the matrix instruction has written it.  20 idle clocks per direction.)
  asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 3" : "+v"(G[0]), "+v"(G[1]));  // (tied to G: stays behind its producers)
  if (r == (FWD ? 31 : 0)) {
#pragma unroll
    for (int p = 0; p < 2; ++p)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x4_t x = {G[p][4 * g], G[p][4 * g + 1], G[p][4 * g + 2], G[p][4 * g + 3]};
        *reinterpret_cast<f32x4_t*>(sc + 32 * h + 16 * p + 4 * g) = x;
      }
  }
  wave_lds_sync();
}

// Operands of one direction for this wave's tile, the publication of what other tiles need from it, and the diagonal
// score tile (masked to the pairs the direction sees and rounded to fp16 pairs: the B operand of the value product).
//   qh: q^ = q exp(G)      (B operand of every score product of this wave; kept)
//   k^ = k exp(T - G)      (published to kreg unless null, piece by piece)
//   D  = exp(T)            (published to dtab, fp16, channel order)
// fp16 form (GENERAL false): the diagonal tile uses k' = k exp(-G) against q^; returns (wave-uniform) whether some
// channel's tile total is outside the form's range.
// General form: inputs carry the power-of-two scales 2^-eq, 2^-ek; the diagonal tile uses the half-anchored pair
// q~ = q exp(G - T/2), k~ = k exp(T/2 - G) as bf16 hi + lo, three MFMA terms per k-step.
template <int NG, bool FWD, bool GENERAL>
__device__ __forceinline__ bool prepare_direction(const uint32_t (&gD)[2][8], const u32x4_t (&rawq)[NG],
                                                  const u32x4_t (&rawk)[NG], float* sc, _Float16* dtab, char* kreg,
                                                  int lane, int eq, int ek, u32x4_t (&qh)[NG], u32x4_t (&p16)[2]) {
  constexpr int HC = 8 * NG;
  f32x16_t G[2];
  cumulative_gates<FWD>(gD, lane & 31, lane >> 5, G);
  park_totals<FWD>(G, sc, lane & 31, lane >> 5);
  float tl = sc[lane] * kLog2e;
  bool wide = false;
  if (!GENERAL) wide = __builtin_amdgcn_ballot_w64(!(fabsf(tl) <= kTileRange)) != 0;
  else tl = fmaxf(tl, kExpFloor);
  const float dT = exp2_fast(tl);
  if (GENERAL) sc[lane] = tl;
  {
    const int p = (lane >> 4) & 1, g = (lane >> 2) & 3, m = lane & 3;
    if (g < NG) dtab[HC * (lane >> 5) + 8 * g + 2 * m + p] = (_Float16)dT;
  }
  wave_lds_sync();
  const float* mine = sc + 32 * (lane >> 5);
  const u32x4_t* dmine = reinterpret_cast<const u32x4_t*>(dtab + HC * (lane >> 5));  // this lane half's decays as fp16 pairs
  const float fq = -(float)eq, fk = -(float)ek;
  f32x16_t P = {0.f};
  u32x4_t kc[NG];  // fp16 form: k' = k exp(-G), the diagonal tile's A operand
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    u32x4_t kh;
    f32x4_t d0, d1;
    if (GENERAL) {
      d0 = *reinterpret_cast<const f32x4_t*>(mine + 4 * g);
      d1 = *reinterpret_cast<const f32x4_t*>(mine + 16 + 4 * g);
    }
    if (!GENERAL) {
      // rawq / rawk hold fp16 pairs here; the decay factors are rounded to fp16 and applied as packed products
      // (the diagonal tile's products wait until the loop is through: their 16 accumulators would otherwise sit
      // beside the cumulative gates and the raw rows, which are at their fullest in the first pieces)
      const u32x4_t d16 = dmine[g];
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const int c = 4 * g + m;
        const float x0 = G[0][c] * kLog2e, x1 = G[1][c] * kLog2e;
        const uint32_t a16 = pack_f16x2(exp2_fast(x0), exp2_fast(x1));
        const uint32_t b16 = pack_f16x2(exp2_fast(-x0), exp2_fast(-x1));
        qh[g][m] = mul_f16x2(rawq[g][m], a16);
        kc[g][m] = mul_f16x2(rawk[g][m], b16);
        kh[m] = mul_f16x2(kc[g][m], d16[m]);
      }
    } else {
      u32x4_t qhi, qlo, khi, klo;
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const int c = 4 * g + m;
        const uint32_t wq = rawq[g][m], wk = rawk[g][m];
        const float qv[2] = {bf16lo_to_f32(wq), bf16hi_to_f32(wq)}, kv[2] = {bf16lo_to_f32(wk), bf16hi_to_f32(wk)};
        float qhat[2], khat[2], qt[2], kt[2];
#pragma unroll
        for (int p = 0; p < 2; ++p) {
          const float tl_c = p ? d1[m] : d0[m];
          const float x = fmaxf(G[p][c] * kLog2e, kExpFloor);
          const float an = 0.5f * tl_c;
          qhat[p] = qv[p] * exp2_fast(x + fq);
          khat[p] = kv[p] * exp2_fast(tl_c - x + fk);
          qt[p] = qv[p] * exp2_fast(x - an + fq);
          kt[p] = kv[p] * exp2_fast(an - x + fk);
        }
        qh[g][m] = pack_f16x2(qhat[0], qhat[1]);
        kh[m] = pack_f16x2(khat[0], khat[1]);
        qhi[m] = pack_bf16x2(qt[0], qt[1]);
        khi[m] = pack_bf16x2(kt[0], kt[1]);
        qlo[m] = pack_bf16x2(qt[0] - bf16lo_to_f32(qhi[m]), qt[1] - bf16hi_to_f32(qhi[m]));
        klo[m] = pack_bf16x2(kt[0] - bf16lo_to_f32(khi[m]), kt[1] - bf16hi_to_f32(khi[m]));
      }
      P = mfma(khi, qhi, P);
      P = mfma(klo, qhi, P);
      P = mfma(khi, qlo, P);
    }
    if (kreg) *reinterpret_cast<u32x4_t*>(unit_ptr(kreg, g, lane)) = kh;
  }
  if (!GENERAL) {
    VIG_PHASE();
#pragma unroll
    for (int g = 0; g < NG; ++g) P = mfma_f16(kc[g], qh[g], P);
  }
  // keep the pairs the direction sees (P^T[j, i]: lane = column i, register 4g+m = row 8g + 4h + m: the token of slot
  // pair x of k-step t, as in the triangular operand), round to fp16
  // (token masks rebuilt from an opaque lane: shared with the triangular operands above they would be carried, and
  // spilled, across the whole loop)
  int lane_m = lane;
  asm volatile("" : "+v"(lane_m));
  const uint32_t kh = keep_bits<FWD>(lane_m & 31, lane_m >> 5);
  const u32x4_t m0 = keep_masks<0>(kh), m1 = keep_masks<1>(kh);
#pragma unroll
  for (int x = 0; x < 4; ++x) {
    const int c = 4 * (x >> 1) + 2 * (x & 1);
    p16[0][x] = pack_f16x2(P[c], P[c + 1]) & m0[x];
    p16[1][x] = pack_f16x2(P[8 + c], P[8 + c + 1]) & m1[x];
  }
  return wide;
}

// O^T[pv] += V^T (fragments vf[t][pv] of one key tile) x P^T given as fp16 pairs
__device__ __forceinline__ void apply_values16(const u32x4_t (&p16)[2], const u32x4_t (&vf)[2][2], f32x16_t (&O)[2]) {
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    O[0] = mfma_f16(vf[t][0], p16[t], O[0]);
    O[1] = mfma_f16(vf[t][1], p16[t], O[1]);
  }
}

// O^T[pv] += V^T x P^T, P rounded once to fp16
__device__ __forceinline__ void apply_values(const f32x16_t& P, const u32x4_t (&vf)[2][2], f32x16_t (&O)[2]) {
  u32x4_t p16[2];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const int c = 4 * (2 * t + (x >> 1)) + 2 * (x & 1);
      p16[t][x] = pack_f16x2(P[c], P[c + 1]);
    }
  apply_values16(p16, vf, O);
}

// One outward walk of a wave over the key tiles of one direction: tiles ti-1 .. 0 (FWD) or ti+1 .. NT-1.  q^ picks up
// the total decay of every tile it passes (fp16 x fp16, every factor at most one).
template <int NG, bool FWD>
__device__ __forceinline__ void walk_tiles(char* lds, const TileLds<NG>& lay, int ti, int NT, int lane,
                                           u32x4_t (&qh)[NG], f32x16_t (&O)[2]) {
  const int h = lane >> 5;
  constexpr int HC = 8 * NG;
  const int kbase = FWD ? lay.kf : lay.kb - TileLds<NG>::KB;  // reverse regions start at tile 1
  const char* dbase = lds + lay.d + (FWD ? 0 : NT * 128) + 2 * HC * h;
  const int n = FWD ? ti : NT - 1 - ti;
#pragma unroll 1
  for (int s = 1; s <= n; ++s) {
    const int j = FWD ? ti - s : ti + s;
    if (s > 1) {  // the tile passed last: j + 1 forward, j - 1 reverse
      const char* dp = dbase + (FWD ? j + 1 : j - 1) * 128;
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const u32x4_t d = *reinterpret_cast<const u32x4_t*>(dp + 16 * g);
#pragma unroll
        for (int m = 0; m < 4; ++m) qh[g][m] = mul_f16x2(qh[g][m], d[m]);
      }
    }
    char* kreg = lds + kbase + j * TileLds<NG>::KB;
    char* vreg = lds + lay.v + j * TileLds<NG>::VB;
    u32x4_t kf[NG];
#pragma unroll
    for (int g = 0; g < NG; ++g) kf[g] = *reinterpret_cast<const u32x4_t*>(unit_ptr(kreg, g, lane));
    u32x4_t vf[2][2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int pv = 0; pv < 2; ++pv) vf[t][pv] = *reinterpret_cast<const u32x4_t*>(unit_ptr(vreg, 2 * t + pv, lane));
    const f32x16_t P = score_tile16<NG>(kf, qh);
    apply_values(P, vf, O);
  }
}

// Long sequences: what the state entering the segment (from the left for the forward direction, from the right for
// the reverse one) adds to this wave's tile,  O^T[pv] += S_in^T q^,  q^ anchored at the segment's edge.  The slot holds
// S_in in the matrix cores' register order: unit (pk, pv, g), lane, m is S_in[k channel 32h + 8g + 2m + pk][v column of
// accumulator lane r, half pv], so two units make the A operand of k-step g as they are.  The state goes in as fp16:
// directly while the scan saw nothing above 2^14, scaled by a power of two otherwise (`shift`, wave-uniform), the
// product then passing through an accumulator of its own.  extra: power of two the result still needs (general form).
template <int NG, bool FWD>
__device__ __forceinline__ void apply_state(const float* slot, const float* top16, const char* dtab_edge, bool cross,
                                            int lane, int extra, u32x4_t (&qh)[NG], f32x16_t (&O)[2]) {
  if (cross) {  // q^ over the segment's edge tile (tile 0 forward, the last one reverse)
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      const u32x4_t d = *reinterpret_cast<const u32x4_t*>(dtab_edge + 16 * g);
#pragma unroll
      for (int m = 0; m < 4; ++m) qh[g][m] = mul_f16x2(qh[g][m], d[m]);
    }
  }
  float top = lane < kGlaScanMaxima ? top16[lane] : 0.f;
  top = wave_max(top);
  const int ex = (int)((__float_as_uint(top) >> 23) & 0xffu) - 127;  // (inf / nan: 128, the result is not finite anyway)
  const int shift = __builtin_amdgcn_readfirstlane(max(ex - 13, -30));
  // (directly down to a top of 2^-4: smaller entries keep their weight relative to it in fp16's subnormal range)
  if (shift <= 0 && shift >= -17 && extra == 0) {
    // (two k-steps' worth of the state in flight at a time: sixteen registers)
#pragma unroll
    for (int pv = 0; pv < 2; ++pv)
#pragma unroll
      for (int g0 = 0; g0 < NG; g0 += 2) {
        f32x4_t a[2], b[2];
#pragma unroll
        for (int g = 0; g < 2; ++g) {
          a[g] = *reinterpret_cast<const f32x4_t*>(slot + (((0 * 2 + pv) * 4 + g0 + g) * 64 + lane) * 4);
          b[g] = *reinterpret_cast<const f32x4_t*>(slot + (((1 * 2 + pv) * 4 + g0 + g) * 64 + lane) * 4);
        }
#pragma unroll
        for (int g = 0; g < 2; ++g) {
          u32x4_t f;
#pragma unroll
          for (int m = 0; m < 4; ++m) f[m] = pack_f16x2(a[g][m], b[g][m]);
          O[pv] = mfma_f16(f, qh[g0 + g], O[pv]);
        }
      }
    return;
  }
  const float pre = __builtin_amdgcn_exp2f(-(float)shift), post = __builtin_amdgcn_exp2f((float)(shift + extra));
#pragma unroll
  for (int pv = 0; pv < 2; ++pv) {
    f32x16_t acc = {0.f};
    f32x4_t a[NG], b[NG];
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      a[g] = *reinterpret_cast<const f32x4_t*>(slot + (((0 * 2 + pv) * 4 + g) * 64 + lane) * 4);
      b[g] = *reinterpret_cast<const f32x4_t*>(slot + (((1 * 2 + pv) * 4 + g) * 64 + lane) * 4);
    }
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      u32x4_t f;
#pragma unroll
      for (int m = 0; m < 4; ++m) f[m] = pack_f16x2(a[g][m] * pre, b[g][m] * pre);
      acc = mfma_f16(f, qh[g], acc);
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) O[pv][i] = __builtin_fmaf(acc[i], post, O[pv][i]);
  }
}

// Fused locality gate: y = o * sigmoid(conv3x3(o)) per channel on the gw x gh token grid (zero padding), o being the
// bf16-rounded output.  The whole slab's outputs are staged in LDS where the tiles lay.  (A function of its own: its
// 72 weight registers stay out of the main path's allocation.)
__device__ __forceinline__ void locality_gate_epilogue(f32x16_t O0, f32x16_t O1, float os, char* lds, const float* gate_w,
                                                    rsrc_t o_rsrc, int gw, int gh, int ti, int NT, int lane_w) {
  struct { int gw, gh; const float* gate_w; rsrc_t o; } cx{gw, gh, gate_w, o_rsrc};
  const f32x16_t O[2] = {O0, O1};
    // ---- fused locality gate: y = o * sigmoid(conv3x3(o)) per channel on the gw x gh token grid (zero padding), o
    // being the bf16-rounded output.  The whole slab's outputs are staged in LDS where the tiles lay. ----
    const int pw = cx.gw + 2;
    char* cells = lds;
    float* wlds = reinterpret_cast<float*>(lds + pw * (cx.gh + 2) * kGateCell);
    const float inv_w = 1.0f / (float)cx.gw;
    // the head's stencil weights, fetched by the first 144 threads while the other waves finish their walks
    f32x4_t w4 = {0.f, 0.f, 0.f, 0.f};
    const bool w_mine = ti * 64 + lane_w < 64 * 9 / 4;
    if (w_mine) w4 = reinterpret_cast<const f32x4_t*>(cx.gate_w)[ti * 64 + lane_w];
    lds_barrier();  // every wave is done with the tiles
    if (w_mine) reinterpret_cast<f32x4_t*>(wlds)[ti * 64 + lane_w] = w4;
    // (workgroups of fewer than three waves: the rest of the 144 pieces)
    for (int idx = ti * 64 + lane_w + 64 * NT; idx < 64 * 9 / 4; idx += 64 * NT)
      reinterpret_cast<f32x4_t*>(wlds)[idx] = reinterpret_cast<const f32x4_t*>(cx.gate_w)[idx];
    // The rounded outputs are staged as fp16 pairs (every bf16 value down to 2^-17 is an fp16 value), so that the
    // stencil's multiply-adds read them in place (v_fma_mix_f32: fp16 x fp32 + fp32, the same fp32 arithmetic as on
    // unpacked values, without the unpacking).
    {
      const int T = 32 * ti + (lane_w & 31);
      if (T < cx.gw * cx.gh) {
        const int y = (int)(((float)T + 0.5f) * inv_w), x = T - __mul24(y, cx.gw);
        const int cell_i = (y + 1) * pw + x + 1;
        char* cell = cells + cell_i * kGateCell;
        const int hb = 4 * (lane_w >> 5);
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) {
          u32x4_t w;
#pragma unroll
          for (int m = 0; m < 4; ++m) {
            const uint32_t b = pack_bf16x2(O[0][4 * gq + m] * os, O[1][4 * gq + m] * os);
            w[m] = pack_f16x2(bf16lo_to_f32(b), bf16hi_to_f32(b));
          }
          *reinterpret_cast<u32x4_t*>(cell + 16 * (hb + gq)) = w;
        }
      }
    }
    const int oct = lane_w & 7, tl = lane_w >> 3;
    {  // the border cells, by the whole workgroup: top row, bottom row, then the two ends of every other row
      const int nborder = 2 * pw + 2 * cx.gh;
      const u32x4_t zero = {0u, 0u, 0u, 0u};
      for (int bc = ti * 8 + tl; bc < nborder; bc += 8 * NT) {
        int py, px;
        if (bc < 2 * pw) {
          py = bc < pw ? 0 : cx.gh + 1;
          px = bc < pw ? bc : bc - pw;
        } else {
          const int j = bc - 2 * pw;
          py = 1 + (j >> 1);
          px = (j & 1) ? pw - 1 : 0;
        }
        *reinterpret_cast<u32x4_t*>(cells + (py * pw + px) * kGateCell + 16 * oct) = zero;
      }
    }
    lds_barrier();  // the slab's outputs, the zero border and the weights are staged
    float wreg[8][9];
    {
      const f32x4_t* wp = reinterpret_cast<const f32x4_t*>(wlds + oct * 72);
#pragma unroll
      for (int i = 0; i < 18; ++i) {
        const f32x4_t x = wp[i];
#pragma unroll
        for (int m = 0; m < 4; ++m) wreg[(4 * i + m) / 9][(4 * i + m) % 9] = x[m];
      }
    }
#pragma unroll 1
    for (int i = 0; i < 4; ++i) {
      const int row = tl + 8 * i;
      const int T = 32 * ti + row;
      if (T < cx.gw * cx.gh) {
        const int y = (int)(((float)T + 0.5f) * inv_w), x = T - __mul24(y, cx.gw);
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        u32x4_t ctr = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int di = 0; di < 3; ++di) {
          const char* rowp = cells + ((y + di) * pw + x) * kGateCell + 16 * oct;  // padded cell of tap (di - 1, -1)
#pragma unroll
          for (int dj = 0; dj < 3; ++dj) {
            const u32x4_t w = *reinterpret_cast<const u32x4_t*>(rowp + dj * kGateCell);
#pragma unroll
            for (int m = 0; m < 4; ++m) {
              asm("v_fma_mix_f32 %0, %1, %2, %0 op_sel:[0,0,0] op_sel_hi:[1,0,0]"
                  : "+v"(acc[2 * m]) : "v"(w[m]), "v"(wreg[2 * m][di * 3 + dj]));
              asm("v_fma_mix_f32 %0, %1, %2, %0 op_sel:[1,0,0] op_sel_hi:[1,0,0]"
                  : "+v"(acc[2 * m + 1]) : "v"(w[m]), "v"(wreg[2 * m + 1][di * 3 + dj]));
            }
            if (di == 1 && dj == 1) ctr = w;
          }
        }
        u32x4_t out;
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          const uint32_t cw = ctr[m];
          const float s0 = sigmoidf_(acc[2 * m]), s1 = sigmoidf_(acc[2 * m + 1]);
          float y0, y1;  // the centre values, read as fp16 halves in place
          asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel:[0,0,0] op_sel_hi:[1,0,0]" : "=v"(y0) : "v"(cw), "v"(s0));
          asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(y1) : "v"(cw), "v"(s1));
          out[m] = pack_bf16x2(y0, y1);
        }
        __builtin_amdgcn_raw_buffer_store_b128(out, cx.o, (unsigned)row * 128u + 16u * oct, 0, 0);
      }
    }
}

// Everything one wave does for its slab.  The fp16 form (GENERAL false) returns true, for every wave of the workgroup
// alike and before anything is stored, when some tile of the slab is outside its range.
template <int NG, bool BIDIR, bool PITCHED, bool GENERAL, bool GATE, bool CHAIN>
__device__ __forceinline__ bool tile_pass(const TileCtx& cx) {
  const int lane = cx.lane, r = lane & 31, h = lane >> 5;
  const int ti = cx.ti, NT = cx.NT;
  const TileLds<NG> lay(NT, GATE ? gate_stage_bytes(cx.gw, cx.gh) : 0);
  char* lds = cx.lds;
  char* vregion = lds + lay.v + ti * TileLds<NG>::VB;
  float* sc = reinterpret_cast<float*>(lds + lay.scratch + ti * 256);
  float* guard = reinterpret_cast<float*>(lds + lay.guard);
  _Float16* dtab_f = reinterpret_cast<_Float16*>(lds + lay.d + ti * 128);
  _Float16* dtab_b = reinterpret_cast<_Float16*>(lds + lay.d + (NT + ti) * 128);

  // ---- loads: v and gates as transposed dwords, q / k rows ----
  uint32_t gDf[2][8], gDb[2][8], vD[2][8];
  u32x4_t rawq[NG], rawk[NG];
  if (PITCHED) issue_tdwords_pitched<0, 2, 4>(cx.v, r, h, cx.v_pitch, vD);
  else issue_tdwords<0, 2, 4>(cx.v, r, h, vD);
  issue_tdwords<0, 2, NG>(cx.gf, r, h, gDf);
  if (PITCHED) {
    issue_raw_tile_pitched<NG>(cx.q, 0, r, h, cx.q_pitch, rawq);
    issue_raw_tile_pitched<NG>(cx.k, 0, r, h, cx.k_pitch, rawk);
  } else {
    issue_raw_tile<NG>(cx.q, 0, r, h, rawq);
    issue_raw_tile<NG>(cx.k, 0, r, h, rawk);
  }
  if (BIDIR) issue_tdwords<0, 2, NG>(cx.gb, r, h, gDb);
  // ---- magnitudes (Gram matrices of the raw rows); values: bf16 pairs -> fp16 pairs, published ----
  int eq = 0, ek = 0, ev = 0;
  bool veto = false;
  {
    u32x4_t vraw[2][2];
    finish_tfrags<2>(vD, vraw);
    f32x4acc_t gq = {0.f, 0.f, 0.f, 0.f}, gk = gq, gv = gq;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int p = 0; p < 2; ++p) gram_acc(vraw[t][p], gv);
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      gram_acc(rawq[g], gq);
      gram_acc(rawk[g], gk);
    }
    const float mq = fmaxf(fmaxf(fabsf(gq[0]), fabsf(gq[1])), fmaxf(fabsf(gq[2]), fabsf(gq[3])));
    const float mk = fmaxf(fmaxf(fabsf(gk[0]), fabsf(gk[1])), fmaxf(fabsf(gk[2]), fabsf(gk[3])));
    const float mv = fmaxf(fmaxf(fabsf(gv[0]), fabsf(gv[1])), fmaxf(fabsf(gv[2]), fabsf(gv[3])));
    if (!GENERAL) {
      veto = __builtin_amdgcn_ballot_w64(!(mq < kMaxSquaresQ) || !(mk < kMaxSquaresK) || !(mv < kMaxSquaresV)) != 0;
    } else {
      // slab-wide scales for k and v (their tiles meet every wave's queries), a scale of its own for this wave's q
      const float wq = wave_max(mq), wk = wave_max(mk), wv = wave_max(mv);
      if (lane == 0) {
        guard[4 * ti + 1] = wk;
        guard[4 * ti + 2] = wv;
      }
      lds_barrier();
      float sk = 0.f, sv = 0.f;
      for (int t = 0; t < NT; ++t) {
        sk = fmaxf(sk, guard[4 * t + 1]);
        sv = fmaxf(sv, guard[4 * t + 2]);
      }
      eq = scale_exponent(wq, 10);
      ek = scale_exponent(sk, 10);
      ev = scale_exponent(sv, 20);
    }
    if (!GENERAL) {  // bf16 pairs -> fp16 pairs (exact for the magnitudes the guard admits)
#pragma unroll
      for (int g = 0; g < NG; ++g)
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          rawq[g][m] = pack_f16x2(bf16lo_to_f32(rawq[g][m]), bf16hi_to_f32(rawq[g][m]));
          rawk[g][m] = pack_f16x2(bf16lo_to_f32(rawk[g][m]), bf16hi_to_f32(rawk[g][m]));
        }
    }
    const float vs = GENERAL ? __builtin_amdgcn_exp2f(-(float)ev) : 1.0f;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        u32x4_t f;
#pragma unroll
        for (int x = 0; x < 4; ++x) {
          const uint32_t w = vraw[t][p][x];
          f[x] = GENERAL ? pack_f16x2(bf16lo_to_f32(w) * vs, bf16hi_to_f32(w) * vs)
                         : pack_f16x2(bf16lo_to_f32(w), bf16hi_to_f32(w));
        }
        *reinterpret_cast<u32x4_t*>(unit_ptr(vregion, 2 * t + p, lane)) = f;
      }
  }
  VIG_PHASE();
  // ---- both directions: operands, publication, diagonal scores ----
  u32x4_t qhf[NG], qhb[NG];
  u32x4_t p16[2];
  {
    char* kreg = ti < NT - 1 ? lds + lay.kf + ti * TileLds<NG>::KB : nullptr;
    if (prepare_direction<NG, true, GENERAL>(gDf, rawq, rawk, sc, dtab_f, kreg, lane, eq, ek, qhf, p16)) veto = true;
  }
  VIG_PHASE();
  if (BIDIR) {
    char* kreg = ti > 0 ? lds + lay.kb + (ti - 1) * TileLds<NG>::KB : nullptr;
    u32x4_t pb[2];
    if (GENERAL) {
      // (opaque copies: the unpacked halves of the raw rows are rebuilt here instead of being carried, 64 registers
      // wide, from the forward direction's loop)
#pragma unroll
      for (int g = 0; g < NG; ++g)
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          asm volatile("" : "+v"(rawq[g][m]));
          asm volatile("" : "+v"(rawk[g][m]));
        }
    }
    // (lane-derived constants of this direction are built here, not carried from the top of the kernel)
    int lane_b = lane;
    asm volatile("" : "+v"(lane_b));
    if (prepare_direction<NG, false, GENERAL>(gDb, rawq, rawk, sc, dtab_b, kreg, lane_b, eq, ek, qhb, pb)) veto = true;
    // (the two directions meet on the pairs j = i only: one more fp16 rounding there)
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int x = 0; x < 4; ++x) p16[t][x] = add_f16x2(p16[t][x], pb[t][x]);
  }
  VIG_PHASE();
  // ---- diagonal tile ----
  f32x16_t O[2] = {f32x16_t{0.f}, f32x16_t{0.f}};
  {
    wave_lds_sync();
    u32x4_t vf[2][2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int pv = 0; pv < 2; ++pv) vf[t][pv] = *reinterpret_cast<const u32x4_t*>(unit_ptr(vregion, 2 * t + pv, lane));
    apply_values16(p16, vf, O);
  }
  if (!GENERAL && lane == 0) guard[4 * ti] = veto ? 1.0f : 0.0f;
  lds_barrier();  // every tile's k^, V and decays are visible
  if (!GENERAL) {
    const float mine = lane < NT ? guard[4 * lane] : 0.0f;
    if (__builtin_amdgcn_ballot_w64(mine != 0.0f) != 0) return true;
  }
  // (from here on a wave holds what the others wait for, its slot on the CU included: ahead of the waves of the other
  // workgroup that are still preparing operands; measured 3 % on the Dk = 32 layer shape, nothing at Dk = 64)
  __builtin_amdgcn_s_setprio(2);
  // ---- the other tiles, outwards ----
  int lane_w = lane;
  asm volatile("" : "+v"(lane_w));
  walk_tiles<NG, true>(lds, lay, ti, NT, lane_w, qhf, O);
  // (general form: the state's term joins accumulators that carry 2^-(eq + ek + ev); q^ carries 2^-eq itself)
  if (CHAIN)
    apply_state<NG, true>(cx.state_in, cx.state_top, lds + lay.d + 16 * NG * (lane_w >> 5), ti > 0, lane_w,
                          GENERAL ? -(ek + ev) : 0, qhf, O);
  if (BIDIR) walk_tiles<NG, false>(lds, lay, ti, NT, lane_w, qhb, O);
  if (CHAIN && BIDIR)
    apply_state<NG, false>(cx.state_in + kGlaStateFloats, cx.state_top + kGlaScanMaxima,
                           lds + lay.d + (NT + NT - 1) * 128 + 16 * NG * (lane_w >> 5), ti < NT - 1, lane_w,
                           GENERAL ? -(ek + ev) : 0, qhb, O);
  float os = cx.oscale;
  if (GENERAL) os *= __builtin_amdgcn_exp2f((float)(eq + ek + ev));
  if (GATE) {
    locality_gate_epilogue(O[0], O[1], os, lds, cx.gate_w, cx.o, cx.gw, cx.gh, ti, NT, lane_w);
    return false;
  }
  // ---- store: lane (r, h) holds channels [32h, 32h + 32) of token r; rows beyond the sequence are dropped ----
#pragma unroll
  for (int gq = 0; gq < 4; ++gq) {
    u32x4_t x;
#pragma unroll
    for (int m = 0; m < 4; ++m) x[m] = pack_bf16x2(O[0][4 * gq + m] * os, O[1][4 * gq + m] * os);
    __builtin_amdgcn_raw_buffer_store_b128(x, cx.o, (unsigned)(lane_w & 31) * 128u + 64u * (lane_w >> 5) + 16u * gq, 0, 0);
  }
  return false;
}

template <int NG, bool BIDIR, bool PITCHED, bool GATE, bool CHAIN>
__device__ __forceinline__ TileCtx make_tile_ctx(const uint16_t* q, const uint16_t* k, const uint16_t* v,
                                                 const uint16_t* gf, const uint16_t* gb, uint16_t* o,
                                                 const TileGeo& geo, float oscale, const float* gate_w, char* lds) {
  constexpr int DK = 16 * NG;
  TileCtx cx;
  cx.lds = lds;
  cx.gw = GATE ? geo.gw : 0, cx.gh = GATE ? geo.gh : 0;
  // (slab = batch element * heads + head)
  cx.gate_w = GATE ? gate_w + (size_t)((int)blockIdx.x % geo.heads) * (64 * 9) : nullptr;
  cx.ti = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  cx.lane = threadIdx.x & 63;
  cx.NT = geo.NT;
  cx.oscale = oscale;
  // (long sequences: grid (sequence, segment), a segment = NT tiles; tiles past the end hold no token)
  const int seq = blockIdx.x;
  const int seg = CHAIN ? (int)blockIdx.y : 0;
  const int tok = 32 * (seg * geo.NT + cx.ti);
  // (the clamp from both sides compiles to a vector instruction: back to a scalar, or every descriptor built from it
  // counts as divergent and every load gets a loop around it)
  const int nvalid = CHAIN ? __builtin_amdgcn_readfirstlane(max(0, min(32, geo.L - tok))) : min(32, geo.L - tok);
  const size_t off = (size_t)seq * geo.L + tok;  // in tokens
  cx.state_in = CHAIN ? geo.states + ((size_t)seq * geo.nseg + seg) * 2 * kGlaStateFloats : nullptr;
  cx.state_top = CHAIN ? geo.maxima + (size_t)seq * 2 * kGlaScanMaxima : nullptr;
  if (PITCHED) {
    const int b = seq / geo.H, hd = seq - b * geo.H;
    cx.q_pitch = 2u * (unsigned)geo.sq[2], cx.k_pitch = 2u * (unsigned)geo.sk[2], cx.v_pitch = 2u * (unsigned)geo.sv[2];
    cx.q = chunk_rsrc(q + b * geo.sq[0] + hd * geo.sq[1] + (long long)tok * geo.sq[2], nvalid, cx.q_pitch);
    cx.k = chunk_rsrc(k + b * geo.sk[0] + hd * geo.sk[1] + (long long)tok * geo.sk[2], nvalid, cx.k_pitch);
    cx.v = chunk_rsrc(v + b * geo.sv[0] + hd * geo.sv[1] + (long long)tok * geo.sv[2], nvalid, cx.v_pitch);
  } else {
    cx.q_pitch = cx.k_pitch = 2 * DK, cx.v_pitch = 128;
    cx.q = chunk_rsrc(q + off * DK, nvalid, 2 * DK);
    cx.k = chunk_rsrc(k + off * DK, nvalid, 2 * DK);
    cx.v = chunk_rsrc(v + off * 64, nvalid, 128);
  }
  cx.gf = chunk_rsrc(gf + off * DK, nvalid, 2 * DK);
  cx.gb = chunk_rsrc(BIDIR ? gb + off * DK : gf, BIDIR ? nvalid : 0, 2 * DK);
  cx.o = chunk_rsrc(o + off * 64, nvalid, 128);
  return cx;
}

// The kernel's argument block as the hardware lays it out (every argument at its natural alignment).
struct TileKernArgs {
  const uint16_t *q, *k, *v, *gf, *gb;
  uint16_t* o;
  TileGeo geo;
  float oscale;
  const float* gate_w;
};

static_assert(offsetof(TileKernArgs, geo) == 6 * sizeof(void*) && offsetof(TileKernArgs, oscale) == 48 + sizeof(TileGeo) &&
                  offsetof(TileKernArgs, gate_w) == 48 + sizeof(TileGeo) + 8 && alignof(TileGeo) == 8,
              "TileKernArgs has to mirror the parameter list of gla_tile_kernel");

// The general form as a function of its own: its register needs stay out of the fp16 form's allocation.  It reads
// the kernel's arguments from the argument block itself (ka: the kernel's own kernarg segment pointer; the builtin
// yields null inside a called function): handed over as parameters, the geometry would need a copy in per-lane
// memory, and the compiler writes that copy at the top of the kernel, for every wave, redo or not.
template <int NG, bool BIDIR, bool PITCHED, bool GATE, bool CHAIN>
__device__ __noinline__ void tile_pass_general(const TileKernArgs* ka_in) {
#if defined(__HIP_DEVICE_COMPILE__)  // (the host pass has no constant address space to copy the geometry from)
  // (a called function gets its arguments in vector registers: back to scalars, or every argument read through the
  // pointer, and every descriptor built from one, counts as divergent and each load gets a loop around it; the LDS
  // base is named here again for the same reason: a pointer handed over would be a generic one)
  extern __shared__ __align__(16) char lds[];
  const uint64_t kp = reinterpret_cast<uint64_t>(ka_in);
  // (constant address space: scalar loads)
  typedef const TileKernArgs __attribute__((address_space(4))) * KernArgPtr;
  const KernArgPtr ka = (KernArgPtr)(((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(kp >> 32)) << 32) |
                                     (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)kp));
  const TileGeo geo = ka->geo;
  const TileCtx cx = make_tile_ctx<NG, BIDIR, PITCHED, GATE, CHAIN>(ka->q, ka->k, ka->v, ka->gf, ka->gb, ka->o, geo,
                                                                     ka->oscale, ka->gate_w, lds);
  tile_pass<NG, BIDIR, PITCHED, true, GATE, CHAIN>(cx);
#endif
}

}  // namespace

template <int NG, bool BIDIR, bool PITCHED, bool GATE, bool CHAIN = false>
__global__ __launch_bounds__(512, 4) void gla_tile_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ k,
                                                          const uint16_t* __restrict__ v,
                                                          const uint16_t* __restrict__ gf,
                                                          const uint16_t* __restrict__ gb, uint16_t* __restrict__ o,
                                                          TileGeo geo, float oscale,
                                                          const float* __restrict__ gate_w) {
  extern __shared__ __align__(16) char lds[];
  bool redo = true;
  if (!geo.wide) {
    const TileCtx cx = make_tile_ctx<NG, BIDIR, PITCHED, GATE, CHAIN>(q, k, v, gf, gb, o, geo, oscale, gate_w, lds);
    redo = tile_pass<NG, BIDIR, PITCHED, false, GATE, CHAIN>(cx);
  }
  if (redo)
    tile_pass_general<NG, BIDIR, PITCHED, GATE, CHAIN>((const TileKernArgs*)__builtin_amdgcn_kernarg_segment_ptr());
}

// The general form alone, for launches whose caller knows the gates to be strong: with 256 registers per wave (one
// workgroup per CU) it keeps its unpacked operands in registers, which the function above, bound to the fp16 form's
// 128, has to send through per-lane memory.
template <int NG, bool BIDIR, bool PITCHED, bool GATE, bool CHAIN = false>
__global__ __launch_bounds__(512, 2) void gla_tile_wide_kernel(const uint16_t* __restrict__ q,
                                                               const uint16_t* __restrict__ k,
                                                               const uint16_t* __restrict__ v,
                                                               const uint16_t* __restrict__ gf,
                                                               const uint16_t* __restrict__ gb, uint16_t* __restrict__ o,
                                                               TileGeo geo, float oscale,
                                                               const float* __restrict__ gate_w) {
  extern __shared__ __align__(16) char lds[];
  const TileCtx cx = make_tile_ctx<NG, BIDIR, PITCHED, GATE, CHAIN>(q, k, v, gf, gb, o, geo, oscale, gate_w, lds);
  tile_pass<NG, BIDIR, PITCHED, true, GATE, CHAIN>(cx);
}

constexpr int kTileMaxLds = 160 * 1024;

bool gla_tiles_supported(const GlaArgs& a) {
  if (!(a.io_dtype == 1 && a.gate_dtype == 1 && (a.Dk == 64 || a.Dk == 32) && a.Dv == 64 && a.L <= 256 &&
        !a.init_state && !a.final_state && !a.state_pass))
    return false;
  if (a.gate_w) {  // fused locality gate: both directions, plain tensors, the padded grid has to fit in LDS
    if (!a.g_bwd || a.q_strides || a.k_strides || a.v_strides || a.gate_cols <= 0 || a.gate_rows <= 0 ||
        (long long)a.gate_cols * a.gate_rows != a.L)
      return false;
    if (TileLds<4>((a.L + 31) / 32, gate_stage_bytes(a.gate_cols, a.gate_rows)).total > kTileMaxLds) return false;
  }
  return true;
}

template <int NG, bool BIDIR, bool PITCHED, bool GATE, bool CHAIN = false>
static int launch_tiles_t(const GlaArgs& a, const TileGeo& geo, int dev) {
  constexpr int kMaxDevices = 64;
  static bool attr_done_dev[kMaxDevices] = {};
  const void* kf = reinterpret_cast<const void*>(gla_tile_kernel<NG, BIDIR, PITCHED, GATE, CHAIN>);
  const void* kw = reinterpret_cast<const void*>(gla_tile_wide_kernel<NG, BIDIR, PITCHED, GATE, CHAIN>);
  if (!attr_done_dev[dev]) {
    if (hipFuncSetAttribute(kf, hipFuncAttributeMaxDynamicSharedMemorySize, kTileMaxLds) != hipSuccess) return -5;
    if (hipFuncSetAttribute(kw, hipFuncAttributeMaxDynamicSharedMemorySize, kTileMaxLds) != hipSuccess) return -5;
    attr_done_dev[dev] = true;
  }
  const TileLds<NG> lay(geo.NT, GATE ? gate_stage_bytes(geo.gw, geo.gh) : 0);
  if (lay.total > kTileMaxLds) return -95;
  if (geo.wide)
    hipLaunchKernelGGL((gla_tile_wide_kernel<NG, BIDIR, PITCHED, GATE, CHAIN>), dim3(a.B * a.H, CHAIN ? geo.nseg : 1),
                       dim3(64 * geo.NT), lay.total, a.stream,
                       (const uint16_t*)a.q, (const uint16_t*)a.k, (const uint16_t*)a.v, (const uint16_t*)a.g_fwd,
                       (const uint16_t*)a.g_bwd, (uint16_t*)a.o, geo, a.scale * a.out_scale, a.gate_w);
  else
    hipLaunchKernelGGL((gla_tile_kernel<NG, BIDIR, PITCHED, GATE, CHAIN>), dim3(a.B * a.H, CHAIN ? geo.nseg : 1),
                       dim3(64 * geo.NT), lay.total, a.stream,
                       (const uint16_t*)a.q, (const uint16_t*)a.k, (const uint16_t*)a.v, (const uint16_t*)a.g_fwd,
                       (const uint16_t*)a.g_bwd, (uint16_t*)a.o, geo, a.scale * a.out_scale, a.gate_w);
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

int launch_gla_tiles(const GlaArgs& a) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return -5;
  TileGeo geo{};
  geo.L = a.L;
  geo.NT = (a.L + 31) / 32;
  geo.H = a.H;
  geo.wide = a.wide_gates;
  const bool pitched = a.q_strides || a.k_strides || a.v_strides;
  if (pitched) {
    const long long* given[3] = {a.q_strides, a.k_strides, a.v_strides};
    long long* dst[3] = {geo.sq, geo.sk, geo.sv};
    const int D[3] = {a.Dk, a.Dk, a.Dv};
    for (int i = 0; i < 3; ++i) {
      if (given[i] && given[i][2] != 0) {
        // rows 16-byte aligned, pitches within the descriptors' 32-bit extents
        for (int j = 0; j < 3; ++j)
          if (given[i][j] <= 0 || given[i][j] % 8 != 0) return -22;
        if (given[i][2] > (1 << 20)) return -22;
        dst[i][0] = given[i][0], dst[i][1] = given[i][1], dst[i][2] = given[i][2];
      } else {
        dst[i][0] = (long long)a.H * a.L * D[i], dst[i][1] = (long long)a.L * D[i], dst[i][2] = D[i];
      }
    }
  }
  const bool bidir = a.g_bwd != nullptr;
  if (a.gate_w) {
    geo.gw = a.gate_cols, geo.gh = a.gate_rows, geo.heads = a.H;
    return a.Dk == 64 ? launch_tiles_t<4, true, false, true>(a, geo, dev) : launch_tiles_t<2, true, false, true>(a, geo, dev);
  }
  geo.heads = 1;
  if (a.Dk == 64) {
    if (pitched)
      return bidir ? launch_tiles_t<4, true, true, false>(a, geo, dev) : launch_tiles_t<4, false, true, false>(a, geo, dev);
    return bidir ? launch_tiles_t<4, true, false, false>(a, geo, dev) : launch_tiles_t<4, false, false, false>(a, geo, dev);
  }
  if (pitched)
    return bidir ? launch_tiles_t<2, true, true, false>(a, geo, dev) : launch_tiles_t<2, false, true, false>(a, geo, dev);
  return bidir ? launch_tiles_t<2, true, false, false>(a, geo, dev) : launch_tiles_t<2, false, false, false>(a, geo, dev);
}

bool gla_tiles_chain_supported(const GlaArgs& a) {
  return a.io_dtype == 1 && a.gate_dtype == 1 && (a.Dk == 64 || a.Dk == 32) && a.Dv == 64 && a.L > 256 && !a.init_state &&
         !a.final_state && !a.state_pass && !a.gate_w && !a.q_strides && !a.k_strides && !a.v_strides &&
         gla_tile_segments(a.L) <= 65535;
}

int launch_gla_tiles_chain(const GlaArgs& a, const float* states, const float* maxima) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return -5;
  if (!gla_tiles_chain_supported(a) || !states || !maxima) return -22;
  TileGeo geo{};
  geo.L = a.L;
  geo.NT = gla_tile_segment_tiles(a.L);
  geo.H = a.H;
  geo.wide = a.wide_gates;
  geo.heads = 1;
  geo.nseg = gla_tile_segments(a.L);
  geo.states = states;
  geo.maxima = maxima;
  const bool bidir = a.g_bwd != nullptr;
  if (a.Dk == 64)
    return bidir ? launch_tiles_t<4, true, false, false, true>(a, geo, dev) : launch_tiles_t<4, false, false, false, true>(a, geo, dev);
  return bidir ? launch_tiles_t<2, true, false, false, true>(a, geo, dev) : launch_tiles_t<2, false, false, false, true>(a, geo, dev);
}

}  // namespace vig
