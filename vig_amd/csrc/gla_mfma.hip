// Bidirectional chunked GLA forward on bf16 MFMA tiles (gfx950), Dk = Dv = 64.
//
// One workgroup (4 waves) per (batch, head) slab of up to 256 tokens; wave w owns a
// contiguous chunk of ceil(L/4) <= 64 tokens.  Per direction a wave
//   1. forms the chunk-local cumulative log-gates G with a triangular-ones MFMA
//      (bf16 gates are exact MFMA inputs, the sums accumulate in fp32),
//   2. builds end-anchored operands q~ = s*q*exp(G - G_end) (>= |sq|) and
//      k~ = k*exp(G_end - G) (<= |k|), split into bf16 hi + lo,
//   3. computes the masked intra-chunk scores P^T = k~ q~^T with three MFMA terms
//      (hi*hi + lo*hi + hi*lo) and P V with P split hi + lo  (V is exact bf16),
//   4. accumulates the chunk's state contribution U = k~^T V  [Dk x Dv] fp32.
// The four U's meet once per direction in LDS; each wave folds the ones before it
// (after it, for the reverse direction) into its incoming state S_in and adds
// q~ (exp(G_end) * S_in) to its outputs.  Outputs of both directions are summed in
// the MFMA accumulators and stored once.
//
// Chunk algebra follows flash-linear-attention/fla/ops/gla/chunk_util.py:9-78 and
// chunk_fuse.py:76-97,245-254 (here with 64-token chunks, an end anchor so that the
// state update needs no second set of factors, and matrix-core intra-chunk scores);
// the two directions share q/k/v registers as in recurrent_fuse.py:19-148.
//
// Register layouts (lane l: r = l & 31, h = l >> 5), v_mfma_f32_32x32x16_bf16:
//   A/B operand: lane supplies index r and contraction slots e = 0..7 (4 VGPRs);
//   C/D: lane holds column r, register c = 4*g + m holds row 8*g + 4*h + m.
// "Transposed" fragments (tokens in the contraction slots) are read as one dword =
// two adjacent channels per token and de-interleaved with v_perm_b32; lane-row rho
// reads channel pair cpair(rho), chosen so that every accumulator ends up holding
// 32 contiguous channels (32*h + 8*g + 2*m + p) of one token.
#include "common.h"
#include "launch.h"

namespace vig {

namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kKtStride = 72;                      // bf16 elements per k~ row in LDS (144 B: conflict-free b128 writes)
constexpr int kKtBytes = 64 * kKtStride * 2;       // per wave
constexpr int kSlotBytes = 16 * 1024;              // one published U (64x64 fp32)
constexpr int kLdsKt = 0;
constexpr int kLdsSlots = 4 * kKtBytes;            // 36864
constexpr int kLdsDvec = kLdsSlots + 3 * kSlotBytes;  // 86016
constexpr int kLdsTotal = kLdsDvec + 4 * 64 * 4;   // + 1 KB decay vectors

__device__ __forceinline__ f32x16_t mfma(const u32x4_t& a, const u32x4_t& b, const f32x16_t& c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0,
                                                 0, 0);
}

__device__ __forceinline__ int cpair(int rho) { return (((rho >> 2) & 1) << 4) | ((rho >> 3) << 2) | (rho & 3); }

// token held by contraction slot e of k-step t for lane half h
__device__ __forceinline__ int jmap(int t, int h, int e) { return 16 * t + 4 * h + (e & 3) + 8 * (e >> 2); }

__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }

// Transposed fragments of a row-major [tokens][64] bf16 tile (global memory): frag[t][p] is the operand
// whose lane index is channel 2*cpair(r)+p and whose slots are the 8 tokens jmap(t,h,.).
__device__ __forceinline__ void load_tfrags_global(const uint16_t* rows, int nvalid, int r, int h,
                                                   u32x4_t (&frag)[4][2]) {
  const int c2 = 2 * cpair(r);
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    uint32_t D[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int tok = jmap(t, h, e);
      D[e] = tok < nvalid ? *reinterpret_cast<const uint32_t*>(rows + (size_t)tok * 64 + c2) : 0u;
    }
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      frag[t][0][x] = __builtin_amdgcn_perm(D[2 * x + 1], D[2 * x], 0x05040100u);
      frag[t][1][x] = __builtin_amdgcn_perm(D[2 * x + 1], D[2 * x], 0x07060302u);
    }
  }
}

// Same, one k-step, from the wave's k~ scratch in LDS.
__device__ __forceinline__ void load_tfrag_lds(const uint16_t* kt, int t, int r, int h, u32x4_t (&frag)[2]) {
  const int c2 = 2 * cpair(r);
  uint32_t D[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int tok = jmap(t, h, e);
    D[e] = *reinterpret_cast<const uint32_t*>(kt + tok * kKtStride + c2);
  }
#pragma unroll
  for (int x = 0; x < 4; ++x) {
    frag[0][x] = __builtin_amdgcn_perm(D[2 * x + 1], D[2 * x], 0x05040100u);
    frag[1][x] = __builtin_amdgcn_perm(D[2 * x + 1], D[2 * x], 0x07060302u);
  }
}

// B operand of the cumulative-sum MFMA: ones where token slot j is on the kept side of column token i.
template <bool FWD>
__device__ __forceinline__ u32x4_t tri_frag(int t, int it, int r, int h) {
  const int i = 32 * it + r;
  u32x4_t f;
#pragma unroll
  for (int x = 0; x < 4; ++x) {
    const int j0 = jmap(t, h, 2 * x), j1 = jmap(t, h, 2 * x + 1);
    const bool b0 = FWD ? (j0 <= i) : (j0 >= i);
    const bool b1 = FWD ? (j1 <= i) : (j1 >= i);
    f[x] = (b0 ? 0x00003F80u : 0u) | (b1 ? 0x3F800000u : 0u);
  }
  return f;
}

struct Operands {
  u32x4_t qh[4], ql[4], kh[4], kl[4];  // one 32-token tile, [k-step]
};

// q~ / k~ of one 32-token tile, split into bf16 hi (round to nearest) + lo (the fp32 remainder, rounded).
__device__ __forceinline__ void make_operands(const u32x4_t (&qraw)[4], const u32x4_t (&kraw)[4],
                                              const f32x16_t (&G)[2], const float (&gend2)[2][16], float l2scale,
                                              Operands& op) {
#pragma unroll
  for (int g = 0; g < 4; ++g) {
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int c = 4 * g + m;
      float qt[2], kt[2];
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        const float Gv = G[p][c];
        const float xq = __builtin_fmaf(Gv, kLog2e, l2scale - gend2[p][c]);
        const float xk = __builtin_fmaf(Gv, -kLog2e, gend2[p][c]);
        const float qf = p ? bf16hi_to_f32(qraw[g][m]) : bf16lo_to_f32(qraw[g][m]);
        const float kf = p ? bf16hi_to_f32(kraw[g][m]) : bf16lo_to_f32(kraw[g][m]);
        qt[p] = qf * exp2_fast(xq);
        kt[p] = kf * exp2_fast(xk);
      }
      const uint32_t qhi = pack_bf16x2(qt[0], qt[1]);
      const uint32_t khi = pack_bf16x2(kt[0], kt[1]);
      op.qh[g][m] = qhi;
      op.kh[g][m] = khi;
      op.ql[g][m] = pack_bf16x2(qt[0] - bf16lo_to_f32(qhi), qt[1] - bf16hi_to_f32(qhi));
      op.kl[g][m] = pack_bf16x2(kt[0] - bf16lo_to_f32(khi), kt[1] - bf16hi_to_f32(khi));
    }
  }
}

// P^T tile = k~ (rows j) x q~ (columns i), three-term split product.
__device__ __forceinline__ f32x16_t score_tile(const Operands& kop, const Operands& qop) {
  f32x16_t acc = {0.f};
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) {
    acc = mfma(kop.kh[ks], qop.qh[ks], acc);
    acc = mfma(kop.kl[ks], qop.qh[ks], acc);
    acc = mfma(kop.kh[ks], qop.ql[ks], acc);
  }
  return acc;
}

// O^T[p][it] += V^T (k-steps of token tile jt) x P^T tile, with P split hi + lo.
// MASK: 0 none, 1 keep j <= i (forward diagonal tile), 2 keep j >= i (reverse diagonal tile).
template <int MASK>
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

__device__ __forceinline__ void store_kt(uint16_t* kt, int row, int h, const u32x4_t (&kh)[4]) {
#pragma unroll
  for (int g = 0; g < 4; ++g) *reinterpret_cast<u32x4_t*>(kt + row * kKtStride + 32 * h + 8 * g) = kh[g];
}

// One direction of one wave's chunk: intra-chunk outputs into O, hi q~ fragments kept for the
// inter-chunk product, chunk state contribution U, and the chunk's total log-decay gend (natural log)
// for the lane's 32 channels.
template <bool FWD>
__device__ __forceinline__ void direction_pass(const uint16_t* grows, int nvalid, int r, int h, float l2scale,
                                               const u32x4_t (&qraw)[2][4], const u32x4_t (&kraw)[2][4],
                                               const u32x4_t (&vfrag)[4][2], f32x16_t (&O)[2][2],
                                               u32x4_t (&qkeep)[2][4], float (&gend)[2][16], f32x16_t (&U)[2][2],
                                               uint16_t* kt) {
  // ---- cumulative log-gates G[it][p] via triangular-ones MFMA ----
  f32x16_t G[2][2];
  {
    u32x4_t gfrag[4][2];
    load_tfrags_global(grows, nvalid, r, h, gfrag);
    const u32x4_t ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      f32x16_t g0 = {0.f}, g1 = {0.f};
      if (FWD) {
        // tokens i of tile 0 see j in tile 0 (masked); tile 1 sees all of tile 0 and masked tile 1
        g0 = mfma(gfrag[0][p], tri_frag<true>(0, 0, r, h), g0);
        g0 = mfma(gfrag[1][p], tri_frag<true>(1, 0, r, h), g0);
        g1 = mfma(gfrag[0][p], ones, g1);
        g1 = mfma(gfrag[1][p], ones, g1);
        g1 = mfma(gfrag[2][p], tri_frag<true>(2, 1, r, h), g1);
        g1 = mfma(gfrag[3][p], tri_frag<true>(3, 1, r, h), g1);
      } else {
        g0 = mfma(gfrag[0][p], tri_frag<false>(0, 0, r, h), g0);
        g0 = mfma(gfrag[1][p], tri_frag<false>(1, 0, r, h), g0);
        g0 = mfma(gfrag[2][p], ones, g0);
        g0 = mfma(gfrag[3][p], ones, g0);
        g1 = mfma(gfrag[2][p], tri_frag<false>(2, 1, r, h), g1);
        g1 = mfma(gfrag[3][p], tri_frag<false>(3, 1, r, h), g1);
      }
      G[0][p] = g0;
      G[1][p] = g1;
    }
  }
  // ---- anchor: G at the last token (forward) / first token (reverse) of the chunk, same channels per lane half ----
  float gend2[2][16];
  {
    const int src = ((FWD ? 31 : 0) + 32 * h) << 2;
#pragma unroll
    for (int p = 0; p < 2; ++p) {
#pragma unroll
      for (int c = 0; c < 16; ++c) {
        const float a = FWD ? G[1][p][c] : G[0][p][c];
        const float e = __int_as_float(__builtin_amdgcn_ds_bpermute(src, __float_as_int(a)));
        gend[p][c] = e;
        gend2[p][c] = e * kLog2e;
      }
    }
  }
  // ---- intra-chunk scores, tile by tile ----
  constexpr int TA = FWD ? 0 : 1;  // first tile walked
  constexpr int TB = FWD ? 1 : 0;
  Operands a, b;
  make_operands(qraw[TA], kraw[TA], G[TA], gend2, l2scale, a);
  apply_scores<FWD ? 1 : 2>(score_tile(a, a), TA, r, h, vfrag, O[0][TA], O[1][TA]);
  store_kt(kt, 32 * TA + r, h, a.kh);
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) qkeep[TA][ks] = a.qh[ks];
  make_operands(qraw[TB], kraw[TB], G[TB], gend2, l2scale, b);
  apply_scores<0>(score_tile(a, b), TA, r, h, vfrag, O[0][TB], O[1][TB]);
  apply_scores<FWD ? 1 : 2>(score_tile(b, b), TB, r, h, vfrag, O[0][TB], O[1][TB]);
  store_kt(kt, 32 * TB + r, h, b.kh);
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) qkeep[TB][ks] = b.qh[ks];
  __syncthreads();
  // ---- chunk state contribution U[p'][pv] = k~^T V ----
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) U[i][j] = f32x16_t{0.f};
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    u32x4_t ktf[2];
    load_tfrag_lds(kt, t, r, h, ktf);
#pragma unroll
    for (int pk = 0; pk < 2; ++pk)
#pragma unroll
      for (int pv = 0; pv < 2; ++pv) U[pk][pv] = mfma(ktf[pk], vfrag[t][pv], U[pk][pv]);
  }
}

__device__ __forceinline__ void publish_state(char* lds, int slot, int lane, const f32x16_t (&U)[2][2]) {
  char* base = lds + kLdsSlots + slot * kSlotBytes;
#pragma unroll
  for (int pk = 0; pk < 2; ++pk)
#pragma unroll
    for (int pv = 0; pv < 2; ++pv)
#pragma unroll
      for (int cq = 0; cq < 4; ++cq) {
        f32x4_t x = {U[pk][pv][4 * cq], U[pk][pv][4 * cq + 1], U[pk][pv][4 * cq + 2], U[pk][pv][4 * cq + 3]};
        *reinterpret_cast<f32x4_t*>(base + (((pk * 2 + pv) * 4 + cq) * 64 + lane) * 16) = x;
      }
}

__device__ __forceinline__ void publish_decay(char* lds, int w, int r, int h, const float (&gend)[2][16]) {
  if (r == 0) {
    float* d = reinterpret_cast<float*>(lds + kLdsDvec) + w * 64 + 32 * h;
#pragma unroll
    for (int p = 0; p < 2; ++p)
#pragma unroll
      for (int c = 0; c < 16; ++c) d[8 * (c >> 2) + 2 * (c & 3) + p] = gend[p][c];
  }
}

// S = exp(gend_w') * S + U_w'  for one published chunk w'
__device__ __forceinline__ void fold_state(const char* lds, int slot, int wsrc, int lane, int h, f32x16_t (&S)[2][2]) {
  const float* d = reinterpret_cast<const float*>(lds + kLdsDvec) + wsrc * 64 + 32 * h;
  const char* base = lds + kLdsSlots + slot * kSlotBytes;
#pragma unroll
  for (int pk = 0; pk < 2; ++pk) {
    float dec[16];
#pragma unroll
    for (int c = 0; c < 16; ++c) dec[c] = exp2_fast(d[8 * (c >> 2) + 2 * (c & 3) + pk] * kLog2e);
#pragma unroll
    for (int pv = 0; pv < 2; ++pv)
#pragma unroll
      for (int cq = 0; cq < 4; ++cq) {
        const f32x4_t u = *reinterpret_cast<const f32x4_t*>(base + (((pk * 2 + pv) * 4 + cq) * 64 + lane) * 16);
#pragma unroll
        for (int m = 0; m < 4; ++m) S[pk][pv][4 * cq + m] = __builtin_fmaf(S[pk][pv][4 * cq + m], dec[4 * cq + m], u[m]);
      }
  }
}

// O^T += (exp(gend) * S_in)^T-fragments x q~hi
__device__ __forceinline__ void inter_product(const f32x16_t (&S)[2][2], const float (&gend)[2][16],
                                              const u32x4_t (&qkeep)[2][4], f32x16_t (&O)[2][2]) {
  float dec[2][16];
#pragma unroll
  for (int p = 0; p < 2; ++p)
#pragma unroll
    for (int c = 0; c < 16; ++c) dec[p][c] = exp2_fast(gend[p][c] * kLog2e);
#pragma unroll
  for (int pv = 0; pv < 2; ++pv) {
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      u32x4_t sf;
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const int c = 4 * ks + m;
        sf[m] = pack_bf16x2(S[0][pv][c] * dec[0][c], S[1][pv][c] * dec[1][c]);
      }
#pragma unroll
      for (int it = 0; it < 2; ++it) O[pv][it] = mfma(sf, qkeep[it][ks], O[pv][it]);
    }
  }
}

}  // namespace

__global__ __launch_bounds__(256) void gla_mfma_slab_kernel(const uint16_t* __restrict__ q,
                                                            const uint16_t* __restrict__ k,
                                                            const uint16_t* __restrict__ v,
                                                            const uint16_t* __restrict__ gf,
                                                            const uint16_t* __restrict__ gb,
                                                            uint16_t* __restrict__ o, int L, float scale,
                                                            float out_scale) {
  extern __shared__ __align__(16) char lds[];
  const int tid = threadIdx.x;
  const int w = tid >> 6, lane = tid & 63;
  const int r = lane & 31, h = lane >> 5;
  const size_t slab = (size_t)blockIdx.x * L * 64;
  const int cw = (L + 3) >> 2;  // tokens per wave (<= 64)
  const int row0 = w * cw;
  const int nvalid = min(max(L - row0, 0), cw);
  const size_t base = slab + (size_t)row0 * 64;
  uint16_t* kt = reinterpret_cast<uint16_t*>(lds + kLdsKt + w * kKtBytes);
  const float l2scale = __log2f(scale);

  // raw q, k rows (lane = token of each 32-token tile, 32 contiguous channels) and transposed V fragments
  u32x4_t qraw[2][4], kraw[2][4];
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int row = 32 * it + r;
    const bool ok = row < nvalid;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const size_t off = base + (size_t)row * 64 + 32 * h + 8 * g;
      const u32x4_t z = {0u, 0u, 0u, 0u};
      qraw[it][g] = ok ? *reinterpret_cast<const u32x4_t*>(q + off) : z;
      kraw[it][g] = ok ? *reinterpret_cast<const u32x4_t*>(k + off) : z;
    }
  }
  u32x4_t vfrag[4][2];
  load_tfrags_global(v + base, nvalid, r, h, vfrag);

  f32x16_t O[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) O[i][j] = f32x16_t{0.f};

  u32x4_t qkeep[2][4];
  float gend[2][16];
  f32x16_t U[2][2];

  // ------------------------------ forward direction ------------------------------
  direction_pass<true>(gf + base, nvalid, r, h, l2scale, qraw, kraw, vfrag, O, qkeep, gend, U, kt);
  if (w < 3) publish_state(lds, w, lane, U);
  publish_decay(lds, w, r, h, gend);
  __syncthreads();
  if (w > 0) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) U[i][j] = f32x16_t{0.f};
    for (int ws = 0; ws < w; ++ws) fold_state(lds, ws, ws, lane, h, U);
    inter_product(U, gend, qkeep, O);
  }
  __syncthreads();

  // ------------------------------ reverse direction ------------------------------
  if (gb != nullptr) {
    direction_pass<false>(gb + base, nvalid, r, h, l2scale, qraw, kraw, vfrag, O, qkeep, gend, U, kt);
    if (w > 0) publish_state(lds, w - 1, lane, U);
    publish_decay(lds, w, r, h, gend);
    __syncthreads();
    if (w < 3) {
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) U[i][j] = f32x16_t{0.f};
      for (int ws = 3; ws > w; --ws) fold_state(lds, ws - 1, ws, lane, h, U);
      inter_product(U, gend, qkeep, O);
    }
  }

  // ------------------------------ store ------------------------------
#pragma unroll
  for (int it = 0; it < 2; ++it) {
    const int row = 32 * it + r;
    if (row < nvalid) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x4_t x;
#pragma unroll
        for (int m = 0; m < 4; ++m)
          x[m] = pack_bf16x2(O[0][it][4 * g + m] * out_scale, O[1][it][4 * g + m] * out_scale);
        *reinterpret_cast<u32x4_t*>(o + base + (size_t)row * 64 + 32 * h + 8 * g) = x;
      }
    }
  }
}

bool gla_mfma_supported(const GlaArgs& a) {
  return a.io_dtype == 1 && a.gate_dtype == 1 && a.Dk == 64 && a.Dv == 64 && a.L <= 256 && a.scale > 0.f;
}

size_t gla_mfma_workspace(int, int, int, int, int) { return 0; }

int launch_gla_mfma(const GlaArgs& a) {
  static bool attr_set = false;
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(gla_mfma_slab_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, kLdsTotal) != hipSuccess)
      return -5;
    attr_set = true;
  }
  hipLaunchKernelGGL(gla_mfma_slab_kernel, dim3(a.B * a.H), dim3(256), kLdsTotal, a.stream, (const uint16_t*)a.q,
                     (const uint16_t*)a.k, (const uint16_t*)a.v, (const uint16_t*)a.g_fwd, (const uint16_t*)a.g_bwd,
                     (uint16_t*)a.o, a.L, a.scale, a.out_scale);
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

}  // namespace vig
