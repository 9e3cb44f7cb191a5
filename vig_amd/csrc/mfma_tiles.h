// Building blocks shared by the MFMA kernels (gfx950, v_mfma_f32_32x32x16_bf16): fragment layouts, loads through
// buffer descriptors, transposed fragments, LDS helpers.
//
// Register layouts (lane l: r = l & 31, h = l >> 5):
//   A/B operand: lane supplies index r and contraction slots e = 0..7 (4 VGPRs);
//   C/D: lane holds column r, register c = 4*g + m holds row 8*g + 4*h + m.
// "Transposed" fragments (tokens in the contraction slots) are read as one dword = two adjacent channels per token
// and de-interleaved with v_perm_b32; lane-row rho reads channel pair cpair(rho), chosen so that every accumulator
// ends up holding 32 contiguous channels (32*h + 8*g + 2*m + p) of one token.
#pragma once
#include "common.h"

namespace vig {
namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kKtStride = 72;                // bf16 elements per k~ row in LDS (144 B: conflict-free b128 writes)

__device__ __forceinline__ f32x16_t mfma(const u32x4_t& a, const u32x4_t& b, const f32x16_t& c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0,
                                                 0, 0);
}


// Channel pair read by lane-row rho of a transposed fragment whose rows span 16*NG channels (NG = 4: 64 channels,
// every row used; NG = 2: 32 channels, rows 16..31 carry no channel and are zero).  With it, accumulator register
// 4*g + m of lane half h holds channel 8*NG*h + 8*g + 2*m + p.
template <int NG>
__device__ __forceinline__ int cpair(int rho) { return (((rho >> 2) & 1) * (4 * NG)) | ((rho >> 3) << 2) | (rho & 3); }
template <int NG>
__device__ __forceinline__ bool row_has_channel(int rho) { return (rho >> 3) < NG; }

// token held by contraction slot e of k-step t for lane half h
__device__ __forceinline__ int jmap(int t, int h, int e) { return 16 * t + 4 * h + (e & 3) + 8 * (e >> 2); }

__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }

// LDS traffic inside one wave (k~ rows written by token lanes, read back by channel lanes): the LDS pipe is in
// order per wave, so only the compiler has to be kept from reordering.
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Workgroup barrier that orders LDS traffic only: global loads issued before it (the next slab's prefetch)
// stay in flight across it, which a full __syncthreads() fence would drain.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// ---------------------------------------------------------------------------------------------------------
// Loads.  Every tensor chunk is addressed through a raw buffer descriptor whose extent is the chunk's valid rows:
// the hardware returns zero for anything beyond it, so padding rows need neither clamped addresses nor selects
// (zero gates, keys and values are exactly what padding tokens have to contribute), and token offsets travel as
// instruction immediates.
// ---------------------------------------------------------------------------------------------------------
typedef __amdgpu_buffer_rsrc_t rsrc_t;

// descriptor of `rows` rows of `row_bytes` starting at p (p and rows are wave-uniform)
__device__ __forceinline__ rsrc_t chunk_rsrc(const void* p, int rows, int row_bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, rows * row_bytes, 0x00020000);
}
constexpr unsigned kOutOfRange = 0x40000000u;  // byte offset no descriptor of this kernel covers

// raw dwords of the transposed fragments of k-steps [T0, T0+NT): D[t][e] = channels (2*cpair(r), +1) of token
// jmap(t,h,e); lane rows that carry no channel (NG = 2, rows 16..31) read zeros
template <int T0, int NT, int NG>
__device__ __forceinline__ void issue_tdwords(rsrc_t rows, int r, int h, uint32_t (&D)[NT][8]) {
  constexpr unsigned RB = 32u * NG;  // bytes per row
  const unsigned base = row_has_channel<NG>(r) ? (4u * h) * RB + 4u * cpair<NG>(r) : kOutOfRange;
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int e = 0; e < 8; ++e)
      D[t][e] = __builtin_amdgcn_raw_buffer_load_b32(rows, base + (unsigned)jmap(T0 + t, 0, e) * RB, 0, 0);
}

// the same for rows that lie `pitch` bytes apart (a head's channels inside wider token rows): the token offsets travel
// in the scalar offset operand instead of the immediate
template <int T0, int NT, int NG>
__device__ __forceinline__ void issue_tdwords_pitched(rsrc_t rows, int r, int h, unsigned pitch, uint32_t (&D)[NT][8]) {
  const unsigned base = row_has_channel<NG>(r) ? (4u * h) * pitch + 4u * cpair<NG>(r) : kOutOfRange;
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int e = 0; e < 8; ++e)
      D[t][e] = __builtin_amdgcn_raw_buffer_load_b32(rows, base, (unsigned)jmap(T0 + t, 0, e) * pitch, 0);
}

// fragments from raw dwords: frag[t][p] has lane index = channel 2*cpair(r)+p, slots = tokens jmap(t,h,.)
template <int NT>
__device__ __forceinline__ void finish_tfrags(const uint32_t (&D)[NT][8], u32x4_t (&frag)[NT][2]) {
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      frag[t][0][x] = __builtin_amdgcn_perm(D[t][2 * x + 1], D[t][2 * x], 0x05040100u);
      frag[t][1][x] = __builtin_amdgcn_perm(D[t][2 * x + 1], D[t][2 * x], 0x07060302u);
    }
}

// raw rows of one 32-token tile: lane (r, h) reads token 32*it + r, channels [8*NG*h, +8*NG) as NG 16-byte pieces
template <int NG>
__device__ __forceinline__ void issue_raw_tile(rsrc_t rows, int it, int r, int h, u32x4_t (&raw)[NG]) {
  constexpr unsigned RB = 32u * NG;
  const unsigned base = (unsigned)r * RB + (16u * NG) * h;
#pragma unroll
  for (int gq = 0; gq < NG; ++gq)
    raw[gq] = __builtin_amdgcn_raw_buffer_load_b128(rows, base + (unsigned)it * 32u * RB + 16u * gq, 0, 0);
}

template <int NG>
__device__ __forceinline__ void issue_raw_tile_pitched(rsrc_t rows, int it, int r, int h, unsigned pitch,
                                                       u32x4_t (&raw)[NG]) {
  const unsigned base = (unsigned)r * pitch + (16u * NG) * h;
#pragma unroll
  for (int gq = 0; gq < NG; ++gq)
    raw[gq] = __builtin_amdgcn_raw_buffer_load_b128(rows, base + 16u * gq, (unsigned)it * 32u * pitch, 0);
}

// one k-step of transposed fragments from the wave's k~ scratch in LDS
template <int NG, int STRIDE = kKtStride>
__device__ __forceinline__ void load_tfrag_lds(const uint16_t* kt, int t, int r, int h, u32x4_t (&frag)[2]) {
  const bool row_ok = row_has_channel<NG>(r);
  const int c2 = row_ok ? 2 * cpair<NG>(r) : 0;
  uint32_t D[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const uint32_t d = *reinterpret_cast<const uint32_t*>(kt + jmap(t, h, e) * STRIDE + c2);
    D[e] = (NG == 4 || row_ok) ? d : 0u;
  }
#pragma unroll
  for (int x = 0; x < 4; ++x) {
    frag[0][x] = __builtin_amdgcn_perm(D[2 * x + 1], D[2 * x], 0x05040100u);
    frag[1][x] = __builtin_amdgcn_perm(D[2 * x + 1], D[2 * x], 0x07060302u);
  }
}

// B operand of the cumulative-sum MFMA: ones where token slot j is on the kept side of column token i (STRICT: the
// token itself is not kept).
template <bool FWD, bool STRICT = false>
__device__ __forceinline__ u32x4_t tri_frag(int t, int it, int r, int h) {
  const int i = 32 * it + r;
  u32x4_t f;
#pragma unroll
  for (int x = 0; x < 4; ++x) {
    const int j0 = jmap(t, h, 2 * x), j1 = jmap(t, h, 2 * x + 1);
    const bool b0 = STRICT ? (FWD ? (j0 < i) : (j0 > i)) : (FWD ? (j0 <= i) : (j0 >= i));
    const bool b1 = STRICT ? (FWD ? (j1 < i) : (j1 > i)) : (FWD ? (j1 <= i) : (j1 >= i));
    f[x] = (b0 ? 0x00003F80u : 0u) | (b1 ? 0x3F800000u : 0u);
  }
  return f;
}

template <int NG, int STRIDE = kKtStride>
__device__ __forceinline__ void store_kt(uint16_t* kt, int row, int h, const u32x4_t (&kh)[NG]) {
#pragma unroll
  for (int g = 0; g < NG; ++g) *reinterpret_cast<u32x4_t*>(kt + row * STRIDE + 8 * NG * h + 8 * g) = kh[g];
}

// ---- fp16 operands, magnitude guard, split-bf16 operands, LDS units (shared by the forward kernels) ----
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
__device__ __forceinline__ f32x16_t mfma_f16(const u32x4_t& a, const u32x4_t& b, const f32x16_t& c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0,
                                                0, 0);
}
__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi) {
  f32x2_t x = {lo, hi};
  f16x2_t y = __builtin_convertvector(x, f16x2_t);  // round to nearest even
  return __builtin_bit_cast(uint32_t, y);
}
// elementwise product of two fp16 pairs (operands by value: a bit cast straight from a vector element reads the
// vector's first word)
__device__ __forceinline__ uint32_t mul_f16x2(uint32_t a, uint32_t b) {
  return __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2_t, a) * __builtin_bit_cast(f16x2_t, b));
}

__device__ __forceinline__ uint32_t add_f16x2(uint32_t a, uint32_t b) {
  return __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2_t, a) + __builtin_bit_cast(f16x2_t, b));
}

// Magnitude guard of the fp16 score variant.  Raw bf16 rows go through a 16x16x32 matrix instruction as both
// operands: whatever the slot assignment, the result is a Gram matrix whose diagonal entries are sums of squares that
// cover every value fed in and whose other entries are no larger than the largest diagonal one.  Eight passes and four
// accumulator registers per step, no vector work until the one comparison at the end.
typedef float f32x4acc_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void gram_acc(const u32x4_t& raw, f32x4acc_t& acc) {
  acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, raw), __builtin_bit_cast(bf16x8_t, raw), acc,
                                                0, 0, 0);
}
template <int NG>
struct HalfOps {
  u32x4_t h[NG], l[NG];  // bf16 hi / lo fragments of one 32-token tile, per k-step (16 channels)
};

// q~ (ISQ) or k~ of one 32-token tile: raw * exp(+-(G - G_end)), split into bf16 hi (round to nearest) and
// lo (the fp32 remainder, rounded).  Padding rows arrive as zeros and stay zero (their exponents are finite).
template <bool ISQ, int NG>
__device__ __forceinline__ void make_half(const u32x4_t (&raw)[NG], const f32x16_t (&G)[2],
                                          const float* gend2 /* LDS, this lane half: [p][16] */, HalfOps<NG>& op) {
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    const f32x4_t a0 = *reinterpret_cast<const f32x4_t*>(gend2 + 4 * g);
    const f32x4_t a1 = *reinterpret_cast<const f32x4_t*>(gend2 + 16 + 4 * g);
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int c = 4 * g + m;
      const uint32_t w = raw[g][m];
      float t[2];
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        const float an = p ? a1[m] : a0[m];
        const float x = ISQ ? __builtin_fmaf(G[p][c], kLog2e, -an) : __builtin_fmaf(G[p][c], -kLog2e, an);
        const float f = p ? bf16hi_to_f32(w) : bf16lo_to_f32(w);
        t[p] = f * exp2_fast(x);
      }
      const uint32_t hi = pack_bf16x2(t[0], t[1]);
      op.h[g][m] = hi;
      op.l[g][m] = pack_bf16x2(t[0] - bf16lo_to_f32(hi), t[1] - bf16hi_to_f32(hi));
    }
  }
}

// P^T tile = k~ (rows j) x q~ (columns i) on fp16 operands.
template <int NG>
__device__ __forceinline__ f32x16_t score_tile16(const u32x4_t (&k16)[NG], const u32x4_t (&q16)[NG]) {
  f32x16_t acc = {0.f};
#pragma unroll
  for (int ks = 0; ks < NG; ++ks) acc = mfma_f16(k16[ks], q16[ks], acc);
  return acc;
}

// P^T tile = k~ (rows j) x q~ (columns i), three-term split product.
template <int NG>
__device__ __forceinline__ f32x16_t score_tile(const HalfOps<NG>& kop, const HalfOps<NG>& qop) {
  f32x16_t acc = {0.f};
#pragma unroll
  for (int ks = 0; ks < NG; ++ks) {
    acc = mfma(kop.h[ks], qop.h[ks], acc);
    acc = mfma(kop.l[ks], qop.h[ks], acc);
    acc = mfma(kop.h[ks], qop.l[ks], acc);
  }
  return acc;
}

// LDS "unit" u of a region = 64 lanes x 16 B, register-native: lane l owns bytes [(u*64 + l)*16, +16).
__device__ __forceinline__ char* unit_ptr(char* region, int u, int lane) { return region + (u * 64 + lane) * 16; }



}  // namespace
}  // namespace vig
