// Elementwise / stencil neighbours of the GLA op: direction-wise gate preparation,
// the 3x3 depthwise stencil on the token grid, the sigmoid locality gate and the
// RMS-norm blend epilogue.  All are HBM-bound: each element is read once with
// 16-byte (bf16 x8) or 16-byte (f32 x4) accesses along the channel dimension and
// written once; stencil neighbours come from L1/L2.
#include "common.h"
#include "launch.h"

namespace vig {

// ---------------------------------------------------------------------------
// vector-of-8 channel access (one 16-byte transaction for bf16, two for f32)
// ---------------------------------------------------------------------------
template <typename T> struct Vec8;
template <> struct Vec8<uint16_t> {
  static __device__ __forceinline__ void load(const uint16_t* p, float (&x)[8]) {
    const u32x4_t r = *reinterpret_cast<const u32x4_t*>(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[2 * i] = bf16lo_to_f32(r[i]);
      x[2 * i + 1] = bf16hi_to_f32(r[i]);
    }
  }
  static __device__ __forceinline__ void store(uint16_t* p, const float (&x)[8]) {
    u32x4_t r;
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = pack_bf16x2(x[2 * i], x[2 * i + 1]);
    *reinterpret_cast<u32x4_t*>(p) = r;
  }
};
template <> struct Vec8<float> {
  static __device__ __forceinline__ void load(const float* p, float (&x)[8]) {
    const f32x4_t a = *reinterpret_cast<const f32x4_t*>(p);
    const f32x4_t b = *reinterpret_cast<const f32x4_t*>(p + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[i] = a[i];
      x[4 + i] = b[i];
    }
  }
  static __device__ __forceinline__ void store(float* p, const float (&x)[8]) {
    f32x4_t a, b;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a[i] = x[i];
      b[i] = x[4 + i];
    }
    *reinterpret_cast<f32x4_t*>(p) = a;
    *reinterpret_cast<f32x4_t*>(p + 4) = b;
  }
};

// ---------------------------------------------------------------------------
// direction-wise gate preparation
//   in  [B, L, 2*H*Dk]  ->  out [2, B, H, L, Dk],  logsigmoid(x) * inv_norm, clamp
// One workgroup owns 32 consecutive tokens of one batch element: it reads their rows (contiguous, 2*H*Dk channels
// each) with 16-byte accesses and writes, per (direction, head), a contiguous run of 32 tokens x Dk.  A thread keeps
// one channel octet for all its tokens, so the layout arithmetic is done once per thread.
// ---------------------------------------------------------------------------
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void dirgate_kernel(const TI* __restrict__ in, TO* __restrict__ out, int B, int L,
                                                       int H, int Dk, float inv_norm, float clamp_min, int use_clamp) {
  const int nv = 2 * H * Dk / 8;         // channel octets per token row
  const int dk8 = Dk >> 3;
  const int b = blockIdx.y;
  const int l0 = blockIdx.x * 32;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // 64 octet lanes x 4 token lanes
  for (int cv = tx; cv < nv; cv += 64) {
    const int d8 = cv % dk8, hh = (cv / dk8) % H, dir = cv / (dk8 * H);
    const TI* src = in + ((size_t)b * L) * (size_t)(nv * 8) + (size_t)cv * 8;
    TO* dst = out + ((((size_t)dir * B + b) * H + hh) * L) * (size_t)Dk + (size_t)d8 * 8;
    for (int t = ty; t < 32; t += 4) {
      const int l = l0 + t;
      if (l >= L) break;
      float x[8];
      Vec8<TI>::load(src + (size_t)l * (nv * 8), x);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        // logsigmoid(x) = min(x,0) - log(1 + exp(-|x|)); hardware exp/log are accurate to ~1e-7 absolute here
        float yv = logsigmoidf_(x[j]);
        yv *= inv_norm;
        if (use_clamp) yv = fmaxf(yv, clamp_min);
        x[j] = yv;
      }
      Vec8<TO>::store(dst + (size_t)l * Dk, x);
    }
  }
}

// Backward of the gate preparation: d_in[b, l, c] = d_out[dir, b, h, l, d] * inv_norm * sigmoid(-x), zero where the
// forward clamped (x = in[b, l, c]; d/dx logsigmoid(x) = sigmoid(-x)).
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void dirgate_bwd_kernel(const TI* __restrict__ in, const TO* __restrict__ d_out,
                                                           TI* __restrict__ d_in, int B, int L, int H, int Dk,
                                                           float inv_norm, float clamp_min, int use_clamp) {
  const int nv = 2 * H * Dk / 8;
  const int dk8 = Dk >> 3;
  const int b = blockIdx.y;
  const int l0 = blockIdx.x * 32;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int cv = tx; cv < nv; cv += 64) {
    const int d8 = cv % dk8, hh = (cv / dk8) % H, dir = cv / (dk8 * H);
    const size_t rows = ((size_t)b * L) * (size_t)(nv * 8) + (size_t)cv * 8;
    const TO* grad = d_out + ((((size_t)dir * B + b) * H + hh) * L) * (size_t)Dk + (size_t)d8 * 8;
    for (int t = ty; t < 32; t += 4) {
      const int l = l0 + t;
      if (l >= L) break;
      float x[8], g[8];
      Vec8<TI>::load(in + rows + (size_t)l * (nv * 8), x);
      Vec8<TO>::load(grad + (size_t)l * Dk, g);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const bool clamped = use_clamp && logsigmoidf_(x[j]) * inv_norm < clamp_min;
        x[j] = clamped ? 0.f : g[j] * inv_norm * sigmoidf_(-x[j]);
      }
      Vec8<TI>::store(d_in + rows + (size_t)l * (nv * 8), x);
    }
  }
}

int launch_dirgate_bwd(const void* in, const void* d_out, void* d_in, int B, int L, int H, int Dk, float inv_norm,
                       float clamp_min, int in_dtype, int out_dtype, hipStream_t stream) {
  const int use_clamp = clamp_min == clamp_min;  // NaN disables
  if (B > 65535) return -22;
  const dim3 grid((L + 31) / 32, B), block(256);
#define VIG_DGB_CASE(TI, TO)                                                                                       \
  hipLaunchKernelGGL((dirgate_bwd_kernel<TI, TO>), grid, block, 0, stream, (const TI*)in, (const TO*)d_out, (TI*)d_in, \
                     B, L, H, Dk, inv_norm, clamp_min, use_clamp)
  if (in_dtype == 0 && out_dtype == 0) VIG_DGB_CASE(float, float);
  else if (in_dtype == 0 && out_dtype == 1) VIG_DGB_CASE(float, uint16_t);
  else if (in_dtype == 1 && out_dtype == 0) VIG_DGB_CASE(uint16_t, float);
  else VIG_DGB_CASE(uint16_t, uint16_t);
#undef VIG_DGB_CASE
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

template <typename TI, typename TO>
static int launch_dirgate_t(const void* in, void* out, int B, int L, int H, int Dk, float inv_norm,
                            float clamp_min, hipStream_t stream) {
  const int use_clamp = clamp_min == clamp_min;  // NaN disables
  if (B > 65535) return -22;
  hipLaunchKernelGGL((dirgate_kernel<TI, TO>), dim3((L + 31) / 32, B), dim3(256), 0, stream, (const TI*)in, (TO*)out, B,
                     L, H, Dk, inv_norm, clamp_min, use_clamp);
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

int launch_dirgate(const void* in, void* out, int B, int L, int H, int Dk, float inv_norm, float clamp_min,
                   int in_dtype, int out_dtype, hipStream_t stream) {
  if (in_dtype == 0 && out_dtype == 0) return launch_dirgate_t<float, float>(in, out, B, L, H, Dk, inv_norm, clamp_min, stream);
  if (in_dtype == 0 && out_dtype == 1) return launch_dirgate_t<float, uint16_t>(in, out, B, L, H, Dk, inv_norm, clamp_min, stream);
  if (in_dtype == 1 && out_dtype == 0) return launch_dirgate_t<uint16_t, float>(in, out, B, L, H, Dk, inv_norm, clamp_min, stream);
  return launch_dirgate_t<uint16_t, uint16_t>(in, out, B, L, H, Dk, inv_norm, clamp_min, stream);
}

// ---------------------------------------------------------------------------
// direction-wise gate preparation with the second (rank -> 2*H*Dk) layer of the gate projection inside:
//   low [B, L, 16] (rows ld elements apart), w1 [2*H*Dk, 16], b1 [2*H*Dk]
//   x = low . w1^T + b1, rounded to the storage type of `low` (what the separate layer would have stored),
//   out [2, B, H, L, Dk] = logsigmoid(x) * inv_norm, clamp
// The rank-16 product is 16 multiply-adds per output, far below what the output write costs, so the [B, L, 2*H*Dk]
// intermediate never goes to memory.  One workgroup owns 32 consecutive tokens of one batch element; their low-rank
// rows sit in LDS as f32; a thread keeps the 8x16 weights of one channel octet in registers for all its tokens.
// ---------------------------------------------------------------------------
constexpr int kGateRank = 16;

template <typename T> struct Stored;  // value after a round trip through the storage type
template <> struct Stored<float> { static __device__ __forceinline__ float of(float x) { return x; } };
template <> struct Stored<uint16_t> {
  static __device__ __forceinline__ float of(float x) { return bf16_to_f32(f32_to_bf16(x)); }
};

template <typename TI, typename TO>
__global__ __launch_bounds__(256) void dirgate_lowrank_kernel(const TI* __restrict__ low, long long ld,
                                                               const TI* __restrict__ w1, const TI* __restrict__ b1,
                                                               TO* __restrict__ out, int B, int L, int H, int Dk,
                                                               float inv_norm, float clamp_min, int use_clamp) {
  constexpr int R = kGateRank, TOK = 32;
  __shared__ float lowf[TOK][R];
  const int nv = 2 * H * Dk / 8;  // channel octets per token row
  const int dk8 = Dk >> 3;
  const int b = blockIdx.y;
  const int l0 = blockIdx.x * TOK;
  if (threadIdx.x < TOK * (R / 8)) {
    const int t = threadIdx.x / (R / 8), part = threadIdx.x % (R / 8);
    float x[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (l0 + t < L) Vec8<TI>::load(low + ((size_t)b * L + l0 + t) * (size_t)ld + part * 8, x);
#pragma unroll
    for (int j = 0; j < 8; ++j) lowf[t][part * 8 + j] = x[j];
  }
  __syncthreads();
  const int per = nv < 256 ? nv : 256;  // threads side by side on one token
  const int groups = 256 / per;         // tokens in flight
  const int oc = threadIdx.x % per, tg = threadIdx.x / per;
  if (tg >= groups) return;
  for (int cv = oc; cv < nv; cv += per) {
    float w[8][R], bias[8];
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int p = 0; p < R / 8; ++p) {
        float x[8];
        Vec8<TI>::load(w1 + ((size_t)cv * 8 + j) * R + p * 8, x);
#pragma unroll
        for (int i = 0; i < 8; ++i) w[j][p * 8 + i] = x[i];
      }
    Vec8<TI>::load(b1 + (size_t)cv * 8, bias);
    const int d8 = cv % dk8, hh = (cv / dk8) % H, dir = cv / (dk8 * H);
    TO* dst = out + ((((size_t)dir * B + b) * H + hh) * L) * (size_t)Dk + (size_t)d8 * 8;
    for (int t = tg; t < TOK; t += groups) {
      const int l = l0 + t;
      if (l >= L) break;
      float acc[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const float xr = lowf[t][r];
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] = __builtin_fmaf(xr, w[j][r], acc[j]);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float x = Stored<TI>::of(acc[j] + bias[j]);
        float yv = logsigmoidf_(x);
        yv *= inv_norm;
        yv = fmaxf(yv, clamp_min);  // (no clamp: clamp_min is NaN and fmaxf returns the other operand)
        acc[j] = yv;
      }
      Vec8<TO>::store(dst + (size_t)l * Dk, acc);
    }
  }
}

// The same for bf16 inputs on the matrix cores: one v_mfma_f32_32x32x16_bf16 is the whole rank-16 product of 32
// channels x 32 tokens.  Operand A holds weight rows, operand B the tokens' low-rank rows, both read straight from
// memory as one 16-byte load per lane (lane = (row r, contraction half h) supplies elements 8h..8h+7 of its row).
// Accumulator register 4g+m of lane (r, h) holds matrix row 8g+4h+m of column r; matrix row i is given channel
// 16*((i>>2)&1) + 4*(i>>3) + (i&3) of the tile, so that lane (r, h) ends up with channels 16h..16h+15 of token r:
// 32 contiguous bytes of the head-major output.  Tokens are numbered over B*L; a workgroup owns NTG groups of 32 and
// its four waves take the channel tiles in turn, each weight tile serving all the groups.  Needs Dk % 16 == 0 (a 16-channel run stays inside one head).
template <typename TO, int NTG>
__global__ __launch_bounds__(256) void dirgate_lowrank_mfma_kernel(const uint16_t* __restrict__ low, long long ld,
                                                                    const uint16_t* __restrict__ w1,
                                                                    const uint16_t* __restrict__ b1,
                                                                    TO* __restrict__ out, long long ntok, int B, int L,
                                                                    int H, int Dk, float inv_norm, float clamp_min,
                                                                    int use_clamp) {
  constexpr int R = kGateRank;
  (void)use_clamp;  // (a NaN clamp_min already means "no clamp" to fmaxf)
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 31, h = lane >> 5;
  // NTG groups of 32 tokens per workgroup: their low-rank rows are fetched first, a weight tile serves all of them
  u32x4_t xb[NTG];
  bool tok_ok[NTG];
  size_t row_off[NTG];  // (b*H*L + l) * Dk of the token: head hh adds hh*L*Dk
#pragma unroll
  for (int g = 0; g < NTG; ++g) {
    const unsigned tok = (blockIdx.x * NTG + g) * 32u + r;  // the launch keeps B*L below 2^31
    tok_ok[g] = tok < (unsigned)ntok;
    const unsigned tokc = tok_ok[g] ? tok : (unsigned)ntok - 1;
    xb[g] = *reinterpret_cast<const u32x4_t*>(low + (size_t)tokc * (size_t)ld + 8 * h);
    const unsigned b = tokc / (unsigned)L, l = tokc - b * (unsigned)L;
    row_off[g] = ((size_t)b * H * L + l) * (size_t)Dk;
  }
  const int chan_of_row = 16 * ((r >> 2) & 1) + 4 * (r >> 3) + (r & 3);
  const int ntiles = 2 * H * Dk / 32;
  const size_t dir_stride = (size_t)B * H * L * Dk;
  // a tile's weights and biases are requested one tile ahead (a wave walks tiles wave, wave + 4, ...)
  auto request = [&](int tile, u32x4_t& wa, u32x4_t& blo, u32x4_t& bhi) {
    const int c0 = min(tile, ntiles - 1) * 32;
    wa = *reinterpret_cast<const u32x4_t*>(w1 + (size_t)(c0 + chan_of_row) * R + 8 * h);
    blo = *reinterpret_cast<const u32x4_t*>(b1 + c0 + 16 * h);
    bhi = *reinterpret_cast<const u32x4_t*>(b1 + c0 + 16 * h + 8);
  };
  u32x4_t wa_next, blo_next, bhi_next;
  request(wave, wa_next, blo_next, bhi_next);
  const float inv_dk = 1.0f / (float)Dk, inv_h = 1.0f / (float)H;
  for (int tile = wave; tile < ntiles; tile += 4) {
    const int c0 = tile * 32;
    const u32x4_t wa = wa_next, blo = blo_next, bhi = bhi_next;
    request(tile + 4, wa_next, blo_next, bhi_next);
    float bias[16];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      bias[2 * j] = bf16lo_to_f32(blo[j]), bias[2 * j + 1] = bf16hi_to_f32(blo[j]);
      bias[8 + 2 * j] = bf16lo_to_f32(bhi[j]), bias[8 + 2 * j + 1] = bf16hi_to_f32(bhi[j]);
    }
    const int c = c0 + 16 * h;  // first of this lane's 16 channels
    // (quotients by float reciprocals: exact for channel numbers below 2^20, a fraction of the integer division's cost)
    const int cd = (int)(((float)c + 0.5f) * inv_dk), d = c - cd * Dk;
    const int dir = (int)(((float)cd + 0.5f) * inv_h), hh = cd - dir * H;
    TO* const dst0 = out + (size_t)dir * dir_stride + (size_t)hh * L * Dk + d;
#pragma unroll
    for (int g = 0; g < NTG; ++g) {
      f32x16_t acc;
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[j] = 0.f;
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, wa),
                                                    __builtin_bit_cast(bf16x8_t, xb[g]), acc, 0, 0, 0);
      float lo[8], hi[8];
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const float x = Stored<uint16_t>::of(acc[j] + bias[j]);
        float yv = logsigmoidf_(x);
        yv *= inv_norm;
        yv = fmaxf(yv, clamp_min);  // (no clamp: clamp_min is NaN and fmaxf returns the other operand)
        if (j < 8) lo[j] = yv;
        else hi[j - 8] = yv;
      }
      if (tok_ok[g]) {
        TO* dst = dst0 + row_off[g];
        Vec8<TO>::store(dst, lo);
        Vec8<TO>::store(dst + 8, hi);
      }
    }
  }
}

template <typename TI, typename TO>
static int launch_dirgate_lowrank_t(const void* low, long long ld, const void* w1, const void* b1, void* out, int B,
                                    int L, int H, int Dk, float inv_norm, float clamp_min, hipStream_t stream) {
  const int use_clamp = clamp_min == clamp_min;  // NaN disables
  if (B > 65535) return -22;
  hipLaunchKernelGGL((dirgate_lowrank_kernel<TI, TO>), dim3((L + 31) / 32, B), dim3(256), 0, stream, (const TI*)low, ld,
                     (const TI*)w1, (const TI*)b1, (TO*)out, B, L, H, Dk, inv_norm, clamp_min, use_clamp);
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

int launch_dirgate_lowrank(const void* low, long long ld, const void* w1, const void* b1, void* out, int B, int L,
                           int H, int Dk, int rank, float inv_norm, float clamp_min, int in_dtype, int out_dtype,
                           hipStream_t stream) {
  if (rank != kGateRank) return -95;
  if (in_dtype == 1 && Dk % 16 == 0 && (long long)B * L < 0x7fffffffLL - 64 && 2LL * H * Dk <= (1 << 20)) {
    const int use_clamp = clamp_min == clamp_min;  // NaN disables
    const long long ntok = (long long)B * L;
    constexpr int kGroups = 1;  // token groups of 32 per workgroup (two measured no faster)
    const dim3 grid((unsigned)((ntok + 32 * kGroups - 1) / (32 * kGroups))), block(256);
    if (out_dtype == 1)
      hipLaunchKernelGGL((dirgate_lowrank_mfma_kernel<uint16_t, kGroups>), grid, block, 0, stream, (const uint16_t*)low, ld,
                         (const uint16_t*)w1, (const uint16_t*)b1, (uint16_t*)out, ntok, B, L, H, Dk, inv_norm,
                         clamp_min, use_clamp);
    else
      hipLaunchKernelGGL((dirgate_lowrank_mfma_kernel<float, kGroups>), grid, block, 0, stream, (const uint16_t*)low, ld,
                         (const uint16_t*)w1, (const uint16_t*)b1, (float*)out, ntok, B, L, H, Dk, inv_norm,
                         clamp_min, use_clamp);
    return hipGetLastError() == hipSuccess ? 0 : -5;
  }
  if (in_dtype == 0 && out_dtype == 0) return launch_dirgate_lowrank_t<float, float>(low, ld, w1, b1, out, B, L, H, Dk, inv_norm, clamp_min, stream);
  if (in_dtype == 0 && out_dtype == 1) return launch_dirgate_lowrank_t<float, uint16_t>(low, ld, w1, b1, out, B, L, H, Dk, inv_norm, clamp_min, stream);
  if (in_dtype == 1 && out_dtype == 0) return launch_dirgate_lowrank_t<uint16_t, float>(low, ld, w1, b1, out, B, L, H, Dk, inv_norm, clamp_min, stream);
  return launch_dirgate_lowrank_t<uint16_t, uint16_t>(low, ld, w1, b1, out, B, L, H, Dk, inv_norm, clamp_min, stream);
}

// ---------------------------------------------------------------------------
// 3x3 depthwise stencil on the token grid, channels-last.  One workgroup owns one image (or one head slab), a
// group of 64 channels and a band of grid rows: it stages the band plus a one-cell halo all around in LDS, with
// zeros where the halo leaves the grid (coalesced 16-byte loads, every input byte leaves L2 once, and no tap needs a
// bounds check or a clamped address).  Thread = (channel octet, token lane) keeps the 8x9 weights of its channels
// in registers and walks the band's tokens lane, lane+32, ...
//   GATE = false:  y = conv(x) (+bias) (SiLU optional)          x, y [N, h*w, C] with row stride `stride` elements
//   GATE = true :  y = x * sigmoid(conv(x))                      (bias / SiLU unused)
// weights [Ctot, 9] f32.
// ---------------------------------------------------------------------------
constexpr int kStencilGroup = 64;  // channels per workgroup

template <typename T, bool GATE>
__global__ __launch_bounds__(256) void stencil3x3_kernel(const T* __restrict__ x, const float* __restrict__ wt,
                                                          const float* __restrict__ bias, T* __restrict__ y, int h, int w,
                                                          int stride, int groups_per_image, int wmod, int cgroup,
                                                          int band_rows, int silu) {
  extern __shared__ __align__(16) char smem[];
  T* tile = reinterpret_cast<T*>(smem);  // [(band_rows + 2) * (w + 2)][64]
  const int oct = threadIdx.x & 7, tl = threadIdx.x >> 3;  // 8 octets x 32 token lanes
  const int img = blockIdx.x / groups_per_image, grp = blockIdx.x % groups_per_image;
  const int r0 = blockIdx.y * band_rows;  // first output row of the band
  const int r1 = min(r0 + band_rows, h);
  const int L = h * w, pw = w + 2;
  const bool ch_ok = grp * kStencilGroup + oct * 8 < cgroup;  // channel tail of the last group
  const size_t base = (size_t)img * L * stride + (size_t)grp * kStencilGroup + oct * 8;
  // ---- this thread's 8 x 9 weights: 72 consecutive floats, fetched (as 16-byte loads) ahead of the staging loop
  // so that their latency runs under it ----
  const int wch = (blockIdx.x / groups_per_image % wmod) * cgroup + grp * kStencilGroup + oct * 8;  // first weight channel
  float wreg[8][9];
  float breg[8];
  if (ch_ok) {
    float* wflat = &wreg[0][0];
#pragma unroll
    for (int i = 0; i < 18; ++i) {
      const f32x4_t v = *reinterpret_cast<const f32x4_t*>(wt + (size_t)wch * 9 + 4 * i);
#pragma unroll
      for (int e = 0; e < 4; ++e) wflat[4 * i + e] = v[e];
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) breg[j] = (!GATE && bias) ? bias[wch + j] : 0.f;
  }
  // ---- stage padded cells (pr, pc) <-> grid (r0 - 1 + pr, pc - 1) ----
  // kBatch cells per thread are in flight at a time: the loads of a batch are issued before the first LDS store waits
  constexpr int kBatch = sizeof(T) == 2 ? 8 : 4;
  const int ncell = (r1 - r0 + 2) * pw;
  for (int t0 = tl; t0 < ncell; t0 += 32 * kBatch) {
    Raw8<T> cell[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int t = t0 + 32 * u;
      const int pr = t / pw, pc = t - pr * pw;
      const int r = r0 - 1 + pr, c = pc - 1;
      cell[u].zero();
      if (t < ncell && ch_ok && r >= 0 && r < h && c >= 0 && c < w)
        cell[u].load(x + base + (size_t)(r * w + c) * stride);
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int t = t0 + 32 * u;
      if (t < ncell) cell[u].store(tile + t * kStencilGroup + oct * 8);
    }
  }
  __syncthreads();
  if (!ch_ok) return;
  const int nout = (r1 - r0) * w;
  for (int t = tl; t < nout; t += 32) {
    const int rl = t / w, c = t - rl * w;
    const T* p = tile + (rl * pw + c) * kStencilGroup + oct * 8;  // padded cell of tap (-1, -1)
    float acc[8], ctr[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = breg[j], ctr[j] = 0.f;
#pragma unroll
    for (int di = 0; di < 3; ++di) {
#pragma unroll
      for (int dj = 0; dj < 3; ++dj) {
        float xv[8];
        Vec8<T>::load(p + (di * pw + dj) * kStencilGroup, xv);
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] = __builtin_fmaf(xv[j], wreg[j][di * 3 + dj], acc[j]);
        if (GATE && di == 1 && dj == 1) {
#pragma unroll
          for (int j = 0; j < 8; ++j) ctr[j] = xv[j];
        }
      }
    }
    if (GATE) {
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] = ctr[j] * sigmoidf_(acc[j]);
    } else if (silu) {
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] = acc[j] * sigmoidf_(acc[j]);
    }
    Vec8<T>::store(y + base + (size_t)((r0 + rl) * w + c) * stride, acc);
  }
}

template <typename T, bool GATE>
static int launch_stencil(const void* x, const float* wt, const float* bias, void* y, int images, int h, int w,
                          int stride, int wmod, int cgroup, int silu, hipStream_t stream) {
  // rows per band so that (band + 2) x (w + 2) padded cells x 64 channels fit 48 KB of LDS
  const int row_bytes = (w + 2) * kStencilGroup * (int)sizeof(T);
  int band = 48 * 1024 / row_bytes - 2;
  if (band < 1) return -95;
  if (band > h) band = h;
  const int nband = (h + band - 1) / band;
  const int groups = (cgroup + kStencilGroup - 1) / kStencilGroup;
  const size_t lds = (size_t)(band + 2) * row_bytes;
  hipLaunchKernelGGL((stencil3x3_kernel<T, GATE>), dim3(images * groups, nband), dim3(256), lds, stream, (const T*)x, wt,
                     bias, (T*)y, h, w, stride, groups, wmod, cgroup, band, silu);
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

int launch_dwconv3x3(const void* x, const float* wt, const float* bias, void* y, int B, int h, int w, int C,
                     int silu, int io_dtype, hipStream_t stream) {
  // every batch element is an image of C channels; all images share the C weight channels
  if (io_dtype == 0) return launch_stencil<float, false>(x, wt, bias, y, B, h, w, C, 1, C, silu, stream);
  return launch_stencil<uint16_t, false>(x, wt, bias, y, B, h, w, C, 1, C, silu, stream);
}

int launch_locality_gate(const void* o, const float* wt, void* y, int B, int H, int h, int w, int Dv, int io_dtype,
                         hipStream_t stream) {
  if (Dv > 64) return -95;
  // every (batch, head) slab is an "image" of Dv channels; head hd uses weight channels [hd*Dv, hd*Dv + Dv)
  if (io_dtype == 0) return launch_stencil<float, true>(o, wt, nullptr, y, B * H, h, w, Dv, H, Dv, 0, stream);
  return launch_stencil<uint16_t, true>(o, wt, nullptr, y, B * H, h, w, Dv, H, Dv, 0, stream);
}

// ---------------------------------------------------------------------------
// RMS-norm blend epilogue.  One group of Dv/8 lanes owns one (b, l, head) row of
// Dv values; the two mean-squares are reduced with lane shuffles inside the group.
//   y[b,l,hd*Dv+d] = rms(o[b,hd,l,:])*w_g*s + rms(local[b,l,hd,:])*w_l*(1-s)
// One workgroup owns 32 consecutive tokens of one batch element; a thread keeps one channel octet (head, d8) for
// all its tokens, so the layout arithmetic and the norm weights are set up once per thread.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void locality_blend_kernel(const T* __restrict__ o, const T* __restrict__ loc,
                                                              const T* __restrict__ glin,
                                                              const float* __restrict__ wg,
                                                              const float* __restrict__ wl, T* __restrict__ y,
                                                              int H, int L, int Dv, long long ldg, float eps,
                                                              int silu_out) {
  const int d8n = Dv >> 3;  // lanes per row: 4 (Dv=32) or 8 (Dv=64); divides 64, so groups never straddle a wave
  const int nv = H * d8n;   // channel octets per token row
  const int b = blockIdx.y;
  const int l0 = blockIdx.x * 32;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const float inv_dv = 1.0f / (float)Dv;
  for (int cv0 = 0; cv0 < nv; cv0 += 64) {
    const int cv = cv0 + tx;
    const bool has = cv < nv;  // lanes past the row still take part in the shuffles of their (inactive) group
    const int cvc = has ? cv : 0;
    const int hd = cvc / d8n, d8 = cvc - hd * d8n;
    float w_g[8], w_l[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) w_g[j] = wg[d8 * 8 + j], w_l[j] = wl[d8 * 8 + j];
    const T* po = o + (((size_t)b * H + hd) * L) * (size_t)Dv + d8 * 8;
    const size_t row0 = ((size_t)b * L) * (size_t)(nv * 8) + (size_t)cvc * 8;
    const T* pg = glin + ((size_t)b * L) * (size_t)ldg + (size_t)cvc * 8;  // g_lin rows are ldg elements apart
    for (int t = ty; t < 32; t += 4) {
      const int l = l0 + t;
      if (l >= L) break;  // uniform over the wave: a wave shares its token
      float xo[8], xl[8], xg[8];
      const size_t tok = row0 + (size_t)l * (nv * 8);
      Vec8<T>::load(po + (size_t)l * Dv, xo);
      Vec8<T>::load(loc + tok, xl);
      Vec8<T>::load(pg + (size_t)l * ldg, xg);
      float so = 0.f, sl = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) so += xo[j] * xo[j], sl += xl[j] * xl[j];
      for (int m = 1; m < d8n; m <<= 1) {
        so += __shfl_xor(so, m);
        sl += __shfl_xor(sl, m);
      }
      const float ro = rsqrtf(so * inv_dv + eps);
      const float rl = rsqrtf(sl * inv_dv + eps);
      float out[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float s = sigmoidf_(xg[j]);
        float v = xo[j] * ro * w_g[j] * s + xl[j] * rl * w_l[j] * (1.f - s);
        if (silu_out) v = v * sigmoidf_(v);
        out[j] = v;
      }
      if (has) Vec8<T>::store(y + tok, out);
    }
  }
}

int launch_locality_blend(const void* o, const void* loc, const void* glin, const float* wg, const float* wl, void* y,
                          int B, int H, int L, int Dv, long long ldg, float eps, int silu_out, int io_dtype,
                          hipStream_t stream) {
  if (B > 65535) return -22;
  const dim3 grid((L + 31) / 32, B), block(256);
  if (io_dtype == 0)
    hipLaunchKernelGGL((locality_blend_kernel<float>), grid, block, 0, stream, (const float*)o, (const float*)loc,
                       (const float*)glin, wg, wl, (float*)y, H, L, Dv, ldg, eps, silu_out);
  else
    hipLaunchKernelGGL((locality_blend_kernel<uint16_t>), grid, block, 0, stream, (const uint16_t*)o,
                       (const uint16_t*)loc, (const uint16_t*)glin, wg, wl, (uint16_t*)y, H, L, Dv, ldg, eps, silu_out);
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

// ---------------------------------------------------------------------------
// Weight and bias gradients of the depthwise 3x3 convolution on token-major rows x, dy [B, h*w, C]:
//   dw[c, ky, kx] = sum over b, y, x of dy[b, y, x, c] * x[b, y+ky-1, x+kx-1, c]   (zero padding),  db[c] = sum dy
// A thread keeps one channel octet and walks every fourth token of its workgroup's share of one image with 9 * 8 + 8
// sums in registers (the nine neighbour rows come from cache: every row is read by its nine neighbours); the four
// token lanes combine through LDS in a fixed order and the workgroup leaves one row of `partials`
// [workgroups, 10 * C] (columns c*9 + tap, then 9*C + c for the bias), which a column sum finishes.
// ---------------------------------------------------------------------------
constexpr int kWgradSplit = 4;  // workgroups per image

template <typename T>
__global__ __launch_bounds__(256) void dwconv3x3_wgrad_kernel(const T* __restrict__ x, const T* __restrict__ dy,
                                                              float* __restrict__ partials, int h, int w, int C,
                                                              int tiles_per_wg) {
  __shared__ float red[64][81];
  const int L = h * w, nv = C >> 3;
  const int b = blockIdx.y;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int ntiles = (L + 31) / 32;
  const int tile0 = blockIdx.x * tiles_per_wg;
  const int tile1 = tile0 + tiles_per_wg < ntiles ? tile0 + tiles_per_wg : ntiles;
  float* prow = partials + ((size_t)b * gridDim.x + blockIdx.x) * ((size_t)C * 10);
  for (int cv0 = 0; cv0 < nv; cv0 += 64) {
    const int cv = cv0 + tx;
    const bool has = cv < nv;
    float acc[10][8];
#pragma unroll
    for (int k = 0; k < 10; ++k)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[k][j] = 0.f;
    if (has) {
      const T* px = x + (size_t)b * L * C + (size_t)cv * 8;
      const T* pd = dy + (size_t)b * L * C + (size_t)cv * 8;
      for (int tile = tile0; tile < tile1; ++tile) {
        for (int t = ty; t < 32; t += 4) {
          const int l = tile * 32 + t;
          if (l >= L) break;
          const int yy = l / w, xx = l - yy * w;
          float g[8];
          Vec8<T>::load(pd + (size_t)l * C, g);
#pragma unroll
          for (int j = 0; j < 8; ++j) acc[9][j] += g[j];
#pragma unroll
          for (int ky = 0; ky < 3; ++ky) {
#pragma unroll
            for (int kx = 0; kx < 3; ++kx) {
              const int y2 = yy + ky - 1, x2 = xx + kx - 1;
              if (y2 >= 0 && y2 < h && x2 >= 0 && x2 < w) {
                float v[8];
                Vec8<T>::load(px + (size_t)(y2 * w + x2) * C, v);
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[ky * 3 + kx][j] = __builtin_fmaf(g[j], v[j], acc[ky * 3 + kx][j]);
              }
            }
          }
        }
      }
    }
    for (int r = 0; r < 4; ++r) {  // the four token lanes add in turn
      if (ty == r) {
#pragma unroll
        for (int k = 0; k < 10; ++k)
#pragma unroll
          for (int j = 0; j < 8; ++j) red[tx][k * 8 + j] = (r == 0 ? 0.f : red[tx][k * 8 + j]) + acc[k][j];
      }
      __syncthreads();
    }
    if (has) {
      for (int k = ty * 20; k < ty * 20 + 20; ++k) {
        const int tap = k >> 3, j = k & 7;
        const size_t col = tap < 9 ? ((size_t)cv * 8 + j) * 9 + tap : (size_t)C * 9 + (size_t)cv * 8 + j;
        prow[col] = red[tx][k];
      }
    }
    __syncthreads();
  }
}

int launch_column_sum(const float* partials, float* out, int n, int C, hipStream_t stream);

size_t dwconv3x3_wgrad_workspace(int B, int C) { return (size_t)B * kWgradSplit * C * 10 * sizeof(float); }

int launch_dwconv3x3_wgrad(const void* x, const void* dy, float* dw_db, void* workspace, int B, int h, int w, int C,
                           int io_dtype, hipStream_t stream) {
  if (B > 65535 || C % 8 != 0 || (long long)h * w > 0x7fffffffLL - 64 || (long long)C * 10 > 0x7fffffffLL) return -22;
  const int ntiles = (h * w + 31) / 32;
  const int split = ntiles < kWgradSplit ? ntiles : kWgradSplit;
  const int tiles_per_wg = (ntiles + split - 1) / split;
  const dim3 grid(split, B), block(256);
  float* partials = static_cast<float*>(workspace);
  if (io_dtype == 0)
    hipLaunchKernelGGL((dwconv3x3_wgrad_kernel<float>), grid, block, 0, stream, (const float*)x, (const float*)dy,
                       partials, h, w, C, tiles_per_wg);
  else
    hipLaunchKernelGGL((dwconv3x3_wgrad_kernel<uint16_t>), grid, block, 0, stream, (const uint16_t*)x,
                       (const uint16_t*)dy, partials, h, w, C, tiles_per_wg);
  if (hipGetLastError() != hipSuccess) return -5;
  return launch_column_sum(partials, dw_db, split * B, C * 10, stream);
}

// ---------------------------------------------------------------------------
// Backward of the RMS-norm blend epilogue, same thread layout as the forward.  With s = sig(g_lin),
// on = rms(o) * w_g, ln = rms(local) * w_l, y0 = on * s + ln * (1 - s), y = silu_out ? y0 * sig(y0) : y0:
//   dy0 = dy * d(y)/d(y0),  d_on = dy0 * s,  d_ln = dy0 * (1 - s),  d_glin = dy0 * (on - ln) * s * (1 - s),
//   d_o = rms_backward(o, w_g, d_on),  d_local = rms_backward(local, w_l, d_ln)   (per (token, head) row of Dv),
//   dw_g[d] = sum d_on * o * r_o,  dw_l[d] = sum d_ln * local * r_l   over batch, tokens and heads.
// The weight gradients leave as one row of `partials` [workgroups, 2 * Dv] per workgroup (threads park their sums in
// LDS and 2 * Dv threads add the ones of their channel, in a fixed order), which a column sum finishes.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void locality_blend_bwd_kernel(
    const T* __restrict__ o, const T* __restrict__ loc, const T* __restrict__ glin, const float* __restrict__ wg,
    const float* __restrict__ wl, const T* __restrict__ dy, T* __restrict__ d_o, T* __restrict__ d_loc,
    T* __restrict__ d_glin, float* __restrict__ partials, int H, int L, int Dv, long long ldg, float eps,
    int silu_out) {
  __shared__ float park[256][17];  // per thread: 8 dw_g + 8 dw_l sums of its channel octet (17: bank spread)
  const int d8n = Dv >> 3;
  const int nv = H * d8n;
  const int b = blockIdx.y;
  const int l0 = blockIdx.x * 32;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const float inv_dv = 1.0f / (float)Dv;
  float total = 0.f;  // threads 0 .. 2*Dv-1: their channel's weight-gradient sum over the whole workgroup
  for (int cv0 = 0; cv0 < nv; cv0 += 64) {
    const int cv = cv0 + tx;
    const bool has = cv < nv;
    const int cvc = has ? cv : 0;
    const int hd = cvc / d8n, d8 = cvc - hd * d8n;
    float w_g[8], w_l[8], dwg[8], dwl[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) w_g[j] = wg[d8 * 8 + j], w_l[j] = wl[d8 * 8 + j], dwg[j] = 0.f, dwl[j] = 0.f;
    const size_t head_off = (((size_t)b * H + hd) * L) * (size_t)Dv + d8 * 8;
    const size_t row0 = ((size_t)b * L) * (size_t)(nv * 8) + (size_t)cvc * 8;
    const T* pg = glin + ((size_t)b * L) * (size_t)ldg + (size_t)cvc * 8;
    for (int t = ty; t < 32; t += 4) {
      const int l = l0 + t;
      if (l >= L) break;  // uniform over the wave
      float xo[8], xl[8], xg[8], g[8];
      const size_t tok = row0 + (size_t)l * (nv * 8);
      Vec8<T>::load(o + head_off + (size_t)l * Dv, xo);
      Vec8<T>::load(loc + tok, xl);
      Vec8<T>::load(pg + (size_t)l * ldg, xg);
      Vec8<T>::load(dy + tok, g);
      float so = 0.f, sl = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) so += xo[j] * xo[j], sl += xl[j] * xl[j];
      for (int m = 1; m < d8n; m <<= 1) {
        so += __shfl_xor(so, m);
        sl += __shfl_xor(sl, m);
      }
      const float ro = rsqrtf(so * inv_dv + eps);
      const float rl = rsqrtf(sl * inv_dv + eps);
      float don[8], dln[8], dgl[8];
      float mo = 0.f, ml = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float s = sigmoidf_(xg[j]);
        const float on = xo[j] * ro * w_g[j], ln = xl[j] * rl * w_l[j];
        float dy0 = g[j];
        if (silu_out) {
          const float y0 = on * s + ln * (1.f - s);
          const float sy = sigmoidf_(y0);
          dy0 *= sy * (1.f + y0 * (1.f - sy));
        }
        don[j] = dy0 * s;
        dln[j] = dy0 * (1.f - s);
        dgl[j] = dy0 * (on - ln) * s * (1.f - s);
        mo = __builtin_fmaf(don[j] * w_g[j], xo[j], mo);
        ml = __builtin_fmaf(dln[j] * w_l[j], xl[j], ml);
      }
      for (int m = 1; m < d8n; m <<= 1) {
        mo += __shfl_xor(mo, m);
        ml += __shfl_xor(ml, m);
      }
      const float co = ro * ro * mo * inv_dv, cl = rl * rl * ml * inv_dv;
      float eo[8], el[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        eo[j] = ro * (don[j] * w_g[j] - xo[j] * co);
        el[j] = rl * (dln[j] * w_l[j] - xl[j] * cl);
        if (has) {
          dwg[j] = __builtin_fmaf(don[j] * ro, xo[j], dwg[j]);
          dwl[j] = __builtin_fmaf(dln[j] * rl, xl[j], dwl[j]);
        }
      }
      if (has) {
        Vec8<T>::store(d_o + head_off + (size_t)l * Dv, eo);
        Vec8<T>::store(d_loc + tok, el);
        Vec8<T>::store(d_glin + tok, dgl);
      }
    }
    // combine the threads of one channel: thread (which, d) adds, in thread order, the parked sums of every thread
    // whose octet holds channel d
    __syncthreads();  // the previous round's readers are done
#pragma unroll
    for (int j = 0; j < 8; ++j) park[threadIdx.x][j] = dwg[j], park[threadIdx.x][8 + j] = dwl[j];
    __syncthreads();
    if (threadIdx.x < 2 * Dv) {
      const int which = threadIdx.x / Dv, d = threadIdx.x - which * Dv;
      const int want = d >> 3, slot = 8 * which + (d & 7);
      // octet index of thread t in this round: ((cv0 + (t & 63)) % d8n), cv0 a multiple of 64 and d8n dividing 64
      for (int t = want; t < 256; t += d8n) total += park[t][slot];
    }
  }
  if (threadIdx.x < 2 * Dv)
    partials[((size_t)blockIdx.y * gridDim.x + blockIdx.x) * (size_t)(2 * Dv) + threadIdx.x] = total;
}

size_t locality_blend_bwd_workspace(int B, int L, int Dv) {
  return (size_t)B * ((L + 31) / 32) * 2 * Dv * sizeof(float);
}

int launch_locality_blend_bwd(const void* o, const void* loc, const void* glin, const float* wg, const float* wl,
                              const void* dy, void* d_o, void* d_loc, void* d_glin, float* dw, void* workspace, int B,
                              int H, int L, int Dv, long long ldg, float eps, int silu_out, int io_dtype,
                              hipStream_t stream) {
  if (B > 65535 || (long long)B * ((L + 31) / 32) > 0x7fffffffLL) return -22;
  const dim3 grid((L + 31) / 32, B), block(256);
  float* partials = static_cast<float*>(workspace);
  if (io_dtype == 0)
    hipLaunchKernelGGL((locality_blend_bwd_kernel<float>), grid, block, 0, stream, (const float*)o, (const float*)loc,
                       (const float*)glin, wg, wl, (const float*)dy, (float*)d_o, (float*)d_loc, (float*)d_glin,
                       partials, H, L, Dv, ldg, eps, silu_out);
  else
    hipLaunchKernelGGL((locality_blend_bwd_kernel<uint16_t>), grid, block, 0, stream, (const uint16_t*)o,
                       (const uint16_t*)loc, (const uint16_t*)glin, wg, wl, (const uint16_t*)dy, (uint16_t*)d_o,
                       (uint16_t*)d_loc, (uint16_t*)d_glin, partials, H, L, Dv, ldg, eps, silu_out);
  if (hipGetLastError() != hipSuccess) return -5;
  return launch_column_sum(partials, dw, (int)(grid.x * grid.y), 2 * Dv, stream);
}

}  // namespace vig
