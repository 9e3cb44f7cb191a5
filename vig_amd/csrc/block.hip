// Row-wise kernels of the ViG block around the GLA op: residual-add + RMS norm, the head-major split of the
// fused q/k/v projection and the SwiGLU product.  All are HBM-bound: every element is read once and written once
// with 16-byte accesses, arithmetic in fp32.
#include <type_traits>

#include "common.h"
#include "launch.h"

namespace vig {

namespace {

// eight consecutive channels, one 16-byte transaction for bf16 and two for f32
template <typename T> struct Oct;
template <> struct Oct<uint16_t> {
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
  static __device__ __forceinline__ float round(float v) { return bf16_to_f32(f32_to_bf16(v)); }
};
template <> struct Oct<float> {
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
  static __device__ __forceinline__ float round(float v) { return v; }
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

}  // namespace

// ---------------------------------------------------------------------------
// residual-add + RMS norm, one wave per row of C channels (C % 8 == 0, C <= 64 * 8 * NV):
//   s = x (+ residual), in fp32;  residual_out = s;  y = s * rsqrt(mean(s^2) + eps) * weight
// round_sum: s is first rounded to the storage type (the value an explicit add would have stored) and the
// rounded value is normalised.
// ---------------------------------------------------------------------------
template <typename T, int NV>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const T* __restrict__ x, const T* __restrict__ residual,
                                                      const float* __restrict__ weight, T* __restrict__ y,
                                                      T* __restrict__ residual_out, int rows, int C, float eps,
                                                      int round_sum) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int nvec = C >> 3;
  const size_t base = (size_t)row * C;
  float s[NV][8];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = lane + 64 * i;
    if (v < nvec) {
      Oct<T>::load(x + base + 8 * v, s[i]);
      if (residual) {
        float rr[8];
        Oct<T>::load(residual + base + 8 * v, rr);
#pragma unroll
        for (int j = 0; j < 8; ++j) s[i][j] += rr[j];
      }
      if (round_sum) {
#pragma unroll
        for (int j = 0; j < 8; ++j) s[i][j] = Oct<T>::round(s[i][j]);
      }
      if (residual_out) Oct<T>::store(residual_out + base + 8 * v, s[i]);
#pragma unroll
      for (int j = 0; j < 8; ++j) ss = __builtin_fmaf(s[i][j], s[i][j], ss);
    }
  }
  ss = wave_sum(ss);
  const float rstd = 1.0f / sqrtf(ss / (float)C + eps);
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = lane + 64 * i;
    if (v < nvec) {
      float w[8];
      Oct<float>::load(weight + 8 * v, w);
#pragma unroll
      for (int j = 0; j < 8; ++j) s[i][j] = s[i][j] * rstd * w[j];
      Oct<T>::store(y + base + 8 * v, s[i]);
    }
  }
}

template <typename T>
static int launch_rmsnorm_t(const void* x, const void* residual, const float* weight, void* y, void* residual_out,
                            int rows, int C, float eps, int round_sum, hipStream_t stream) {
  const dim3 grid((rows + 3) / 4), block(256);
  const int nvec = C / 8;
#define VIG_RMS_CASE(NV)                                                                                          \
  hipLaunchKernelGGL((rmsnorm_kernel<T, NV>), grid, block, 0, stream, (const T*)x, (const T*)residual, weight, \
                     (T*)y, (T*)residual_out, rows, C, eps, round_sum)
  if (nvec <= 64) VIG_RMS_CASE(1);
  else if (nvec <= 128) VIG_RMS_CASE(2);
  else if (nvec <= 256) VIG_RMS_CASE(4);
  else VIG_RMS_CASE(8);
#undef VIG_RMS_CASE
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

int launch_rmsnorm(const void* x, const void* residual, const float* weight, void* y, void* residual_out, int rows,
                   int C, float eps, int round_sum, int io_dtype, hipStream_t stream) {
  if (C % 8 != 0 || C > 4096) return -95;
  return io_dtype == 1 ? launch_rmsnorm_t<uint16_t>(x, residual, weight, y, residual_out, rows, C, eps, round_sum, stream)
                       : launch_rmsnorm_t<float>(x, residual, weight, y, residual_out, rows, C, eps, round_sum, stream);
}

// ---------------------------------------------------------------------------
// LayerNorm over the last dimension with an optional SiLU behind it (the norms of the patch embedding, applied to
// channels-last feature maps):  y = (x - mean) * rsqrt(var + eps) * weight + bias, var the biased variance; with
// silu the normalised value is first rounded to the storage type (the separate activation reads stored values).
// Two neighbours ride along: pre_bias [C] is added to x first (the bias of the convolution in front, the sum rounded
// to the storage type as that convolution would have stored it), and post_add [post_rows, C] is added to the result
// of row r at its row r % post_rows (the position table behind the last norm; the normalised value is rounded to
// the storage type first, as the separate add reads it).
// GROUP lanes own one row (GROUP = 32 for C <= 256: two rows per wave keep the lanes busy at small C), each lane
// holds NV channel octets; mean and variance are two reductions over registers, as torch computes them.
// ---------------------------------------------------------------------------
template <int GROUP>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
  for (int off = GROUP / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

template <typename T, int NV, int GROUP>
__global__ __launch_bounds__(256) void layernorm_kernel(const T* __restrict__ x, const float* __restrict__ weight,
                                                        const float* __restrict__ bias, T* __restrict__ y,
                                                        long long rows, int C, float eps, int silu,
                                                        const float* __restrict__ pre_bias,
                                                        const T* __restrict__ post_add, int post_rows) {
  constexpr int kRowsPerBlock = 256 / GROUP;
  const int gl = threadIdx.x % GROUP;
  const long long row = (long long)blockIdx.x * kRowsPerBlock + threadIdx.x / GROUP;
  const bool row_ok = row < rows;  // lanes of a missing row still take part in the shuffles of their wave
  const int nvec = C >> 3;
  const size_t base = (size_t)(row_ok ? row : 0) * C;
  float s[NV][8];
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = gl + GROUP * i;
    if (v < nvec) {
      Oct<T>::load(x + base + 8 * v, s[i]);
      if (pre_bias) {
        float pb[8];
        Oct<float>::load(pre_bias + 8 * v, pb);
#pragma unroll
        for (int j = 0; j < 8; ++j) s[i][j] = Oct<T>::round(s[i][j] + pb[j]);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) sum += s[i][j];
    }
  }
  const float mean = group_sum<GROUP>(sum) / (float)C;
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = gl + GROUP * i;
    if (v < nvec) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        s[i][j] -= mean;
        ss = __builtin_fmaf(s[i][j], s[i][j], ss);
      }
    }
  }
  const float rstd = 1.0f / sqrtf(group_sum<GROUP>(ss) / (float)C + eps);
  if (!row_ok) return;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = gl + GROUP * i;
    if (v < nvec) {
      float w[8], b[8];
      Oct<float>::load(weight + 8 * v, w);
      Oct<float>::load(bias + 8 * v, b);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float r = __builtin_fmaf(s[i][j] * rstd, w[j], b[j]);
        if (silu) {
          r = Oct<T>::round(r);
          r = r * sigmoidf_(r);
        }
        s[i][j] = r;
      }
      if (post_add) {
        float pa[8];
        Oct<T>::load(post_add + (size_t)(row % post_rows) * C + 8 * v, pa);
#pragma unroll
        for (int j = 0; j < 8; ++j) s[i][j] = Oct<T>::round(s[i][j]) + pa[j];
      }
      Oct<T>::store(y + base + 8 * v, s[i]);
    }
  }
}

template <typename T>
static int launch_layernorm_t(const void* x, const float* weight, const float* bias, void* y, long long rows, int C,
                              float eps, int silu, const float* pre_bias, const void* post_add, int post_rows,
                              hipStream_t stream) {
  const int nvec = C / 8;
#define VIG_LN_CASE(NV, GROUP)                                                                                       \
  hipLaunchKernelGGL((layernorm_kernel<T, NV, GROUP>), dim3((unsigned)((rows + 256 / GROUP - 1) / (256 / GROUP))), \
                     dim3(256), 0, stream, (const T*)x, weight, bias, (T*)y, rows, C, eps, silu, pre_bias,      \
                     (const T*)post_add, post_rows)
  if (nvec <= 32) VIG_LN_CASE(1, 32);
  else if (nvec <= 64) VIG_LN_CASE(1, 64);
  else if (nvec <= 128) VIG_LN_CASE(2, 64);
  else if (nvec <= 256) VIG_LN_CASE(4, 64);
  else VIG_LN_CASE(8, 64);
#undef VIG_LN_CASE
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

int launch_layernorm(const void* x, const float* weight, const float* bias, void* y, long long rows, int C, float eps,
                     int silu, const float* pre_bias, const void* post_add, int post_rows, int io_dtype,
                     hipStream_t stream) {
  if (C % 8 != 0 || C > 4096 || (rows + 3) / 4 > 0x7fffffffLL) return -95;
  return io_dtype == 1
             ? launch_layernorm_t<uint16_t>(x, weight, bias, y, rows, C, eps, silu, pre_bias, post_add, post_rows, stream)
             : launch_layernorm_t<float>(x, weight, bias, y, rows, C, eps, silu, pre_bias, post_add, post_rows, stream);
}

// ---------------------------------------------------------------------------
// head-major split of the fused projection:
//   qkv [B, L, H*Dk | H*Dk | H*Dv]  ->  q, k [B, H, L, Dk],  v [B, H, L, Dv]
// A token's row may sit inside a wider row of `ld` elements (the columns of a larger projection).
// One workgroup owns 32 consecutive tokens of one batch element: whole rows are read, and every (tensor, head)
// receives a contiguous run of 32 tokens.
// ---------------------------------------------------------------------------
template <typename T, bool MERGE>  // MERGE: the backward, head-major gradients gathered into token-major rows
__global__ __launch_bounds__(256) void split_heads_kernel(typename std::conditional<MERGE, T, const T>::type* __restrict__ qkv,
                                                          typename std::conditional<MERGE, const T, T>::type* __restrict__ q,
                                                          typename std::conditional<MERGE, const T, T>::type* __restrict__ k,
                                                          typename std::conditional<MERGE, const T, T>::type* __restrict__ v,
                                                          int B, int L, int H, int Dk, int Dv, long long ld) {
  const int K = H * Dk, V = H * Dv;
  const int row = 2 * K + V;
  const int nv = row >> 3;
  const int b = blockIdx.y;
  const int l0 = blockIdx.x * 32;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int cv = tx; cv < nv; cv += 64) {
    const int ch = cv * 8;
    typename std::conditional<MERGE, const T, T>::type* head;
    int D, c;
    if (ch < K) { head = q; D = Dk; c = ch; }
    else if (ch < 2 * K) { head = k; D = Dk; c = ch - K; }
    else { head = v; D = Dv; c = ch - 2 * K; }
    const int hh = c / D, d = c - hh * D;
    auto* rows = qkv + ((size_t)b * L) * (size_t)ld + ch;
    auto* slab = head + (((size_t)b * H + hh) * L) * (size_t)D + d;
    for (int t = ty; t < 32; t += 4) {
      const int l = l0 + t;
      if (l >= L) break;
      float x[8];
      if constexpr (MERGE) {
        Oct<T>::load(slab + (size_t)l * D, x);
        Oct<T>::store(rows + (size_t)l * ld, x);
      } else {
        Oct<T>::load(rows + (size_t)l * ld, x);
        Oct<T>::store(slab + (size_t)l * D, x);
      }
    }
  }
}

int launch_split_heads(const void* qkv, void* q, void* k, void* v, int B, int L, int H, int Dk, int Dv, long long ld,
                       int io_dtype, hipStream_t stream) {
  if (Dk % 8 != 0 || Dv % 8 != 0 || B > 65535) return -95;
  const dim3 grid((L + 31) / 32, B), block(256);
  if (io_dtype == 1)
    hipLaunchKernelGGL((split_heads_kernel<uint16_t, false>), grid, block, 0, stream, (const uint16_t*)qkv,
                       (uint16_t*)q, (uint16_t*)k, (uint16_t*)v, B, L, H, Dk, Dv, ld);
  else
    hipLaunchKernelGGL((split_heads_kernel<float, false>), grid, block, 0, stream, (const float*)qkv, (float*)q,
                       (float*)k, (float*)v, B, L, H, Dk, Dv, ld);
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

// the backward of the split: dq, dk, dv (head-major) -> d_qkv [B, L, H*(2*Dk+Dv)] packed rows
int launch_merge_heads(const void* dq, const void* dk, const void* dv, void* dqkv, int B, int L, int H, int Dk, int Dv,
                       int io_dtype, hipStream_t stream) {
  if (Dk % 8 != 0 || Dv % 8 != 0 || B > 65535) return -95;
  const dim3 grid((L + 31) / 32, B), block(256);
  const long long ld = (long long)H * (2 * Dk + Dv);
  if (io_dtype == 1)
    hipLaunchKernelGGL((split_heads_kernel<uint16_t, true>), grid, block, 0, stream, (uint16_t*)dqkv,
                       (const uint16_t*)dq, (const uint16_t*)dk, (const uint16_t*)dv, B, L, H, Dk, Dv, ld);
  else
    hipLaunchKernelGGL((split_heads_kernel<float, true>), grid, block, 0, stream, (float*)dqkv, (const float*)dq,
                       (const float*)dk, (const float*)dv, B, L, H, Dk, Dv, ld);
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

// ---------------------------------------------------------------------------
// SwiGLU product:  in [rows, 2*I] = (gate | up)  ->  out [rows, I] = gate * up / (1 + exp(-gate))
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void swiglu_kernel(const T* __restrict__ in, T* __restrict__ out, long long nvec,
                                                     int I8) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= nvec) return;
  const long long row = i / I8;
  const int c = (int)(i - row * I8) * 8;
  const size_t I = (size_t)I8 * 8;
  float g[8], u[8];
  Oct<T>::load(in + (size_t)row * 2 * I + c, g);
  Oct<T>::load(in + (size_t)row * 2 * I + I + c, u);
#pragma unroll
  for (int j = 0; j < 8; ++j) g[j] = g[j] * u[j] * sigmoidf_(g[j]);
  Oct<T>::store(out + (size_t)row * I + c, g);
}

int launch_swiglu(const void* in, void* out, long long rows, int I, int io_dtype, hipStream_t stream) {
  if (I % 8 != 0) return -95;
  const long long nvec = rows * (I / 8);
  const dim3 grid((unsigned)((nvec + 255) / 256)), block(256);
  if (io_dtype == 1)
    hipLaunchKernelGGL(swiglu_kernel<uint16_t>, grid, block, 0, stream, (const uint16_t*)in, (uint16_t*)out, nvec, I / 8);
  else
    hipLaunchKernelGGL(swiglu_kernel<float>, grid, block, 0, stream, (const float*)in, (float*)out, nvec, I / 8);
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

// ---------------------------------------------------------------------------
// Backward of the SwiGLU product:  d_gate = dy * up * sig(gate) * (1 + gate * (1 - sig(gate))),
// d_up = dy * gate * sig(gate), written as d_gate_up [rows, 2*I] = (d_gate | d_up).
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const T* __restrict__ in, const T* __restrict__ dy,
                                                         T* __restrict__ din, long long nvec, int I8) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= nvec) return;
  const long long row = i / I8;
  const int c = (int)(i - row * I8) * 8;
  const size_t I = (size_t)I8 * 8;
  float g[8], u[8], d[8];
  Oct<T>::load(in + (size_t)row * 2 * I + c, g);
  Oct<T>::load(in + (size_t)row * 2 * I + I + c, u);
  Oct<T>::load(dy + (size_t)row * I + c, d);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float sg = sigmoidf_(g[j]);
    const float du = d[j] * g[j] * sg;
    g[j] = d[j] * u[j] * sg * (1.f + g[j] * (1.f - sg));
    u[j] = du;
  }
  Oct<T>::store(din + (size_t)row * 2 * I + c, g);
  Oct<T>::store(din + (size_t)row * 2 * I + I + c, u);
}

int launch_swiglu_bwd(const void* in, const void* dy, void* din, long long rows, int I, int io_dtype,
                      hipStream_t stream) {
  if (I % 8 != 0) return -95;
  const long long nvec = rows * (I / 8);
  if ((nvec + 255) / 256 > 0x7fffffffLL) return -95;
  const dim3 grid((unsigned)((nvec + 255) / 256)), block(256);
  if (io_dtype == 1)
    hipLaunchKernelGGL(swiglu_bwd_kernel<uint16_t>, grid, block, 0, stream, (const uint16_t*)in, (const uint16_t*)dy,
                       (uint16_t*)din, nvec, I / 8);
  else
    hipLaunchKernelGGL(swiglu_bwd_kernel<float>, grid, block, 0, stream, (const float*)in, (const float*)dy,
                       (float*)din, nvec, I / 8);
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

// ---------------------------------------------------------------------------
// Backward of the residual-add + RMS norm.  s is the stored sum that was normalised (x, or x + residual as the
// forward returned it), dy the gradient of y, d_sum (optional) the gradient arriving at the returned sum:
//   r = rsqrt(mean(s^2) + eps),  g = dy * weight,
//   ds = r * (g - s * r^2 * mean(g * s)) + d_sum         (the gradient of x and of the residual alike)
//   dweight[c] = sum over rows of dy[c] * s[c] * r
// One wave per row, sixteen waves a workgroup (eight a SIMD: the kernel is a chain of load -> reduce -> store per
// row, and only occupancy hides it); workgroups walk the rows a grid apart and keep their share of dweight in
// registers; the waves of a workgroup combine through LDS into one row of `partials` [gridDim.x, C], which a second
// kernel sums (no atomics: the result does not depend on the order the workgroups finish in).
// ---------------------------------------------------------------------------
constexpr int kRmsBwdWaves = 16;

template <typename T, int NV>
__global__ __launch_bounds__(64 * kRmsBwdWaves) void rmsnorm_bwd_kernel(const T* __restrict__ s_in, const float* __restrict__ weight,
                                                          const T* __restrict__ dy, const T* __restrict__ d_sum,
                                                          T* __restrict__ ds, float* __restrict__ partials, int rows,
                                                          int C, float eps) {
  extern __shared__ __align__(16) float red[];  // [kRmsBwdWaves][C], only with partials
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nvec = C >> 3;
  float w[NV][8], dw[NV][8];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = lane + 64 * i;
#pragma unroll
    for (int j = 0; j < 8; ++j) dw[i][j] = 0.f, w[i][j] = 0.f;
    if (v < nvec) Oct<float>::load(weight + 8 * v, w[i]);
  }
  const float inv_c = 1.0f / (float)C;
  for (int row = blockIdx.x * kRmsBwdWaves + wave; row < rows; row += gridDim.x * kRmsBwdWaves) {
    const size_t base = (size_t)row * C;
    float s[NV][8], g[NV][8];
    float ss = 0.f, gs = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = lane + 64 * i;
#pragma unroll
      for (int j = 0; j < 8; ++j) s[i][j] = 0.f, g[i][j] = 0.f;
      if (v < nvec) {
        Oct<T>::load(s_in + base + 8 * v, s[i]);
        Oct<T>::load(dy + base + 8 * v, g[i]);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        ss = __builtin_fmaf(s[i][j], s[i][j], ss);
        gs = __builtin_fmaf(g[i][j] * w[i][j], s[i][j], gs);
      }
    }
    ss = wave_sum(ss);
    gs = wave_sum(gs);
    const float rstd = 1.0f / sqrtf(ss * inv_c + eps);
    const float coef = rstd * rstd * gs * inv_c;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = lane + 64 * i;
      if (v < nvec) {
        float o[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          dw[i][j] = __builtin_fmaf(g[i][j] * rstd, s[i][j], dw[i][j]);
          o[j] = rstd * (g[i][j] * w[i][j] - s[i][j] * coef);
        }
        if (d_sum) {
          float e[8];
          Oct<T>::load(d_sum + base + 8 * v, e);
#pragma unroll
          for (int j = 0; j < 8; ++j) o[j] += e[j];
        }
        Oct<T>::store(ds + base + 8 * v, o);
      }
    }
  }
  if (!partials) return;  // uniform over the grid
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int v = lane + 64 * i;
    if (v < nvec) Oct<float>::store(red + wave * C + 8 * v, dw[i]);
  }
  __syncthreads();
  for (int c = threadIdx.x; c < C; c += 64 * kRmsBwdWaves) {
    float acc = 0.f;
#pragma unroll
    for (int k = 0; k < kRmsBwdWaves; ++k) acc += red[k * C + c];
    partials[(size_t)blockIdx.x * C + c] = acc;
  }
}

// out[c] = sum over the n rows of partials [n, C]: a workgroup takes 64 columns, its 16 waves a sixteenth of the rows each
__global__ __launch_bounds__(1024) void column_sum_kernel(const float* __restrict__ partials, float* __restrict__ out,
                                                          int n, int C) {
  __shared__ float red[16][64];
  const int lane = threadIdx.x & 63, slice = threadIdx.x >> 6;
  const int c = blockIdx.x * 64 + lane;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  if (c < C) {
    int i = slice;
    for (; i + 48 < n; i += 64) {
#pragma unroll
      for (int k = 0; k < 4; ++k) acc[k] += partials[(size_t)(i + 16 * k) * C + c];
    }
    for (; i < n; i += 16) acc[0] += partials[(size_t)i * C + c];
  }
  red[slice][lane] = (acc[0] + acc[1]) + (acc[2] + acc[3]);
  __syncthreads();
  if (slice == 0 && c < C) {
    float t = 0.f;
#pragma unroll
    for (int k = 0; k < 16; ++k) t += red[k][lane];
    out[c] = t;
  }
}

int launch_column_sum(const float* partials, float* out, int n, int C, hipStream_t stream) {
  hipLaunchKernelGGL(column_sum_kernel, dim3((C + 63) / 64), dim3(1024), 0, stream, partials, out, n, C);
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

static int rmsnorm_bwd_grid(long long rows) {
  const long long want = (rows + kRmsBwdWaves - 1) / kRmsBwdWaves;
  return (int)(want < 512 ? want : 512);
}

size_t rmsnorm_bwd_workspace(long long rows, int C) { return (size_t)rmsnorm_bwd_grid(rows) * C * sizeof(float); }

template <typename T>
static int launch_rmsnorm_bwd_t(const void* s, const float* weight, const void* dy, const void* d_sum, void* ds,
                                float* dweight, float* partials, int rows, int C, float eps, hipStream_t stream) {
  const int grid = rmsnorm_bwd_grid(rows);
  const size_t lds = dweight ? (size_t)kRmsBwdWaves * C * sizeof(float) : 0;
  float* part = dweight ? partials : nullptr;
  const int nvec = C / 8;
#define VIG_RMSB_CASE(NV)                                                                                     \
  hipLaunchKernelGGL((rmsnorm_bwd_kernel<T, NV>), dim3(grid), dim3(64 * kRmsBwdWaves), lds, stream, (const T*)s, \
                     weight, (const T*)dy, (const T*)d_sum, (T*)ds, part, rows, C, eps)
  if (nvec <= 64) VIG_RMSB_CASE(1);
  else VIG_RMSB_CASE(2);
#undef VIG_RMSB_CASE
  if (hipGetLastError() != hipSuccess) return -5;
  if (dweight) {
    return launch_column_sum(partials, dweight, grid, C, stream);
  }
  return 0;
}

int launch_rmsnorm_bwd(const void* s, const float* weight, const void* dy, const void* d_sum, void* ds, float* dweight,
                       void* workspace, long long rows, int C, float eps, int io_dtype, hipStream_t stream) {
  if (C % 8 != 0 || C > 1024 || rows > 0x7fffffffLL - 8192) return -95;  // 16 rows of C floats in 64 KB of LDS
  return io_dtype == 1 ? launch_rmsnorm_bwd_t<uint16_t>(s, weight, dy, d_sum, ds, dweight, (float*)workspace,
                                                        (int)rows, C, eps, stream)
                       : launch_rmsnorm_bwd_t<float>(s, weight, dy, d_sum, ds, dweight, (float*)workspace, (int)rows,
                                                     C, eps, stream);
}

// ---------------------------------------------------------------------------
// Channel padding / cropping of bf16 rows:  dst[row, c] = c < src_c ? src[row, c] : 0  for c < dst_c.
// Used to run head shapes narrower than the matrix-core kernel's (Dk 16, Dv 32) on it: zero q, k and v channels
// contribute nothing, zero log-gates mean no decay, and the surplus output channels are cropped.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void pad_channels_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst,
                                                           long long nvec, int src_c8, int dst_c8) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;  // one 16-byte piece of dst
  if (i >= nvec) return;
  const long long row = i / dst_c8;
  const int c8 = (int)(i - row * dst_c8);
  u32x4_t x = {0u, 0u, 0u, 0u};
  if (c8 < src_c8) x = *reinterpret_cast<const u32x4_t*>(src + ((size_t)row * src_c8 + c8) * 8);
  *reinterpret_cast<u32x4_t*>(dst + (size_t)i * 8) = x;
}

// Several tensors of the same row count in one launch (blockIdx.y = tensor).
constexpr int kMaxPadJobs = 6;
struct PadJobs {
  const uint16_t* src[kMaxPadJobs];
  uint16_t* dst[kMaxPadJobs];
  int src_c8[kMaxPadJobs], dst_c8[kMaxPadJobs];
};
__global__ __launch_bounds__(256) void pad_channels_multi_kernel(PadJobs jobs, long long rows) {
  const int j = blockIdx.y;
  const int dst_c8 = jobs.dst_c8[j], src_c8 = jobs.src_c8[j];
  const long long nvec = rows * dst_c8;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (long long)gridDim.x * 256) {
    const long long row = i / dst_c8;
    const int c8 = (int)(i - row * dst_c8);
    u32x4_t x = {0u, 0u, 0u, 0u};
    if (c8 < src_c8) x = *reinterpret_cast<const u32x4_t*>(jobs.src[j] + ((size_t)row * src_c8 + c8) * 8);
    *reinterpret_cast<u32x4_t*>(jobs.dst[j] + (size_t)i * 8) = x;
  }
}

int launch_pad_channels_multi(const void* const* src, void* const* dst, const int* src_c, const int* dst_c, int n,
                              long long rows, hipStream_t stream) {
  if (n < 1 || n > kMaxPadJobs || rows <= 0) return -95;
  PadJobs jobs{};
  int max_c8 = 0;
  for (int j = 0; j < n; ++j) {
    if (src_c[j] % 8 != 0 || dst_c[j] % 8 != 0) return -95;
    jobs.src[j] = (const uint16_t*)src[j];
    jobs.dst[j] = (uint16_t*)dst[j];
    jobs.src_c8[j] = src_c[j] / 8;
    jobs.dst_c8[j] = dst_c[j] / 8;
    if (jobs.dst_c8[j] > max_c8) max_c8 = jobs.dst_c8[j];
  }
  const long long nvec = rows * max_c8;
  const long long blocks = (nvec + 255) / 256;
  hipLaunchKernelGGL(pad_channels_multi_kernel, dim3((unsigned)(blocks < 65536 ? blocks : 65536), n), dim3(256), 0,
                     stream, jobs, rows);
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

int launch_pad_channels(const void* src, void* dst, long long rows, int src_c, int dst_c, hipStream_t stream) {
  if (src_c % 8 != 0 || dst_c % 8 != 0 || rows <= 0) return -95;
  const long long nvec = rows * (dst_c / 8);
  hipLaunchKernelGGL(pad_channels_kernel, dim3((unsigned)((nvec + 255) / 256)), dim3(256), 0, stream,
                     (const uint16_t*)src, (uint16_t*)dst, nvec, src_c / 8, dst_c / 8);
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

}  // namespace vig
