// Shared device helpers for the gfx950 GLA kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vig {

typedef __bf16 bf16_t;
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// bf16 <-> f32 through the native type: hipcc lowers the narrowing conversion to
// the round-to-nearest-even hardware convert of gfx950.
__device__ __forceinline__ float bf16_to_f32(uint16_t b) {
  return __uint_as_float(((uint32_t)b) << 16);
}
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  bf16_t h = (bf16_t)f;
  return __builtin_bit_cast(uint16_t, h);
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  f32x2_t x = {lo, hi};
  bf16x2_t y = __builtin_convertvector(x, bf16x2_t);
  return __builtin_bit_cast(uint32_t, y);
}
__device__ __forceinline__ float bf16lo_to_f32(uint32_t p) { return __uint_as_float(p << 16); }
__device__ __forceinline__ float bf16hi_to_f32(uint32_t p) { return __uint_as_float(p & 0xffff0000u); }

// eight channels as stored (no conversion): what a kernel that only moves them keeps in registers
template <typename T> struct Raw8;
template <> struct Raw8<uint16_t> {
  u32x4_t a;
  __device__ __forceinline__ void zero() { a = u32x4_t{0u, 0u, 0u, 0u}; }
  __device__ __forceinline__ void load(const uint16_t* p) { a = *reinterpret_cast<const u32x4_t*>(p); }
  __device__ __forceinline__ void store(uint16_t* p) const { *reinterpret_cast<u32x4_t*>(p) = a; }
  __device__ __forceinline__ void unpack(float (&x)[8]) const {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[2 * i] = bf16lo_to_f32(a[i]);
      x[2 * i + 1] = bf16hi_to_f32(a[i]);
    }
  }
};
template <> struct Raw8<float> {
  f32x4_t a, b;
  __device__ __forceinline__ void zero() { a = b = f32x4_t{0.f, 0.f, 0.f, 0.f}; }
  __device__ __forceinline__ void load(const float* p) {
    a = *reinterpret_cast<const f32x4_t*>(p);
    b = *reinterpret_cast<const f32x4_t*>(p + 4);
  }
  __device__ __forceinline__ void store(float* p) const {
    *reinterpret_cast<f32x4_t*>(p) = a;
    *reinterpret_cast<f32x4_t*>(p + 4) = b;
  }
  __device__ __forceinline__ void unpack(float (&x)[8]) const {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[i] = a[i];
      x[4 + i] = b[i];
    }
  }
};

// Typed element access used by the dtype-generic (non-MFMA) kernels.
template <typename T> struct Elem;
template <> struct Elem<float> {
  static __device__ __forceinline__ float load(const float* p) { return *p; }
  static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
};
template <> struct Elem<uint16_t> {  // bf16 storage
  static __device__ __forceinline__ float load(const uint16_t* p) { return bf16_to_f32(*p); }
  static __device__ __forceinline__ void store(uint16_t* p, float v) { *p = f32_to_bf16(v); }
};

// (hardware reciprocal, 1 ulp: a full-precision division costs ten instructions more per value)
// e^-|..| style arguments only need the bare hardware instructions (2^x and log2 x, 1 ulp): results below the
// normal range flush to zero, which is exact enough next to 1, and the guards the library versions wrap around them
// (range tests, rescaling) cost more than the instructions themselves.
__device__ __forceinline__ float exp_fast(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }
__device__ __forceinline__ float sigmoidf_(float x) { return __builtin_amdgcn_rcpf(1.0f + exp_fast(-x)); }
// log(sigmoid(x)) = min(x, 0) - log(1 + e^-|x|); the log's argument lies in [1, 2]
__device__ __forceinline__ float logsigmoidf_(float x) {
  return fminf(x, 0.f) - 0.6931471805599453f * __builtin_amdgcn_logf(1.f + exp_fast(-fabsf(x)));
}

}  // namespace vig
