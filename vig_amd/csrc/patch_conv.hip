// First convolution of ViG's v2 patch embedding (classification/models/vig.py:651: kernel 9, stride 8, padding 1,
// 3 input channels) as an implicit GEMM on the matrix cores, reading the images in the [B, C, H, W] layout they
// arrive in and writing channels-last rows [B, OH, OW, Cout] -- what the LayerNorm kernel behind it consumes.
//
// One workgroup produces one output row (b, oy): OW <= 32 pixels x Cout channels.  Its input is the slab of
// Cin * KH image rows (27 for 3 channels x 9 kernel rows); each goes to LDS shifted by one element, so that input
// column ix sits at element ix + 1 and element 0 is the left padding: pixel ox then finds its 16 kernel columns
// (9 real ones, the weights of the others are zero) at elements 8*ox .. 8*ox+15, two aligned 16-byte reads.  The
// contraction runs over (channel, kernel row) steps of 16 kernel columns: one v_mfma_f32_32x32x16_bf16 per step with
// the weights (matrix rows = output channels) in registers for the life of the workgroup and the pixels as columns.
// Matrix rows are assigned channels so that a lane ends with 16 consecutive channels of one pixel (32 contiguous
// bytes).  The one-element shift costs no unaligned access: a lane takes the last element of its left neighbour's
// 16-byte chunk (a lane shuffle) and funnel-shifts its own chunk behind it.
#include "common.h"
#include "launch.h"

namespace vig {

namespace {

constexpr int kPcStride = 8;       // convolution stride = elements per pixel step in a staged row
constexpr int kPcRowElems = 272;   // staged row: 32 chunks of 8 elements written per step, 16 more that stay zero
constexpr int kPcKW = 16;          // kernel columns per contraction step (weights beyond the real width are zero)

template <int KS, int NW>  // KS = Cin * KH contraction steps, NW = Cout / 32 waves
__global__ __launch_bounds__(512) void patch_conv_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ wp,
                                                         uint16_t* __restrict__ y, int Cin, int H, int W, int KH, int OH,
                                                         int OW, int Cout, int nrows) {
  extern __shared__ __align__(16) char smem[];
  uint16_t* slab = reinterpret_cast<uint16_t*>(smem);  // [KS][kPcRowElems]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  constexpr int nwaves = NW;
  const int r = lane & 31, h = lane >> 5;
  // the columns no step writes (and, until the first step, everything) read as zero
  for (int i = threadIdx.x; i < KS * kPcRowElems / 8; i += blockDim.x)
    reinterpret_cast<u32x4_t*>(slab)[i] = u32x4_t{0u, 0u, 0u, 0u};
  // this wave's 32 output channels: matrix row i holds channel 16*((i>>2)&1) + 4*(i>>3) + (i&3) of the tile, which
  // leaves lane (r, h) with channels 16h .. 16h+15 of pixel r in its accumulator registers
  const int chan_of_row = 16 * ((r >> 2) & 1) + 4 * (r >> 3) + (r & 3);
  u32x4_t wf[KS];
#pragma unroll
  for (int t = 0; t < KS; ++t)
    wf[t] = *reinterpret_cast<const u32x4_t*>(wp + ((size_t)(32 * wave + chan_of_row) * KS + t) * kPcKW + 8 * h);
  __syncthreads();
  // image rows of the slab a thread fetches: half-wave (wave, h) takes slab rows 2*p + h, p = wave, wave + nwaves, ..;
  // the chunks of the next output row are in flight while the current one is multiplied
  constexpr int kMaxP = ((KS + 1) / 2 + NW - 1) / NW;  // row pairs per wave
  auto fetch = [&](int row, u32x4_t (&v)[kMaxP]) {
    const int b = row / OH, oy = row - b * OH;
#pragma unroll
    for (int i = 0; i < kMaxP; ++i) {
      const int t = 2 * (wave + i * nwaves) + h;
      const int c = t / KH, ky = t - c * KH;
      const int iy = oy * kPcStride - 1 + ky;
      v[i] = u32x4_t{0u, 0u, 0u, 0u};
      if (row < nrows && t < KS && iy >= 0 && iy < H && r * 8 < W)
        v[i] = *reinterpret_cast<const u32x4_t*>(x + (((size_t)b * Cin + c) * H + iy) * (size_t)W + r * 8);
    }
  };
  u32x4_t v[kMaxP];
  fetch(blockIdx.x, v);
  for (int row = blockIdx.x; row < nrows; row += gridDim.x) {
    // ---- stage the slab: lane r = 16-byte chunk r of its image row, shifted by one element ----
#pragma unroll
    for (int i = 0; i < kMaxP; ++i) {
      const int t = 2 * (wave + i * nwaves) + h;
      uint32_t prev = __shfl_up(v[i][3], 1, 32);  // the left neighbour's last pair; chunk 0 has the padding there
      if (r == 0) prev = 0u;
      u32x4_t o;
      o[0] = __builtin_amdgcn_alignbit(v[i][0], prev, 16);
      o[1] = __builtin_amdgcn_alignbit(v[i][1], v[i][0], 16);
      o[2] = __builtin_amdgcn_alignbit(v[i][2], v[i][1], 16);
      o[3] = __builtin_amdgcn_alignbit(v[i][3], v[i][2], 16);
      if (t < KS) *reinterpret_cast<u32x4_t*>(slab + t * kPcRowElems + r * 8) = o;
    }
    __syncthreads();
    fetch(row + gridDim.x, v);
    // ---- pixels x channels: KS contraction steps ----
    f32x16_t acc;
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[j] = 0.f;
#pragma unroll
    for (int t = 0; t < KS; ++t) {
      const u32x4_t px = *reinterpret_cast<const u32x4_t*>(slab + t * kPcRowElems + r * kPcStride + 8 * h);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, wf[t]),
                                                    __builtin_bit_cast(bf16x8_t, px), acc, 0, 0, 0);
    }
    u32x4_t lo, hi;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      lo[j] = pack_bf16x2(acc[2 * j], acc[2 * j + 1]);
      hi[j] = pack_bf16x2(acc[8 + 2 * j], acc[8 + 2 * j + 1]);
    }
    if (r < OW) {
      uint16_t* dst = y + ((size_t)row * OW + r) * (size_t)Cout + 32 * wave + 16 * h;
      *reinterpret_cast<u32x4_t*>(dst) = lo;
      *reinterpret_cast<u32x4_t*>(dst + 8) = hi;
    }
    __syncthreads();  // the next step's staging overwrites the slab
  }
}

}  // namespace

bool patch_conv_supported(int Cin, int H, int W, int KH, int KW, int stride, int padding, int Cout) {
  if (stride != kPcStride || padding != 1 || KW < 1 || KW > kPcKW || Cin * KH != 27) return false;
  if (W % 8 != 0 || W > 248 || H < 1) return false;
  const int OW = (W + 2 - KW) / stride + 1;
  return OW >= 1 && OW <= 32 && Cout % 32 == 0 && Cout >= 64 && Cout <= 256;  // two to eight waves
}

int launch_patch_conv(const void* x, const void* w_packed, void* y, int B, int Cin, int H, int W, int KH, int KW,
                      int Cout, hipStream_t stream) {
  if (!patch_conv_supported(Cin, H, W, KH, KW, kPcStride, 1, Cout)) return -95;
  const int OH = (H + 2 - KH) / kPcStride + 1, OW = (W + 2 - KW) / kPcStride + 1;
  if (OH < 1 || (long long)B * OH > 0x7fffffffLL - 4096 || Cout / 32 < 2) return -95;
  const int nrows = B * OH;
  const int grid = nrows < 512 ? nrows : 512;  // two workgroups a CU; each walks rows grid apart
  const size_t lds = (size_t)27 * kPcRowElems * sizeof(uint16_t);
#define VIG_PC_CASE(NW)                                                                                            \
  case NW:                                                                                                         \
    hipLaunchKernelGGL((patch_conv_kernel<27, NW>), dim3(grid), dim3(64 * NW), lds, stream, (const uint16_t*)x, \
                       (const uint16_t*)w_packed, (uint16_t*)y, Cin, H, W, KH, OH, OW, Cout, nrows);              \
    break
  switch (Cout / 32) {
    VIG_PC_CASE(2);
    VIG_PC_CASE(3);
    VIG_PC_CASE(4);
    VIG_PC_CASE(5);
    VIG_PC_CASE(6);
    VIG_PC_CASE(7);
    VIG_PC_CASE(8);
    default:
      return -95;
  }
#undef VIG_PC_CASE
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

}  // namespace vig
