// gate_proj and the SwiGLU product of the block's MLP in one kernel, for contractions as short as the hidden size
// (K = 16 * KS <= 384):
//   out[t, c] = g * sigmoid(g) * u,   g = A[t, :] . W[c, :],   u = A[t, :] . W[I + c, :]      (W = [2*I, K])
// bf16 operands, fp32 accumulation, bf16 out; the product is taken on g and u rounded to bf16, the values the
// separate layer would have stored (flash-linear-attention/fla/modules/activations.py:109-113 on the two halves of
// gate_proj's output, classification/models/vig.py:492-495), so the [T, 2*I] intermediate never exists.
//
// With K this short a wave's whole slice of W fits in registers: a wave keeps the 32 gate rows and the 32 matching
// up rows of one channel tile as matrix-instruction A operands for the life of the workgroup, eight waves cover 256
// channels, and the workgroup streams 32-token tiles of A through LDS, double-buffered: the next tile travels from
// memory straight into its buffer (direct-to-LDS loads, whole token rows per wave, no registers) during the matrix
// instructions of the current one, and every 16-byte LDS read, issued three k-steps ahead of its use, feeds two
// v_mfma_f32_32x32x16_bf16.  The two waves of a SIMD take turns on its matrix and vector pipes (see the loop).  Matrix
// rows are assigned channels so that a lane ends with 16 consecutive channels of one token (32 contiguous bytes).
// Workgroups of the same column group are spread over the token tiles; the column groups of one token tile run on the
// same XCD (workers are a multiple of the XCD count apart in block index), so a tile of A leaves HBM once.
#include "common.h"
#include "launch.h"

namespace vig {

namespace {

constexpr int kLinWaves = 8;

template <int KS>
__global__ __launch_bounds__(64 * kLinWaves) void linear_swiglu_kernel(const uint16_t* __restrict__ A,
                                                                       const uint16_t* __restrict__ W,
                                                                       uint16_t* __restrict__ out, int T, int I,
                                                                       int nworkers) {
  constexpr int K = 16 * KS;
  constexpr int kThreads = 64 * kLinWaves;
  constexpr int kCols = K / 8;                 // 16-byte chunks per token row
  constexpr int kRow = K + 8;                  // LDS row stride in elements (conflict-free 16-byte reads)
  constexpr int kPer = 32 / kLinWaves;         // token rows per wave
  static_assert(kCols <= 64 && 32 % kLinWaves == 0, "a wave loads whole token rows");
  extern __shared__ __align__(16) char smem[];
  uint16_t* buf = reinterpret_cast<uint16_t*>(smem);  // [2][32][kRow]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, h = lane >> 5;
  const int cg = blockIdx.x / nworkers, worker = blockIdx.x - cg * nworkers;
  const int ct = cg * kLinWaves + wave;  // this wave's channel tile
  const bool have = 32 * ct < I;
  // matrix row i holds channel 16*((i>>2)&1) + 4*(i>>3) + (i&3) of the tile: lane (r, h) ends with channels 16h..16h+15
  const int chan_of_row = 16 * ((r >> 2) & 1) + 4 * (r >> 3) + (r & 3);
  u32x4_t wg[KS], wu[KS];
  {
    const uint16_t* pg = W + (size_t)(have ? 32 * ct + chan_of_row : 0) * K + 8 * h;
    const uint16_t* pu = pg + (size_t)I * K;
#pragma unroll
    for (int t = 0; t < KS; ++t) {
      wg[t] = *reinterpret_cast<const u32x4_t*>(pg + 16 * t);
      wu[t] = *reinterpret_cast<const u32x4_t*>(pu + 16 * t);
    }
  }
  const int ntiles_t = (T + 31) / 32;
  // A tile travels from memory straight into its LDS buffer (no registers): lane i of a wave lands 16 i bytes behind
  // the wave's base, so a wave loads whole token rows (the first K/8 lanes, one 16-byte chunk each) to the rows' padded
  // places.  Token rows past the end are not requested: their rows of the buffer keep old data, and their products
  // are never stored.
  typedef __attribute__((address_space(3))) void* lds_ptr_t;
  auto fetch = [&](int tile, int which) {
    if (tile >= ntiles_t) return;
    char* base = reinterpret_cast<char*>(buf + which * (32 * kRow));
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
      const int row = i * kLinWaves + wave;
      if (lane < kCols && tile * 32 + row < T)
        __builtin_amdgcn_global_load_lds(A + (size_t)tile * (32 * K) + (size_t)row * K + lane * 8,
                                         (lds_ptr_t)(base + row * (kRow * 2)), 16, 0, 0);
    }
  };
  f32x16_t g, u;
#pragma unroll
  for (int j = 0; j < 16; ++j) g[j] = 0.f, u[j] = 0.f;
  // SwiGLU on the rounded gate and up values of one finished tile, 16 consecutive channels of one token per lane
  auto epilogue = [&](int etile) {
    u32x4_t lo, hi;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float y[2];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const float gs = bf16_to_f32(f32_to_bf16(g[2 * j + e])), us = bf16_to_f32(f32_to_bf16(u[2 * j + e]));
        y[e] = gs * us * sigmoidf_(gs);
      }
      const uint32_t pk = pack_bf16x2(y[0], y[1]);
      if (j < 4) lo[j] = pk;
      else hi[j - 4] = pk;
    }
    const int token = etile * 32 + r;
    if (have && token < T) {
      uint16_t* dst = out + (size_t)token * I + 32 * ct + 16 * h;
      *reinterpret_cast<u32x4_t*>(dst) = lo;
      *reinterpret_cast<u32x4_t*>(dst + 8) = hi;
    }
  };
  // this tile's products: operand reads run kAhead k-steps ahead of the matrix instructions that use them
  auto products = [&](const uint16_t* mine) {
#pragma unroll
    for (int j = 0; j < 16; ++j) g[j] = 0.f, u[j] = 0.f;
    const uint16_t* xrow = mine + r * kRow + 8 * h;
    constexpr int kAhead = 3;
    u32x4_t x[kAhead];
#pragma unroll
    for (int t = 0; t < kAhead; ++t) x[t] = *reinterpret_cast<const u32x4_t*>(xrow + 16 * t);
#pragma unroll
    for (int t = 0; t < KS; ++t) {
      const u32x4_t xt = x[t % kAhead];
      g = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, wg[t]), __builtin_bit_cast(bf16x8_t, xt),
                                                  g, 0, 0, 0);
      u = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, wu[t]), __builtin_bit_cast(bf16x8_t, xt),
                                                  u, 0, 0, 0);
      if (t + kAhead < KS) x[t % kAhead] = *reinterpret_cast<const u32x4_t*>(xrow + 16 * (t + kAhead));
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  fetch(worker, 0);
  int cur = 0;
  for (int tile = worker; tile < ntiles_t; tile += nworkers, cur ^= 1) {
    const uint16_t* mine = buf + cur * (32 * kRow);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this thread's chunks of the tile have landed
    __syncthreads();  // the tile is complete; the other buffer was last read before the previous barrier
    fetch(tile + nworkers, cur ^ 1);
    // The two waves of a SIMD (w and w + 4) take turns on its two pipes: the lower wave runs this tile's matrix
    // instructions first and its SwiGLU epilogue after; the upper wave first runs the epilogue of its PREVIOUS tile
    // (its accumulators waited in registers) and then this tile's matrix instructions.  So one wave's vector work
    // runs under the other's matrix work in both halves of a tile's time, with one barrier per tile as before.
    if (wave < kLinWaves / 2) {
      products(mine);
      epilogue(tile);  // (straight-line after the matrix instructions: no run-time branch in between)
    } else {
      if (tile > worker) epilogue(tile - nworkers);
      products(mine);
    }
  }
  if (wave >= kLinWaves / 2 && worker < ntiles_t)  // the upper waves' last tile
    epilogue(worker + ((ntiles_t - 1 - worker) / nworkers) * nworkers);
}

template <int KS>
int launch_linear_swiglu_t(const void* A, const void* W, void* out, long long T, int I, int num_cu, hipStream_t stream) {
  constexpr int K = 16 * KS;
  const size_t lds = (size_t)2 * 32 * (K + 8) * sizeof(uint16_t);
  const int ncg = (I / 32 + kLinWaves - 1) / kLinWaves;
  const long long ntiles_t = (T + 31) / 32;
  // one workgroup a CU; workers a multiple of 8 so that the column groups of a token tile share an XCD
  int nworkers = num_cu / ncg / 8 * 8;
  if (nworkers < 8) nworkers = 8;
  if (nworkers > ntiles_t) nworkers = (int)ntiles_t;
  hipLaunchKernelGGL((linear_swiglu_kernel<KS>), dim3(ncg * nworkers), dim3(64 * kLinWaves), lds, stream,
                     (const uint16_t*)A, (const uint16_t*)W, (uint16_t*)out, (int)T, I, nworkers);
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

// ---------------------------------------------------------------------------
// The mixer's epilogue and o_proj in one kernel:
//   y[t, h, :] = rms(o[b, h, l, :]) w_g sigmoid(g) + rms(loc[t, h, :]) w_l (1 - sigmoid(g))   (optionally y <- y sigmoid(y)),
//   out[t, :]  = y[t, :] . W[c, :]                                   (W = o_proj.weight [C, H*Dv], K = H*Dv = 16 * KS)
// with t = b*L + l, the head norms over the Dv = 64 channels of a (token, head), g = g_lin rows of pitch ldg
// (classification/models/vig.py:444-463).  y is rounded to bf16 as the separate blend kernel would store it and never
// leaves the chip: the workgroup computes a 32-token tile of it straight into the LDS buffer the matrix instructions
// read (double-buffered).  The o / loc / g octets of the next tile travel from memory straight into thread-private
// LDS slots (no registers: lane i of a wave lands at the wave's slot base + 16 i) while the matrix instructions of the
// current tile run.  NW waves hold TPW 32-channel tiles of W each as matrix-instruction operands for the life of the
// workgroup, so one workgroup makes whole output rows (C = 32 * TPW * NW) and every tile of y is computed once.
// ---------------------------------------------------------------------------
// value of the lane a DPP control names (inside a row of 16 lanes)
template <int CTRL>
__device__ __forceinline__ float lane_permuted(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

// This wave's LDS writes done, then the barrier, and nothing else: global requests and stores issued before it stay in
// flight.  (A fence would drain them: the compiler counts loads that land in LDS as LDS writes.  Whoever reads what
// such a load brings waits for it by itself.)
__device__ __forceinline__ void tile_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <int KS, int NW, int TPW>
__global__ __launch_bounds__(64 * NW) void blend_linear_kernel(const uint16_t* __restrict__ o,
                                                              const uint16_t* __restrict__ loc,
                                                              const uint16_t* __restrict__ glin,
                                                              const float* __restrict__ w_g,
                                                              const float* __restrict__ w_l,
                                                              const uint16_t* __restrict__ W,
                                                              uint16_t* __restrict__ out, int T, int L, int H,
                                                              long long ldg, float eps, int silu_out) {
  constexpr int K = 16 * KS;
  constexpr int C = 32 * TPW * NW;             // TPW 32-channel tiles of W per wave
  constexpr int kThreads = 64 * NW;
  constexpr int kCols = K / 8;                 // channel octets per token row
  constexpr int kRow = K + 8;                  // LDS row stride in elements (conflict-free 16-byte reads)
  constexpr int kChunks = 32 * kCols;          // channel octets of a 32-token tile
  constexpr int kPer = kChunks / kThreads;     // octets per thread
  static_assert(kChunks % kThreads == 0, "whole octets per thread");
  static_assert(kThreads % kCols == 0, "a thread's octets share their column");
  extern __shared__ __align__(16) char smem[];
  uint16_t* buf = reinterpret_cast<uint16_t*>(smem);  // [2][32][kRow]
  float* wnorm = reinterpret_cast<float*>(smem + (size_t)2 * 32 * kRow * sizeof(uint16_t));  // w_g | w_l, 64 floats each
  // thread-private slots for the fetched octets of the tile that comes next: [octet i][o, loc, g][thread]
  u32x4_t* park = reinterpret_cast<u32x4_t*>(smem + (size_t)2 * 32 * kRow * sizeof(uint16_t) + 128 * sizeof(float));
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, h = lane >> 5;
  if (tid < 128) wnorm[tid] = tid < 64 ? w_g[tid] : w_l[tid - 64];
  // matrix row i holds channel 16*((i>>2)&1) + 4*(i>>3) + (i&3) of the tile: lane (r, h) ends with channels 16h..16h+15
  const int chan_of_row = 16 * ((r >> 2) & 1) + 4 * (r >> 3) + (r & 3);
  u32x4_t wt[TPW][KS];  // channel tiles TPW * wave ..
#pragma unroll
  for (int j = 0; j < TPW; ++j) {
    const uint16_t* pw = W + (size_t)(32 * (TPW * wave + j) + chan_of_row) * K + 8 * h;
#pragma unroll
    for (int t = 0; t < KS; ++t) wt[j][t] = *reinterpret_cast<const u32x4_t*>(pw + 16 * t);
  }
  const int ntiles_t = (T + 31) / 32;
  const float* wg8 = wnorm + ((tid % kCols) & 7) * 8;  // (kThreads % kCols == 0: a thread's octets share their column)
  const float* wl8 = wg8 + 64;
  typedef __attribute__((address_space(3))) void* lds_ptr_t;
  // requests this thread's octets of a tile into its slots; tokens past the end are not requested (their rows of y
  // hold whatever the slots held: their products are never stored)
  const int col = tid % kCols, row0 = tid / kCols;  // this thread's octets: column col of rows row0 + kRowStep * i
  constexpr int kRowStep = kThreads / kCols;
  const size_t o_col = ((size_t)(col >> 3) * L) * 64 + (col & 7) * 8;  // head col / 8, channels 8 (col % 8) ..
  const size_t o_batch = (size_t)H * L * 64;
  auto fetch = [&](int tile) {
#pragma unroll 1
    for (int i = 0; i < kPer; ++i) {  // (one octet's addresses at a time: the weight tiles leave few registers)
      const int t = tile * 32 + row0 + kRowStep * i;
      if (tile < ntiles_t && t < T) {
        const unsigned b = (unsigned)t / (unsigned)L, l = (unsigned)t - b * (unsigned)L;
        char* slot = reinterpret_cast<char*>(park + (i * 3) * kThreads + wave * 64);  // (wave-uniform; lanes 16 B apart)
        __builtin_amdgcn_global_load_lds(o + b * o_batch + (size_t)l * 64 + o_col, (lds_ptr_t)slot, 16, 0, 0);
        __builtin_amdgcn_global_load_lds(loc + (size_t)t * K + col * 8, (lds_ptr_t)(slot + kThreads * 16), 16, 0, 0);
        __builtin_amdgcn_global_load_lds(glin + (size_t)t * ldg + col * 8, (lds_ptr_t)(slot + 2 * kThreads * 16), 16, 0, 0);
      }
    }
  };
  const int nworkers = gridDim.x;
  // the blend of this thread's octets of a tile (they wait in its slots), straight into the tile's operand buffer
  auto blend = [&](uint16_t* mine) {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the octets are in their slots
#pragma unroll 1
    for (int i = 0; i < kPer; ++i) {
      const u32x4_t po = park[(i * 3 + 0) * kThreads + tid], pl = park[(i * 3 + 1) * kThreads + tid],
                    pg = park[(i * 3 + 2) * kThreads + tid];
      float fo[8], fl[8], fg[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        fo[2 * j] = bf16_to_f32((uint16_t)(po[j] & 0xffffu)), fo[2 * j + 1] = bf16_to_f32((uint16_t)(po[j] >> 16));
        fl[2 * j] = bf16_to_f32((uint16_t)(pl[j] & 0xffffu)), fl[2 * j + 1] = bf16_to_f32((uint16_t)(pl[j] >> 16));
        fg[2 * j] = bf16_to_f32((uint16_t)(pg[j] & 0xffffu)), fg[2 * j + 1] = bf16_to_f32((uint16_t)(pg[j] >> 16));
      }
      float so = 0.f, sl = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) so += fo[j] * fo[j], sl += fl[j] * fl[j];
      // the eight lanes of a (token, head): lane ^ 1, lane ^ 2 inside the quad, then the other quad of the eight
      so += lane_permuted<0xB1>(so), sl += lane_permuted<0xB1>(sl);    // quad_perm:[1,0,3,2]
      so += lane_permuted<0x4E>(so), sl += lane_permuted<0x4E>(sl);    // quad_perm:[2,3,0,1]
      so += lane_permuted<0x141>(so), sl += lane_permuted<0x141>(sl);  // row_half_mirror
      const float ro = rsqrtf(so * (1.0f / 64.0f) + eps);
      const float rl = rsqrtf(sl * (1.0f / 64.0f) + eps);
      float e[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float sg = sigmoidf_(fg[j]);
        e[j] = fo[j] * ro * wg8[j] * sg + fl[j] * rl * wl8[j] * (1.f - sg);
      }
      if (silu_out) {
        asm volatile("");  // (a real branch: as a select, the second sigmoid is computed for every caller)
#pragma unroll
        for (int j = 0; j < 8; ++j) e[j] = e[j] * sigmoidf_(e[j]);
      }
      u32x4_t y;
#pragma unroll
      for (int j = 0; j < 4; ++j) y[j] = pack_bf16x2(e[2 * j], e[2 * j + 1]);
      *reinterpret_cast<u32x4_t*>(mine + (row0 + kRowStep * i) * kRow + col * 8) = y;
    }
  };
  // this wave's products of a staged tile, and its rows of the result
  auto products = [&](const uint16_t* mine, int tile) {
    f32x16_t acc[TPW];
#pragma unroll
    for (int j = 0; j < TPW; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[j][e] = 0.f;
    const uint16_t* xrow = mine + r * kRow + 8 * h;
    constexpr int kAhead = TPW == 2 ? 3 : 1;  // operand reads this many k-steps ahead of the matrix instructions that
                                              // use them, where the registers allow
    u32x4_t x[kAhead];
#pragma unroll
    for (int t = 0; t < kAhead; ++t) x[t] = *reinterpret_cast<const u32x4_t*>(xrow + 16 * t);
#pragma unroll
    for (int t = 0; t < KS; ++t) {
      const u32x4_t xt = x[t % kAhead];
#pragma unroll
      for (int j = 0; j < TPW; ++j)
        acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, wt[j][t]),
                                                         __builtin_bit_cast(bf16x8_t, xt), acc[j], 0, 0, 0);
      if (t + kAhead < KS) x[t % kAhead] = *reinterpret_cast<const u32x4_t*>(xrow + 16 * (t + kAhead));
      if (TPW == 2) __builtin_amdgcn_sched_barrier(0);
    }
    // (no run-time branch between the matrix instructions and the first read of their results)
    const int token = tile * 32 + r;
#pragma unroll
    for (int j = 0; j < TPW; ++j) {
      u32x4_t lo, hi;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        lo[e] = pack_bf16x2(acc[j][2 * e], acc[j][2 * e + 1]);
        hi[e] = pack_bf16x2(acc[j][8 + 2 * e], acc[j][8 + 2 * e + 1]);
      }
      if (token < T) {
        uint16_t* dst = out + (size_t)token * C + 32 * (TPW * wave + j) + 16 * h;
        *reinterpret_cast<u32x4_t*>(dst) = lo;
        *reinterpret_cast<u32x4_t*>(dst + 8) = hi;
      }
    }
  };
  // The waves take turns on the two pipes of their SIMD: waves 4 .. 7 (one per SIMD) first blend their octets of the
  // NEXT tile into the other buffer and then run this tile's matrix instructions; the other waves multiply first and
  // blend after (measured: 55.7 -> 52.7 us per layer at B256; the other split of the waves gained half of that).  One barrier per tile: behind it every wave has finished with tile i - 1's buffer
  // (being refilled now) and tile i's is complete.
  __syncthreads();  // the norm weights are in place
  fetch(blockIdx.x);
  blend(buf);
  fetch(blockIdx.x + nworkers);
  tile_barrier();
  int cur = 0;
  for (int tile = blockIdx.x; tile < ntiles_t; tile += nworkers, cur ^= 1) {
    const uint16_t* mine = buf + cur * (32 * kRow);
    uint16_t* next = buf + (cur ^ 1) * (32 * kRow);
    const bool more = tile + nworkers < ntiles_t;
    if ((wave >> 2) != 1) {
      products(mine, tile);
      if (more) {
        blend(next);
        fetch(tile + 2 * nworkers);
      }
    } else {
      if (more) {
        blend(next);
        fetch(tile + 2 * nworkers);
      }
      products(mine, tile);
    }
    tile_barrier();  // (the requests for the tile after the next and this tile's stores stay in flight)
  }
}

template <int KS, int NW, int TPW>
int launch_blend_linear_t(const void* o, const void* loc, const void* glin, const float* w_g, const float* w_l,
                          const void* W, void* out, long long T, int L, int H, long long ldg, float eps, int silu_out,
                          int num_cu, int dev, hipStream_t stream) {
  constexpr int K = 16 * KS;
  const size_t lds = (size_t)2 * 32 * (K + 8) * sizeof(uint16_t) + 128 * sizeof(float) +
                     (size_t)(32 * K / 8) * 3 * sizeof(u32x4_t);
  const long long ntiles_t = (T + 31) / 32;
  const int grid = ntiles_t < num_cu ? (int)ntiles_t : num_cu;
  static bool attr_done[64] = {};
  if (!attr_done[dev]) {  // (per device; concurrent first calls only repeat an idempotent setting)
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(blend_linear_kernel<KS, NW, TPW>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return -5;
    attr_done[dev] = true;
  }
  hipLaunchKernelGGL((blend_linear_kernel<KS, NW, TPW>), dim3(grid), dim3(64 * NW), lds, stream, (const uint16_t*)o,
                     (const uint16_t*)loc, (const uint16_t*)glin, w_g, w_l, (const uint16_t*)W, (uint16_t*)out, (int)T, L,
                     H, ldg, eps, silu_out);
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

}  // namespace

// o_proj of a square block (d_model = H * Dv) with 64-channel heads, at the widths the weights fit the registers
bool blend_linear_supported(int H, int Dv, int C) { return Dv == 64 && C == H * Dv && (C == 384 || C == 192); }

int launch_blend_linear(const void* o, const void* loc, const void* glin, const float* w_g, const float* w_l,
                        const void* W, void* out, int B, int H, int L, int Dv, int C, long long ldg, float eps,
                        int silu_out, hipStream_t stream) {
  if (!blend_linear_supported(H, Dv, C) || B <= 0 || L <= 0 || (long long)B * L > 0x7fffffffLL - 64 || ldg % 8 != 0 ||
      ldg < C)
    return -95;
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return -5;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return -5;
  const int num_cu = n > 0 ? n : 256;
  const long long T = (long long)B * L;
  // twelve waves with one weight tile each (three per SIMD at 168 registers) at the wider size, six at the narrower
  return C == 384 ? launch_blend_linear_t<24, 12, 1>(o, loc, glin, w_g, w_l, W, out, T, L, H, ldg, eps, silu_out, num_cu, dev, stream)
                  : launch_blend_linear_t<12, 6, 1>(o, loc, glin, w_g, w_l, W, out, T, L, H, ldg, eps, silu_out, num_cu, dev, stream);
}

bool linear_swiglu_supported(int K, int I) { return (K == 384 || K == 192) && I % 32 == 0 && I >= 32; }

int launch_linear_swiglu(const void* A, const void* W, void* out, long long T, int K, int I, hipStream_t stream) {
  if (!linear_swiglu_supported(K, I) || T <= 0 || T > 0x7fffffffLL - 64) return -95;
  constexpr int kMaxDevices = 64;
  static int num_cu_dev[kMaxDevices] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return -5;
  if (num_cu_dev[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return -5;
    num_cu_dev[dev] = n > 0 ? n : 256;
  }
  return K == 384 ? launch_linear_swiglu_t<24>(A, W, out, T, I, num_cu_dev[dev], stream)
                  : launch_linear_swiglu_t<12>(A, W, out, T, I, num_cu_dev[dev], stream);
}

}  // namespace vig

