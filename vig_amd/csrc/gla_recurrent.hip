// Token-recurrent bidirectional GLA forward in fp32 arithmetic (exact path).
//
// One workgroup of 4 waves per (batch*head, 64-column tile of Dv).  Wave w owns
// Dk/4 state rows, lane owns one state column, so the [Dk x Dv] fp32 state lives
// in registers (Dk/4 per lane) and never touches memory.  Tokens are staged
// through LDS in blocks of TB; the per-token partial read-outs of the four waves
// meet in LDS once per block.  The forward sweep parks its fp32 output in `acc`
// (the output tensor itself when it is fp32, else caller workspace); the reverse
// sweep adds its own and writes the final value, the same thread touching the
// same element in both sweeps.
//
// Semantics follow flash-linear-attention/fla/ops/gla/naive.py:33-41,48-56 and
// the merged inference kernel recurrent_fuse.py:99-142 (decay, add k v^T, read
// out with the scaled q), with independent gates per direction.
#include "common.h"
#include "launch.h"

namespace vig {

template <typename TIO, typename TG, int DKG, int TB>
__global__ __launch_bounds__(256) void gla_recurrent_kernel(
    const TIO* __restrict__ q, const TIO* __restrict__ k, const TIO* __restrict__ v,
    const TG* __restrict__ gf, const TG* __restrict__ gb, TIO* o,
    float* acc, int L, int Dv, float scale, float out_scale, const float* __restrict__ init_state,
    float* __restrict__ final_state) {
  constexpr int DK = DKG * 4;
  __shared__ float sq[TB][DK];
  __shared__ float sk[TB][DK];
  __shared__ float sa[TB][DK];
  __shared__ float sv[TB][64];
  __shared__ float so[4][TB][64];

  const int tid = threadIdx.x;
  const int w = tid >> 6;
  const int lane = tid & 63;
  const int bh = blockIdx.x;
  const int dv0 = blockIdx.y * 64;
  const int dv = dv0 + lane;
  const bool dv_ok = dv < Dv;
  const size_t qk_base = (size_t)bh * L * DK;
  const size_t vo_base = (size_t)bh * L * Dv;
  const int nblk = (L + TB - 1) / TB;
  const int npass = gb ? 2 : 1;

  for (int pass = 0; pass < npass; ++pass) {
    const TG* g = pass ? gb : gf;
    float S[DKG];
#pragma unroll
    for (int j = 0; j < DKG; ++j) S[j] = 0.f;
    // causal op: the state may start from a caller-supplied value (fla/ops/gla/chunk_fuse.py:70-72)
    if (init_state && pass == 0 && dv_ok) {
#pragma unroll
      for (int j = 0; j < DKG; ++j) S[j] = init_state[((size_t)bh * DK + w * DKG + j) * Dv + dv];
    }

    for (int ib = 0; ib < nblk; ++ib) {
      const int blk = pass ? (nblk - 1 - ib) : ib;
      const int t0 = blk * TB;
      for (int idx = tid; idx < TB * DK; idx += 256) {
        const int t = idx / DK, d = idx % DK;
        const int tok = t0 + t;
        float fq = 0.f, fk = 0.f, fa = 1.f;
        if (tok < L) {
          const size_t off = qk_base + (size_t)tok * DK + d;
          fq = Elem<TIO>::load(q + off) * scale;
          fk = Elem<TIO>::load(k + off);
          fa = __expf(Elem<TG>::load(g + off));
        }
        sq[t][d] = fq;
        sk[t][d] = fk;
        sa[t][d] = fa;
      }
      for (int idx = tid; idx < TB * 64; idx += 256) {
        const int t = idx >> 6, c = idx & 63;
        const int tok = t0 + t;
        float fv = 0.f;
        if (tok < L && dv0 + c < Dv) fv = Elem<TIO>::load(v + vo_base + (size_t)tok * Dv + dv0 + c);
        sv[t][c] = fv;
      }
      __syncthreads();

#pragma unroll 1
      for (int it = 0; it < TB; ++it) {
        const int t = pass ? (TB - 1 - it) : it;
        const float vv = sv[t][lane];
        float po = 0.f;
#pragma unroll
        for (int j = 0; j < DKG; ++j) {
          const int d = w * DKG + j;
          S[j] = S[j] * sa[t][d] + sk[t][d] * vv;
          po += sq[t][d] * S[j];
        }
        so[w][t][lane] = po;
      }
      __syncthreads();

      for (int t = w; t < TB; t += 4) {
        const int tok = t0 + t;
        if (tok < L && dv_ok) {
          const float s = (so[0][t][lane] + so[1][t][lane]) + (so[2][t][lane] + so[3][t][lane]);
          const size_t off = vo_base + (size_t)tok * Dv + dv;
          if (npass == 2 && pass == 0) {
            acc[off] = s;
          } else if (npass == 2) {
            Elem<TIO>::store(o + off, out_scale * (acc[off] + s));
          } else {
            Elem<TIO>::store(o + off, out_scale * s);
          }
        }
      }
      __syncthreads();
    }
    // ... and be handed back after the last token (chunk_fuse.py:99-101); padding tokens of the last block are no-ops
    if (final_state && pass == 0 && dv_ok) {
#pragma unroll
      for (int j = 0; j < DKG; ++j) final_state[((size_t)bh * DK + w * DKG + j) * Dv + dv] = S[j];
    }
  }
}

template <typename TIO, typename TG>
static int launch_recurrent_t(const GlaArgs& a) {
  constexpr int TB = 16;
  dim3 grid(a.B * a.H, (a.Dv + 63) / 64), block(256);
  float* acc = nullptr;
  if (a.g_bwd) {
    acc = sizeof(TIO) == 4 ? (float*)a.o : (float*)a.workspace;
  }
#define VIG_LAUNCH_REC(DKG)                                                                   \
  hipLaunchKernelGGL((gla_recurrent_kernel<TIO, TG, DKG, TB>), grid, block, 0, a.stream,      \
                     (const TIO*)a.q, (const TIO*)a.k, (const TIO*)a.v, (const TG*)a.g_fwd,   \
                     (const TG*)a.g_bwd, (TIO*)a.o, acc, a.L, a.Dv, a.scale, a.out_scale, a.init_state,   \
                     a.final_state)
  switch (a.Dk) {
    case 16: VIG_LAUNCH_REC(4); break;
    case 32: VIG_LAUNCH_REC(8); break;
    case 64: VIG_LAUNCH_REC(16); break;
    case 128: VIG_LAUNCH_REC(32); break;
    default: return -95;
  }
#undef VIG_LAUNCH_REC
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

int launch_gla_recurrent(const GlaArgs& a) {
  if (a.io_dtype == 0) {
    return a.gate_dtype == 0 ? launch_recurrent_t<float, float>(a) : launch_recurrent_t<float, uint16_t>(a);
  }
  return a.gate_dtype == 0 ? launch_recurrent_t<uint16_t, float>(a) : launch_recurrent_t<uint16_t, uint16_t>(a);
}

size_t gla_recurrent_workspace(int B, int H, int L, int Dv, int io_dtype) {
  return io_dtype == 0 ? 0 : (size_t)B * H * L * Dv * sizeof(float);
}

}  // namespace vig
