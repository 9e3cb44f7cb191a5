// Token-recurrent backward of the bidirectional GLA op in fp32 arithmetic.
//
// One workgroup of 4 waves per (batch*head).  Per direction it makes two sweeps over the tokens, staged through LDS
// in blocks of TB, with the [Dk x Dv] state (and its adjoint) held in registers in two layouts at once:
//   layout A: lane = state column (dv), wave w owns Dk/4 rows   -> sums over dk are in-thread + across waves
//   layout B: lane = state row (dk),    wave w owns Dv/4 columns -> sums over dv are in-thread + across waves
// so no per-token cross-lane reduction is needed; the four waves' partial sums meet in LDS once per block.
//   sweep 1 (the direction's walk order):  S_t = a_t*S + k_t v_t^T (layout B);  dq_t = scale * S_t do_t
//   sweep 2 (the opposite order):          dS_t = (scale*q_t) do_t^T + a_t'*dS_t' (both layouts, t' = token walked
//                                           after t);  dk_t = dS_t v_t (layout B);  dv_t = dS_t^T k_t (layout A);
//                                           dG_t = q_t*dq_t - k_t*dk_t;  dg_t = running sum of dG along sweep 2.
// dq of a direction is parked in the caller workspace between the sweeps; dk, dv (and dq) of the first direction are
// parked there as fp32 until the second direction adds its own and writes the typed results, the same thread
// touching the same element both times.
//
// Same derivatives as flash-linear-attention/fla/ops/gla/chunk_fuse.py:413-518 (dq, dk, dv by the adjoint state,
// gate gradient as q*dq - k*dk followed by a reversed cumulative sum, :505-518), per token instead of per chunk
// and for both directions of classification/models/vig.py:407-426 in natural token order.
#include "common.h"
#include "launch.h"

namespace vig {

struct GlaBwdArgs {
  const void *q, *k, *v, *g_fwd, *g_bwd, *d_o;
  void *dq, *dk, *dv, *dg_fwd, *dg_bwd;
  void* workspace;
  int B, H, L, Dk, Dv;
  float scale, out_scale;
  int io_dtype, gate_dtype;
  hipStream_t stream;
  const int* only_flagged;  // null: every slab; else one int per (batch, head): slabs with 0 are skipped
};

template <typename TIO, typename TG, int DK, int DV, int TB>
__global__ __launch_bounds__(256) void gla_backward_kernel(
    const TIO* __restrict__ q, const TIO* __restrict__ k, const TIO* __restrict__ v, const TG* __restrict__ gf,
    const TG* __restrict__ gb, const TIO* __restrict__ d_o, TIO* dq, TIO* dk, TIO* dv, TG* dgf, TG* dgb,
    float* ws_dq, float* ws_acc_k, float* ws_acc_v, int L, float scale, float out_scale,
    const int* __restrict__ only_flagged) {
  // second pass behind the matrix-core kernel: only the slabs it left out (uniform per workgroup, before any barrier)
  if (only_flagged && only_flagged[blockIdx.x] == 0) return;
  constexpr int DKG = DK / 4;  // rows per wave, layout A
  constexpr int DVG = DV / 4;  // columns per wave, layout B
  __shared__ __align__(16) float sq[TB][DK];   // scale * q
  __shared__ __align__(16) float sk[TB][DK];
  __shared__ __align__(16) float sa[TB][DK];   // exp(g)
  __shared__ __align__(16) float sv[TB][DV];
  __shared__ __align__(16) float sd[TB][DV];   // out_scale * do
  __shared__ float pk[4][TB][DK];              // partial sums over dv quarters (layout B): dq in sweep 1, dk in sweep 2
  __shared__ float pv[4][TB][DV];              // partial sums over dk quarters (layout A): dv in sweep 2

  const int tid = threadIdx.x;
  const int w = tid >> 6, lane = tid & 63;
  const size_t bh = blockIdx.x;
  const size_t qk_base = bh * (size_t)L * DK;
  const size_t vo_base = bh * (size_t)L * DV;
  const int nblk = (L + TB - 1) / TB;
  const int ndir = gb ? 2 : 1;
  const bool row_ok = lane < DK;  // layout B lanes that own a state row
  const bool col_ok = lane < DV;  // layout A lanes that own a state column

  auto stage = [&](const TG* g, int t0, bool with_q) {
    for (int idx = tid; idx < TB * DK; idx += 256) {
      const int t = idx / DK, d = idx % DK;
      const int tok = t0 + t;
      float fq = 0.f, fk = 0.f, fa = 1.f;
      if (tok < L) {
        const size_t off = qk_base + (size_t)tok * DK + d;
        if (with_q) fq = Elem<TIO>::load(q + off) * scale;
        fk = Elem<TIO>::load(k + off);
        fa = __expf(Elem<TG>::load(g + off));
      }
      sq[t][d] = fq;
      sk[t][d] = fk;
      sa[t][d] = fa;
    }
    for (int idx = tid; idx < TB * DV; idx += 256) {
      const int t = idx / DV, c = idx % DV;
      const int tok = t0 + t;
      float fv = 0.f, fd = 0.f;
      if (tok < L) {
        fv = Elem<TIO>::load(v + vo_base + (size_t)tok * DV + c);
        fd = Elem<TIO>::load(d_o + vo_base + (size_t)tok * DV + c) * out_scale;
      }
      sv[t][c] = fv;
      sd[t][c] = fd;
    }
  };

  for (int dir = 0; dir < ndir; ++dir) {
    const TG* g = dir ? gb : gf;
    TG* dg = dir ? dgb : dgf;
    const bool rev = dir == 1;              // the direction walks tokens L-1 .. 0
    const bool last_dir = dir == ndir - 1;  // writes the typed dq, dk, dv
    float* my_dq = ws_dq + ((size_t)dir * gridDim.x + bh) * (size_t)L * DK;

    // ---- sweep 1: state in layout B, dq of this direction to the workspace ----
    {
      float Sb[DVG];
#pragma unroll
      for (int j = 0; j < DVG; ++j) Sb[j] = 0.f;
      for (int ib = 0; ib < nblk; ++ib) {
        const int blk = rev ? nblk - 1 - ib : ib;
        const int t0 = blk * TB;
        stage(g, t0, false);
        __syncthreads();
        if (row_ok) {
#pragma unroll 1
          for (int it = 0; it < TB; ++it) {
            const int t = rev ? TB - 1 - it : it;
            const float a = sa[t][lane], kk = sk[t][lane];
            float p = 0.f;
#pragma unroll
            for (int j = 0; j < DVG; ++j) {
              Sb[j] = Sb[j] * a + kk * sv[t][w * DVG + j];
              p += Sb[j] * sd[t][w * DVG + j];
            }
            pk[w][t][lane] = p;
          }
        }
        __syncthreads();
        for (int idx = tid; idx < TB * DK; idx += 256) {
          const int t = idx / DK, d = idx % DK;
          const int tok = t0 + t;
          if (tok < L) my_dq[(size_t)tok * DK + d] = scale * ((pk[0][t][d] + pk[1][t][d]) + (pk[2][t][d] + pk[3][t][d]));
        }
        __syncthreads();
      }
    }

    // ---- sweep 2: adjoint state in both layouts; dk, dv, dg (and the typed dq) ----
    {
      float dSa[DKG], dSb[DVG];
#pragma unroll
      for (int j = 0; j < DKG; ++j) dSa[j] = 0.f;
#pragma unroll
      for (int j = 0; j < DVG; ++j) dSb[j] = 0.f;
      float run = 0.f;  // running sum of dG for channel `lane` (wave 0 only)
      for (int ib = 0; ib < nblk; ++ib) {
        const int blk = rev ? ib : nblk - 1 - ib;
        const int t0 = blk * TB;
        stage(g, t0, true);
        __syncthreads();
#pragma unroll 1
        for (int it = 0; it < TB; ++it) {
          const int t = rev ? it : TB - 1 - it;
          if (col_ok) {  // layout A: rows w*DKG.., column lane
            const float dd = sd[t][lane];
            float p = 0.f;
#pragma unroll
            for (int j = 0; j < DKG; ++j) {
              const int d = w * DKG + j;
              dSa[j] += sq[t][d] * dd;
              p += dSa[j] * sk[t][d];
              dSa[j] *= sa[t][d];
            }
            pv[w][t][lane] = p;
          }
          if (row_ok) {  // layout B: row lane, columns w*DVG..
            const float qq = sq[t][lane], a = sa[t][lane];
            float p = 0.f;
#pragma unroll
            for (int j = 0; j < DVG; ++j) {
              const int c = w * DVG + j;
              dSb[j] += qq * sd[t][c];
              p += dSb[j] * sv[t][c];
              dSb[j] *= a;
            }
            pk[w][t][lane] = p;
          }
        }
        __syncthreads();
        // dv of this block
        for (int idx = tid; idx < TB * DV; idx += 256) {
          const int t = idx / DV, c = idx % DV;
          const int tok = t0 + t;
          if (tok < L) {
            float s = (pv[0][t][c] + pv[1][t][c]) + (pv[2][t][c] + pv[3][t][c]);
            const size_t off = vo_base + (size_t)tok * DV + c;
            if (ndir == 2 && !last_dir) {
              ws_acc_v[off] = s;
            } else {
              if (ndir == 2) s += ws_acc_v[off];
              Elem<TIO>::store(dv + off, s);
            }
          }
        }
        // dk, dq of this block
        for (int idx = tid; idx < TB * DK; idx += 256) {
          const int t = idx / DK, d = idx % DK;
          const int tok = t0 + t;
          if (tok < L) {
            float s = (pk[0][t][d] + pk[1][t][d]) + (pk[2][t][d] + pk[3][t][d]);
            pk[0][t][d] = s;  // this direction's dk, for the gate gradient below (same thread wrote and reads it)
            const size_t off = qk_base + (size_t)tok * DK + d;
            if (ndir == 2 && !last_dir) {
              ws_acc_k[off] = s;
            } else {
              float sq_ = my_dq[(size_t)tok * DK + d];
              if (ndir == 2) {
                s += ws_acc_k[off];
                sq_ += ws_dq[bh * (size_t)L * DK + (size_t)tok * DK + d];  // the first direction's dq
              }
              Elem<TIO>::store(dk + off, s);
              Elem<TIO>::store(dq + off, sq_);
            }
          }
        }
        __syncthreads();
        // gate gradient: running sum of q*dq - k*dk along this sweep, one channel per lane of wave 0
        if (w == 0 && row_ok) {
#pragma unroll 1
          for (int it = 0; it < TB; ++it) {
            const int t = rev ? it : TB - 1 - it;
            const int tok = t0 + t;
            if (tok < L) {
              const size_t off = qk_base + (size_t)tok * DK + lane;
              const float qv = Elem<TIO>::load(q + off);  // unscaled q: my_dq already carries the scale
              run += qv * my_dq[(size_t)tok * DK + lane] - sk[t][lane] * pk[0][t][lane];
              Elem<TG>::store(dg + off, run);
            }
          }
        }
        __syncthreads();
      }
    }
  }
}

template <typename TIO, typename TG, int DK, int DV>
static int launch_bwd_t(const GlaBwdArgs& a) {
  constexpr int TB = 16;
  const size_t n_qk = (size_t)a.B * a.H * a.L * DK, n_v = (size_t)a.B * a.H * a.L * DV;
  const int ndir = a.g_bwd ? 2 : 1;
  float* ws = (float*)a.workspace;
  float* ws_dq = ws;
  float* ws_acc_k = ws + (size_t)ndir * n_qk;
  float* ws_acc_v = ws_acc_k + n_qk;
  (void)n_v;
  hipLaunchKernelGGL((gla_backward_kernel<TIO, TG, DK, DV, TB>), dim3(a.B * a.H), dim3(256), 0, a.stream,
                     (const TIO*)a.q, (const TIO*)a.k, (const TIO*)a.v, (const TG*)a.g_fwd, (const TG*)a.g_bwd,
                     (const TIO*)a.d_o, (TIO*)a.dq, (TIO*)a.dk, (TIO*)a.dv, (TG*)a.dg_fwd, (TG*)a.dg_bwd, ws_dq,
                     ws_acc_k, ws_acc_v, a.L, a.scale, a.out_scale, a.only_flagged);
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

template <typename TIO, typename TG>
static int launch_bwd_d(const GlaBwdArgs& a) {
#define VIG_BWD_CASE(K, V) \
  if (a.Dk == K && a.Dv == V) return launch_bwd_t<TIO, TG, K, V>(a)
  VIG_BWD_CASE(16, 32);
  VIG_BWD_CASE(32, 32);
  VIG_BWD_CASE(32, 64);
  VIG_BWD_CASE(64, 32);
  VIG_BWD_CASE(64, 64);
#undef VIG_BWD_CASE
  return -95;
}

// fp32 scratch of the recurrent kernel, then one flag per slab for the matrix-core kernel
static size_t recurrent_floats(int B, int H, int L, int Dk, int Dv, int bidir) {
  const size_t n_qk = (size_t)B * H * L * Dk, n_v = (size_t)B * H * L * Dv;
  return bidir ? 3 * n_qk + n_v : n_qk;
}
// ... and, 256-byte aligned behind the flags, what the matrix-core kernel needs for sequences longer than one slab
static size_t flags_end(int B, int H, int L, int Dk, int Dv, int bidir) {
  const size_t n = recurrent_floats(B, H, L, Dk, Dv, bidir) * sizeof(float) + (size_t)B * H * sizeof(int);
  return (n + 255) / 256 * 256;
}
size_t gla_backward_workspace(int B, int H, int L, int Dk, int Dv, int bidir) {
  const size_t seg = gla_backward_mfma_workspace(B, H, L, Dk, Dv);
  if (seg == 0) return recurrent_floats(B, H, L, Dk, Dv, bidir) * sizeof(float) + (size_t)B * H * sizeof(int);
  return flags_end(B, H, L, Dk, Dv, bidir) + seg;
}

int launch_gla_backward(const void* q, const void* k, const void* v, const void* g_fwd, const void* g_bwd,
                        const void* d_o, void* dq, void* dk, void* dv, void* dg_fwd, void* dg_bwd, void* workspace,
                        int B, int H, int L, int Dk, int Dv, float scale, float out_scale, int io_dtype,
                        int gate_dtype, bool exact, hipStream_t stream) {
  GlaBwdArgs a{q, k, v, g_fwd, g_bwd, d_o, dq, dk, dv, dg_fwd, dg_bwd, workspace, B, H, L, Dk, Dv,
               scale, out_scale, io_dtype, gate_dtype, stream, nullptr};
  if (!exact && gla_backward_mfma_supported(B, H, L, Dk, Dv, io_dtype, gate_dtype, g_bwd != nullptr)) {
    int* flags = reinterpret_cast<int*>((float*)workspace + recurrent_floats(B, H, L, Dk, Dv, g_bwd != nullptr));
    void* seg_ws = (char*)workspace + flags_end(B, H, L, Dk, Dv, g_bwd != nullptr);
    const int rc = launch_gla_backward_mfma(q, k, v, g_fwd, g_bwd, d_o, dq, dk, dv, dg_fwd, dg_bwd, flags, seg_ws, B,
                                            H, L, Dk, scale * out_scale, stream);
    if (rc != 0) return rc;
    a.only_flagged = flags;  // slabs with gates beyond the matrix-core kernel's range
  }
  if (io_dtype == 0) return gate_dtype == 0 ? launch_bwd_d<float, float>(a) : launch_bwd_d<float, uint16_t>(a);
  return gate_dtype == 0 ? launch_bwd_d<uint16_t, float>(a) : launch_bwd_d<uint16_t, uint16_t>(a);
}

}  // namespace vig
