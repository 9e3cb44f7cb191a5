// PyTorch-ROCm extension over the C ABI of libvig_gla.so (include/vig_gla.h): one operator per forward entry point
// (namespace vig_amd), plus the eval-mode GLA block as one operator.  Host code only: it checks the tensors
// (device, dtype, layout, 16-byte alignment), takes outputs and workspaces from torch's caching allocator, passes the
// current HIP stream of the tensors' device and turns status codes into exceptions.  No kernel lives here.
//
// The operators mirror the reference's call sites: the op signatures of flash-linear-attention/fla/ops/gla/
// chunk_fuse.py:554-596 and recurrent_fuse.py:631-676, and the eval branch of GatedLinearAttention.forward
// (classification/models/vig.py:427-463).
#include <ATen/ATen.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/library.h>

#include <cmath>
#include <limits>
#include <tuple>

#include "../../include/vig_gla.h"

namespace {

using at::Tensor;
using c10::optional;

int dt(const Tensor& t) {
  if (t.scalar_type() == at::kFloat) return VIG_F32;
  if (t.scalar_type() == at::kBFloat16) return VIG_BF16;
  TORCH_CHECK(false, "vig_amd: unsupported dtype ", t.scalar_type(), "; float32 and bfloat16 are built");
}

void check_dev(const Tensor& t, const Tensor& ref, const char* name) {
  TORCH_CHECK(t.is_cuda(), "vig_amd: ", name, " must be a GPU tensor (there is no CPU path)");
  TORCH_CHECK(t.device() == ref.device(), "vig_amd: ", name, " is on ", t.device(), ", expected ", ref.device());
}

// dense row-major tensor on a 16-byte boundary (the kernels move 16 bytes per access)
void check_dense(const Tensor& t, const Tensor& ref, const char* name) {
  check_dev(t, ref, name);
  TORCH_CHECK(t.is_contiguous(), "vig_amd: ", name, " must be contiguous");
  TORCH_CHECK(reinterpret_cast<uintptr_t>(t.data_ptr()) % 16 == 0, "vig_amd: ", name, " must start on a 16-byte boundary");
}

void check_f32_vec(const Tensor& t, const Tensor& ref, int64_t n, const char* name) {
  check_dense(t, ref, name);
  TORCH_CHECK(t.scalar_type() == at::kFloat && t.numel() == n, "vig_amd: ", name, " must be float32 with ", n, " elements");
}

// [B, L, C] whose token rows may be a column block of a wider contiguous [B, L, W] tensor: returns the row stride
int64_t token_row_stride(const Tensor& t, const Tensor& ref, const char* name) {
  check_dev(t, ref, name);
  TORCH_CHECK(t.dim() == 3, "vig_amd: ", name, " must be [B, L, C]");
  const int64_t L = t.size(1), C = t.size(2), ld = t.stride(1);
  TORCH_CHECK(t.stride(2) == 1 && ld >= C && (t.size(0) == 1 || t.stride(0) == L * ld), "vig_amd: ", name,
              " must have contiguous token rows at a constant distance");
  TORCH_CHECK((ld * t.element_size()) % 16 == 0 && reinterpret_cast<uintptr_t>(t.data_ptr()) % 16 == 0, "vig_amd: ", name,
              ": token rows must keep 16-byte alignment");
  return ld;
}

void* stream_of(const Tensor& t) { return c10::hip::getCurrentHIPStream(t.device().index()).stream(); }

void check_rc(int rc, const char* what) {
  TORCH_CHECK(rc == VIG_OK, what, " failed: ", vig_gla_strerror(rc), " (code ", rc, ")");
}

Tensor workspace(size_t bytes, const Tensor& like) {
  return at::empty({static_cast<int64_t>(bytes ? bytes : 16)}, like.options().dtype(at::kByte));
}

float resolve_scale(double scale, int64_t Dk) { return scale < 0 ? 1.0f / std::sqrt((float)Dk) : (float)scale; }

struct GlaDims {
  int B, H, L, Dk, Dv;
};
GlaDims gla_check(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& gf, const optional<Tensor>& gb) {
  TORCH_CHECK(q.dim() == 4 && v.dim() == 4, "vig_amd: q, k, g must be [B,H,L,Dk] and v [B,H,L,Dv]");
  check_dense(q, q, "q");
  check_dense(k, q, "k");
  check_dense(v, q, "v");
  check_dense(gf, q, "g_fwd");
  TORCH_CHECK(k.sizes() == q.sizes() && gf.sizes() == q.sizes() && v.sizes().slice(0, 3) == q.sizes().slice(0, 3),
              "vig_amd: shape mismatch between q, k, v, g");
  TORCH_CHECK(k.scalar_type() == q.scalar_type() && v.scalar_type() == q.scalar_type(), "vig_amd: q, k, v must share a dtype");
  if (gb) {
    check_dense(*gb, q, "g_bwd");
    TORCH_CHECK(gb->sizes() == gf.sizes() && gb->scalar_type() == gf.scalar_type(), "vig_amd: g_bwd must match g_fwd");
  }
  return {(int)q.size(0), (int)q.size(1), (int)q.size(2), (int)q.size(3), (int)v.size(3)};
}

// mode 0: default dispatch, 1: wide-range scores first (strong gates), 2: fp32-arithmetic token-recurrent kernel
Tensor gla_bidir_fwd(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& g_fwd, const optional<Tensor>& g_bwd,
                     double scale, double out_scale, int64_t mode) {
  const GlaDims d = gla_check(q, k, v, g_fwd, g_bwd);
  const c10::DeviceGuard guard(q.device());
  Tensor o = at::empty({d.B, d.H, d.L, d.Dv}, q.options());
  const int io = dt(q), gd = dt(g_fwd);
  size_t need;
  if (mode == 2) need = (g_bwd && io != VIG_F32) ? (size_t)d.B * d.H * d.L * d.Dv * 4 : 0;
  else need = vig_gla_bidir_fwd_workspace_for(d.B, d.H, d.L, d.Dk, d.Dv, io, gd, g_bwd ? 1 : 0);
  Tensor ws;
  if (need) ws = workspace(need, q);
  auto fn = mode == 2 ? vig_gla_bidir_fwd_exact : (mode == 1 ? vig_gla_bidir_fwd_wide : vig_gla_bidir_fwd);
  check_rc(fn(q.data_ptr(), k.data_ptr(), v.data_ptr(), g_fwd.data_ptr(), g_bwd ? g_bwd->data_ptr() : nullptr, o.data_ptr(),
              need ? ws.data_ptr() : nullptr, need, d.B, d.H, d.L, d.Dk, d.Dv, resolve_scale(scale, d.Dk), (float)out_scale,
              io, gd, stream_of(q)),
           "vig_gla_bidir_fwd");
  return o;
}

Tensor gla_bidir_locgate_fwd(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& g_fwd, const Tensor& g_bwd,
                             const Tensor& weight, int64_t grid_h, int64_t grid_w, double scale, double out_scale) {
  const GlaDims d = gla_check(q, k, v, g_fwd, g_bwd);
  check_f32_vec(weight, q, (int64_t)d.H * d.Dv * 9, "weight");
  const c10::DeviceGuard guard(q.device());
  Tensor y = at::empty({d.B, d.H, d.L, d.Dv}, q.options());
  check_rc(vig_gla_bidir_locgate_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), g_fwd.data_ptr(), g_bwd.data_ptr(),
                                     weight.data_ptr<float>(), y.data_ptr(), d.B, d.H, d.L, d.Dk, d.Dv, (int)grid_h,
                                     (int)grid_w, resolve_scale(scale, d.Dk), (float)out_scale, dt(q), dt(g_fwd),
                                     stream_of(q)),
           "vig_gla_bidir_locgate_fwd");
  return y;
}

std::tuple<Tensor, optional<Tensor>> gla_causal_state_fwd(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& g,
                                                const optional<Tensor>& initial_state, bool output_final_state,
                                                double scale, bool exact) {
  const GlaDims d = gla_check(q, k, v, g, c10::nullopt);
  if (initial_state) {
    check_dense(*initial_state, q, "initial_state");
    TORCH_CHECK(initial_state->scalar_type() == at::kFloat && initial_state->dim() == 4 &&
                    initial_state->size(0) == d.B && initial_state->size(1) == d.H &&
                    initial_state->size(2) == d.Dk && initial_state->size(3) == d.Dv,
                "vig_amd: initial_state must be float32 [B,H,Dk,Dv]");
  }
  const c10::DeviceGuard guard(q.device());
  Tensor o = at::empty({d.B, d.H, d.L, d.Dv}, q.options());
  optional<Tensor> fin;
  if (output_final_state) fin = at::empty({d.B, d.H, d.Dk, d.Dv}, q.options().dtype(at::kFloat));
  const float* s0 = initial_state ? initial_state->data_ptr<float>() : nullptr;
  float* s1 = output_final_state ? fin->data_ptr<float>() : nullptr;
  const int io = dt(q), gd = dt(g);
  if (exact) {
    check_rc(vig_gla_causal_state_fwd_exact(q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(), o.data_ptr(), s0, s1,
                                            d.B, d.H, d.L, d.Dk, d.Dv, resolve_scale(scale, d.Dk), 1.0f, io, gd,
                                            stream_of(q)),
             "vig_gla_causal_state_fwd_exact");
  } else {
    const size_t need = vig_gla_causal_state_fwd_workspace(d.B, d.H, d.L, d.Dk, d.Dv, io, gd);
    Tensor ws;
    if (need) ws = workspace(need, q);
    check_rc(vig_gla_causal_state_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(), o.data_ptr(), s0, s1,
                                      need ? ws.data_ptr() : nullptr, need, d.B, d.H, d.L, d.Dk, d.Dv,
                                      resolve_scale(scale, d.Dk), 1.0f, io, gd, stream_of(q)),
             "vig_gla_causal_state_fwd");
  }
  return {o, fin};
}

std::tuple<Tensor, Tensor, Tensor, Tensor, optional<Tensor>> gla_bidir_bwd(const Tensor& q, const Tensor& k, const Tensor& v,
                                                                 const Tensor& g_fwd, const optional<Tensor>& g_bwd,
                                                                 const Tensor& d_o, double scale, double out_scale,
                                                                 bool exact) {
  const GlaDims d = gla_check(q, k, v, g_fwd, g_bwd);
  check_dense(d_o, q, "d_o");
  TORCH_CHECK(d_o.sizes() == v.sizes() && d_o.scalar_type() == q.scalar_type(), "vig_amd: d_o must match the output");
  const c10::DeviceGuard guard(q.device());
  Tensor dq = at::empty_like(q), dk = at::empty_like(k), dv = at::empty_like(v), dgf = at::empty_like(g_fwd);
  optional<Tensor> dgb;
  if (g_bwd) dgb = at::empty_like(*g_bwd);
  const size_t need = exact ? vig_gla_bidir_bwd_workspace(d.B, d.H, d.L, d.Dk, d.Dv, g_bwd ? 1 : 0)
                            : vig_gla_bidir_bwd_workspace_for(d.B, d.H, d.L, d.Dk, d.Dv, dt(q), dt(g_fwd), g_bwd ? 1 : 0);
  TORCH_CHECK(need > 0, "vig_gla_bidir_bwd: shape Dk=", d.Dk, ", Dv=", d.Dv, " is not built");
  Tensor ws = workspace(need, q);
  auto fn = exact ? vig_gla_bidir_bwd_exact : vig_gla_bidir_bwd;
  check_rc(fn(q.data_ptr(), k.data_ptr(), v.data_ptr(), g_fwd.data_ptr(), g_bwd ? g_bwd->data_ptr() : nullptr,
              d_o.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dgf.data_ptr(),
              g_bwd ? dgb->data_ptr() : nullptr, ws.data_ptr(), need, d.B, d.H, d.L, d.Dk, d.Dv,
              resolve_scale(scale, d.Dk), (float)out_scale, dt(q), dt(g_fwd), stream_of(q)),
           "vig_gla_bidir_bwd");
  return {dq, dk, dv, dgf, dgb};
}

float clamp_arg(const optional<double>& c) { return c ? (float)*c : std::numeric_limits<float>::quiet_NaN(); }

Tensor dirgate_fwd(const Tensor& gk_lin, int64_t H, double normalizer, const optional<double>& clamp_min) {
  TORCH_CHECK(gk_lin.dim() == 3, "vig_amd: gk_lin must be [B, L, 2*H*Dk]");
  check_dense(gk_lin, gk_lin, "gk_lin");
  const int64_t B = gk_lin.size(0), L = gk_lin.size(1), C2 = gk_lin.size(2);
  TORCH_CHECK(H > 0 && C2 % (2 * H) == 0, "vig_amd: last dimension must be 2*H*Dk");
  const int64_t Dk = C2 / (2 * H);
  const c10::DeviceGuard guard(gk_lin.device());
  Tensor out = at::empty({2, B, H, L, Dk}, gk_lin.options());
  check_rc(vig_dirgate_fwd(gk_lin.data_ptr(), out.data_ptr(), (int)B, (int)L, (int)H, (int)Dk, (float)(1.0 / normalizer),
                           clamp_arg(clamp_min), dt(gk_lin), dt(out), stream_of(gk_lin)),
           "vig_dirgate_fwd");
  return out;
}

Tensor dirgate_lowrank_fwd(const Tensor& gk_low, const Tensor& w_up, const Tensor& b_up, int64_t H, double normalizer,
                           const optional<double>& clamp_min) {
  const int64_t ld = token_row_stride(gk_low, gk_low, "gk_low");
  check_dense(w_up, gk_low, "w_up");
  check_dense(b_up, gk_low, "b_up");
  const int64_t B = gk_low.size(0), L = gk_low.size(1), R = gk_low.size(2), C2 = w_up.size(0);
  TORCH_CHECK(w_up.dim() == 2 && w_up.size(1) == R && b_up.numel() == C2 && H > 0 && C2 % (2 * H) == 0,
              "vig_amd: w_up must be [2*H*Dk, rank] and b_up [2*H*Dk]");
  TORCH_CHECK(w_up.scalar_type() == gk_low.scalar_type() && b_up.scalar_type() == gk_low.scalar_type(),
              "vig_amd: gk_low, w_up and b_up must share a dtype");
  const int64_t Dk = C2 / (2 * H);
  const c10::DeviceGuard guard(gk_low.device());
  Tensor out = at::empty({2, B, H, L, Dk}, gk_low.options());
  check_rc(vig_dirgate_lowrank_fwd(gk_low.data_ptr(), ld, w_up.data_ptr(), b_up.data_ptr(), out.data_ptr(), (int)B, (int)L,
                                   (int)H, (int)Dk, (int)R, (float)(1.0 / normalizer), clamp_arg(clamp_min), dt(gk_low),
                                   dt(out), stream_of(gk_low)),
           "vig_dirgate_lowrank_fwd");
  return out;
}

Tensor dwconv3x3_fwd(const Tensor& x, const Tensor& weight, const optional<Tensor>& bias, int64_t h, int64_t w, bool silu) {
  TORCH_CHECK(x.dim() == 3 && x.size(1) == h * w, "vig_amd: x must be [B, h*w, C]");
  check_dense(x, x, "x");
  const int64_t C = x.size(2);
  check_f32_vec(weight, x, C * 9, "weight");
  if (bias) check_f32_vec(*bias, x, C, "bias");
  const c10::DeviceGuard guard(x.device());
  Tensor y = at::empty_like(x);
  check_rc(vig_dwconv3x3_fwd(x.data_ptr(), weight.data_ptr<float>(), bias ? bias->data_ptr<float>() : nullptr, y.data_ptr(),
                             (int)x.size(0), (int)h, (int)w, (int)C, silu ? 1 : 0, dt(x), stream_of(x)),
           "vig_dwconv3x3_fwd");
  return y;
}

Tensor locality_gate_fwd(const Tensor& o, const Tensor& weight, int64_t h, int64_t w) {
  TORCH_CHECK(o.dim() == 4 && o.size(2) == h * w, "vig_amd: o must be [B, H, h*w, Dv]");
  check_dense(o, o, "o");
  check_f32_vec(weight, o, o.size(1) * o.size(3) * 9, "weight");
  const c10::DeviceGuard guard(o.device());
  Tensor y = at::empty_like(o);
  check_rc(vig_locality_gate_fwd(o.data_ptr(), weight.data_ptr<float>(), y.data_ptr(), (int)o.size(0), (int)o.size(1), (int)h,
                                 (int)w, (int)o.size(3), dt(o), stream_of(o)),
           "vig_locality_gate_fwd");
  return y;
}

// o_proj(locality_blend(...)) in one kernel where the library builds it (bf16, 64-channel heads, square o_proj of
// width 384 or 192); the two steps otherwise.
Tensor locality_blend_fwd(const Tensor& o, const Tensor& local, const Tensor& g_lin, const Tensor& w_g, const Tensor& w_l,
                          double eps, bool silu_out);
Tensor locality_blend_linear_fwd(const Tensor& o, const Tensor& local, const Tensor& g_lin, const Tensor& w_g,
                                 const Tensor& w_l, const Tensor& weight, double eps, bool silu_out) {
  TORCH_CHECK(o.dim() == 4 && weight.dim() == 2, "vig_amd: o must be [B, H, L, Dv], weight [C, H*Dv]");
  const int64_t B = o.size(0), H = o.size(1), L = o.size(2), Dv = o.size(3), C = weight.size(0);
  const bool fused = o.scalar_type() == at::kBFloat16 && weight.scalar_type() == at::kBFloat16 && Dv == 64 &&
                     weight.size(1) == H * Dv && C == H * Dv && (C == 384 || C == 192) && weight.is_contiguous() &&
                     reinterpret_cast<uintptr_t>(weight.data_ptr()) % 16 == 0;
  if (!fused) return at::linear(locality_blend_fwd(o, local, g_lin, w_g, w_l, eps, silu_out), weight);
  check_dense(o, o, "o");
  check_dense(local, o, "local");
  const int64_t ldg = token_row_stride(g_lin, o, "g_lin");
  TORCH_CHECK(local.dim() == 3 && local.size(0) == B && local.size(1) == L && local.size(2) == H * Dv &&
                  g_lin.size(0) == B && g_lin.size(1) == L && g_lin.size(2) == H * Dv,
              "vig_amd: local and g_lin must be [B, L, H*Dv]");
  TORCH_CHECK(local.scalar_type() == o.scalar_type() && g_lin.scalar_type() == o.scalar_type(),
              "vig_amd: o, local, g_lin must share a dtype");
  check_f32_vec(w_g, o, Dv, "w_g");
  check_f32_vec(w_l, o, Dv, "w_l");
  const c10::DeviceGuard guard(o.device());
  Tensor out = at::empty({B, L, C}, o.options());
  check_rc(vig_locality_blend_linear_fwd(o.data_ptr(), local.data_ptr(), g_lin.data_ptr(), w_g.data_ptr<float>(),
                                         w_l.data_ptr<float>(), weight.data_ptr(), out.data_ptr(), (int)B, (int)H, (int)L,
                                         (int)Dv, (int)C, ldg, (float)eps, silu_out ? 1 : 0, dt(o), stream_of(o)),
           "vig_locality_blend_linear_fwd");
  return out;
}

Tensor locality_blend_fwd(const Tensor& o, const Tensor& local, const Tensor& g_lin, const Tensor& w_g, const Tensor& w_l,
                          double eps, bool silu_out) {
  TORCH_CHECK(o.dim() == 4, "vig_amd: o must be [B, H, L, Dv]");
  check_dense(o, o, "o");
  check_dense(local, o, "local");
  const int64_t B = o.size(0), H = o.size(1), L = o.size(2), Dv = o.size(3);
  const int64_t ldg = token_row_stride(g_lin, o, "g_lin");
  TORCH_CHECK(local.dim() == 3 && local.size(0) == B && local.size(1) == L && local.size(2) == H * Dv &&
                  g_lin.size(0) == B && g_lin.size(1) == L && g_lin.size(2) == H * Dv,
              "vig_amd: local and g_lin must be [B, L, H*Dv]");
  TORCH_CHECK(local.scalar_type() == o.scalar_type() && g_lin.scalar_type() == o.scalar_type(),
              "vig_amd: o, local, g_lin must share a dtype");
  check_f32_vec(w_g, o, Dv, "w_g");
  check_f32_vec(w_l, o, Dv, "w_l");
  const c10::DeviceGuard guard(o.device());
  Tensor y = at::empty_like(local);
  check_rc(vig_locality_blend_fwd(o.data_ptr(), local.data_ptr(), g_lin.data_ptr(), w_g.data_ptr<float>(),
                                  w_l.data_ptr<float>(), y.data_ptr(), (int)B, (int)H, (int)L, (int)Dv, ldg, (float)eps,
                                  silu_out ? 1 : 0, dt(o), stream_of(o)),
           "vig_locality_blend_fwd");
  return y;
}

// returns (y, sum): sum = x + residual when a residual is given, else nothing (the sum is x itself)
std::tuple<Tensor, optional<Tensor>> rmsnorm_fwd(const Tensor& x, const optional<Tensor>& residual, const Tensor& weight, double eps,
                                       bool round_sum) {
  check_dense(x, x, "x");
  const int64_t C = x.size(-1), rows = x.numel() / C;
  check_f32_vec(weight, x, C, "weight");
  if (residual) {
    check_dense(*residual, x, "residual");
    TORCH_CHECK(residual->sizes() == x.sizes() && residual->scalar_type() == x.scalar_type(),
                "vig_amd: residual must match x in shape and dtype");
  }
  const c10::DeviceGuard guard(x.device());
  Tensor y = at::empty_like(x);
  optional<Tensor> sum;
  if (residual) sum = at::empty_like(x);
  check_rc(vig_rmsnorm_fwd(x.data_ptr(), residual ? residual->data_ptr() : nullptr, weight.data_ptr<float>(), y.data_ptr(),
                           residual ? sum->data_ptr() : nullptr, rows, (int)C, (float)eps, round_sum ? 1 : 0, dt(x),
                           stream_of(x)),
           "vig_rmsnorm_fwd");
  return {y, sum};
}

Tensor layernorm_fwd(const Tensor& x, const Tensor& weight, const Tensor& bias, double eps, bool silu,
                     const optional<Tensor>& pre_bias, const optional<Tensor>& post_add) {
  check_dense(x, x, "x");
  const int64_t C = x.size(-1), rows = x.numel() / C;
  check_f32_vec(weight, x, C, "weight");
  check_f32_vec(bias, x, C, "bias");
  if (pre_bias) check_f32_vec(*pre_bias, x, C, "pre_bias");
  int64_t prow = 0;
  if (post_add) {
    check_dense(*post_add, x, "post_add");
    TORCH_CHECK(post_add->scalar_type() == x.scalar_type() && post_add->numel() % C == 0, "vig_amd: post_add must be [P, C] in x's dtype");
    prow = post_add->numel() / C;
    TORCH_CHECK(prow > 0 && rows % prow == 0, "vig_amd: post_add's row count must divide x's");
  }
  const c10::DeviceGuard guard(x.device());
  Tensor y = at::empty_like(x);
  check_rc(vig_layernorm_fwd(x.data_ptr(), weight.data_ptr<float>(), bias.data_ptr<float>(), y.data_ptr(), rows, (int)C,
                             (float)eps, silu ? 1 : 0, pre_bias ? pre_bias->data_ptr<float>() : nullptr,
                             post_add ? post_add->data_ptr() : nullptr, (int)prow, dt(x), stream_of(x)),
           "vig_layernorm_fwd");
  return y;
}

std::tuple<Tensor, Tensor, Tensor> split_heads_fwd(const Tensor& qkv, int64_t H, int64_t Dk, int64_t Dv) {
  const int64_t ld = token_row_stride(qkv, qkv, "qkv");
  const int64_t B = qkv.size(0), L = qkv.size(1);
  TORCH_CHECK(qkv.size(2) == H * (2 * Dk + Dv), "vig_amd: last dimension must be H*(2*Dk+Dv)");
  const c10::DeviceGuard guard(qkv.device());
  Tensor q = at::empty({B, H, L, Dk}, qkv.options()), k = at::empty({B, H, L, Dk}, qkv.options());
  Tensor v = at::empty({B, H, L, Dv}, qkv.options());
  check_rc(vig_split_heads_fwd(qkv.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), (int)B, (int)L, (int)H, (int)Dk,
                               (int)Dv, ld, dt(qkv), stream_of(qkv)),
           "vig_split_heads_fwd");
  return {q, k, v};
}

Tensor swiglu_fwd(const Tensor& gate_up) {
  check_dense(gate_up, gate_up, "gate_up");
  const int64_t I = gate_up.size(-1) / 2, rows = gate_up.numel() / (2 * I);
  const c10::DeviceGuard guard(gate_up.device());
  auto shape = gate_up.sizes().vec();
  shape.back() = I;
  Tensor out = at::empty(shape, gate_up.options());
  check_rc(vig_swiglu_fwd(gate_up.data_ptr(), out.data_ptr(), rows, (int)I, dt(gate_up), stream_of(gate_up)), "vig_swiglu_fwd");
  return out;
}

Tensor linear_swiglu_fwd(const Tensor& x, const Tensor& weight) {
  check_dense(x, x, "x");
  check_dense(weight, x, "weight");
  TORCH_CHECK(weight.dim() == 2 && weight.size(1) == x.size(-1) && weight.scalar_type() == x.scalar_type(),
              "vig_amd: weight must be [2*I, K] in x's dtype");
  const int64_t K = weight.size(1), I = weight.size(0) / 2;
  const c10::DeviceGuard guard(x.device());
  auto shape = x.sizes().vec();
  shape.back() = I;
  Tensor y = at::empty(shape, x.options());
  check_rc(vig_linear_swiglu_fwd(x.data_ptr(), weight.data_ptr(), y.data_ptr(), x.numel() / K, (int)K, (int)I, dt(x),
                                 stream_of(x)),
           "vig_linear_swiglu_fwd");
  return y;
}

Tensor patch_conv_fwd(const Tensor& x, const Tensor& w_packed, int64_t KH, int64_t KW, int64_t stride, int64_t padding) {
  TORCH_CHECK(x.dim() == 4 && w_packed.dim() == 3, "vig_amd: x must be [B, Cin, H, W] and w_packed [Cout, Cin*KH, 16]");
  check_dense(x, x, "x");
  check_dense(w_packed, x, "w_packed");
  const int64_t B = x.size(0), Cin = x.size(1), H = x.size(2), W = x.size(3), Cout = w_packed.size(0);
  TORCH_CHECK(w_packed.size(1) == Cin * KH && w_packed.size(2) == 16 && w_packed.scalar_type() == x.scalar_type(),
              "vig_amd: w_packed must be [Cout, Cin*KH, 16] in x's dtype");
  const int64_t OH = (H + 2 * padding - KH) / stride + 1, OW = (W + 2 * padding - KW) / stride + 1;
  const c10::DeviceGuard guard(x.device());
  Tensor y = at::empty({B, OH, OW, Cout}, x.options());
  check_rc(vig_patch_conv_fwd(x.data_ptr(), w_packed.data_ptr(), y.data_ptr(), (int)B, (int)Cin, (int)H, (int)W, (int)KH,
                              (int)KW, (int)stride, (int)padding, (int)Cout, dt(x), stream_of(x)),
           "vig_patch_conv_fwd");
  return y;
}

// Eval-mode token mixer of one GLA block on x [B, L, C] (classification/models/vig.py:427-463), every step between the
// projections on the library's kernels: depthwise conv, ONE stacked projection (qkv | g | low-rank gate rows, as the
// caller stacked them), head split, gate preparation with the rank-16 up-projection inside, the bidirectional GLA,
// both head norms + sigmoid blend, o_proj.  One operator call per block instead of eight.
Tensor gla_block_mix(const Tensor& x, int64_t grid_h, int64_t grid_w, const Tensor& conv_w, const optional<Tensor>& conv_b,
                     bool act_in_conv, const Tensor& w_in, const Tensor& b_in, int64_t H, int64_t Dk, int64_t Dv,
                     const Tensor& w_up, const Tensor& b_up, double normalizer, const optional<double>& clamp_min,
                     const Tensor& w_gnorm, const Tensor& w_lnorm, double eps, bool out_act, const Tensor& w_o,
                     double out_scale) {
  Tensor xs = dwconv3x3_fwd(x, conv_w, conv_b, grid_h, grid_w, act_in_conv);
  Tensor z = at::linear(xs, w_in, b_in);
  const int64_t n0 = H * (2 * Dk + Dv), n1 = n0 + H * Dv, rank = w_up.size(1);
  TORCH_CHECK(z.size(-1) >= n1 + rank, "vig_amd: stacked projection is narrower than qkv | g | gate rows");
  Tensor gates = dirgate_lowrank_fwd(z.narrow(-1, n1, rank), w_up, b_up, H, normalizer, clamp_min);
  Tensor o;
  const int64_t B = z.size(0), L = z.size(1), ld = z.size(-1);
  if (z.scalar_type() == at::kBFloat16 && gates.scalar_type() == at::kBFloat16 && L <= 256 && (Dk == 32 || Dk == 64) &&
      Dv == 64 && ld % 8 == 0 && z.is_contiguous() && reinterpret_cast<uintptr_t>(z.data_ptr()) % 16 == 0) {
    // the matrix-core slab kernel reads q, k, v in place from the projection's rows: no head-major copies
    const c10::DeviceGuard guard(z.device());
    o = at::empty({B, H, L, Dv}, z.options());
    const long long sqk[3] = {(long long)(L * ld), (long long)Dk, (long long)ld};
    const long long sv[3] = {(long long)(L * ld), (long long)Dv, (long long)ld};
    const auto* base = static_cast<const at::BFloat16*>(z.data_ptr());
    Tensor gf = gates.select(0, 0), gb = gates.select(0, 1);
    check_rc(vig_gla_bidir_fwd_strided(base, base + H * Dk, base + 2 * H * Dk, gf.data_ptr(), gb.data_ptr(), o.data_ptr(),
                                       (int)B, (int)H, (int)L, (int)Dk, (int)Dv, sqk, sqk, sv,
                                       resolve_scale(-1.0, (int)Dk), (float)out_scale, VIG_BF16, VIG_BF16, stream_of(z)),
             "vig_gla_bidir_fwd_strided");
  } else {
    auto qkv = split_heads_fwd(z.narrow(-1, 0, n0), H, Dk, Dv);
    o = gla_bidir_fwd(std::get<0>(qkv), std::get<1>(qkv), std::get<2>(qkv), gates.select(0, 0), gates.select(0, 1), -1.0,
                      out_scale, 0);
  }
  return locality_blend_linear_fwd(o, xs, z.narrow(-1, n0, H * Dv), w_gnorm, w_lnorm, w_o, eps, out_act);
}

// One eval-mode GLA block in the carried form (classification/models/vig.py:582-608 with the closing residual add of
// the previous block folded into this block's first norm): takes (branch, residual) with hidden = residual + branch
// and returns the next such pair.  attn_norm -> mixer -> residual add + mlp_norm (prenorm) -> gate_proj + SwiGLU ->
// down_proj, one operator call per block.
std::tuple<Tensor, Tensor> gla_block_carry(const Tensor& branch, const optional<Tensor>& residual, const Tensor& w_attn_norm,
                                           double norm_eps, int64_t grid_h, int64_t grid_w, const Tensor& conv_w,
                                           const optional<Tensor>& conv_b, bool act_in_conv, const Tensor& w_in,
                                           const Tensor& b_in, int64_t H, int64_t Dk, int64_t Dv, const Tensor& w_up,
                                           const Tensor& b_up, double normalizer, const optional<double>& clamp_min,
                                           const Tensor& w_gnorm, const Tensor& w_lnorm, double eps, bool out_act,
                                           const Tensor& w_o, double out_scale, const Tensor& w_mlp_norm,
                                           const Tensor& w_gate, const Tensor& w_down) {
  // the explicit add of the reference stores a rounded sum and attn_norm normalises that (vig.py:598,606)
  auto n1 = rmsnorm_fwd(branch, residual, w_attn_norm, norm_eps, true);
  const Tensor hidden = std::get<1>(n1) ? *std::get<1>(n1) : branch;
  Tensor a = gla_block_mix(std::get<0>(n1), grid_h, grid_w, conv_w, conv_b, act_in_conv, w_in, b_in, H, Dk, Dv, w_up, b_up,
                           normalizer, clamp_min, w_gnorm, w_lnorm, eps, out_act, w_o, out_scale);
  auto n2 = rmsnorm_fwd(a, hidden, w_mlp_norm, norm_eps, false);
  const Tensor& h = std::get<0>(n2);
  const int64_t K = w_gate.size(1), I = w_gate.size(0) / 2;
  Tensor m;
  if (h.scalar_type() == at::kBFloat16 && w_gate.scalar_type() == at::kBFloat16 && (K == 384 || K == 192) && I % 32 == 0)
    m = linear_swiglu_fwd(h, w_gate);  // no [.., 2*I] intermediate
  else
    m = swiglu_fwd(at::linear(h, w_gate));
  return {at::linear(m, w_down), *std::get<1>(n2)};
}

}  // namespace

TORCH_LIBRARY(vig_amd, m) {
  m.def("gla_bidir_fwd(Tensor q, Tensor k, Tensor v, Tensor g_fwd, Tensor? g_bwd, float scale, float out_scale, int mode) -> Tensor",
        &gla_bidir_fwd);
  m.def("gla_bidir_locgate_fwd(Tensor q, Tensor k, Tensor v, Tensor g_fwd, Tensor g_bwd, Tensor weight, int grid_h, int grid_w, float scale, float out_scale) -> Tensor",
        &gla_bidir_locgate_fwd);
  m.def("gla_causal_state_fwd(Tensor q, Tensor k, Tensor v, Tensor g, Tensor? initial_state, bool output_final_state, float scale, bool exact) -> (Tensor, Tensor?)",
        &gla_causal_state_fwd);
  m.def("gla_bidir_bwd(Tensor q, Tensor k, Tensor v, Tensor g_fwd, Tensor? g_bwd, Tensor d_o, float scale, float out_scale, bool exact) -> (Tensor, Tensor, Tensor, Tensor, Tensor?)",
        &gla_bidir_bwd);
  m.def("dirgate_fwd(Tensor gk_lin, int num_heads, float normalizer, float? clamp_min) -> Tensor", &dirgate_fwd);
  m.def("dirgate_lowrank_fwd(Tensor gk_low, Tensor w_up, Tensor b_up, int num_heads, float normalizer, float? clamp_min) -> Tensor",
        &dirgate_lowrank_fwd);
  m.def("dwconv3x3_fwd(Tensor x, Tensor weight, Tensor? bias, int h, int w, bool silu) -> Tensor", &dwconv3x3_fwd);
  m.def("locality_gate_fwd(Tensor o, Tensor weight, int h, int w) -> Tensor", &locality_gate_fwd);
  m.def("locality_blend_fwd(Tensor o, Tensor local, Tensor g_lin, Tensor w_g, Tensor w_l, float eps, bool silu_out) -> Tensor",
        &locality_blend_fwd);
  m.def("rmsnorm_fwd(Tensor x, Tensor? residual, Tensor weight, float eps, bool round_sum) -> (Tensor, Tensor?)", &rmsnorm_fwd);
  m.def("layernorm_fwd(Tensor x, Tensor weight, Tensor bias, float eps, bool silu, Tensor? pre_bias, Tensor? post_add) -> Tensor",
        &layernorm_fwd);
  m.def("split_heads_fwd(Tensor qkv, int num_heads, int head_qk_dim, int head_v_dim) -> (Tensor, Tensor, Tensor)",
        &split_heads_fwd);
  m.def("swiglu_fwd(Tensor gate_up) -> Tensor", &swiglu_fwd);
  m.def("linear_swiglu_fwd(Tensor x, Tensor weight) -> Tensor", &linear_swiglu_fwd);
  m.def("locality_blend_linear_fwd(Tensor o, Tensor local, Tensor g_lin, Tensor w_g, Tensor w_l, Tensor weight, float eps, "
        "bool silu_out) -> Tensor",
        &locality_blend_linear_fwd);
  m.def("patch_conv_fwd(Tensor x, Tensor w_packed, int kh, int kw, int stride, int padding) -> Tensor", &patch_conv_fwd);
  m.def("gla_block_mix(Tensor x, int grid_h, int grid_w, Tensor conv_w, Tensor? conv_b, bool act_in_conv, Tensor w_in, Tensor b_in, int num_heads, int head_qk_dim, int head_v_dim, Tensor w_up, Tensor b_up, float normalizer, float? clamp_min, Tensor w_gnorm, Tensor w_lnorm, float eps, bool out_act, Tensor w_o, float out_scale) -> Tensor",
        &gla_block_mix);
  m.def("gla_block_carry(Tensor branch, Tensor? residual, Tensor w_attn_norm, float norm_eps, int grid_h, int grid_w, Tensor conv_w, Tensor? conv_b, bool act_in_conv, Tensor w_in, Tensor b_in, int num_heads, int head_qk_dim, int head_v_dim, Tensor w_up, Tensor b_up, float normalizer, float? clamp_min, Tensor w_gnorm, Tensor w_lnorm, float eps, bool out_act, Tensor w_o, float out_scale, Tensor w_mlp_norm, Tensor w_gate, Tensor w_down) -> (Tensor, Tensor)",
        &gla_block_carry);
}
