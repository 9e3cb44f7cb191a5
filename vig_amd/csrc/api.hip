// C ABI of the library (declared in include/vig_gla.h): argument validation and
// dispatch only.  Nothing here allocates, frees or synchronises.
#include "../../include/vig_gla.h"
#include "launch.h"
#include <mutex>

namespace vig {
int launch_dirgate(const void* in, void* out, int B, int L, int H, int Dk, float inv_norm, float clamp_min,
                   int in_dtype, int out_dtype, hipStream_t stream);
int launch_dirgate_bwd(const void* in, const void* d_out, void* d_in, int B, int L, int H, int Dk, float inv_norm,
                       float clamp_min, int in_dtype, int out_dtype, hipStream_t stream);
int launch_merge_heads(const void* dq, const void* dk, const void* dv, void* dqkv, int B, int L, int H, int Dk, int Dv,
                       int io_dtype, hipStream_t stream);
size_t dwconv3x3_wgrad_workspace(int B, int C);
int launch_dwconv3x3_wgrad(const void* x, const void* dy, float* dw_db, void* workspace, int B, int h, int w, int C,
                           int io_dtype, hipStream_t stream);
int launch_dwconv3x3(const void* x, const float* wt, const float* bias, void* y, int B, int h, int w, int C,
                     int silu, int io_dtype, hipStream_t stream);
int launch_dirgate_lowrank(const void* low, long long ld, const void* w1, const void* b1, void* out, int B, int L,
                           int H, int Dk, int rank, float inv_norm, float clamp_min, int in_dtype, int out_dtype,
                           hipStream_t stream);
int launch_locality_gate(const void* o, const float* wt, void* y, int B, int H, int h, int w, int Dv, int io_dtype,
                         hipStream_t stream);
int launch_locality_blend(const void* o, const void* loc, const void* glin, const float* wg, const float* wl, void* y,
                          int B, int H, int L, int Dv, long long ldg, float eps, int silu_out, int io_dtype,
                          hipStream_t stream);
size_t locality_blend_bwd_workspace(int B, int L, int Dv);
int launch_locality_blend_bwd(const void* o, const void* loc, const void* glin, const float* wg, const float* wl,
                              const void* dy, void* d_o, void* d_loc, void* d_glin, float* dw, void* workspace, int B,
                              int H, int L, int Dv, long long ldg, float eps, int silu_out, int io_dtype,
                              hipStream_t stream);
int launch_rmsnorm(const void* x, const void* residual, const float* weight, void* y, void* residual_out, int rows,
                   int C, float eps, int round_sum, int io_dtype, hipStream_t stream);
int launch_layernorm(const void* x, const float* weight, const float* bias, void* y, long long rows, int C, float eps,
                     int silu, const float* pre_bias, const void* post_add, int post_rows, int io_dtype,
                     hipStream_t stream);
int launch_split_heads(const void* qkv, void* q, void* k, void* v, int B, int L, int H, int Dk, int Dv, long long ld,
                       int io_dtype, hipStream_t stream);
int launch_swiglu(const void* in, void* out, long long rows, int I, int io_dtype, hipStream_t stream);
int launch_swiglu_bwd(const void* in, const void* dy, void* din, long long rows, int I, int io_dtype,
                      hipStream_t stream);
size_t rmsnorm_bwd_workspace(long long rows, int C);
int launch_rmsnorm_bwd(const void* s, const float* weight, const void* dy, const void* d_sum, void* ds, float* dweight,
                       void* workspace, long long rows, int C, float eps, int io_dtype, hipStream_t stream);
bool blend_linear_supported(int H, int Dv, int C);
int launch_blend_linear(const void* o, const void* loc, const void* glin, const float* w_g, const float* w_l,
                        const void* W, void* out, int B, int H, int L, int Dv, int C, long long ldg, float eps,
                        int silu_out, hipStream_t stream);
bool linear_swiglu_supported(int K, int I);
int launch_linear_swiglu(const void* A, const void* W, void* out, long long T, int K, int I, hipStream_t stream);
bool patch_conv_supported(int Cin, int H, int W, int KH, int KW, int stride, int padding, int Cout);
int launch_patch_conv(const void* x, const void* w_packed, void* y, int B, int Cin, int H, int W, int KH, int KW,
                      int Cout, hipStream_t stream);
int launch_pad_channels(const void* src, void* dst, long long rows, int src_c, int dst_c, hipStream_t stream);
int launch_pad_channels_multi(const void* const* src, void* const* dst, const int* src_c, const int* dst_c, int n,
                              long long rows, hipStream_t stream);
int launch_gla_backward(const void* q, const void* k, const void* v, const void* g_fwd, const void* g_bwd,
                        const void* d_o, void* dq, void* dk, void* dv, void* dg_fwd, void* dg_bwd, void* workspace,
                        int B, int H, int L, int Dk, int Dv, float scale, float out_scale, int io_dtype,
                        int gate_dtype, bool exact, hipStream_t stream);
size_t gla_backward_workspace(int B, int H, int L, int Dk, int Dv, int bidir);
}  // namespace vig

static bool dtype_ok(int d) { return d == VIG_F32 || d == VIG_BF16; }

// rows read with 16-byte vector loads: the base and the distance between rows have to keep that alignment
static bool strided_rows_ok(const void* base, long long ld_elems, int dtype) {
  const long long elem = dtype == VIG_BF16 ? 2 : 4;
  return (reinterpret_cast<uintptr_t>(base) % 16) == 0 && (ld_elems * elem) % 16 == 0;
}
// every tensor is moved 16 bytes per access: a pointer off that boundary is refused (null, for an optional tensor, passes)
template <typename... P>
static bool aligned16(P... p) {
  return ((reinterpret_cast<uintptr_t>(static_cast<const void*>(p)) % 16 == 0) && ...);
}
static bool dk_ok(int d) { return d == 16 || d == 32 || d == 64 || d == 128; }
static bool dv_ok(int d) { return d == 32 || d == 64 || d == 128; }

extern "C" {

const char* vig_gla_version(void) { return "vig_gla 0.1 gfx950"; }

const char* vig_gla_strerror(int code) {
  switch (code) {
    case VIG_OK: return "ok";
    case VIG_EINVAL: return "invalid argument";
    case VIG_ENOTSUP: return "shape or dtype combination not built";
    case VIG_ENOSPC: return "workspace too small";
    case VIG_ELAUNCH: return "HIP launch error";
    default: return "unknown error";
  }
}

static int fill_args(vig::GlaArgs& a, const void* q, const void* k, const void* v, const void* g_fwd,
                     const void* g_bwd, void* o, void* workspace, size_t workspace_bytes, int B, int H, int L,
                     int Dk, int Dv, float scale, float out_scale, int io_dtype, int gate_dtype, void* stream) {
  if (!q || !k || !v || !g_fwd || !o) return VIG_EINVAL;
  if (!aligned16(q, k, v, g_fwd, g_bwd, o, workspace)) return VIG_EINVAL;
  if (B <= 0 || H <= 0 || L <= 0) return VIG_EINVAL;
  if ((long long)B * H > 2147483647LL) return VIG_EINVAL;
  if (!dtype_ok(io_dtype) || !dtype_ok(gate_dtype)) return VIG_ENOTSUP;
  if (!dk_ok(Dk) || !dv_ok(Dv)) return VIG_ENOTSUP;
  a = vig::GlaArgs{q, k, v, g_fwd, g_bwd, o, workspace, workspace_bytes, B, H, L, Dk, Dv,
                   scale, out_scale, io_dtype, gate_dtype, (hipStream_t)stream};
  return VIG_OK;
}

// HierViG's head shape (Dk 16, Dv 32) rides the matrix-core kernel zero-padded to Dk 32 / Dv 64 once the sequence is
// long enough for that to beat the token-recurrent kernel (measured: 1.5x at L = 196, 10x at L = 3136).
constexpr int kPadMinL = 128;
static bool padded_shape(int L, int Dk, int Dv, int io_dtype, int gate_dtype, bool bidir) {
  return bidir && io_dtype == VIG_BF16 && gate_dtype == VIG_BF16 && Dk == 16 && Dv == 32 && L >= kPadMinL;
}
static size_t padded_elems_qk(int B, int H, int L) { return (size_t)B * H * L * 32; }
static size_t padded_elems_v(int B, int H, int L) { return (size_t)B * H * L * 64; }
static size_t padded_workspace(int B, int H, int L) {
  // q, k, g_fwd, g_bwd padded to 32 channels, v and o to 64, then the matrix-core kernel's own workspace
  return (4 * padded_elems_qk(B, H, L) + 2 * padded_elems_v(B, H, L)) * sizeof(uint16_t) +
         vig::gla_mfma_workspace(B, H, L, 32, 64);
}

// What the path vig_gla_bidir_fwd dispatches to for exactly these arguments needs.
static size_t fwd_workspace_exact(int B, int H, int L, int Dk, int Dv, int io_dtype, int gate_dtype, bool bidir) {
  if (io_dtype == VIG_BF16 && gate_dtype == VIG_BF16 && (Dk == 64 || Dk == 32) && Dv == 64)
    return vig::gla_mfma_workspace(B, H, L, Dk, Dv);
  if (padded_shape(L, Dk, Dv, io_dtype, gate_dtype, bidir)) return padded_workspace(B, H, L);
  return bidir ? vig::gla_recurrent_workspace(B, H, L, Dv, io_dtype) : 0;
}

size_t vig_gla_bidir_fwd_workspace_for(int B, int H, int L, int Dk, int Dv, int io_dtype, int gate_dtype,
                                       int bidirectional) {
  if (B <= 0 || H <= 0 || L <= 0 || !dtype_ok(io_dtype) || !dtype_ok(gate_dtype)) return 0;
  return fwd_workspace_exact(B, H, L, Dk, Dv, io_dtype, gate_dtype, bidirectional != 0);
}

size_t vig_gla_bidir_fwd_workspace(int B, int H, int L, int Dk, int Dv, int io_dtype) {
  if (B <= 0 || H <= 0 || L <= 0) return 0;
  // The largest requirement over the paths the dispatcher may take for this shape.
  size_t need = vig::gla_recurrent_workspace(B, H, L, Dv, io_dtype);
  if (padded_shape(L, Dk, Dv, io_dtype, VIG_BF16, true)) {
    const size_t p = padded_workspace(B, H, L);
    if (p > need) need = p;
  }
  if (io_dtype == VIG_BF16) {
    const size_t m = vig::gla_mfma_workspace(B, H, L, Dk, Dv);
    if (m > need) need = m;
  }
  return need;
}

static int gla_bidir_fwd(const void* q, const void* k, const void* v, const void* g_fwd, const void* g_bwd, void* o,
                         void* workspace, size_t workspace_bytes, int B, int H, int L, int Dk, int Dv, float scale,
                         float out_scale, int io_dtype, int gate_dtype, void* stream, int wide_gates) {
  vig::GlaArgs a;
  const int rc = fill_args(a, q, k, v, g_fwd, g_bwd, o, workspace, workspace_bytes, B, H, L, Dk, Dv, scale,
                           out_scale, io_dtype, gate_dtype, stream);
  if (rc != VIG_OK) return rc;
  a.wide_gates = wide_gates;
  if (vig::gla_mfma_supported(a)) {
    // (the segment scan of long sequences puts sequence x direction on grid.y)
    if (L > 256 && (long long)B * H * (g_bwd ? 2 : 1) > 65535) return VIG_ENOTSUP;
    if (vig::gla_mfma_workspace(B, H, L, Dk, Dv) > workspace_bytes) return VIG_ENOSPC;
    if (vig::gla_mfma_workspace(B, H, L, Dk, Dv) > 0 && !workspace) return VIG_EINVAL;
    return vig::launch_gla_mfma(a);
  }
  if (padded_shape(L, Dk, Dv, io_dtype, gate_dtype, g_bwd != nullptr) && workspace &&
      workspace_bytes >= padded_workspace(B, H, L)) {
    // (a caller that sized the workspace for the recurrent kernel only still gets that kernel below)
    const size_t nqk = padded_elems_qk(B, H, L), nv = padded_elems_v(B, H, L);
    uint16_t* p = static_cast<uint16_t*>(workspace);
    uint16_t *qp = p, *kp = p + nqk, *gfp = p + 2 * nqk, *gbp = p + 3 * nqk, *vp = p + 4 * nqk, *op = vp + nv;
    const long long rows = (long long)B * H * L;
    hipStream_t st = (hipStream_t)stream;
    const void* srcs[5] = {q, k, g_fwd, g_bwd, v};
    void* dsts[5] = {qp, kp, gfp, gbp, vp};
    const int src_c[5] = {16, 16, 16, 16, 32}, dst_c[5] = {32, 32, 32, 32, 64};
    int e = vig::launch_pad_channels_multi(srcs, dsts, src_c, dst_c, 5, rows, st);
    if (e) return e;
    vig::GlaArgs b = a;
    b.q = qp, b.k = kp, b.v = vp, b.g_fwd = gfp, b.g_bwd = gbp, b.o = op;
    b.Dk = 32, b.Dv = 64;
    b.workspace = op + nv;
    b.workspace_bytes = vig::gla_mfma_workspace(B, H, L, 32, 64);
    e = vig::launch_gla_mfma(b);
    if (e) return e;
    return vig::launch_pad_channels(op, o, rows, 64, 32, st);
  }
  const size_t need = g_bwd ? vig::gla_recurrent_workspace(B, H, L, Dv, io_dtype) : 0;
  if (need > workspace_bytes) return VIG_ENOSPC;
  if (need > 0 && !workspace) return VIG_EINVAL;
  return vig::launch_gla_recurrent(a);
}

int vig_gla_bidir_fwd(const void* q, const void* k, const void* v, const void* g_fwd, const void* g_bwd, void* o,
                      void* workspace, size_t workspace_bytes, int B, int H, int L, int Dk, int Dv, float scale,
                      float out_scale, int io_dtype, int gate_dtype, void* stream) {
  return gla_bidir_fwd(q, k, v, g_fwd, g_bwd, o, workspace, workspace_bytes, B, H, L, Dk, Dv, scale, out_scale,
                       io_dtype, gate_dtype, stream, 0);
}

// q, k, v read in place from wider rows (e.g. the column blocks of a stacked projection's output): the matrix-core slab
// kernel with the rows' pitches in scalar registers; no workspace.
int vig_gla_bidir_fwd_strided(const void* q, const void* k, const void* v, const void* g_fwd, const void* g_bwd, void* o,
                              int B, int H, int L, int Dk, int Dv, const long long* q_strides,
                              const long long* k_strides, const long long* v_strides, float scale, float out_scale,
                              int io_dtype, int gate_dtype, void* stream) {
  if (!q_strides || !k_strides || !v_strides) return VIG_EINVAL;
  vig::GlaArgs a;
  const int rc = fill_args(a, q, k, v, g_fwd, g_bwd, o, nullptr, 0, B, H, L, Dk, Dv, scale, out_scale, io_dtype,
                           gate_dtype, stream);
  if (rc != VIG_OK) return rc;
  if (!vig::gla_mfma_supported(a) || L > 256) return VIG_ENOTSUP;
  a.q_strides = q_strides, a.k_strides = k_strides, a.v_strides = v_strides;
  return vig::launch_gla_mfma(a);
}

// The causal op with a state carried in and / or out.
static size_t causal_state_workspace(int B, int H, int L, int Dk, int Dv, int io_dtype, int gate_dtype) {
  if (io_dtype == VIG_BF16 && gate_dtype == VIG_BF16 && (Dk == 64 || Dk == 32) && Dv == 64)
    return vig::gla_mfma_state_workspace(B, H, L, Dk, Dv);
  return 0;  // the token-recurrent kernel keeps the state in registers
}

size_t vig_gla_causal_state_fwd_workspace(int B, int H, int L, int Dk, int Dv, int io_dtype, int gate_dtype) {
  if (B <= 0 || H <= 0 || L <= 0 || !dtype_ok(io_dtype) || !dtype_ok(gate_dtype)) return 0;
  return causal_state_workspace(B, H, L, Dk, Dv, io_dtype, gate_dtype);
}

static int causal_state_fwd(const void* q, const void* k, const void* v, const void* g, void* o,
                            const float* initial_state, float* final_state, void* workspace, size_t workspace_bytes,
                            int B, int H, int L, int Dk, int Dv, float scale, float out_scale, int io_dtype,
                            int gate_dtype, void* stream, bool exact) {
  vig::GlaArgs a;
  const int rc = fill_args(a, q, k, v, g, nullptr, o, workspace, workspace_bytes, B, H, L, Dk, Dv, scale, out_scale,
                           io_dtype, gate_dtype, stream);
  if (rc != VIG_OK) return rc;
  if (!aligned16(initial_state, final_state)) return VIG_EINVAL;
  a.init_state = initial_state;
  a.final_state = final_state;
  if (!exact && vig::gla_mfma_supported(a)) {
    if ((long long)B * H > 65535) return VIG_ENOTSUP;  // (the segment scan puts the sequences on grid.y)
    const size_t need = vig::gla_mfma_state_workspace(B, H, L, Dk, Dv);
    if (need > workspace_bytes) return VIG_ENOSPC;
    if (!workspace) return VIG_EINVAL;
    return vig::launch_gla_mfma(a);
  }
  return vig::launch_gla_recurrent(a);
}

int vig_gla_causal_state_fwd(const void* q, const void* k, const void* v, const void* g, void* o,
                             const float* initial_state, float* final_state, void* workspace, size_t workspace_bytes,
                             int B, int H, int L, int Dk, int Dv, float scale, float out_scale, int io_dtype,
                             int gate_dtype, void* stream) {
  return causal_state_fwd(q, k, v, g, o, initial_state, final_state, workspace, workspace_bytes, B, H, L, Dk, Dv, scale,
                          out_scale, io_dtype, gate_dtype, stream, false);
}

// Same contract, always the fp32-arithmetic token-recurrent kernel (no workspace).
int vig_gla_causal_state_fwd_exact(const void* q, const void* k, const void* v, const void* g, void* o,
                                   const float* initial_state, float* final_state, int B, int H, int L, int Dk, int Dv,
                                   float scale, float out_scale, int io_dtype, int gate_dtype, void* stream) {
  return causal_state_fwd(q, k, v, g, o, initial_state, final_state, nullptr, 0, B, H, L, Dk, Dv, scale, out_scale,
                          io_dtype, gate_dtype, stream, true);
}

// Same contract and results to the same bar; for callers whose gates are known to be strong (see the header).
int vig_gla_bidir_fwd_wide(const void* q, const void* k, const void* v, const void* g_fwd, const void* g_bwd, void* o,
                           void* workspace, size_t workspace_bytes, int B, int H, int L, int Dk, int Dv, float scale,
                           float out_scale, int io_dtype, int gate_dtype, void* stream) {
  return gla_bidir_fwd(q, k, v, g_fwd, g_bwd, o, workspace, workspace_bytes, B, H, L, Dk, Dv, scale, out_scale,
                       io_dtype, gate_dtype, stream, 1);
}

// ---- vig_gla_bidir_fwd for callers that cannot allocate: the workspace is a device array of this library ----
// One copy per GPU, held from the first launch of the library on that GPU until the process ends.
constexpr size_t kScratchBytes = VIG_GLA_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
// The array's name is only a host-side handle: its address on each device is looked up once, with that device current.
constexpr int kScratchMaxDevices = 64;
static void* scratch_ptr[kScratchMaxDevices] = {};
static std::mutex scratch_mutex;

// `owned`: a device pointer of the call (q).  The array that serves a call is the one of the GPU that holds the
// call's tensors, which has to be the current device (the kernels are launched there, and the symbol lookup answers
// for the current device only): a caller on another device is refused instead of being handed the wrong GPU's array.
static int scratch_for_current_device(void** out, const void* owned) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kScratchMaxDevices) return VIG_ELAUNCH;
  hipPointerAttribute_t attr;
  if (hipPointerGetAttributes(&attr, owned) == hipSuccess) {
    if (attr.type == hipMemoryTypeDevice && attr.device != dev) return VIG_EINVAL;
  } else {
    (void)hipGetLastError();  // (an unregistered pointer: the launch itself will report it)
  }
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (!scratch_ptr[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return VIG_ELAUNCH;
    scratch_ptr[dev] = p;
  }
  *out = scratch_ptr[dev];
  return VIG_OK;
}

size_t vig_gla_bidir_fwd_noalloc_max_workspace(void) { return kScratchBytes; }

int vig_gla_bidir_fwd_noalloc(const void* q, const void* k, const void* v, const void* g_fwd, const void* g_bwd,
                              void* o, int B, int H, int L, int Dk, int Dv, float scale, float out_scale,
                              int io_dtype, int gate_dtype, void* stream) {
  if (B <= 0 || H <= 0 || L <= 0) return VIG_EINVAL;
  if (!dtype_ok(io_dtype) || !dtype_ok(gate_dtype)) return VIG_ENOTSUP;
  // what the dispatched path of vig_gla_bidir_fwd needs; shapes whose need exceeds the array are refused, not shrunk
  const size_t need = fwd_workspace_exact(B, H, L, Dk, Dv, io_dtype, gate_dtype, g_bwd != nullptr);
  if (need > kScratchBytes) return VIG_ENOSPC;
  void* ws = nullptr;
  if (need > 0) {
    const int rc = scratch_for_current_device(&ws, q);
    if (rc != VIG_OK) return rc;
  }
  // Every kernel behind vig_gla_bidir_fwd writes the part of the workspace it later reads (segment states, padded
  // copies, the reverse direction's partial outputs) before reading it: nothing has to start at zero.
  return gla_bidir_fwd(q, k, v, g_fwd, g_bwd, o, ws, need, B, H, L, Dk, Dv, scale, out_scale, io_dtype, gate_dtype,
                       stream, 0);
}

// vig_gla_bidir_fwd followed by vig_locality_gate_fwd in one kernel: y = o * sigmoid(conv3x3(o)) with o the rounded
// GLA output, never written to memory.  Only shapes of the bf16 MFMA path with the whole sequence in one slab.
int vig_gla_bidir_locgate_fwd(const void* q, const void* k, const void* v, const void* g_fwd, const void* g_bwd,
                              const float* gate_weight, void* y, int B, int H, int L, int Dk, int Dv, int grid_h,
                              int grid_w, float scale, float out_scale, int io_dtype, int gate_dtype, void* stream) {
  vig::GlaArgs a;
  const int rc = fill_args(a, q, k, v, g_fwd, g_bwd, y, nullptr, 0, B, H, L, Dk, Dv, scale, out_scale, io_dtype,
                           gate_dtype, stream);
  if (rc != VIG_OK) return rc;
  if (!gate_weight || !g_bwd || grid_h <= 0 || grid_w <= 0 || (long long)grid_h * grid_w != L) return VIG_EINVAL;
  if (!aligned16(gate_weight)) return VIG_EINVAL;
  if (!vig::gla_mfma_supported(a) || vig::gla_mfma_workspace(B, H, L, Dk, Dv) > 0 ||
      !vig::gla_mfma_gate_grid_ok(grid_h, grid_w))
    return VIG_ENOTSUP;
  a.gate_w = gate_weight;
  a.gate_rows = grid_h;
  a.gate_cols = grid_w;
  return vig::launch_gla_mfma(a);
}

// Same contract as vig_gla_bidir_fwd, but always takes the fp32-arithmetic
// token-recurrent kernel (the exact path), whatever the dtypes.
int vig_gla_bidir_fwd_exact(const void* q, const void* k, const void* v, const void* g_fwd, const void* g_bwd,
                            void* o, void* workspace, size_t workspace_bytes, int B, int H, int L, int Dk, int Dv,
                            float scale, float out_scale, int io_dtype, int gate_dtype, void* stream) {
  vig::GlaArgs a;
  const int rc = fill_args(a, q, k, v, g_fwd, g_bwd, o, workspace, workspace_bytes, B, H, L, Dk, Dv, scale,
                           out_scale, io_dtype, gate_dtype, stream);
  if (rc != VIG_OK) return rc;
  const size_t need = g_bwd ? vig::gla_recurrent_workspace(B, H, L, Dv, io_dtype) : 0;
  if (need > workspace_bytes) return VIG_ENOSPC;
  if (need > 0 && !workspace) return VIG_EINVAL;
  return vig::launch_gla_recurrent(a);
}

int vig_dirgate_fwd(const void* gk_lin, void* g_out, int B, int L, int H, int Dk, float inv_normalizer,
                    float clamp_min, int in_dtype, int out_dtype, void* stream) {
  if (!gk_lin || !g_out || B <= 0 || L <= 0 || H <= 0 || Dk <= 0) return VIG_EINVAL;
  if (!aligned16(gk_lin, g_out)) return VIG_EINVAL;
  if (!dtype_ok(in_dtype) || !dtype_ok(out_dtype) || (Dk % 8) != 0) return VIG_ENOTSUP;
  return vig::launch_dirgate(gk_lin, g_out, B, L, H, Dk, inv_normalizer, clamp_min, in_dtype, out_dtype,
                             (hipStream_t)stream);
}

int vig_dirgate_bwd(const void* gk_lin, const void* d_g, void* d_gk_lin, int B, int L, int H, int Dk,
                    float inv_normalizer, float clamp_min, int in_dtype, int out_dtype, void* stream) {
  if (!gk_lin || !d_g || !d_gk_lin || B <= 0 || L <= 0 || H <= 0 || Dk <= 0) return VIG_EINVAL;
  if (!aligned16(gk_lin, d_g, d_gk_lin)) return VIG_EINVAL;
  if (!dtype_ok(in_dtype) || !dtype_ok(out_dtype) || (Dk % 8) != 0) return VIG_ENOTSUP;
  return vig::launch_dirgate_bwd(gk_lin, d_g, d_gk_lin, B, L, H, Dk, inv_normalizer, clamp_min, in_dtype, out_dtype,
                                 (hipStream_t)stream);
}

int vig_split_heads_bwd(const void* dq, const void* dk, const void* dv, void* d_qkv, int B, int L, int H, int Dk,
                        int Dv, int io_dtype, void* stream) {
  if (!dq || !dk || !dv || !d_qkv || B <= 0 || L <= 0 || H <= 0 || Dk <= 0 || Dv <= 0) return VIG_EINVAL;
  if (!aligned16(dq, dk, dv, d_qkv)) return VIG_EINVAL;
  if (!dtype_ok(io_dtype) || (Dk % 8) != 0 || (Dv % 8) != 0 || B > 65535) return VIG_ENOTSUP;
  return vig::launch_merge_heads(dq, dk, dv, d_qkv, B, L, H, Dk, Dv, io_dtype, (hipStream_t)stream);
}

int vig_dirgate_lowrank_fwd(const void* gk_low, long long low_row_stride, const void* w_up, const void* b_up,
                            void* g_out, int B, int L, int H, int Dk, int rank, float inv_normalizer, float clamp_min,
                            int in_dtype, int out_dtype, void* stream) {
  if (!gk_low || !w_up || !b_up || !g_out || B <= 0 || L <= 0 || H <= 0 || Dk <= 0 || rank <= 0) return VIG_EINVAL;
  if (!dtype_ok(in_dtype) || !dtype_ok(out_dtype) || (Dk % 8) != 0 || rank != 16) return VIG_ENOTSUP;
  const long long ld = low_row_stride > 0 ? low_row_stride : rank;
  if (ld < rank || !strided_rows_ok(gk_low, ld, in_dtype) || !strided_rows_ok(w_up, rank, in_dtype) ||
      !strided_rows_ok(b_up, 8, in_dtype) || !aligned16(g_out))
    return VIG_EINVAL;
  return vig::launch_dirgate_lowrank(gk_low, ld, w_up, b_up, g_out, B, L, H, Dk, rank, inv_normalizer, clamp_min,
                                     in_dtype, out_dtype, (hipStream_t)stream);
}

int vig_dwconv3x3_fwd(const void* x, const float* weight, const float* bias, void* y, int B, int h, int w, int C,
                      int silu, int io_dtype, void* stream) {
  if (!x || !weight || !y || B <= 0 || h <= 0 || w <= 0 || C <= 0 || x == y) return VIG_EINVAL;
  if (!aligned16(x, weight, bias, y)) return VIG_EINVAL;
  if (!dtype_ok(io_dtype) || (C % 8) != 0) return VIG_ENOTSUP;
  return vig::launch_dwconv3x3(x, weight, bias, y, B, h, w, C, silu, io_dtype, (hipStream_t)stream);
}

size_t vig_dwconv3x3_bwd_weight_workspace(int B, int C) {
  if (B <= 0 || C <= 0) return 0;
  return vig::dwconv3x3_wgrad_workspace(B, C);
}

int vig_dwconv3x3_bwd_weight(const void* x, const void* dy, float* dw_db, void* workspace, size_t workspace_bytes,
                             int B, int h, int w, int C, int io_dtype, void* stream) {
  if (!x || !dy || !dw_db || B <= 0 || h <= 0 || w <= 0 || C <= 0) return VIG_EINVAL;
  if (!aligned16(x, dy, dw_db, workspace)) return VIG_EINVAL;
  if (!dtype_ok(io_dtype) || (C % 8) != 0) return VIG_ENOTSUP;
  if (!workspace || workspace_bytes < vig::dwconv3x3_wgrad_workspace(B, C)) return VIG_ENOSPC;
  return vig::launch_dwconv3x3_wgrad(x, dy, dw_db, workspace, B, h, w, C, io_dtype, (hipStream_t)stream);
}

int vig_locality_gate_fwd(const void* o, const float* weight, void* y, int B, int H, int h, int w, int Dv,
                          int io_dtype, void* stream) {
  if (!o || !weight || !y || B <= 0 || H <= 0 || h <= 0 || w <= 0 || o == y) return VIG_EINVAL;
  if (!aligned16(o, weight, y)) return VIG_EINVAL;
  if (!dtype_ok(io_dtype) || (Dv % 8) != 0 || Dv <= 0) return VIG_ENOTSUP;
  return vig::launch_locality_gate(o, weight, y, B, H, h, w, Dv, io_dtype, (hipStream_t)stream);
}

int vig_locality_blend_fwd(const void* o, const void* local, const void* g_lin, const float* w_g, const float* w_l,
                           void* y, int B, int H, int L, int Dv, long long g_row_stride, float eps, int silu_out,
                           int io_dtype, void* stream) {
  if (!o || !local || !g_lin || !w_g || !w_l || !y || B <= 0 || H <= 0 || L <= 0) return VIG_EINVAL;
  if (!aligned16(o, local, w_g, w_l, y)) return VIG_EINVAL;
  if (!dtype_ok(io_dtype) || !(Dv == 32 || Dv == 64)) return VIG_ENOTSUP;
  const long long ldg = g_row_stride > 0 ? g_row_stride : (long long)H * Dv;
  if (ldg < (long long)H * Dv || !strided_rows_ok(g_lin, ldg, io_dtype)) return VIG_EINVAL;
  return vig::launch_locality_blend(o, local, g_lin, w_g, w_l, y, B, H, L, Dv, ldg, eps, silu_out, io_dtype,
                                    (hipStream_t)stream);
}

size_t vig_locality_blend_bwd_workspace(int B, int L, int Dv) {
  if (B <= 0 || L <= 0 || !(Dv == 32 || Dv == 64)) return 0;
  return vig::locality_blend_bwd_workspace(B, L, Dv);
}

int vig_locality_blend_bwd(const void* o, const void* local, const void* g_lin, const float* w_g, const float* w_l,
                           const void* dy, void* d_o, void* d_local, void* d_glin, float* dw, void* workspace,
                           size_t workspace_bytes, int B, int H, int L, int Dv, long long g_row_stride, float eps,
                           int silu_out, int io_dtype, void* stream) {
  if (!o || !local || !g_lin || !w_g || !w_l || !dy || !d_o || !d_local || !d_glin || !dw || B <= 0 || H <= 0 ||
      L <= 0)
    return VIG_EINVAL;
  if (!aligned16(o, local, w_g, w_l, dy, d_o, d_local, d_glin, dw, workspace)) return VIG_EINVAL;
  if (!dtype_ok(io_dtype) || !(Dv == 32 || Dv == 64)) return VIG_ENOTSUP;
  const long long ldg = g_row_stride > 0 ? g_row_stride : (long long)H * Dv;
  if (ldg < (long long)H * Dv || !strided_rows_ok(g_lin, ldg, io_dtype)) return VIG_EINVAL;
  if (!workspace || workspace_bytes < vig::locality_blend_bwd_workspace(B, L, Dv)) return VIG_ENOSPC;
  return vig::launch_locality_blend_bwd(o, local, g_lin, w_g, w_l, dy, d_o, d_local, d_glin, dw, workspace, B, H, L,
                                        Dv, ldg, eps, silu_out, io_dtype, (hipStream_t)stream);
}

int vig_rmsnorm_fwd(const void* x, const void* residual, const float* weight, void* y, void* residual_out,
                    long long rows, int C, float eps, int round_sum, int io_dtype, void* stream) {
  if (!x || !weight || !y || rows <= 0 || C <= 0 || rows > 0x7fffffffLL) return VIG_EINVAL;
  if (!aligned16(x, residual, weight, y, residual_out)) return VIG_EINVAL;
  if (!dtype_ok(io_dtype) || (C % 8) != 0 || C > 4096) return VIG_ENOTSUP;
  return vig::launch_rmsnorm(x, residual, weight, y, residual_out, (int)rows, C, eps, round_sum, io_dtype,
                             (hipStream_t)stream);
}

int vig_layernorm_fwd(const void* x, const float* weight, const float* bias, void* y, long long rows, int C,
                      float eps, int silu, const float* pre_bias, const void* post_add, int post_rows, int io_dtype,
                      void* stream) {
  if (!x || !weight || !bias || !y || rows <= 0 || C <= 0 || (post_add && post_rows <= 0)) return VIG_EINVAL;
  if (!aligned16(x, weight, bias, y, pre_bias, post_add)) return VIG_EINVAL;
  if (!dtype_ok(io_dtype) || (C % 8) != 0 || C > 4096) return VIG_ENOTSUP;
  return vig::launch_layernorm(x, weight, bias, y, rows, C, eps, silu, pre_bias, post_add, post_rows, io_dtype,
                               (hipStream_t)stream);
}

int vig_split_heads_fwd(const void* qkv, void* q, void* k, void* v, int B, int L, int H, int Dk, int Dv,
                        long long qkv_row_stride, int io_dtype, void* stream) {
  if (!qkv || !q || !k || !v || B <= 0 || L <= 0 || H <= 0 || Dk <= 0 || Dv <= 0) return VIG_EINVAL;
  if (!aligned16(q, k, v)) return VIG_EINVAL;
  if (!dtype_ok(io_dtype) || (Dk % 8) != 0 || (Dv % 8) != 0 || B > 65535) return VIG_ENOTSUP;
  const long long packed = (long long)H * (2 * Dk + Dv);
  const long long ld = qkv_row_stride > 0 ? qkv_row_stride : packed;
  if (ld < packed || !strided_rows_ok(qkv, ld, io_dtype)) return VIG_EINVAL;
  return vig::launch_split_heads(qkv, q, k, v, B, L, H, Dk, Dv, ld, io_dtype, (hipStream_t)stream);
}

int vig_patch_conv_fwd(const void* x, const void* w_packed, void* y, int B, int Cin, int H, int W, int KH, int KW,
                       int stride, int padding, int Cout, int io_dtype, void* stream) {
  if (!x || !w_packed || !y || B <= 0 || Cin <= 0 || H <= 0 || W <= 0 || KH <= 0 || KW <= 0 || Cout <= 0) return VIG_EINVAL;
  if (io_dtype != VIG_BF16 || !vig::patch_conv_supported(Cin, H, W, KH, KW, stride, padding, Cout)) return VIG_ENOTSUP;
  if (!strided_rows_ok(x, W, io_dtype) || !strided_rows_ok(w_packed, 16, io_dtype) || !strided_rows_ok(y, Cout, io_dtype))
    return VIG_EINVAL;
  return vig::launch_patch_conv(x, w_packed, y, B, Cin, H, W, KH, KW, Cout, (hipStream_t)stream);
}

int vig_locality_blend_linear_fwd(const void* o, const void* local, const void* g_lin, const float* w_g,
                                  const float* w_l, const void* weight, void* out, int B, int H, int L, int Dv, int C,
                                  long long g_row_stride, float eps, int silu_out, int io_dtype, void* stream) {
  if (!o || !local || !g_lin || !w_g || !w_l || !weight || !out || B <= 0 || H <= 0 || L <= 0) return VIG_EINVAL;
  if (!aligned16(o, local, w_g, w_l, weight, out)) return VIG_EINVAL;
  if (io_dtype != VIG_BF16 || !vig::blend_linear_supported(H, Dv, C)) return VIG_ENOTSUP;
  const long long ldg = g_row_stride > 0 ? g_row_stride : (long long)H * Dv;
  if (ldg < (long long)H * Dv || !strided_rows_ok(g_lin, ldg, io_dtype)) return VIG_EINVAL;
  return vig::launch_blend_linear(o, local, g_lin, w_g, w_l, weight, out, B, H, L, Dv, C, ldg, eps, silu_out,
                                  (hipStream_t)stream);
}

int vig_linear_swiglu_fwd(const void* x, const void* weight, void* y, long long rows, int K, int I, int io_dtype,
                          void* stream) {
  if (!x || !weight || !y || rows <= 0 || K <= 0 || I <= 0) return VIG_EINVAL;
  if (io_dtype != VIG_BF16 || !vig::linear_swiglu_supported(K, I)) return VIG_ENOTSUP;
  if (!strided_rows_ok(x, K, io_dtype) || !strided_rows_ok(weight, K, io_dtype) || !strided_rows_ok(y, I, io_dtype))
    return VIG_EINVAL;
  return vig::launch_linear_swiglu(x, weight, y, rows, K, I, (hipStream_t)stream);
}

int vig_swiglu_fwd(const void* gate_up, void* out, long long rows, int I, int io_dtype, void* stream) {
  if (!gate_up || !out || rows <= 0 || I <= 0) return VIG_EINVAL;
  if (!aligned16(gate_up, out)) return VIG_EINVAL;
  if (!dtype_ok(io_dtype) || (I % 8) != 0) return VIG_ENOTSUP;
  return vig::launch_swiglu(gate_up, out, rows, I, io_dtype, (hipStream_t)stream);
}

int vig_swiglu_bwd(const void* gate_up, const void* dy, void* d_gate_up, long long rows, int I, int io_dtype,
                   void* stream) {
  if (!gate_up || !dy || !d_gate_up || rows <= 0 || I <= 0) return VIG_EINVAL;
  if (!aligned16(gate_up, dy, d_gate_up)) return VIG_EINVAL;
  if (!dtype_ok(io_dtype) || (I % 8) != 0) return VIG_ENOTSUP;
  return vig::launch_swiglu_bwd(gate_up, dy, d_gate_up, rows, I, io_dtype, (hipStream_t)stream);
}

size_t vig_rmsnorm_bwd_workspace(long long rows, int C) {
  if (rows <= 0 || C <= 0) return 0;
  return vig::rmsnorm_bwd_workspace(rows, C);
}

int vig_rmsnorm_bwd(const void* sum, const float* weight, const void* dy, const void* d_sum, void* ds, float* dweight,
                    void* workspace, size_t workspace_bytes, long long rows, int C, float eps, int io_dtype,
                    void* stream) {
  if (!sum || !weight || !dy || !ds || rows <= 0 || C <= 0 || rows > 0x7fffffffLL) return VIG_EINVAL;
  if (!aligned16(sum, weight, dy, d_sum, ds, dweight, workspace)) return VIG_EINVAL;
  if (!dtype_ok(io_dtype) || (C % 8) != 0 || C > 1024) return VIG_ENOTSUP;
  if (dweight && (!workspace || workspace_bytes < vig::rmsnorm_bwd_workspace(rows, C))) return VIG_ENOSPC;
  return vig::launch_rmsnorm_bwd(sum, weight, dy, d_sum, ds, dweight, workspace, rows, C, eps, io_dtype,
                                 (hipStream_t)stream);
}

static bool bwd_shape_ok(int Dk, int Dv) {
  return (Dk == 16 && Dv == 32) || (Dk == 32 && (Dv == 32 || Dv == 64)) || (Dk == 64 && (Dv == 32 || Dv == 64));
}

size_t vig_gla_bidir_bwd_workspace(int B, int H, int L, int Dk, int Dv, int bidirectional) {
  if (B <= 0 || H <= 0 || L <= 0 || !bwd_shape_ok(Dk, Dv)) return 0;
  return vig::gla_backward_workspace(B, H, L, Dk, Dv, bidirectional);
}

// The backward of HierViG's head shape rides the matrix-core kernels the way its forward does: q, k, both gates and
// their four gradients padded to 32 channels, v, d_o and dv to 64, then the backward's own workspace at 32 / 64.
static size_t padded_bwd_tensors(int B, int H, int L) {
  const size_t n = (8 * padded_elems_qk(B, H, L) + 3 * padded_elems_v(B, H, L)) * sizeof(uint16_t);
  return (n + 255) / 256 * 256;
}
static size_t padded_bwd_workspace(int B, int H, int L) {
  return padded_bwd_tensors(B, H, L) + vig::gla_backward_workspace(B, H, L, 32, 64, 1);
}

size_t vig_gla_bidir_bwd_workspace_for(int B, int H, int L, int Dk, int Dv, int io_dtype, int gate_dtype,
                                       int bidirectional) {
  if (B <= 0 || H <= 0 || L <= 0 || !bwd_shape_ok(Dk, Dv) || !dtype_ok(io_dtype) || !dtype_ok(gate_dtype)) return 0;
  if (padded_shape(L, Dk, Dv, io_dtype, gate_dtype, bidirectional != 0)) return padded_bwd_workspace(B, H, L);
  return vig::gla_backward_workspace(B, H, L, Dk, Dv, bidirectional);
}

static int gla_bidir_bwd(const void* q, const void* k, const void* v, const void* g_fwd, const void* g_bwd,
                         const void* d_o, void* dq, void* dk, void* dv, void* dg_fwd, void* dg_bwd, void* workspace,
                         size_t workspace_bytes, int B, int H, int L, int Dk, int Dv, float scale, float out_scale,
                         int io_dtype, int gate_dtype, bool exact, void* stream) {
  if (!q || !k || !v || !g_fwd || !d_o || !dq || !dk || !dv || !dg_fwd || (g_bwd && !dg_bwd) || B <= 0 || H <= 0 ||
      L <= 0)
    return VIG_EINVAL;
  if (!aligned16(q, k, v, g_fwd, g_bwd, d_o, dq, dk, dv, dg_fwd, dg_bwd, workspace)) return VIG_EINVAL;
  if ((long long)B * H > 2147483647LL) return VIG_EINVAL;
  if (!dtype_ok(io_dtype) || !dtype_ok(gate_dtype) || !bwd_shape_ok(Dk, Dv)) return VIG_ENOTSUP;
  if (!exact && padded_shape(L, Dk, Dv, io_dtype, gate_dtype, g_bwd != nullptr) && workspace &&
      workspace_bytes >= padded_bwd_workspace(B, H, L)) {
    // (a caller that sized the workspace with vig_gla_bidir_bwd_workspace gets the recurrent kernel below)
    const size_t nqk = padded_elems_qk(B, H, L), nv = padded_elems_v(B, H, L);
    uint16_t* p = static_cast<uint16_t*>(workspace);
    uint16_t *qp = p, *kp = p + nqk, *gfp = p + 2 * nqk, *gbp = p + 3 * nqk, *dqp = p + 4 * nqk, *dkp = p + 5 * nqk,
             *dgfp = p + 6 * nqk, *dgbp = p + 7 * nqk, *vp = p + 8 * nqk, *dop = vp + nv, *dvp = dop + nv;
    const long long rows = (long long)B * H * L;
    hipStream_t st = (hipStream_t)stream;
    {
      const void* srcs[6] = {q, k, g_fwd, g_bwd, v, d_o};
      void* dsts[6] = {qp, kp, gfp, gbp, vp, dop};
      const int src_c[6] = {16, 16, 16, 16, 32, 32}, dst_c[6] = {32, 32, 32, 32, 64, 64};
      const int e = vig::launch_pad_channels_multi(srcs, dsts, src_c, dst_c, 6, rows, st);
      if (e) return e;
    }
    const int e = vig::launch_gla_backward(qp, kp, vp, gfp, gbp, dop, dqp, dkp, dvp, dgfp, dgbp,
                                           (char*)workspace + padded_bwd_tensors(B, H, L), B, H, L, 32, 64, scale,
                                           out_scale, io_dtype, gate_dtype, false, st);
    if (e) return e;
    const void* srcs[5] = {dqp, dkp, dgfp, dgbp, dvp};
    void* dsts[5] = {dq, dk, dg_fwd, dg_bwd, dv};
    const int src_c[5] = {32, 32, 32, 32, 64}, dst_c[5] = {16, 16, 16, 16, 32};
    return vig::launch_pad_channels_multi(srcs, dsts, src_c, dst_c, 5, rows, st);
  }
  const size_t need = vig::gla_backward_workspace(B, H, L, Dk, Dv, g_bwd != nullptr);
  if (!workspace || workspace_bytes < need) return VIG_ENOSPC;
  return vig::launch_gla_backward(q, k, v, g_fwd, g_bwd, d_o, dq, dk, dv, dg_fwd, dg_bwd, workspace, B, H, L, Dk, Dv,
                                  scale, out_scale, io_dtype, gate_dtype, exact, (hipStream_t)stream);
}

int vig_gla_bidir_bwd(const void* q, const void* k, const void* v, const void* g_fwd, const void* g_bwd,
                      const void* d_o, void* dq, void* dk, void* dv, void* dg_fwd, void* dg_bwd, void* workspace,
                      size_t workspace_bytes, int B, int H, int L, int Dk, int Dv, float scale, float out_scale,
                      int io_dtype, int gate_dtype, void* stream) {
  return gla_bidir_bwd(q, k, v, g_fwd, g_bwd, d_o, dq, dk, dv, dg_fwd, dg_bwd, workspace, workspace_bytes, B, H, L, Dk,
                       Dv, scale, out_scale, io_dtype, gate_dtype, false, stream);
}

// Same contract, always the fp32-arithmetic token-recurrent kernel.
int vig_gla_bidir_bwd_exact(const void* q, const void* k, const void* v, const void* g_fwd, const void* g_bwd,
                            const void* d_o, void* dq, void* dk, void* dv, void* dg_fwd, void* dg_bwd,
                            void* workspace, size_t workspace_bytes, int B, int H, int L, int Dk, int Dv, float scale,
                            float out_scale, int io_dtype, int gate_dtype, void* stream) {
  return gla_bidir_bwd(q, k, v, g_fwd, g_bwd, d_o, dq, dk, dv, dg_fwd, dg_bwd, workspace, workspace_bytes, B, H, L, Dk,
                       Dv, scale, out_scale, io_dtype, gate_dtype, true, stream);
}

}  // extern "C"
