/*
 * vig_gla.h -- C ABI of the MI355X (gfx950) bidirectional gated-linear-attention
 * forward path of ViG and its two neighbours (direction-wise gate preparation,
 * 2D locality gate).
 *
 * Conventions shared by every entry point
 *   - every pointer is DEVICE memory owned by the caller; nothing is allocated,
 *     freed or synchronised inside; work is enqueued on `stream`
 *     (a hipStream_t passed as void*; NULL = the null stream);
 *   - tensors are dense row-major with the innermost dimension contiguous;
 *   - every tensor, weight vector and workspace starts on a 16-byte boundary
 *     (the kernels move 16 bytes per access); a pointer off it is VIG_EINVAL;
 *   - return value: 0 on success, a negative VIG_E* code otherwise
 *     (vig_gla_strerror() gives the text); a failed call enqueues nothing;
 *   - dtype codes: VIG_F32 = 0, VIG_BF16 = 1.
 *
 * Citations name the reference (hustvl/ViG) interface each entry point replaces.
 */
#ifndef VIG_GLA_H_
#define VIG_GLA_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VIG_F32 0
#define VIG_BF16 1

#define VIG_OK 0
#define VIG_EINVAL (-22)  /* bad argument (null or misaligned pointer, non-positive size) */
#define VIG_ENOTSUP (-95) /* shape / dtype combination not built */
#define VIG_ENOSPC (-28)  /* workspace too small */
#define VIG_ELAUNCH (-5)  /* HIP reported a launch error */

/* Library identification: "vig_gla <version> gfx950". */
const char* vig_gla_version(void);
const char* vig_gla_strerror(int code);

/*
 * Bidirectional GLA forward, both directions in one call, natural token order.
 *
 *   S_i  = diag(exp(gf_i)) S_{i-1} + k_i v_i^T      (i = 0..L-1)
 *   S'_i = diag(exp(gb_i)) S'_{i+1} + k_i v_i^T     (i = L-1..0)
 *   o_i  = out_scale * (scale*q_i)^T (S_i + S'_i)
 *
 * q, k, g_fwd, g_bwd: [B, H, L, Dk]; v, o: [B, H, L, Dv].  g_* are natural-log
 * decays (<= 0).  g_bwd == NULL computes the forward direction only (the causal
 * op).  io_dtype is the type of q, k, v, o; gate_dtype the type of g_*.
 * `workspace` must hold vig_gla_bidir_fwd_workspace(...) bytes (may be NULL when
 * that is 0).
 *
 * Replaces: bid_fused_recurrent_gla (flash-linear-attention/fla/ops/gla/
 * recurrent_fuse.py:659-676, kernel :19-148; out_scale 1/2 from :442),
 * batch_bid_fused_chunk_gla (fla/ops/gla/chunk_fuse.py:574-596) and, with
 * g_bwd == NULL, fused_chunk_gla (chunk_fuse.py:554-572).
 *
 * Built shapes: Dk in {16, 32, 64, 128}, Dv in {32, 64, 128}, any L >= 1.
 *
 * Numeric range of the matrix-core paths (bf16 tensors and gates, Dk in {32, 64},
 * Dv = 64).  q, k and v may hold any finite bf16 values; the kernels check
 * magnitudes and gate totals themselves and switch arithmetic where needed:
 *   L <= 256 (one workgroup per sequence, one wave per 32-token tile): fp16
 *   operands while every tile's gate total stays within about 7 (natural log
 *   units) per channel and rows of q / k / v have sums of squares below 2^15 /
 *   2^10 / 10^8; a sequence outside that is redone by the same workgroup with
 *   power-of-two input scales and split-bf16 diagonal tiles, good for gates down
 *   to about -5 per token (beyond: exponents are clamped, far tokens count as 0).
 *   L > 256 (segments of <= 224 tokens, seven tiles each, chained through states
 *   in the workspace: a state pass, a scan, then the kernel above once more per
 *   segment with the entering states; refused with VIG_ENOTSUP when
 *   B*H*directions > 65535): the same per-tile behaviour for the outputs, and for
 *   the state pass the sum of |g| over any 56 consecutive tokens of one channel
 *   must stay below about 80 (beyond it results may be inf / NaN, never silently
 *   wrong finite numbers).
 * HierViG's head shape (bf16, Dk = 16, Dv = 32, both directions) takes the same
 * paths from L = 128 on, zero-padded to Dk 32 / Dv 64 in the workspace
 * (classification/models/vig_h.py:377-385 with EXPAND_K 0.5, EXPAND_V 1.0).
 * Other combinations run on the
 * fp32-arithmetic kernel, which has no such limit.
 */
int vig_gla_bidir_fwd(const void* q, const void* k, const void* v,
                      const void* g_fwd, const void* g_bwd, void* o,
                      void* workspace, size_t workspace_bytes,
                      int B, int H, int L, int Dk, int Dv,
                      float scale, float out_scale,
                      int io_dtype, int gate_dtype, void* stream);

/*
 * vig_gla_bidir_fwd on q, k, v that are not plain [B, H, L, D] tensors: element (b, h, l, d) of q lies at
 * q + b*q_strides[0] + h*q_strides[1] + l*q_strides[2] + d (likewise k, v; the channels of one (token, head) are
 * contiguous).  For the column blocks of a projection output [B, L, H*(2*Dk + Dv)] read in place that is
 * {L*row, Dk (or Dv), row} with row = H*(2*Dk + Dv), so no head-major copies of q, k, v are made.  g_fwd, g_bwd and o
 * stay plain [B, H, L, D].  Strides are positive multiples of 8 elements (16-byte rows), the token stride at most 2^20.
 * Built for the matrix-core slab kernel only: bf16 tensors and gates, Dk in {32, 64}, Dv = 64, L <= 256 (no workspace);
 * VIG_ENOTSUP otherwise.  Same arithmetic and results as vig_gla_bidir_fwd on contiguous copies.
 *
 * Replaces: the stride arguments of the reference's kernels (s_qk_h, s_qk_t, s_qk_d, s_vo_h, s_vo_t, s_vo_d,
 * flash-linear-attention/fla/ops/gla/chunk_fuse.py:23-38), which its wrapper feeds with contiguous copies
 * (@contiguous, chunk_fuse.py:315) of the head-split views made at classification/models/vig.py:402-406 and :436-438.
 */
int vig_gla_bidir_fwd_strided(const void* q, const void* k, const void* v,
                              const void* g_fwd, const void* g_bwd, void* o,
                              int B, int H, int L, int Dk, int Dv,
                              const long long* q_strides, const long long* k_strides, const long long* v_strides,
                              float scale, float out_scale,
                              int io_dtype, int gate_dtype, void* stream);

/* Workspace that is enough for every gate dtype and for one or two directions (the largest over the kernels the
 * call may dispatch to for this shape and io_dtype). */
size_t vig_gla_bidir_fwd_workspace(int B, int H, int L, int Dk, int Dv, int io_dtype);
/* Workspace of exactly the kernel vig_gla_bidir_fwd / _wide dispatch to for these arguments (bidirectional: g_bwd
 * given): 0 for bf16 tensors and gates with Dk in {32, 64}, Dv = 64, L <= 256. */
size_t vig_gla_bidir_fwd_workspace_for(int B, int H, int L, int Dk, int Dv, int io_dtype, int gate_dtype,
                                       int bidirectional);

/*
 * The causal op (one direction) with a state carried in and / or out:
 *   S_{-1} = initial_state (zero when NULL);  S_i = diag(exp(g_i)) S_{i-1} + k_i v_i^T;  o_i = out_scale * (scale*q_i)^T S_i;
 *   final_state = S_{L-1} (not written when NULL).
 * initial_state, final_state: fp32 [B, H, Dk, Dv], row-major (k channel, then v channel); same tensors, dtypes and
 * shapes as vig_gla_bidir_fwd with g_bwd == NULL.  bf16 tensors and gates with Dk in {32, 64}, Dv = 64 run on the
 * matrix cores as chained segments of up to 256 tokens (state contributions, a scan that starts from initial_state
 * and ends in final_state, outputs); everything else on the fp32-arithmetic token-recurrent kernel.
 * `workspace` must hold vig_gla_causal_state_fwd_workspace(...) bytes (may be NULL when that is 0).
 *
 * Replaces: fused_chunk_gla with initial_state / output_final_state (flash-linear-attention/fla/ops/gla/
 * chunk_fuse.py:554-572; the state enters at :70-72 and leaves at :99-101) and fused_recurrent_gla with the same
 * arguments (fla/ops/gla/recurrent_fuse.py:631-657, kernel :213-218,240-246).
 */
int vig_gla_causal_state_fwd(const void* q, const void* k, const void* v, const void* g, void* o,
                             const float* initial_state, float* final_state,
                             void* workspace, size_t workspace_bytes,
                             int B, int H, int L, int Dk, int Dv,
                             float scale, float out_scale,
                             int io_dtype, int gate_dtype, void* stream);
size_t vig_gla_causal_state_fwd_workspace(int B, int H, int L, int Dk, int Dv, int io_dtype, int gate_dtype);
/* Same contract, always the fp32-arithmetic token-recurrent kernel whatever the dtypes (no workspace): the counterpart
 * of fused_recurrent_gla's state arguments (fla/ops/gla/recurrent_fuse.py:631-657). */
int vig_gla_causal_state_fwd_exact(const void* q, const void* k, const void* v, const void* g, void* o,
                                   const float* initial_state, float* final_state,
                                   int B, int H, int L, int Dk, int Dv,
                                   float scale, float out_scale,
                                   int io_dtype, int gate_dtype, void* stream);

/*
 * Same contract, workspace and accuracy bar as vig_gla_bidir_fwd, for callers who know their gates to be strong.
 * The matrix-core kernel computes on fp16 operands while every 32-token tile's gate total stays within about 7
 * (natural log units) in every channel, and in its wider-range form beyond; it finds out per sequence (or segment),
 * after preparing the fp16 operands in vain, and redoes it at about four times the cost.  This entry point runs the
 * wider-range form alone, in a kernel of its own with twice the registers: about 1.65 times the fp16 form's time
 * whatever the gates (60 against 37 us at B128 H6 L196 Dk64), against 3.8 times through the default entry point when
 * every sequence refuses.  No counterpart
 * in the reference, whose kernels have one arithmetic (fla/ops/gla/chunk_fuse.py:25-101,212-254).
 */
int vig_gla_bidir_fwd_wide(const void* q, const void* k, const void* v,
                           const void* g_fwd, const void* g_bwd, void* o,
                           void* workspace, size_t workspace_bytes,
                           int B, int H, int L, int Dk, int Dv,
                           float scale, float out_scale,
                           int io_dtype, int gate_dtype, void* stream);

/*
 * vig_gla_bidir_fwd without a workspace argument, for callers that cannot allocate device memory: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  Same tensors, dispatch, kernels and
 * results (bit for bit) as vig_gla_bidir_fwd; the workspace is a device array inside the library,
 * VIG_GLA_NOALLOC_SCRATCH_BYTES per GPU, held from the first call on that GPU until the process ends.  A shape whose
 * vig_gla_bidir_fwd_workspace_for(...) exceeds that size returns VIG_ENOSPC and launches nothing (then use
 * vig_gla_bidir_fwd with a workspace of the caller's).  Calls no hipMalloc / hipFree and nothing else that allocates.
 * All calls on one GPU share the one array: calls that overlap in time on the same GPU (two streams, two threads)
 * race on it; serialise them.  The tensors must live on the current device (another device's pointers: VIG_EINVAL).
 * Under HIP graph capture: make one call per device and shape class outside the capture first.  The first call on a
 * device looks up the array's address and sets the kernels' shared-memory attribute (no stream work, but not capturable
 * either); every later call is kernel launches on `stream` only.  It has no counterpart in the reference, whose ops
 * allocate their temporaries through torch (flash-linear-attention/fla/ops/gla/chunk_fuse.py:325-345).
 */
#define VIG_GLA_NOALLOC_SCRATCH_BYTES (16u << 20)
int vig_gla_bidir_fwd_noalloc(const void* q, const void* k, const void* v,
                              const void* g_fwd, const void* g_bwd, void* o,
                              int B, int H, int L, int Dk, int Dv,
                              float scale, float out_scale,
                              int io_dtype, int gate_dtype, void* stream);
size_t vig_gla_bidir_fwd_noalloc_max_workspace(void);

/*
 * Same contract as vig_gla_bidir_fwd, but always runs the fp32-arithmetic
 * token-recurrent kernel whatever the dtypes (bf16 tensors are widened on load,
 * the state and all sums stay fp32).  This is the op-level counterpart of the
 * reference's recurrent kernels (fla/ops/gla/recurrent_fuse.py:19-148,152-246),
 * kept callable for callers that want fp32 state arithmetic on bf16 tensors.
 * Workspace: B*H*L*Dv*4 bytes when io_dtype is bf16 and g_bwd != NULL, else 0.
 */
int vig_gla_bidir_fwd_exact(const void* q, const void* k, const void* v,
                            const void* g_fwd, const void* g_bwd, void* o,
                            void* workspace, size_t workspace_bytes,
                            int B, int H, int L, int Dk, int Dv,
                            float scale, float out_scale,
                            int io_dtype, int gate_dtype, void* stream);

/*
 * Backward of vig_gla_bidir_fwd: given d_o = dL/do [B, H, L, Dv], writes
 *   dq, dk [B, H, L, Dk], dv [B, H, L, Dv] (summed over the directions) in io_dtype and
 *   dg_fwd, dg_bwd [B, H, L, Dk] in gate_dtype (dg_bwd only when g_bwd != NULL).
 * `workspace` must hold vig_gla_bidir_bwd_workspace(...) bytes.
 * Built shapes: (Dk, Dv) in {(16,32), (32,32), (32,64), (64,32), (64,64)}, any L >= 1.
 * Dispatch: bf16 tensors + bf16 gates + Dk in {32, 64} + Dv = 64 (both directions, or the causal op with
 * g_bwd == NULL) -> matrix-core kernel (bf16 operands, fp32 accumulation; gradients within ~1e-2 of their largest
 * magnitude): one quadratic form per (batch, head) for L <= 256; a longer sequence as segments of <= 256 tokens linked
 * by their states (two state passes of the forward kernel, a segment scan, then one quadratic form per segment;
 * B*H*directions <= 65535).  A sequence with a segment whose gate total exceeds ~83 in some channel, and every other
 * case -> fp32-arithmetic token-recurrent kernel.
 *
 * Replaces: FusedChunkGLAFunction.backward (flash-linear-attention/fla/ops/gla/chunk_fuse.py:413-518; gate
 * gradient :505-518) under the flip-concat glue of classification/models/vig.py:407-426, for both directions in
 * natural token order.
 */
int vig_gla_bidir_bwd(const void* q, const void* k, const void* v,
                      const void* g_fwd, const void* g_bwd, const void* d_o,
                      void* dq, void* dk, void* dv, void* dg_fwd, void* dg_bwd,
                      void* workspace, size_t workspace_bytes,
                      int B, int H, int L, int Dk, int Dv,
                      float scale, float out_scale,
                      int io_dtype, int gate_dtype, void* stream);

size_t vig_gla_bidir_bwd_workspace(int B, int H, int L, int Dk, int Dv, int bidirectional);

/*
 * Workspace of the path vig_gla_bidir_bwd takes for exactly these dtypes.  It differs from the query above for
 * HierViG's head shape (Dk 16, Dv 32; classification/models/vig_h.py:521-527) with bf16 tensors and gates, both
 * directions and L >= 128: given this many bytes, the backward runs zero-padded to 32 / 64 channels on the matrix-core
 * kernels (inputs padded, gradients cropped; 20x faster than the token-recurrent kernel at L = 3136); given only the
 * smaller amount of the query above, it runs on the token-recurrent kernel.
 */
size_t vig_gla_bidir_bwd_workspace_for(int B, int H, int L, int Dk, int Dv, int io_dtype, int gate_dtype,
                                       int bidirectional);

/* Same contract as vig_gla_bidir_bwd, always the fp32-arithmetic token-recurrent kernel (the exact path). */
int vig_gla_bidir_bwd_exact(const void* q, const void* k, const void* v,
                            const void* g_fwd, const void* g_bwd, const void* d_o,
                            void* dq, void* dk, void* dv, void* dg_fwd, void* dg_bwd,
                            void* workspace, size_t workspace_bytes,
                            int B, int H, int L, int Dk, int Dv,
                            float scale, float out_scale,
                            int io_dtype, int gate_dtype, void* stream);

/*
 * Direction-wise gate preparation.
 *   gk_lin [B, L, 2*H*Dk]  ->  g_out [2, B, H, L, Dk]
 *   g_out[dir,b,h,l,d] = max(logsigmoid(gk_lin[b,l,dir*H*Dk + h*Dk + d]) * inv_normalizer, clamp_min)
 * clamp_min = NaN disables the clamp.  g_out[0] / g_out[1] are the g_fwd / g_bwd
 * arguments of vig_gla_bidir_fwd.
 *
 * Replaces: classification/models/vig.py:432-441 (chunk(2), cat, rearrange,
 * logsigmoid / gate_logit_normalizer, clamp_min).
 */
int vig_dirgate_fwd(const void* gk_lin, void* g_out, int B, int L, int H, int Dk,
                    float inv_normalizer, float clamp_min,
                    int in_dtype, int out_dtype, void* stream);

/*
 * Backward of vig_dirgate_fwd: d_g [2, B, H, L, Dk] (type out_dtype) -> d_gk_lin [B, L, 2*H*Dk] (type in_dtype),
 *   d_gk_lin = d_g * inv_normalizer * sigmoid(-gk_lin), zero where the forward clamped.
 *
 * Replaces: what autograd derives for classification/models/vig.py:368-371,411-414 (logsigmoid, division, clamp,
 * the direction split and the head rearrange).
 */
int vig_dirgate_bwd(const void* gk_lin, const void* d_g, void* d_gk_lin, int B, int L, int H, int Dk,
                    float inv_normalizer, float clamp_min, int in_dtype, int out_dtype, void* stream);

/*
 * Direction-wise gate preparation with the second layer of the low-rank gate projection inside:
 *   gk_low [B, L, rank] (token rows low_row_stride elements apart, 0 = packed), w_up [2*H*Dk, rank], b_up [2*H*Dk]
 *   x = gk_low . w_up^T + b_up, rounded to in_dtype (what the separate layer would have stored);
 *   g_out [2, B, H, L, Dk] as in vig_dirgate_fwd.  gk_low, w_up and b_up share in_dtype; rank must be 16; bases and
 *   row strides in bytes must be multiples of 16.  The [B, L, 2*H*Dk] intermediate never goes to memory.
 *
 * Replaces: the second nn.Linear of gk_proj (classification/models/vig.py:296-297, applied at vig.py:432) together
 * with vig.py:432-441.
 */
int vig_dirgate_lowrank_fwd(const void* gk_low, long long low_row_stride, const void* w_up, const void* b_up,
                            void* g_out, int B, int L, int H, int Dk, int rank, float inv_normalizer, float clamp_min,
                            int in_dtype, int out_dtype, void* stream);

/*
 * 3x3 depthwise convolution on the token grid, channels-last, zero padding 1.
 *   x [B, L=h*w, C], weight [C, 3, 3] (f32), bias [C] (f32) or NULL -> y [B, L, C]
 *   optional SiLU on the result.
 *
 * Replaces: the in_proj of GatedLinearAttention (classification/models/vig.py:
 * 291-294 applied at :428-430 with the two permutes around it).
 */
int vig_dwconv3x3_fwd(const void* x, const float* weight, const float* bias, void* y,
                      int B, int h, int w, int C, int silu, int io_dtype, void* stream);

/*
 * Weight and bias gradients of vig_dwconv3x3_fwd (without its SiLU) from x and dy [B, h*w, C]:
 *   dw_db fp32 [C*9 + C]: dw[c, ky, kx] = sum dy[b, y, x, c] * x[b, y+ky-1, x+kx-1, c], then db[c] = sum dy[b, y, x, c].
 * The input gradient needs no entry point of its own: it is vig_dwconv3x3_fwd on dy with the nine taps of every
 * channel mirrored through the centre.  `workspace` holds vig_dwconv3x3_bwd_weight_workspace(B, C) bytes
 * (per-workgroup partial sums, added in a fixed order: no atomics).
 *
 * Replaces: the convolution library's depthwise weight-gradient call behind classification/models/vig.py:291-294.
 */
size_t vig_dwconv3x3_bwd_weight_workspace(int B, int C);
int vig_dwconv3x3_bwd_weight(const void* x, const void* dy, float* dw_db, void* workspace, size_t workspace_bytes,
                             int B, int h, int w, int C, int io_dtype, void* stream);

/*
 * Synthetic locality gate of the ViG-B benchmark shape:
 *   y[b,hd,l,d] = o[b,hd,l,d] * sigmoid( dwconv3x3(o on the h x w grid, channel c = hd*Dv+d) )
 * o, y: [B, H, L=h*w, Dv]; weight [H*Dv, 3, 3] f32.  In-place (y == o) is NOT allowed.
 */
int vig_locality_gate_fwd(const void* o, const float* weight, void* y,
                          int B, int H, int h, int w, int Dv, int io_dtype, void* stream);

/*
 * vig_gla_bidir_fwd and vig_locality_gate_fwd in one kernel: the GLA output o = out_scale * (o_fwd + o_bwd) is
 * rounded to bf16, staged on chip, and y = o * sigmoid(dwconv3x3(o)) is what reaches memory (bit-identical to the
 * two calls in a row).  Same tensors as vig_gla_bidir_fwd; weight [H*Dv, 3, 3] f32; L = grid_h * grid_w.
 * Built for bf16 tensors and gates, Dk in {32, 64}, Dv = 64, L <= 256, both directions, and token grids with
 * grid_w <= 62 and grid_h + 2 <= 8 * floor(64 / (grid_w + 2)) (14x14 and 16x16 are); VIG_ENOTSUP otherwise
 * (the caller then makes the two calls).  No workspace.
 *
 * Replaces: the GLA call of classification/models/vig.py:442 followed by the benchmark's sigmoid locality gate
 * (the synthetic restatement of vig.py:291-294,447-454 on the op's own output).
 */
int vig_gla_bidir_locgate_fwd(const void* q, const void* k, const void* v, const void* g_fwd, const void* g_bwd,
                              const float* gate_weight, void* y, int B, int H, int L, int Dk, int Dv,
                              int grid_h, int grid_w, float scale, float out_scale, int io_dtype, int gate_dtype,
                              void* stream);

/*
 * Block epilogue before o_proj:
 *   y[b,l,hd*Dv+d] = rms(o[b,hd,l,:])*w_g * s + rms(local[b,l,hd,:])*w_l * (1-s),  s = sigmoid(g_lin[b,l,hd*Dv+d])
 *   rms(x) = x * rsqrt(mean(x^2) + eps); optional SiLU on y.
 * o [B,H,L,Dv]; local, g_lin, y [B, L, H*Dv]; w_g, w_l [Dv] f32.
 * g_row_stride: elements between consecutive token rows of g_lin (0 = packed, H*Dv), so that g_lin may be a block
 * of columns of a wider projection output; the base and the stride in bytes must be multiples of 16.
 *
 * Replaces: classification/models/vig.py:444-457 (two RMSNorm launches
 * fla/modules/rmsnorm.py:69-125, three rearranges, sigmoid blend, out_act).
 */
int vig_locality_blend_fwd(const void* o, const void* local, const void* g_lin,
                           const float* w_g, const float* w_l, void* y,
                           int B, int H, int L, int Dv, long long g_row_stride, float eps, int silu_out,
                           int io_dtype, void* stream);

/*
 * Backward of vig_locality_blend_fwd from the forward's inputs and dy [B, L, H*Dv]:
 *   d_o [B, H, L, Dv], d_local and d_glin [B, L, H*Dv] (packed), dw fp32 [2, Dv] = (gradient of w_g | of w_l).
 * With s = sigmoid(g_lin), on = rms(o) * w_g, ln = rms(local) * w_l, y0 = on * s + ln * (1 - s):
 *   dy0 = dy * d(y)/d(y0) (SiLU derivative when silu_out), d_on = dy0 * s, d_ln = dy0 * (1 - s),
 *   d_glin = dy0 * (on - ln) * s * (1 - s); d_o and d_local are the RMS-norm backward of d_on and d_ln per
 *   (token, head) row; dw sums d_on * o * r_o and d_ln * local * r_l over batch, tokens and heads.
 * `workspace` holds vig_locality_blend_bwd_workspace(B, L, Dv) bytes (per-workgroup partial sums of dw, added in a
 * fixed order: no atomics).
 *
 * Replaces: what autograd derives for classification/models/vig.py:447-457 in the reference (two fused RMS-norm
 * backward launches, rmsnorm.py:203-296, and the elementwise chain of the blend).
 */
size_t vig_locality_blend_bwd_workspace(int B, int L, int Dv);
int vig_locality_blend_bwd(const void* o, const void* local, const void* g_lin, const float* w_g, const float* w_l,
                           const void* dy, void* d_o, void* d_local, void* d_glin, float* dw, void* workspace,
                           size_t workspace_bytes, int B, int H, int L, int Dv, long long g_row_stride, float eps,
                           int silu_out, int io_dtype, void* stream);

/*
 * Residual-add + RMS norm over the last dimension (rows x C, C % 8 == 0, C <= 4096):
 *   s = x (+ residual) in fp32;  residual_out = s (if not NULL);  y = s * rsqrt(mean(s^2) + eps) * weight
 * residual and residual_out may be NULL; weight [C] f32.  round_sum != 0 first rounds s to the storage
 * type and normalises the rounded value (what `norm(a + b)` on stored tensors computes); round_sum == 0
 * is the fused kernel's arithmetic (the unrounded sum is normalised).
 *
 * Replaces: flash-linear-attention/fla/modules/rmsnorm.py:69-125 (_layer_norm_fwd_1pass_kernel with
 * IS_RMS_NORM, HAS_RESIDUAL, STORE_RESIDUAL_OUT) as used at classification/models/vig.py:598,602-606,896.
 */
int vig_rmsnorm_fwd(const void* x, const void* residual, const float* weight, void* y, void* residual_out,
                    long long rows, int C, float eps, int round_sum, int io_dtype, void* stream);

/*
 * LayerNorm over the last dimension (rows x C, C % 8 == 0, C <= 4096), optional SiLU behind it:
 *   y = (x - mean) * rsqrt(var + eps) * weight + bias   (biased variance, fp32 arithmetic; weight, bias [C] f32)
 *   silu != 0:  y = r * sigmoid(r) with r the normalised value rounded to the storage type
 *   pre_bias [C] f32 or NULL: x + pre_bias, rounded to the storage type, is what gets normalised (the bias of the
 *     convolution in front of the norm);
 *   post_add [post_rows, C] (io dtype) or NULL: row r of the (rounded) result gets post_add[r % post_rows] added
 *     (the position table behind the last norm, post_rows = tokens per image).
 * x and y may be the same buffer.
 *
 * Replaces: LayerNorm2d of the v2 patch embedding on a channels-last feature map with the bias add of the
 * convolution before it, the swish that follows the first one (classification/models/vig.py:619-624, 650-655) and
 * the position-table add behind the second (vig.py:858-865).
 */
int vig_layernorm_fwd(const void* x, const float* weight, const float* bias, void* y, long long rows, int C,
                      float eps, int silu, const float* pre_bias, const void* post_add, int post_rows, int io_dtype,
                      void* stream);

/*
 * Head-major split of the fused q/k/v projection:
 *   qkv [B, L, H*Dk | H*Dk | H*Dv]  ->  q, k [B, H, L, Dk],  v [B, H, L, Dv]   (Dk, Dv multiples of 8)
 * qkv_row_stride: elements between consecutive token rows of qkv (0 = packed), so that qkv may be the leading
 * columns of a wider projection output; the base and the stride in bytes must be multiples of 16.
 *
 * Replaces: classification/models/vig.py:401-409 (torch.split and the three 'b l (h d) -> b h l d'
 * rearranges in front of the GLA op).
 */
int vig_split_heads_fwd(const void* qkv, void* q, void* k, void* v, int B, int L, int H, int Dk, int Dv,
                        long long qkv_row_stride, int io_dtype, void* stream);

/*
 * Backward of vig_split_heads_fwd: dq, dk [B, H, L, Dk] and dv [B, H, L, Dv] gathered into d_qkv
 * [B, L, H*(2*Dk+Dv)] (packed rows), one pass.
 *
 * Replaces: what autograd derives for classification/models/vig.py:401-409 (three rearranges back and a concat).
 */
int vig_split_heads_bwd(const void* dq, const void* dk, const void* dv, void* d_qkv, int B, int L, int H, int Dk,
                        int Dv, int io_dtype, void* stream);

/*
 * SwiGLU product of the MLP:  gate_up [rows, 2*I] = (gate | up)  ->  out [rows, I] = gate * up / (1 + exp(-gate))
 *
 * Replaces: swiglu_fwd (flash-linear-attention/fla/modules/activations.py:109-113) on the two halves of
 * gate_proj's output (classification/models/vig.py:492-495).
 */
int vig_swiglu_fwd(const void* gate_up, void* out, long long rows, int I, int io_dtype, void* stream);

/*
 * Backward of vig_swiglu_fwd: d_gate_up [rows, 2*I] = (d_gate | d_up) from the forward's input and dy [rows, I]:
 *   d_gate = dy * up * sig(gate) * (1 + gate * (1 - sig(gate))),  d_up = dy * gate * sig(gate).
 *
 * Replaces: swiglu_bwd (flash-linear-attention/fla/modules/activations.py:113-119, used by SwiGLUFunction :137-148).
 */
int vig_swiglu_bwd(const void* gate_up, const void* dy, void* d_gate_up, long long rows, int I, int io_dtype,
                   void* stream);

/*
 * Backward of vig_rmsnorm_fwd.  `sum` [rows, C] is the tensor the forward normalised (x, or the x + residual it
 * returned), dy the gradient of y, d_sum (may be NULL) the gradient that arrives at the returned sum:
 *   r = rsqrt(mean(sum^2) + eps),  g = dy * weight,
 *   ds = r * (g - sum * r^2 * mean(g * sum)) + d_sum     -- the gradient of x and of the residual alike
 *   dweight[c] = sum over rows of dy[c] * sum[c] * r     -- fp32 [C]; NULL skips it (and needs no workspace)
 * `workspace` holds vig_rmsnorm_bwd_workspace(rows, C) bytes of per-workgroup partial sums; the result does not
 * depend on scheduling (no atomics).  C % 8 == 0, C <= 1024.
 *
 * Replaces: _layer_norm_bwd_kernel in its RMS mode with residual
 * (flash-linear-attention/fla/modules/rmsnorm.py:203-296, driver :300-387).
 */
size_t vig_rmsnorm_bwd_workspace(long long rows, int C);
int vig_rmsnorm_bwd(const void* sum, const float* weight, const void* dy, const void* d_sum, void* ds, float* dweight,
                    void* workspace, size_t workspace_bytes, long long rows, int C, float eps, int io_dtype,
                    void* stream);

/*
 * gate_proj and the SwiGLU product in one kernel, for a short contraction (K = 384 or 192, the hidden sizes of
 * ViG-S / ViG-T), bf16, fp32 accumulation:
 *   y [rows, I] = swiglu(gate, up) with (gate | up) = x [rows, K] . weight [2*I, K]^T, the product taken on gate and
 *   up rounded to bf16 (what the separate layer stores); I % 32 == 0; x, weight and y packed row-major.
 * Other K or dtypes return VIG_ENOTSUP (use a GEMM library and vig_swiglu_fwd).
 *
 * Replaces: gate_proj followed by swiglu (classification/models/vig.py:492-495,
 * flash-linear-attention/fla/modules/activations.py:109-113) without the [rows, 2*I] intermediate.
 */
int vig_linear_swiglu_fwd(const void* x, const void* weight, void* y, long long rows, int K, int I, int io_dtype,
                          void* stream);

/*
 * vig_locality_blend_fwd and o_proj in one kernel, for square blocks with 64-channel heads at the widths whose weight
 * tiles fit the registers (C = H*Dv = 384 or 192, the hidden sizes of ViG-S / ViG-T), bf16, fp32 accumulation:
 *   out [B*L, C] = y . weight [C, H*Dv]^T with y the blend above, rounded to bf16 as vig_locality_blend_fwd stores
 *   it; y itself is never written.  Arguments as in vig_locality_blend_fwd (Dv = 64, g_row_stride likewise);
 *   weight and out packed row-major.  Other shapes or dtypes return VIG_ENOTSUP (make the two calls).
 *
 * Replaces: classification/models/vig.py:444-463 (head norms, sigmoid blend, out_act, o_proj) without the
 * [B, L, H*Dv] intermediate.
 */
int vig_locality_blend_linear_fwd(const void* o, const void* local, const void* g_lin,
                                  const float* w_g, const float* w_l, const void* weight, void* out,
                                  int B, int H, int L, int Dv, int C, long long g_row_stride, float eps, int silu_out,
                                  int io_dtype, void* stream);

/*
 * First convolution of the v2 patch embedding, without its bias (vig_layernorm_fwd's pre_bias takes that):
 *   x [B, Cin, H, W] (bf16, the layout images arrive in)  ->  y [B, OH, OW, Cout] (bf16, channels-last rows),
 *   OH = (H + 2*padding - KH) / stride + 1, OW likewise.
 *   w_packed [Cout, Cin*KH, 16] bf16: the kernel rows of the [Cout, Cin, KH, KW] weight, each padded with zeros to
 *   16 columns.
 * Built for the reference's stem: stride 8, padding 1, KW <= 16, Cin*KH = 27 (3 channels x 9 rows), W % 8 == 0,
 * W <= 248, Cout a multiple of 32 from 64 to 256; anything else returns VIG_ENOTSUP (use a library convolution).
 *
 * Replaces: the first nn.Conv2d of V2PatchEmbed (classification/models/vig.py:651) and the layout change a
 * channels-last convolution library needs in front of it.
 */
int vig_patch_conv_fwd(const void* x, const void* w_packed, void* y, int B, int Cin, int H, int W, int KH, int KW,
                       int stride, int padding, int Cout, int io_dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* VIG_GLA_H_ */
