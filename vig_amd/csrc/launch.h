// Host-side argument block and launcher prototypes shared by the C ABI and the kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

namespace vig {

struct GlaArgs {
  const void* q;
  const void* k;
  const void* v;
  const void* g_fwd;
  const void* g_bwd;  // may be null: forward direction only
  void* o;
  void* workspace;
  size_t workspace_bytes;
  int B, H, L, Dk, Dv;
  float scale, out_scale;
  int io_dtype, gate_dtype;  // 0 = f32, 1 = bf16
  hipStream_t stream;
  // fused locality gate (bf16 MFMA path only): o * sigmoid(conv3x3(o)) on the gate_rows x gate_cols token grid is
  // stored instead of o; weights [H*Dv, 9] f32.  Null: plain output.
  const float* gate_w = nullptr;
  int gate_rows = 0, gate_cols = 0;
  // bf16 MFMA path: the caller expects gates beyond the fp16 score variant's range (|chunk total| > ~8 nat in some
  // channel): start with the split-bf16 variant instead of finding out on the first segment of every workgroup
  int wide_gates = 0;
  // causal op only (g_bwd null): fp32 [B, H, Dk, Dv] state before the first token / after the last one; null: zero / not wanted
  const float* init_state = nullptr;
  float* final_state = nullptr;
  // bf16 MFMA path, any L: run state passes alone into `workspace`, per (sequence, segment, direction)
  // kGlaStateFloats floats, no scan, no outputs.  1: the forward's pass on (k, v, gates).  2 (both directions only):
  // that pass and, behind its slots, the gradient-state pass of the backward on (q for k, `o` read as the output
  // gradient for v, the two directions' gates exchanged, cumulative gates exclusive of each token's own gate).
  int state_pass = 0;
  // bf16 MFMA path: q, k, v that are not plain [B, H, L, D] tensors: element strides (batch, head, token) with the
  // channels of a (token, head) contiguous, e.g. column blocks of a projection output [B, L, H*(2*Dk + Dv)] read in
  // place.  Null (or token stride 0): plain layout.  Strides are multiples of 8 elements.
  const long long* q_strides = nullptr;
  const long long* k_strides = nullptr;
  const long long* v_strides = nullptr;
};

// Per (sequence, segment, direction) slot of a state pass: the 64 x 64 state contribution in the matrix cores' register
// order (element ((u*64 + lane)*4 + m): unit u = (pk*2 + pv)*4 + cq), then the segment's 64 per-channel decays.
constexpr int kGlaStateFloats = 64 * 64 + 64;
// Segments of a long sequence: ceil(L / 256) of them, ceil(L / nseg) tokens each (the last one possibly fewer).
inline int gla_segments(int L) { return (L + 255) / 256; }
inline int gla_segment_len(int L) { return (L + gla_segments(L) - 1) / gla_segments(L); }
// The forward of a long sequence, when its output pass is the tile-pair kernel: segments of whole 32-token tiles, at
// most 7 of them (one wave each, two workgroups per CU); the last segment of a sequence may hold fewer tokens, down to
// none in its trailing tiles.
inline int gla_tile_segments(int L) { return (L + 223) / 224; }
inline int gla_tile_segment_tiles(int L) { return ((L + gla_tile_segments(L) - 1) / gla_tile_segments(L) + 31) / 32; }
// Behind the state slots of a scanned workspace: per (sequence, direction) 16 partial maxima of |state entering a
// segment| (one per block of the scan), for consumers that read the states as fp16.
constexpr int kGlaScanMaxima = 16;

// fp32-arithmetic token-recurrent path (any supported dtype combination).
int launch_gla_recurrent(const GlaArgs& a);
size_t gla_recurrent_workspace(int B, int H, int L, int Dv, int io_dtype);

// bf16 MFMA chunked path (bf16 io and gates).
bool gla_mfma_supported(const GlaArgs& a);
int launch_gla_mfma(const GlaArgs& a);
// bf16 tile-pair path for whole-sequence slabs (L <= 256): one wave per 32-token tile, both directions per wave.
bool gla_tiles_supported(const GlaArgs& a);
int launch_gla_tiles(const GlaArgs& a);
// the same kernel as the output pass of a long sequence (L > 256): one workgroup per (sequence, segment), the states
// entering the segments (scanned slots, kGlaStateFloats floats per (sequence, segment, direction)) and their maxima
// (kGlaScanMaxima floats per (sequence, direction)) in `states` / `maxima`
bool gla_tiles_chain_supported(const GlaArgs& a);
int launch_gla_tiles_chain(const GlaArgs& a, const float* states, const float* maxima);
bool gla_mfma_gate_grid_ok(int rows, int cols);  // token grids the fused locality gate takes
size_t gla_mfma_workspace(int B, int H, int L, int Dk, int Dv);
size_t gla_mfma_state_workspace(int B, int H, int L, int Dk, int Dv);  // causal op with an initial / final state

// bf16 matrix-core backward (quadratic form per slab, or per <= 256-token segment of a longer sequence with the
// segments chained through states); flags[b*H + h] = 1 marks sequences it left to the recurrent kernel.
// seg_workspace: gla_backward_mfma_workspace() bytes, used for L > 256 only.
bool gla_backward_mfma_supported(int B, int H, int L, int Dk, int Dv, int io_dtype, int gate_dtype, bool bidir);
size_t gla_backward_mfma_workspace(int B, int H, int L, int Dk, int Dv);
int launch_gla_backward_mfma(const void* q, const void* k, const void* v, const void* gf, const void* gb,
                             const void* d_o, void* dq, void* dk, void* dv, void* dgf, void* dgb, int* flags,
                             void* seg_workspace, int B, int H, int L, int Dk, float s, hipStream_t stream);

}  // namespace vig
