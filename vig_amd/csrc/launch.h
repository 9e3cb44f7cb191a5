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
};

// fp32-arithmetic token-recurrent path (any supported dtype combination).
int launch_gla_recurrent(const GlaArgs& a);
size_t gla_recurrent_workspace(int B, int H, int L, int Dv, int io_dtype);

// bf16 MFMA chunked path (bf16 io and gates).
bool gla_mfma_supported(const GlaArgs& a);
int launch_gla_mfma(const GlaArgs& a);
size_t gla_mfma_workspace(int B, int H, int L, int Dk, int Dv);

}  // namespace vig
