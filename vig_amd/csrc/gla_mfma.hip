// bf16 MFMA chunked path: placeholder until the kernel lands.
#include "common.h"
#include "launch.h"
namespace vig {
bool gla_mfma_supported(const GlaArgs&) { return false; }
int launch_gla_mfma(const GlaArgs&) { return -95; }
size_t gla_mfma_workspace(int, int, int, int, int) { return 0; }
}  // namespace vig
