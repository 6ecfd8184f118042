// Matrix-core (MFMA) attention kernels for 16-bit element types.
#include <hip/hip_runtime.h>

#include "va_internal.h"
#include "va_launch.h"

bool va_mfma_supported(int dtype, int head_dim, int gqa) {
  (void)dtype; (void)head_dim; (void)gqa;
  return false;
}
int va_mfma_max_q_tile(int gqa) { return 16 / (gqa > 16 ? 16 : gqa); }
int va_mfma_default_q_tile(int gqa, bool has_chain) { (void)has_chain; return va_mfma_max_q_tile(gqa); }

namespace va {
int launch_mfma(const AttnArgs&, int, int, int, hipStream_t) {
  return va_fail(VA_ERR_ARG, "matrix-core path not available for this configuration");
}
}  // namespace va
