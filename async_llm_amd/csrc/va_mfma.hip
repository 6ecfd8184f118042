// Matrix-core (MFMA) view attention for 16-bit element types on gfx950: eligibility, tile
// limits and the launch of the two kernels.
//
//   * streaming kernel (va_mfma_stream.hip): query tiles of up to 16 MFMA rows (row = tile row
//     R / G, head R % G with G = q heads per kv head), i.e. decode tiles of 16/G requests that
//     read the same KV run, and short prefill tiles.  Bound by HBM.
//   * wide kernel (va_mfma_wide.hip): query tiles of up to 128 MFMA rows for view-conditioned
//     prefill.  Bound by the matrix pipe.
// A plan lists its wide items first; each kind gets one launch.
#include <hip/hip_runtime.h>

#include "va_internal.h"
#include "va_launch.h"

bool va_mfma_supported(int dtype, int head_dim, int gqa) {
  if (dtype != VA_BF16 && dtype != VA_F16) return false;
  if (head_dim != 64 && head_dim != 128 && head_dim != 256) return false;
  return gqa == 1 || gqa == 2 || gqa == 4 || gqa == 8 || gqa == 16;
}
int va_mfma_max_q_tile(int gqa) { return 16 / gqa; }
int va_mfma_default_q_tile(int gqa, bool has_chain) {
  (void)has_chain;
  return 16 / gqa;
}
int va_mfma_wide_q_tile(int gqa, int head_dim) { return (head_dim == 256 ? 128 : 256) / gqa; }

namespace va {

int launch_mfma(const AttnArgs& a_in, int dtype, int n_items, int n_wide, int n_wide_slots, int q_tile,
                hipStream_t stream) {
  AttnArgs a = a_in;
  const int g = a.num_q_heads / a.num_kv_heads;
  if (!va_mfma_supported(dtype, a.head_dim, g))
    return va_fail(VA_ERR_ARG, "matrix-core path does not support this dtype/head_dim/group size");
  if (q_tile * g > 16) return va_fail(VA_ERR_ARG, "plan tile of %d rows x %d heads exceeds 16 MFMA rows", q_tile, g);
  if (a.rope.rotary_dim % 16) return va_fail(VA_ERR_ARG, "matrix-core path needs rotary_dim to be a multiple of 16");
  if (a.q_row_stride % 8 || a.pool_row_stride % 8 || (uintptr_t)a.q % 16 || (uintptr_t)a.k_pool % 16 ||
      (uintptr_t)a.v_pool % 16)
    return va_fail(VA_ERR_ARG, "matrix-core path needs 16-byte aligned rows");
  // the query staging reads the cos|sin entries of a unit in 16-byte loads
  if (a.rope.mode == VA_ROPE_TABLE && a.rope.rotary_dim > 0 && (uintptr_t)a.rope.cos_sin % 16)
    return va_fail(VA_ERR_ARG, "matrix-core path needs a 16-byte aligned cos|sin table");
  // the streaming kernel addresses a tile's rows with 32-bit byte offsets from its first row
  if (a.pool_row_stride * 2 * 16 > 0x7fffffffLL) return va_fail(VA_ERR_ARG, "pool rows too far apart");
  if (n_wide > 0 && n_wide_slots > 0) {
    const int rc = launch_mfma_wide(a, dtype, n_wide_slots, stream);
    if (rc) return rc;
  }
  a.items += (long long)n_wide * VA_ITEM_WORDS;
  return launch_mfma_stream(a, dtype, n_items - n_wide, stream);
}

}  // namespace va
