// Kernel argument blocks and launchers shared between translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "va_device.h"

namespace va {

struct AttnArgs {
  const void* q;
  long long q_row_stride;  // elements between query rows
  const void* k_pool;
  const void* v_pool;
  long long pool_row_stride;  // elements between token slots
  const int32_t* items;
  const int32_t* links;
  const int32_t* qrefs;
  const int32_t* kv_indices;
  const int64_t* sub_worker;
  const int64_t* sub_loc;
  long long sub_loc_axis_stride;
  void* out;
  float* lse;
  int lse_base2;
  float* part_acc;  // [n_partials, Hq, D]
  float* part_ml;   // [n_partials, Hq, 2]  (running max in log2 units, sum)
  int num_q_heads, num_kv_heads, head_dim, page_size;
  RopeDev rope;
  float scale_log2;  // log2(e) / sqrt(head_dim)
  const int32_t* qref_rows;  // sub_worker[qrefs[k]], precomputed by the planner
  const int32_t* wide_slots;  // [n_wide_slots + 1]: the wide items each workgroup of the wide launch runs
};

struct MergeArgs {
  const int32_t* row_indptr;
  const int32_t* row_ids;
  const int32_t* row_flags;
  const float* part_acc;
  const float* part_ml;
  void* out;
  float* lse;
  int lse_base2;
  int num_q_heads, head_dim;
};

// Validate a rotation description and turn it into its device form.
int make_rope(const VaRope* rope, int head_dim, RopeDev* out);

// Matrix-core attention (launched from va_mfma.hip).
// `n_wide` leading items are wide tiles (va_mfma_wide.hip: `n_wide_slots` workgroups per kv head, each
// running the items a.wide_slots gives it), the rest narrow ones (va_mfma_stream.hip).
int launch_mfma(const AttnArgs& a, int dtype, int n_items, int n_wide, int n_wide_slots, int q_tile,
                hipStream_t stream);
int launch_mfma_wide(const AttnArgs& a, int dtype, int n_slots, hipStream_t stream);
int launch_mfma_stream(const AttnArgs& a, int dtype, int n_items, hipStream_t stream);

}  // namespace va
