/*
 * viewattn.h -- C ABI of libviewattn.so: cache-view attention for MI355X (gfx950).
 *
 * The library replaces, for AsyncLLM's view-attention path, everything the
 * reference hands to third-party CUDA code or to torch elementwise ops inside
 * SharedCacheAttention.forward:
 *
 *   reference (python/minisgl/...)                          entry point here
 *   ------------------------------------------------------  ------------------
 *   shared_cache/rope_correction.py:15-54,                  va_rope
 *     shared_cache/attention.py:241-280 (_rope/_rope_mrope)
 *   attention.py:645-649 + kernel/store.py:30-42 +          va_store_kv_rope
 *     kernel/csrc/jit/store.cu:27-125 (K rotate + KV store)
 *   FlashInfer wrapper.plan(...) attention.py:390-426,      va_plan_count,
 *     574-604 (work decomposition of the planned tables)    va_plan_build
 *   attention.py:652-703 (q gather + per-segment rotate,    va_attention
 *     BatchDecode run x2, pad-scatter, merge_states) and
 *     attention.py:705-752 (BatchPrefill run x2, merge)
 *   attention_graph.py:14-290 (fixed-capacity graph        va_plan_capacity,
 *     buffers) + attention.py:212-239 (workspace sizing)    va_plan_fixed_words,
 *                                                           va_plan_build_fixed
 *   session.py:470-528 (block merge / append: KV copy and   va_copy_shift_kv
 *     key shift into the left block's position frame)
 *
 * Conventions: every function returns 0 on success or a negative VA_ERR_*;
 * va_last_error() returns a thread-local message for the last failure.  All
 * pointers named *_dev are device pointers on the current HIP device; *_host are
 * host pointers.  The library allocates nothing: the caller owns every buffer
 * (workspace included) and the stream.  Its only state besides the last error
 * message is the scratch array of va_attention_static (one copy per GPU).
 * `stream` is a hipStream_t passed as void*.
 */
#ifndef VIEWATTN_H
#define VIEWATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#define VA_API __attribute__((visibility("default")))
#else
#define VA_API
#endif

#define VA_OK 0
#define VA_ERR_ARG (-1)       /* inconsistent or unsupported argument */
#define VA_ERR_CAPACITY (-2)  /* caller-provided buffer too small */
#define VA_ERR_HIP (-3)       /* a HIP runtime call failed */

/* element types of q/k/v/out and of the KV pool */
#define VA_F32 0
#define VA_F16 1
#define VA_BF16 2

/* rotation modes */
#define VA_ROPE_TABLE 0 /* 1-D neox RoPE from an fp32 cos|sin table (rope_correction.py) */
#define VA_ROPE_MROPE 1 /* interleaved 3-axis mRoPE, cos/sin computed from inv_freq      */

/* kernel families for va_attention / va_plan_* */
#define VA_KERNEL_AUTO 0
#define VA_KERNEL_GENERIC 1 /* vector-ALU path, any dtype                            */
#define VA_KERNEL_MFMA 2    /* bf16/f16 matrix-core path                             */

typedef struct VaShape {
  int32_t num_q_heads;
  int32_t num_kv_heads;
  int32_t head_dim;
  int32_t page_size; /* tokens per page of the pool */
  int32_t dtype;     /* VA_F32 / VA_F16 / VA_BF16 */
} VaShape;

typedef struct VaRope {
  int32_t mode;          /* VA_ROPE_TABLE / VA_ROPE_MROPE */
  int32_t rotary_dim;    /* leading head dims that rotate (pairs i, i+rotary_dim/2) */
  const float* cos_sin_dev; /* [max_pos, rotary_dim] fp32: cos | sin  (TABLE)       */
  int32_t max_pos;       /* rows of the table; |position| is clamped to max_pos-1  */
  int32_t section_h;     /* mrope_section[1] (MROPE)                                */
  int32_t section_w;     /* mrope_section[2] (MROPE)                                */
  const float* inv_freq_dev; /* [rotary_dim/2] fp32 (MROPE)                         */
} VaRope;

VA_API const char* va_last_error(void);
VA_API int va_version(void);

/*
 * va_rope: y[i, h, :] = R(pos[i]) x[i, h, :] for i < n_rows, h < n_heads.
 * pos_dev is int64 [n_rows] (pos_axis_stride == 0) or [3, n_rows] with
 * pos_axis_stride elements between axes (mRoPE with genuine 3-D positions).
 * x/y rows are x_row_stride / y_row_stride ELEMENTS apart; heads are
 * contiguous (head_dim apart).  In-place (y == x) is allowed.
 * Replaces rope_correction.py:15-54 and attention.py:241-280.
 */
VA_API int va_rope(const void* x_dev, void* y_dev, const int64_t* pos_dev, int64_t pos_axis_stride,
            int64_t n_rows, int32_t n_heads, int32_t head_dim, int32_t dtype,
            int64_t x_row_stride, int64_t y_row_stride, const VaRope* rope, void* stream);

/*
 * va_store_kv_rope: for every row i with out_loc[i] >= 0 write
 *   k_pool[out_loc[i]] = R(pos[i]) k[i]   and   v_pool[out_loc[i]] = v[i]
 * (rows with a negative slot are skipped: store.cu:44-46).  out_loc is int32 or
 * int64 (out_loc_is_i64).  Pool rows are pool_row_stride elements apart and
 * hold num_kv_heads*head_dim elements.  Replaces attention.py:645-649 +
 * store.cu:27-57 in one pass (the rotated key is never materialised).
 */
VA_API int va_store_kv_rope(const void* k_dev, const void* v_dev, int64_t k_row_stride,
                     int64_t v_row_stride, void* k_pool_dev, void* v_pool_dev,
                     int64_t pool_row_stride, const void* out_loc_dev, int32_t out_loc_is_i64,
                     const int64_t* pos_dev, int64_t pos_axis_stride, int64_t n_rows,
                     const VaShape* shape, const VaRope* rope, void* stream);

/* ---------------------------------------------------------------------------
 * Work decomposition (host).  Input: the planned sub-request tables, exactly the
 * integer tensors the reference hands to FlashInfer's plan():
 *   sub-request s reads KV entries kv_indptr[s]..kv_indptr[s+1] of kv_indices
 *   (page numbers, or token slots when VA_SUB_SLOTS is set: the page_size=1
 *   aux wrapper of attention.py:412-426), seq_lens[s] tokens, and serves the
 *   query sub-rows qo_indptr[s]..qo_indptr[s+1] (indices into sub_worker /
 *   sub_loc).  flags[s]: VA_SUB_CAUSAL = bottom-right aligned causal mask
 *   (attention.py:586-602).  chain[s] >= 0 ties the sub-requests of one prefill
 *   request together (same query rows, merged in-kernel); chain[s] < 0 marks a
 *   stand-alone (decode) sub-request, which may be batched with other
 *   sub-requests that read the identical page list.
 * ------------------------------------------------------------------------- */
#define VA_SUB_CAUSAL 1
#define VA_SUB_SLOTS 2

typedef struct VaSubRequests {
  int32_t n_sub;
  int32_t n_subrows;          /* == qo_indptr[n_sub] */
  int32_t n_rows;             /* output rows (workers / new tokens) */
  const int32_t* qo_indptr;   /* [n_sub+1] host */
  const int32_t* kv_indptr;   /* [n_sub+1] host */
  const int32_t* kv_indices;  /* [kv_indptr[n_sub]] host; NULL when the table only exists on the
                                 device: readers of one KV list are then not batched into shared tiles */
  const int32_t* seq_lens;    /* [n_sub] host */
  const int32_t* flags;       /* [n_sub] host */
  const int32_t* chain;       /* [n_sub] host */
  const int64_t* sub_worker;  /* [n_subrows] host: output row of each sub-row */
} VaSubRequests;

typedef struct VaPlanParams {
  int32_t kernel;        /* VA_KERNEL_*; AUTO picks by dtype/shape            */
  int32_t q_tile;        /* 0 = library default for the chosen kernel         */
  int32_t kv_chunk;      /* 0 = derive from the launch's total KV tokens      */
  int32_t target_items;  /* 0 = default (work items wanted per kv head)       */
  int32_t wide_tile;     /* rows of a wide query tile: 0 = default (prefill tiles; decode readers of one
                            block only where the re-reads saved outweigh a second launch), >0 = this many
                            rows, decode readers included, <0 = never */
} VaPlanParams;

typedef struct VaPlanCounts {
  int32_t kernel;        /* resolved kernel family */
  int32_t q_tile;        /* resolved */
  int32_t kv_chunk;      /* resolved */
  int32_t n_items;       /* work items incl. padding (multiple of 8) */
  int32_t n_links;
  int32_t n_qrefs;
  int32_t n_partials;    /* partial (row, item) slots the launch will write */
  int32_t n_row_parts;   /* length of row_part_ids */
  int32_t plan_words;    /* int32 words va_plan_build writes                 */
  int32_t wide_tile;     /* resolved rows of a wide tile (0: none)           */
  int32_t n_wide_items;  /* items served by the wide kernel                  */
  int64_t workspace_bytes; /* device scratch va_attention needs for this plan */
  int32_t n_wide_slots;  /* workgroups per kv head of the wide launch (a multiple of 8): a slot
                            runs one wide item, or several pieces of equal total length */
} VaPlanCounts;

/* Size the plan (no output besides *counts). */
VA_API int va_plan_count(const VaSubRequests* subs, const VaShape* shape, const VaPlanParams* params,
                  VaPlanCounts* counts);

/*
 * Build the plan into plan_host (capacity plan_capacity_words int32 words, at
 * least counts->plan_words).  The blob is position independent: copy it to the
 * device verbatim and pass the device copy to va_attention.  Layout (int32
 * words): header[24] | items[n_items*16] | links[n_links*8] | qrefs[n_qrefs] |
 * qref_rows[n_qrefs] | row_part_indptr[n_rows+1] | row_part_ids[n_row_parts] |
 * row_flags[n_rows] | wide_slots[n_wide_slots+1].  (An item carries a copy of its first link, and qref_rows
 * the output row of every qrefs entry: both shorten the chain of dependent loads
 * at the start of a workgroup.)
 * A link whose token range no other query tile of the launch reads carries the
 * flag "read once" (its rows are then requested as non-temporal loads, which
 * stream through the die's L2 as lines to evict first); the header also holds
 * the number of waves per workgroup of the merge launch, chosen from the
 * partial states per row (from the capacity, for a fixed plan).
 * Items are in launch order, laid out for the 8 dies of an MI355X (workgroup b
 * of a launch runs on die b % 8): wide items first, then narrow ones, each
 * class padded with empty items (n_q = 0) to a multiple of 8; n_items and
 * n_wide_items count the padding.  A caller may skip va_plan_count and build
 * into a buffer of its own guess: when it is too small the call returns
 * VA_ERR_CAPACITY and *counts holds the size to retry with.
 */
VA_API int va_plan_build(const VaSubRequests* subs, const VaShape* shape, const VaPlanParams* params,
                  int32_t* plan_host, int64_t plan_capacity_words, VaPlanCounts* counts);

/*
 * Fixed-capacity plans, for launches that are recorded once and replayed (HIP
 * graphs): the reference keeps such plans in fixed slot geometry
 * (shared_cache/attention_graph.py:14-121 decode, :127-290 prefill; workspace
 * sizing attention.py:212-239).  Here the geometry that must not change between
 * replays is what va_attention derives from the plan header: the number of
 * workgroups of each launch, the merge grid and the section offsets.
 * va_plan_build_fixed lays the sections out at offsets given by `capacity` alone
 * and pads the item lists with empty items, so every plan built with the same
 * capacity has the same header and va_attention issues the same launches on the
 * same buffers; only the contents of the plan blob (and of kv_indices,
 * sub_worker, sub_loc) change.  (Three informational header words differ from a packed
 * plan's: the sub-row and empty-row counts hold max_qrefs and max_rows, and the
 * KV chunk, which is chosen per plan, reads 0; counts->kv_chunk has it.)  Rows beyond subs->n_rows, up to max_rows, get
 * out = 0 and lse = -inf.  A plan that does not fit returns VA_ERR_CAPACITY and
 * names the section.
 */
typedef struct VaPlanCapacity {
  int32_t max_items;       /* narrow work items, a multiple of 8            */
  int32_t max_wide_items;  /* wide work items, a multiple of 8 (may be 0)   */
  int32_t max_links;
  int32_t max_qrefs;
  int32_t max_partials;    /* sizes the workspace                           */
  int32_t max_row_parts;
  int32_t max_rows;        /* rows of `out` the launch covers               */
} VaPlanCapacity;

/*
 * What a fixed-capacity launch must be able to hold, in the planner's own terms.
 * The reference sizes its graph buffers from (workers, depth, max_pages) for decode
 * (attention_graph.py:15-31) and (workers, depth, rows, max_pages) for prefill
 * (attention_graph.py:137-163):
 *   decode : max_sub_requests = max_sub_rows = workers * (depth + 1), max_rows = workers
 *   prefill: max_chains = workers, max_chain_members = depth + 1, max_chain_rows = rows,
 *            max_rows = rows
 * va_plan_capacity turns them into section sizes that no plan within the limits can
 * exceed (the KV chunk is chosen per plan, so page counts do not enter; kv_indices is
 * the caller's buffer).  params->kv_chunk must be 0.
 */
typedef struct VaPlanLimits {
  int32_t max_sub_requests;   /* stand-alone (decode) sub-requests, empty ones included */
  int32_t max_sub_rows;       /* their query rows in total                               */
  int32_t max_chains;         /* prefill requests                                        */
  int32_t max_chain_members;  /* sub-requests per prefill request                        */
  int32_t max_chain_rows;     /* new tokens of all prefill requests together             */
  int32_t max_rows;           /* rows of `out`                                           */
} VaPlanLimits;

VA_API int va_plan_capacity(const VaShape* shape, const VaPlanParams* params, const VaPlanLimits* limits,
                     VaPlanCapacity* capacity);

/* int32 words of a fixed-capacity plan blob */
VA_API int64_t va_plan_fixed_words(const VaPlanCapacity* capacity);

VA_API int va_plan_build_fixed(const VaSubRequests* subs, const VaShape* shape, const VaPlanParams* params,
                        const VaPlanCapacity* capacity, int32_t* plan_host, int64_t plan_capacity_words,
                        VaPlanCounts* counts);

/*
 * va_copy_shift_kv: block merge / append.  For every layer l < num_layers and
 * token i < n_tokens
 *   k_pool_l[dst[i]] = round(R(position_shift) float(k_pool_l[src[i]]))
 *   v_pool_l[dst[i]] = v_pool_l[src[i]]
 * where layer l's pools start l * layer_stride ELEMENTS after k_pool_dev /
 * v_pool_dev (num_layers = 1 for pools that are separate allocations), slots are
 * int64 on the device and the rotation uses position_shift on all three mRoPE
 * axes.  position_shift == 0 is a plain copy (rope may be NULL).  The keys are
 * rotated as fp32 copies and rounded once, as the reference does.  Source and
 * destination slots must be disjoint sets: the reference gathers everything
 * before it scatters, this kernel does not.
 * Replaces session.py:470-528 (_copy_block, _copy_slots, _shift_keys_): per
 * layer index_select + index_copy_ of K and V, then gather, fp32 rotation and
 * scatter of the copied keys.
 */
VA_API int va_copy_shift_kv(void* k_pool_dev, void* v_pool_dev, int64_t pool_row_stride, int64_t layer_stride,
                     int32_t num_layers, const int64_t* src_slots_dev, const int64_t* dst_slots_dev,
                     int64_t n_tokens, int64_t position_shift, const VaShape* shape, const VaRope* rope,
                     void* stream);

/*
 * va_attention: out[r, h, :] = softmax over the whole view of row r, i.e. the
 * LSE merge over all sub-requests (and KV chunks) that serve row r of
 *   softmax(R(sub_loc[i]) q[sub_worker[i], h] . K_s^T / sqrt(head_dim)) V_s .
 * q is [n_q_rows, num_q_heads, head_dim] unrotated, rows q_row_stride elements
 * apart; the pool is [num_slots, num_kv_heads, head_dim] with slot stride
 * pool_row_stride elements; out is [n_rows, num_q_heads*head_dim] contiguous;
 * lse_dev (optional, may be NULL) is fp32 [n_rows, num_q_heads]: natural-log
 * logsumexp of the scaled scores, or log2 when lse_base2 != 0.
 * sub_loc_dev is int64 [n_subrows] (sub_loc_axis_stride == 0) or [3, n_subrows].
 * plan_dev / kv_indices_dev / sub_worker_dev are device copies of the host
 * tables the plan was built from.  Rows no sub-request serves get out = 0 and
 * lse = -inf.  workspace_dev must hold counts.workspace_bytes.
 */
VA_API int va_attention(const void* q_dev, int64_t q_row_stride, const void* k_pool_dev,
                 const void* v_pool_dev, int64_t pool_row_stride, const int32_t* plan_dev,
                 const int32_t* plan_header_host, const int32_t* kv_indices_dev,
                 const int64_t* sub_worker_dev, const int64_t* sub_loc_dev,
                 int64_t sub_loc_axis_stride, void* out_dev, float* lse_dev, int32_t lse_base2,
                 void* workspace_dev, int64_t workspace_bytes, const VaShape* shape,
                 const VaRope* rope, void* stream);

/*
 * va_attention_static: va_attention for callers that cannot allocate or bring a
 * workspace -- code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  It has no counterpart in the reference.  Same arguments and
 * results as va_attention without workspace_dev / workspace_bytes: the partial
 * softmax states go to an array of VA_STATIC_SCRATCH_BYTES that the library
 * holds on every GPU it runs on until the process ends.  The call allocates
 * nothing (no hipMalloc / hipFree, no allocating library routine).  A plan whose
 * partial states need more (n_partials * num_q_heads * (head_dim + 2) * 4 bytes)
 * is rejected with VA_ERR_CAPACITY.  Every call on a GPU shares that GPU's
 * array: nothing in it has to start at zero (each slot is written before the
 * merge reads it), but calls that overlap on one GPU -- two streams, two
 * threads -- race; run them in stream order.  The first call on a device looks
 * up the array's device address; make it outside graph capture.
 */
#define VA_STATIC_SCRATCH_BYTES (32u << 20)
VA_API int va_attention_static(const void* q_dev, int64_t q_row_stride, const void* k_pool_dev,
                        const void* v_pool_dev, int64_t pool_row_stride, const int32_t* plan_dev,
                        const int32_t* plan_header_host, const int32_t* kv_indices_dev,
                        const int64_t* sub_worker_dev, const int64_t* sub_loc_dev,
                        int64_t sub_loc_axis_stride, void* out_dev, float* lse_dev, int32_t lse_base2,
                        const VaShape* shape, const VaRope* rope, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* VIEWATTN_H */
