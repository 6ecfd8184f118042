// Device-side helpers shared by the view-attention kernels (gfx950, wave64).
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/viewattn.h"
#include "va_plan.h"

namespace va {

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kNegBig = -1.0e30f;  // finite stand-in for -inf in running maxima

// ---- element types --------------------------------------------------------
struct F32 {
  using storage = float;
  static constexpr int kId = VA_F32;
  static __device__ __forceinline__ float load(const storage& v) { return v; }
  static __device__ __forceinline__ storage store(float f) { return f; }
};
struct F16 {
  using storage = __half;
  static constexpr int kId = VA_F16;
  static __device__ __forceinline__ float load(const storage& v) { return __half2float(v); }
  static __device__ __forceinline__ storage store(float f) { return __float2half_rn(f); }
};
struct BF16 {
  using storage = uint16_t;
  static constexpr int kId = VA_BF16;
  static __device__ __forceinline__ float load(const storage& v) {
    return __uint_as_float((uint32_t)v << 16);
  }
  // round to nearest even, NaN kept quiet (same rule as torch's float -> bfloat16): the hardware's
  // conversion (v_cvt_pk_bf16_f32) -- in integer arithmetic the rounding with its test for NaN took a
  // dozen instructions and a branch per element, most of what rotating a query tile cost
  static __device__ __forceinline__ storage store(float f) { return __builtin_bit_cast(storage, (__bf16)f); }
};

template <typename E>
__device__ __forceinline__ float round_through(float f) {
  return E::load(E::store(f));
}

// ---- rotation -------------------------------------------------------------
struct RopeDev {
  int mode;
  int rotary_dim;
  int half;  // rotary_dim / 2
  const float* cos_sin;
  int max_pos;
  int section_h3;  // 3 * mrope_section[1]
  int section_w3;  // 3 * mrope_section[2]
  const float* inv_freq;
};

struct Pos3 {
  long long t, h, w;
};

__device__ __forceinline__ Pos3 load_pos(const int64_t* pos, int64_t axis_stride, int64_t i) {
  Pos3 p;
  p.t = pos[i];
  if (axis_stride) {
    p.h = pos[axis_stride + i];
    p.w = pos[2 * axis_stride + i];
  } else {
    p.h = p.w = p.t;
  }
  return p;
}

__device__ __forceinline__ float mul_rounded(float a, float b);

// cos/sin of rotary pair `i` (0 <= i < half) at position `p`.
//  TABLE: row |p| (clamped to the table) of the fp32 cos|sin cache, sine negated for
//         negative p  (reference rope_correction.py:36-42).
//  MROPE: angle = float(axis position) * inv_freq[i]; pair i takes the height axis when
//         i % 3 == 1 and i < 3*section[1], the width axis when i % 3 == 2 and
//         i < 3*section[2], the temporal axis otherwise  (reference attention.py:267-277).
__device__ __forceinline__ void rope_cos_sin(const RopeDev& r, const Pos3& p, int i, float& c, float& s) {
  if (r.mode == VA_ROPE_TABLE) {
    long long a = p.t < 0 ? -p.t : p.t;
    if (a > r.max_pos - 1) a = r.max_pos - 1;
    const float* row = r.cos_sin + a * (long long)r.rotary_dim;
    c = row[i];
    s = row[r.half + i];
    if (p.t < 0) s = -s;
  } else {
    const int m = i % 3;
    long long q = p.t;
    if (m == 1 && i < r.section_h3) q = p.h;
    if (m == 2 && i < r.section_w3) q = p.w;
    const float angle = mul_rounded((float)q, r.inv_freq[i]);
    c = cosf(angle);
    s = sinf(angle);
  }
}

// Rotate the pair (x1, x2) = (x[i], x[i + half]) and round to the element type.
//  TABLE: fp32 arithmetic, one rounding at the end (rope_correction.py:47-54).
//  MROPE: cos/sin are first cast to the element type and every product and the sum
//         are rounded to it, as torch does for `x*cos + rotate_half(x)*sin` on a
//         low-precision tensor (attention.py:276-279).
// A product that the compiler may not fuse into a following add (the reference
// computes rotations with separately rounded multiplies and adds).
__device__ __forceinline__ float mul_rounded(float a, float b) {
  float p = a * b;
  asm volatile("" : "+v"(p));
  return p;
}

template <typename E>
__device__ __forceinline__ void rope_pair(const RopeDev& r, float c, float s, float x1, float x2,
                                          float& y1, float& y2) {
  if (r.mode == VA_ROPE_TABLE) {
    y1 = round_through<E>(mul_rounded(c, x1) - mul_rounded(s, x2));
    y2 = round_through<E>(mul_rounded(c, x2) + mul_rounded(s, x1));
  } else {
    const float ce = round_through<E>(c), se = round_through<E>(s);
    y1 = round_through<E>(round_through<E>(mul_rounded(x1, ce)) + round_through<E>(mul_rounded(-x2, se)));
    y2 = round_through<E>(round_through<E>(mul_rounded(x2, ce)) + round_through<E>(mul_rounded(x1, se)));
  }
}

// ---- wave reductions ------------------------------------------------------
template <int kLanes>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
  for (int off = kLanes / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

// Workgroup -> (work item, kv head).  The hardware hands workgroup b of a launch to die b % 8
// (8 dies, one L2 each).  The planner lays the items out so that item i belongs on die i % 8;
// here the kv heads of an item are placed at consecutive turns of that same die, so the
// workgroups that read the same tokens (one per head: adjacent 2*D-byte pieces of each pool
// row) run on one die at the same time.  n_items is a multiple of 8.
struct ItemHead {
  int item, head;
};
__device__ __forceinline__ ItemHead item_and_head(unsigned b, int num_kv_heads) {
  const unsigned die = b & 7u, turn = b >> 3;
  const unsigned head = turn % (unsigned)num_kv_heads, slot = turn / (unsigned)num_kv_heads;
  return ItemHead{(int)(slot * 8u + die), (int)head};
}

// physical slot of token t of a sub-request
__device__ __forceinline__ long long kv_slot(const int32_t* kv_indices, int kv_begin, int t, int page_size,
                                             bool slots) {
  if (slots) return kv_indices[kv_begin + t];
  const int page = t / page_size;
  return (long long)kv_indices[kv_begin + page] * page_size + (t - page * page_size);
}

}  // namespace va
