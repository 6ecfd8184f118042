// Matrix-core helpers shared by the narrow and the wide attention kernels.
#pragma once
#include <hip/hip_runtime.h>

#include "va_device.h"

typedef __bf16 va_bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 va_f16x8 __attribute__((ext_vector_type(8)));
typedef float va_f32x4 __attribute__((ext_vector_type(4)));

typedef float va_f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t va_u32x4 __attribute__((ext_vector_type(4)));  // 16 bytes as a plain vector (registers, LDS)
typedef uint32_t va_u32x2 __attribute__((ext_vector_type(2)));
typedef short va_i16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 va_f16x4 __attribute__((ext_vector_type(4)));

namespace va {

template <typename E>
struct Mma;
template <>
struct Mma<BF16> {
  template <typename A, typename B>
  static __device__ __forceinline__ va_f32x16 run32(const A& a, const B& b, va_f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(va_bf16x8, a), __builtin_bit_cast(va_bf16x8, b),
                                                   c, 0, 0, 0);
  }
  // Same product with the accumulator pinned in the accumulation registers (AGPRs).  Written as
  // assembly because the register allocator otherwise treats AGPRs as spill space for a long-lived
  // accumulator and copies all of it to VGPRs and back around every tile.  Only the long-lived
  // output accumulators are driven this way: nothing but further products touches them between
  // the start of a work item and accumulator_fence(), which every other reader must call first
  // (it carries the accumulators through, so no read can be moved in front of it).  The compiler
  // cannot insert wait states for an instruction it does not see, and the matrix pipe must not
  // read an operand in the two wait states after a vector-ALU instruction wrote it (the transposed
  // V fragment, the packed P, or a register copy placed in front of the statement): every product
  // issued from assembly therefore carries its own `s_nop 1`.  Products whose results the vector
  // ALU reads next (the scores) go through run32, which the compiler sees and guards both ways.
  static __device__ __forceinline__ void run32_acc(const va_u32x4& a, const va_u32x4& b, va_f32x16& c) {
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
  template <typename A, typename B>
  static __device__ __forceinline__ va_f32x4 run(const A& a, const B& b, va_f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(va_bf16x8, a), __builtin_bit_cast(va_bf16x8, b),
                                                   c, 0, 0, 0);
  }
  // 16x16x16: four contraction elements per lane
  static __device__ __forceinline__ va_f32x4 run16(const va_u32x2& a, const va_u32x2& b, va_f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(va_i16x4, a), __builtin_bit_cast(va_i16x4, b),
                                                     c, 0, 0, 0);
  }
  // both conversions in one instruction (v_cvt_pk_bf16_f32, round to nearest even)
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, bf16x2));
  }
};
template <>
struct Mma<F16> {
  template <typename A, typename B>
  static __device__ __forceinline__ va_f32x16 run32(const A& a, const B& b, va_f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(va_f16x8, a), __builtin_bit_cast(va_f16x8, b), c,
                                                  0, 0, 0);
  }
  static __device__ __forceinline__ void run32_acc(const va_u32x4& a, const va_u32x4& b, va_f32x16& c) {
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
  template <typename A, typename B>
  static __device__ __forceinline__ va_f32x4 run(const A& a, const B& b, va_f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(va_f16x8, a), __builtin_bit_cast(va_f16x8, b), c,
                                                  0, 0, 0);
  }
  static __device__ __forceinline__ va_f32x4 run16(const va_u32x2& a, const va_u32x2& b, va_f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(va_f16x4, a), __builtin_bit_cast(va_f16x4, b), c,
                                                 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, f16x2));
  }
};

// One 16-byte piece (dims [d0, d0+8)) of a query head row, rotated for position `p` and
// rounded to the element type; pieces beyond rotary_dim pass through.  rotary_dim is a
// multiple of 16 here, so a piece never straddles the two rotary halves.
template <typename E>
__device__ __forceinline__ uint4 rotated_query_piece(const RopeDev& rope, const typename E::storage* qh, int d0,
                                                     const Pos3& p) {
  using S = typename E::storage;
  if (d0 >= rope.rotary_dim) return *(const uint4*)(qh + d0);
  const bool first = d0 < rope.half;
  const int i0 = first ? d0 : d0 - rope.half;
  const uint4 ra = *(const uint4*)(qh + i0);
  const uint4 rb = *(const uint4*)(qh + i0 + rope.half);
  const uint32_t wa[4] = {ra.x, ra.y, ra.z, ra.w}, wb[4] = {rb.x, rb.y, rb.z, rb.w};
  uint32_t out[4];
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    float y[2];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const S xa = __builtin_bit_cast(S, (uint16_t)(wa[w] >> (16 * b)));
      const S xb = __builtin_bit_cast(S, (uint16_t)(wb[w] >> (16 * b)));
      float cs, sn, y1, y2;
      rope_cos_sin(rope, p, i0 + 2 * w + b, cs, sn);
      rope_pair<E>(rope, cs, sn, E::load(xa), E::load(xb), y1, y2);
      y[b] = first ? y1 : y2;
    }
    out[w] = Mma<E>::pack(y[0], y[1]);  // y is already representable: the conversion is exact
  }
  return make_uint4(out[0], out[1], out[2], out[3]);
}

// Two 16-byte pieces of a rotated query head row at once.  Unit x of a row (0 <= x < D/16) covers
// the rotary pair of pieces (x, x + rotary_dim/16) -- both halves of the same eight rotations, so
// the inputs, the cos/sin entries and the products are shared -- or, past the rotary part, two
// adjacent pieces that pass through.  c0/c1 receive the piece indices.
template <typename E>
__device__ __forceinline__ void rotated_query_unit(const RopeDev& rope, const typename E::storage* qh, int x,
                                                   const Pos3& p, int& c0, int& c1, uint4& o0, uint4& o1) {
  using S = typename E::storage;
  const int pair_units = rope.rotary_dim / 16;
  if (x >= pair_units) {
    c0 = rope.rotary_dim / 8 + 2 * (x - pair_units);
    c1 = c0 + 1;
    o0 = *(const uint4*)(qh + 8 * c0);
    o1 = *(const uint4*)(qh + 8 * c1);
    return;
  }
  c0 = x;
  c1 = x + pair_units;
  const int i0 = 8 * x;
  const uint4 ra = *(const uint4*)(qh + i0);
  const uint4 rb = *(const uint4*)(qh + i0 + rope.half);
  const uint32_t wa[4] = {ra.x, ra.y, ra.z, ra.w}, wb[4] = {rb.x, rb.y, rb.z, rb.w};
  uint32_t lo[4], hi[4];
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    float y1[2], y2[2];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const S xa = __builtin_bit_cast(S, (uint16_t)(wa[w] >> (16 * b)));
      const S xb = __builtin_bit_cast(S, (uint16_t)(wb[w] >> (16 * b)));
      float cs, sn;
      rope_cos_sin(rope, p, i0 + 2 * w + b, cs, sn);
      rope_pair<E>(rope, cs, sn, E::load(xa), E::load(xb), y1[b], y2[b]);
    }
    lo[w] = Mma<E>::pack(y1[0], y1[1]);  // already representable: the conversions are exact
    hi[w] = Mma<E>::pack(y2[0], y2[1]);
  }
  o0 = make_uint4(lo[0], lo[1], lo[2], lo[3]);
  o1 = make_uint4(hi[0], hi[1], hi[2], hi[3]);
}

// The same unit in two steps for the cos|sin table, for callers that stage several rows at once:
// `load` sends every memory request of the unit (the two query pieces and the sixteen table
// entries), `finish` rotates.  A caller that loads a batch of rows before it finishes the first
// pays the memory latency once per batch instead of once per row.  The unit must be rotary
// (x < rotary_dim / 16); pieces past the rotary part are plain copies.
template <typename E>
struct TableQueryUnit {
  uint4 ra, rb;
  float4 c[2], s[2];
  __device__ __forceinline__ void load(const RopeDev& rope, const typename E::storage* qh, int x, const Pos3& p) {
    const int i0 = 8 * x;
    ra = *(const uint4*)(qh + i0);
    rb = *(const uint4*)(qh + i0 + rope.half);
    long long a = p.t < 0 ? -p.t : p.t;
    if (a > rope.max_pos - 1) a = rope.max_pos - 1;
    // rows of the table and their halves start on 32-byte boundaries (rotary_dim is a multiple of 16)
    const float* row = rope.cos_sin + a * (long long)rope.rotary_dim + i0;
    c[0] = *(const float4*)row;
    c[1] = *(const float4*)(row + 4);
    s[0] = *(const float4*)(row + rope.half);
    s[1] = *(const float4*)(row + rope.half + 4);
  }
  __device__ __forceinline__ void finish(const RopeDev& rope, const Pos3& p, uint4& o0, uint4& o1) const {
    using S = typename E::storage;
    const uint32_t wa[4] = {ra.x, ra.y, ra.z, ra.w}, wb[4] = {rb.x, rb.y, rb.z, rb.w};
    const float ct[8] = {c[0].x, c[0].y, c[0].z, c[0].w, c[1].x, c[1].y, c[1].z, c[1].w};
    const float st[8] = {s[0].x, s[0].y, s[0].z, s[0].w, s[1].x, s[1].y, s[1].z, s[1].w};
    uint32_t lo[4], hi[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      float y1[2], y2[2];
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const S xa = __builtin_bit_cast(S, (uint16_t)(wa[w] >> (16 * b)));
        const S xb = __builtin_bit_cast(S, (uint16_t)(wb[w] >> (16 * b)));
        const float sn = p.t < 0 ? -st[2 * w + b] : st[2 * w + b];
        // the table mode's arithmetic of rope_pair: fp32, one rounding at the end
        y1[b] = mul_rounded(ct[2 * w + b], E::load(xa)) - mul_rounded(sn, E::load(xb));
        y2[b] = mul_rounded(ct[2 * w + b], E::load(xb)) + mul_rounded(sn, E::load(xa));
      }
      lo[w] = Mma<E>::pack(y1[0], y1[1]);  // the one rounding (to nearest even, as E::store rounds)
      hi[w] = Mma<E>::pack(y2[0], y2[1]);
    }
    o0 = make_uint4(lo[0], lo[1], lo[2], lo[3]);
    o1 = make_uint4(hi[0], hi[1], hi[2], hi[3]);
  }
};

// Wait until the matrix pipe has written the results of the products issued from assembly
// (run32_acc) into the accumulators `o`, before anything but another product touches them.  A
// 32x32x16 product runs for 8 passes of 4 clocks and its result needs 3 more wait states to reach
// the register file (11 in all, whatever was issued before it has finished by then as the pipe
// works in order); kAccumulatorWaitStates adds a margin.  The statement takes every accumulator as
// an in-out operand: a later read depends on it and so cannot be scheduled in front of it, and
// neither can a copy the register allocator makes for such a read.
constexpr int kMfma32Passes = 8;
constexpr int kAccumulatorWaitStates = kMfma32Passes + 3 + 4;
static_assert(kAccumulatorWaitStates <= 16, "one s_nop holds at most 16 wait states");
template <int kCount>
__device__ __forceinline__ void accumulator_fence(va_f32x16* o) {
  static_assert(kCount == 2 || kCount == 4 || kCount == 8 || kCount == 16, "accumulators per wave");
  if constexpr (kCount == 16) {
    asm volatile("s_nop %16"
                 : "+a"(o[0]), "+a"(o[1]), "+a"(o[2]), "+a"(o[3]), "+a"(o[4]), "+a"(o[5]), "+a"(o[6]), "+a"(o[7]),
                   "+a"(o[8]), "+a"(o[9]), "+a"(o[10]), "+a"(o[11]), "+a"(o[12]), "+a"(o[13]), "+a"(o[14]), "+a"(o[15])
                 : "n"(kAccumulatorWaitStates - 1));
  } else if constexpr (kCount == 8) {
    asm volatile("s_nop %8"
                 : "+a"(o[0]), "+a"(o[1]), "+a"(o[2]), "+a"(o[3]), "+a"(o[4]), "+a"(o[5]), "+a"(o[6]), "+a"(o[7])
                 : "n"(kAccumulatorWaitStates - 1));
  } else if constexpr (kCount == 4) {
    asm volatile("s_nop %4" : "+a"(o[0]), "+a"(o[1]), "+a"(o[2]), "+a"(o[3]) : "n"(kAccumulatorWaitStates - 1));
  } else {
    asm volatile("s_nop %2" : "+a"(o[0]), "+a"(o[1]) : "n"(kAccumulatorWaitStates - 1));
  }
}

// Workgroup barrier for the tile ring.  __syncthreads() carries a fence that waits for ALL
// outstanding memory operations, which would drain the loads of the tiles still in flight; this
// one waits until at most `n` of the wave's vector memory operations (the pool -> LDS loads) are
// outstanding, and for the wave's own LDS traffic, before it joins the barrier.  The "memory"
// clobber keeps the compiler from moving LDS accesses or loads across it.
template <int n>
__device__ __forceinline__ void ring_barrier() {
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(n) : "memory");
}
// The same, handing back a zero that exists only after the barrier: a value combined with it cannot
// be touched (and so cannot be waited for) before the barrier.
template <int n>
__device__ __forceinline__ int ring_barrier_zero() {
  int zero;
  asm volatile("s_waitcnt vmcnt(%1) lgkmcnt(0)\n\ts_barrier\n\ts_mov_b32 %0, 0" : "=s"(zero) : "n"(n) : "memory");
  return zero;
}
constexpr int kAnyInFlight = 63;  // vmcnt(63): no wait on vector memory at all

// One wave-level pool -> LDS load: lane l's 16 bytes at `src` land at LDS byte address
// `lds_base + 16 l` (lds_base is wave-uniform and travels in M0).  Written as assembly on purpose:
// when the compiler sees such a load it makes every later LDS read wait for ALL of them
// (it cannot tell the ring's buffers apart), which would serialise the ring.  Completion is
// tracked by hand instead, with the vmcnt values of ring_barrier.  M0 is a reserved register the
// compiler manages itself and cannot be named as a clobber, so every statement puts back the value
// it found: a value the compiler keeps live in M0 across the statement stays intact.
__device__ __forceinline__ void load_to_lds(const void* src, uint32_t lds_base) {
  uint32_t saved;
  asm volatile(
      "s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\t"
      "global_load_lds_dwordx4 %1, off\n\t"
      "s_mov_b32 m0, %0"
      : "=&s"(saved)
      : "v"(src), "s"(lds_base)
      : "memory");
}
// The same load marked non-temporal: rows that one workgroup reads once (a block no other query
// tile shares) are streamed through the caches as lines to evict first, so that they do not push
// out the rows that several tiles read (a block shared by many views, held in the die's L2).
// Measured on one MI355X: a pure stream (eight views of 131 072 tokens, nothing shared) 5.74 -> 6.29 TB/s;
// it is the nt bit that does it, the sc0 / sc1 bits beside it change nothing.
__device__ __forceinline__ void load_to_lds_once(const void* src, uint32_t lds_base) {
  uint32_t saved;
  asm volatile(
      "s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\t"
      "global_load_lds_dwordx4 %1, off nt\n\t"
      "s_mov_b32 m0, %0"
      : "=&s"(saved)
      : "v"(src), "s"(lds_base)
      : "memory");
}
// The same with a wave-uniform base address and a 32-bit per-lane byte offset (no vector ALU work
// to form 64-bit addresses).
__device__ __forceinline__ void load_to_lds(const void* base, uint32_t lane_offset, uint32_t lds_base) {
  uint32_t saved;
  asm volatile(
      "s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %2\n\t"
      "s_mov_b32 m0, %0"
      : "=&s"(saved)
      : "v"(lane_offset), "s"(base), "s"(lds_base)
      : "memory");
}
// Two loads of per-lane addresses behind ONE setting of M0, the second landing 1024 bytes after
// the first: the instruction's immediate offset is added to the pool address AND to the LDS
// address, so the caller passes the second address with 1024 taken off.
__device__ __forceinline__ void load_pair_to_lds(const void* src0, const void* src1_minus_1024, uint32_t lds_base) {
  uint32_t saved;
  asm volatile(
      "s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\ts_nop 0\n\t"
      "global_load_lds_dwordx4 %1, off\n\t"
      "global_load_lds_dwordx4 %2, off offset:1024\n\t"
      "s_mov_b32 m0, %0"
      : "=&s"(saved)
      : "v"(src0), "v"(src1_minus_1024), "s"(lds_base)
      : "memory");
}
// Up to four loads of "uniform base + per-lane offset" behind one setting of M0: load u of a group
// lands 1024 u bytes further on when its per-lane offset has had 1024 u taken off beforehand
// (grouped_lane_offset).
__device__ __forceinline__ uint32_t grouped_lane_offset(uint32_t lane_offset, int u) { return lane_offset - 1024u * (u % 4); }
template <int kCount>
__device__ __forceinline__ void load_group_to_lds(const void* base, const uint32_t* adjusted_offsets, uint32_t lds_base) {
  static_assert(kCount == 1 || kCount == 2 || kCount == 4, "loads per group");
  uint32_t saved;
  if constexpr (kCount == 4) {
    asm volatile(
        "s_mov_b32 %0, m0\n\ts_mov_b32 m0, %6\n\ts_nop 0\n\t"
        "global_load_lds_dwordx4 %1, %5\n\t"
        "global_load_lds_dwordx4 %2, %5 offset:1024\n\t"
        "global_load_lds_dwordx4 %3, %5 offset:2048\n\t"
        "global_load_lds_dwordx4 %4, %5 offset:3072\n\t"
        "s_mov_b32 m0, %0"
        : "=&s"(saved)
        : "v"(adjusted_offsets[0]), "v"(adjusted_offsets[1]), "v"(adjusted_offsets[2]), "v"(adjusted_offsets[3]),
          "s"(base), "s"(lds_base)
        : "memory");
  } else if constexpr (kCount == 2) {
    asm volatile(
        "s_mov_b32 %0, m0\n\ts_mov_b32 m0, %4\n\ts_nop 0\n\t"
        "global_load_lds_dwordx4 %1, %3\n\t"
        "global_load_lds_dwordx4 %2, %3 offset:1024\n\t"
        "s_mov_b32 m0, %0"
        : "=&s"(saved)
        : "v"(adjusted_offsets[0]), "v"(adjusted_offsets[1]), "s"(base), "s"(lds_base)
        : "memory");
  } else {
    load_to_lds(base, adjusted_offsets[0], lds_base);
  }
}
__device__ __forceinline__ uint32_t lds_address(const void* p) {
  return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)p;
}

}  // namespace va
