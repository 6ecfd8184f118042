// libviewattn.so: C ABI, rotation/store kernel, vector-ALU attention kernel and
// the partial-state merge kernel.  The matrix-core kernels live in va_mfma_stream.hip and va_mfma_wide.hip.
#include <hip/hip_runtime.h>

#include <type_traits>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>

#include "../../include/viewattn.h"
#include "va_device.h"
#include "va_internal.h"
#include "va_launch.h"
#include "va_plan.h"

// ---------------------------------------------------------------------------
// errors
// ---------------------------------------------------------------------------
static thread_local char g_error[512] = "";

int va_fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

extern "C" const char* va_last_error(void) { return g_error; }
extern "C" int va_version(void) { return 1; }

int64_t va_workspace_bytes_for(int64_t n_partials, int num_q_heads, int head_dim) {
  // accumulators [n_partials, Hq, D] fp32, then (max, sum) [n_partials, Hq, 2] fp32
  return n_partials * num_q_heads * ((int64_t)head_dim + 2) * (int64_t)sizeof(float);
}

static int check_hip(hipError_t e, const char* what) {
  if (e == hipSuccess) return VA_OK;
  return va_fail(VA_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

namespace va {

int make_rope(const VaRope* rope, int head_dim, RopeDev* out) {
  if (!rope) return va_fail(VA_ERR_ARG, "null rope description");
  if (rope->rotary_dim < 0 || rope->rotary_dim > head_dim || (rope->rotary_dim & 1))
    return va_fail(VA_ERR_ARG, "rotary_dim %d must be even and within head_dim %d", rope->rotary_dim, head_dim);
  out->mode = rope->mode;
  out->rotary_dim = rope->rotary_dim;
  out->half = rope->rotary_dim / 2;
  out->cos_sin = rope->cos_sin_dev;
  out->max_pos = rope->max_pos;
  out->section_h3 = 3 * rope->section_h;
  out->section_w3 = 3 * rope->section_w;
  out->inv_freq = rope->inv_freq_dev;
  if (rope->rotary_dim == 0) return VA_OK;
  if (rope->mode == VA_ROPE_TABLE) {
    if (!rope->cos_sin_dev || rope->max_pos <= 0) return va_fail(VA_ERR_ARG, "table rotation needs cos_sin and max_pos > 0");
  } else if (rope->mode == VA_ROPE_MROPE) {
    if (!rope->inv_freq_dev) return va_fail(VA_ERR_ARG, "mRoPE rotation needs inv_freq");
  } else {
    return va_fail(VA_ERR_ARG, "unknown rotation mode %d", rope->mode);
  }
  return VA_OK;
}

// ---------------------------------------------------------------------------
// rotate (+ optional scatter of K and V rows into the pool)
// ---------------------------------------------------------------------------
// One workgroup per input row.  The row's heads are rotated pairwise
// (i, i + rotary_dim/2) so the operation is safe in place; dims beyond
// rotary_dim pass through.  With a destination table the rotated row goes to
// pool row dst[i] (negative: the row is skipped, reference store.cu:44-46) and
// the value row is copied beside it.
template <typename E>
__global__ __launch_bounds__(256) void rope_store_kernel(
    const typename E::storage* __restrict__ x, const typename E::storage* __restrict__ v,
    typename E::storage* y, typename E::storage* v_out, long long x_stride, long long v_stride,
    long long y_stride, const void* dst, int dst_is_i64, const int64_t* pos, long long pos_axis_stride,
    long long n_rows, int n_heads, int head_dim, RopeDev rope) {
  const long long row = blockIdx.x;
  if (row >= n_rows) return;
  long long out_row = row;
  if (dst) {
    out_row = dst_is_i64 ? ((const long long*)dst)[row] : (long long)((const int*)dst)[row];
    if (out_row < 0) return;
  }
  const typename E::storage* xr = x + row * x_stride;
  typename E::storage* yr = y + out_row * y_stride;
  const int half = rope.half;
  if (half > 0) {
    const Pos3 p = load_pos(pos, pos_axis_stride, row);
    for (int e = threadIdx.x; e < n_heads * half; e += blockDim.x) {
      const int h = e / half, i = e - h * half;
      float c, s;
      rope_cos_sin(rope, p, i, c, s);
      const float x1 = E::load(xr[h * head_dim + i]);
      const float x2 = E::load(xr[h * head_dim + half + i]);
      float y1, y2;
      rope_pair<E>(rope, c, s, x1, x2, y1, y2);
      yr[h * head_dim + i] = E::store(y1);
      yr[h * head_dim + half + i] = E::store(y2);
    }
  }
  const int tail = head_dim - rope.rotary_dim;
  if (tail > 0 && (const void*)xr != (const void*)yr) {
    for (int e = threadIdx.x; e < n_heads * tail; e += blockDim.x) {
      const int h = e / tail, i = e - h * tail;
      yr[h * head_dim + rope.rotary_dim + i] = xr[h * head_dim + rope.rotary_dim + i];
    }
  }
  if (v) {
    const typename E::storage* vr = v + row * v_stride;
    typename E::storage* vo = v_out + out_row * y_stride;
    for (int e = threadIdx.x; e < n_heads * head_dim; e += blockDim.x) vo[e] = vr[e];
  }
}

// The same in 16-byte pieces, for rows whose addresses, strides and rotary half are multiples of
// a piece (the reference's store kernel copies with 16-byte vectors too: store.cu:42-54).  Thread j
// of a row takes key unit j -- a rotary pair of pieces (dims [i0, i0 + kVec) and the same dims half
// a rotary_dim further: one thread reads both, rotates element by element with the arithmetic of
// rope_pair, writes both, so in place is safe) or a piece past the rotary part -- and value piece j;
// all of a thread's loads are issued before its first store.  Consecutive threads take consecutive
// pieces of consecutive rows: a workgroup covers one row or several, whatever the row length.
template <typename E>
__global__ __launch_bounds__(256) void rope_store_vec_kernel(
    const typename E::storage* __restrict__ x, const typename E::storage* __restrict__ v,
    typename E::storage* y, typename E::storage* v_out, long long x_stride, long long v_stride,
    long long y_stride, const void* dst, int dst_is_i64, const int64_t* pos, long long pos_axis_stride,
    long long n_rows, int n_heads, int head_dim, RopeDev rope, int pair_units, int key_units, int units) {
  using S = typename E::storage;
  constexpr int kVec = 16 / sizeof(S);
  union Piece {
    uint4 raw;
    S e[kVec];
  };
  const unsigned idx = blockIdx.x * 256u + threadIdx.x;  // the launcher keeps rows * units within 32 bits
  const long long row = idx / (unsigned)units;
  if (row >= n_rows) return;
  const int u = (int)(idx - (unsigned)row * (unsigned)units);
  long long out_row = row;
  if (dst) {
    out_row = dst_is_i64 ? ((const long long*)dst)[row] : (long long)((const int*)dst)[row];
    if (out_row < 0) return;
  }
  const S* xr = x + row * x_stride;
  S* yr = y + out_row * y_stride;
  const bool has_value = v != nullptr && u < n_heads * (head_dim / kVec);
  Piece val, xa, xb, ya, yb;
  if (has_value) val.raw = *(const uint4*)(v + row * v_stride + u * kVec);
  int ea = -1, eb = -1;  // element offsets of the key pieces this thread writes
  if (u < pair_units) {
    const int per_head = rope.half / kVec;
    const int h = u / per_head, i0 = (u - h * per_head) * kVec;
    ea = h * head_dim + i0;
    eb = ea + rope.half;
    xa.raw = *(const uint4*)(xr + ea);
    xb.raw = *(const uint4*)(xr + eb);
    const Pos3 p = load_pos(pos, pos_axis_stride, row);
    float cs[kVec], sns[kVec];
    if (rope.mode == VA_ROPE_TABLE) {
      // the kVec cosines and sines of this piece in 16-byte loads (the launcher has checked the table's alignment)
      long long a = p.t < 0 ? -p.t : p.t;
      if (a > rope.max_pos - 1) a = rope.max_pos - 1;
      const float* trow = rope.cos_sin + a * (long long)rope.rotary_dim + i0;
#pragma unroll
      for (int k = 0; k < kVec; k += 4) {
        const float4 c4 = *(const float4*)(trow + k), s4 = *(const float4*)(trow + rope.half + k);
        cs[k] = c4.x, cs[k + 1] = c4.y, cs[k + 2] = c4.z, cs[k + 3] = c4.w;
        sns[k] = s4.x, sns[k + 1] = s4.y, sns[k + 2] = s4.z, sns[k + 3] = s4.w;
      }
      if (p.t < 0) {
#pragma unroll
        for (int k = 0; k < kVec; ++k) sns[k] = -sns[k];
      }
    } else {
#pragma unroll
      for (int k = 0; k < kVec; ++k) rope_cos_sin(rope, p, i0 + k, cs[k], sns[k]);
    }
#pragma unroll
    for (int k = 0; k < kVec; ++k) {
      float y1, y2;
      const float c = cs[k], sn = sns[k];
      rope_pair<E>(rope, c, sn, E::load(xa.e[k]), E::load(xb.e[k]), y1, y2);
      ya.e[k] = E::store(y1);
      yb.e[k] = E::store(y2);
    }
  } else if (u < key_units) {  // a key piece past the rotary part
    const int t = u - pair_units, per_head = (head_dim - rope.rotary_dim) / kVec;
    ea = (t / per_head) * head_dim + rope.rotary_dim + (t % per_head) * kVec;
    ya.raw = *(const uint4*)(xr + ea);
  }
  if (has_value) *(uint4*)(v_out + out_row * y_stride + u * kVec) = val.raw;
  if (ea >= 0) *(uint4*)(yr + ea) = ya.raw;
  if (eb >= 0) *(uint4*)(yr + eb) = yb.raw;
}

template <typename E>
int launch_rope_store(const void* x, const void* v, void* y, void* v_out, long long x_stride,
                      long long v_stride, long long y_stride, const void* dst, int dst_is_i64,
                      const int64_t* pos, long long pos_axis_stride, long long n_rows, int n_heads,
                      int head_dim, const RopeDev& rope, hipStream_t stream) {
  using S = typename E::storage;
  constexpr int kVec = 16 / sizeof(S);
  if (n_rows == 0) return VA_OK;
  if (n_rows > 0x7fffffffLL) return va_fail(VA_ERR_ARG, "too many rows");
  auto piecewise = [&](const void* ptr, long long stride) {
    return ptr == nullptr || ((uintptr_t)ptr % 16 == 0 && stride % kVec == 0);
  };
  const bool table_ok = rope.mode != VA_ROPE_TABLE || (kVec % 4 == 0 && (uintptr_t)rope.cos_sin % 16 == 0 &&
                                                      rope.rotary_dim % 4 == 0 && rope.half % 4 == 0);
  const bool vec = head_dim % kVec == 0 && rope.half % kVec == 0 && piecewise(x, x_stride) && piecewise(y, y_stride) &&
                   piecewise(v, v_stride) && piecewise(v_out, y_stride) && table_ok;
  if (vec) {
    const bool copy_tail = x != y || dst != nullptr;
    const int pair_units = n_heads * (rope.half / kVec);
    const int key_units = pair_units + (copy_tail ? n_heads * ((head_dim - rope.rotary_dim) / kVec) : 0);
    const int units = v ? n_heads * (head_dim / kVec) : key_units;  // (key_units <= the pieces of a row)
    if (units > 0 && n_rows * units < 0x7fffff00LL) {
      const long long blocks = (n_rows * units + 255) / 256;
      hipLaunchKernelGGL(rope_store_vec_kernel<E>, dim3((unsigned)blocks), dim3(256), 0, stream, (const S*)x,
                         (const S*)v, (S*)y, (S*)v_out, x_stride, v_stride, y_stride, dst, dst_is_i64, pos,
                         pos_axis_stride, n_rows, n_heads, head_dim, rope, pair_units, key_units, units);
      return check_hip(hipGetLastError(), "rope/store launch");
    }
    if (units == 0) return VA_OK;
  }
  hipLaunchKernelGGL(rope_store_kernel<E>, dim3((unsigned)n_rows), dim3(256), 0, stream, (const S*)x,
                     (const S*)v, (S*)y, (S*)v_out, x_stride, v_stride, y_stride, dst, dst_is_i64, pos,
                     pos_axis_stride, n_rows, n_heads, head_dim, rope);
  return check_hip(hipGetLastError(), "rope/store launch");
}

// ---------------------------------------------------------------------------
// vector-ALU attention: any element type, head_dim in {16..256} (power of two)
// ---------------------------------------------------------------------------
// One workgroup (4 waves) per (work item, kv head).  Tile rows are taken one
// after the other; for each, heads are processed in blocks of kHB.  A token's
// K (then V) row is read by kLPT adjacent lanes with 16-byte loads, so a wave
// streams 64/kLPT tokens per step and the four waves interleave tokens.  Every
// lane group keeps its own online-softmax state; states are merged across lane
// groups by shuffles and across waves through LDS when the chain ends.
constexpr int kHB = 4;          // q heads per pass
constexpr int kGenThreads = 256;
constexpr int kGenWaves = kGenThreads / kWave;
constexpr int kGenAhead = 4;     // steps of the token walk whose loads are in flight together

template <typename E, int kD>
__global__ __launch_bounds__(kGenThreads) void attn_generic_kernel(AttnArgs a) {
  using S = typename E::storage;
  constexpr int kVec = 16 / sizeof(S);
  constexpr int kLPT = kD / kVec;  // lanes per token
  constexpr int kTPW = kWave / kLPT;
  static_assert(kLPT >= 1 && kLPT <= kWave, "head_dim out of range for this element type");

  __shared__ float q_s[kHB][kD];
  __shared__ float acc_s[kGenWaves][kHB][kD];
  __shared__ float ml_s[kGenWaves][kHB][2];

  const ItemHead where = item_and_head(blockIdx.x, a.num_kv_heads);
  const int32_t* item = a.items + (long long)where.item * VA_ITEM_WORDS;
  const int hk = where.head;
  const int G = a.num_q_heads / a.num_kv_heads;
  const int n_q = item[VA_I_N_Q];
  if (n_q == 0) return;  // padding item: keeps the launch order aligned with the die round-robin
  const int part_base = item[VA_I_PART_BASE];
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int li = lane % kLPT;   // which 16-byte piece of the row
  const int lg = lane / kLPT;   // token within the wave step
  const S* kp = (const S*)a.k_pool;
  const S* vp = (const S*)a.v_pool;

  for (int iq = 0; iq < n_q; ++iq) {
    long long out_row = -1;
    for (int hb = 0; hb < G; hb += kHB) {
      float m[kHB], l[kHB], acc[kHB][kVec];
#pragma unroll
      for (int g = 0; g < kHB; ++g) {
        m[g] = kNegBig;
        l[g] = 0.f;
#pragma unroll
        for (int e = 0; e < kVec; ++e) acc[g][e] = 0.f;
      }
      for (int li_ = 0; li_ < item[VA_I_N_LINKS]; ++li_) {
        const int32_t* link = a.links + (long long)(item[VA_I_LINK_BEGIN] + li_) * VA_LINK_WORDS;
        const int lflags = link[VA_L_FLAGS];
        const int subrow = (lflags & VA_LINK_INDIRECT) ? a.qrefs[link[VA_L_QREF] + iq] : link[VA_L_QREF] + iq;
        const long long src_row = a.sub_worker[subrow];
        out_row = src_row;
        const Pos3 p = load_pos(a.sub_loc, a.sub_loc_axis_stride, subrow);

        // rotate this row's query for the link, rounded to the element type
        __syncthreads();
        for (int e = threadIdx.x; e < kHB * kD; e += kGenThreads) {
          const int g = e / kD, d = e - g * kD;
          float val = 0.f;
          if (hb + g < G) {
            const S* qh = (const S*)a.q + src_row * a.q_row_stride + (long long)(hk * G + hb + g) * kD;
            if (d < a.rope.rotary_dim) {
              const int i = d < a.rope.half ? d : d - a.rope.half;
              float c, s;
              rope_cos_sin(a.rope, p, i, c, s);
              float y1, y2;
              rope_pair<E>(a.rope, c, s, E::load(qh[i]), E::load(qh[i + a.rope.half]), y1, y2);
              val = d < a.rope.half ? y1 : y2;
            } else {
              val = E::load(qh[d]);
            }
          }
          q_s[g][d] = val;
        }
        __syncthreads();
        float qr[kHB][kVec];
#pragma unroll
        for (int g = 0; g < kHB; ++g)
#pragma unroll
          for (int e = 0; e < kVec; ++e) qr[g][e] = q_s[g][li * kVec + e];

        const int t_end = min(link[VA_L_TOK_END], link[VA_L_CAUSAL_BASE] + iq + 1);
        const int kv_begin = link[VA_L_KV_BEGIN];
        const bool slots = lflags & VA_LINK_SLOTS;
        // kGenAhead steps of the walk at a time: their page lookups first, then their K and V rows, all
        // in flight together -- a step by itself is a chain of two dependent trips to memory, and at
        // decode sizes (a few hundred tokens per workgroup) the kernel is nothing but that chain
        for (int t0 = link[VA_L_TOK_BEGIN] + wave * kTPW; t0 < t_end; t0 += kGenAhead * kGenWaves * kTPW) {
          bool live[kGenAhead];
          long long off[kGenAhead];
          uint4 kraw[kGenAhead], vraw[kGenAhead];
#pragma unroll
          for (int u = 0; u < kGenAhead; ++u) {
            const int t = t0 + u * kGenWaves * kTPW + lg;
            live[u] = t < t_end;
            const long long slot = kv_slot(a.kv_indices, kv_begin, live[u] ? t : t_end - 1, a.page_size, slots);
            off[u] = slot * a.pool_row_stride + (long long)hk * kD + li * kVec;
          }
#pragma unroll
          for (int u = 0; u < kGenAhead; ++u) {
            kraw[u] = make_uint4(0, 0, 0, 0);
            vraw[u] = make_uint4(0, 0, 0, 0);
            if (live[u]) {
              kraw[u] = *(const uint4*)(kp + off[u]);
              vraw[u] = *(const uint4*)(vp + off[u]);
            }
          }
#pragma unroll
          for (int u = 0; u < kGenAhead; ++u) {
            if (t0 + u * kGenWaves * kTPW >= t_end) break;  // (wave-uniform: the step lies past the range)
            float sc[kHB];
            const S* ke = (const S*)&kraw[u];
            const S* ve = (const S*)&vraw[u];
            float kf[kVec], vf[kVec];
#pragma unroll
            for (int e = 0; e < kVec; ++e) {
              kf[e] = E::load(ke[e]);
              vf[e] = E::load(ve[e]);
            }
#pragma unroll
            for (int g = 0; g < kHB; ++g) {
              float d = 0.f;
#pragma unroll
              for (int e = 0; e < kVec; ++e) d = fmaf(qr[g][e], kf[e], d);
              d = group_sum<kLPT>(d);
              sc[g] = live[u] ? d * a.scale_log2 : -INFINITY;
            }
#pragma unroll
            for (int g = 0; g < kHB; ++g) {
              const float m_new = fmaxf(m[g], sc[g]);
              const float alpha = exp2f(m[g] - m_new);
              const float pr = exp2f(sc[g] - m_new);
              m[g] = m_new;
              l[g] = l[g] * alpha + pr;
#pragma unroll
              for (int e = 0; e < kVec; ++e) acc[g][e] = fmaf(pr, vf[e], acc[g][e] * alpha);
            }
          }
        }
      }

      // merge the lane groups of the wave
#pragma unroll
      for (int off = kLPT; off < kWave; off <<= 1) {
#pragma unroll
        for (int g = 0; g < kHB; ++g) {
          const float m_o = __shfl_xor(m[g], off, kWave);
          const float l_o = __shfl_xor(l[g], off, kWave);
          const float m_new = fmaxf(m[g], m_o);
          const float sa = exp2f(m[g] - m_new), sb = exp2f(m_o - m_new);
          l[g] = l[g] * sa + l_o * sb;
#pragma unroll
          for (int e = 0; e < kVec; ++e) {
            const float a_o = __shfl_xor(acc[g][e], off, kWave);
            acc[g][e] = acc[g][e] * sa + a_o * sb;
          }
          m[g] = m_new;
        }
      }
      __syncthreads();
      if (lg == 0) {
#pragma unroll
        for (int g = 0; g < kHB; ++g) {
#pragma unroll
          for (int e = 0; e < kVec; ++e) acc_s[wave][g][li * kVec + e] = acc[g][e];
          if (li == 0) {
            ml_s[wave][g][0] = m[g];
            ml_s[wave][g][1] = l[g];
          }
        }
      }
      __syncthreads();
      // merge the waves and emit
      for (int e = threadIdx.x; e < kHB * kD; e += kGenThreads) {
        const int g = e / kD, d = e - g * kD;
        if (hb + g >= G) continue;
        float mm = kNegBig;
#pragma unroll
        for (int w = 0; w < kGenWaves; ++w) mm = fmaxf(mm, ml_s[w][g][0]);
        float ll = 0.f, av = 0.f;
#pragma unroll
        for (int w = 0; w < kGenWaves; ++w) {
          const float sw = exp2f(ml_s[w][g][0] - mm);
          ll += ml_s[w][g][1] * sw;
          av += acc_s[w][g][d] * sw;
        }
        const int hq = hk * G + hb + g;
        if (part_base < 0) {
          S* o = (S*)a.out + (out_row * a.num_q_heads + hq) * (long long)kD;
          o[d] = E::store(ll > 0.f ? av / ll : 0.f);
          if (d == 0 && a.lse) {
            const float lse2 = ll > 0.f ? mm + log2f(ll) : -INFINITY;
            a.lse[out_row * a.num_q_heads + hq] = a.lse_base2 ? lse2 : lse2 * kLn2;
          }
        } else {
          const long long slot = (long long)(part_base + iq) * a.num_q_heads + hq;
          a.part_acc[slot * kD + d] = av;
          if (d == 0) {
            a.part_ml[slot * 2 + 0] = mm;
            a.part_ml[slot * 2 + 1] = ll;
          }
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// merge of partial states: one workgroup of kMergeWaves waves per (row, q head)
// ---------------------------------------------------------------------------
// The launch is short and made of dependent loads (row list -> partial states), so it is laid out
// for latency: wave w folds partials w, w + kMergeWaves, ... of the row, eight per round (the last
// round exactly what is left) with all their loads in flight together, and the running states meet
// in LDS.  Lane l owns dims l, l + 64, ...
// Four waves for a decode batch (few rows, up to dozens of partial states each); one wave when the
// rows are many (split prefill tiles: thousands of rows of a few states each), where four times as
// many rows in flight per CU count for more than the parallel fold.
template <typename E, int kMergeWaves>
__global__ __launch_bounds__(64 * kMergeWaves) void merge_kernel(MergeArgs a) {
  using S = typename E::storage;
  const long long row = blockIdx.x;
  const int hq = blockIdx.y;
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int flags = a.row_flags[row];
  if (flags & VA_ROW_DIRECT) return;
  S* o = (S*)a.out + (row * a.num_q_heads + hq) * (long long)a.head_dim;
  if (flags & VA_ROW_EMPTY) {
    for (int d = threadIdx.x; d < a.head_dim; d += 64 * kMergeWaves) o[d] = E::store(0.f);
    if (threadIdx.x == 0 && a.lse) a.lse[row * a.num_q_heads + hq] = -INFINITY;
    return;
  }
  const int b = a.row_indptr[row], e = a.row_indptr[row + 1];
  const int n_d = (a.head_dim + 63) / 64;  // dims per lane: d = lane + 64*k (at most 4 for D = 256)
  float mm = kNegBig, ll = 0.f;
  float av[4] = {0.f, 0.f, 0.f, 0.f};
  // fold partials i0, i0 + kMergeWaves, ... (n of them): all loads first, then the fold in order
  auto fold = [&](int i0, auto n_tag) __attribute__((always_inline)) {
    constexpr int n = decltype(n_tag)::value;
    float mp[n], lp[n], ap[n][4];
#pragma unroll
    for (int u = 0; u < n; ++u) {
      const long long slot = (long long)a.row_ids[i0 + u * kMergeWaves] * a.num_q_heads + hq;
      mp[u] = a.part_ml[slot * 2];
      lp[u] = a.part_ml[slot * 2 + 1];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int d = lane + 64 * k;
        ap[u][k] = (k < n_d && d < a.head_dim) ? a.part_acc[slot * a.head_dim + d] : 0.f;
      }
    }
#pragma unroll
    for (int u = 0; u < n; ++u) {
      const float m_new = fmaxf(mm, mp[u]);
      const float sa = exp2f(mm - m_new), sb = exp2f(mp[u] - m_new);
      ll = ll * sa + lp[u] * sb;
#pragma unroll
      for (int k = 0; k < 4; ++k) av[k] = av[k] * sa + ap[u][k] * sb;
      mm = m_new;
    }
  };
  // this wave's partials, eight per round; the last round takes exactly what is left (a split
  // prefill row has two or three states: a padded round of eight would quadruple its loads)
  int i0 = b + wave;
  int mine = i0 < e ? (e - i0 + kMergeWaves - 1) / kMergeWaves : 0;
  for (; mine >= 8; mine -= 8, i0 += 8 * kMergeWaves) fold(i0, std::integral_constant<int, 8>{});
  if (mine & 4) {
    fold(i0, std::integral_constant<int, 4>{});
    i0 += 4 * kMergeWaves;
  }
  if (mine & 2) {
    fold(i0, std::integral_constant<int, 2>{});
    i0 += 2 * kMergeWaves;
  }
  if (mine & 1) fold(i0, std::integral_constant<int, 1>{});
  if constexpr (kMergeWaves > 1) {
    // fold the waves' states: wave 0 collects
    __shared__ float s_ml[kMergeWaves][2];
    __shared__ float s_av[kMergeWaves][4][64];
    if (wave > 0) {
      if (lane == 0) {
        s_ml[wave][0] = mm;
        s_ml[wave][1] = ll;
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) s_av[wave][k][lane] = av[k];
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int w = 1; w < kMergeWaves; ++w) {
      const float mw = s_ml[w][0], lw = s_ml[w][1];
      const float m_new = fmaxf(mm, mw);
      const float sa = exp2f(mm - m_new), sb = exp2f(mw - m_new);
      ll = ll * sa + lw * sb;
#pragma unroll
      for (int k = 0; k < 4; ++k) av[k] = av[k] * sa + s_av[w][k][lane] * sb;
      mm = m_new;
    }
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int d = lane + 64 * k;
    if (d < a.head_dim) o[d] = E::store(ll > 0.f ? av[k] / ll : 0.f);
  }
  if (lane == 0 && a.lse) {
    const float lse2 = ll > 0.f ? mm + log2f(ll) : -INFINITY;
    a.lse[row * a.num_q_heads + hq] = a.lse_base2 ? lse2 : lse2 * kLn2;
  }
}

template <typename E>
int launch_generic(const AttnArgs& a, int n_items, hipStream_t stream) {
  const dim3 grid((unsigned)n_items * (unsigned)a.num_kv_heads), block(kGenThreads);
  constexpr int kMaxD = 16 / sizeof(typename E::storage) * 64;
  switch (a.head_dim) {
#define VA_CASE(D)                                                              \
  case D:                                                                       \
    if constexpr (D <= kMaxD && D >= 16 / (int)sizeof(typename E::storage)) {   \
      hipLaunchKernelGGL((attn_generic_kernel<E, D>), grid, block, 0, stream, a); \
      break;                                                                    \
    }                                                                           \
    return va_fail(VA_ERR_ARG, "head_dim %d unsupported for this element type", a.head_dim);
    VA_CASE(16)
    VA_CASE(32)
    VA_CASE(64)
    VA_CASE(128)
    VA_CASE(256)
#undef VA_CASE
    default:
      return va_fail(VA_ERR_ARG, "head_dim %d unsupported (16, 32, 64, 128 or 256)", a.head_dim);
  }
  return check_hip(hipGetLastError(), "attention launch");
}

// `waves`: waves per (row, q head) workgroup, chosen by the planner (plan header).
template <typename E>
int launch_merge(const MergeArgs& a, int n_rows, int waves, hipStream_t stream) {
  const dim3 grid((unsigned)n_rows, (unsigned)a.num_q_heads);
  switch (waves) {
    case 1:
      hipLaunchKernelGGL((merge_kernel<E, 1>), grid, dim3(64), 0, stream, a);
      break;
    case 4:
      hipLaunchKernelGGL((merge_kernel<E, 4>), grid, dim3(256), 0, stream, a);
      break;
    case 8:
      hipLaunchKernelGGL((merge_kernel<E, 8>), grid, dim3(512), 0, stream, a);
      break;
    case 16:
      hipLaunchKernelGGL((merge_kernel<E, 16>), grid, dim3(1024), 0, stream, a);
      break;
    default:
      return va_fail(VA_ERR_ARG, "plan header: %d merge waves (1, 4, 8 or 16)", waves);
  }
  return check_hip(hipGetLastError(), "merge launch");
}

}  // namespace va

// ---------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------
#define VA_DISPATCH_DTYPE(dtype, CALL)                                  \
  switch (dtype) {                                                      \
    case VA_F32: { using E = va::F32; CALL; } break;                    \
    case VA_F16: { using E = va::F16; CALL; } break;                    \
    case VA_BF16: { using E = va::BF16; CALL; } break;                  \
    default: return va_fail(VA_ERR_ARG, "unknown dtype %d", (int)(dtype)); \
  }

extern "C" int va_rope(const void* x_dev, void* y_dev, const int64_t* pos_dev, int64_t pos_axis_stride,
                       int64_t n_rows, int32_t n_heads, int32_t head_dim, int32_t dtype,
                       int64_t x_row_stride, int64_t y_row_stride, const VaRope* rope, void* stream) {
  if (n_rows < 0 || n_heads <= 0 || head_dim <= 0) return va_fail(VA_ERR_ARG, "bad shape");
  if (n_rows == 0) return VA_OK;
  if (!x_dev || !y_dev || !pos_dev) return va_fail(VA_ERR_ARG, "null pointer");
  va::RopeDev r;
  int rc = va::make_rope(rope, head_dim, &r);
  if (rc) return rc;
  VA_DISPATCH_DTYPE(dtype, rc = va::launch_rope_store<E>(x_dev, nullptr, y_dev, nullptr, x_row_stride, 0,
                                                         y_row_stride, nullptr, 0, pos_dev, pos_axis_stride,
                                                         n_rows, n_heads, head_dim, r, (hipStream_t)stream));
  return rc;
}

extern "C" int va_store_kv_rope(const void* k_dev, const void* v_dev, int64_t k_row_stride,
                                int64_t v_row_stride, void* k_pool_dev, void* v_pool_dev,
                                int64_t pool_row_stride, const void* out_loc_dev, int32_t out_loc_is_i64,
                                const int64_t* pos_dev, int64_t pos_axis_stride, int64_t n_rows,
                                const VaShape* shape, const VaRope* rope, void* stream) {
  if (!shape) return va_fail(VA_ERR_ARG, "null shape");
  if (n_rows < 0) return va_fail(VA_ERR_ARG, "bad shape");
  if (n_rows == 0) return VA_OK;
  if (!k_dev || !v_dev || !k_pool_dev || !v_pool_dev || !out_loc_dev || !rope)
    return va_fail(VA_ERR_ARG, "null pointer");
  if (!pos_dev && rope->rotary_dim > 0) return va_fail(VA_ERR_ARG, "rotation needs positions");
  va::RopeDev r;
  int rc = va::make_rope(rope, shape->head_dim, &r);
  if (rc) return rc;
  VA_DISPATCH_DTYPE(shape->dtype,
                    rc = va::launch_rope_store<E>(k_dev, v_dev, k_pool_dev, v_pool_dev, k_row_stride, v_row_stride,
                                                  pool_row_stride, out_loc_dev, out_loc_is_i64, pos_dev,
                                                  pos_axis_stride, n_rows, shape->num_kv_heads, shape->head_dim, r,
                                                  (hipStream_t)stream));
  return rc;
}

// Both attention entry points: `workspace_dev` is the caller's buffer (va_attention) or this
// device's copy of the library's own scratch array (va_attention_static).
static int attention_launches(const void* q_dev, int64_t q_row_stride, const void* k_pool_dev,
                              const void* v_pool_dev, int64_t pool_row_stride, const int32_t* plan_dev,
                              const int32_t* plan_header_host, const int32_t* kv_indices_dev,
                              const int64_t* sub_worker_dev, const int64_t* sub_loc_dev,
                              int64_t sub_loc_axis_stride, void* out_dev, float* lse_dev, int32_t lse_base2,
                              void* workspace_dev, int64_t workspace_bytes, const VaShape* shape,
                              const VaRope* rope, void* stream) {
  if (!shape || !plan_header_host || !plan_dev) return va_fail(VA_ERR_ARG, "null plan or shape");
  const int32_t* h = plan_header_host;
  if (h[VA_H_MAGIC] != VA_PLAN_MAGIC) return va_fail(VA_ERR_ARG, "plan header has no magic word");
  const int n_rows = h[VA_H_N_ROWS], n_items = h[VA_H_N_ITEMS], n_partials = h[VA_H_N_PARTIALS];
  if (n_rows == 0) return VA_OK;
  // the kernels map workgroup -> (item, head) assuming each launch covers a multiple of 8 items
  if (n_items % 8 || h[VA_H_N_WIDE] % 8 || h[VA_H_N_WIDE] < 0 || h[VA_H_N_WIDE] > n_items)
    return va_fail(VA_ERR_ARG, "plan header: item counts (%d, %d wide) are not padded to the 8 dies", n_items,
                   h[VA_H_N_WIDE]);
  if (h[VA_H_N_WIDE_SLOTS] % 8 || h[VA_H_N_WIDE_SLOTS] < 0 || h[VA_H_N_WIDE_SLOTS] > h[VA_H_N_WIDE])
    return va_fail(VA_ERR_ARG, "plan header: %d wide slots for %d wide items", h[VA_H_N_WIDE_SLOTS], h[VA_H_N_WIDE]);
  if (!out_dev) return va_fail(VA_ERR_ARG, "null out");
  if (n_items > 0 && (!q_dev || !k_pool_dev || !v_pool_dev || !sub_worker_dev || !sub_loc_dev || !kv_indices_dev))
    return va_fail(VA_ERR_ARG, "null pointer");
  if (shape->num_kv_heads <= 0 || shape->num_q_heads % shape->num_kv_heads)
    return va_fail(VA_ERR_ARG, "num_q_heads must be a multiple of num_kv_heads");
  const int64_t need = va_workspace_bytes_for(n_partials, shape->num_q_heads, shape->head_dim);
  if (need > 0 && (!workspace_dev || workspace_bytes < need))
    return va_fail(VA_ERR_CAPACITY, "workspace needs %lld bytes, got %lld", (long long)need, (long long)workspace_bytes);
  va::RopeDev r;
  int rc = va::make_rope(rope, shape->head_dim, &r);
  if (rc) return rc;

  va::AttnArgs a;
  a.q = q_dev;
  a.q_row_stride = q_row_stride;
  a.k_pool = k_pool_dev;
  a.v_pool = v_pool_dev;
  a.pool_row_stride = pool_row_stride;
  a.items = plan_dev + h[VA_H_OFF_ITEMS];
  a.links = plan_dev + h[VA_H_OFF_LINKS];
  a.qrefs = plan_dev + h[VA_H_OFF_QREFS];
  a.qref_rows = plan_dev + h[VA_H_OFF_QREF_ROWS];
  a.wide_slots = plan_dev + h[VA_H_OFF_WIDE_SLOTS];
  a.kv_indices = kv_indices_dev;
  a.sub_worker = sub_worker_dev;
  a.sub_loc = sub_loc_dev;
  a.sub_loc_axis_stride = sub_loc_axis_stride;
  a.out = out_dev;
  a.lse = lse_dev;
  a.lse_base2 = lse_base2;
  a.part_acc = (float*)workspace_dev;
  a.part_ml = (float*)workspace_dev + (int64_t)n_partials * shape->num_q_heads * shape->head_dim;
  a.num_q_heads = shape->num_q_heads;
  a.num_kv_heads = shape->num_kv_heads;
  a.head_dim = shape->head_dim;
  a.page_size = shape->page_size;
  a.rope = r;
  a.scale_log2 = va::kLog2e / sqrtf((float)shape->head_dim);
  hipStream_t s = (hipStream_t)stream;

  if (n_items > 0) {
    if (h[VA_H_KERNEL] == VA_KERNEL_MFMA) {
      rc = va::launch_mfma(a, shape->dtype, n_items, h[VA_H_N_WIDE], h[VA_H_N_WIDE_SLOTS], h[VA_H_Q_TILE], s);
    } else {
      VA_DISPATCH_DTYPE(shape->dtype, rc = va::launch_generic<E>(a, n_items, s));
    }
    if (rc) return rc;
  }
  if (n_partials > 0 || h[VA_H_N_EMPTY_ROWS] > 0) {
    va::MergeArgs m;
    m.row_indptr = plan_dev + h[VA_H_OFF_ROW_INDPTR];
    m.row_ids = plan_dev + h[VA_H_OFF_ROW_IDS];
    m.row_flags = plan_dev + h[VA_H_OFF_ROW_FLAGS];
    m.part_acc = a.part_acc;
    m.part_ml = a.part_ml;
    m.out = out_dev;
    m.lse = lse_dev;
    m.lse_base2 = lse_base2;
    m.num_q_heads = shape->num_q_heads;
    m.head_dim = shape->head_dim;
    VA_DISPATCH_DTYPE(shape->dtype, rc = va::launch_merge<E>(m, n_rows, h[VA_H_MERGE_WAVES], s));
  }
  return rc;
}

extern "C" int va_attention(const void* q_dev, int64_t q_row_stride, const void* k_pool_dev,
                            const void* v_pool_dev, int64_t pool_row_stride, const int32_t* plan_dev,
                            const int32_t* plan_header_host, const int32_t* kv_indices_dev,
                            const int64_t* sub_worker_dev, const int64_t* sub_loc_dev,
                            int64_t sub_loc_axis_stride, void* out_dev, float* lse_dev, int32_t lse_base2,
                            void* workspace_dev, int64_t workspace_bytes, const VaShape* shape,
                            const VaRope* rope, void* stream) {
  return attention_launches(q_dev, q_row_stride, k_pool_dev, v_pool_dev, pool_row_stride, plan_dev, plan_header_host,
                            kv_indices_dev, sub_worker_dev, sub_loc_dev, sub_loc_axis_stride, out_dev, lse_dev,
                            lse_base2, workspace_dev, workspace_bytes, shape, rope, stream);
}

// ---------------------------------------------------------------------------
// va_attention_static: the same launches over a scratch array the library owns
// ---------------------------------------------------------------------------
// Partial softmax states of rows served by several work items live here instead of in a caller's
// workspace.  Every GPU the library runs on holds its own copy of the array, at its own address,
// until the process ends.  In host code the array's name only stands for the symbol: the address
// kernels may use is looked up once per device (hipGetSymbolAddress, with that device current) and
// kept; nothing below passes the name itself to a kernel.
static __device__ __align__(256) unsigned char scratch[VA_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {nullptr};

// Device address of the current device's copy of `scratch` (NULL on failure, error recorded).
void* static_scratch_of_current_device() {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess || device < 0 || device >= kMaxDevices) {
    va_fail(VA_ERR_HIP, "static scratch: no current device (%s)", hipGetErrorString(e));
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[device]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      va_fail(VA_ERR_HIP, "static scratch: hipGetSymbolAddress on device %d: %s", device, hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptr[device] = ptr;
  }
  return g_scratch_ptr[device];
}
}  // namespace

extern "C" int va_attention_static(const void* q_dev, int64_t q_row_stride, const void* k_pool_dev,
                                   const void* v_pool_dev, int64_t pool_row_stride, const int32_t* plan_dev,
                                   const int32_t* plan_header_host, const int32_t* kv_indices_dev,
                                   const int64_t* sub_worker_dev, const int64_t* sub_loc_dev,
                                   int64_t sub_loc_axis_stride, void* out_dev, float* lse_dev, int32_t lse_base2,
                                   const VaShape* shape, const VaRope* rope, void* stream) {
  if (!shape || !plan_header_host) return va_fail(VA_ERR_ARG, "null plan or shape");
  if (plan_header_host[VA_H_MAGIC] != VA_PLAN_MAGIC) return va_fail(VA_ERR_ARG, "plan header has no magic word");
  const int64_t need = va_workspace_bytes_for(plan_header_host[VA_H_N_PARTIALS], shape->num_q_heads, shape->head_dim);
  if (need > (int64_t)VA_STATIC_SCRATCH_BYTES)
    return va_fail(VA_ERR_CAPACITY,
                   "va_attention_static: the plan's %d partial states need %lld bytes of scratch, the library's "
                   "array holds %lld; use va_attention with a workspace of the caller's",
                   plan_header_host[VA_H_N_PARTIALS], (long long)need, (long long)VA_STATIC_SCRATCH_BYTES);
  void* ptr = static_scratch_of_current_device();
  if (!ptr) return VA_ERR_HIP;
  return attention_launches(q_dev, q_row_stride, k_pool_dev, v_pool_dev, pool_row_stride, plan_dev, plan_header_host,
                            kv_indices_dev, sub_worker_dev, sub_loc_dev, sub_loc_axis_stride, out_dev, lse_dev,
                            lse_base2, ptr, (int64_t)VA_STATIC_SCRATCH_BYTES, shape, rope, stream);
}
