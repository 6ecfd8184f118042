// Block merge / append: copy the K and V rows of a run of tokens to other pool slots, in every
// layer, moving the copied keys into the destination block's position frame on the way.
//
// The reference does this per layer with index_select + index_copy_ for K and V and then a second
// gather, an fp32 rotation and a scatter for the keys (session.py:470-528); here one launch reads
// every source row once and writes every destination row once.  Bound by HBM:
// 4 * layers * kv_heads * head_dim * sizeof(element) bytes per token.
//
// Work split: a workgroup owns kTokens consecutive tokens of one layer.  A thread owns one 16-byte
// piece position of the row -- a rotary pair piece of K (elements [8j, 8j+8) of a head and their
// partners half a rotary_dim further), a pass-through piece of K, or a piece of V -- and walks the
// tokens with it, so the cos/sin of its pair (the shift is the same for every token) stay in
// registers.  Loads of four tokens are issued before the first store: the pool is read and written
// through the same pointer, so the compiler cannot reorder them itself.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "va_device.h"
#include "va_internal.h"
#include "va_launch.h"

namespace va {

#ifndef VA_COPY_TOKENS
#define VA_COPY_TOKENS 16
#endif
#ifndef VA_COPY_BATCH
#define VA_COPY_BATCH 4
#endif
constexpr int kCopyTokens = VA_COPY_TOKENS;  // tokens per workgroup
constexpr int kCopyBatch = VA_COPY_BATCH;    // tokens whose loads are in flight together

template <typename S, int kVec>
struct alignas(kVec * sizeof(S) == 16 ? 16 : alignof(S)) Piece {
  S v[kVec];
};

// 16-byte pieces travel as non-temporal loads and stores: every row is read once and written once,
// nothing of it is worth a place in the caches (two 16 384-token blocks over four layers: 259 -> 247 us).
typedef uint32_t va_copy_u32x4 __attribute__((ext_vector_type(4)));

template <typename S, int kVec>
__device__ __forceinline__ Piece<S, kVec> load_piece(const S* p) {
  Piece<S, kVec> out;
  if constexpr (kVec * sizeof(S) == 16) {
    *reinterpret_cast<va_copy_u32x4*>(out.v) = __builtin_nontemporal_load(reinterpret_cast<const va_copy_u32x4*>(p));
  } else {
#pragma unroll
    for (int i = 0; i < kVec; ++i) out.v[i] = p[i];
  }
  return out;
}

template <typename S, int kVec>
__device__ __forceinline__ void store_piece(S* p, const Piece<S, kVec>& x) {
  if constexpr (kVec * sizeof(S) == 16) {
    __builtin_nontemporal_store(*reinterpret_cast<const va_copy_u32x4*>(x.v), reinterpret_cast<va_copy_u32x4*>(p));
  } else {
#pragma unroll
    for (int i = 0; i < kVec; ++i) p[i] = x.v[i];
  }
}

struct CopyArgs {
  void* k_pool;
  void* v_pool;
  long long pool_row_stride;  // elements between token slots
  long long layer_stride;     // elements between the pools of consecutive layers
  const int64_t* src;
  const int64_t* dst;
  long long n_tokens;
  long long shift;  // position shift of the copied keys (0: plain copy)
  int num_kv_heads, head_dim;
  RopeDev rope;
};

template <typename E, int kVec>
__global__ __launch_bounds__(1024) void copy_shift_kernel(CopyArgs a) {
  using S = typename E::storage;
  using P = Piece<S, kVec>;
  const long long layer = blockIdx.y;
  const long long t0 = (long long)blockIdx.x * kCopyTokens;
  const int n_tok = (int)min((long long)kCopyTokens, a.n_tokens - t0);
  S* kp = (S*)a.k_pool + layer * a.layer_stride;
  S* vp = (S*)a.v_pool + layer * a.layer_stride;
  const int D = a.head_dim;
  const bool rotate = a.shift != 0 && a.rope.half > 0;
  const int half = rotate ? a.rope.half : 0;
  const int pair_pieces = half / kVec;                 // per head
  const int pass_pieces = (D - 2 * half) / kVec;       // per head: K pieces that are only copied
  const int n_pair = a.num_kv_heads * pair_pieces;
  const int n_pass = a.num_kv_heads * pass_pieces;
  const int n_v = a.num_kv_heads * D / kVec;
  const Pos3 pos{a.shift, a.shift, a.shift};

  for (int task = threadIdx.x; task < n_pair + n_pass + n_v; task += blockDim.x) {
    if (task < n_pair) {
      const int h = task / pair_pieces, j = task - h * pair_pieces;
      const long long off = (long long)h * D + (long long)j * kVec;
      float c[kVec], s[kVec];
#pragma unroll
      for (int e = 0; e < kVec; ++e) rope_cos_sin(a.rope, pos, j * kVec + e, c[e], s[e]);
      for (int b = 0; b < n_tok; b += kCopyBatch) {
        P x1[kCopyBatch], x2[kCopyBatch];
#pragma unroll
        for (int u = 0; u < kCopyBatch; ++u) {
          if (b + u < n_tok) {
            const S* row = kp + a.src[t0 + b + u] * a.pool_row_stride + off;
            x1[u] = load_piece<S, kVec>(row);
            x2[u] = load_piece<S, kVec>(row + half);
          }
        }
#pragma unroll
        for (int u = 0; u < kCopyBatch; ++u) {
          if (b + u < n_tok) {
            P y1, y2;
#pragma unroll
            for (int e = 0; e < kVec; ++e) {
              // the reference rotates float copies of the keys and rounds once (session.py:519-527)
              float r1, r2;
              rope_pair<F32>(a.rope, c[e], s[e], E::load(x1[u].v[e]), E::load(x2[u].v[e]), r1, r2);
              y1.v[e] = E::store(r1);
              y2.v[e] = E::store(r2);
            }
            S* row = kp + a.dst[t0 + b + u] * a.pool_row_stride + off;
            store_piece<S, kVec>(row, y1);
            store_piece<S, kVec>(row + half, y2);
          }
        }
      }
    } else {
      // plain pieces: the rest of K, then V
      S* pool = kp;
      long long off;
      int t = task - n_pair;
      if (t < n_pass) {
        const int h = t / pass_pieces, j = t - h * pass_pieces;
        off = (long long)h * D + 2 * half + (long long)j * kVec;
      } else {
        pool = vp;
        off = (long long)(t - n_pass) * kVec;
      }
      for (int b = 0; b < n_tok; b += kCopyBatch) {
        P x[kCopyBatch];
#pragma unroll
        for (int u = 0; u < kCopyBatch; ++u)
          if (b + u < n_tok) x[u] = load_piece<S, kVec>(pool + a.src[t0 + b + u] * a.pool_row_stride + off);
#pragma unroll
        for (int u = 0; u < kCopyBatch; ++u)
          if (b + u < n_tok) store_piece<S, kVec>(pool + a.dst[t0 + b + u] * a.pool_row_stride + off, x[u]);
      }
    }
  }
}

template <typename E>
static int launch_copy_shift(const CopyArgs& a, int num_layers, hipStream_t stream) {
  using S = typename E::storage;
  constexpr int kWide = 16 / (int)sizeof(S);
  const bool rotate = a.shift != 0 && a.rope.half > 0;
  const int half = rotate ? a.rope.half : 0;
  auto aligned = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
  const bool wide = a.head_dim % kWide == 0 && half % kWide == 0 && a.pool_row_stride % kWide == 0 &&
                    a.layer_stride % kWide == 0 && aligned(a.k_pool) && aligned(a.v_pool);
  const int vec = wide ? kWide : 1;
  const long long tasks = (long long)a.num_kv_heads * (half / vec + (a.head_dim - 2 * half) / vec + a.head_dim / vec);
  const unsigned threads = (unsigned)std::min<long long>(1024, (tasks + 63) / 64 * 64);
  const long long groups = (a.n_tokens + kCopyTokens - 1) / kCopyTokens;
  if (groups > 0x7fffffffLL || num_layers > 65535) return va_fail(VA_ERR_ARG, "too many tokens or layers for one launch");
  const dim3 grid((unsigned)groups, (unsigned)num_layers);
  if (wide) {
    hipLaunchKernelGGL((copy_shift_kernel<E, kWide>), grid, dim3(threads), 0, stream, a);
  } else {
    hipLaunchKernelGGL((copy_shift_kernel<E, 1>), grid, dim3(threads), 0, stream, a);
  }
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? VA_OK : va_fail(VA_ERR_HIP, "copy/shift launch: %s", hipGetErrorString(e));
}

}  // namespace va

extern "C" int va_copy_shift_kv(void* k_pool_dev, void* v_pool_dev, int64_t pool_row_stride, int64_t layer_stride,
                                int32_t num_layers, const int64_t* src_slots_dev, const int64_t* dst_slots_dev,
                                int64_t n_tokens, int64_t position_shift, const VaShape* shape, const VaRope* rope,
                                void* stream) {
  if (!shape) return va_fail(VA_ERR_ARG, "null shape");
  if (n_tokens < 0 || num_layers < 0) return va_fail(VA_ERR_ARG, "negative count");
  if (n_tokens == 0 || num_layers == 0) return VA_OK;
  if (!k_pool_dev || !v_pool_dev || !src_slots_dev || !dst_slots_dev) return va_fail(VA_ERR_ARG, "null pointer");
  if (shape->num_kv_heads <= 0 || shape->head_dim <= 0) return va_fail(VA_ERR_ARG, "bad shape");
  if (pool_row_stride < (int64_t)shape->num_kv_heads * shape->head_dim)
    return va_fail(VA_ERR_ARG, "pool rows overlap: stride %lld < %d elements", (long long)pool_row_stride,
                   shape->num_kv_heads * shape->head_dim);
  va::CopyArgs a;
  a.k_pool = k_pool_dev;
  a.v_pool = v_pool_dev;
  a.pool_row_stride = pool_row_stride;
  a.layer_stride = layer_stride;
  a.src = src_slots_dev;
  a.dst = dst_slots_dev;
  a.n_tokens = n_tokens;
  a.shift = position_shift;
  a.num_kv_heads = shape->num_kv_heads;
  a.head_dim = shape->head_dim;
  if (position_shift != 0) {
    const int rc = va::make_rope(rope, shape->head_dim, &a.rope);
    if (rc) return rc;
  } else {
    a.rope = va::RopeDev{};
  }
  switch (shape->dtype) {
    case VA_F32:
      return va::launch_copy_shift<va::F32>(a, num_layers, (hipStream_t)stream);
    case VA_F16:
      return va::launch_copy_shift<va::F16>(a, num_layers, (hipStream_t)stream);
    case VA_BF16:
      return va::launch_copy_shift<va::BF16>(a, num_layers, (hipStream_t)stream);
    default:
      return va_fail(VA_ERR_ARG, "unknown dtype %d", (int)shape->dtype);
  }
}
