// Matrix-core (MFMA) view attention for 16-bit element types on gfx950.
//
// One workgroup of four waves per (work item, kv head).  The item's query tile
// is at most 16 MFMA rows: row j = (tile row j / G, head j % G) with G = q heads
// per kv head, so a decode tile batches 16/G requests that read the same KV run.
// Each wave streams every fourth 32-token tile of the chain:
//
//   S^T[token, row]  = K[token, :] . Q^T[:, row]        v_mfma_f32_16x16x32, K as the A operand
//   online softmax per row (row = lane % 16, so all of a lane's scores share a row)
//   O^T[dim, row]   += V^T[dim, token] . P^T[token, row] V as the A operand, P as the B operand
//
// K fragments are loaded straight into the A-operand layout (16 bytes per lane).
// The S^T accumulator layout (lane holds tokens 4*(lane/16)+r of each 16-token
// half) is exactly the B-operand layout of P once the contraction index of the
// second product is permuted accordingly, so P never moves between lanes.  V is
// loaded so that the 16 lanes of a group read one contiguous run of a token row;
// the 8-token x (D/16)-dim block each lane holds is transposed in registers with
// v_perm_b32 into A operands.  The query tile is rotated for the current link
// (sub-request) by all 256 threads into LDS and read back as B operands.
//
// Memory pipeline: the K registers are free as soon as the scores are computed
// and the V registers as soon as the output is updated, so the loads of the next
// tile's K are issued right after Q.K^T and those of its V right after P.V; a
// wave always has 16-32 KB of loads in flight while it computes, at no register
// cost.  Page-table entries are wave-uniform when the page size is a multiple of
// 16 (a 16-token half tile never straddles a page) and are fetched with scalar
// loads one tile ahead.
//
// Wave states are merged through LDS; the result goes to `out` or to a partial
// slot for the merge kernel.
#include <hip/hip_runtime.h>

#include "va_internal.h"
#include "va_launch.h"
#include "va_mfma_common.h"

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
int va_mfma_wide_q_tile(int gqa) { return 128 / gqa; }

namespace va {

constexpr int kMfmaThreads = 256;
constexpr int kMfmaWaves = 4;
constexpr int kTileTokens = 32;

#ifndef VA_MFMA_MIN_BLOCKS
#define VA_MFMA_MIN_BLOCKS 2  // workgroups per CU the register allocation must allow
#endif

#if VA_NARROW_EXPERIMENT == 2  // per-workgroup timeline: start, prologue end, loop end, end, hardware id
__device__ unsigned long long va_debug_times[5 * 16384];
extern "C" __attribute__((visibility("default"))) int va_debug_read(void* host, size_t bytes) {
  return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(va_debug_times), bytes);
}
#define VA_STAMP(k) \
  if (threadIdx.x == 0 && blockIdx.x < 16384) va_debug_times[5 * blockIdx.x + (k)] = wall_clock64();
#else
#define VA_STAMP(k)
#endif

template <typename E, int kD>
__global__ __launch_bounds__(kMfmaThreads, VA_MFMA_MIN_BLOCKS) void attn_mfma_kernel(AttnArgs a) {
  VA_STAMP(0)
#if VA_NARROW_EXPERIMENT == 2
  if (threadIdx.x == 0 && blockIdx.x < 16384)
    va_debug_times[5 * blockIdx.x + 4] = __builtin_amdgcn_s_getreg(4 | (31 << 11)) |
                                         ((unsigned long long)__builtin_amdgcn_s_getreg(20 | (31 << 11)) << 32);
#endif
  using S = typename E::storage;
  constexpr int kSteps = kD / 32;     // contraction steps of Q.K^T
  constexpr int kDimTiles = kD / 16;  // 16-dim tiles of the output
  constexpr int kChunks = kD / 8;     // 16-byte pieces of a head row
  constexpr int kVDw = kD / 32;       // dwords of a V token a lane holds (D/16 dims)
  constexpr int kStride = kMfmaWaves * kTileTokens;

  __shared__ va_u32x4 q_s[16][kChunks + 1];
  __shared__ float o_s[2][16][kD + 4];
  __shared__ float ml_s[2][16][2];

  const ItemHead where = item_and_head(blockIdx.x, a.num_kv_heads);
  const int32_t* item = a.items + (long long)where.item * VA_ITEM_WORDS;
  const int hk = where.head;
  const int G = a.num_q_heads / a.num_kv_heads;
  const int n_q = item[VA_I_N_Q];
  if (n_q == 0) return;  // padding item: keeps the launch order aligned with the die round-robin
  const int part_base = item[VA_I_PART_BASE];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int lane = tid % kWave;
  const int j = lane % 16;   // MFMA row of this lane: tile row j / G, head j % G
  const int kg = lane / 16;  // contraction group
  const int row_iq = j / G;
  const S* kp = (const S*)a.k_pool + (long long)hk * kD + 8 * kg;         // + row*stride + 32*s
  const S* vp = (const S*)a.v_pool + (long long)hk * kD + j * (kD / 16);  // + row*stride
  const int P = a.page_size;

  float m_run = kNegBig, l_run = 0.f;
  va_f32x4 o[kDimTiles];
#pragma unroll
  for (int t = 0; t < kDimTiles; ++t) o[t] = va_f32x4{0.f, 0.f, 0.f, 0.f};

  for (int li = 0; li < item[VA_I_N_LINKS]; ++li) {
    const int32_t* link = a.links + (long long)(item[VA_I_LINK_BEGIN] + li) * VA_LINK_WORDS;
    const int lflags = link[VA_L_FLAGS];
    const int qref = link[VA_L_QREF];
    const int kv_begin = link[VA_L_KV_BEGIN];
    const int tok_end = link[VA_L_TOK_END];
    const int causal_base = link[VA_L_CAUSAL_BASE];
    const bool slots = lflags & VA_LINK_SLOTS;
    const bool uniform_pages = !slots && (P % 16 == 0);

    // ---- rotate the query tile for this link into LDS ----
    __syncthreads();
    for (int idx = tid; idx < 16 * kChunks; idx += kMfmaThreads) {
      const int jr = idx / kChunks, c = idx - jr * kChunks;
      const int iq = jr / G, g = jr - iq * G;
      va_u32x4 packed = {0, 0, 0, 0};
      if (iq < n_q) {
        const int subrow = (lflags & VA_LINK_INDIRECT) ? a.qrefs[qref + iq] : qref + iq;
        const long long src_row = a.sub_worker[subrow];
        const S* qh = (const S*)a.q + src_row * a.q_row_stride + (long long)(hk * G + g) * kD;
        const Pos3 p = load_pos(a.sub_loc, a.sub_loc_axis_stride, subrow);
        const uint4 piece = rotated_query_piece<E>(a.rope, qh, c * 8, p);
        packed = va_u32x4{piece.x, piece.y, piece.z, piece.w};
      }
      q_s[jr][c] = packed;
    }
    __syncthreads();

    // visible range of this link for the tile and for this lane's row
    const int t_stop = min(tok_end, causal_base + n_q);
    const int t_row = min(tok_end, causal_base + row_iq + 1);
    const int t_last = t_stop - 1;

    // Pool rows of the two 16-token halves of the tile starting at t0 (uniform pages):
    // row of token min(t0 + 16u, t_last) rounded down to its 16-token group.  Every
    // clamped token of the half lies in that group, so lanes only add their offset.
    auto half_rows = [&](int t0, long long (&rows)[2]) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int t = min(t0 + 16 * u, t_last);
        const int page = __builtin_amdgcn_readfirstlane(a.kv_indices[kv_begin + t / P]);
        rows[u] = (long long)page * P + ((t % P) & ~15);
      }
    };
    // K fragments: lane (j, kg) holds dims [32s + 8kg, +8) of tokens t0 + j and t0 + 16 + j.
    auto load_k = [&](int t0, const long long (&rows)[2], va_u32x4 (&kf)[2][kSteps]) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int t = min(t0 + 16 * u + j, t_last);
        const long long row = uniform_pages ? rows[u] + (t & 15) : kv_slot(a.kv_indices, kv_begin, t, P, slots);
        const S* kr = kp + row * a.pool_row_stride;
#pragma unroll
        for (int s = 0; s < kSteps; ++s) kf[u][s] = *(const va_u32x4*)(kr + 32 * s);
      }
    };
    // V block: lane (j, kg) holds dims [j*D/16, +D/16) of the 8 tokens it scores:
    // t0 + 16*(e/4) + 4*kg + e%4, e = 0..7.
    auto load_v = [&](int t0, const long long (&rows)[2], uint32_t (&vraw)[8][kVDw]) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int t = min(t0 + 16 * (e / 4) + 4 * kg + (e % 4), t_last);
        const long long row = uniform_pages ? rows[e / 4] + (t & 15) : kv_slot(a.kv_indices, kv_begin, t, P, slots);
        const S* vr = vp + row * a.pool_row_stride;
        if constexpr (kVDw == 8) {
          const va_u32x4 x = *(const va_u32x4*)vr, y = *(const va_u32x4*)(vr + 8);
          vraw[e][0] = x[0]; vraw[e][1] = x[1]; vraw[e][2] = x[2]; vraw[e][3] = x[3];
          vraw[e][4] = y[0]; vraw[e][5] = y[1]; vraw[e][6] = y[2]; vraw[e][7] = y[3];
        } else if constexpr (kVDw == 4) {
          const va_u32x4 x = *(const va_u32x4*)vr;
          vraw[e][0] = x[0]; vraw[e][1] = x[1]; vraw[e][2] = x[2]; vraw[e][3] = x[3];
        } else {
          const uint2 x = *(const uint2*)vr;
          vraw[e][0] = x.x; vraw[e][1] = x.y;
        }
      }
    };

    VA_STAMP(1)
    int t0 = link[VA_L_TOK_BEGIN] + wave * kTileTokens;
    if (t0 < t_stop) {
      va_u32x4 kf[2][kSteps];
      uint32_t vraw[8][kVDw];
      long long rows[2] = {0, 0};
      if (uniform_pages) half_rows(t0, rows);
      load_k(t0, rows, kf);
      load_v(t0, rows, vraw);
      while (true) {
        const int tn = t0 + kStride;
        const bool more = tn < t_stop;
        if (more && uniform_pages) half_rows(tn, rows);

        // ---- scores: S^T = K . Q^T ----
        va_f32x4 sc[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          sc[u] = va_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s = 0; s < kSteps; ++s) sc[u] = Mma<E>::run(kf[u][s], q_s[j][4 * s + kg], sc[u]);
        }
        if (more) load_k(tn, rows, kf);  // K registers are free again

        // ---- online softmax (row = lane % 16) ----
        float tile_max = -INFINITY;
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int t = t0 + 16 * u + 4 * kg + r;
            const float v = t < t_row ? sc[u][r] * a.scale_log2 : -INFINITY;
            sc[u][r] = v;
            tile_max = fmaxf(tile_max, v);
          }
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, kWave));
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, kWave));
        const float m_new = fmaxf(m_run, tile_max);
        const float alpha = exp2f(m_run - m_new);
        m_run = m_new;
        float psum = 0.f;
        float pr[8];
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float p = exp2f(sc[u][r] - m_new);
            pr[4 * u + r] = p;
            psum += p;
          }
        l_run = l_run * alpha + psum;
        if (__any(alpha != 1.f)) {
#pragma unroll
          for (int t = 0; t < kDimTiles; ++t) o[t] *= alpha;
        }
        const va_u32x4 pf = {Mma<E>::pack(pr[0], pr[1]), Mma<E>::pack(pr[2], pr[3]), Mma<E>::pack(pr[4], pr[5]),
                             Mma<E>::pack(pr[6], pr[7])};

        // ---- O^T += V^T . P^T, one 16-dim tile at a time; tile T takes element T of the lane's run ----
#pragma unroll
        for (int t = 0; t < kDimTiles; ++t) {
          const int w = t / 2;
          const uint32_t sel = (t & 1) ? 0x07060302u : 0x05040100u;
          const va_u32x4 vf = {__builtin_amdgcn_perm(vraw[1][w], vraw[0][w], sel),
                               __builtin_amdgcn_perm(vraw[3][w], vraw[2][w], sel),
                               __builtin_amdgcn_perm(vraw[5][w], vraw[4][w], sel),
                               __builtin_amdgcn_perm(vraw[7][w], vraw[6][w], sel)};
          o[t] = Mma<E>::run(vf, pf, o[t]);
        }
        if (!more) break;
        load_v(tn, rows, vraw);  // V registers are free again
        t0 = tn;
      }
    }
  }

  VA_STAMP(2)
  // row sums live spread over the four contraction groups
  l_run += __shfl_xor(l_run, 16, kWave);
  l_run += __shfl_xor(l_run, 32, kWave);

  // ---- merge the four waves: (2,3) -> LDS, (0,1) fold them in, 1 -> LDS, 0 folds and emits ----
  auto spill = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < kDimTiles; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) o_s[buf][j][(4 * kg + r) * (kD / 16) + t] = o[t][r];
    if (kg == 0) {
      ml_s[buf][j][0] = m_run;
      ml_s[buf][j][1] = l_run;
    }
  };
  auto fold = [&](int buf) __attribute__((always_inline)) {
    const float m_o = ml_s[buf][j][0], l_o = ml_s[buf][j][1];
    const float m_new = fmaxf(m_run, m_o);
    const float sa = exp2f(m_run - m_new), sb = exp2f(m_o - m_new);
    l_run = l_run * sa + l_o * sb;
    m_run = m_new;
#pragma unroll
    for (int t = 0; t < kDimTiles; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) o[t][r] = o[t][r] * sa + o_s[buf][j][(4 * kg + r) * (kD / 16) + t] * sb;
  };
  __syncthreads();
  if (wave >= 2) spill(wave - 2);
  __syncthreads();
  if (wave < 2) fold(wave);
  __syncthreads();
  if (wave == 1) spill(0);
  __syncthreads();
  if (wave == 0) {
    fold(0);
    spill(1);
  }
  __syncthreads();

  // ---- emit: all threads, coalesced over the head dimension ----
  const int32_t* link0 = a.links + (long long)item[VA_I_LINK_BEGIN] * VA_LINK_WORDS;
  for (int idx = tid; idx < 16 * kD; idx += kMfmaThreads) {
    const int jr = idx / kD, d = idx - jr * kD;
    const int iq = jr / G, g = jr - iq * G;
    if (iq >= n_q) continue;
    const int hq = hk * G + g;
    const float mm = ml_s[1][jr][0], ll = ml_s[1][jr][1];
    const float av = o_s[1][jr][d];
    if (part_base < 0) {
      const int subrow = (link0[VA_L_FLAGS] & VA_LINK_INDIRECT) ? a.qrefs[link0[VA_L_QREF] + iq] : link0[VA_L_QREF] + iq;
      const long long out_row = a.sub_worker[subrow];
      ((S*)a.out)[(out_row * a.num_q_heads + hq) * (long long)kD + d] = E::store(ll > 0.f ? av / ll : 0.f);
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
  VA_STAMP(3)
}

template <typename E>
static int launch_mfma_typed(const AttnArgs& a, int n_items, hipStream_t stream) {
  if (n_items == 0) return VA_OK;
  const dim3 grid((unsigned)n_items * (unsigned)a.num_kv_heads), block(kMfmaThreads);
  switch (a.head_dim) {
    case 64:
      hipLaunchKernelGGL((attn_mfma_kernel<E, 64>), grid, block, 0, stream, a);
      break;
    case 128:
      hipLaunchKernelGGL((attn_mfma_kernel<E, 128>), grid, block, 0, stream, a);
      break;
    case 256:
      hipLaunchKernelGGL((attn_mfma_kernel<E, 256>), grid, block, 0, stream, a);
      break;
    default:
      return va_fail(VA_ERR_ARG, "matrix-core path supports head_dim 64, 128, 256");
  }
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? VA_OK : va_fail(VA_ERR_HIP, "attention launch: %s", hipGetErrorString(e));
}

int launch_mfma(const AttnArgs& a_in, int dtype, int n_items, int n_wide, int q_tile, hipStream_t stream) {
  AttnArgs a = a_in;
  const int g = a.num_q_heads / a.num_kv_heads;
  if (!va_mfma_supported(dtype, a.head_dim, g))
    return va_fail(VA_ERR_ARG, "matrix-core path does not support this dtype/head_dim/group size");
  if (q_tile * g > 16) return va_fail(VA_ERR_ARG, "plan tile of %d rows x %d heads exceeds 16 MFMA rows", q_tile, g);
  if (a.rope.rotary_dim % 16) return va_fail(VA_ERR_ARG, "matrix-core path needs rotary_dim to be a multiple of 16");
  if (a.q_row_stride % 8 || a.pool_row_stride % 8)
    return va_fail(VA_ERR_ARG, "matrix-core path needs 16-byte aligned rows");
  if (n_wide > 0) {
    const int rc = launch_mfma_wide(a, dtype, n_wide, stream);
    if (rc) return rc;
  }
  a.items += (long long)n_wide * VA_ITEM_WORDS;
  const int n_narrow = n_items - n_wide;
#if VA_NARROW_REGISTER_PATH  // the older register-staged kernel, kept for comparison builds
  return dtype == VA_BF16 ? launch_mfma_typed<BF16>(a, n_narrow, stream) : launch_mfma_typed<F16>(a, n_narrow, stream);
#else
  return launch_mfma_stream(a, dtype, n_narrow, stream);
#endif
}

}  // namespace va
