// Wide matrix-core view attention: query tiles of up to 128 MFMA rows.
//
// Used where many query rows meet the same keys: view-conditioned prefill
// (128/G new tokens x G heads per workgroup) and decode over a block shared by
// more than 16/G requests.  One workgroup of four waves per (work item, kv head);
// wave w owns MFMA rows [32w, 32w+32) (row R = tile row R / G, head R % G) and
// all four waves walk the same 32-token K/V tiles, which are staged once per
// workgroup in LDS (double buffered: the global loads of tile i+1 are in flight
// while tile i is computed, one barrier per tile).
//
//   S^T[32 tokens, 32 rows] = K . Q^T     16 x v_mfma_f32_32x32x16 (D = 256), K from LDS as the A operand,
//                                         the wave's rotated queries pinned in registers as B operands
//   online softmax per row (row = lane % 32; the other half-wave holds the other 16 tokens)
//   O^T[D, 32 rows] += V^T . P^T          2 token steps x D/32 dim tiles; P is already laid out as the B operand
//                                         (the token order of the contraction is chosen to match the S^T
//                                         accumulator), V rows are read from LDS as 8 tokens x D/32 dims per
//                                         lane and transposed in registers with v_perm_b32
//
// The query tile of the current link is rotated by all 256 threads into the (not yet
// used) tile buffers, then each wave pulls its 32 rows into registers.
#include <hip/hip_runtime.h>

#include "va_internal.h"
#include "va_launch.h"
#include "va_mfma_common.h"

namespace va {

constexpr int kWideThreads = 256;
constexpr int kWideRows = 128;   // MFMA rows per workgroup
constexpr int kWideTokens = 32;  // tokens per K/V tile

template <int kD>
constexpr int wide_lds_bytes() {
  // two buffers x (K tile + V tile) x 32 tokens x padded row; the same bytes hold the rotated
  // query tile (128 rows) before streaming starts
  return 2 * 2 * kWideTokens * (kD / 8 + 1) * 16;
}

template <typename E, int kD>
__global__ __launch_bounds__(kWideThreads, 1) void attn_mfma_wide_kernel(AttnArgs a) {
  using S = typename E::storage;
  constexpr int kSteps = kD / 16;     // contraction steps of K.Q^T (32x32x16)
  constexpr int kDimTiles = kD / 32;  // 32-dim tiles of the output = dims a lane owns per V token
  constexpr int kChunks = kD / 8;     // 16-byte pieces of a head row
  constexpr int kRow = kChunks + 1;   // padded LDS row, in 16-byte units
  constexpr int kVDw = kD / 64;       // dwords of a V token a lane reads (D/32 dims)

  extern __shared__ va_u32x4 smem[];
  // buffer b: K tile at smem + b*2*32*kRow, V tile 32*kRow further
  auto k_tile = [&](int b) __attribute__((always_inline)) { return smem + (b * 2) * kWideTokens * kRow; };
  auto v_tile = [&](int b) __attribute__((always_inline)) { return smem + (b * 2 + 1) * kWideTokens * kRow; };

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
  const int j = lane % 32;  // row within the wave's 32 rows / token within a tile / dim group
  const int h = lane / 32;  // half-wave: contraction group
  const int my_row = 32 * wave + j;
  const int row_iq = my_row / G;
  const int wave_iq_last = min(n_q - 1, (32 * wave + 31) / G);  // last tile row this wave serves
  const S* kp = (const S*)a.k_pool + (long long)hk * kD;
  const S* vp = (const S*)a.v_pool + (long long)hk * kD;
  const int P = a.page_size;

  float m_run = kNegBig, l_run = 0.f;
  va_f32x16 o[kDimTiles];
#pragma unroll
  for (int t = 0; t < kDimTiles; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[t][r] = 0.f;

  for (int li = 0; li < item[VA_I_N_LINKS]; ++li) {
    const int32_t* link = a.links + (long long)(item[VA_I_LINK_BEGIN] + li) * VA_LINK_WORDS;
    const int lflags = link[VA_L_FLAGS];
    const int qref = link[VA_L_QREF];
    const int kv_begin = link[VA_L_KV_BEGIN];
    const int tok_begin = link[VA_L_TOK_BEGIN];
    const int tok_end = link[VA_L_TOK_END];
    const int causal_base = link[VA_L_CAUSAL_BASE];
    const bool slots = lflags & VA_LINK_SLOTS;

    // ---- rotate the whole query tile for this link into LDS (aliases the tile buffers) ----
    __syncthreads();
    for (int idx = tid; idx < kWideRows * kChunks; idx += kWideThreads) {
      const int R = idx / kChunks, c = idx - R * kChunks;
      const int iq = R / G, g = R - iq * G;
      va_u32x4 packed = {0, 0, 0, 0};
      if (iq < n_q) {
        const int subrow = (lflags & VA_LINK_INDIRECT) ? a.qrefs[qref + iq] : qref + iq;
        const long long src_row = a.sub_worker[subrow];
        const S* qh = (const S*)a.q + src_row * a.q_row_stride + (long long)(hk * G + g) * kD;
        const Pos3 p = load_pos(a.sub_loc, a.sub_loc_axis_stride, subrow);
        const uint4 piece = rotated_query_piece<E>(a.rope, qh, c * 8, p);
        packed = va_u32x4{piece.x, piece.y, piece.z, piece.w};
      }
      smem[R * kRow + c] = packed;
    }
    __syncthreads();
    va_u32x4 qf[kSteps];  // B operands: row my_row, dims [16s + 8h, +8)
#pragma unroll
    for (int s = 0; s < kSteps; ++s) qf[s] = smem[my_row * kRow + 2 * s + h];
    __syncthreads();

    const int t_stop = min(tok_end, causal_base + n_q);             // tokens any row of the tile sees
    const int t_row = min(tok_end, causal_base + row_iq + 1);       // tokens this lane's row sees
    // tokens any row of this wave sees (none if the wave's rows lie beyond the tile)
    const int t_wave = (32 * wave) / G < n_q ? min(tok_end, causal_base + wave_iq_last + 1) : -0x7fffffff;
    const int t_last = t_stop - 1;
    // tokens EVERY real row of this wave sees: tiles ending below it need no masking
    const int t_wave_min = min(tok_end, causal_base + (32 * wave) / G + 1);

    // global -> registers -> LDS.  Thread (ld_tok, ld_c) moves piece ld_c of tokens ld_tok + kTokStep*i of
    // both the K and the V tile: rows are contiguous over threads, K and V share the row lookup.
    constexpr int kTokStep = kWideThreads / kChunks;  // tokens per round of loads
    constexpr int kRounds = kWideTokens / kTokStep;
    const int ld_tok = tid / kChunks, ld_c = tid - ld_tok * kChunks;
    // a 16-token half tile lies inside one page only if the link starts on a 16-token boundary
    const bool uniform_pages = !slots && (P % 16 == 0) && (tok_begin % 16 == 0);
    va_u32x4 stage_k[kRounds], stage_v[kRounds];
    auto fetch = [&](int t0) __attribute__((always_inline)) {
      if (uniform_pages) {
        // a 16-token half tile lies in one page: two wave-uniform page-table reads per tile
        long long half_row[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int t = min(t0 + 16 * u, t_last);
          const int page = __builtin_amdgcn_readfirstlane(a.kv_indices[kv_begin + t / P]);
          half_row[u] = (long long)page * P + ((t % P) & ~15);
        }
#pragma unroll
        for (int i = 0; i < kRounds; ++i) {
          const int tok = ld_tok + kTokStep * i;
          const int t = min(t0 + tok, t_last);
          const long long off = ((tok < 16 ? half_row[0] : half_row[1]) + (t & 15)) * a.pool_row_stride + 8 * ld_c;
          stage_k[i] = *(const va_u32x4*)(kp + off);
          stage_v[i] = *(const va_u32x4*)(vp + off);
        }
      } else {
        long long off[kRounds];
#pragma unroll
        for (int i = 0; i < kRounds; ++i) {
          const int t = min(t0 + ld_tok + kTokStep * i, t_last);
          off[i] = kv_slot(a.kv_indices, kv_begin, t, P, slots) * a.pool_row_stride + 8 * ld_c;
        }
#pragma unroll
        for (int i = 0; i < kRounds; ++i) {
          stage_k[i] = *(const va_u32x4*)(kp + off[i]);
          stage_v[i] = *(const va_u32x4*)(vp + off[i]);
        }
      }
    };
    auto commit = [&](int b) __attribute__((always_inline)) {
      va_u32x4* kt = k_tile(b);
      va_u32x4* vt = v_tile(b);
#pragma unroll
      for (int i = 0; i < kRounds; ++i) {
        const int at = (ld_tok + kTokStep * i) * kRow + ld_c;
        kt[at] = stage_k[i];
        vt[at] = stage_v[i];
      }
    };

    int t0 = tok_begin;
    int buf = 0;
    if (t0 < t_stop) {
      fetch(t0);
      commit(0);
      __syncthreads();
    }
    for (; t0 < t_stop; t0 += kWideTokens) {
      const bool more = t0 + kWideTokens < t_stop;
#if VA_WIDE_EXPERIMENT != 1
      if (more) fetch(t0 + kWideTokens);
#endif

#if VA_WIDE_EXPERIMENT == 2
      if (false) {
#else
      if (t0 < t_wave) {
#endif
        const va_u32x4* kt = k_tile(buf);
        const va_u32x4* vt = v_tile(buf);
        // ---- scores.  K fragments are read from LDS in groups of four, two groups ahead of the
        // MFMAs that consume them, so the matrix pipe never waits on an LDS round trip. ----
        constexpr int kGroups = kSteps / 4;
        va_u32x4 kfr[2][4];
        auto read_group = [&](int g, va_u32x4 (&dst)[4]) __attribute__((always_inline)) {
#pragma unroll
          for (int q = 0; q < 4; ++q) dst[q] = kt[j * kRow + 2 * (4 * g + q) + h];
        };
        read_group(0, kfr[0]);
        if constexpr (kGroups > 1) read_group(1, kfr[1]);
        va_f32x16 sc;
#pragma unroll
        for (int r = 0; r < 16; ++r) sc[r] = 0.f;
        __builtin_amdgcn_sched_barrier(0);  // keep the reads ahead of the MFMAs (the scheduler would sink them)
#pragma unroll
        for (int g = 0; g < kGroups; ++g) {
#pragma unroll
          for (int q = 0; q < 4; ++q) sc = Mma<E>::run32(kfr[g & 1][q], qf[4 * g + q], sc);
          if (g + 2 < kGroups) read_group(g + 2, kfr[g & 1]);
          __builtin_amdgcn_sched_barrier(0);
        }

        // ---- online softmax: reg r holds token t0 + (r/4)*8 + 4h + r%4 of row my_row.  Interior
        // tiles (every row of the wave sees all 32 tokens) skip the masking; the scale is folded
        // into the exponent: p = 2^(s*c - m). ----
        float tile_max = -INFINITY;
        if (t0 + kWideTokens <= t_wave_min) {
#pragma unroll
          for (int r = 0; r < 16; ++r) tile_max = fmaxf(tile_max, sc[r]);
        } else {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int t = t0 + (r / 4) * 8 + 4 * h + (r % 4);
            sc[r] = t < t_row ? sc[r] : -INFINITY;
            tile_max = fmaxf(tile_max, sc[r]);
          }
        }
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, kWave));
        const float m_new = fmaxf(m_run, tile_max * a.scale_log2);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        m_run = m_new;
        float psum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          sc[r] = __builtin_amdgcn_exp2f(fmaf(sc[r], a.scale_log2, -m_new));
          psum += sc[r];
        }
        l_run = l_run * alpha + psum;
        if (__any(alpha != 1.f)) {
#pragma unroll
          for (int t = 0; t < kDimTiles; ++t) o[t] *= alpha;
        }

        // ---- O^T += V^T . P^T over two 16-token steps ----
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
          const va_u32x4 pf = {Mma<E>::pack(sc[8 * kk + 0], sc[8 * kk + 1]), Mma<E>::pack(sc[8 * kk + 2], sc[8 * kk + 3]),
                               Mma<E>::pack(sc[8 * kk + 4], sc[8 * kk + 5]), Mma<E>::pack(sc[8 * kk + 6], sc[8 * kk + 7])};
          // the lane's 8 tokens of this step, D/32 dims each (dims j*D/32 ..)
          uint32_t vraw[8][kVDw];
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int tok = (2 * kk + e / 4) * 8 + 4 * h + (e % 4);
            if constexpr (kVDw == 4) {
              const va_u32x4 x = vt[tok * kRow + j];
              vraw[e][0] = x[0]; vraw[e][1] = x[1]; vraw[e][2] = x[2]; vraw[e][3] = x[3];
            } else if constexpr (kVDw == 2) {
              const uint2 x = ((const uint2*)(vt + tok * kRow))[j];
              vraw[e][0] = x.x; vraw[e][1] = x.y;
            } else {
              vraw[e][0] = ((const uint32_t*)(vt + tok * kRow))[j];
            }
          }
#pragma unroll
          for (int t = 0; t < kDimTiles; ++t) {
            const int w = t / 2;
            const uint32_t sel = (t & 1) ? 0x07060302u : 0x05040100u;
            const va_u32x4 vf = {__builtin_amdgcn_perm(vraw[1][w], vraw[0][w], sel), __builtin_amdgcn_perm(vraw[3][w], vraw[2][w], sel),
                                 __builtin_amdgcn_perm(vraw[5][w], vraw[4][w], sel), __builtin_amdgcn_perm(vraw[7][w], vraw[6][w], sel)};
            o[t] = Mma<E>::run32(vf, pf, o[t]);
          }
        }
      }

#if VA_WIDE_EXPERIMENT != 1
      if (more) commit(buf ^ 1);
#endif
      __syncthreads();
      buf ^= 1;
    }
  }

  l_run += __shfl_xor(l_run, 32, kWave);

  // ---- emit: accumulator reg r of dim tile T is dim ((r/4)*8 + 4h + r%4) * D/32 + T of row my_row ----
  if (row_iq < n_q) {
    const int g = my_row - row_iq * G;
    const int hq = hk * G + g;
    const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
    if (part_base < 0) {
      const int32_t* link0 = a.links + (long long)item[VA_I_LINK_BEGIN] * VA_LINK_WORDS;
      const int subrow =
          (link0[VA_L_FLAGS] & VA_LINK_INDIRECT) ? a.qrefs[link0[VA_L_QREF] + row_iq] : link0[VA_L_QREF] + row_iq;
      const long long out_row = a.sub_worker[subrow];
      S* orow = (S*)a.out + (out_row * a.num_q_heads + hq) * (long long)kD;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int d0 = ((r / 4) * 8 + 4 * h + (r % 4)) * kDimTiles;
        uint32_t w[kDimTiles / 2];
#pragma unroll
        for (int t = 0; t < kDimTiles / 2; ++t) w[t] = Mma<E>::pack(o[2 * t][r] * inv, o[2 * t + 1][r] * inv);
        if constexpr (kDimTiles == 8) {
          *(uint4*)(orow + d0) = make_uint4(w[0], w[1], w[2], w[3]);
        } else if constexpr (kDimTiles == 4) {
          *(uint2*)(orow + d0) = make_uint2(w[0], w[1]);
        } else {
          *(uint32_t*)(orow + d0) = w[0];
        }
      }
      if (h == 0 && a.lse) {
        const float lse2 = l_run > 0.f ? m_run + log2f(l_run) : -INFINITY;
        a.lse[out_row * a.num_q_heads + hq] = a.lse_base2 ? lse2 : lse2 * kLn2;
      }
    } else {
      const long long slot = (long long)(part_base + row_iq) * a.num_q_heads + hq;
      float* prow = a.part_acc + slot * kD;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int d0 = ((r / 4) * 8 + 4 * h + (r % 4)) * kDimTiles;
#pragma unroll
        for (int t = 0; t < kDimTiles; ++t) prow[d0 + t] = o[t][r];
      }
      if (h == 0) {
        a.part_ml[slot * 2 + 0] = m_run;
        a.part_ml[slot * 2 + 1] = l_run;
      }
    }
  }
}

template <typename E, int kD>
static int launch_wide_one(const AttnArgs& a, int n_items, hipStream_t stream) {
  constexpr int bytes = wide_lds_bytes<kD>();
  static bool configured = false;  // raising the limit is idempotent; a race only repeats the call
  if (!configured) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_mfma_wide_kernel<E, kD>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) return va_fail(VA_ERR_HIP, "raising the LDS limit: %s", hipGetErrorString(e));
    configured = true;
  }
  const dim3 grid((unsigned)n_items * (unsigned)a.num_kv_heads), block(kWideThreads);
  hipLaunchKernelGGL((attn_mfma_wide_kernel<E, kD>), grid, block, bytes, stream, a);
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? VA_OK : va_fail(VA_ERR_HIP, "wide attention launch: %s", hipGetErrorString(e));
}

template <typename E>
static int launch_wide_typed(const AttnArgs& a, int n_items, hipStream_t stream) {
  switch (a.head_dim) {
    case 64:
      return launch_wide_one<E, 64>(a, n_items, stream);
    case 128:
      return launch_wide_one<E, 128>(a, n_items, stream);
    case 256:
      return launch_wide_one<E, 256>(a, n_items, stream);
    default:
      return va_fail(VA_ERR_ARG, "matrix-core path supports head_dim 64, 128, 256");
  }
}

int launch_mfma_wide(const AttnArgs& a, int dtype, int n_items, hipStream_t stream) {
  if (n_items == 0) return VA_OK;
  return dtype == VA_BF16 ? launch_wide_typed<BF16>(a, n_items, stream) : launch_wide_typed<F16>(a, n_items, stream);
}

}  // namespace va
