// Streaming matrix-core view attention: query tiles of up to 16 MFMA rows (decode and short
// prefill tiles), K/V streamed from the pool straight into LDS.
//
// The kernel is bound by HBM, so it is built around keeping pool reads in flight:
//   * K/V tiles (16 tokens) go global -> LDS with global_load_lds_dwordx4: no registers hold
//     data in flight, so a workgroup needs few of them and three or four workgroups share a CU, which
//     covers one workgroup's set-up and write-out with the others' streaming;
//   * every wave-level load covers whole, contiguous head rows (64 lanes x 16 B);
//   * each workgroup keeps a ring of tile buffers: a buffer is refilled as soon as its tile has
//     been consumed, so all but the tile being computed are in flight;
//   * the first tiles of a link are requested before its query tile is rotated (a chain of
//     dependent loads).
// One workgroup = 4 waves per (work item, kv head).  All four waves compute the (cheap) scores
// of a tile, S^T[16 tokens, 16 rows] = K . Q^T with v_mfma_f32_16x16x32 (K from LDS as the A
// operand, the rotated query tile pinned in registers as B operands), and the same online
// softmax; for O^T += V^T . P^T each wave owns a slice of the head dimension
// (v_mfma_f32_16x16x16, V rows read from LDS and transposed in registers with v_perm_b32, P
// already laid out as the B operand), so the waves never have to be merged and results leave
// straight from registers.
//
// LDS rows are not padded (the loads write 1 KB runs); bank conflicts are avoided by storing
// 16-byte piece c of tile row r at position c ^ swz(r), which costs nothing: the lane that
// fills position p simply fetches piece p ^ swz(r) from the pool.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "va_internal.h"
#include "va_launch.h"
#include "va_mfma_common.h"

namespace va {

constexpr int kStreamThreads = 256;
constexpr int kStreamWaves = 4;
constexpr int kStreamTok = 16;  // tokens per tile

#ifndef VA_STREAM_BUFFERS_256
#define VA_STREAM_BUFFERS_256 3
#endif
#ifndef VA_STREAM_BLOCKS_256
#define VA_STREAM_BLOCKS_256 3
#endif

template <int kD>
struct StreamShape {
  static constexpr int kChunks = kD / 8;                     // 16-byte pieces of a head row
  static constexpr int kSteps = kD / 32;                     // contraction steps of K.Q^T
  static constexpr int kRowsPerLoad = kWave / kChunks;       // tile rows one wave-level load covers
  static constexpr int kLoadsPerKind = kStreamTok / kRowsPerLoad;  // loads per K (or V) tile
  static constexpr int kLoadsPerWave = 2 * kLoadsPerKind / kStreamWaves;
  static constexpr int kTileUnits = kStreamTok * kChunks;    // 16-byte units of a K (or V) tile
  static constexpr int kBuffers = kD == 256 ? VA_STREAM_BUFFERS_256 : 4;         // ring depth: 48 KB at D=256, 32 KB, 16 KB
  static constexpr int kMinBlocks = kD == 256 ? VA_STREAM_BLOCKS_256 : 4;       // workgroups per CU (registers and LDS allow)
  static constexpr int kPvWaves = kD >= 128 ? 4 : 2;         // waves that own a slice of the head dim
  static constexpr int kDimsPerWave = kD / kPvWaves;
  static constexpr int kRun = kDimsPerWave / 16;             // contiguous dims a lane reads per V token
  static constexpr int kLdsBytes = kBuffers * 2 * kTileUnits * 16;
  static_assert(kLoadsPerWave >= 1 && kRun >= 2 && kRun <= 4, "unsupported head_dim");
};

// position swizzle of tile row r (see the header comment)
template <int kD>
__device__ __forceinline__ int swz(int r) {
  if constexpr (kD >= 128) return (r ^ ((r & 4) << 1)) & 15;
  return (r >> 1) & 7;
}


// max over the four lanes l, l ^ 16, l ^ 32, l ^ 48 (the contraction groups of an MFMA row) with the two
// row-swapping instructions of gfx950, no trip through the LDS crossbar: with both operands x,
// v_permlane16_swap leaves (rows 0 0 2 2, rows 1 1 3 3) of x and v_permlane32_swap (low low, high high).
__device__ __forceinline__ float max_over_contraction_groups(float x) {
  const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

template <typename E, int kD>
__global__ __launch_bounds__(kStreamThreads, StreamShape<kD>::kMinBlocks) void attn_stream_kernel(AttnArgs a) {
  using S = typename E::storage;
  using Sh = StreamShape<kD>;
  constexpr int kChunks = Sh::kChunks, kSteps = Sh::kSteps, kTileUnits = Sh::kTileUnits, kBuffers = Sh::kBuffers;
  constexpr int kRun = Sh::kRun;

  extern __shared__ va_u32x4 ring[];  // buffer b: K tile at ring + 2b * kTileUnits, V tile kTileUnits further

  const ItemHead where = item_and_head(blockIdx.x, a.num_kv_heads);
  // The whole item (its first link travels in it) in ONE round of scalar loads: fetched word by word
  // where each was first needed, the item cost three dependent trips to memory before the first tile
  // could be requested.
  typedef int va_i32x4 __attribute__((ext_vector_type(4)));
  int item[VA_ITEM_WORDS];
  {
    const __attribute__((address_space(4))) va_i32x4* words =
        (const __attribute__((address_space(4))) va_i32x4*)(a.items + (long long)where.item * VA_ITEM_WORDS);
#pragma unroll
    for (int w = 0; w < VA_ITEM_WORDS / 4; ++w) {
      const va_i32x4 x = words[w];
      item[4 * w + 0] = x[0];
      item[4 * w + 1] = x[1];
      item[4 * w + 2] = x[2];
      item[4 * w + 3] = x[3];
    }
  }
  const int hk = where.head;
  const int G = a.num_q_heads / a.num_kv_heads;
  const int n_q = item[VA_I_N_Q];
  if (n_q == 0) return;  // padding item: keeps the launch order aligned with the die round-robin
  const int part_base = item[VA_I_PART_BASE];
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int lane = tid % kWave;
  const int j = lane % 16;   // MFMA row of this lane: tile row j / G, head j % G; also the token it fetches K for
  const int kg = lane / 16;  // contraction group
  const int row_iq = j / G;
  const bool pv_wave = wave < Sh::kPvWaves;
  const S* kp = (const S*)a.k_pool + (long long)hk * kD;
  const S* vp = (const S*)a.v_pool + (long long)hk * kD;
  const int P = a.page_size;
  const bool pow2_pages = (P & (P - 1)) == 0;
  const int p_shift = __builtin_ctz(P);  // t / P and t % P as shift and mask (power-of-two pages)

  // This lane's part of wave-level load u of a tile: tile row, and byte offset of the piece it
  // fetches within the head row (the piece that belongs at the lane's LDS position).
  int ld_row[Sh::kLoadsPerWave], ld_byte[Sh::kLoadsPerWave];
#pragma unroll
  for (int u = 0; u < Sh::kLoadsPerWave; ++u) {
    const int q = (wave * Sh::kLoadsPerWave + u) % Sh::kLoadsPerKind;
    ld_row[u] = q * Sh::kRowsPerLoad + lane / kChunks;
    ld_byte[u] = 16 * ((lane % kChunks) ^ swz<kD>(ld_row[u]));
  }
  // LDS byte offsets (within a tile) of what this lane reads.  The swizzle only touches the low
  // four bits of a position, so contraction steps s and s + 4 are 256 bytes apart.
  constexpr int kKBases = kSteps < 4 ? kSteps : 4;
  int k_byte[kKBases], v_byte[4];
#pragma unroll
  for (int s = 0; s < kKBases; ++s) k_byte[s] = 16 * (j * kChunks + ((4 * s + kg) ^ swz<kD>(j)));
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int row = 4 * kg + r;
    const int dim = wave * Sh::kDimsPerWave + kRun * j;  // first dim of the lane's run, within the head
    v_byte[r] = 16 * (row * kChunks + ((dim / 8) ^ swz<kD>(row))) + 2 * (dim % 8);
  }
  const char* lds = (const char*)ring;
  constexpr int kBufferBytes = 2 * kTileUnits * 16;
  const int row_bytes = (int)a.pool_row_stride * (int)sizeof(S);

  float m_run = kNegBig, l_run = 0.f;
  va_f32x4 o[kRun];
#pragma unroll
  for (int t = 0; t < kRun; ++t) o[t] = va_f32x4{0.f, 0.f, 0.f, 0.f};

  for (int li = 0; li < item[VA_I_N_LINKS]; ++li) {
    // the first link travels with the item
    int link[VA_LINK_WORDS];
    if (li == 0) {
#pragma unroll
      for (int w = 0; w < VA_LINK_WORDS; ++w) link[w] = item[VA_I_LINK0 + w];
    } else {
      const __attribute__((address_space(4))) va_i32x4* words = (const __attribute__((address_space(4))) va_i32x4*)(
          a.links + (long long)(item[VA_I_LINK_BEGIN] + li) * VA_LINK_WORDS);
#pragma unroll
      for (int w = 0; w < VA_LINK_WORDS / 4; ++w) {
        const va_i32x4 x = words[w];
        link[4 * w + 0] = x[0];
        link[4 * w + 1] = x[1];
        link[4 * w + 2] = x[2];
        link[4 * w + 3] = x[3];
      }
    }
    const int lflags = link[VA_L_FLAGS];
    const int qref = link[VA_L_QREF];
    const int kv_begin = link[VA_L_KV_BEGIN];
    const int tok_begin = link[VA_L_TOK_BEGIN];
    const int tok_end = link[VA_L_TOK_END];
    const int causal_base = link[VA_L_CAUSAL_BASE];
    const bool slots = lflags & VA_LINK_SLOTS;
    // no other query tile reads these rows: they are requested as lines to evict first
    const bool read_once = lflags & VA_LINK_ONCE;
    // a 16-token tile lies inside one page: one wave-uniform page read per tile
    const bool uniform_pages = !slots && pow2_pages && P >= 16 && (tok_begin % 16 == 0);

    const int t_stop = min(tok_end, causal_base + n_q);        // tokens any row of the tile sees
    const int t_row = min(tok_end, causal_base + row_iq + 1);  // tokens this lane's row sees
    const int t_last = t_stop - 1;
    const int n_tiles = t_stop > tok_begin ? (t_stop - tok_begin + kStreamTok - 1) / kStreamTok : 0;

    // Request tile i (tokens tok_begin + 16 i ..) into ring buffer i % kBuffers.  Rows past the
    // visible range re-read the last visible token (their scores are masked).
    // page of tile i (uniform page tables).  Read through the constant address space: the table is
    // read-only for the kernel, and this keeps the lookup a scalar load (a vector load would have
    // to be waited for together with every tile load in flight).
    auto page_of = [&](int i) __attribute__((always_inline)) {
      return ((const __attribute__((address_space(4))) int32_t*)a.kv_indices)[kv_begin + ((tok_begin + i * kStreamTok) >> p_shift)];
    };
    auto issue = [&](int i, auto uniform_tag, auto once_tag, int page) __attribute__((always_inline)) {
      constexpr bool kUniform = decltype(uniform_tag)::value;
      constexpr bool kOnce = decltype(once_tag)::value;
      const int t0 = tok_begin + i * kStreamTok;
      va_u32x4* buf = ring + (i % kBuffers) * 2 * kTileUnits;
      long long base_byte = 0;  // wave-uniform: pool byte offset of the tile's first token
      if constexpr (kUniform) {
        base_byte = (((long long)page << p_shift) + (t0 & (P - 1))) * row_bytes;
      }
      const int last_row = t_last - t0;  // rows beyond it are clamped
#pragma unroll
      for (int u = 0; u < Sh::kLoadsPerWave; ++u) {
        const int q = wave * Sh::kLoadsPerWave + u;  // wave-uniform
        const bool is_v = q >= Sh::kLoadsPerKind;
        const int first_row = (is_v ? q - Sh::kLoadsPerKind : q) * Sh::kRowsPerLoad;
        const int r = min(ld_row[u], last_row);
        const char* src;
        if constexpr (kUniform) {
          src = (const char*)(is_v ? vp : kp) + base_byte + (uint32_t)(r * row_bytes + ld_byte[u]);
        } else {
          src = (const char*)(is_v ? vp : kp) + kv_slot(a.kv_indices, kv_begin, t0 + r, P, slots) * row_bytes +
                ld_byte[u];
        }
        const va_u32x4* dst = buf + (is_v ? kTileUnits : 0) + first_row * kChunks;  // + lane, implied by the load
        if constexpr (kOnce) {
          load_to_lds_once(src, __builtin_amdgcn_readfirstlane(lds_address(dst)));
        } else {
          load_to_lds(src, __builtin_amdgcn_readfirstlane(lds_address(dst)));
        }
      }
    };

    // ---- set-up: first tiles on their way, then the query tile ----
    __syncthreads();  // every wave is done with the previous link's buffers
    auto first_tiles = [&](auto uniform_tag, auto once_tag) __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < kBuffers - 1; ++i)
        if (i < n_tiles) issue(i, uniform_tag, once_tag, decltype(uniform_tag)::value ? page_of(i) : 0);
    };
    // (one instance of the requests and of the tile loop per page-table kind and per cache policy,
    // so that none carries the others' branches)
    auto per_kind = [&](auto&& body) __attribute__((always_inline)) {
      if (uniform_pages) {
        if (read_once) {
          body(std::true_type{}, std::true_type{});
        } else {
          body(std::true_type{}, std::false_type{});
        }
      } else {
        if (read_once) {
          body(std::false_type{}, std::true_type{});
        } else {
          body(std::false_type{}, std::false_type{});
        }
      }
    };
    per_kind(first_tiles);

    // rotate the query tile into the last buffer (not yet in use), swizzled like a K tile
    va_u32x4* q_stage = ring + (kBuffers - 1) * 2 * kTileUnits;
    for (int idx = tid; idx < 16 * (kChunks / 2); idx += kStreamThreads) {  // two pieces per step
      const int jr = idx / (kChunks / 2), x = idx - jr * (kChunks / 2);
      const int iq = jr / G, g = jr - iq * G;
      int c0 = 2 * x, c1 = 2 * x + 1;
      uint4 p0 = make_uint4(0, 0, 0, 0), p1 = p0;
      if (iq < n_q) {
        // indirect links find sub-row and query row side by side in the plan; direct ones ask sub_worker
        const bool indirect = lflags & VA_LINK_INDIRECT;
        const int subrow = indirect ? a.qrefs[qref + iq] : qref + iq;
        const long long src_row = indirect ? (long long)a.qref_rows[qref + iq] : a.sub_worker[subrow];
        const S* qh = (const S*)a.q + src_row * a.q_row_stride + (long long)(hk * G + g) * kD;
        const Pos3 p = load_pos(a.sub_loc, a.sub_loc_axis_stride, subrow);
        if (a.rope.mode == VA_ROPE_TABLE && x < a.rope.rotary_dim / 16) {
          // the table entries of the unit in four 16-byte loads
          TableQueryUnit<E> unit;
          unit.load(a.rope, qh, x, p);
          unit.finish(a.rope, p, p0, p1);
          c0 = x;
          c1 = x + a.rope.rotary_dim / 16;
        } else {
          rotated_query_unit<E>(a.rope, qh, x, p, c0, c1, p0, p1);
        }
      }
      q_stage[jr * kChunks + (c0 ^ swz<kD>(jr))] = va_u32x4{p0.x, p0.y, p0.z, p0.w};
      q_stage[jr * kChunks + (c1 ^ swz<kD>(jr))] = va_u32x4{p1.x, p1.y, p1.z, p1.w};
    }
    ring_barrier<kAnyInFlight>();
    va_u32x4 qf[kSteps];  // B operands: row j, dims [32s + 8kg, +8)
#pragma unroll
    for (int s = 0; s < kSteps; ++s) qf[s] = q_stage[j * kChunks + ((4 * s + kg) ^ swz<kD>(j))];
    ring_barrier<kAnyInFlight>();  // the staging buffer may be refilled now

    // ---- the tile loop ----
    auto stream = [&](auto uniform_tag, auto once_tag) __attribute__((always_inline)) {
    if (kBuffers - 1 < n_tiles) issue(kBuffers - 1, uniform_tag, once_tag, decltype(uniform_tag)::value ? page_of(kBuffers - 1) : 0);
    for (int i = 0; i < n_tiles; ++i) {
      // This wave's loads of tile i have landed once at most the loads of the tiles requested
      // after it are outstanding; the barrier then covers the other waves' loads.
      if (i + kBuffers - 1 < n_tiles) {
        ring_barrier<(kBuffers - 1) * Sh::kLoadsPerWave>();
      } else {
        ring_barrier<0>();
      }

      const bool refill = i + kBuffers < n_tiles;
      int next_page = 0;
      const int t0 = tok_begin + i * kStreamTok;
      const char* kt = lds + (i % kBuffers) * kBufferBytes;
      const char* vt = kt + kTileUnits * 16;
      if (pv_wave) {
        // scores: S^T = K . Q^T; lane (j, kg) supplies dims [32s + 8kg, +8) of token t0 + j
        // every K fragment is requested before the first product (left to itself the compiler reads
        // them one by one into one set of registers: an LDS latency per product)
        va_u32x4 kfr[kSteps];
#pragma unroll
        for (int s = 0; s < kSteps; ++s) kfr[s] = *(const va_u32x4*)(kt + k_byte[s % 4] + 256 * (s / 4));
        __builtin_amdgcn_sched_barrier(0);
        va_f32x4 sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < kSteps; ++s) sc = Mma<E>::run(kfr[s], qf[s], sc);

        // The page of the tile requested at the end of this iteration is looked up here: the softmax and
        // the products below cover the latency -- and not before the score products, because a scalar
        // load in flight shares its counter with the LDS reads, which then could only be waited for
        // all at once (every K fragment read a full LDS latency of its own).
        if (decltype(uniform_tag)::value && refill) next_page = page_of(i + kBuffers);
        // online softmax: this lane holds tokens t0 + 4kg + r of row j
        float tile_max = -INFINITY;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float v = (t0 + 4 * kg + r) < t_row ? sc[r] * a.scale_log2 : -INFINITY;
          sc[r] = v;
          tile_max = fmaxf(tile_max, v);
        }
        tile_max = max_over_contraction_groups(tile_max);
        const float m_new = fmaxf(m_run, tile_max);
        // (the bare instruction: results below 2^-126 become 0 instead of denormal)
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        m_run = m_new;
        float pr[4], psum = 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          pr[r] = __builtin_amdgcn_exp2f(sc[r] - m_new);
          psum += pr[r];
        }
        l_run = l_run * alpha + psum;
#pragma unroll
        for (int t = 0; t < kRun; ++t) o[t] *= alpha;
        const va_u32x2 pf = {Mma<E>::pack(pr[0], pr[1]), Mma<E>::pack(pr[2], pr[3])};

        // O^T += V^T . P^T on this wave's slice: the lane reads kRun dims of its 4 tokens and
        // dim tile T takes element T of each run
        uint32_t vraw[4][kRun / 2];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if constexpr (kRun == 4) {
            const uint2 x = *(const uint2*)(vt + v_byte[r]);
            vraw[r][0] = x.x;
            vraw[r][1] = x.y;
          } else {
            vraw[r][0] = *(const uint32_t*)(vt + v_byte[r]);
          }
        }
#pragma unroll
        for (int t = 0; t < kRun; ++t) {
          const int w = t / 2;
          const uint32_t sel = (t & 1) ? 0x07060302u : 0x05040100u;
          const va_u32x2 vf = {__builtin_amdgcn_perm(vraw[1][w], vraw[0][w], sel),
                               __builtin_amdgcn_perm(vraw[3][w], vraw[2][w], sel)};
          o[t] = Mma<E>::run16(vf, pf, o[t]);
        }
      }
      else if (decltype(uniform_tag)::value && refill) {
        next_page = page_of(i + kBuffers);  // (waves that only load, at head_dim 64)
      }
      // refill this tile's buffer once every wave has consumed it
      if (refill) {
        ring_barrier<kAnyInFlight>();
        issue(i + kBuffers, uniform_tag, once_tag, next_page);
      }
    }
    };
    per_kind(stream);
  }

  // row sums live spread over the four contraction groups
  l_run += __shfl_xor(l_run, 16, kWave);
  l_run += __shfl_xor(l_run, 32, kWave);

  // ---- emit from registers: o[T][r] is dim 4*kRun*kg + kRun*r + T of the wave's slice, row j ----
  if (pv_wave && row_iq < n_q) {
    const int g = j - row_iq * G;
    const int hq = hk * G + g;
    const int d0 = wave * Sh::kDimsPerWave + 4 * kRun * kg;
    if (part_base < 0) {
      const int qref0 = item[VA_I_LINK0 + VA_L_QREF];
      const long long out_row = (item[VA_I_LINK0 + VA_L_FLAGS] & VA_LINK_INDIRECT) ? (long long)a.qref_rows[qref0 + row_iq]
                                                                                   : a.sub_worker[qref0 + row_iq];
      S* orow = (S*)a.out + (out_row * a.num_q_heads + hq) * (long long)kD + d0;
      const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
      uint32_t w[2 * kRun];
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int t = 0; t < kRun; t += 2) w[(kRun * r + t) / 2] = Mma<E>::pack(o[t][r] * inv, o[t + 1][r] * inv);
#pragma unroll
      for (int x = 0; x < 2 * kRun; x += 4) *(uint4*)(orow + 2 * x) = make_uint4(w[x], w[x + 1], w[x + 2], w[x + 3]);
      if (wave == 0 && kg == 0 && a.lse) {
        const float lse2 = l_run > 0.f ? m_run + log2f(l_run) : -INFINITY;
        a.lse[out_row * a.num_q_heads + hq] = a.lse_base2 ? lse2 : lse2 * kLn2;
      }
    } else {
      const long long slot = (long long)(part_base + row_iq) * a.num_q_heads + hq;
      float* prow = a.part_acc + slot * kD + d0;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if constexpr (kRun == 4) {
          *(float4*)(prow + 4 * r) = make_float4(o[0][r], o[1][r], o[2][r], o[3][r]);
        } else {
          *(float2*)(prow + 2 * r) = make_float2(o[0][r], o[1][r]);
        }
      }
      if (wave == 0 && kg == 0) {
        a.part_ml[slot * 2 + 0] = m_run;
        a.part_ml[slot * 2 + 1] = l_run;
      }
    }
  }
}

template <typename E, int kD>
static int launch_stream_one(const AttnArgs& a, int n_items, hipStream_t stream) {
  const dim3 grid((unsigned)n_items * (unsigned)a.num_kv_heads), block(kStreamThreads);
  if constexpr (StreamShape<kD>::kLdsBytes > 64 * 1024) {  // (deeper rings than the default need the limit raised)
    static bool configured = false;  // raising the limit is idempotent; a race only repeats the call
    if (!configured) {
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_stream_kernel<E, kD>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, StreamShape<kD>::kLdsBytes);
      if (e != hipSuccess) return va_fail(VA_ERR_HIP, "raising the LDS limit: %s", hipGetErrorString(e));
      configured = true;
    }
  }
  hipLaunchKernelGGL((attn_stream_kernel<E, kD>), grid, block, StreamShape<kD>::kLdsBytes, stream, a);
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? VA_OK : va_fail(VA_ERR_HIP, "streaming attention launch: %s", hipGetErrorString(e));
}

template <typename E>
static int launch_stream_typed(const AttnArgs& a, int n_items, hipStream_t stream) {
  switch (a.head_dim) {
    case 64:
      return launch_stream_one<E, 64>(a, n_items, stream);
    case 128:
      return launch_stream_one<E, 128>(a, n_items, stream);
    case 256:
      return launch_stream_one<E, 256>(a, n_items, stream);
    default:
      return va_fail(VA_ERR_ARG, "matrix-core path supports head_dim 64, 128, 256");
  }
}

int launch_mfma_stream(const AttnArgs& a, int dtype, int n_items, hipStream_t stream) {
  if (n_items == 0) return VA_OK;
  return dtype == VA_BF16 ? launch_stream_typed<BF16>(a, n_items, stream)
                          : launch_stream_typed<F16>(a, n_items, stream);
}

}  // namespace va
