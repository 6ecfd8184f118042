// Wide matrix-core view attention: query tiles of 128 (head_dim 256) or 256 MFMA rows, for
// view-conditioned prefill (rows / G new tokens x G heads per workgroup).
//
// One workgroup of four waves per (slot, kv head), one wave per SIMD; a slot is one work item, or
// several pieces of tiles whose walks add up to the same number of tokens in every slot, run one
// after the other.  Wave w owns one
// (head_dim 256) or two blocks of 32 MFMA rows (row R = tile row R / G, head R % G).  All waves walk
// the same 32-token K/V tiles, which travel pool -> LDS directly (global_load_lds_dwordx4) into a
// ring of four buffers: two tiles are in flight while the scores of a third and the products of a
// fourth are computed, one barrier per tile.
//
//   S^T[32 tokens, 32 rows] = K . Q^T    v_mfma_f32_32x32x16, K from LDS as the A operand; each K
//                                        fragment is read once and used for all row blocks, whose
//                                        rotated queries are pinned in registers as B operands
//   softmax per row against a reference maximum that is raised only when a tile exceeds it by far
//   (row = lane % 32; the other half-wave holds the other 16 tokens)
//   O^T[D, 32 rows] += V^T . P^T         2 token steps x D/32 dim tiles; P is already laid out as
//                                        the B operand; V^T fragments come from transposing LDS
//                                        reads (ds_read_b64_tr_b16), each serving all row blocks
//
// The loop is a hand-ordered software pipeline: the scores of tile i + 1 run on the matrix pipe
// under the exponentials of tile i (each taken of scale * score - reference, formed in fp32 right
// in front of it), the products of tile i under the maxima of tile i + 1.  Interior tiles of a link
// take a branch-free ring step, in a loop of their own.
// V tiles and the staged query tile keep whole rows in LDS, unpadded and swizzled (piece c of row r
// at position c ^ swz(r)); K tiles land in fragment order (8-token x 128-byte blocks, see the load
// pattern in the kernel), so that the K reads of a tile share one address register.  The query tile
// is rotated by all 256 threads, one row block of every wave (128 rows) at a time, into the two
// ring buffers that are not yet in use.
#include <hip/hip_runtime.h>

#include "va_internal.h"
#include "va_launch.h"
#include "va_mfma_common.h"

namespace va {

constexpr int kWideThreads = 256;
constexpr float kWideRaise = 14.f;  // a tile maximum this far above the reference (log2 units) raises it
constexpr int kWideWaves = 4;
constexpr int kWideTokens = 32;  // tokens per K/V tile
#ifndef VA_WIDE_BUFFERS
#define VA_WIDE_BUFFERS 4
#endif
constexpr int kWideBuffers = VA_WIDE_BUFFERS;  // ring depth: kWideBuffers - 2 tiles in flight
constexpr int kWideAhead = kWideBuffers - 2;    // a ring step requests the tile this far ahead

template <int kD>
struct WideShape {
  static constexpr int kChunks = kD / 8;     // 16-byte pieces of a head row
  static constexpr int kSteps = kD / 16;     // contraction steps of K.Q^T (32x32x16)
  static constexpr int kDimTiles = kD / 32;  // 32-dim tiles of the output
  static constexpr int kRowBytes = kChunks * 16;
  static constexpr int kRowsPerLoad = kWave / kChunks;              // tile rows one wave-level load covers
  static constexpr int kLoadsPerKind = kWideTokens / kRowsPerLoad;  // loads per K (or V) tile
  static constexpr int kLoadsPerWave = 2 * kLoadsPerKind / kWideWaves;
  static constexpr int kTileBytes = kWideTokens * kRowBytes;  // a K (or V) tile
  static constexpr int kBufferBytes = 2 * kTileBytes;
  static constexpr int kLdsBytes = kWideBuffers * kBufferBytes;  // 128 KB at D = 256
  // 32-row blocks per wave.  Two blocks halve the LDS bytes read per flop, but the state of a row
  // (D fp32 accumulators + D 16-bit query elements) then fills the register file at D = 256:
  // 64 rows need 256 + 128 of the 512 registers before any operand is staged, and the compiler
  // spills.  D = 256 therefore runs one block per wave.
  static constexpr int kBlocks = kD == 256 ? 1 : 2;
  static constexpr int kWaveRows = 32 * kBlocks;
  static constexpr int kTileRows = kWideWaves * kWaveRows;  // MFMA rows per workgroup
  static_assert(128 * kRowBytes == 2 * kBufferBytes, "one row block of every wave fills two ring buffers");
};

template <int kD>
__device__ __forceinline__ int wide_swz(int r) {
  if constexpr (kD >= 128) return r & 15;
  return (r >> 1) & 7;
}

// Ring buffer of a tile (tile numbers are never negative: the unsigned remainder is one instruction
// for a power-of-two ring, the signed one five).
__device__ __forceinline__ uint32_t ring_slot(int tile) { return (uint32_t)tile % (uint32_t)kWideBuffers; }

// V tiles are read with transposing loads (16 lanes fetch 4 tokens x 16 dims, 32 bytes per token):
// moving token r's pieces by 2 (r % 4) puts the four rows of such a fetch side by side in one
// 128-byte window.
__device__ __forceinline__ int wide_vswz(int r) { return (r & 3) << 1; }

// A transposing LDS read (ds_read_b64_tr_b16).  Within every group of 16 lanes, lane s supplies
// the address of four 16-bit elements E[s][0..3]; lane i receives E[i / 4 + 4 k][i % 4], k = 0..3.
// With lane s pointed at token T + s / 4, dims c + 4 (s % 4) .. + 3, lane i therefore receives
// dim c + i of tokens T .. T + 3: four consecutive contraction elements of one row of V^T.
__device__ __forceinline__ va_u32x2 lds_read_tr16(uint32_t lds_byte_address) {
  typedef short v4s __attribute__((ext_vector_type(4)));
  const v4s r = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (__attribute__((address_space(3))) v4s*)(uintptr_t)lds_byte_address);
  return __builtin_bit_cast(va_u32x2, r);
}

// max over the two half-waves (lanes l and l ^ 32) without touching LDS
__device__ __forceinline__ float half_wave_max(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

template <typename E, int kD>
__global__ __launch_bounds__(kWideThreads, 1) void attn_mfma_wide_kernel(AttnArgs a) {
  using S = typename E::storage;
  using Sh = WideShape<kD>;
  constexpr int kChunks = Sh::kChunks, kSteps = Sh::kSteps, kDimTiles = Sh::kDimTiles;
  constexpr int kRowBytes = Sh::kRowBytes, kL = Sh::kLoadsPerWave, kB = Sh::kBlocks, kWaveRows = Sh::kWaveRows;

  extern __shared__ va_u32x4 smem[];
  const char* lds = (const char*)smem;

  // workgroup -> (slot, kv head); the slot's items are run one after the other
  // The slots of a die run in groups of up to 32 under ONE kv head at a time (a die has 32 compute
  // units): neighbouring slots hold neighbouring query tiles of one request, which walk the same
  // K/V rows, so the die's L2 holds one head's stream at a time instead of all of them.
  ItemHead where;
  {
    const unsigned die = blockIdx.x & 7u, turn = blockIdx.x >> 3, per_die = gridDim.x / (8u * a.num_kv_heads);
    unsigned g = 32;
    while (per_die % g) g >>= 1;
    const unsigned block = turn / (g * a.num_kv_heads), within = turn % (g * a.num_kv_heads);
    where = ItemHead{(int)((block * g + within % g) * 8u + die), (int)(within / g)};
  }
  const int item_begin = a.wide_slots[where.item], item_end = a.wide_slots[where.item + 1];
  const int hk = where.head;
  const int G = a.num_q_heads / a.num_kv_heads;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int lane = tid % kWave;
  const int j = lane % 32;         // row within a 32-row block / token within a tile / dim group
  const int h = lane / 32;         // half-wave: contraction group
  const int row0 = kWaveRows * wave + j;  // this lane's row in block 0; block 1 is 32 further
  int row_iq[kB];
#pragma unroll
  for (int b = 0; b < kB; ++b) row_iq[b] = (row0 + 32 * b) / G;
  const S* kp = (const S*)a.k_pool + (long long)hk * kD;
  const S* vp = (const S*)a.v_pool + (long long)hk * kD;
  const int P = a.page_size;
  const bool pow2_pages = (P & (P - 1)) == 0;
  const int p_shift = __builtin_ctz(P);  // t / P and t % P as shift and mask (power-of-two pages)
  const int row_bytes = (int)a.pool_row_stride * (int)sizeof(S);
  // bytes of a page, for the offsets of plain tiles: such tiles need the figure to fit 32 bits
  const bool page_fits = ((unsigned long long)(uint32_t)row_bytes << p_shift) <= 0xffffffffull;
  const uint32_t page_bytes = (uint32_t)row_bytes << p_shift;

  // This lane's part of a wave-level load (64 lanes x 16 bytes land as one 1 KB run in LDS; which
  // piece of the pool a lane fetches is free).  Waves 0 and 1 load K halves, waves 2 and 3 V halves.
  //   V: load u covers kRowsPerLoad whole rows, piece c of row r at position c ^ vswz(r).
  //   K: fragment order.  Load u of a half is the block (8 rows R, 128-byte column g) = the operands
  //      of four contraction steps for eight tokens: lane 16 s2 + 8 (h ^ R % 2) + j3 fetches row
  //      8 R + j3, piece 8 g + 2 s2 + h.  The block of step s = 4 g + s2 thus lies 256 s bytes into
  //      the 8-row region of R, and the fragment reads of a tile are ONE per-lane address plus
  //      immediates; 16 consecutive lanes (served together) read 256 consecutive bytes, the flip of
  //      h in odd R keeps the two regions they straddle on different banks.
  const bool wave_is_v = wave >= 2;
  constexpr int kColumns = kChunks / 8;  // 128-byte columns of a row
  const int ld_row0 = lane / kChunks;
  const int ld_x0 = (lane % kChunks) ^ wide_vswz(ld_row0);
  auto ld_row = [&](int u) __attribute__((always_inline)) {  // row within the wave's 16-token half
    return wave_is_v ? u * Sh::kRowsPerLoad + ld_row0 : 8 * (u / kColumns) + lane % 8;
  };
  auto ld_piece = [&](int u) __attribute__((always_inline)) {
    return wave_is_v ? (ld_x0 ^ wide_vswz(u * Sh::kRowsPerLoad))
                     : 8 * (u % kColumns) + 2 * (lane / 16) + (((lane / 8) ^ (u / kColumns)) & 1);
  };
  // The loads of a plain tile (uniform pages, inside the visible range) go out in groups of up to four
  // behind one setting of M0, as a wave-uniform base plus a per-lane offset that never changes.  A
  // group's immediate offsets move the pool address as well: the per-lane offsets have them taken
  // off beforehand (grouped_lane_offset) and carry a bias, which the base gives back, to stay positive.
  constexpr int kLoadBias = 3072;
  uint32_t ld_off[kL];
#pragma unroll
  for (int u = 0; u < kL; ++u)
    ld_off[u] = grouped_lane_offset((uint32_t)(ld_row(u) * row_bytes + 16 * ld_piece(u) + kLoadBias), u);
  constexpr int kLoadGroup = kL >= 4 ? 4 : kL;
  auto issue_plain = [&](const char* base, uint32_t dst) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < kL; u += kLoadGroup) load_group_to_lds<kLoadGroup>(base, ld_off + u, dst + u * 1024);
  };
  // LDS offsets of what this lane reads from a tile
  const int k_lane_byte = (j / 8) * 8 * kRowBytes + 128 * ((h ^ (j / 8)) & 1) + 16 * (j % 8);
  // V^T fragments come from transposing reads.  For dim tile t (dims 32t .. 32t+31) and 16-token
  // step kk the lane needs, as contraction elements 0..3 and 4..7, tokens 16kk + 4h + 0..3 and
  // 16kk + 8 + 4h + 0..3 of dim 32t + lane % 32 (the token order P^T has in its registers): two
  // reads, in each of which this lane points at token row `v_row` (+ 16kk, + 8) and at 4 dims of
  // the tile's 16-dim half lane / 16 % 2.  The swizzle folds into two per-lane bases, one for even
  // and one for odd t; everything else is an immediate offset.
  const int v_sub = lane % 16;
  const int v_row = 4 * h + v_sub / 4;
  const int v_swz = wide_vswz(v_row);
  const int v_piece = (2 * ((lane / 16) % 2) + (v_sub % 4) / 2) ^ (v_swz & 2);
  const int v_base = v_row * kRowBytes + 16 * v_piece + 8 * (v_sub % 2);
  const int v_even = v_base + 64 * (v_swz >> 2), v_odd = v_base + 64 * (1 ^ (v_swz >> 2));
  const uint32_t lds_base = lds_address(lds);

  for (int item_index = item_begin; item_index < item_end; ++item_index) {
  const int32_t* item = a.items + (long long)item_index * VA_ITEM_WORDS;
  const int n_q = item[VA_I_N_Q];
  if (n_q == 0) continue;  // padding item
  const int part_base = item[VA_I_PART_BASE];
  const bool wave_active = (kWaveRows * wave) / G < n_q;  // the wave owns real rows

  float m_ref[kB], m_tile[kB], l_run[kB];  // reference maximum (log2 units), last tile maximum, row sum
  float raise_above[kB];                    // m_ref + kWideRaise: what a tile's maximum is tested against
  va_f32x16 o[kB][kDimTiles];
#pragma unroll
  for (int b = 0; b < kB; ++b) {
    m_ref[b] = kNegBig;
    m_tile[b] = kNegBig;
    raise_above[b] = kNegBig + kWideRaise;
    l_run[b] = 0.f;
#pragma unroll
    for (int t = 0; t < kDimTiles; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[b][t][r] = 0.f;
  }

  for (int li = 0; li < item[VA_I_N_LINKS]; ++li) {
    const int32_t* link = a.links + (long long)(item[VA_I_LINK_BEGIN] + li) * VA_LINK_WORDS;
    const int lflags = link[VA_L_FLAGS];
    const int qref = link[VA_L_QREF];
    const int kv_begin = link[VA_L_KV_BEGIN];
    const int tok_begin = link[VA_L_TOK_BEGIN];
    const int tok_end = link[VA_L_TOK_END];
    const int causal_base = link[VA_L_CAUSAL_BASE];
    const bool slots = lflags & VA_LINK_SLOTS;
    // a 16-token half tile lies inside one page only if the link starts on a 16-token boundary
    const bool uniform_pages = !slots && pow2_pages && page_fits && P >= 16 && (tok_begin % 16 == 0);

    const int t_stop = min(tok_end, causal_base + n_q);  // tokens any row of the tile sees
    const int t_last = t_stop - 1;
    int t_row[kB];
#pragma unroll
    for (int b = 0; b < kB; ++b) t_row[b] = min(tok_end, causal_base + row_iq[b] + 1);
    // tokens any row of this wave sees, and tokens EVERY real row of it sees (no masking below that)
    const int wave_iq_last = min(n_q - 1, (kWaveRows * wave + kWaveRows - 1) / G);
    const int t_wave = wave_active ? min(tok_end, causal_base + wave_iq_last + 1) : -0x7fffffff;
    const int t_wave_min = min(tok_end, causal_base + (kWaveRows * wave) / G + 1);
    const int n_tiles = t_stop > tok_begin ? (t_stop - tok_begin + kWideTokens - 1) / kWideTokens : 0;

    // Loads of a tile.  Wave w fetches one 16-token half of the K tile (w = 0, 1) or of the V tile
    // (w = 2, 3): kL wave-level loads of kRowsPerLoad rows each.  With uniform pages the half lies
    // in one page, so the wave needs ONE scalar page lookup per tile and every load is a
    // wave-uniform base plus a per-lane offset that never changes (ld_off); tiles that reach past
    // the visible range, and page tables with pages under 16 tokens or slot lists, look every
    // row up per lane instead (rows past the range re-read the last visible token; their scores
    // are masked).
    const int wave_half = wave & 1;
    const char* wave_pool = (const char*)(wave_is_v ? vp : kp);
    const char* wave_plain = wave_pool - kLoadBias;  // base of plain loads: the per-lane offsets carry the bias
    const uint32_t wave_lds = __builtin_amdgcn_readfirstlane(lds_address(lds)) + (wave_is_v ? Sh::kTileBytes : 0) +
                              wave_half * 16 * kRowBytes;
    // pool row of this wave's half of tile i (uniform pages, tile inside the visible range); read
    // through the constant address space so that the lookup stays a scalar load
    // (as a byte offset: page x bytes of a page + row in the page x bytes of a row, a 32 x 32 -> 64 bit
    // product and a 32-bit one; the row number times the row size would be a 64 x 32 bit product, six
    // scalar instructions in every ring step)
    auto half_offset = [&](int page, int t) __attribute__((always_inline)) {
      return (unsigned long long)(uint32_t)page * page_bytes + (uint32_t)(t & (P - 1)) * (uint32_t)row_bytes;
    };
    auto half_row = [&](int i) __attribute__((always_inline)) {
      const int t = tok_begin + i * kWideTokens + 16 * wave_half;
      const int page = ((const __attribute__((address_space(4))) int32_t*)a.kv_indices)[kv_begin + (t >> p_shift)];
      return half_offset(page, t);
    };
    auto tile_is_plain = [&](int i) __attribute__((always_inline)) {
      return uniform_pages && tok_begin + (i + 1) * kWideTokens - 1 <= t_last;
    };
    auto issue = [&](int i, unsigned long long row) __attribute__((always_inline)) {
      const uint32_t dst = wave_lds + ring_slot(i) * Sh::kBufferBytes;
      if (tile_is_plain(i)) {
        const char* base = wave_plain + row;
        issue_plain(base, dst);
      } else {
        const int t0 = tok_begin + i * kWideTokens + 16 * wave_half;
#pragma unroll
        for (int u = 0; u < kL; ++u) {
          const int t = min(t0 + ld_row(u), t_last);
          const int piece = 16 * ld_piece(u);
          load_to_lds(wave_pool + kv_slot(a.kv_indices, kv_begin, t, P, slots) * row_bytes + piece, dst + u * 1024);
        }
      }
    };
    auto issue_now = [&](int i) __attribute__((always_inline)) { issue(i, tile_is_plain(i) ? half_row(i) : 0); };

    // ---- set-up: first two tiles on their way, then the query tile (staged in buffers 2 and 3) ----
    __syncthreads();  // every wave is done with the previous link's buffers
#pragma unroll
    for (int i = 0; i < kWideAhead; ++i)
      if (i < n_tiles) issue_now(i);
    va_u32x4* q_stage = (va_u32x4*)(lds + kWideAhead * Sh::kBufferBytes);
    va_u32x4 qf[kB][kSteps];  // B operands: row of block b, dims [16s + 8h, +8)
#pragma unroll
    for (int pass = 0; pass < kB; ++pass) {
      if (a.rope.mode == VA_ROPE_TABLE) {
        // Every thread stages one unit (two pieces) of kIts rows.  The sub-row numbers are fetched
        // for all rows at once, source rows and positions, then pieces and table entries, for
        // kBatch rows at once: a row's chain of dependent loads (sub-row -> source row and position
        // -> query pieces and cos|sin entries) is paid once per batch, not once per row (row by row
        // this set-up was an eighth of the kernel on long views of many blocks).
        constexpr int kUnits = kChunks / 2, kRowStep = kWideThreads / kUnits, kIts = 128 / kRowStep;
        constexpr int kBatch = kIts < 4 ? kIts : 4;
        static_assert(kWideThreads % kUnits == 0 && 128 % kRowStep == 0 && kIts % kBatch == 0, "staging pattern");
        const int x = tid % kUnits, rl0 = tid / kUnits;
        const int pair_units = a.rope.rotary_dim / 16;
        const bool rotary = x < pair_units;
        const int c0 = rotary ? x : a.rope.rotary_dim / 8 + 2 * (x - pair_units);
        const int c1 = rotary ? x + pair_units : c0 + 1;
        bool live[kIts];
        int subrow[kIts];
#pragma unroll
        for (int it = 0; it < kIts; ++it) {
          const int Rl = rl0 + it * kRowStep;
          const int R = kWaveRows * (Rl / 32) + 32 * pass + Rl % 32;  // block `pass` of every wave
          const int iq = R / G;
          live[it] = iq < n_q;
          const int iqc = live[it] ? iq : 0;  // rows past the tile stage row 0's numbers and are zeroed below
          subrow[it] = (lflags & VA_LINK_INDIRECT) ? a.qrefs[qref + iqc] : qref + iqc;
        }
#pragma unroll
        for (int it0 = 0; it0 < kIts; it0 += kBatch) {
          const S* qh[kBatch];
          Pos3 pos[kBatch];
#pragma unroll
          for (int jj = 0; jj < kBatch; ++jj) {
            const int Rl = rl0 + (it0 + jj) * kRowStep;
            const int R = kWaveRows * (Rl / 32) + 32 * pass + Rl % 32;
            const int iq = R / G, g = R - iq * G;
            const long long src_row = a.sub_worker[subrow[it0 + jj]];
            qh[jj] = (const S*)a.q + src_row * a.q_row_stride + (long long)(hk * G + g) * kD;
            pos[jj] = load_pos(a.sub_loc, a.sub_loc_axis_stride, subrow[it0 + jj]);
          }
          uint4 p0[kBatch], p1[kBatch];
          if (rotary) {
            TableQueryUnit<E> unit[kBatch];
#pragma unroll
            for (int jj = 0; jj < kBatch; ++jj) unit[jj].load(a.rope, qh[jj], x, pos[jj]);
#pragma unroll
            for (int jj = 0; jj < kBatch; ++jj) unit[jj].finish(a.rope, pos[jj], p0[jj], p1[jj]);
          } else {
#pragma unroll
            for (int jj = 0; jj < kBatch; ++jj) {
              p0[jj] = *(const uint4*)(qh[jj] + 8 * c0);
              p1[jj] = *(const uint4*)(qh[jj] + 8 * c1);
            }
          }
#pragma unroll
          for (int jj = 0; jj < kBatch; ++jj) {
            const int Rl = rl0 + (it0 + jj) * kRowStep;
            if (!live[it0 + jj]) p0[jj] = p1[jj] = make_uint4(0, 0, 0, 0);
            q_stage[Rl * kChunks + (c0 ^ wide_swz<kD>(Rl))] = va_u32x4{p0[jj].x, p0[jj].y, p0[jj].z, p0[jj].w};
            q_stage[Rl * kChunks + (c1 ^ wide_swz<kD>(Rl))] = va_u32x4{p1[jj].x, p1[jj].y, p1[jj].z, p1[jj].w};
          }
        }
      } else {
        // mRoPE computes its cosines and sines (no table to wait for): row by row
        for (int idx = tid; idx < 128 * (kChunks / 2); idx += kWideThreads) {  // two pieces per step
          const int Rl = idx / (kChunks / 2), x = idx - Rl * (kChunks / 2);
          const int R = kWaveRows * (Rl / 32) + 32 * pass + Rl % 32;  // block `pass` of every wave
          const int iq = R / G, g = R - iq * G;
          int c0 = 2 * x, c1 = 2 * x + 1;
          uint4 p0 = make_uint4(0, 0, 0, 0), p1 = p0;
          if (iq < n_q) {
            const int subrow = (lflags & VA_LINK_INDIRECT) ? a.qrefs[qref + iq] : qref + iq;
            const long long src_row = a.sub_worker[subrow];
            const S* qh = (const S*)a.q + src_row * a.q_row_stride + (long long)(hk * G + g) * kD;
            const Pos3 p = load_pos(a.sub_loc, a.sub_loc_axis_stride, subrow);
            rotated_query_unit<E>(a.rope, qh, x, p, c0, c1, p0, p1);
          }
          q_stage[Rl * kChunks + (c0 ^ wide_swz<kD>(Rl))] = va_u32x4{p0.x, p0.y, p0.z, p0.w};
          q_stage[Rl * kChunks + (c1 ^ wide_swz<kD>(Rl))] = va_u32x4{p1.x, p1.y, p1.z, p1.w};
        }
      }
      ring_barrier<kAnyInFlight>();
      {
        const int Rl = 32 * wave + j;
#pragma unroll
        for (int s = 0; s < kSteps; ++s) qf[pass][s] = q_stage[Rl * kChunks + ((2 * s + h) ^ wide_swz<kD>(Rl))];
      }
      ring_barrier<kAnyInFlight>();  // staging rows may be overwritten now
    }

    // ---- the tile loop ----
    // Reference maximum.  The softmax runs against a per-row REFERENCE maximum m_ref that is
    // raised only when a tile's maximum exceeds it by more than kWideRaise (in log2 units):
    // p = exp2(s - m_ref) then stays below 2^kWideRaise, harmless for the 16-bit P operand and the
    // fp32 sums, and any consistent reference gives the same softmax.  Raising m_ref means
    // rescaling the D fp32 accumulators of every row, vector-ALU work on registers that otherwise
    // only the matrix pipe touches; it happens on the first tile and then hardly ever, so it is
    // kept out of the hot loop: the steady loop is left, the accumulators are rescaled, the tile is
    // computed, the steady loop is entered again.  (One wave per SIMD issues an instruction every four
    // clocks or so whatever its kind: the steady loop's own control being a counter and one test,
    // instead of the general loop's flags, is worth 2 % of the kernel.)
    //
    // Software pipeline.  One wave per SIMD means nothing but this wave's own instruction order
    // can keep the matrix pipe busy, so the loop body is written as pieces pinned in order with
    // scheduling barriers: while the scores of tile i+1 are computed (matrix pipe), the
    // exponentials of tile i run on the vector ALU; while the products P.V of tile i run, the V
    // fragments of the next product are transposed.
    //
    // Ring.  ring_step(k): wait until tile k has landed for the whole workgroup (one barrier) and
    // request tile k + 2 into the buffer of tile k - 2, which every wave has left by then.  Every
    // wave makes every step exactly once, in order; a step is made just before tile k is first
    // needed (its K, for the scores computed one iteration ahead).
    const int n_vis = t_wave > tok_begin ? min(n_tiles, (t_wave - tok_begin + kWideTokens - 1) / kWideTokens) : 0;
    int next_step = 0;
    // The pool row of the tile a step requests is looked up a whole step earlier (a scalar load whose
    // result is not touched before the next step): its latency never shows.
    auto row_of = [&](int tile) __attribute__((always_inline)) {
      return (tile < n_tiles && tile_is_plain(tile)) ? half_row(tile) : 0ull;
    };
    unsigned long long row_ahead = row_of(kWideAhead);
    auto ring_step = [&]() __attribute__((always_inline)) {
      const int k = next_step++;
      const bool refill = k + kWideAhead < n_tiles;
      const unsigned long long row = row_ahead;
      row_ahead = row_of(k + 1 + kWideAhead);
      // only the loads of the tiles requested after tile k (up to kWideAhead - 1 of them) may still be outstanding
      if (k + kWideAhead - 1 < n_tiles) {
        ring_barrier<(kWideAhead - 1) * kL>();
      } else if (kWideAhead > 2 && k + 1 < n_tiles) {
        ring_barrier<kL>();
      } else {
        ring_barrier<0>();
      }
      if (refill) issue(k + kWideAhead, row);
    };

    // The same step for the steady part of a link (uniform pages; the requested tile and the one
    // after it inside the visible range): no case distinctions, and the page lookup for the next
    // step is sent before the barrier and first touched after it, so its latency passes under the wait.
    const __attribute__((address_space(4))) char* link_pages =
        (const __attribute__((address_space(4))) char*)(a.kv_indices + kv_begin);
    auto ring_step_steady = [&]() __attribute__((always_inline)) {
      const int k = next_step++;
      const unsigned long long row = row_ahead;
      const int t = tok_begin + (k + 1 + kWideAhead) * kWideTokens + 16 * wave_half;
      // (base of the link's page list + an unsigned 32-bit byte offset: a scalar load with a register offset)
      const int page = *(const __attribute__((address_space(4))) int32_t*)(link_pages + ((uint32_t)(t >> p_shift) << 2));
      // The K half of the buffer refilled here was last read two steps ago (the scores of a tile are computed
      // an iteration ahead of its products), and every wave has passed a barrier since: the waves that load K
      // send their requests BEFORE the barrier, in the time they would otherwise only wait, and out of step
      // with the waves that load V, which must wait for the products of the previous iteration to end.
      int zero;
      const uint32_t dst = wave_lds + ring_slot(k + kWideAhead) * Sh::kBufferBytes;
      const char* base = wave_plain + row;
      if (!wave_is_v) {
        issue_plain(base, dst);
        zero = ring_barrier_zero<kWideAhead * kL>();
      } else {
        zero = ring_barrier_zero<(kWideAhead - 1) * kL>();
        issue_plain(base, dst);
      }
      row_ahead = half_offset(page + zero, t);
    };
    // iterations [1, i_steady_end) may take it: tiles i + 1 + kWideAhead and i + 2 + kWideAhead are plain,
    // tile i is unmasked for every row of the wave and a next tile exists
    int i_steady_end = 0;
    if (uniform_pages) {
      const int plain_tiles = (t_last + 1 - tok_begin) / kWideTokens;  // tiles 0 .. plain_tiles - 1 are plain
      const int unmasked_tiles = t_wave_min > tok_begin ? (t_wave_min - tok_begin) / kWideTokens : 0;
      i_steady_end = min(min(plain_tiles - 2 - kWideAhead, unmasked_tiles), n_vis - 1);
    }

    // Scores of two tiles: the exponentials of one are taken in place while the products of the next
    // accumulate into the other; which is which alternates from tile to tile.
    va_f32x16 sc[kB];       // scores, then probabilities, of the current tile (between tiles)
    va_f32x16 sc_next[kB];  // scores of the next tile
    // K fragments: at most eight in registers; the fragment eight steps on is requested as one is consumed
    constexpr int kKRing = kSteps < 8 ? kSteps : 8;
    va_u32x4 kf[kKRing];
    auto read_k_fragment = [&](int tile, int s) __attribute__((always_inline)) {
      const char* kt = lds + ring_slot(tile) * Sh::kBufferBytes;
      kf[s % kKRing] = *(const va_u32x4*)(kt + k_lane_byte + 256 * s);
    };
    auto read_k = [&](int tile) __attribute__((always_inline)) {
#pragma unroll
      for (int s = 0; s < kKRing; ++s) read_k_fragment(tile, s);
    };
    auto score_step = [&](int tile, int s, auto& into) __attribute__((always_inline)) {
#pragma unroll
      for (int b = 0; b < kB; ++b) {
        // through the builtin: the compiler sees these products and keeps the wait states between
        // them and the vector-ALU instructions that feed them or read their results
        into[b] = Mma<E>::run32(kf[s % kKRing], qf[b][s], s == 0 ? va_f32x16{} : into[b]);
      }
      if (s + kKRing < kSteps) read_k_fragment(tile, s + kKRing);
    };

    if (n_vis > 0) {  // scores of tile 0
      ring_step();
      read_k(0);
#pragma unroll
      for (int s = 0; s < kSteps; ++s) score_step(0, s, sc);
    }
    // maximum of the (unmasked) scores of the next tile per lane, gathered piecewise between the
    // P.V products of the current one, whose matrix work leaves the vector ALU idle
    float early_max[kB];
    bool early_max_valid = false;
#pragma unroll
    for (int b = 0; b < kB; ++b) early_max[b] = 0.f;
    // One tile: phase A and phase B below, on the scores in `cur`, leaving those of the next tile in `nxt`.
    // The steady part of a link runs it in a loop of its own, whose control is a counter and the test for
    // a raised reference; every other tile (the first, masked ones, the last, the one after a raised
    // reference) goes through the general step further down.
    auto tile_body = [&](int i, auto& cur, auto& nxt) __attribute__((always_inline)) {

      // V^T fragments of this tile, kVAhead of them in flight: fragment idx = (step kk, dim tile t)
      const uint32_t vt = lds_base + ring_slot(i) * Sh::kBufferBytes + Sh::kTileBytes;
      const uint32_t vt_even = vt + v_even, vt_odd = vt + v_odd;
      constexpr int kFrags = 2 * kDimTiles;
      constexpr int kMaxFirst = kFrags > 2 ? 2 : kFrags - 1;  // first product the early maxima follow
      constexpr int kVAhead = kFrags < 4 ? kFrags : 4;
      va_u32x4 vfr[kVAhead];
      auto read_vfrag = [&](int idx) __attribute__((always_inline)) {
        const int kk = idx / kDimTiles, t = idx % kDimTiles;
        const uint32_t at = ((t & 1) ? vt_odd : vt_even) + 128 * (t / 2) + kk * 16 * kRowBytes;
        const va_u32x2 lo = lds_read_tr16(at), hi = lds_read_tr16(at + 8 * kRowBytes);
        vfr[idx % kVAhead] = va_u32x4{lo[0], lo[1], hi[0], hi[1]};
      };
      // ---- phase A: scores of tile i + 1 (matrix pipe) under the exponentials of tile i ----
      float sum[kB];
#pragma unroll
      for (int b = 0; b < kB; ++b) sum[b] = 0.f;
      // Piece r: the exponential of element r; the sum takes element r - 1 (an exponential's result
      // is not ready for the very next instruction) and odd pieces pack the finished pair into P.
      uint32_t pw[kB][8];
      auto exp_piece = [&](int r) __attribute__((always_inline)) {
#pragma unroll
        for (int b = 0; b < kB; ++b) {
          // raw score -> exponent in fp32, as the reference scales its scores.  (The multiply-add sits here,
          // in the shadow of a score product, rather than under the P.V products, whose slots are full: there
          // it costs 3.4 % of the kernel, here 0.8 %.  Staging the query times the scale instead makes it
          // free, but rounds other numbers than the reference does: out of tolerance once scores reach +-20.)
          cur[b][r] = __builtin_amdgcn_exp2f(fmaf(cur[b][r], a.scale_log2, -m_ref[b]));
          if (r > 0) sum[b] += cur[b][r - 1];
          if (r >= 2 && r % 2 == 0) pw[b][r / 2 - 1] = Mma<E>::pack(cur[b][r - 2], cur[b][r - 1]);
        }
      };
      constexpr int kPiecesPerStep = 16 / kSteps > 0 ? 16 / kSteps : 1;  // exponentials between two score steps
      // The last visible tile runs the same instructions: its "next scores" come from whatever
      // the following ring buffer holds and are never looked at (sixteen idle products per link
      // against a second copy of this phase and the register moves where the two would meet).
      read_k(i + 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        if (r % kPiecesPerStep == 0) score_step(i + 1, r / kPiecesPerStep, nxt);
        __builtin_amdgcn_sched_barrier(0);
        exp_piece(r);
        // the first V fragments are requested once half of the K fragments have been consumed: the
        // counter of outstanding LDS reads holds fifteen, and a wait for the first K fragment
        // with more than that in flight becomes a wait for the excess as well
        if (r == 8) {
#pragma unroll
          for (int idx = 0; idx < kVAhead; ++idx) read_vfrag(idx);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int b = 0; b < kB; ++b) {
        l_run[b] += sum[b] + cur[b][15];
        pw[b][7] = Mma<E>::pack(cur[b][14], cur[b][15]);
      }

      // ---- phase B: O^T += V^T . P^T over two 16-token steps; a fragment serves all row blocks,
      // and once it has been used the fragment kVAhead further on is requested ----
      va_u32x4 pf[2][kB];
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int b = 0; b < kB; ++b)
          pf[kk][b] = va_u32x4{pw[b][4 * kk + 0], pw[b][4 * kk + 1], pw[b][4 * kk + 2], pw[b][4 * kk + 3]};
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int idx = 0; idx < kFrags; ++idx) {
        const int kk = idx / kDimTiles, t = idx % kDimTiles;
#pragma unroll
        for (int b = 0; b < kB; ++b) {
          Mma<E>::run32_acc(vfr[idx % kVAhead], pf[kk][b], o[b][t]);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (idx + kVAhead < kFrags) read_vfrag(idx + kVAhead);
        // Elements of the next tile's scores folded into early_max after this product: the 15
        // comparisons are spread over the products from the third on (the last score product was
        // issued well before, so its results have been written).
        if (idx >= kMaxFirst) {
#pragma unroll
          for (int e = 1; e < 16; ++e) {
            if (kMaxFirst + (e - 1) * (kFrags - kMaxFirst) / 15 != idx) continue;
#pragma unroll
            for (int b = 0; b < kB; ++b)
              early_max[b] = fmaxf(e == 1 ? nxt[b][0] : early_max[b], nxt[b][e]);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    // The reference of the rows is raised to the maxima of the tile in `cur` (m_tile, log2 units): what was
    // accumulated against the old reference is rescaled; the tile's raw scores stay as they are.
    auto raise_reference = [&](int i, auto& cur) __attribute__((always_inline)) {
      accumulator_fence<kB * kDimTiles>(&o[0][0]);
#pragma unroll
      for (int b = 0; b < kB; ++b) {
        const float m_new = fmaxf(m_ref[b], m_tile[b]);
        const float alpha = __builtin_amdgcn_exp2f(m_ref[b] - m_new);
        m_ref[b] = m_new;
        raise_above[b] = m_new + kWideRaise;
        l_run[b] *= alpha;
#pragma unroll
        for (int t = 0; t < kDimTiles; ++t) o[b][t] *= alpha;
        const int t0 = tok_begin + i * kWideTokens;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const bool visible = (t0 + (r / 4) * 8 + 4 * h + (r % 4)) < t_row[b];
          cur[b][r] = visible ? cur[b][r] : -INFINITY;
        }
      }
    };
    // the test of the steady part: the maxima were gathered under the previous products, nothing is masked
    auto steady_test = [&]() __attribute__((always_inline)) {
      bool raise = false;
#pragma unroll
      for (int b = 0; b < kB; ++b) {
        m_tile[b] = half_wave_max(early_max[b]) * a.scale_log2;
        raise = raise || m_tile[b] > raise_above[b];
      }
      return (bool)__any(raise);
    };

    int i = 0;
    while (i < n_vis) {
      bool raise = false;
      if (i >= 1 && i < i_steady_end) {
        // steady part
        do {
          ring_step_steady();
          raise = steady_test();
          if (raise) break;
          tile_body(i, sc, sc_next);
#pragma unroll
          for (int b = 0; b < kB; ++b) sc[b] = sc_next[b];
          ++i;
        } while (i < i_steady_end);
        early_max_valid = true;  // (a next tile exists throughout the steady part)
        if (!raise) continue;
      } else {
        const int t0 = tok_begin + i * kWideTokens;
        if (i + 1 < n_tiles) ring_step();  // tile i + 1 has landed
        // mask and find the tile maxima; reg r of a block is token t0 + (r/4)*8 + 4h + r%4 of its row
        const bool masked = t0 + kWideTokens > t_wave_min;
#pragma unroll
        for (int b = 0; b < kB; ++b) {
          if (masked) {
#pragma unroll
            for (int r = 0; r < 16; ++r)
              sc[b][r] = (t0 + (r / 4) * 8 + 4 * h + (r % 4)) < t_row[b] ? sc[b][r] : -INFINITY;
          }
          // the tile maximum (raw): from the maxima found under the previous products, or, for a masked or
          // first tile, from sc
          float tile_max = early_max[b];
          if (masked || !early_max_valid) {
            tile_max = sc[b][0];
#pragma unroll
            for (int r = 1; r < 16; ++r) tile_max = fmaxf(tile_max, sc[b][r]);
          }
          m_tile[b] = half_wave_max(tile_max) * a.scale_log2;
          raise = raise || m_tile[b] > raise_above[b];
        }
        raise = __any(raise);
      }
      if (raise) raise_reference(i, sc);
      tile_body(i, sc, sc_next);
#pragma unroll
      for (int b = 0; b < kB; ++b) sc[b] = sc_next[b];
      early_max_valid = i + 1 < n_vis;
      ++i;
    }
    while (next_step < n_tiles) ring_step();  // tiles this wave does not see: keep in step with the others
  }

  accumulator_fence<kB * kDimTiles>(&o[0][0]);
  // ---- emit: accumulator reg r of dim tile t is dim 32t + (r/4)*8 + 4h + r%4 of the lane's row ----
#pragma unroll
  for (int b = 0; b < kB; ++b) {
    float l = l_run[b];
    {
      const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(l), __float_as_uint(l), false, false);
      l = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    }
    const int my_row = row0 + 32 * b;
    const int iq = row_iq[b];
    if (iq >= n_q) continue;
    const int g = my_row - iq * G;
    const int hq = hk * G + g;
    const float inv = l > 0.f ? 1.f / l : 0.f;
    if (part_base < 0) {
      const int32_t* link0 = a.links + (long long)item[VA_I_LINK_BEGIN] * VA_LINK_WORDS;
      const int subrow = (link0[VA_L_FLAGS] & VA_LINK_INDIRECT) ? a.qrefs[link0[VA_L_QREF] + iq] : link0[VA_L_QREF] + iq;
      const long long out_row = a.sub_worker[subrow];
      S* orow = (S*)a.out + (out_row * a.num_q_heads + hq) * (long long)kD;
#pragma unroll
      for (int t = 0; t < kDimTiles; ++t)
#pragma unroll
        for (int r = 0; r < 16; r += 4) {  // four consecutive dims
          const int d0 = 32 * t + (r / 4) * 8 + 4 * h;
          *(uint2*)(orow + d0) = make_uint2(Mma<E>::pack(o[b][t][r] * inv, o[b][t][r + 1] * inv),
                                            Mma<E>::pack(o[b][t][r + 2] * inv, o[b][t][r + 3] * inv));
        }
      if (h == 0 && a.lse) {
        const float lse2 = l > 0.f ? m_ref[b] + log2f(l) : -INFINITY;
        a.lse[out_row * a.num_q_heads + hq] = a.lse_base2 ? lse2 : lse2 * kLn2;
      }
    } else {
      const long long slot = (long long)(part_base + iq) * a.num_q_heads + hq;
      float* prow = a.part_acc + slot * kD;
#pragma unroll
      for (int t = 0; t < kDimTiles; ++t)
#pragma unroll
        for (int r = 0; r < 16; r += 4)
          *(float4*)(prow + 32 * t + (r / 4) * 8 + 4 * h) = make_float4(o[b][t][r], o[b][t][r + 1], o[b][t][r + 2], o[b][t][r + 3]);
      if (h == 0) {
        a.part_ml[slot * 2 + 0] = m_ref[b];
        a.part_ml[slot * 2 + 1] = l;
      }
    }
  }
  }  // items of the slot
}

template <typename E, int kD>
static int launch_wide_one(const AttnArgs& a, int n_items, hipStream_t stream) {
  constexpr int bytes = WideShape<kD>::kLdsBytes;
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
