// Host-side work decomposition for view attention.
//
// Takes the planned sub-request tables of one launch (what the reference feeds
// to FlashInfer's plan(): python/minisgl/shared_cache/attention.py:390-426 for
// decode, :574-604 for prefill) and cuts them into work items sized for the
// 256 CUs of an MI355X:
//   * stand-alone (decode) sub-requests that read the identical page list are
//     batched into one query tile, so a block shared by many views is streamed
//     once per tile instead of once per reader;
//   * long KV runs are split into chunks (split-KV); every (row, chunk) yields a
//     partial softmax state that the merge kernel folds together with the
//     row's other segments -- the same LSE merge the reference performs across
//     segments (attention.py:694-703);
//   * the sub-requests of one prefill request are chained so a query tile walks
//     all of its segments in one workgroup, carrying the online softmax in
//     registers (no per-segment scratch as in attention.py:736-751).
#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <numeric>
#include <unordered_map>
#include <vector>

#include "../../include/viewattn.h"
#include "va_internal.h"
#include "va_plan.h"

namespace {

struct Item {
  int32_t link_begin, n_links, n_q, part_base, tokens, kind;
  int32_t unit;  // items that stream the same K/V chunk share a unit (planner only, not serialised)
  int32_t slot;  // wide items packed into one workgroup share a slot, -1: none (planner only)
};
constexpr int kXcds = 8;  // accelerator dies of an MI355X, each with its own L2; workgroup b runs on die b % 8
struct Link {
  int32_t kv_begin, tok_begin, tok_end, qref, causal_base, flags;
};

struct Built {
  std::vector<Item> items;
  std::vector<Link> links;
  std::vector<int32_t> qrefs;
  std::vector<int32_t> row_indptr;
  std::vector<int32_t> row_ids;
  std::vector<int32_t> row_flags;
  std::vector<int32_t> wide_slots;  // indptr over the wide items: the items of each workgroup of the wide launch
  int32_t n_partials = 0;
  int32_t kernel = 0, q_tile = 0, kv_chunk = 0, wide_tile = 0, n_wide = 0;
};

inline int32_t round_up(int64_t x, int32_t m) { return (int32_t)(((x + m - 1) / m) * m); }

int check_subs(const VaSubRequests* s, const VaShape* shape) {
  if (!s || !shape) return va_fail(VA_ERR_ARG, "null argument");
  if (s->n_sub < 0 || s->n_rows < 0 || s->n_subrows < 0) return va_fail(VA_ERR_ARG, "negative count");
  if (s->n_sub > 0 && (!s->qo_indptr || !s->kv_indptr || !s->seq_lens || !s->flags || !s->chain))
    return va_fail(VA_ERR_ARG, "null sub-request table");
  if (s->n_subrows > 0 && !s->sub_worker) return va_fail(VA_ERR_ARG, "null sub_worker");
  if (shape->num_kv_heads <= 0 || shape->num_q_heads % shape->num_kv_heads)
    return va_fail(VA_ERR_ARG, "num_q_heads must be a multiple of num_kv_heads");
  if (shape->page_size <= 0) return va_fail(VA_ERR_ARG, "page_size must be positive");
  if (s->n_sub > 0) {
    if (s->qo_indptr[0] != 0 || s->kv_indptr[0] != 0) return va_fail(VA_ERR_ARG, "indptr must start at 0");
    if (s->qo_indptr[s->n_sub] != s->n_subrows)
      return va_fail(VA_ERR_ARG, "qo_indptr[-1]=%d != n_subrows=%d", s->qo_indptr[s->n_sub], s->n_subrows);
  }
  for (int32_t i = 0; i < s->n_sub; ++i) {
    const int32_t nq = s->qo_indptr[i + 1] - s->qo_indptr[i];
    const int32_t ne = s->kv_indptr[i + 1] - s->kv_indptr[i];
    if (nq < 0 || ne < 0) return va_fail(VA_ERR_ARG, "indptr not monotone at sub-request %d", i);
    const int32_t len = s->seq_lens[i];
    const int64_t cap = (s->flags[i] & VA_SUB_SLOTS) ? ne : (int64_t)ne * shape->page_size;
    if (len < 0 || len > cap)
      return va_fail(VA_ERR_ARG, "sub-request %d: seq_len %d does not fit its %d kv entries", i, len, ne);
    if ((s->flags[i] & VA_SUB_CAUSAL) && nq > len)
      return va_fail(VA_ERR_ARG, "sub-request %d: causal with more query rows (%d) than keys (%d)", i, nq, len);
  }
  for (int32_t i = 0; i < s->n_subrows; ++i)
    if (s->sub_worker[i] < 0 || s->sub_worker[i] >= s->n_rows)
      return va_fail(VA_ERR_ARG, "sub_worker[%d]=%lld outside [0,%d)", i, (long long)s->sub_worker[i], s->n_rows);
  return VA_OK;
}

int resolve_kernel(const VaShape* shape, const VaPlanParams* p) {
  int kernel = p ? p->kernel : VA_KERNEL_AUTO;
  const int g = shape->num_q_heads / shape->num_kv_heads;
  const bool mfma_ok = va_mfma_supported(shape->dtype, shape->head_dim, g);
  if (kernel == VA_KERNEL_AUTO) kernel = mfma_ok ? VA_KERNEL_MFMA : VA_KERNEL_GENERIC;
  if (kernel == VA_KERNEL_MFMA && !mfma_ok) return -1;
  if (kernel != VA_KERNEL_MFMA && kernel != VA_KERNEL_GENERIC) return -1;
  return kernel;
}

// Visible tokens of a causal/non-causal sub-request for tile rows [a, b).
inline int32_t visible_end(int32_t len, int32_t nq, bool causal, int32_t b) {
  return causal ? std::min(len, len - nq + b) : len;
}

// `cap`, when given, bounds the number of entries a die may receive in each class, so that a plan
// whose real items fit the capacity still fits it after the per-die padding.
int build(const VaSubRequests* s, const VaShape* shape, const VaPlanParams* params, Built& out,
          const VaPlanCapacity* cap = nullptr) {
  int rc = check_subs(s, shape);
  if (rc) return rc;
  const int kernel = resolve_kernel(shape, params);
  if (kernel < 0) return va_fail(VA_ERR_ARG, "requested kernel family does not support this dtype/shape");
  const int g = shape->num_q_heads / shape->num_kv_heads;
  int q_tile = params && params->q_tile > 0 ? params->q_tile : 0;
  const int q_tile_max = kernel == VA_KERNEL_MFMA ? va_mfma_max_q_tile(g) : 64;
  const bool has_chain = std::any_of(s->chain, s->chain + s->n_sub, [](int32_t c) { return c >= 0; });
  if (q_tile == 0) q_tile = kernel == VA_KERNEL_MFMA ? va_mfma_default_q_tile(g, has_chain) : 1;
  if (q_tile > q_tile_max) return va_fail(VA_ERR_ARG, "q_tile %d exceeds the kernel's maximum %d", q_tile, q_tile_max);
  // Wide tiles (matrix-core path only): query tiles of more than q_tile rows are served by the
  // wide kernel, whose four waves share every K/V tile through LDS.
  int wide_tile = 0;
  if (kernel == VA_KERNEL_MFMA && !(params && params->wide_tile < 0)) {
    wide_tile = params && params->wide_tile > 0 ? params->wide_tile : va_mfma_wide_q_tile(g, shape->head_dim);
    if (wide_tile > va_mfma_wide_q_tile(g, shape->head_dim))
      return va_fail(VA_ERR_ARG, "wide_tile %d exceeds the kernel's maximum %d", wide_tile, va_mfma_wide_q_tile(g, shape->head_dim));
    if (wide_tile <= q_tile) wide_tile = 0;
  }
  // Cut n query rows into tiles: wide ones while more than q_tile rows remain, then narrow ones.
  auto cut_tiles = [&](int64_t n, std::vector<std::pair<int32_t, int32_t>>& tiles, bool allow_wide = true) {
    tiles.clear();
    int64_t a = 0;
    while (a < n) {
      const int64_t left = n - a;
      const int64_t take = (allow_wide && wide_tile && left > q_tile) ? std::min<int64_t>(left, wide_tile) : std::min<int64_t>(left, q_tile);
      tiles.emplace_back((int32_t)a, (int32_t)(a + take));
      a += take;
    }
  };
  std::vector<std::pair<int32_t, int32_t>> tiles;
  // Decode groups (readers of one shared block): whether a group is cut into wide tiles is decided per
  // group once the groups are known (group_is_wide below); narrow tiles are emitted chunk-major, so the
  // tiles that stream the same chunk run side by side and share it in L2.
  const bool wide_on_request = params && params->wide_tile > 0;
  const int target = params && params->target_items > 0 ? params->target_items
                                                        : std::max(64, 2048 / shape->num_kv_heads);
  const int gran = 64;  // chunk boundaries are multiples of this many tokens

  // ---- stand-alone sub-requests: batch readers of identical KV lists ----
  struct Group {
    int32_t rep;                  // representative sub-request
    std::vector<int32_t> subrows; // sub-row ids of all members, in order
  };
  std::vector<Group> groups;
  {
    std::unordered_map<uint64_t, std::vector<int32_t>> by_hash;  // hash -> group ids
    for (int32_t i = 0; i < s->n_sub; ++i) {
      if (s->chain[i] >= 0) continue;
      const int32_t nq = s->qo_indptr[i + 1] - s->qo_indptr[i];
      if (nq == 0 || s->seq_lens[i] == 0) continue;
      if (s->flags[i] & VA_SUB_CAUSAL)
        return va_fail(VA_ERR_ARG, "sub-request %d: causal sub-requests must belong to a chain", i);
      const int32_t b = s->kv_indptr[i], ne = s->kv_indptr[i + 1] - b;
      int32_t gid = -1;
      uint64_t h = 0;
      // readers are batched by comparing their KV lists; without a host copy of the lists
      // (kv_indices == NULL) every sub-request stands alone
      const bool can_group = q_tile > 1 && s->kv_indices && ne > 0;
      if (can_group) {
        h = (uint64_t)(uint32_t)s->kv_indices[b] * 0x9E3779B97F4A7C15ull ^
            ((uint64_t)(uint32_t)s->seq_lens[i] << 32) ^ (uint64_t)(uint32_t)(ne * 31 + s->flags[i]);
        auto it = by_hash.find(h);
        if (it != by_hash.end()) {
          for (int32_t cand : it->second) {
            const int32_t r = groups[cand].rep;
            const int32_t rb = s->kv_indptr[r], rn = s->kv_indptr[r + 1] - rb;
            if (rn == ne && s->seq_lens[r] == s->seq_lens[i] && s->flags[r] == s->flags[i] &&
                !std::memcmp(s->kv_indices + rb, s->kv_indices + b, sizeof(int32_t) * ne)) {
              gid = cand;
              break;
            }
          }
        }
      }
      if (gid < 0) {
        gid = (int32_t)groups.size();
        groups.push_back(Group{i, {}});
        if (can_group) by_hash[h].push_back(gid);
      }
      for (int32_t r = s->qo_indptr[i]; r < s->qo_indptr[i + 1]; ++r) groups[gid].subrows.push_back(r);
    }
  }

  // Wide tiles for a group.  n readers in narrow tiles stream their block ceil(n / q_tile) times (once
  // from memory, then from the die's L2), in wide tiles wide_tile / q_tile times less often -- but wide
  // tiles run in a launch of their own, whose workgroups each stage a whole tile of queries and write a
  // whole tile of partial states.  Measured at 16 q / 4 kv heads, head_dim 256, bf16 (q_tile 4, wide_tile
  // 32 readers): 64 readers of an 8192-token block save 0.47 GB of such re-reads and the launch costs what
  // they cost (401 -> 403 us); 128 readers of it save 0.94 GB (797 -> 759 us), 64 readers of a 32768-token
  // block 1.9 GB (494 -> 443 us).  So: on request always; otherwise (plans of free size only) when the
  // groups that would each save a fair share together save more than 0.64 GB.
  std::vector<char> group_is_wide(groups.size(), wide_on_request && wide_tile > 0);
  if (!wide_on_request && wide_tile > 0 && !cap) {
    const int64_t token_bytes = 2ll * shape->num_kv_heads * shape->head_dim * (shape->dtype == VA_F32 ? 4 : 2);
    constexpr int64_t kWorthALaunch = 640ll << 20, kFairShare = kWorthALaunch / 8;
    std::vector<int64_t> saved(groups.size(), 0);
    int64_t total = 0;
    for (size_t gi = 0; gi < groups.size(); ++gi) {
      const int64_t n = (int64_t)groups[gi].subrows.size();
      if (n <= q_tile) continue;
      cut_tiles(n, tiles, true);
      saved[gi] = ((n + q_tile - 1) / q_tile - (int64_t)tiles.size()) * s->seq_lens[groups[gi].rep] * token_bytes;
      if (saved[gi] >= kFairShare) total += saved[gi];
    }
    if (total >= kWorthALaunch)
      for (size_t gi = 0; gi < groups.size(); ++gi) group_is_wide[gi] = saved[gi] >= kFairShare;
  }

  // ---- chains: sub-requests of one prefill request, in table order ----
  std::vector<std::vector<int32_t>> chains;
  {
    std::unordered_map<int32_t, int32_t> chain_index;
    for (int32_t i = 0; i < s->n_sub; ++i) {
      const int32_t c = s->chain[i];
      if (c < 0) continue;
      auto it = chain_index.find(c);
      if (it == chain_index.end()) {
        it = chain_index.emplace(c, (int32_t)chains.size()).first;
        chains.emplace_back();
      }
      chains[it->second].push_back(i);
    }
    for (auto& ch : chains) {
      const int32_t nq = s->qo_indptr[ch[0] + 1] - s->qo_indptr[ch[0]];
      for (int32_t m : ch) {
        if (s->qo_indptr[m + 1] - s->qo_indptr[m] != nq)
          return va_fail(VA_ERR_ARG, "chain %d: members disagree on the number of query rows", s->chain[m]);
        for (int32_t r = 0; r < nq; ++r)
          if (s->sub_worker[s->qo_indptr[m] + r] != s->sub_worker[s->qo_indptr[ch[0]] + r])
            return va_fail(VA_ERR_ARG, "chain %d: members disagree on output rows", s->chain[m]);
      }
    }
  }

  // ---- total tokens -> chunk size for split-KV ----
  int64_t total_tokens = 0;
  for (auto& gr : groups) {
    cut_tiles((int64_t)gr.subrows.size(), tiles, group_is_wide[&gr - &groups[0]]);
    total_tokens += (int64_t)tiles.size() * s->seq_lens[gr.rep];
  }
  int64_t chain_tiles = 0, chain_tokens = 0, wide_chain_tokens = 0;
  for (auto& ch : chains) {
    const int32_t nq = s->qo_indptr[ch[0] + 1] - s->qo_indptr[ch[0]];
    cut_tiles(nq, tiles);
    for (auto& tl : tiles) {
      ++chain_tiles;
      int64_t walked = 0;
      for (int32_t m : ch) walked += std::max(0, visible_end(s->seq_lens[m], nq, s->flags[m] & VA_SUB_CAUSAL, tl.second));
      chain_tokens += walked;
      if (tl.second - tl.first > q_tile) wide_chain_tokens += walked;
    }
  }
  // (the chunk cuts the runs of stand-alone sub-requests only -- chains are cut by budgets of their own,
  // below -- so it is sized from their tokens alone: in a mixed batch the prefill chunks' long walks
  // would otherwise triple it, and the decode items would run in two long rounds instead of four short ones)
  int32_t kv_chunk = params && params->kv_chunk > 0 ? round_up(params->kv_chunk, gran) : 0;
  if (kv_chunk == 0) {
    const int64_t per_item = (total_tokens + target - 1) / target;
    // No chunk under four granules as a rule (an item's set-up is worth a few hundred tokens) -- unless the
    // launch holds so few tokens that such chunks would leave most of the machine idle: then the time of
    // the launch is the walk of ONE item, a chain of dependent trips to memory, and shorter walks side by
    // side (down to one granule) are what shortens it.
    const int64_t spread = (total_tokens + (256 / shape->num_kv_heads) - 1) / std::max(1, 256 / shape->num_kv_heads);
    const int64_t least = std::min<int64_t>(4 * gran, std::max<int64_t>(gran, round_up(spread, gran)));
    kv_chunk = round_up(std::max<int64_t>(per_item, least), gran);
  }

  out.kernel = kernel;
  out.q_tile = q_tile;
  out.kv_chunk = kv_chunk;
  out.wide_tile = wide_tile;

  // contributions per output row decide direct-vs-partial
  std::vector<int32_t> row_count(s->n_rows, 0);
  struct Pending {
    int32_t item;
    std::vector<int32_t> rows;  // output row per tile row
  };
  std::vector<Pending> pend;

  int32_t next_unit = 0;
  auto emit = [&](int32_t n_q, const std::vector<Link>& links, std::vector<int32_t>&& rows, int32_t unit = -1,
                  int32_t slot = -1) {
    int32_t tokens = 0;
    for (auto& l : links) tokens += l.tok_end - l.tok_begin;
    Item it{(int32_t)out.links.size(), (int32_t)links.size(), n_q, -1, tokens, n_q > q_tile ? 1 : 0,
            unit >= 0 ? unit : next_unit++, n_q > q_tile ? slot : -1};
    out.links.insert(out.links.end(), links.begin(), links.end());
    for (int32_t r : rows) ++row_count[r];
    pend.push_back(Pending{(int32_t)out.items.size(), std::move(rows)});
    out.items.push_back(it);
  };

  // Wide decode tiles run in their own launch (one workgroup per CU at a time), so their
  // runs are cut finer: enough chunks for about one workgroup per CU.
  int64_t wide_group_tokens = 0;
  for (auto& gr : groups) {
    cut_tiles((int64_t)gr.subrows.size(), tiles, group_is_wide[&gr - &groups[0]]);
    for (auto& tl : tiles)
      if (tl.second - tl.first > q_tile) wide_group_tokens += s->seq_lens[gr.rep];
  }
  const int wide_items_wanted = std::max(1, 256 / shape->num_kv_heads);
  const int32_t wide_chunk = std::min<int32_t>(
      kv_chunk, round_up(std::max<int64_t>((wide_group_tokens + wide_items_wanted - 1) / wide_items_wanted, 2 * gran), gran));

  for (auto& gr : groups) {
    const int32_t rep = gr.rep;
    const int32_t len = s->seq_lens[rep];
    cut_tiles((int64_t)gr.subrows.size(), tiles, group_is_wide[&gr - &groups[0]]);
    // A run that a single query tile reads is fetched once per kv head and never again: its rows are
    // requested as lines to evict first, so that they stream through the die's L2 without pushing
    // out the rows that several tiles read side by side (a block shared by many views).
    const int32_t lflags = VA_LINK_INDIRECT | ((s->flags[rep] & VA_SUB_SLOTS) ? VA_LINK_SLOTS : 0) |
                           (tiles.size() == 1 ? VA_LINK_ONCE : 0);
    std::vector<int32_t> tile_qref;
    for (auto& tl : tiles) {
      tile_qref.push_back((int32_t)out.qrefs.size());
      out.qrefs.insert(out.qrefs.end(), gr.subrows.begin() + tl.first, gr.subrows.begin() + tl.second);
    }
    auto emit_range = [&](size_t ti, int32_t t0, int32_t t1, int32_t unit = -1) {
      const size_t a = tiles[ti].first, b = tiles[ti].second;
      std::vector<int32_t> rows;
      for (size_t r = a; r < b; ++r) rows.push_back((int32_t)s->sub_worker[gr.subrows[r]]);
      emit((int32_t)(b - a), {Link{s->kv_indptr[rep], t0, t1, tile_qref[ti], VA_NO_CAUSAL, lflags}}, std::move(rows), unit);
    };
    auto chunk_len = [&](int32_t chunk) {
      const int32_t n_chunks = (len + chunk - 1) / chunk;
      return round_up((len + n_chunks - 1) / n_chunks, gran);
    };
    // narrow tiles: chunk-major; wide tiles: their own (finer) chunking
    const int32_t per = chunk_len(kv_chunk);
    // The last chunk of a run is cut in two: every run then contributes short items, which the
    // launch order puts last, so the launch does not end on a round of full-length items.
    std::vector<int32_t> cuts{0};
    for (int32_t t0 = per; t0 < len; t0 += per) cuts.push_back(t0);
    if (len - cuts.back() >= 4 * gran) cuts.push_back(cuts.back() + round_up((len - cuts.back()) / 2, gran));
    cuts.push_back(len);
    for (size_t ci = 0; ci + 1 < cuts.size(); ++ci) {
      if (cuts[ci] >= cuts[ci + 1]) continue;
      const int32_t unit = next_unit++;  // the narrow tiles of one chunk: same die, side by side
      for (size_t ti = 0; ti < tiles.size(); ++ti)
        if (tiles[ti].second - tiles[ti].first <= q_tile) emit_range(ti, cuts[ci], cuts[ci + 1], unit);
    }
    const int32_t per_w = chunk_len(wide_chunk);
    for (size_t ti = 0; ti < tiles.size(); ++ti)
      if (tiles[ti].second - tiles[ti].first > q_tile)
        for (int32_t t0 = 0; t0 < len; t0 += per_w) emit_range(ti, t0, std::min(len, t0 + per_w));
  }

  // Chains.  When the tiles of all chains are many (several rounds of one workgroup per CU) every
  // tile is one work item and the hardware hands them out as CUs fall free.  When they are few --
  // a handful of prefill chunks in a continuous batch, whose views differ in length by a factor
  // of thirty -- whole tiles cannot fill the machine evenly, so the walks of the wide tiles, laid end
  // to end, are cut into equal budgets instead, for a launch of one workgroup ("slot") per CU.  A slot
  // runs its pieces one after the other; a tile cut in pieces yields partial states that the merge
  // kernel folds.  Every slot then costs the same (the cost of a wide tile is its tokens, all its rows
  // share each K/V tile, plus a set-up per segment) and the launch is one even round, where 2.25
  // rounds of uneven items used to take the time of three.
  // Narrow tiles of chains (the last rows of a request) are cut by a token budget, one item a piece.
  const int64_t slots_wanted = std::max(1, 256 / shape->num_kv_heads);
  int64_t chain_budget = INT64_MAX;
  // A piece of a wide tile stages its query tile once per segment of the view it walks (the query is
  // rotated for every block anew), which costs about as much as walking `seg_cost` tokens: the packing
  // charges every (piece, segment) to the room it fills.  A remainder that would cost less than
  // `min_piece` stays with the piece before it.
  const int32_t seg_cost = 10 * gran;
  const int32_t min_piece = 6 * gran;
  if (chain_tiles > 0 && chain_tiles < 4 * slots_wanted) {
    // The budget cuts the walks of the NARROW chain tiles only (wide tiles are packed in bundles by
    // budgets of their own, below), so it is their tokens that size it: a narrow tile of t tokens
    // yields at most t / budget + 1 pieces, all narrow tiles together at most `want` <= target more
    // pieces than there are tiles -- which is the bound a fixed-capacity plan relies on.  (Sized from
    // the wide tiles' tokens, a one-row chunk over a long view beside a short wide chunk was cut
    // into hundreds of pieces.)
    const int64_t want = std::max<int64_t>(1, std::min<int64_t>(target, slots_wanted));
    const int64_t narrow_chain_tokens = chain_tokens - wide_chain_tokens;
    chain_budget = std::max<int64_t>((narrow_chain_tokens + want - 1) / want, 16 * gran);
  }
  // cuts inside a segment keep to multiples of 16 tokens where the kernels profit (pages of 16
  // tokens or more: a piece that starts on such a boundary is fetched with uniform loads)
  const bool align_cuts = shape->page_size >= 16 && (shape->page_size & (shape->page_size - 1)) == 0;
  const bool pack = chain_budget != INT64_MAX;
  const int32_t slot_room = pack ? round_up(chain_budget + (align_cuts ? 15 : 0), gran) : 0;  // narrow tiles of chains

  // Wide tiles are packed in LOCKSTEP BUNDLES.  The query tiles of one chunk all stream the chunk's
  // view; packed one after the other into slots they would walk it at different places at any one
  // time, and each would fetch it from HBM for itself.  So the workgroup slots are taken in groups of
  // `lanes` (the slots that run side by side on one die), up to `lanes` neighbouring tiles of a chain
  // form a bundle, and a bundle's walk is cut ONCE, for all its tiles alike: the lanes of a group walk
  // the same tokens at the same time, one of them fetches a K/V tile from HBM and the others find
  // it in the die's L2.  A bundle of m <= lanes / 2 tiles has its walk cut into f = lanes / m parts
  // that run side by side (lane = part * m + tile), so a short chain still fills the group.
  const int64_t want_slots = pack ? std::max<int64_t>(1, std::min<int64_t>(target, slots_wanted)) : 1;
  const int32_t lanes = (int32_t)std::max<int64_t>(1, want_slots / kXcds);
  const int32_t groups_wanted = (int32_t)std::min<int64_t>(want_slots, kXcds);
  struct Bundle {
    int32_t first = 0, m = 0, f = 1;  // tiles [first, first + m) of the chain; f parts side by side
    int32_t part = 0;                 // walk positions per part
    std::vector<int32_t> subs;        // the chain members any tile of the bundle sees
    std::vector<int32_t> off;         // walk position of each member's first token
    std::vector<int32_t> starts;      // positions within a part where some lane starts a member (sorted)
    // What positions [x0, x1) cost the slowest lane of the bundle: its tokens, and a set-up (worth
    // `seg` tokens) for the segment it is in at x0 and for every member that starts inside its range.
    int64_t cost(int64_t x0, int64_t x1, int32_t seg) const {
      int64_t most = 0;
      for (int32_t g = 0; g < f; ++g) {
        int64_t n = 1;
        for (int32_t o : off) {
          const int64_t x = (int64_t)o - (int64_t)g * part;
          n += x > x0 && x < x1;
        }
        most = std::max(most, n);
      }
      return (x1 - x0) + seg * most;
    }
  };
  auto make_bundle = [&](const std::vector<int32_t>& ch, int32_t nq, int32_t first, int32_t m) {
    Bundle bd;
    bd.first = first;
    bd.m = m;
    const int32_t b_last = tiles[first + m - 1].second;  // the last tile sees most
    int64_t pos = 0;
    for (int32_t sub : ch) {
      const int32_t vis = visible_end(s->seq_lens[sub], nq, s->flags[sub] & VA_SUB_CAUSAL, b_last);
      if (vis <= 0) continue;
      bd.subs.push_back(sub);
      bd.off.push_back((int32_t)pos);
      pos += align_cuts ? round_up(vis, 16) : vis;  // every member starts at a multiple of 16: so do all cuts within it
    }
    if (pos == 0) return bd;
    bd.f = (int32_t)std::max<int64_t>(1, std::min<int64_t>(lanes / m, pos / (8 * gran)));
    bd.part = bd.f == 1 ? (int32_t)pos : round_up((pos + bd.f - 1) / bd.f, 16);
    for (int32_t g = 0; g < bd.f; ++g)
      for (int32_t o : bd.off) {
        const int64_t x = (int64_t)o - (int64_t)g * bd.part;
        if (x > 0 && x < bd.part) bd.starts.push_back((int32_t)x);
      }
    std::sort(bd.starts.begin(), bd.starts.end());
    bd.starts.erase(std::unique(bd.starts.begin(), bd.starts.end()), bd.starts.end());
    return bd;
  };
  // bundles of a chain's tile list (as cut_tiles left it in `tiles`)
  auto bundles_of = [&](const std::vector<int32_t>& ch, int32_t nq, std::vector<Bundle>& out_bundles) {
    out_bundles.clear();
    int32_t n_wide_tiles = 0;
    while (n_wide_tiles < (int32_t)tiles.size() && tiles[n_wide_tiles].second - tiles[n_wide_tiles].first > q_tile) ++n_wide_tiles;
    for (int32_t first = 0; first < n_wide_tiles; first += lanes) {
      Bundle bd = make_bundle(ch, nq, first, std::min(lanes, n_wide_tiles - first));
      if (bd.part > 0) out_bundles.push_back(std::move(bd));
    }
  };
  std::vector<Bundle> bundles;
  int64_t wide_walk = 0, wide_cost = 0;  // positions of all bundles; with their set-ups
  if (pack) {
    for (auto& ch : chains) {
      const int32_t nq = s->qo_indptr[ch[0] + 1] - s->qo_indptr[ch[0]];
      cut_tiles(nq, tiles);
      bundles_of(ch, nq, bundles);
      for (auto& bd : bundles) {
        wide_walk += bd.part;
        wide_cost += bd.cost(0, bd.part, seg_cost);
      }
    }
  }
  // The room of a new group is the even share of what is still to be placed over the groups still
  // to be opened, so that a group closed early (less than min_piece of its room left) or run over (a
  // bundle's short remainder kept with the piece before it) is made up for by the groups after it,
  // and their number never exceeds the number wanted.
  const int64_t group_budget = pack ? std::max<int64_t>((wide_walk + groups_wanted - 1) / groups_wanted, 16 * gran) : 0;
  int64_t groups_left = pack ? std::max<int64_t>(1, (wide_walk + group_budget - 1) / group_budget) : 0;
  // What is still to be placed, set-ups included: every segment of every bundle, and one more for
  // every group boundary (it falls inside some segment, which is then staged on both sides).  An
  // estimate on the high side leaves the LAST group short, one on the low side would leave it long --
  // and the longest group is the time of the launch.
  int64_t wide_left = wide_cost + seg_cost * (groups_left - 1);
  auto next_wide_room = [&]() -> int64_t {
    if (groups_left <= 1) return INT32_MAX;  // the last group takes whatever is left
    const int64_t share = std::max<int64_t>((wide_left + groups_left - 1) / groups_left, seg_cost + min_piece);
    --groups_left;
    return round_up(share + (align_cuts ? 15 : 0), 16);
  };
  int32_t wide_group = 0;                              // the group being filled
  int64_t wide_room = pack ? next_wide_room() : 0;  // the room left in it: it carries over from bundle to bundle
  // Cut a bundle's walk where the room of the current group ends; close(x0, x1, group) takes every piece.
  auto cut_bundle = [&](const Bundle& bd, auto&& close) {
    // no tiny last piece: a remainder that would cost less than `small` stays with the piece before it
    // (small next to a group's share: the group that keeps it runs that much longer than the others)
    const int64_t small = std::min<int64_t>(min_piece + seg_cost, group_budget / 8);
    int64_t x = 0;
    while (x < bd.part) {
      if (wide_room < seg_cost + min_piece) {  // too little left for a piece worth its set-up
        ++wide_group;
        wide_room = next_wide_room();
      }
      // the furthest end the room pays for: between two starts the cost grows by one per position
      int64_t x1 = bd.part;
      if (bd.cost(x, bd.part, seg_cost) > wide_room) {
        int64_t from = x;  // cost(x, from) fits
        for (size_t i = 0; i <= bd.starts.size(); ++i) {
          const int64_t to = i < bd.starts.size() ? bd.starts[i] : bd.part;
          if (to <= x) continue;
          const int64_t c = bd.cost(x, to, seg_cost);
          if (c <= wide_room) {
            from = to;
            continue;
          }
          x1 = std::max(from, to - (c - wide_room));
          break;
        }
        if (align_cuts) x1 = x1 / 16 * 16;  // x and every start are multiples of 16
        if (x1 <= x) x1 = std::min<int64_t>(bd.part, x + 16);
        if (x1 < bd.part && bd.cost(x1, bd.part, seg_cost) < small) x1 = bd.part;
      }
      close(x, x1, wide_group);
      const int64_t c = bd.cost(x, x1, seg_cost);
      wide_room -= c;
      wide_left -= c;
      x = x1;
    }
  };

  // Cut a narrow tile's walk (links in walking order) into budgets of `slot_room` tokens, one item a
  // piece; a remainder of less than min_piece stays with the piece before it.
  auto cut_walk = [&](const std::vector<Link>& walk, auto&& close) {
    int32_t room = slot_room;
    int64_t left = 0;  // tokens of the walk not yet in a piece
    for (auto& l : walk) left += l.tok_end - l.tok_begin;
    auto fit_room = [&]() {
      if (left > room && left - room < min_piece) room = (int32_t)left;
    };
    fit_room();
    std::vector<Link> cur;
    auto close_piece = [&]() {
      if (!cur.empty()) close(cur);
      cur.clear();
    };
    for (auto l : walk) {
      const bool aligned = align_cuts && !(l.flags & VA_LINK_SLOTS);
      while (l.tok_begin < l.tok_end) {
        int32_t take = std::min(room, l.tok_end - l.tok_begin);
        if (aligned && take < l.tok_end - l.tok_begin) take = take / 16 * 16;  // l.tok_begin is a multiple of 16: segments start at 0, cuts keep it so
        if (take <= 0) {  // no room left to go on here: the piece ends
          if (!cur.empty() && left < min_piece) {  // ... unless what is left is too little for a piece of its own
            room = (int32_t)left;
            continue;
          }
          close_piece();
          room = slot_room;
          fit_room();
          continue;
        }
        Link piece = l;
        piece.tok_end = l.tok_begin + take;
        cur.push_back(piece);
        l.tok_begin += take;
        left -= take;
        room -= take;
        if (room <= 0 && left > 0) {
          if (left < min_piece) {  // too little for a piece of its own: it stays with this one
            room = (int32_t)left;
            continue;
          }
          close_piece();
          room = slot_room;
          fit_room();
        }
      }
    }
    close_piece();
  };

  for (auto& ch : chains) {
    const int32_t nq = s->qo_indptr[ch[0] + 1] - s->qo_indptr[ch[0]];
    cut_tiles(nq, tiles);
    // the links of tile rows [a, b), clipped to walk positions [lo, hi) of a bundle (all of them without one)
    auto tile_links = [&](int32_t a, int32_t b, const Bundle* bd, int64_t lo, int64_t hi) {
      std::vector<Link> links;
      size_t k = 0;
      for (int32_t m : ch) {
        const bool causal = s->flags[m] & VA_SUB_CAUSAL;
        const int32_t len = s->seq_lens[m];
        int32_t t0 = 0, t1 = visible_end(len, nq, causal, b);
        if (bd) {
          if (k >= bd->subs.size() || bd->subs[k] != m) continue;  // no tile of the bundle sees this member
          const int64_t off = bd->off[k++];
          t0 = (int32_t)(std::max<int64_t>(lo, off) - off);
          t1 = (int32_t)(std::min<int64_t>(hi, off + t1) - off);
        }
        if (t1 <= t0) continue;
        const int32_t cbase = causal ? len - nq + a : VA_NO_CAUSAL;
        links.push_back(Link{s->kv_indptr[m], t0, t1, s->qo_indptr[m] + a, cbase,
                             (s->flags[m] & VA_SUB_SLOTS) ? VA_LINK_SLOTS : 0});
      }
      return links;
    };
    auto tile_rows = [&](int32_t a, int32_t b) {
      std::vector<int32_t> rows;
      for (int32_t r = a; r < b; ++r) rows.push_back((int32_t)s->sub_worker[s->qo_indptr[ch[0]] + r]);
      return rows;
    };
    if (pack) {
      bundles_of(ch, nq, bundles);
      for (auto& bd : bundles) {
        cut_bundle(bd, [&](int64_t x0, int64_t x1, int32_t group) {
          for (int32_t g = 0; g < bd.f; ++g)
            for (int32_t j = 0; j < bd.m; ++j) {
              const int32_t a = tiles[bd.first + j].first, b = tiles[bd.first + j].second;
              const std::vector<Link> links = tile_links(a, b, &bd, (int64_t)g * bd.part + x0, (int64_t)g * bd.part + x1);
              if (!links.empty()) emit(b - a, links, tile_rows(a, b), -1, group * lanes + g * bd.m + j);
            }
        });
      }
    }
    for (auto& tl : tiles) {
      const int32_t a = tl.first, b = tl.second;
      if (pack && b - a > q_tile) continue;  // packed above
      const std::vector<Link> all = tile_links(a, b, nullptr, 0, 0);
      if (all.empty()) continue;
      if (!pack) {
        emit(b - a, all, tile_rows(a, b));
        continue;
      }
      cut_walk(all, [&](const std::vector<Link>& cur) { emit(b - a, cur, tile_rows(a, b)); });
    }
  }

  // ---- partial slots and the per-row merge lists ----
  std::vector<std::vector<int32_t>> parts_of_row(s->n_rows);
  for (auto& p : pend) {
    bool direct = true;
    for (int32_t r : p.rows) direct = direct && row_count[r] == 1;
    Item& it = out.items[p.item];
    if (direct) {
      it.part_base = -1;
    } else {
      it.part_base = out.n_partials;
      for (size_t i = 0; i < p.rows.size(); ++i) parts_of_row[p.rows[i]].push_back(out.n_partials + (int32_t)i);
      out.n_partials += (int32_t)p.rows.size();
    }
  }
  out.row_indptr.assign(s->n_rows + 1, 0);
  out.row_flags.assign(s->n_rows, 0);
  for (int32_t r = 0; r < s->n_rows; ++r) {
    out.row_indptr[r + 1] = out.row_indptr[r] + (int32_t)parts_of_row[r].size();
    out.row_ids.insert(out.row_ids.end(), parts_of_row[r].begin(), parts_of_row[r].end());
    if (row_count[r] == 0) out.row_flags[r] = VA_ROW_EMPTY;
    else if (parts_of_row[r].empty()) out.row_flags[r] = VA_ROW_DIRECT;
  }

  // Launch order.  Wide items first (their own launch), then narrow ones.  The hardware hands
  // workgroup b of a launch to die b % 8, and each die has its own L2, so within a class:
  //   * units (the tiles that stream one K/V chunk) are dealt to the 8 dies, heaviest first, each
  //     to the least loaded die, and stay together there: the chunk is fetched from HBM by one
  //     tile and found in that die's L2 by the others;
  //   * after a first round of mixed sizes a die runs its units longest item first, so the tail of
  //     the launch is made of short items;
  //   * position p of the class holds entry p / 8 of die p % 8; dies with fewer entries are
  //     padded with empty items (n_q = 0, the kernels return at once), which also keeps the
  //     class a multiple of 8 long so the next kv head starts on die 0 again.
  std::vector<Item> sorted;
  sorted.reserve(out.items.size() + 2 * kXcds);
  for (int kind = 1; kind >= 0; --kind) {
    struct Unit {
      int64_t cost = 0, item_cost = 0;
      std::vector<int32_t> members;
    };
    std::vector<Unit> units;
    std::unordered_map<int32_t, int32_t> unit_index;
    for (int32_t i = 0; i < (int32_t)out.items.size(); ++i) {
      const Item& it = out.items[i];
      if (it.kind != kind) continue;
      auto at = unit_index.find(it.unit);
      if (at == unit_index.end()) {
        at = unit_index.emplace(it.unit, (int32_t)units.size()).first;
        units.emplace_back();
      }
      Unit& u = units[at->second];
      const int64_t cost = it.tokens;  // a tile streams its tokens once whatever its row count
      u.cost += cost;
      u.item_cost = std::max(u.item_cost, cost);
      u.members.push_back(i);
    }
    if (units.empty()) continue;
    if (kind == 1 && std::any_of(out.items.begin(), out.items.end(), [](const Item& it) { return it.kind == 1 && it.slot >= 0; })) {
      // Packed wide pieces: slot id = group * lanes + lane.  Every group costs the same, and its
      // lanes walk the same tokens at the same pace: group g goes to die g % 8 as a whole, where
      // the K/V its lanes share is fetched from HBM once and found in that die's L2 by the others.
      // Wide items outside the packing get slots of their own on the die with the fewest.
      std::vector<std::vector<int32_t>> by_slot;
      for (int32_t i = 0; i < (int32_t)out.items.size(); ++i) {
        const Item& it = out.items[i];
        if (it.kind != 1 || it.slot < 0) continue;
        if ((size_t)it.slot >= by_slot.size()) by_slot.resize(it.slot + 1);
        by_slot[it.slot].push_back(i);
      }
      std::vector<std::vector<int32_t>> die_slots[kXcds];
      for (size_t k = 0; k < by_slot.size(); ++k)
        if (!by_slot[k].empty()) die_slots[(k / lanes) % kXcds].push_back(std::move(by_slot[k]));
      for (int32_t i = 0; i < (int32_t)out.items.size(); ++i) {
        if (out.items[i].kind != 1 || out.items[i].slot >= 0) continue;
        int least = 0;
        for (int d = 1; d < kXcds; ++d)
          if (die_slots[d].size() < die_slots[least].size()) least = d;
        die_slots[least].push_back({i});
      }
      size_t per_die = 0;
      for (int d = 0; d < kXcds; ++d) per_die = std::max(per_die, die_slots[d].size());
      // slot k of the launch runs on die k % 8 (the kernel maps its workgroups that way)
      out.wide_slots.assign(1, 0);
      for (size_t k = 0; k < per_die * kXcds; ++k) {
        const auto& on_die = die_slots[k % kXcds];
        if (k / kXcds < on_die.size())
          for (int32_t m : on_die[k / kXcds]) sorted.push_back(out.items[m]);
        out.wide_slots.push_back((int32_t)sorted.size());
      }
      const Item padding{0, 0, 0, -1, 0, 1, -1, -1};
      // (outside every slot; a launch has at least as many items as slots)
      while (sorted.size() % kXcds || sorted.size() + 1 < out.wide_slots.size()) sorted.push_back(padding);
      out.n_wide = (int32_t)sorted.size();
      continue;
    }
    std::vector<int32_t> by_cost(units.size());
    std::iota(by_cost.begin(), by_cost.end(), 0);
    std::stable_sort(by_cost.begin(), by_cost.end(), [&](int32_t x, int32_t y) { return units[x].cost > units[y].cost; });
    int64_t load[kXcds] = {0};
    int64_t room[kXcds];
    std::fill(room, room + kXcds, cap ? (kind ? cap->max_wide_items : cap->max_items) / kXcds : INT32_MAX);
    std::vector<int32_t> die_units[kXcds];
    // least loaded die that still has room for `n` entries (-1: none)
    auto pick_die = [&](int64_t n) {
      int best = -1;
      for (int d = 0; d < kXcds; ++d)
        if (room[d] >= n && (best < 0 || load[d] < load[best])) best = d;
      return best;
    };
    auto place = [&](int32_t u, int die) {
      die_units[die].push_back(u);
      load[die] += units[u].cost;
      room[die] -= (int64_t)units[u].members.size();
    };
    for (size_t k = 0; k < by_cost.size(); ++k) {
      const int32_t u = by_cost[k];
      int die = pick_die((int64_t)units[u].members.size());
      if (die >= 0) {
        place(u, die);
        continue;
      }
      // No die has room for the whole unit (fixed capacity only): its tiles go one by one to dies
      // that have room, at the price of fetching the chunk once per die.  When even that fails the
      // plan is over capacity, which the serializer reports; keep every item in the launch order.
      const std::vector<int32_t> members = units[u].members;
      units[u].members.clear();
      units[u].cost = units[u].item_cost = 0;
      for (int32_t m : members) {
        Unit single;
        single.cost = single.item_cost = out.items[m].tokens;
        single.members.push_back(m);
        units.push_back(single);
        die = pick_die(1);
        if (die < 0) die = (int)(std::min_element(load, load + kXcds) - load);
        place((int32_t)units.size() - 1, die);
      }
    }
    std::vector<int32_t> die_items[kXcds];
    size_t depth = 0;
    for (int d = 0; d < kXcds; ++d) {
      std::stable_sort(die_units[d].begin(), die_units[d].end(),
                       [&](int32_t x, int32_t y) { return units[x].item_cost > units[y].item_cost; });
      // Workgroups that start together and stream the same number of tokens also finish together,
      // and while they all write results and set up their next item the memory system idles.  So
      // the first round of a die (the items that start at once: 64 workgroup slots) is a spread
      // sample of all its sizes; their staggered ends keep the later rounds out of step.
      const size_t n_u = die_units[d].size();
      const size_t first_round = std::min<size_t>(n_u, std::max(1, 64 / shape->num_kv_heads));
      if (first_round > 1 && n_u > first_round) {
        std::vector<int32_t> head, rest;
        std::vector<char> picked(n_u, 0);
        for (size_t k = 0; k < first_round; ++k) picked[k * (n_u - 1) / (first_round - 1)] = 1;
        for (size_t i = 0; i < n_u; ++i) (picked[i] ? head : rest).push_back(die_units[d][i]);
        head.insert(head.end(), rest.begin(), rest.end());
        die_units[d].swap(head);
      }
      for (int32_t u : die_units[d])
        die_items[d].insert(die_items[d].end(), units[u].members.begin(), units[u].members.end());
      depth = std::max(depth, die_items[d].size());
    }
    const Item padding{0, 0, 0, -1, 0, kind, -1, -1};
    for (size_t slot = 0; slot < depth; ++slot)
      for (int d = 0; d < kXcds; ++d)
        sorted.push_back(slot < die_items[d].size() ? out.items[die_items[d][slot]] : padding);
    if (kind == 1) {  // one workgroup per wide item
      out.n_wide = (int32_t)sorted.size();
      out.wide_slots.resize(out.n_wide + 1);
      std::iota(out.wide_slots.begin(), out.wide_slots.end(), 0);
    }
  }
  out.items.swap(sorted);
  if (out.wide_slots.empty()) out.wide_slots.assign(1, 0);
  return VA_OK;
}

void fill_counts(const Built& b, const VaSubRequests* s, const VaShape* shape, VaPlanCounts* c) {
  c->kernel = b.kernel;
  c->q_tile = b.q_tile;
  c->kv_chunk = b.kv_chunk;
  c->wide_tile = b.wide_tile;
  c->n_wide_items = b.n_wide;
  c->n_items = (int32_t)b.items.size();
  c->n_links = (int32_t)b.links.size();
  c->n_qrefs = (int32_t)b.qrefs.size();
  c->n_partials = b.n_partials;
  c->n_row_parts = (int32_t)b.row_ids.size();
  c->n_wide_slots = (int32_t)b.wide_slots.size() - 1;
  c->plan_words = VA_PLAN_HEADER_WORDS + c->n_items * VA_ITEM_WORDS + c->n_links * VA_LINK_WORDS +
                  2 * c->n_qrefs + (s->n_rows + 1) + c->n_row_parts + s->n_rows + (c->n_wide_slots + 1);
  c->workspace_bytes = va_workspace_bytes_for(b.n_partials, shape->num_q_heads, shape->head_dim);
}

}  // namespace

extern "C" int va_plan_count(const VaSubRequests* subs, const VaShape* shape, const VaPlanParams* params,
                             VaPlanCounts* counts) {
  if (!counts) return va_fail(VA_ERR_ARG, "null counts");
  Built b;
  int rc = build(subs, shape, params, b);
  if (rc) return rc;
  fill_counts(b, subs, shape, counts);
  return VA_OK;
}

// Serialise a built plan.  With `cap` the sections sit at offsets that depend on the capacity
// alone and the item lists are padded to it; otherwise they are packed.
static int write_plan(const Built& b, const VaSubRequests* subs, const VaShape* shape, const VaPlanCapacity* cap,
                      int32_t* plan_host, int64_t plan_capacity_words, VaPlanCounts* counts) {
  VaPlanCounts c;
  fill_counts(b, subs, shape, &c);
  const int32_t n_narrow = c.n_items - c.n_wide_items;
  int32_t cap_wide = c.n_wide_items, cap_narrow = n_narrow, cap_links = c.n_links, cap_qrefs = c.n_qrefs,
          cap_row_parts = c.n_row_parts, cap_rows = subs->n_rows, cap_partials = c.n_partials;
  if (cap) {
    if (cap->max_items % 8 || cap->max_wide_items % 8 || cap->max_items < 0 || cap->max_wide_items < 0)
      return va_fail(VA_ERR_ARG, "capacity: item counts must be non-negative multiples of 8");
#define VA_FITS(have, room, what) \
  if ((have) > (room)) return va_fail(VA_ERR_CAPACITY, "plan exceeds the fixed capacity: %d %s, room for %d", (have), what, (room));
    VA_FITS(c.n_wide_items, cap->max_wide_items, "wide work items")
    VA_FITS(n_narrow, cap->max_items, "work items")
    VA_FITS(c.n_links, cap->max_links, "links")
    VA_FITS(c.n_qrefs, cap->max_qrefs, "query references")
    VA_FITS(c.n_partials, cap->max_partials, "partial states")
    VA_FITS(c.n_row_parts, cap->max_row_parts, "row parts")
    VA_FITS(subs->n_rows, cap->max_rows, "rows")
#undef VA_FITS
    cap_wide = cap->max_wide_items; cap_narrow = cap->max_items; cap_links = cap->max_links; cap_qrefs = cap->max_qrefs;
    cap_row_parts = cap->max_row_parts; cap_rows = cap->max_rows; cap_partials = cap->max_partials;
    c.n_items = cap_wide + cap_narrow;
    c.n_wide_items = cap_wide;
    c.n_wide_slots = cap_wide;  // a fixed plan launches one workgroup per wide item it has room for
    c.n_links = cap_links;
    c.n_qrefs = cap_qrefs;
    c.n_partials = cap_partials;
    c.n_row_parts = cap_row_parts;
    c.plan_words = (int32_t)va_plan_fixed_words(cap);
    c.workspace_bytes = va_workspace_bytes_for(cap_partials, shape->num_q_heads, shape->head_dim);
  }
  if (plan_capacity_words < c.plan_words) {
    if (counts) *counts = c;  // the caller learns the size it needs
    return va_fail(VA_ERR_CAPACITY, "plan needs %d words, buffer holds %lld", c.plan_words,
                   (long long)plan_capacity_words);
  }
  int32_t* h = plan_host;
  std::memset(h, 0, sizeof(int32_t) * (size_t)c.plan_words);
  int32_t off = VA_PLAN_HEADER_WORDS;
  h[VA_H_MAGIC] = VA_PLAN_MAGIC;
  h[VA_H_KERNEL] = c.kernel;
  h[VA_H_Q_TILE] = c.q_tile;
  h[VA_H_KV_CHUNK] = cap ? 0 : c.kv_chunk;  // chosen per plan: not part of a fixed plan's header (see counts)
  h[VA_H_N_WIDE] = cap_wide;
  h[VA_H_WIDE_TILE] = c.wide_tile;
  h[VA_H_N_ITEMS] = cap_wide + cap_narrow;
  h[VA_H_N_LINKS] = cap_links;
  h[VA_H_N_QREFS] = cap_qrefs;
  h[VA_H_N_PARTIALS] = cap_partials;
  h[VA_H_N_ROW_PARTS] = cap_row_parts;
  h[VA_H_N_ROWS] = cap_rows;
  // a fixed plan's header depends on the capacity alone: these two words hold their upper bounds
  h[VA_H_N_SUBROWS] = cap ? cap_qrefs : subs->n_subrows;
  h[VA_H_N_EMPTY_ROWS] = cap ? cap_rows : (int32_t)std::count(b.row_flags.begin(), b.row_flags.end(), VA_ROW_EMPTY);
  h[VA_H_OFF_ITEMS] = off;
  auto write_item = [&](int32_t at, const Item& it) {
    int32_t* w = plan_host + off + at * VA_ITEM_WORDS;
    w[VA_I_LINK_BEGIN] = it.link_begin;
    w[VA_I_N_LINKS] = it.n_links;
    w[VA_I_N_Q] = it.n_q;
    w[VA_I_PART_BASE] = it.part_base;
    w[VA_I_TOKENS] = it.tokens;
    w[VA_I_KIND] = it.kind;
    if (it.n_links > 0) {
      const Link& l = b.links[it.link_begin];
      int32_t* lw = w + VA_I_LINK0;
      lw[VA_L_KV_BEGIN] = l.kv_begin;
      lw[VA_L_TOK_BEGIN] = l.tok_begin;
      lw[VA_L_TOK_END] = l.tok_end;
      lw[VA_L_QREF] = l.qref;
      lw[VA_L_CAUSAL_BASE] = l.causal_base;
      lw[VA_L_FLAGS] = l.flags;
    }
  };
  for (int32_t i = 0; i < b.n_wide; ++i) write_item(i, b.items[i]);
  for (int32_t i = b.n_wide; i < cap_wide; ++i) write_item(i, Item{0, 0, 0, -1, 0, 1, -1, -1});
  for (int32_t i = 0; i < n_narrow; ++i) write_item(cap_wide + i, b.items[b.n_wide + i]);
  for (int32_t i = n_narrow; i < cap_narrow; ++i) write_item(cap_wide + i, Item{0, 0, 0, -1, 0, 0, -1, -1});
  off += (cap_wide + cap_narrow) * VA_ITEM_WORDS;
  h[VA_H_OFF_LINKS] = off;
  for (size_t i = 0; i < b.links.size(); ++i) {
    const Link& l = b.links[i];
    int32_t* w = plan_host + off + (int32_t)i * VA_LINK_WORDS;
    w[VA_L_KV_BEGIN] = l.kv_begin;
    w[VA_L_TOK_BEGIN] = l.tok_begin;
    w[VA_L_TOK_END] = l.tok_end;
    w[VA_L_QREF] = l.qref;
    w[VA_L_CAUSAL_BASE] = l.causal_base;
    w[VA_L_FLAGS] = l.flags;
  }
  off += cap_links * VA_LINK_WORDS;
  h[VA_H_OFF_QREFS] = off;
  std::copy(b.qrefs.begin(), b.qrefs.end(), plan_host + off);
  off += cap_qrefs;
  h[VA_H_OFF_QREF_ROWS] = off;
  for (size_t i = 0; i < b.qrefs.size(); ++i) plan_host[off + i] = (int32_t)subs->sub_worker[b.qrefs[i]];
  off += cap_qrefs;
  h[VA_H_OFF_ROW_INDPTR] = off;
  std::copy(b.row_indptr.begin(), b.row_indptr.end(), plan_host + off);
  for (int32_t r = subs->n_rows; r < cap_rows; ++r) plan_host[off + r + 1] = b.row_indptr.back();
  off += cap_rows + 1;
  h[VA_H_OFF_ROW_IDS] = off;
  std::copy(b.row_ids.begin(), b.row_ids.end(), plan_host + off);
  off += cap_row_parts;
  h[VA_H_OFF_ROW_FLAGS] = off;
  std::copy(b.row_flags.begin(), b.row_flags.end(), plan_host + off);
  for (int32_t r = subs->n_rows; r < cap_rows; ++r) plan_host[off + r] = VA_ROW_EMPTY;
  off += cap_rows;
  // The waves of a merge workgroup split a row's states, so rows of many states (long views cut
  // into many chunks) get more waves; when the rows are many (split prefill tiles: thousands of
  // rows of a few states each) one wave per row keeps more rows in flight.  A fixed plan decides
  // from its capacity, a packed one from its counts: either way the word is part of the header the
  // launches are derived from.  Measured on one MI355X: 17 states per row take 9.9 / 14.7 / 20.6 us
  // with 4 / 8 / 16 waves, 72 per row 16.4 / 12.0 / 9.5 us.
  {
    const int64_t rows = std::max<int64_t>(1, cap ? cap_rows : subs->n_rows);
    const int64_t per_row = (cap ? cap_row_parts : c.n_row_parts) / rows;
    h[VA_H_MERGE_WAVES] = rows * shape->num_q_heads >= 8192 ? 1 : per_row >= 48 ? 16 : per_row >= 28 ? 8 : 4;
  }
  h[VA_H_N_WIDE_SLOTS] = c.n_wide_slots;
  h[VA_H_OFF_WIDE_SLOTS] = off;
  std::copy(b.wide_slots.begin(), b.wide_slots.end(), plan_host + off);
  for (int32_t k = (int32_t)b.wide_slots.size(); k <= c.n_wide_slots; ++k) plan_host[off + k] = b.wide_slots.back();
  off += c.n_wide_slots + 1;
  if (counts) *counts = c;
  return VA_OK;
}

extern "C" int va_plan_build(const VaSubRequests* subs, const VaShape* shape, const VaPlanParams* params,
                             int32_t* plan_host, int64_t plan_capacity_words, VaPlanCounts* counts) {
  if (!plan_host) return va_fail(VA_ERR_ARG, "null plan buffer");
  Built b;
  int rc = build(subs, shape, params, b);
  if (rc) return rc;
  return write_plan(b, subs, shape, nullptr, plan_host, plan_capacity_words, counts);
}

extern "C" int64_t va_plan_fixed_words(const VaPlanCapacity* cap) {
  if (!cap) return 0;
  return (int64_t)VA_PLAN_HEADER_WORDS + ((int64_t)cap->max_items + cap->max_wide_items) * VA_ITEM_WORDS +
         (int64_t)cap->max_links * VA_LINK_WORDS + 2 * (int64_t)cap->max_qrefs + (cap->max_rows + 1) +
         cap->max_row_parts + cap->max_rows + (cap->max_wide_items + 1);
}

// Upper bounds of every plan section for a workload within `lim`, following the rules of build():
//   * stand-alone sub-requests: a group of readers is cut into tiles x chunks with
//     chunk >= total_tokens / target, plus one for the halved last chunk, so items <= 2 tiles + target
//     with tiles <= sub-requests; every item carries one link; a query row enters the partial list
//     once per chunk of its run;
//   * chains: tiles of up to wide_tile rows (the last one of a chain may be narrow); a narrow tile
//     is split into round(its tokens / budget) pieces with budget >= all chain tokens / target; wide
//     tiles are cut in bundles of `lanes` tiles, at most 7 cuts of at most `lanes` items each with
//     8 x lanes <= target, and a chain's last bundle may be walked in up to `lanes` parts side by
//     side; so items <= tiles + chains x lanes + target per class; a tile has one link per member plus
//     one per cut or part; a split tile's rows enter the partial list once per piece.
extern "C" int va_plan_capacity(const VaShape* shape, const VaPlanParams* params, const VaPlanLimits* lim,
                                VaPlanCapacity* capacity) {
  if (!shape || !lim || !capacity) return va_fail(VA_ERR_ARG, "null argument");
  if (params && params->kv_chunk > 0)
    return va_fail(VA_ERR_ARG, "fixed-capacity plans choose their KV chunk themselves: kv_chunk must be 0");
  if (lim->max_sub_requests < 0 || lim->max_sub_rows < lim->max_sub_requests || lim->max_chains < 0 ||
      lim->max_chain_members < 0 || lim->max_chain_rows < 0 || lim->max_rows <= 0)
    return va_fail(VA_ERR_ARG, "limits: negative count, no rows, or fewer query rows than sub-requests");
  if (shape->num_kv_heads <= 0 || shape->num_q_heads % shape->num_kv_heads)
    return va_fail(VA_ERR_ARG, "num_q_heads must be a multiple of num_kv_heads");
  const int kernel = resolve_kernel(shape, params);
  if (kernel < 0) return va_fail(VA_ERR_ARG, "requested kernel family does not support this dtype/shape");
  const int g = shape->num_q_heads / shape->num_kv_heads;
  const int64_t q_tile = params && params->q_tile > 0 ? params->q_tile
                                                      : (kernel == VA_KERNEL_MFMA ? va_mfma_default_q_tile(g, false) : 1);
  int64_t wide_tile = 0;
  if (kernel == VA_KERNEL_MFMA && !(params && params->wide_tile < 0)) {
    wide_tile = params && params->wide_tile > 0 ? params->wide_tile : va_mfma_wide_q_tile(g, shape->head_dim);
    if (wide_tile <= q_tile) wide_tile = 0;
  }
  const bool wide_groups = params && params->wide_tile > 0 && wide_tile > 0;
  const int64_t target = params && params->target_items > 0 ? params->target_items
                                                            : std::max(64, 2048 / shape->num_kv_heads);
  const int64_t subs = lim->max_sub_requests, sub_rows = lim->max_sub_rows;
  const int64_t chains = lim->max_chains, members = lim->max_chain_members, chain_rows = lim->max_chain_rows;

  int64_t narrow = 0, wide = 0, links = 0, qrefs = 0, partials = 0;
  if (subs > 0) {
    narrow += 2 * sub_rows + target;  // tiles <= query rows; the halved last chunk adds one item per tile
    // wide decode tiles are cut at min(chunk, their tokens / (256 / kv heads))
    if (wide_groups) wide += sub_rows + target + 256;
    qrefs += sub_rows;
    // a query row is in one tile; that tile has at most 1 + len / chunk chunks, and the sum of
    // len / chunk over tiles is at most target (times the tile's rows when counted per row)
    partials += 2 * sub_rows + (q_tile + (wide_groups ? wide_tile : 0)) * (target + 256);
  }
  if (chains > 0 && chain_rows > 0) {
    const int64_t tile_rows = wide_tile ? wide_tile : q_tile;
    const int64_t tiles = chain_rows / tile_rows + chains;  // per chain: floor(rows / tile) + 1
    // the last bundle of a chain may hold fewer tiles than a group has lanes and be walked in parts
    // side by side: up to `lanes` items, one more link each and `lanes` x tile rows more partial states
    const int64_t lanes = std::max<int64_t>(1, std::min<int64_t>(target, std::max(1, 256 / shape->num_kv_heads)) / kXcds);
    if (wide_tile) {
      wide += tiles + chains * lanes + target;
      narrow += chains + target;
    } else {
      narrow += tiles + target;
    }
    const int64_t chain_items = tiles + target + (wide_tile ? chains * (lanes + 1) + target : 0);
    links += tiles * members + chain_items;
    partials += chain_rows + tile_rows * (target + (wide_tile ? chains * lanes : 0));
  }
  links += narrow + wide;
  auto round8 = [](int64_t x) { return (x + 7) / 8 * 8; };
  const int64_t limit = INT32_MAX / 64;
  if (narrow > limit || wide > limit || links > limit || partials > limit)
    return va_fail(VA_ERR_CAPACITY, "limits describe a plan too large for 32-bit tables");
  capacity->max_items = (int32_t)round8(narrow);
  capacity->max_wide_items = (int32_t)round8(wide);
  capacity->max_links = (int32_t)links;
  capacity->max_qrefs = (int32_t)qrefs;
  capacity->max_partials = (int32_t)partials;
  capacity->max_row_parts = (int32_t)partials;
  capacity->max_rows = lim->max_rows;
  return VA_OK;
}

extern "C" int va_plan_build_fixed(const VaSubRequests* subs, const VaShape* shape, const VaPlanParams* params,
                                   const VaPlanCapacity* cap, int32_t* plan_host, int64_t plan_capacity_words,
                                   VaPlanCounts* counts) {
  if (!plan_host || !cap) return va_fail(VA_ERR_ARG, "null plan buffer or capacity");
  if (cap->max_items % kXcds || cap->max_wide_items % kXcds || cap->max_items < 0 || cap->max_wide_items < 0)
    return va_fail(VA_ERR_ARG, "capacity: item counts must be non-negative multiples of 8");
  Built b;
  int rc = build(subs, shape, params, b, cap);
  if (rc) return rc;
  return write_plan(b, subs, shape, cap, plan_host, plan_capacity_words, counts);
}
