// Plan blob layout shared by the host planner and the kernels.
//
// A plan turns the sub-request tables of one launch into work items.  One work
// item is one workgroup per kv head: a tile of query rows walking a chain of
// KV ranges ("links").  Each link is a token range of one sub-request; the
// query tile is re-rotated at every link start because each sub-request has
// its own rotation offset per row.
#pragma once
#include <stdint.h>

#define VA_PLAN_MAGIC 0x56415031  // "VAP1"
#define VA_PLAN_HEADER_WORDS 24
#define VA_ITEM_WORDS 16
#define VA_LINK_WORDS 8

// header word indices
enum {
  VA_H_MAGIC = 0,
  VA_H_KERNEL,
  VA_H_Q_TILE,
  VA_H_KV_CHUNK,
  VA_H_N_ITEMS,
  VA_H_N_LINKS,
  VA_H_N_QREFS,
  VA_H_N_PARTIALS,
  VA_H_N_ROW_PARTS,
  VA_H_N_ROWS,
  VA_H_OFF_ITEMS,
  VA_H_OFF_LINKS,
  VA_H_OFF_QREFS,
  VA_H_OFF_ROW_INDPTR,
  VA_H_OFF_ROW_IDS,
  VA_H_OFF_ROW_FLAGS,
  VA_H_N_EMPTY_ROWS,   // rows no sub-request serves
  VA_H_N_SUBROWS,
  VA_H_N_WIDE,     // items [0, n_wide) are wide tiles, the rest narrow
  VA_H_WIDE_TILE,
  VA_H_OFF_QREF_ROWS,  // parallel to qrefs: the query/output row of each entry (sub_worker[qrefs[k]])
  VA_H_N_WIDE_SLOTS,   // workgroups per kv head of the wide launch (a multiple of 8)
  VA_H_OFF_WIDE_SLOTS, // [n_wide_slots + 1]: slot s runs the wide items [indptr[s], indptr[s + 1]) one after the other
  VA_H_MERGE_WAVES,    // waves per (row, q head) workgroup of the merge launch: 1, 4, 8 or 16
};

// item word indices
enum {
  VA_I_LINK_BEGIN = 0,
  VA_I_N_LINKS,
  VA_I_N_Q,        // query rows in the tile
  VA_I_PART_BASE,  // first partial slot (one per query row), or -1: write `out` directly
  VA_I_TOKENS,     // KV tokens the item walks (scheduling weight)
  VA_I_KIND,       // 1: wide tile (more rows than the streaming kernel's tile)
  VA_I_LINK0 = 8,  // words 8..15: a copy of the item's first link, so that a kernel finds it with the
                   // same load as the item (one level less in the chain of dependent loads at its start)
};

// link word indices
enum {
  VA_L_KV_BEGIN = 0,  // first entry of the sub-request's page (or slot) list in kv_indices
  VA_L_TOK_BEGIN,     // token range within the sub-request
  VA_L_TOK_END,
  VA_L_QREF,          // base sub-row id, or offset into qrefs when VA_LINK_INDIRECT
  VA_L_CAUSAL_BASE,   // token t is visible to tile row i iff t <= causal_base + i
  VA_L_FLAGS,
};

#define VA_LINK_INDIRECT 1  // sub-row of tile row i is qrefs[qref + i], else qref + i
#define VA_LINK_SLOTS 2     // kv_indices entries are token slots (page size 1)
#define VA_LINK_ONCE 4      // no other query tile of the launch reads this token range (per kv head the rows are
                            // fetched exactly once): the streaming kernel requests them non-temporally

#define VA_NO_CAUSAL 0x3fffffff

// row flags
#define VA_ROW_DIRECT 1  // an item writes this row's output itself
#define VA_ROW_EMPTY 2   // nothing serves the row: merge kernel writes zeros
