// Host-side bookkeeping of the block pool that is worth doing in native code: the compaction plan of a
// block table (a few passes over the table; in interpreted code they took longer than the copy they plan).
#include <vector>

#include "common.h"

using namespace pace_kv;

extern "C" int32_t pace_kv_plan_compaction(int32_t* block_table, int32_t table_stride, const int64_t* n_blocks, int32_t batch,
                                           int32_t num_blocks, int32_t* moves, int32_t capacity, int32_t apply, int32_t* refs) {
  const char* who = "pace_kv_plan_compaction";
  PACE_REQUIRE(batch >= 0 && table_stride >= 1 && num_blocks >= 1 && capacity >= 0, "%s: bad batch (%d), table_stride (%d), num_blocks (%d) or capacity (%d)",
               who, batch, table_stride, num_blocks, capacity);
  if (batch == 0) return 0;
  PACE_REQUIRE(block_table && n_blocks && (moves || capacity == 0) && (!apply || refs), "%s: NULL pointer", who);
  // Live ids as a bitmap, walked a word at a time (count-trailing-zeros): a byte per id and a test per id cost more
  // in mispredicted branches (which ids are live is random) than everything else here together.
  const size_t words = ((size_t)num_blocks + 63) / 64;
  std::vector<uint64_t> live(words, 0);
  for (int b = 0; b < batch; ++b) {
    PACE_REQUIRE(n_blocks[b] >= 0 && n_blocks[b] <= table_stride, "%s: sequence %d uses %lld of %d table entries", who, b,
                 (long long)n_blocks[b], table_stride);
    const int32_t* row = block_table + (int64_t)b * table_stride;
    uint32_t bad = 0;
    for (int64_t j = 0; j < n_blocks[b]; ++j) {
      const uint32_t id = (uint32_t)row[j];
      bad |= id >= (uint32_t)num_blocks;
      if (id < (uint32_t)num_blocks) live[id >> 6] |= 1ull << (id & 63);
    }
    PACE_REQUIRE(!bad, "%s: a block id of sequence %d is outside the pool", who, b);
  }
  int32_t n_live = 0;
  for (size_t w = 0; w < words; ++w) n_live += __builtin_popcountll(live[w]);
  // sources: live ids >= n_live, ascending; destinations: free ids < n_live, ascending (as many of each)
  auto bits_from = [&](size_t w, int32_t first, bool want_live) {  // word w with the ids below `first` taken out
    uint64_t v = want_live ? live[w] : ~live[w];
    if ((int64_t)w * 64 < first) v &= first - (int64_t)w * 64 >= 64 ? 0 : ~0ull << (first - (int64_t)w * 64);
    return v;
  };
  int32_t n_moves = 0;
  for (size_t w = (size_t)n_live / 64; w < words; ++w) n_moves += __builtin_popcountll(bits_from(w, n_live, true));
  PACE_REQUIRE(n_moves <= capacity, "%s: %d moves do not fit the capacity of %d", who, n_moves, capacity);
  std::vector<int32_t> remap;
  if (apply) {
    remap.resize((size_t)num_blocks);
    for (int32_t id = 0; id < num_blocks; ++id) remap[id] = id;
  }
  {
    int32_t k = 0;
    for (size_t w = (size_t)n_live / 64; w < words; ++w)
      for (uint64_t v = bits_from(w, n_live, true); v; v &= v - 1) moves[2 * k++] = (int32_t)(w * 64 + __builtin_ctzll(v));
    // a free id below n_live exists for every live id at or above it (the ids past the pool's end in the last word
    // read as free, but they are never below n_live)
    k = 0;
    for (size_t w = 0; k < n_moves; ++w)
      for (uint64_t v = bits_from(w, 0, false); v && k < n_moves; v &= v - 1) moves[2 * k++ + 1] = (int32_t)(w * 64 + __builtin_ctzll(v));
    if (apply)
      for (int32_t i = 0; i < n_moves; ++i) remap[moves[2 * i]] = moves[2 * i + 1];
  }
  if (apply) {
    for (int32_t id = 0; id < num_blocks; ++id) refs[id] = 0;
    for (int b = 0; b < batch; ++b) {
      int32_t* row = block_table + (int64_t)b * table_stride;
      for (int64_t j = 0; j < n_blocks[b]; ++j) {
        row[j] = remap[row[j]];
        ++refs[row[j]];
      }
    }
  }
  return n_moves;
}

extern "C" int pace_kv_apply_moves(int32_t* block_table, int32_t table_stride, const int64_t* n_blocks, int32_t batch,
                                   int32_t num_blocks, const int32_t* moves, int32_t n_moves, int32_t* refs) {
  const char* who = "pace_kv_apply_moves";
  PACE_REQUIRE(batch >= 0 && table_stride >= 1 && num_blocks >= 1 && n_moves >= 0, "%s: bad batch (%d), table_stride (%d), num_blocks (%d) or n_moves (%d)",
               who, batch, table_stride, num_blocks, n_moves);
  PACE_REQUIRE((batch == 0 || (block_table && n_blocks)) && (n_moves == 0 || moves) && refs, "%s: NULL pointer", who);
  std::vector<int32_t> remap((size_t)num_blocks);
  for (int32_t id = 0; id < num_blocks; ++id) remap[id] = id, refs[id] = 0;
  for (int32_t k = 0; k < n_moves; ++k) {
    const int32_t src = moves[2 * k], dst = moves[2 * k + 1];
    PACE_REQUIRE(src >= 0 && src < num_blocks && dst >= 0 && dst < num_blocks, "%s: move %d (%d -> %d) is outside the pool", who, k, src, dst);
    remap[src] = dst;
  }
  for (int b = 0; b < batch; ++b) {
    PACE_REQUIRE(n_blocks[b] >= 0 && n_blocks[b] <= table_stride, "%s: sequence %d uses %lld of %d table entries", who, b,
                 (long long)n_blocks[b], table_stride);
    int32_t* row = block_table + (int64_t)b * table_stride;
    for (int64_t j = 0; j < n_blocks[b]; ++j) {
      PACE_REQUIRE(row[j] >= 0 && row[j] < num_blocks, "%s: block id %d of sequence %d is outside the pool", who, row[j], b);
      row[j] = remap[row[j]];
      ++refs[row[j]];
    }
  }
  return PACE_KV_OK;
}

// The same plan from the allocator's own record of which ids are free (one byte per id, non-zero = free): no walk
// over the table.  Eight flags become eight bits with one multiplication; the plan is then two walks over the bitmap.
extern "C" int32_t pace_kv_plan_compaction_flags(const uint8_t* is_free, int32_t num_blocks, int32_t* moves, int32_t capacity) {
  const char* who = "pace_kv_plan_compaction_flags";
  PACE_REQUIRE(is_free && num_blocks >= 1 && capacity >= 0 && (moves || capacity == 0), "%s: bad num_blocks (%d), capacity (%d) or NULL pointer", who,
               num_blocks, capacity);
  const size_t words = ((size_t)num_blocks + 63) / 64;
  static thread_local std::vector<uint64_t> live;
  live.assign(words, 0);
  int32_t id = 0;
  for (; id + 8 <= num_blocks; id += 8) {
    uint64_t x;
    __builtin_memcpy(&x, is_free + id, 8);
    // bytes to 0 / 1 (a flag is any non-zero value), then bit i of the product's top byte is byte i of x
    x = ((x | ((x & 0x7f7f7f7f7f7f7f7full) + 0x7f7f7f7f7f7f7f7full)) >> 7) & 0x0101010101010101ull;
    const uint64_t free_bits = (x * 0x0102040810204080ull) >> 56;
    live[(size_t)id >> 6] |= (~free_bits & 0xffull) << (id & 63);
  }
  for (; id < num_blocks; ++id)
    if (!is_free[id]) live[(size_t)id >> 6] |= 1ull << (id & 63);
  int32_t n_live = 0;
  for (size_t w = 0; w < words; ++w) n_live += __builtin_popcountll(live[w]);
  auto bits_from = [&](size_t w, int32_t first, bool want_live) {  // word w with the ids below `first` taken out
    uint64_t v = want_live ? live[w] : ~live[w];
    if ((int64_t)w * 64 < first) v &= first - (int64_t)w * 64 >= 64 ? 0 : ~0ull << (first - (int64_t)w * 64);
    return v;
  };
  int32_t n_moves = 0;
  for (size_t w = (size_t)n_live / 64; w < words; ++w) n_moves += __builtin_popcountll(bits_from(w, n_live, true));
  PACE_REQUIRE(n_moves <= capacity, "%s: %d moves do not fit the capacity of %d", who, n_moves, capacity);
  int32_t k = 0;
  for (size_t w = (size_t)n_live / 64; w < words; ++w)
    for (uint64_t v = bits_from(w, n_live, true); v; v &= v - 1) moves[2 * k++] = (int32_t)(w * 64 + __builtin_ctzll(v));
  k = 0;
  for (size_t w = 0; k < n_moves; ++w)
    for (uint64_t v = bits_from(w, 0, false); v && k < n_moves; v &= v - 1) moves[2 * k++ + 1] = (int32_t)(w * 64 + __builtin_ctzll(v));
  return n_moves;
}

// Rewrite the table for moves whose data is being copied, moving the bookkeeping along instead of recounting it:
// the owners of a moved block go with it (refs), its old id becomes free and its new one used (is_free), and the
// free list is written out afresh, lowest ids on top (free_stack [num_blocks], *n_free entries, the stack's top
// last).  Sources must be live, destinations free, and no id may occur twice: then only table entries that name a
// source change.
extern "C" int pace_kv_apply_moves_tracked(int32_t* block_table, int32_t table_stride, const int64_t* n_blocks, int32_t batch,
                                           int32_t num_blocks, const int32_t* moves, int32_t n_moves, int32_t* refs, uint8_t* is_free,
                                           int32_t* free_stack, int32_t* n_free) {
  const char* who = "pace_kv_apply_moves_tracked";
  PACE_REQUIRE(batch >= 0 && table_stride >= 1 && num_blocks >= 1 && n_moves >= 0, "%s: bad batch (%d), table_stride (%d), num_blocks (%d) or n_moves (%d)",
               who, batch, table_stride, num_blocks, n_moves);
  PACE_REQUIRE((batch == 0 || (block_table && n_blocks)) && (n_moves == 0 || moves) && refs && is_free && free_stack && n_free, "%s: NULL pointer", who);
  // new id of every id: itself, but for the sources.  (A full map read without a test per table entry: which entries
  // name a moved block is as good as random, and a mispredicted branch per entry cost more than the map.)
  static thread_local std::vector<int32_t> remap, identity;
  if (identity.size() < (size_t)num_blocks) {
    const size_t had = identity.size();
    identity.resize((size_t)num_blocks);
    for (size_t i = had; i < identity.size(); ++i) identity[i] = (int32_t)i;
  }
  remap.resize((size_t)num_blocks);
  __builtin_memcpy(remap.data(), identity.data(), (size_t)num_blocks * sizeof(int32_t));
  // marks while the moves are checked: 2 = a source, 3 = a destination (restored if a move is refused)
  int32_t k = 0;
  bool ok = true;
  for (; k < n_moves && ok; ++k) {
    const int32_t src = moves[2 * k], dst = moves[2 * k + 1];
    ok = src >= 0 && src < num_blocks && dst >= 0 && dst < num_blocks && src != dst && is_free[src] == 0 && is_free[dst] == 1;
    if (ok) is_free[src] = 2, is_free[dst] = 3, remap[src] = dst;
  }
  if (!ok) {
    for (int32_t i = 0; i + 1 < k; ++i) is_free[moves[2 * i]] = 0, is_free[moves[2 * i + 1]] = 1;
    PACE_REQUIRE(false, "%s: move %d (%d -> %d) does not take a live block to a free one, or names an id twice", who, k - 1, moves[2 * (k - 1)],
                 moves[2 * (k - 1) + 1]);
  }
  for (int b = 0; b < batch; ++b) {
    const int64_t nb = n_blocks[b] < 0 ? 0 : (n_blocks[b] > table_stride ? table_stride : n_blocks[b]);
    int32_t* row = block_table + (int64_t)b * table_stride;
    for (int64_t j = 0; j < nb; ++j) {
      const uint32_t id = (uint32_t)row[j];
      const bool in_pool = id < (uint32_t)num_blocks;  // (an id outside the pool stays as it is)
      const int32_t mapped = remap[in_pool ? id : 0u];
      row[j] = in_pool ? mapped : row[j];
    }
  }
  for (k = 0; k < n_moves; ++k) {
    const int32_t src = moves[2 * k], dst = moves[2 * k + 1];
    refs[dst] = refs[src], refs[src] = 0;
    is_free[src] = 1, is_free[dst] = 0;
  }
  int32_t top = 0;
  for (int32_t id = num_blocks - 1; id >= 0; --id) {  // (branch-free: which ids are free is as good as random)
    free_stack[top] = id;
    top += is_free[id] != 0;
  }
  *n_free = top;
  return PACE_KV_OK;
}
