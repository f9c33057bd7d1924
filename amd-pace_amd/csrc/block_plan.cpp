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
