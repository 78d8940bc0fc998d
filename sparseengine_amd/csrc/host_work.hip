// Host side of the matrix-core attention kernels: the work lists of a step (no device code).
//
// The same rules as kernels/attention_work.py, which holds their description and a numpy
// implementation that the tests compare this one with, list for list.  It exists because the lists
// are built once per step on the critical path: a decode step of one request runs about 2 ms on the
// GPU, and a hundred microseconds of array-library overhead per step are then worth removing.
//
// Two calls: `se_attention_work_plan` decides every item's class, key ranges and partial slots and
// returns the lengths of the three lists; `se_attention_work_fill` writes them.
#include <algorithm>
#include <cstdint>
#include <numeric>
#include <vector>

namespace {

constexpr int UNIT_FIELDS = 8;
constexpr int TASK_FIELDS = 6;
constexpr int BLOCK_UNIT_FIELDS = 12;

struct Rules {  // order of the `rules` argument
  int64_t target_waves, min_split_keys, max_splits, tiles_per_block, tiled_max_head_dim, target_blocks,
      min_block_keys, prefix_per_portion;
};

// per item: in_blocks, rows (tiles or blocks), splits, chunk, first_key, base
constexpr int PLAN_FIELDS = 6;

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

int64_t keys_per_unit(const std::vector<int64_t>& units_per_item, const std::vector<int64_t>& reach,
                      int kv_heads, int64_t wanted, int64_t least) {
  int64_t in_flight = 0, ranges_at_least = 0, keys = 0;
  for (size_t i = 0; i < reach.size(); ++i) in_flight += units_per_item[i];
  if (in_flight * kv_heads >= wanted) return int64_t(1) << 30;
  for (size_t i = 0; i < reach.size(); ++i) ranges_at_least += units_per_item[i] * (reach[i] / least);
  if (ranges_at_least * kv_heads < wanted / 2) least = std::max<int64_t>(32, least / 2);
  for (size_t i = 0; i < reach.size(); ++i) keys += units_per_item[i] * reach[i];
  const int64_t share = ceil_div(keys * kv_heads, wanted);
  return std::max(least, ceil_div(share, 32) * 32);
}

}  // namespace

extern "C" {

// plan: int64 [items, PLAN_FIELDS]; counts: int64 [4] = units, tasks, block units, partial slots
int se_attention_work_plan(const int64_t* q_len, const int64_t* ctx_len, int items, int group,
                           int kv_heads, int window, int head_dim, const int64_t* rules_in,
                           int64_t* plan, int64_t* counts) {
  if (items < 0 || group <= 0 || kv_heads <= 0) return -1;
  Rules r{rules_in[0], rules_in[1], rules_in[2], rules_in[3], rules_in[4], rules_in[5], rules_in[6], rules_in[7]};
  const bool blocks_allowed = head_dim > 0 && head_dim % 32 == 0 && head_dim <= r.tiled_max_head_dim;
  std::vector<int64_t> tiles(items), reach(items), nblocks(items), alone(items), cut_blocks(items);
  int64_t whole = 0;      // blocks of items that are never cut into key ranges
  for (int i = 0; i < items; ++i) {
    if (q_len[i] < 1 || q_len[i] > ctx_len[i]) return -2;   // an item's new tokens are part of its context
    tiles[i] = (q_len[i] * group + 15) / 16;
    reach[i] = window ? std::min<int64_t>(ctx_len[i], window + q_len[i]) : ctx_len[i];
    const bool in_blocks = blocks_allowed && tiles[i] >= r.tiles_per_block / 2;
    plan[i * PLAN_FIELDS + 0] = in_blocks;
    nblocks[i] = in_blocks ? ceil_div(tiles[i], r.tiles_per_block) : 0;
    alone[i] = in_blocks ? 0 : tiles[i];
    // the keys of a portion that is most of what it reads (a whole prompt) are not cut into ranges
    const bool cut = in_blocks && reach[i] - q_len[i] >= r.prefix_per_portion * q_len[i];
    cut_blocks[i] = cut ? nblocks[i] : 0;
    whole += cut ? 0 : nblocks[i];
  }
  whole *= kv_heads;
  const int64_t block_keys = r.target_blocks > whole
      ? keys_per_unit(cut_blocks, reach, kv_heads, r.target_blocks - whole, r.min_block_keys)
      : int64_t(1) << 30;
  const int64_t wave_keys = keys_per_unit(alone, reach, kv_heads, r.target_waves, r.min_split_keys);
  int64_t units = 0, tasks = 0, blocks = 0, slots = 0;
  for (int i = 0; i < items; ++i) {
    const bool in_blocks = plan[i * PLAN_FIELDS + 0] != 0;
    const int64_t keys = in_blocks ? (cut_blocks[i] ? block_keys : int64_t(1) << 30) : wave_keys;
    const int64_t first_key = std::max<int64_t>(0, ctx_len[i] - reach[i]) / 32 * 32;
    const int64_t span = ctx_len[i] - first_key;
    int64_t splits = std::min(std::max<int64_t>(ceil_div(reach[i], keys), 1), r.max_splits);
    int64_t chunk = ceil_div(ceil_div(span, splits), 32) * 32;
    if (splits > 1) {
      splits = ceil_div(span, std::max<int64_t>(chunk, 1));
    }
    if (splits <= 1) {
      splits = 1;
      chunk = span;
    }
    const int64_t rows = in_blocks ? nblocks[i] : alone[i];
    plan[i * PLAN_FIELDS + 1] = rows;
    plan[i * PLAN_FIELDS + 2] = splits;
    plan[i * PLAN_FIELDS + 3] = chunk;
    plan[i * PLAN_FIELDS + 4] = first_key;
    plan[i * PLAN_FIELDS + 5] = slots;
    (in_blocks ? blocks : units) += rows * splits;
    if (splits > 1) {
      tasks += tiles[i];
      slots += tiles[i] * splits;
    }
  }
  counts[0] = units;
  counts[1] = tasks;
  counts[2] = blocks;
  counts[3] = slots;
  return 0;
}

int se_attention_work_fill(const int64_t* q_len, const int64_t* ctx_len, int items, int group,
                           int window, const int64_t* rules_in, const int64_t* plan, int32_t* units,
                           int32_t* tasks, int32_t* blocks) {
  const int64_t tiles_per_block = rules_in[3];
  std::vector<std::vector<int32_t>> block_records;  // sorted longest first below
  std::vector<int64_t> block_length;
  int64_t q_start = 0;
  for (int i = 0; i < items; ++i) {
    const bool in_blocks = plan[i * PLAN_FIELDS + 0] != 0;
    const int64_t rows = plan[i * PLAN_FIELDS + 1], splits = plan[i * PLAN_FIELDS + 2],
                  chunk = plan[i * PLAN_FIELDS + 3], first_key = plan[i * PLAN_FIELDS + 4],
                  base = plan[i * PLAN_FIELDS + 5];
    const int64_t tiles = (q_len[i] * group + 15) / 16;
    const int64_t per_row = in_blocks ? tiles_per_block : 1;
    for (int64_t row = 0; row < rows; ++row)
      for (int64_t s = 0; s < splits; ++s) {
        int32_t rec[BLOCK_UNIT_FIELDS] = {0};
        const int64_t begin = first_key + s * chunk;
        rec[0] = i;
        rec[1] = static_cast<int32_t>(row * per_row);
        rec[2] = static_cast<int32_t>(begin);
        rec[3] = static_cast<int32_t>(std::min(begin + chunk, ctx_len[i]));
        rec[4] = splits > 1 ? static_cast<int32_t>(base + row * per_row * splits + s) : -1;
        rec[5] = static_cast<int32_t>(q_start);
        rec[6] = static_cast<int32_t>(q_len[i]);
        rec[7] = static_cast<int32_t>(ctx_len[i]);
        if (!in_blocks) {
          std::copy(rec, rec + UNIT_FIELDS, units);
          units += UNIT_FIELDS;
          continue;
        }
        rec[8] = static_cast<int32_t>(splits);
        const int64_t pos0 = ctx_len[i] - q_len[i];
        const int64_t last_key = pos0 + ((rec[1] + tiles_per_block) * 16 - 1) / group;
        const int64_t end = std::min(std::min(last_key + 1, ctx_len[i]), static_cast<int64_t>(rec[3]));
        int64_t from = begin;
        if (window) from = std::max(from, pos0 + (static_cast<int64_t>(rec[1]) * 16) / group - window + 1);
        block_length.push_back(std::max<int64_t>(end - from, 0));
        block_records.emplace_back(rec, rec + BLOCK_UNIT_FIELDS);
      }
    if (splits > 1)
      for (int64_t tile = 0; tile < tiles; ++tile) {
        tasks[0] = i;
        tasks[1] = static_cast<int32_t>(tile);
        tasks[2] = static_cast<int32_t>(base + tile * splits);
        tasks[3] = static_cast<int32_t>(splits);
        tasks[4] = static_cast<int32_t>(q_start);
        tasks[5] = static_cast<int32_t>(q_len[i]);
        tasks += TASK_FIELDS;
      }
    q_start += q_len[i];
  }
  std::vector<size_t> order(block_records.size());
  std::iota(order.begin(), order.end(), size_t(0));
  std::stable_sort(order.begin(), order.end(),
                   [&](size_t a, size_t b) { return block_length[a] > block_length[b]; });
  for (size_t k : order) {
    std::copy(block_records[k].begin(), block_records[k].end(), blocks);
    blocks += BLOCK_UNIT_FIELDS;
  }
  return 0;
}

}  // extern "C"
