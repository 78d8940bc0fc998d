"""Work list of the matrix-core attention kernels (host side, numpy).

For one step and one (query heads per kv head) ratio: the rows of every item are cut into tiles
of 16.  A step with enough tiles to fill the chip (prompt portions) goes to the kernel that shares
keys and values through shared memory: a unit is a run of ``TILES_PER_BLOCK`` tiles of one item.
A step with few tiles (decoding) goes to the kernel with one wavefront per unit: every tile's keys
are cut into equal ranges (multiples of 32 keys) and a merge task per tile combines them.
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

UNIT_FIELDS = 8      # item, row_tile, key_begin, key_end, partial_slot (-1: none), q_start, q_len, ctx_len
TASK_FIELDS = 6      # item, row_tile, first_slot, num_splits, q_start, q_len
# Measured on MI355X (48:8 heads of 128, pages of 64): one wavefront per SIMD is the sweet spot.
# 8 requests x 2048 keys take 20 us in 16 ranges of 128 keys against 24 us in 32 of 64; 64 requests
# x 2060 keys 102 us in 2 ranges (1024 wavefronts) against 146 us unsplit and 118 us in 4 ranges;
# 64 x 8192 keys 360 us (6.0 TB/s) against 550 us unsplit; 4 x 131072 keys 361 us (5.9 TB/s).
TARGET_WAVES = 1024    # wavefronts wanted in flight (256 CUs x 4 SIMDs)
TILED_MIN_WAVES = 2048 # tiles x kv heads from which prompt portions take the shared-memory kernel
MIN_SPLIT_KEYS = 128   # keys of a range; 64 when ranges of 128 would leave most of the chip idle (one request)
MAX_SPLITS = 256      # what the merge kernel's shared memory holds
TILES_PER_BLOCK = 8   # row tiles of one block of the shared-memory kernel
TILED_MAX_HEAD_DIM = 128


@dataclass
class AttentionWork:
    """Both lists may be non-empty: a step's prompt portions go to the block kernel, its single
    tokens (whose few rows would leave a block mostly idle over a whole context) to the other."""
    units: np.ndarray        # int32 [num_units, UNIT_FIELDS]: (tile, key range) for one wavefront each
    tasks: np.ndarray        # int32 [num_tasks, TASK_FIELDS]: merges of split tiles
    num_slots: int           # partial results the units write
    block_units: np.ndarray  # int32 [num_block_units, UNIT_FIELDS]: runs of TILES_PER_BLOCK tiles for a block
    tiles_per_block: int = TILES_PER_BLOCK


@dataclass
class DeviceAttentionWork:
    """An ``AttentionWork`` whose lists lie in device memory (int32 tensors)."""
    units: object
    num_units: int
    tasks: object
    num_tasks: int
    num_slots: int
    block_units: object
    num_block_units: int
    tiles_per_block: int


def _record(rows: int, item, tile, begin, end, slot, q_start, q_len, ctx) -> np.ndarray:
    block = np.zeros((rows, UNIT_FIELDS), dtype=np.int32)
    for column, value in enumerate((item, tile, begin, end, slot, q_start, q_len, ctx)):
        block[:, column] = value
    return block


def build_attention_work(q_len, ctx_len, group: int, kv_heads: int, window: int = 0,
                         target_waves: int = TARGET_WAVES, head_dim: int = 0) -> AttentionWork:
    """``head_dim``: 0 keeps every step on the one-wavefront kernel (callers that do not know it)."""
    q_len = np.asarray(q_len, dtype=np.int64)
    ctx_len = np.asarray(ctx_len, dtype=np.int64)
    q_start = np.concatenate(([0], np.cumsum(q_len)[:-1]))      # items' tokens lie one after the other
    tiles = (q_len * group + 15) // 16
    empty = np.zeros((0, UNIT_FIELDS), np.int32)

    # blocks of TILES_PER_BLOCK tiles pay off for items with many rows (prompt portions) in a step that
    # fills the chip; items with few rows keep one wavefront per tile and split their keys
    in_blocks = np.zeros(len(tiles), dtype=bool)
    if (head_dim and head_dim % 32 == 0 and head_dim <= TILED_MAX_HEAD_DIM
            and int(tiles.sum()) * kv_heads >= TILED_MIN_WAVES and int(tiles.sum()) >= 4 * len(tiles)):
        in_blocks = tiles >= TILES_PER_BLOCK // 2
    block_units = empty
    if in_blocks.any():
        blocks = []
        for item in np.nonzero(in_blocks)[0].tolist():
            first = np.arange(0, int(tiles[item]), TILES_PER_BLOCK, dtype=np.int32)
            blocks.append(_record(first.size, item, first, 0, ctx_len[item], -1, q_start[item], q_len[item],
                                  ctx_len[item]))
        block_units = np.concatenate(blocks)
        # longest first: a block's work grows with the position of its rows, and the blocks that are
        # started last decide when the kernel ends
        pos0 = ctx_len - q_len
        reach = pos0[block_units[:, 0]] + ((block_units[:, 1].astype(np.int64) + TILES_PER_BLOCK) * 16 - 1) // group
        keys = np.minimum(reach + 1, ctx_len[block_units[:, 0]])
        if window:
            keys = np.minimum(keys, window + TILES_PER_BLOCK * 16 // group + 1)
        block_units = block_units[np.argsort(-keys, kind="stable")]

    rest = np.nonzero(~in_blocks)[0].tolist()
    waves = int(tiles[~in_blocks].sum()) * kv_heads
    want = 1 if waves >= target_waves else -(-target_waves // max(waves, 1))
    units, tasks, slot = [], [], 0
    for item in rest:
        n_tiles, ctx = int(tiles[item]), int(ctx_len[item])
        reach = min(ctx, window + int(q_len[item])) if window else ctx     # keys a tile can read
        min_keys = MIN_SPLIT_KEYS
        if waves * (reach // min_keys) < target_waves // 2:
            min_keys //= 2
        splits = max(1, min(want, reach // min_keys, MAX_SPLITS))
        tile_ids = np.arange(n_tiles, dtype=np.int32)
        if splits == 1:
            units.append(_record(n_tiles, item, tile_ids, 0, ctx, -1, q_start[item], q_len[item], ctx))
            continue
        first_key = max(0, ctx - reach) // 32 * 32
        chunk = -(-(-(-(ctx - first_key) // splits)) // 32) * 32
        splits = -(-(ctx - first_key) // chunk)
        begins = first_key + np.arange(splits, dtype=np.int32) * chunk
        block = np.zeros((n_tiles, splits, UNIT_FIELDS), dtype=np.int32)
        block[:, :, 0] = item
        block[:, :, 1] = tile_ids[:, None]
        block[:, :, 2] = begins[None, :]
        block[:, :, 3] = np.minimum(begins + chunk, ctx)[None, :]
        block[:, :, 4] = slot + np.arange(n_tiles * splits, dtype=np.int32).reshape(n_tiles, splits)
        block[:, :, 5], block[:, :, 6], block[:, :, 7] = q_start[item], q_len[item], ctx
        units.append(block.reshape(-1, UNIT_FIELDS))
        task = np.zeros((n_tiles, TASK_FIELDS), dtype=np.int32)
        task[:, 0], task[:, 1], task[:, 3] = item, tile_ids, splits
        task[:, 2] = slot + tile_ids * splits
        task[:, 4], task[:, 5] = q_start[item], q_len[item]
        tasks.append(task)
        slot += n_tiles * splits
    return AttentionWork(np.concatenate(units) if units else empty,
                         np.concatenate(tasks) if tasks else np.zeros((0, TASK_FIELDS), np.int32), slot,
                         block_units)
