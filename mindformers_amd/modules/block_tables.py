"""Host-side block bookkeeping of the paged KV cache, as the generation loop drives it
(mindformers/modules/block_tables.py:24-126, mindformers/modules/cache_engine.py:20-90).  Pure numpy / lists."""
from typing import List

import numpy as np


class BlockMemPool:
    """Block-wise memory pool: blocks are handed out from the front of the free list (cache_engine.py:20-60)."""

    def __init__(self, num_blocks: int, block_size: int):
        self.num_blocks = num_blocks
        self.block_size = block_size
        self.free_blocks = list(range(num_blocks))
        self.used_blocks = []

    def allocate_block(self, num_new_block: int):
        if len(self.free_blocks) < num_new_block:
            raise RuntimeError('block pool is out of memory')
        new_blocks = self.free_blocks[0:num_new_block]
        self.used_blocks += new_blocks
        self.free_blocks = self.free_blocks[num_new_block:]
        return new_blocks

    def free_block(self, block_indices: List[int]):
        for idx in block_indices:
            if idx not in self.used_blocks:
                raise RuntimeError(f"bad block idx, {idx} is not in the used block list.")
            self.free_blocks.append(idx)
            self.used_blocks.remove(idx)


class CacheEngine:
    """Per-sequence block list (cache_engine.py:63-90)."""

    def __init__(self, block_size: int, pool: BlockMemPool = None):
        self.block_size = block_size
        self.pool = pool
        self.num_token = 0
        self.block_table = []

    def prepare_cache(self, num_new_token):
        remained_token = len(self.block_table) * self.block_size - self.num_token
        if remained_token < num_new_token:
            num_new_block = (num_new_token - remained_token + self.block_size - 1) // self.block_size
            self.block_table += self.pool.allocate_block(num_new_block)
        self.num_token += num_new_token

    def release_cache(self):
        self.pool.free_block(self.block_table)
        self.block_table = []
        self.num_token = 0


class BlockTables:
    """Which physical block holds which tokens of each sequence, and the slot each new token is written to
    (block_tables.py:24-126).  Tables are padded with -1 to seq_length // block_size entries."""

    def __init__(self, num_blocks, block_size, seq_length):
        self.num_blocks = num_blocks
        self.block_size = block_size
        self.seq_length = seq_length
        self.max_num_blocks_per_seq = self.seq_length // self.block_size
        self.block_mem_pool = BlockMemPool(self.num_blocks, self.block_size)
        self.cache_engines = []

    def init_cache_engine(self, batch_size):
        self.cache_engines.clear()
        for _ in range(batch_size):
            self.cache_engines.append(CacheEngine(self.block_size, self.block_mem_pool))

    def _padded_tables(self):
        rows = []
        for eng in self.cache_engines:
            rows.append(eng.block_table + [-1] * (self.max_num_blocks_per_seq - len(eng.block_table)))
        return np.array(rows, dtype=np.int32).reshape(len(self.cache_engines), -1)

    def assemble_pa_full_inputs(self, max_input_length, batch_valid_length: np.array, is_finished: List[bool]):
        """Prefill: allocate blocks for every prompt and map each token position to its slot (padding = -1)."""
        bs = batch_valid_length.shape[0]
        for i in range(bs):
            if not is_finished[i]:
                self.cache_engines[i].prepare_cache(int(batch_valid_length[i]))
        block_tables = self._padded_tables()
        pos = np.arange(max_input_length, dtype=np.int64)[None, :]
        valid = pos < np.asarray(batch_valid_length, dtype=np.int64)[:, None]
        blk_idx = np.where(valid, pos // self.block_size, 0)
        width = block_tables.shape[1]
        blk = np.take_along_axis(block_tables, np.minimum(blk_idx, max(width - 1, 0)).astype(np.int64), axis=1) \
            if width else np.zeros_like(blk_idx)
        slots = np.where(valid, blk.astype(np.int64) * self.block_size + pos % self.block_size, -1)
        return block_tables, slots.astype(np.int32).reshape(-1)

    def assemble_pa_inc_inputs(self, batch_valid_length: np.array, is_finished: List[bool]):
        """Decode: one more token per live sequence; slot = table[(L-1) // bs] * bs + (L-1) % bs."""
        bs = batch_valid_length.shape[0]
        slot_mapping = []
        for i in range(bs):
            if not is_finished[i]:
                self.cache_engines[i].prepare_cache(1)
            block_table = self.cache_engines[i].block_table
            cur = int(batch_valid_length[i]) - 1
            index = cur // self.block_size
            if index >= len(block_table):
                index = len(block_table) - 1
            slot_mapping.append(block_table[index] * self.block_size + cur % self.block_size)
        return self._padded_tables(), np.array(slot_mapping, dtype=np.int32)

    def clear_cache(self):
        for cache_engine in self.cache_engines:
            cache_engine.release_cache()
