"""Host-side bookkeeping of the paged KV cache for a generation loop: a pool that hands out physical blocks, the
block list of every sequence, and the two per-step products the kernels consume (padded block tables, slot mapping).

Keeps the public names and call contract of mindformers/modules/block_tables.py:24-126 and
mindformers/modules/cache_engine.py:20-90 (BlockTables / CacheEngine / BlockMemPool and their methods):
  * blocks leave the pool in FIFO order (lowest ids first on a fresh pool) and returned blocks queue at the back;
  * token j of a sequence lives in slot  table[j // block_size] * block_size + j % block_size;
  * tables are padded with -1 to seq_length // block_size entries, padding positions of a prefill get slot -1.
The state is one int32 table [batch, max_blocks] that the sequences fill in place, so a step's tables are a copy of
an array and the decode slots one vectorised expression.
"""
from collections import deque
from typing import List

import numpy as np


class BlockMemPool:
    """Pool of ``num_blocks`` physical cache blocks."""

    def __init__(self, num_blocks: int, block_size: int):
        self.num_blocks = int(num_blocks)
        self.block_size = int(block_size)
        self._queue = deque(range(self.num_blocks))           # free ids, next one to hand out on the left
        self._out = np.zeros(self.num_blocks, dtype=bool)     # handed out and not yet returned

    @property
    def free_blocks(self):
        """Free block ids in the order they will be handed out."""
        return list(self._queue)

    @property
    def used_blocks(self):
        return np.flatnonzero(self._out).tolist()

    def allocate_block(self, num_new_block: int):
        n = int(num_new_block)
        if n > len(self._queue):
            raise RuntimeError(f"KV block pool exhausted: {n} blocks requested, {len(self._queue)} of "
                               f"{self.num_blocks} free")
        ids = [self._queue.popleft() for _ in range(n)]
        self._out[ids] = True
        return ids

    def free_block(self, block_indices: List[int]):
        ids = [int(i) for i in block_indices]
        for i in ids:
            if not (0 <= i < self.num_blocks) or not self._out[i]:
                raise RuntimeError(f"block {i} was not handed out by this pool and cannot be returned")
        self._out[ids] = False
        self._queue.extend(ids)


class CacheEngine:
    """The blocks of one sequence.  ``row`` (optional) is the sequence's row of a shared int32 table that mirrors
    ``block_table`` for the batch-level views."""

    def __init__(self, block_size: int, pool: BlockMemPool = None, row=None):
        self.block_size = int(block_size)
        self.pool = pool
        self.num_token = 0
        self.block_table = []
        self._row = row

    def prepare_cache(self, num_new_token):
        """Make room for ``num_new_token`` more tokens."""
        total = self.num_token + int(num_new_token)
        missing = -(-total // self.block_size) - len(self.block_table)
        if missing > 0:
            if self._row is not None and len(self.block_table) + missing > len(self._row):
                raise ValueError(f"{total} tokens do not fit the {len(self._row)} blocks a sequence may hold")
            fresh = self.pool.allocate_block(missing)
            if self._row is not None:
                self._row[len(self.block_table):len(self.block_table) + missing] = fresh
            self.block_table.extend(fresh)
        self.num_token = total

    def release_cache(self):
        self.pool.free_block(self.block_table)
        if self._row is not None:
            self._row[:] = -1
        self.block_table = []
        self.num_token = 0


class BlockTables:
    """Block tables and slot mappings of a batch."""

    def __init__(self, num_blocks, block_size, seq_length):
        self.num_blocks = num_blocks
        self.block_size = block_size
        self.seq_length = seq_length
        self.max_num_blocks_per_seq = self.seq_length // self.block_size
        self.block_mem_pool = BlockMemPool(self.num_blocks, self.block_size)
        self.cache_engines = []
        self._table = np.full((0, self.max_num_blocks_per_seq), -1, dtype=np.int32)

    def init_cache_engine(self, batch_size):
        self._table = np.full((batch_size, self.max_num_blocks_per_seq), -1, dtype=np.int32)
        self.cache_engines = [CacheEngine(self.block_size, self.block_mem_pool, self._table[i])
                              for i in range(batch_size)]

    def _grow(self, new_tokens, is_finished):
        for eng, n, done in zip(self.cache_engines, new_tokens, is_finished):
            if not done:
                eng.prepare_cache(int(n))

    def assemble_pa_full_inputs(self, max_input_length, batch_valid_length: np.array, is_finished: List[bool]):
        """Prefill: blocks for every live prompt; returns (tables [B, max_blocks], slots [B * max_input_length]) with
        slot -1 at the padding positions of each prompt."""
        lens = np.asarray(batch_valid_length, dtype=np.int64).reshape(-1)
        self._grow(lens, is_finished)
        pos = np.arange(int(max_input_length), dtype=np.int64)[None, :]
        live = pos < lens[:, None]
        width = self._table.shape[1]
        col = np.minimum(pos // self.block_size, max(width - 1, 0))
        blk = self._table[np.arange(len(lens))[:, None], col].astype(np.int64) if width else np.zeros_like(live, np.int64)
        slots = np.where(live, blk * self.block_size + pos % self.block_size, -1)
        return self._table.copy(), slots.astype(np.int32).reshape(-1)

    def assemble_pa_inc_inputs(self, batch_valid_length: np.array, is_finished: List[bool]):
        """Decode: one more token per live sequence, written at position L - 1.  A sequence that stopped growing
        (finished) keeps pointing into its last block; one that never held a block gets slot -1."""
        lens = np.asarray(batch_valid_length, dtype=np.int64).reshape(-1)
        self._grow(np.ones(len(lens), dtype=np.int64), is_finished)
        held = np.fromiter((len(e.block_table) for e in self.cache_engines), dtype=np.int64, count=len(lens))
        last = lens - 1
        col = np.clip(np.minimum(last // self.block_size, held - 1), 0, None)
        blk = self._table[np.arange(len(lens)), col].astype(np.int64)
        slots = np.where(held > 0, blk * self.block_size + last % self.block_size, -1)
        return self._table.copy(), slots.astype(np.int32)

    def clear_cache(self):
        for eng in self.cache_engines:
            eng.release_cache()
