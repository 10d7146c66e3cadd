"""Paged-KV block allocator with ref counts and chained xxh64 prefix hashes
(src/myvllm/engine/block_manager.py:24-139).

Intended semantics where the reference is broken: a freshly allocated block
has ref_count 1 (the reference leaves 0, so deallocate never frees it,
block_manager.py:47-53, 101-105).
"""
from __future__ import annotations

from collections import deque

import numpy as np
import xxhash

from minivllm_amd.engine.sequence import Sequence


class Block:
    def __init__(self, block_id):
        self.block_id = block_id
        self.hash = -1
        self.ref_count = 0
        self.token_ids: list[int] = []

    def update(self, h: int, token_ids: list[int]):
        self.hash = h
        self.token_ids = token_ids

    def reset(self):
        self.hash = -1
        self.ref_count = 1
        self.token_ids = []


class BlockManager:
    def __init__(self, num_blocks: int, block_size: int):
        self.block_size = block_size
        self.blocks = [Block(i) for i in range(num_blocks)]
        self.hash_to_block_id: dict[int, int] = {}
        self.free_block_ids: deque[int] = deque(range(num_blocks))
        self.deferred: list = []          # (sequence, block index) whose hash waits for a token id
        self.used_block_ids: set[int] = set()

    @staticmethod
    def compute_hash(token_ids: list[int], prefix_hash_value: int = -1) -> int:
        """xxh64 over (8-byte little-endian prefix hash, if any) + int32 token bytes (block_manager.py:39-44)."""
        h = xxhash.xxh64()
        if prefix_hash_value != -1:
            h.update(prefix_hash_value.to_bytes(8, "little"))
        h.update(np.array(token_ids, dtype=np.int32).tobytes())
        return h.intdigest()

    def _allocate_block(self, block_id: int) -> Block:
        block = self.blocks[block_id]
        assert block.ref_count == 0, "Block is already allocated"
        # the block is about to hold something else: its old hash must not lead here any more (a later prompt whose
        # block has the same tokens behind ANOTHER prefix would pass the token comparison and share the wrong K/V)
        if block.hash != -1 and self.hash_to_block_id.get(block.hash) == block_id:
            del self.hash_to_block_id[block.hash]
        block.reset()
        self.free_block_ids.remove(block_id)
        self.used_block_ids.add(block_id)
        return block

    def _deallocate_block(self, block_id: int) -> None:
        assert self.blocks[block_id].ref_count == 0, "Block is still in use"
        self.used_block_ids.remove(block_id)
        self.free_block_ids.append(block_id)

    def can_allocate(self, seq: Sequence) -> bool:
        return len(self.free_block_ids) >= seq.num_blocks

    def allocate(self, seq: Sequence) -> None:
        """Fill seq.block_table; full blocks whose chained hash (and tokens) match a cached block are shared."""
        assert not seq.block_table
        h = -1
        cache_miss = False
        for i in range(seq.num_blocks):
            token_ids = seq.block(i)
            h = self.compute_hash(token_ids, h) if len(token_ids) == self.block_size else -1
            block_id = self.hash_to_block_id.get(h, -1)
            if block_id == -1 or self.blocks[block_id].hash != h or self.blocks[block_id].token_ids != token_ids:
                cache_miss = True        # a prefix is only reusable up to the first miss
            if cache_miss:
                block = self._allocate_block(self.free_block_ids[0])
            else:
                seq.num_cached_tokens += self.block_size
                if block_id in self.used_block_ids:
                    block = self.blocks[block_id]
                    block.ref_count += 1
                else:
                    block = self._allocate_block(block_id)
            if h != -1:
                block.update(h, token_ids)
                self.hash_to_block_id[h] = block.block_id
            seq.block_table.append(block.block_id)
        if seq.num_cached_tokens == len(seq):
            # every block hit: the last one is recomputed anyway (identical values into the shared block), so
            # that the step has at least one query token per sequence to take the next-token logits from
            seq.num_cached_tokens -= self.block_size

    def deallocate(self, seq: Sequence) -> None:
        for block_id in reversed(seq.block_table):
            block = self.blocks[block_id]
            block.ref_count -= 1
            if block.ref_count == 0:
                self._deallocate_block(block_id)
        seq.num_cached_tokens = 0
        seq.block_table = []

    def can_append(self, seq: Sequence) -> bool:
        """The token appended last needs a slot; a new block is needed exactly when it starts one
        (len % block_size == 1, block_manager.py:112-115)."""
        return len(self.free_block_ids) >= seq.num_blocks - len(seq.block_table)

    def append(self, seq: Sequence) -> None:
        """Called in a decode step after the previous step's token was appended to ``seq`` and before its
        K/V is stored (block_manager.py:120-139): take a block if that token starts one, and give the last
        block its chained hash once this step fills it, so later prompts can share it."""
        table = seq.block_table
        if len(table) < seq.num_blocks:
            block = self._allocate_block(self.free_block_ids[0])
            table.append(block.block_id)
        last = self.blocks[table[-1]]
        if len(seq) % self.block_size == 0:
            if seq.token_ids[-1] < 0:
                # the token that fills the block is still on its way from the device (engine steps launched ahead
                # of their ids): the hash follows when it arrives
                self.deferred.append((seq, seq.num_blocks - 1))
            else:
                self._hash_block(seq, seq.num_blocks - 1)
        else:
            assert last.hash == -1, "a partial block carries no hash"

    def _hash_block(self, seq: Sequence, index: int) -> None:
        table = seq.block_table
        block = self.blocks[table[index]]
        token_ids = seq.block(index)
        prefix = -1
        if index > 0:
            prefix = self.blocks[table[index - 1]].hash
            if prefix == -1:
                # the block before it was never hashed: chaining from -1 would give this block the hash of a first
                # block and let it be shared behind another prefix; it stays unshared instead
                return
        h = self.compute_hash(token_ids, prefix)
        block.update(h, token_ids)
        self.hash_to_block_id[h] = block.block_id

    def hash_deferred_blocks(self) -> None:
        """Hashes postponed by ``append``; a sequence that was finished or preempted in between has given its
        blocks back and is skipped (its blocks simply stay unshared).  An entry whose block still holds a
        placeholder id stays on the list for the next call."""
        keep = []
        for seq, index in self.deferred:
            if index >= len(seq.block_table) or self.blocks[seq.block_table[index]].hash != -1:
                continue
            if all(t >= 0 for t in seq.block(index)):
                self._hash_block(seq, index)
            else:
                keep.append((seq, index))
        self.deferred = keep
