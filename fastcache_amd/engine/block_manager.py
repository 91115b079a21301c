"""Paged-KV block bookkeeping with release after compression
(nanovllm/engine/block_manager.py:39-169).

Free blocks form a FIFO: allocation takes the head of ``free_block_ids``, release appends to its
tail, so the ids a compression frees come back in table order and are reused last.
"""
from __future__ import annotations

from collections import deque
from typing import Deque, Dict, List, Set

import numpy as np
import xxhash

from .sequence import Sequence


def compute_hash(token_ids: List[int], prefix: int = -1) -> int:
    """xxh64 over the optional 8-byte little-endian prefix hash and the token ids as int64 bytes."""
    h = xxhash.xxh64()
    if prefix != -1:
        h.update(prefix.to_bytes(8, "little"))
    h.update(np.array(token_ids).tobytes())
    return h.intdigest()


class Block:
    __slots__ = ("block_id", "ref_count", "hash", "token_ids")

    def __init__(self, block_id: int):
        self.block_id = block_id
        self.ref_count = 0
        self.hash = -1
        self.token_ids: List[int] = []

    def update(self, hash: int, token_ids: List[int]) -> None:
        assert hash != -1
        self.hash, self.token_ids = hash, token_ids

    def reset(self) -> None:
        self.ref_count, self.hash, self.token_ids = 1, -1, []

    def __repr__(self):
        return f"{(self.block_id, self.ref_count, self.hash)}"


class BlockManager:
    def __init__(self, num_blocks: int, block_size: int):
        self.block_size = block_size
        self.blocks: List[Block] = [Block(i) for i in range(num_blocks)]
        self.hash_to_block_id: Dict[int, int] = {}
        self.free_block_ids: Deque[int] = deque(range(num_blocks))
        self.used_block_ids: Set[int] = set()

    # -- single blocks ---------------------------------------------------------------------------
    def _allocate_block(self, block_id: int) -> Block:
        blk = self.blocks[block_id]
        assert blk.ref_count == 0
        blk.reset()
        self.free_block_ids.remove(block_id)
        self.used_block_ids.add(block_id)
        return blk

    def _deallocate_block(self, block_id: int) -> None:
        assert self.blocks[block_id].ref_count == 0
        self.used_block_ids.remove(block_id)
        self.free_block_ids.append(block_id)

    def _unref(self, block_id: int) -> bool:
        """Drop one reference; returns True when the block went back to the free list."""
        blk = self.blocks[block_id]
        blk.ref_count -= 1
        if blk.ref_count == 0:
            self._deallocate_block(block_id)
            return True
        return False

    # -- whole sequences ---------------------------------------------------------------------------
    def can_allocate(self, seq: Sequence) -> bool:
        return len(self.free_block_ids) >= seq.num_blocks

    def allocate(self, seq: Sequence) -> None:
        """Blocks for a fresh sequence, reusing full blocks whose content hash is already cached."""
        assert not seq.block_table
        h, miss = -1, False
        for i in range(seq.num_blocks):
            tokens = seq.block(i)
            h = compute_hash(tokens, h) if len(tokens) == self.block_size else -1
            block_id = self.hash_to_block_id.get(h, -1)
            if block_id == -1 or self.blocks[block_id].token_ids != tokens:
                miss = True
            if miss:
                block_id = self.free_block_ids[0]
                blk = self._allocate_block(block_id)
            else:
                seq.num_cached_tokens += self.block_size
                if block_id in self.used_block_ids:
                    blk = self.blocks[block_id]
                    blk.ref_count += 1
                else:
                    blk = self._allocate_block(block_id)
            if h != -1:
                blk.update(h, tokens)
                self.hash_to_block_id[h] = block_id
            seq.block_table.append(block_id)

    def deallocate(self, seq: Sequence) -> None:
        for block_id in reversed(seq.block_table):
            self._unref(block_id)
        seq.num_cached_tokens = 0
        seq.block_table.clear()

    # -- decode-time growth (uses the compression-aware KV length) -----------------------------------
    def can_append(self, seq: Sequence) -> bool:
        return len(self.free_block_ids) >= (seq.kv_cache_len % self.block_size == 1)

    def may_append(self, seq: Sequence) -> None:
        table = seq.block_table
        last = self.blocks[table[-1]]
        pos = seq.kv_cache_len % self.block_size
        compressed = seq.is_compressed
        if pos == 1:                                  # first token of a new block
            if not compressed:
                assert last.hash != -1
            block_id = self.free_block_ids[0]
            self._allocate_block(block_id)
            table.append(block_id)
        elif pos == 0:                                # block just filled: publish its hash
            if compressed:
                return                                # compressed content is not prefix-cacheable
            assert last.hash == -1
            tokens = seq.last_block()
            prefix = self.blocks[table[-2]].hash if len(table) > 1 else -1
            h = compute_hash(tokens, prefix)
            last.update(h, tokens)
            self.hash_to_block_id[h] = last.block_id
        elif not compressed:
            assert last.hash == -1

    # -- release after compression -----------------------------------------------------------------
    def free_blocks_after_compression(self, seq: Sequence, blocks_to_keep: int) -> None:
        """Return the table's tail past ``blocks_to_keep`` to the free list and truncate the table."""
        table = seq.block_table
        if len(table) <= blocks_to_keep:
            return
        for block_id in table[blocks_to_keep:]:
            self._unref(block_id)
        seq.block_table = table[:blocks_to_keep]

    def free_specific_blocks(self, block_ids: List[int]) -> None:
        for block_id in block_ids:
            if block_id in self.used_block_ids:
                self._unref(block_id)
