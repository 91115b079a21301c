"""Oracle (test infrastructure): paged-KV bookkeeping around compression.

Restates ``BlockManager`` (nanovllm/engine/block_manager.py:39-169), the compression state of
``Sequence`` (nanovllm/engine/sequence.py:29, 72-98) and ``LlavaLLMEngine._free_compressed_blocks``
(nanovllm/engine/llava_engine.py:274-330) as plain functions over small records, so that the
product's classes can be checked state-for-state.  The prefix-cache hashing of ``allocate`` is
reduced to "every block is a cache miss", which is what a synthetic sequence with unique tokens
sees.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional, Set


@dataclass
class SeqState:
    seq_id: int
    num_tokens: int                      # len(token_ids)
    block_table: List[int] = field(default_factory=list)
    kv_cache_len_override: Optional[int] = None   # Sequence._kv_cache_len (sequence.py:29)

    @property
    def kv_cache_len(self) -> int:       # sequence.py:78-83
        return self.num_tokens if self.kv_cache_len_override is None else self.kv_cache_len_override

    @property
    def is_compressed(self) -> bool:     # sequence.py:90-93
        return self.kv_cache_len_override is not None

    def append_token(self) -> None:      # sequence.py:72-76
        self.num_tokens += 1
        if self.kv_cache_len_override is not None:
            self.kv_cache_len_override += 1


@dataclass
class PoolState:
    num_blocks: int
    block_size: int = 256
    free: Deque[int] = field(default_factory=deque)
    used: Set[int] = field(default_factory=set)
    ref: Dict[int, int] = field(default_factory=dict)
    hash: Dict[int, int] = field(default_factory=dict)

    def __post_init__(self):
        self.free = deque(range(self.num_blocks))          # block_manager.py:45
        self.ref = {i: 0 for i in range(self.num_blocks)}
        self.hash = {i: -1 for i in range(self.num_blocks)}


def _take(pool: PoolState, bid: int) -> None:
    assert pool.ref[bid] == 0                               # block_manager.py:48-54
    pool.ref[bid] = 1
    pool.hash[bid] = -1
    pool.free.remove(bid)
    pool.used.add(bid)


def _release(pool: PoolState, bid: int) -> None:
    assert pool.ref[bid] == 0                               # block_manager.py:56-59
    pool.used.remove(bid)
    pool.free.append(bid)


def allocate(pool: PoolState, seq: SeqState) -> None:
    """``BlockManager.allocate`` with every block a cache miss (block_manager.py:64-87): blocks are
    taken from the head of the free deque."""
    assert not seq.block_table
    for _ in range((seq.num_tokens + pool.block_size - 1) // pool.block_size):
        bid = pool.free[0]
        _take(pool, bid)
        seq.block_table.append(bid)


def can_append(pool: PoolState, seq: SeqState) -> bool:
    """block_manager.py:98-101."""
    return len(pool.free) >= (seq.kv_cache_len % pool.block_size == 1)


def may_append(pool: PoolState, seq: SeqState) -> None:
    """block_manager.py:103-132, the parts that change state for a compressed sequence: a new block
    is taken from the head of the free deque when ``kv_len % block_size == 1``."""
    if seq.kv_cache_len % pool.block_size == 1:
        bid = pool.free[0]
        _take(pool, bid)
        seq.block_table.append(bid)


def free_compressed_blocks(pool: PoolState, seq: SeqState, compressed_len: Optional[int]) -> List[int]:
    """``_free_compressed_blocks`` for one sequence (llava_engine.py:289-325).  Returns the ids that
    went back to the free deque, in order."""
    freed: List[int] = []
    if compressed_len is None:                              # :291-292
        return freed
    seq.kv_cache_len_override = compressed_len              # :295
    keep = (compressed_len + pool.block_size - 1) // pool.block_size   # llava_model_runner.py:821-822
    if keep > 0 and len(seq.block_table) > keep:            # :300-304
        for bid in seq.block_table[keep:]:                  # :306-315
            if bid in pool.used:
                pool.ref[bid] -= 1
                if pool.ref[bid] == 0:
                    _release(pool, bid)
                    freed.append(bid)
        seq.block_table = seq.block_table[:keep]            # :318
        if seq.block_table:                                 # :321-325
            pool.hash[seq.block_table[-1]] = -1
    return freed
