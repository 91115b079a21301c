"""Page accounting for the paged KV pool, with release of a sequence's tail pages after compression.

Behaviour follows nano-vllm's ``BlockManager`` (nanovllm/engine/block_manager.py:39-169) where the engine hooks
depend on it: free pages form a FIFO (taken from the head, returned to the tail, so the pages a compression
releases come back in table order and are reused last), a sequence grows by one page exactly when its KV length
modulo the page size is 1, and full pages of identical token content are shared between sequences.  The members
``blocks`` (records with ``ref_count`` / ``hash`` / ``token_ids``), ``free_block_ids``, ``used_block_ids`` and
``_deallocate_block`` keep the reference's names because its ``_free_compressed_blocks``
(nanovllm/engine/llava_engine.py:274-330) reaches into them; everything else is this build's own arrangement:
the prefix cache is an index from a page's content key to the page, consulted once per allocation for the
longest cached run of leading full pages.
"""
from __future__ import annotations

import hashlib
from array import array
from collections import deque
from typing import Deque, Dict, List, Sequence as Seq, Set

from .sequence import Sequence

NO_KEY = -1      # a page whose content is not (or no longer) known to the prefix cache


def page_key(tokens: Seq[int], parent: int = NO_KEY) -> int:
    """Content key of a FULL page: 64 bits of BLAKE2b over the key of the page before it (absent for the first
    page) and the page's token ids.  Two pages get the same key only when the whole prefix up to and including
    them is the same (up to hash collisions, which ``allocate`` rules out by comparing the tokens)."""
    h = hashlib.blake2b(digest_size=8)
    if parent != NO_KEY:
        h.update(parent.to_bytes(8, "little"))
    h.update(array("q", tokens).tobytes())
    return int.from_bytes(h.digest(), "little")


class Block:
    """One page: how many sequences reference it and, for a full page, its content key and tokens."""
    __slots__ = ("block_id", "ref_count", "hash", "token_ids")

    def __init__(self, block_id: int):
        self.block_id = block_id
        self.ref_count = 0
        self.hash = NO_KEY
        self.token_ids: List[int] = []

    def forget(self) -> None:
        self.hash, self.token_ids = NO_KEY, []

    def __repr__(self):
        return f"Block(id={self.block_id}, refs={self.ref_count}, key={self.hash})"


class BlockManager:
    def __init__(self, num_blocks: int, block_size: int):
        self.block_size = block_size
        self.blocks: List[Block] = [Block(i) for i in range(num_blocks)]
        self.free_block_ids: Deque[int] = deque(range(num_blocks))
        self.used_block_ids: Set[int] = set()
        self._prefix_index: Dict[int, int] = {}        # content key -> page that holds (or last held) that content

    # -- pages ------------------------------------------------------------------------------------------
    def _claim(self, block_id: int) -> Block:
        """Take a page off the free list (wherever it sits there) for one new owner."""
        page = self.blocks[block_id]
        if page.ref_count != 0:
            raise RuntimeError(f"page {block_id} is still referenced")
        self.free_block_ids.remove(block_id)
        self.used_block_ids.add(block_id)
        page.ref_count = 1
        page.forget()
        return page

    def _claim_next(self) -> Block:
        return self._claim(self.free_block_ids[0])

    def _deallocate_block(self, block_id: int) -> None:
        """An unreferenced page goes to the tail of the free list (its content key stays in the index: a later
        request with the same prefix may still find the bytes there)."""
        if self.blocks[block_id].ref_count != 0:
            raise RuntimeError(f"page {block_id} is still referenced")
        self.used_block_ids.discard(block_id)
        self.free_block_ids.append(block_id)

    def _release(self, block_id: int) -> None:
        page = self.blocks[block_id]
        page.ref_count -= 1
        if page.ref_count == 0:
            self._deallocate_block(block_id)

    def _publish(self, page: Block, key: int, tokens: List[int]) -> None:
        page.hash, page.token_ids = key, tokens
        self._prefix_index[key] = page.block_id

    # -- a new sequence ---------------------------------------------------------------------------------
    def can_allocate(self, seq: Sequence) -> bool:
        return seq.num_blocks <= len(self.free_block_ids)

    def allocate(self, seq: Sequence) -> None:
        """Pages for a sequence that has none.  The leading full pages whose content the index already holds are
        shared (their tokens count as cached); from the first page that is not found on, fresh pages are taken
        from the head of the free list.  Every full page ends up published under its key."""
        if seq.block_table:
            raise RuntimeError("sequence already has pages")
        keys, parent = [], NO_KEY
        for i in range(seq.num_blocks):
            tokens = seq.block(i)
            parent = page_key(tokens, parent) if len(tokens) == self.block_size else NO_KEY
            keys.append(parent)
        shared = 0
        for i, key in enumerate(keys):
            held = self._prefix_index.get(key, NO_KEY) if key != NO_KEY else NO_KEY
            if held == NO_KEY or self.blocks[held].token_ids != seq.block(i):
                break
            shared += 1
        for i, key in enumerate(keys):
            if i < shared:
                block_id = self._prefix_index[key]
                if block_id in self.used_block_ids:
                    page = self.blocks[block_id]
                    page.ref_count += 1
                else:                                   # released earlier, bytes still in place: take it back
                    page = self._claim(block_id)
            else:
                page = self._claim_next()
            if key != NO_KEY:
                self._publish(page, key, seq.block(i))
            seq.block_table.append(page.block_id)
        seq.num_cached_tokens += shared * self.block_size

    def deallocate(self, seq: Sequence) -> None:
        """All pages of a finished or pre-empted sequence, last page first."""
        while seq.block_table:
            self._release(seq.block_table.pop())
        seq.num_cached_tokens = 0

    # -- decode-time growth, by the KV length the sequence really holds (compressed or not) ---------------------
    def can_append(self, seq: Sequence) -> bool:
        starts_new_page = seq.kv_cache_len % self.block_size == 1
        return len(self.free_block_ids) >= int(starts_new_page)

    def may_append(self, seq: Sequence) -> None:
        """Called after a token was appended: the first row of a new page needs that page; a page that has just
        become full is published to the prefix cache, unless the sequence is compressed (its rows are no longer
        the prompt's tokens)."""
        fill = seq.kv_cache_len % self.block_size
        if fill == 1:
            seq.block_table.append(self._claim_next().block_id)
        elif fill == 0 and not seq.is_compressed:
            table = seq.block_table
            parent = self.blocks[table[-2]].hash if len(table) > 1 else NO_KEY
            tokens = seq.last_block()
            self._publish(self.blocks[table[-1]], page_key(tokens, parent), tokens)

    # -- pages a compression rewrites ----------------------------------------------------------------------
    def shared_positions(self, seq: Sequence, upto: int) -> List[int]:
        """Positions below ``upto`` of the sequence's table whose page has more than one owner."""
        return [i for i, b in enumerate(seq.block_table[:upto]) if self.blocks[b].ref_count > 1]

    def unshare(self, seq: Sequence, positions: Seq[int]) -> List[tuple]:
        """Give the sequence a page of its own at each of ``positions`` (pages it shares with other sequences):
        a fresh page from the head of the free list replaces the shared one in the table, which loses one owner.
        Returns ``(old page, new page)`` pairs; the caller copies the rows.  Nothing changes when the free list
        is too short."""
        positions = list(positions)
        if len(positions) > len(self.free_block_ids):
            raise RuntimeError(f"sequence {seq.seq_id} shares {len(positions)} pages it is about to rewrite and "
                               f"only {len(self.free_block_ids)} pages are free")
        moved = []
        for i in positions:
            old = seq.block_table[i]
            fresh = self._claim_next()
            seq.block_table[i] = fresh.block_id
            self._release(old)
            moved.append((old, fresh.block_id))
        return moved

    def forget_pages(self, block_ids: Seq[int]) -> None:
        """The rows of these pages no longer are the tokens they were published under: drop their content keys
        from the prefix cache, so that no later request is handed them."""
        for block_id in block_ids:
            page = self.blocks[block_id]
            if page.hash != NO_KEY and self._prefix_index.get(page.hash) == block_id:
                del self._prefix_index[page.hash]
            page.forget()

    # -- release after compression ------------------------------------------------------------------------
    def free_blocks_after_compression(self, seq: Sequence, blocks_to_keep: int) -> None:
        """Give back the table's pages past the first ``blocks_to_keep`` (in table order) and cut the table."""
        tail = seq.block_table[blocks_to_keep:]
        if tail:
            del seq.block_table[blocks_to_keep:]
            for block_id in tail:
                self._release(block_id)

    def free_specific_blocks(self, block_ids: List[int]) -> None:
        """Drop one reference from each listed page that is in use; others are ignored."""
        for block_id in block_ids:
            if block_id in self.used_block_ids:
                self._release(block_id)
