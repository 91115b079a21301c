"""Engine-side hook that turns a finished compression into freed blocks
(``LlavaLLMEngine._free_compressed_blocks``, nanovllm/engine/llava_engine.py:274-330)."""
from __future__ import annotations

from typing import Iterable

from .block_manager import BlockManager
from .kv_runner import PagedKVRunner
from .sequence import Sequence


def free_compressed_blocks(block_manager: BlockManager, model_runner: PagedKVRunner, seqs: Iterable[Sequence],
                           reset_all_kept_hashes: bool = True) -> int:
    """For every sequence the runner has compressed: set ``kv_cache_len``, give the table's tail back
    to the block manager (appended to the free deque in table order), truncate the table and forget
    the prefix-cache hash of the last kept block.  Returns the number of blocks freed.

    ``reset_all_kept_hashes`` also clears the hashes of the other kept blocks, whose contents the
    compression rewrote; the reference leaves them, so a later request with the same prefix could be
    handed compressed data.  Block tables and the free list are the same either way.
    """
    freed = 0
    for seq in seqs:
        rows = model_runner._compressed_lens.get(seq.seq_id)
        if rows is None:
            continue
        seq.kv_cache_len = rows
        keep = model_runner.get_compressed_block_count(seq.seq_id)
        model_runner._blocks_to_free.pop(seq.seq_id, None)
        if keep <= 0:
            continue
        tail = seq.block_table[keep:]
        if tail:
            free_before = len(block_manager.free_block_ids)
            block_manager.free_specific_blocks(tail)      # one owner fewer each; unowned pages join the free list in table order
            freed += len(block_manager.free_block_ids) - free_before
            seq.block_table = seq.block_table[:keep]
        # pages whose rows the compression rewrote must not serve a later request as its prompt prefix: all kept
        # pages (also when no page was freed), or like the reference only the last one of a table that got shorter
        stale = seq.block_table if reset_all_kept_hashes else (seq.block_table[-1:] if tail else [])
        if hasattr(block_manager, "forget_pages"):
            block_manager.forget_pages(stale)             # the content keys leave the prefix index as well
        else:                                             # a manager that only has the reference's fields
            for block_id in stale:
                block_manager.blocks[block_id].hash = -1
                block_manager.blocks[block_id].token_ids = []
    return freed
