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
        c = model_runner._compressed_lens.get(seq.seq_id)
        if c is None:
            continue
        seq.kv_cache_len = c
        keep = model_runner.get_compressed_block_count(seq.seq_id)
        if keep > 0 and len(seq.block_table) > keep:
            for block_id in seq.block_table[keep:]:
                if block_id in block_manager.used_block_ids:
                    blk = block_manager.blocks[block_id]
                    blk.ref_count -= 1
                    if blk.ref_count == 0:
                        block_manager._deallocate_block(block_id)
                        freed += 1
            seq.block_table = seq.block_table[:keep]
            kept = seq.block_table if reset_all_kept_hashes else seq.block_table[-1:]
            for block_id in kept:
                block_manager.blocks[block_id].hash = -1
                block_manager.blocks[block_id].token_ids = []
        model_runner._blocks_to_free.pop(seq.seq_id, None)
    return freed
