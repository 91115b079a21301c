"""Compression spread over decode steps: a few layers per step on a side stream, spliced in at the end.

The reference (pipeline tree) snapshots a sequence's KV after prefill, compresses ``layers_per_step`` layers
of the snapshot after every decode step, and when the last layer is done writes ``compressed ++ rows
generated meanwhile`` back to the sequence's pages (``start_decode_overlap_compression`` /
``step_decode_overlap_compression``, kv-cache pipeline/nanovllm/engine/llava_model_runner.py:1271-1338;
``ZeroOverheadCompressEngine``, kv-cache pipeline/nanovllm/kernels/zero_overhead_compress.py:401-537).

Here no snapshot is taken: the prefill rows of a page never change while decoding appends behind them, so each
chunk is compressed straight from the pages into a staging tensor of the compressed size
(``compressor.paged_forward(..., layers=, out=)``), on a side stream of default priority.  The splice is two
ordered copies per plane: staging -> leading slots, then the rows generated meanwhile from
``[prefill_len, len)`` down to ``[C, C + tail)`` (destination below source, safe in place).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import _lib, ops
from .._lib import FastcacheError
from .kv_runner import PagedKVRunner
from .sequence import Sequence


class DecodeOverlapCompressor:
    def __init__(self, runner: PagedKVRunner, layers_per_step: int = 4,
                 compress_stream: Optional[torch.cuda.Stream] = None):
        self.runner = runner
        self.layers_per_step = max(1, int(layers_per_step))
        self.compress_stream = compress_stream or torch.cuda.Stream(device=runner.device)
        self._tasks: List[dict] = []
        self._decode_overlap_blocks: Dict[int, List[int]] = {}      # seq_id -> block table at start
        self._decode_overlap_prefill_lens: Dict[int, int] = {}

    def pending(self, seq_id: int) -> bool:
        return seq_id in self._decode_overlap_blocks

    def start_decode_overlap_compression(self, seqs: List[Sequence], image_len: Optional[int] = None) -> None:
        """Register the sequences (grouped by length); nothing is enqueued yet."""
        r = self.runner
        comp = r._active_compressor()
        if comp is None:
            return
        if not hasattr(comp, "paged_forward") or not hasattr(comp, "paged_compressed_len"):
            raise FastcacheError("decode-overlap compression needs a compressor with paged_forward(layers=, out=)")
        if image_len is None:
            image_len = r.image_token_len
        groups: Dict[int, List[Sequence]] = {}
        for s in seqs:
            if s.seq_id in self._decode_overlap_blocks:
                continue
            if len(s) < getattr(comp, "min_seq_len", 0):
                continue
            groups.setdefault(len(s), []).append(s)
        for S, group in groups.items():
            it_len = [image_len, max(1, S - image_len)]
            C = comp.paged_compressed_len(S, it_len)
            if C >= S:
                continue
            r._isolate_shared_pages(group, comp, image_len)    # the splice rewrites the leading pages in place
            tables, lens = r._table_and_lens([s.block_table for s in group], [S] * len(group))
            staging = torch.empty((2, r.num_hidden_layers, len(group), r.num_key_value_heads, C, r.head_dim),
                                  dtype=r.kv_cache.dtype, device=r.device)
            ready = torch.cuda.Event()
            ready.record()                               # the prefill that produced these rows
            self._tasks.append(dict(seqs=group, S=S, C=C, it_len=it_len, tables=tables, lens=lens, staging=staging,
                                    next_layer=0, ready=ready, done=None))
            for s in group:
                self._decode_overlap_blocks[s.seq_id] = list(s.block_table)
                self._decode_overlap_prefill_lens[s.seq_id] = S

    def step_decode_overlap_compression(self, seqs: List[Sequence]) -> List[Sequence]:
        """Advance every task that has a sequence in ``seqs`` by ``layers_per_step`` layers; splice the tasks
        that finished and return their sequences (whose ``_compressed_lens`` are now set on the runner)."""
        r = self.runner
        comp = r._active_compressor()
        ids = {s.seq_id for s in seqs}
        completed: List[Sequence] = []
        for task in list(self._tasks):
            if not any(s.seq_id in ids for s in task["seqs"]):
                continue
            L = r.num_hidden_layers
            l0 = task["next_layer"]
            if l0 < L:
                l1 = min(l0 + self.layers_per_step, L)
                if l0 == 0:
                    self.compress_stream.wait_event(task["ready"])
                with torch.cuda.stream(self.compress_stream):
                    extra = {"seq_ids": [s.seq_id for s in task["seqs"]]} if getattr(comp, "wants_seq_ids", False) else {}
                    comp.paged_forward(r.kv_cache, task["tables"], task["lens"], task["S"], task["it_len"],
                                       layers=(l0, l1), out=task["staging"], **extra)
                    if l1 >= L:
                        task["done"] = torch.cuda.Event()
                        task["done"].record(self.compress_stream)
                task["next_layer"] = l1
                if l1 < L:
                    continue
            self._splice(task)
            self._tasks.remove(task)
            completed.extend(task["seqs"])
        return completed

    def _splice(self, task: dict) -> None:
        """On the current stream, after the side stream's last chunk: staging -> pages ``[0, C)``, then the rows
        generated since the start from ``[S, len)`` to ``[C, C + tail)``; bookkeeping on the runner."""
        r = self.runner
        torch.cuda.current_stream().wait_event(task["done"])
        S, C = task["S"], task["C"]
        max_len = task["tables"].shape[1] * r.block_size
        for p in range(2):
            view = _lib.paged_view(r.kv_cache[p], task["tables"], None, max_len)
            ops.copy_tokens(_lib.dense_view(task["staging"][p]), view, 0, C, 0)
        for b, s in enumerate(task["seqs"]):
            tail = max(0, len(s) - S)
            if tail > 0:
                tab, _ = r._table_and_lens([s.block_table], [len(s)])
                width = tab.shape[1] * r.block_size
                for p in range(2):
                    view = _lib.paged_view(r.kv_cache[p], tab, None, width)
                    ops.copy_tokens(view, view, S, tail, C)
            new_len = C + tail
            with r._lock:
                r._compressed_lens[s.seq_id] = new_len
                keep = -(-new_len // r.block_size)
                if len(s.block_table) > keep:
                    r._blocks_to_free[s.seq_id] = s.block_table[keep:]
            self._decode_overlap_blocks.pop(s.seq_id, None)
            self._decode_overlap_prefill_lens.pop(s.seq_id, None)
        task["staging"] = None
