"""The compression hooks of nano-vllm's model runner over a paged KV pool
(nanovllm/engine/llava_model_runner.py: ``allocate_kv_cache`` :498-539, ``prepare_decode``
:637-674, ``compress_kv_cache_batch`` :712-793, ``_extract_kv_cache_fast`` :824-872,
``_write_compressed_kv_cache_fast`` :874-912, ``start_background_compression`` :1046-1094).

The model forward is not part of this build; a ``PagedKVRunner`` owns the pool and offers the same
method names, bookkeeping dictionaries and return values, so an engine loop written against the
reference runner drives it unchanged.  Compressors that expose ``paged_forward`` (every compressor
of this package) are run in place on the pages for all sequences of a batch at once, whatever their
lengths; any other callable goes through extract -> call -> write back, with the copies done by HIP
kernels.
"""
from __future__ import annotations

import threading
import time
from typing import Dict, List, Optional, Sequence as Seq, Tuple

import torch

from .. import _lib, ops
from ..utils.context import set_context
from .sequence import Sequence

LayerKV = Tuple[torch.Tensor, torch.Tensor]


class PagedKVRunner:
    def __init__(self, num_layers: int, num_kv_heads: int, head_dim: int, num_blocks: int, dtype: torch.dtype,
                 device, block_size: int = 256, compressor=None, batched_compressor=None, image_token_len: int = 576,
                 block_manager=None):
        pool = torch.zeros(2, num_layers, num_blocks, block_size, num_kv_heads, head_dim, dtype=dtype,
                           device=torch.device(device))
        self._setup(pool, compressor, batched_compressor, image_token_len, block_manager, None)

    @classmethod
    def adopt(cls, kv_cache: torch.Tensor, compressor=None, batched_compressor=None, image_token_len: int = 576,
              block_manager=None, compressed_lens: Optional[Dict[int, int]] = None) -> "PagedKVRunner":
        """A runner over a pool that already exists (``kv_cache [2, L, blocks, block_size, Hkv, D]``, e.g. the one
        ``LlavaModelRunner.allocate_kv_cache`` made, llava_model_runner.py:526-529) instead of one of its own;
        ``compressed_lens`` lets the host runner and this one share the ``_compressed_lens`` dictionary."""
        if kv_cache.dim() != 6 or kv_cache.shape[0] != 2:
            raise _lib.FastcacheError("kv_cache must be [2, L, num_blocks, block_size, Hkv, D]")
        self = cls.__new__(cls)
        self._setup(kv_cache, compressor, batched_compressor, image_token_len, block_manager, compressed_lens)
        return self

    def _setup(self, kv_cache, compressor, batched_compressor, image_token_len, block_manager, compressed_lens):
        _, L, _, bs, H, D = kv_cache.shape
        self.num_hidden_layers, self.num_key_value_heads, self.head_dim = L, H, D
        self.block_size = bs
        self.device = kv_cache.device
        self.kv_cache = kv_cache
        self.compressor = compressor
        self.batched_compressor = batched_compressor
        self.use_batched_compressor = batched_compressor is not None
        self.image_token_len = image_token_len
        self._compressed_lens: Dict[int, int] = {} if compressed_lens is None else compressed_lens
        self._blocks_to_free: Dict[int, List[int]] = {}
        self._lock = threading.Lock()
        self._compress_stream: Optional[torch.cuda.Stream] = None
        # the page manager, when the caller has one: lets an in-place compression give a sequence its own copy of
        # pages it shares with other sequences (prefix cache) before it rewrites them
        self.block_manager = block_manager
        self._touched = False
        self._watch_enqueues = True
        self._enqueue_mark = _lib.enqueue_count()

    @property
    def _launch_started(self) -> bool:
        """Whether an enqueue since the flag was last cleared may have begun to rewrite cache rows in place: set by
        hand, or read off the library's count of successful entry-point calls (host-side checks that raise before
        the first launch leave it False)."""
        return self._touched or (self._watch_enqueues and _lib.enqueue_count() != self._enqueue_mark)

    @_launch_started.setter
    def _launch_started(self, value: bool) -> None:
        self._touched = bool(value)
        self._enqueue_mark = _lib.enqueue_count()

    # -- tables -----------------------------------------------------------------------------------
    def preare_block_tables(self, seqs: Seq[Sequence]) -> torch.Tensor:
        """int32 ``[B, max blocks]`` right-padded with -1 (llava_model_runner.py:541-549; the
        reference spells it this way)."""
        width = max(len(s.block_table) for s in seqs)
        rows = [s.block_table + [-1] * (width - len(s.block_table)) for s in seqs]
        return torch.tensor(rows, dtype=torch.int32, pin_memory=True).to(self.device, non_blocking=True)

    def _table_and_lens(self, tables: Seq[Seq[int]], lens: Seq[int]):
        width = max(len(t) for t in tables)
        tt = torch.tensor([list(t) + [-1] * (width - len(t)) for t in tables], dtype=torch.int32, device=self.device)
        return tt, torch.tensor(list(lens), dtype=torch.int32, device=self.device)

    # -- paged <-> HuggingFace layout ----------------------------------------------------------------
    def _extract_kv_cache_fast(self, block_table: List[int], seq_len: int) -> List[LayerKV]:
        """One ``(K, V)`` pair per layer, each ``[1, Hkv, S, D]``, copied out of the pages."""
        L, H, D = self.num_hidden_layers, self.num_key_value_heads, self.head_dim
        need = -(-seq_len // self.block_size)
        table = [b for b in block_table[:need] if b >= 0]
        seq_len = min(seq_len, len(table) * self.block_size)
        if seq_len == 0:
            return []
        tt, ll = self._table_and_lens([table], [seq_len])
        out = torch.empty((2, L, 1, H, seq_len, D), dtype=self.kv_cache.dtype, device=self.device)
        for p in range(2):
            ops.copy_tokens(_lib.paged_view(self.kv_cache[p], tt, ll, seq_len), _lib.dense_view(out[p]), 0, seq_len, 0)
        return [(out[0, l], out[1, l]) for l in range(L)]

    def _write_compressed_kv_cache_fast(self, compressed_kv: List[LayerKV], block_table: List[int]) -> None:
        """Write ``[1, Hkv, C, D]`` pairs into the leading blocks of ``block_table``; slots past ``C``
        keep their contents."""
        if not compressed_kv:
            return
        C = compressed_kv[0][0].shape[2]
        table = []
        for b in block_table:
            if b < 0:
                break
            table.append(b)
        C = min(C, len(table) * self.block_size)
        if C == 0:
            return
        tt, ll = self._table_and_lens([table], [C])
        for p in range(2):
            dst = _lib.paged_view(self.kv_cache[p], tt, ll, C)
            layers = [kv[p] for kv in compressed_kv]
            if not ops.copy_tokens_from_layers(layers, dst, C):      # one launch straight from the list
                src = torch.stack(layers)                             # [L, 1, Hkv, C, D]: tensors of mixed geometry
                ops.copy_tokens(_lib.dense_view(src), dst, 0, C, 0)

    # -- pages shared between sequences ----------------------------------------------------------------
    def _pages_rewritten(self, comp, seq_len: int, it_len) -> int:
        """How many leading pages an in-place compression of ``seq_len`` rows writes (all of them when the
        compressor cannot say its output length beforehand)."""
        rows = seq_len
        if hasattr(comp, "paged_compressed_len"):
            try:
                rows = min(seq_len, int(comp.paged_compressed_len(seq_len, it_len)))
            except Exception:
                rows = seq_len
        return -(-rows // self.block_size)

    def _isolate_shared_pages(self, seqs: Seq[Sequence], comp, image_len: int) -> int:
        """Full prompt pages of identical content are shared between sequences (prefix cache).  An in-place
        compression rewrites the leading pages of every sequence of the batch in one launch, so a page that has
        another owner, in the batch or not, must first become the sequence's own: with a page manager attached
        the sequence gets a fresh page and the rows are copied (one ``fc_copy_tokens`` launch per plane for all
        such pages); without one, a batch whose tables name a page twice where it would be rewritten is refused.
        Runs before any row is rewritten; returns the number of pages copied."""
        bm = self.block_manager
        writes = [self._pages_rewritten(comp, len(s), [image_len, max(1, len(s) - image_len)]) for s in seqs]
        if bm is None:
            owners: Dict[int, int] = {}
            for s in seqs:
                for b in set(s.block_table):
                    owners[b] = owners.get(b, 0) + 1
            for s, w in zip(seqs, writes):
                for b in s.block_table[:w]:
                    if b >= 0 and owners[b] > 1:
                        raise _lib.FastcacheError(
                            f"page {b} belongs to several sequences of the batch and sequence {s.seq_id} would "
                            "rewrite it in place; attach the page manager (block_manager=) so that it gets its own copy")
            return 0
        # a page shared only inside the batch stays with the last sequence that names it
        owners = {b: bm.blocks[b].ref_count for s in seqs for b in s.block_table if b >= 0}
        plan = []
        for s, w in zip(seqs, writes):
            mine = []
            for i, b in enumerate(s.block_table[:w]):
                if owners[b] > 1:
                    owners[b] -= 1
                    mine.append(i)
            plan.append((s, mine))
        need = sum(len(p) for _, p in plan)
        if need > len(bm.free_block_ids):
            raise _lib.FastcacheError(f"the batch would rewrite {need} pages it shares with other sequences and only "
                                      f"{len(bm.free_block_ids)} pages are free to copy them to")
        moved = []
        for s, positions in plan:
            moved += bm.unshare(s, positions)
        # From the first launch on, the pages about to be rewritten no longer hold the tokens they were published
        # under.  Their content keys leave the prefix cache now, not when the engine later shortens the tables: with
        # the compression on a side stream, a prefill of the same prompt can be scheduled in between.
        if hasattr(bm, "forget_pages"):
            for s, w in zip(seqs, writes):
                bm.forget_pages([b for b in s.block_table[:w] if b >= 0])
        if moved:
            old = [[a] for a, _ in moved]
            new = [[b] for _, b in moved]
            n = self.block_size
            t_old, ll = self._table_and_lens(old, [n] * len(moved))
            t_new, _ = self._table_and_lens(new, [n] * len(moved))
            for p in range(2):
                ops.copy_tokens(_lib.paged_view(self.kv_cache[p], t_old, ll, n),
                                _lib.paged_view(self.kv_cache[p], t_new, ll, n), 0, n, 0)
        return len(moved)

    # -- compression ---------------------------------------------------------------------------------
    def _active_compressor(self):
        if self.use_batched_compressor and self.batched_compressor is not None:
            return self.batched_compressor
        return self.compressor

    def _compress_enqueue(self, seqs: Seq[Sequence], image_len: int) -> Tuple[int, int]:
        """Enqueue the compression of ``seqs`` on the current stream and update the bookkeeping;
        returns (elements before, elements after)."""
        comp = self._active_compressor()
        L, H, D = self.num_hidden_layers, self.num_key_value_heads, self.head_dim
        orig = after = 0
        result: Dict[int, int] = {}
        if hasattr(comp, "paged_forward"):
            # every sequence of the batch in the same launches, whatever their lengths: the kernels take each
            # sequence's length (and, for the MLPs, its segments) from device arrays
            lens = [len(s) for s in seqs]
            S = max(lens)
            self._isolate_shared_pages(seqs, comp, image_len)           # may edit the tables
            tt, ll = self._table_and_lens([s.block_table for s in seqs], lens)
            it_len = [image_len, max(1, S - image_len)]
            # from here on every successful enqueue counts: a failure after one may leave rows partly rewritten, a
            # failure in the host-side checks before it leaves the cache as it was
            self._watch_enqueues = True
            self._launch_started = False
            extra = {"seq_ids": [s.seq_id for s in seqs]} if getattr(comp, "wants_seq_ids", False) else {}
            C = comp.paged_forward(self.kv_cache, tt, ll, S, it_len, host_lens=lens, **extra)
            per_seq = list(C) if isinstance(C, (list, tuple)) else [C] * len(seqs)
            for s, n, c in zip(seqs, lens, per_seq):
                result[s.seq_id] = c
                orig += 2 * L * H * D * n
                after += 2 * L * H * D * c
        else:
            self._watch_enqueues = False      # the extracts launch copies that leave the pages alone
            self._isolate_shared_pages(seqs, comp, image_len)
            for s in seqs:
                S = len(s)
                hf = self._extract_kv_cache_fast(s.block_table, S)
                it_len = [image_len, max(1, S - image_len)]
                with torch.no_grad():
                    out = comp(hf, it_len=it_len)
                self._launch_started = True   # the write-back below is the first thing that touches the pages
                self._write_compressed_kv_cache_fast(out, s.block_table)
                result[s.seq_id] = out[0][0].shape[2]
                orig += sum(k.numel() + v.numel() for k, v in hf)
                after += sum(k.numel() + v.numel() for k, v in out)
        with self._lock:
            for s in seqs:
                C = result[s.seq_id]
                self._compressed_lens[s.seq_id] = C
                keep = -(-C // self.block_size)
                if len(s.block_table) > keep:
                    self._blocks_to_free[s.seq_id] = s.block_table[keep:]
        return orig, after

    def compress_kv_cache_batch(self, seqs: List[Sequence], image_len: Optional[int] = None) -> Tuple[float, float]:
        """Compress the KV of ``seqs`` in place; returns ``(seconds, elements before / after)`` after a
        device synchronisation (llava_model_runner.py:712-793)."""
        if self._active_compressor() is None:
            return 0.0, 1.0
        if image_len is None:
            image_len = self.image_token_len
        t0 = time.time()
        orig, after = self._compress_enqueue(seqs, image_len)
        torch.cuda.synchronize()
        return time.time() - t0, (orig / after if after > 0 else 1.0)

    def get_blocks_to_free(self, seq_id: int) -> List[int]:
        return self._blocks_to_free.pop(seq_id, [])

    def get_compressed_block_count(self, seq_id: int) -> int:
        if seq_id not in self._compressed_lens:
            return -1
        return -(-self._compressed_lens[seq_id] // self.block_size)

    def clear_compressed_lens(self, seq_ids: Optional[List[int]] = None) -> None:
        with self._lock:
            if seq_ids is None:
                self._compressed_lens.clear()
            else:
                for i in seq_ids:
                    self._compressed_lens.pop(i, None)

    # -- asynchronous variant: one side stream, two events --------------------------------------------
    def start_background_compression(self, seqs: List[Sequence], image_len: Optional[int] = None):
        """Enqueue the compression on the side stream behind everything already on the current stream;
        returns the event that fires when it is done (llava_model_runner.py:1046-1094).  Bookkeeping
        is updated immediately; consumers must ``wait_compression`` before touching those sequences."""
        if self._active_compressor() is None:
            return None
        if image_len is None:
            image_len = self.image_token_len
        if self._compress_stream is None:
            self._compress_stream = torch.cuda.Stream(device=self.device)
        ready = torch.cuda.Event()
        ready.record()
        self._compress_stream.wait_event(ready)
        with torch.cuda.stream(self._compress_stream):
            self._compress_enqueue(seqs, image_len)
            done = torch.cuda.Event()
            done.record(self._compress_stream)
        return done

    def wait_compression(self, event) -> None:
        if event is not None:
            event.synchronize()

    # -- decode metadata ------------------------------------------------------------------------------
    def prepare_decode(self, seqs: List[Sequence]):
        """``positions = context_lens = kv_cache_len``; the new token's slot is position ``kv_cache_len``
        of the sequence (llava_model_runner.py:637-674)."""
        input_ids, positions, slots, lens = [], [], [], []
        for s in seqs:
            n = s.kv_cache_len
            input_ids.append(s.last_token)
            positions.append(n)
            lens.append(n)
            bi, pos = divmod(n, self.block_size)
            blk = s.block_table[bi] if bi < len(s.block_table) else s.block_table[-1]
            slots.append(blk * self.block_size + pos)
        mk = lambda x, dt: torch.tensor(x, dtype=dt, pin_memory=True).to(self.device, non_blocking=True)
        input_ids, positions = mk(input_ids, torch.int64), mk(positions, torch.int64)
        set_context(False, slot_mapping=mk(slots, torch.int32), context_lens=mk(lens, torch.int32),
                    block_tables=self.preare_block_tables(seqs))
        return input_ids, positions
