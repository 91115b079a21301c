"""Compressions that run beside decoding, tracked per sequence.

The protocol is the reference's (``CompressionState`` / ``AsyncCompressionManager``,
nanovllm/engine/llava_model_runner.py:33-196, and ``PipelineAsyncCompressor``,
nanovllm/kernels/batched_compress.py:660-819): work goes to a side stream behind whatever the submitting stream
already holds, every sequence has a state and a completion event, and its compressed length counts as its KV
length only after that event has fired.  The arrangement is this build's: one ``_Ticket`` record per sequence
instead of parallel dictionaries, one enqueue for the whole batch (the paged kernels take sequences of any
lengths together), and a failure mode the in-place kernels need: a compression that fails after its first launch
has rewritten part of the sequence's rows, so that sequence is marked ``FAILED`` and must be prefilled again; only a
failure before any launch leaves the cache intact (state ``NONE``, the reference's "carry on uncompressed").
All streams have the default priority.
"""
from __future__ import annotations

import threading
from dataclasses import dataclass
from enum import Enum
from typing import Callable, Dict, Iterable, List, Optional

import torch

from .._lib import FastcacheError


class CompressionState(Enum):
    NONE = 0          # not compressed (never submitted, or the attempt failed before touching the cache)
    PENDING = 1       # submitted, not yet enqueued
    IN_PROGRESS = 2   # being enqueued on the side stream
    COMPLETED = 3     # enqueued; finished on the device once the sequence's event has fired
    FAILED = 4        # failed after launches were enqueued: the sequence's cache rows are not trustworthy


@dataclass
class _Ticket:
    original_len: int
    state: CompressionState = CompressionState.PENDING
    compressed_len: Optional[int] = None
    done: Optional[torch.cuda.Event] = None

    def finished_on_device(self) -> bool:
        return self.state is CompressionState.COMPLETED and (self.done is None or self.done.query())


class _TicketBook:
    """Thread-safe map seq_id -> ticket with the read-only views the reference's attribute names offer."""

    def __init__(self):
        self._lock = threading.Lock()
        self._tickets: Dict[int, _Ticket] = {}

    def open(self, seq_id: int, original_len: int) -> _Ticket:
        with self._lock:
            t = self._tickets[seq_id] = _Ticket(original_len)
            return t

    def get(self, seq_id: int) -> Optional[_Ticket]:
        with self._lock:
            return self._tickets.get(seq_id)

    def set_state(self, seq_ids: Iterable[int], state: CompressionState) -> None:
        with self._lock:
            for i in seq_ids:
                if i in self._tickets:
                    self._tickets[i].state = state

    def drop(self, seq_id: int) -> None:
        with self._lock:
            self._tickets.pop(seq_id, None)

    def column(self, field: str) -> dict:
        with self._lock:
            return {i: getattr(t, field) for i, t in self._tickets.items() if getattr(t, field) is not None}


class AsyncCompressionManager:
    """``model_runner`` is a ``PagedKVRunner`` (or any object with ``compressor``, ``_compressed_lens`` and
    ``_compress_enqueue(seqs, image_len)``).  A runner may set ``_launch_started`` before its first launch; a
    failure with that flag set marks the batch ``FAILED`` instead of ``NONE``."""

    def __init__(self, model_runner):
        self.model_runner = model_runner
        self.compress_stream = torch.cuda.Stream()
        self._book = _TicketBook()

    # the reference's dictionaries, as snapshots
    @property
    def seq_states(self) -> Dict[int, CompressionState]:
        return self._book.column("state")

    @property
    def seq_original_lens(self) -> Dict[int, int]:
        return self._book.column("original_len")

    @property
    def seq_compressed_lens(self) -> Dict[int, int]:
        return self._book.column("compressed_len")

    @property
    def compress_events(self) -> Dict[int, torch.cuda.Event]:
        return self._book.column("done")

    def start_async_compression(self, seqs: List, image_len: int = 0):
        """Enqueue the compression of ``seqs`` on the side stream, ordered behind the current stream's work."""
        runner = self.model_runner
        if getattr(runner, "compressor", None) is None and getattr(runner, "batched_compressor", None) is None:
            return
        tickets = [self._book.open(s.seq_id, len(s)) for s in seqs]
        ids = [s.seq_id for s in seqs]
        fence = torch.cuda.Event()
        fence.record()
        self.compress_stream.wait_event(fence)
        with torch.cuda.stream(self.compress_stream):
            self._book.set_state(ids, CompressionState.IN_PROGRESS)
            if hasattr(runner, "_launch_started"):
                runner._launch_started = False
            try:
                runner._compress_enqueue(seqs, image_len)
            except Exception as e:
                touched = bool(getattr(runner, "_launch_started", False))
                self._book.set_state(ids, CompressionState.FAILED if touched else CompressionState.NONE)
                print(f"async compression failed for sequences {ids} "
                      f"({'cache rows partly rewritten: prefill them again' if touched else 'cache untouched'}): {e}")
                return
            done = torch.cuda.Event()
            done.record(self.compress_stream)
            for s, t in zip(seqs, tickets):
                t.compressed_len = runner._compressed_lens[s.seq_id]
                t.done = done
            self._book.set_state(ids, CompressionState.COMPLETED)

    def is_compression_complete(self, seq_id: int) -> bool:
        t = self._book.get(seq_id)
        return t is not None and t.finished_on_device()

    def wait_for_compression(self, seq_id: int, timeout_ms: float = 1000) -> None:
        t = self._book.get(seq_id)
        if t is not None and t.done is not None:
            t.done.synchronize()

    def wait_all_compressions(self) -> None:
        self.compress_stream.synchronize()

    def get_effective_kv_len(self, seq) -> int:
        """The compressed length once the sequence's event has fired, its original length before.  A sequence
        whose compression failed half-way has no valid length: that raises."""
        t = self._book.get(seq.seq_id)
        if t is None:
            return len(seq)
        if t.state is CompressionState.FAILED:
            raise FastcacheError(f"sequence {seq.seq_id}: compression failed after rewriting part of its cache; "
                                 "pre-empt it and prefill again")
        if t.finished_on_device() and t.compressed_len is not None:
            return t.compressed_len
        return t.original_len

    def cleanup_seq(self, seq_id: int) -> None:
        self._book.drop(seq_id)


class PipelineAsyncCompressor:
    """``num_streams`` side streams taken in turn, so that the compression of one request overlaps the prefill of
    the next.  The compressor is called on an extracted HuggingFace-layout list and its result handed to
    ``write_callback(compressed_kv, block_table)``; the source pages are only overwritten by that callback, so a
    failure before it leaves them intact (state ``NONE``)."""

    def __init__(self, compressor, num_streams: int = 2):
        self.compressor = compressor
        self.num_streams = num_streams
        self.compress_streams = [torch.cuda.Stream() for _ in range(num_streams)]
        self.current_stream_idx = 0
        self._book = _TicketBook()

    @property
    def seq_states(self) -> Dict[int, CompressionState]:
        return self._book.column("state")

    @property
    def seq_events(self) -> Dict[int, torch.cuda.Event]:
        return self._book.column("done")

    @property
    def seq_compressed_lens(self) -> Dict[int, int]:
        return self._book.column("compressed_len")

    def _get_next_stream(self) -> torch.cuda.Stream:
        stream = self.compress_streams[self.current_stream_idx % self.num_streams]
        self.current_stream_idx = (self.current_stream_idx + 1) % self.num_streams
        return stream

    def submit_compression(self, seq_id: int, kv_cache, block_table: List[int], original_seq_len: int,
                           it_len: List[int], write_callback: Callable) -> torch.cuda.Event:
        """Returns the event that fires when this request's compression and write-back are done."""
        ticket = self._book.open(seq_id, original_seq_len)
        stream = self._get_next_stream()
        fence = torch.cuda.Event()
        fence.record()
        stream.wait_event(fence)
        with torch.cuda.stream(stream):
            ticket.state = CompressionState.IN_PROGRESS
            written = False
            try:
                with torch.no_grad():
                    result = self.compressor(kv_cache, it_len=it_len)
                written = True
                write_callback(result, block_table)
                ticket.compressed_len = result[0][0].shape[2]
                ticket.state = CompressionState.COMPLETED
            except Exception as e:
                ticket.state = CompressionState.FAILED if written else CompressionState.NONE
                print(f"async compression failed seq_id={seq_id}: {e}")
            ticket.done = torch.cuda.Event()
            ticket.done.record(stream)
        return ticket.done

    def is_compression_ready(self, seq_id: int) -> bool:
        t = self._book.get(seq_id)
        return t is not None and t.finished_on_device()

    def wait_compression(self, seq_id: int) -> None:
        t = self._book.get(seq_id)
        if t is not None and t.done is not None:
            t.done.synchronize()

    def get_compressed_len(self, seq_id: int) -> Optional[int]:
        t = self._book.get(seq_id)
        return None if t is None else t.compressed_len

    def cleanup(self, seq_id: int) -> None:
        self._book.drop(seq_id)
