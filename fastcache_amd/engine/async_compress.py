"""Per-sequence tracking of compressions that run beside decoding.

Mirrors ``CompressionState`` / ``AsyncCompressionManager`` (nanovllm/engine/llava_model_runner.py:33-196)
and ``PipelineAsyncCompressor`` (nanovllm/kernels/batched_compress.py:660-819): a side stream does the
compression, every sequence has a state and a completion event, and the compressed length becomes the
effective KV length only once that event has fired.  All streams have the default priority.
"""
from __future__ import annotations

import threading
from enum import Enum
from typing import Callable, Dict, List, Optional, Tuple

import torch


class CompressionState(Enum):
    NONE = 0          # not compressed
    PENDING = 1       # handed to the side stream
    IN_PROGRESS = 2   # being enqueued
    COMPLETED = 3     # enqueued; finished on the device once the sequence's event has fired


class AsyncCompressionManager:
    """``model_runner`` is a ``PagedKVRunner`` (or any object with ``compressor``, ``_compressed_lens`` and
    ``_compress_enqueue(seqs, image_len)``)."""

    def __init__(self, model_runner):
        self.model_runner = model_runner
        self.compress_stream = torch.cuda.Stream()
        self.seq_states: Dict[int, CompressionState] = {}
        self.seq_original_lens: Dict[int, int] = {}
        self.seq_compressed_lens: Dict[int, int] = {}
        self.compress_events: Dict[int, torch.cuda.Event] = {}
        self.temp_kv_buffer: Dict[int, list] = {}     # kept for attribute compatibility; compression is in place
        self.lock = threading.Lock()

    def start_async_compression(self, seqs: List, image_len: int = 0):
        """Enqueue the compression of every sequence on the side stream, behind what the current stream
        holds (llava_model_runner.py:73-98)."""
        runner = self.model_runner
        if getattr(runner, "compressor", None) is None and getattr(runner, "batched_compressor", None) is None:
            return
        with self.lock:
            for seq in seqs:
                self.seq_original_lens[seq.seq_id] = len(seq)
                self.seq_states[seq.seq_id] = CompressionState.PENDING
                self.compress_events[seq.seq_id] = torch.cuda.Event()
        ready = torch.cuda.Event()
        ready.record()
        self.compress_stream.wait_event(ready)
        with torch.cuda.stream(self.compress_stream):
            for seq in seqs:
                self._compress_single_seq_async(seq, image_len)

    def _compress_single_seq_async(self, seq, image_len: int):
        seq_id = seq.seq_id
        with self.lock:
            self.seq_states[seq_id] = CompressionState.IN_PROGRESS
        try:
            self.model_runner._compress_enqueue([seq], image_len)
            compressed = self.model_runner._compressed_lens[seq_id]
            with self.lock:
                self.seq_compressed_lens[seq_id] = compressed
                self.seq_states[seq_id] = CompressionState.COMPLETED
                self.compress_events[seq_id].record(self.compress_stream)
        except Exception as e:  # the reference reports and falls back to the uncompressed cache (:137-140)
            print(f"async compression failed seq_id={seq_id}: {e}")
            with self.lock:
                self.seq_states[seq_id] = CompressionState.NONE

    def is_compression_complete(self, seq_id: int) -> bool:
        with self.lock:
            if self.seq_states.get(seq_id, CompressionState.NONE) != CompressionState.COMPLETED:
                return False
            event = self.compress_events.get(seq_id)
            return True if event is None else event.query()

    def wait_for_compression(self, seq_id: int, timeout_ms: float = 1000):
        event = self.compress_events.get(seq_id)
        if event is not None:
            event.synchronize()

    def wait_all_compressions(self):
        self.compress_stream.synchronize()

    def get_effective_kv_len(self, seq) -> int:
        """Compressed length once the sequence's event has fired, the original length before (:169-187)."""
        seq_id = seq.seq_id
        with self.lock:
            if self.seq_states.get(seq_id, CompressionState.NONE) == CompressionState.COMPLETED:
                event = self.compress_events.get(seq_id)
                if event is not None and event.query():
                    return self.seq_compressed_lens.get(seq_id, len(seq))
            return self.seq_original_lens.get(seq_id, len(seq))

    def cleanup_seq(self, seq_id: int):
        with self.lock:
            self.seq_states.pop(seq_id, None)
            self.seq_original_lens.pop(seq_id, None)
            self.seq_compressed_lens.pop(seq_id, None)
            self.compress_events.pop(seq_id, None)
            self.temp_kv_buffer.pop(seq_id, None)


class PipelineAsyncCompressor:
    """Round-robin over ``num_streams`` side streams so that the compression of one request overlaps the
    prefill of the next (batched_compress.py:668-819)."""

    def __init__(self, compressor, num_streams: int = 2):
        self.compressor = compressor
        self.num_streams = num_streams
        self.compress_streams = [torch.cuda.Stream() for _ in range(num_streams)]
        self.current_stream_idx = 0
        self.seq_states: Dict[int, CompressionState] = {}
        self.seq_events: Dict[int, torch.cuda.Event] = {}
        self.seq_compressed_lens: Dict[int, int] = {}
        self.pending_compressions: Dict[int, Tuple] = {}
        self.lock = threading.Lock()

    def _get_next_stream(self) -> torch.cuda.Stream:
        stream = self.compress_streams[self.current_stream_idx]
        self.current_stream_idx = (self.current_stream_idx + 1) % self.num_streams
        return stream

    def submit_compression(self, seq_id: int, kv_cache, block_table: List[int], original_seq_len: int,
                           it_len: List[int], write_callback: Callable) -> torch.cuda.Event:
        """Compress ``kv_cache`` (HF layout) on the next side stream and hand the result to
        ``write_callback(compressed_kv, block_table)``; returns the completion event (:718-787)."""
        with self.lock:
            self.seq_states[seq_id] = CompressionState.PENDING
        stream = self._get_next_stream()
        main_event = torch.cuda.Event()
        main_event.record()
        stream.wait_event(main_event)
        with torch.cuda.stream(stream):
            with self.lock:
                self.seq_states[seq_id] = CompressionState.IN_PROGRESS
            try:
                with torch.no_grad():
                    compressed_kv = self.compressor(kv_cache, it_len=it_len)
                compressed_len = compressed_kv[0][0].shape[2]
                write_callback(compressed_kv, block_table)
                with self.lock:
                    self.seq_compressed_lens[seq_id] = compressed_len
                    self.seq_states[seq_id] = CompressionState.COMPLETED
            except Exception as e:
                print(f"async compression failed seq_id={seq_id}: {e}")
                with self.lock:
                    self.seq_states[seq_id] = CompressionState.NONE
        done_event = torch.cuda.Event()
        done_event.record(stream)
        with self.lock:
            self.seq_events[seq_id] = done_event
        return done_event

    def is_compression_ready(self, seq_id: int) -> bool:
        with self.lock:
            if self.seq_states.get(seq_id, CompressionState.NONE) != CompressionState.COMPLETED:
                return False
            event = self.seq_events.get(seq_id)
            return True if event is None else event.query()

    def wait_compression(self, seq_id: int):
        with self.lock:
            event = self.seq_events.get(seq_id)
        if event is not None:
            event.synchronize()

    def get_compressed_len(self, seq_id: int) -> Optional[int]:
        with self.lock:
            return self.seq_compressed_lens.get(seq_id)

    def cleanup(self, seq_id: int):
        with self.lock:
            self.seq_states.pop(seq_id, None)
            self.seq_events.pop(seq_id, None)
            self.seq_compressed_lens.pop(seq_id, None)
            self.pending_compressions.pop(seq_id, None)
