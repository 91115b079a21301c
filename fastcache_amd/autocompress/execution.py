"""Stream handling for compression beside decoding (reference: nanovllm/autocompress/execution.py:438-500)."""
from __future__ import annotations

from typing import Optional

import torch


class StreamManager:
    """The main stream and one side stream for compression.  Both have the default priority: the
    reference asks for a low-priority side stream, which this platform does not mix reliably with
    default-priority work; ordering is by events either way."""

    def __init__(self):
        self._main_stream = None
        self._compress_stream = None
        self._initialized = False

    def initialize(self):
        if self._initialized:
            return
        if torch.cuda.is_available():
            self._main_stream = torch.cuda.current_stream()
            self._compress_stream = torch.cuda.Stream()
            self._initialized = True

    def get_main_stream(self):
        self.initialize()
        return self._main_stream

    def get_compress_stream(self):
        self.initialize()
        return self._compress_stream

    def synchronize_compress_to_main(self):
        """The main stream waits for everything enqueued on the compression stream so far."""
        if self._compress_stream is not None:
            event = torch.cuda.Event()
            event.record(self._compress_stream)
            self._main_stream.wait_event(event)


_stream_manager: Optional[StreamManager] = None


def get_stream_manager() -> StreamManager:
    global _stream_manager
    if _stream_manager is None:
        _stream_manager = StreamManager()
    return _stream_manager
