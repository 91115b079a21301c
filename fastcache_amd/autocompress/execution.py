"""The two streams of the compress-beside-decode schedule (the role of the reference's ``StreamManager``,
nanovllm/autocompress/execution.py:438-500).

Both streams have the default priority: the reference asks for a low-priority side stream, which this platform
does not mix reliably with default-priority work; the order between the streams comes from events either way.
"""
from __future__ import annotations

from typing import Optional

import torch


class StreamManager:
    """Created lazily on first use, so that importing the package never touches the GPU."""

    def __init__(self):
        self._streams: Optional[tuple] = None        # (main, compress)

    def _pair(self) -> tuple:
        if self._streams is None:
            if not torch.cuda.is_available():
                return (None, None)
            self._streams = (torch.cuda.current_stream(), torch.cuda.Stream())
        return self._streams

    def initialize(self) -> None:
        self._pair()

    def get_main_stream(self):
        return self._pair()[0]

    def get_compress_stream(self):
        return self._pair()[1]

    def synchronize_compress_to_main(self) -> None:
        """Everything enqueued on the compression stream so far happens before what the main stream gets next."""
        main, side = self._pair()
        if side is not None:
            main.wait_event(side.record_event())


_manager: Optional[StreamManager] = None


def get_stream_manager() -> StreamManager:
    global _manager
    if _manager is None:
        _manager = StreamManager()
    return _manager
