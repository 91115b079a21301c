"""``Sequence`` with the compression-aware KV length (nanovllm/engine/sequence.py:14-98)."""
from __future__ import annotations

import itertools
from enum import Enum, auto
from typing import List, Optional


class SequenceStatus(Enum):
    WAITING = auto()
    RUNNING = auto()
    FINISHED = auto()


class Sequence:
    """A request's tokens, its block table and, once compressed, the number of KV rows it really
    holds (``kv_cache_len``), which then grows by one per generated token."""

    block_size = 256
    counter = itertools.count()

    def __init__(self, token_ids: List[int], sampling_params=None):
        self.seq_id = next(Sequence.counter)
        self.status = SequenceStatus.WAITING
        self.token_ids = list(token_ids)
        self.num_prompt_tokens = len(self.token_ids)
        self._num_cached_tokens = 0
        self.block_table: List[int] = []
        self.temperature = getattr(sampling_params, "temperature", 1.0)
        self.max_tokens = getattr(sampling_params, "max_tokens", 64)
        self.ignore_eos = getattr(sampling_params, "ignore_eos", False)
        self._kv_cache_len: Optional[int] = None      # None = not compressed

    def __len__(self):
        return len(self.token_ids)

    def __lt__(self, other):
        return self.seq_id < other.seq_id

    def __getitem__(self, key):
        return self.token_ids[key]

    @property
    def num_completion_tokens(self) -> int:
        return len(self.token_ids) - self.num_prompt_tokens

    @property
    def num_cached_tokens(self) -> int:
        return self._num_cached_tokens

    @num_cached_tokens.setter
    def num_cached_tokens(self, n: int):
        assert n % self.block_size == 0
        self._num_cached_tokens = n

    @property
    def num_cached_blocks(self) -> int:
        return self._num_cached_tokens // self.block_size

    @property
    def num_blocks(self) -> int:
        return -(-len(self.token_ids) // self.block_size)

    @property
    def last_token(self) -> int:
        return self.token_ids[-1]

    def block(self, i: int) -> List[int]:
        return self.token_ids[i * self.block_size:(i + 1) * self.block_size]

    def last_block(self) -> List[int]:
        return self.token_ids[(self.num_blocks - 1) * self.block_size:]

    def append_token(self, token_id: int) -> None:
        self.token_ids.append(token_id)
        if self._kv_cache_len is not None:
            self._kv_cache_len += 1

    # -- compression state ---------------------------------------------------------------------
    @property
    def kv_cache_len(self) -> int:
        return len(self.token_ids) if self._kv_cache_len is None else self._kv_cache_len

    @kv_cache_len.setter
    def kv_cache_len(self, value: int):
        self._kv_cache_len = value

    @property
    def is_compressed(self) -> bool:
        return self._kv_cache_len is not None

    @property
    def kv_num_blocks(self) -> int:
        return -(-self.kv_cache_len // self.block_size)
