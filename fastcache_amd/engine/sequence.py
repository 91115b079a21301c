"""A request as the scheduler, the page manager and the compression hooks see it.

Attribute and property names are nano-vllm's (nanovllm/engine/sequence.py:14-98): its scheduler, block manager and
model runner read them by name, and the compression path adds ``kv_cache_len`` / ``is_compressed`` /
``kv_num_blocks`` on top.  The state behind them is kept differently here: the tokens, and how many KV rows the
cache holds MORE or FEWER than there are tokens (``_kv_delta``, ``None`` until the first compression), so that
appending a token never has to touch the compression state.
"""
from __future__ import annotations

import itertools
from enum import Enum, auto
from typing import List, Optional


class SequenceStatus(Enum):
    WAITING = auto()
    RUNNING = auto()
    FINISHED = auto()


_ids = itertools.count()


def _pages(n_tokens: int, page: int) -> int:
    return (n_tokens + page - 1) // page


class Sequence:
    block_size = 256          # tokens per page; class-wide, as in the reference

    def __init__(self, token_ids: List[int], sampling_params=None):
        self.seq_id = next(_ids)
        self.status = SequenceStatus.WAITING
        self.token_ids = list(token_ids)
        self.num_prompt_tokens = len(self.token_ids)
        self.block_table: List[int] = []
        self.num_cached_tokens = 0                 # prompt tokens found in the prefix cache (whole pages)
        self._kv_delta: Optional[int] = None       # cache rows minus tokens; None = not compressed
        params = sampling_params
        self.temperature = 1.0 if params is None else getattr(params, "temperature", 1.0)
        self.max_tokens = 64 if params is None else getattr(params, "max_tokens", 64)
        self.ignore_eos = False if params is None else getattr(params, "ignore_eos", False)

    # -- tokens ----------------------------------------------------------------------------------------
    def __len__(self) -> int:
        return len(self.token_ids)

    def __getitem__(self, key):
        return self.token_ids[key]

    def __lt__(self, other: "Sequence") -> bool:
        return self.seq_id < other.seq_id

    def append_token(self, token_id: int) -> None:
        """One more token and, with it, one more cache row (compressed or not: the delta stays)."""
        self.token_ids.append(token_id)

    @property
    def last_token(self) -> int:
        return self.token_ids[-1]

    @property
    def num_completion_tokens(self) -> int:
        return len(self.token_ids) - self.num_prompt_tokens

    # -- pages of tokens (prefill allocation, prefix cache) -----------------------------------------------------
    @property
    def num_blocks(self) -> int:
        return _pages(len(self.token_ids), self.block_size)

    @property
    def num_cached_blocks(self) -> int:
        return self.num_cached_tokens // self.block_size

    def block(self, i: int) -> List[int]:
        lo = i * self.block_size
        return self.token_ids[lo:lo + self.block_size]

    def last_block(self) -> List[int]:
        return self.block(self.num_blocks - 1)

    # -- cache rows (decode-time growth, compression) -----------------------------------------------------------
    @property
    def is_compressed(self) -> bool:
        return self._kv_delta is not None

    @property
    def kv_cache_len(self) -> int:
        """Rows the cache really holds: the token count, or after a compression the compressed length plus the
        tokens generated since."""
        return len(self.token_ids) + (self._kv_delta or 0)

    @kv_cache_len.setter
    def kv_cache_len(self, rows: int) -> None:
        self._kv_delta = rows - len(self.token_ids)

    @property
    def _kv_cache_len(self) -> Optional[int]:
        """The reference's private field: the overriding length, ``None`` while uncompressed."""
        return None if self._kv_delta is None else self.kv_cache_len

    @_kv_cache_len.setter
    def _kv_cache_len(self, rows: Optional[int]) -> None:
        self._kv_delta = None if rows is None else rows - len(self.token_ids)

    @property
    def kv_num_blocks(self) -> int:
        return _pages(self.kv_cache_len, self.block_size)
