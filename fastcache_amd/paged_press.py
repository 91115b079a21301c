"""Score -> select -> compact over a paged KV pool, all layers and sequences per launch.

This is the fused counterpart of the reference's per-sequence loop
``_extract_kv_cache_fast`` -> press -> ``_write_compressed_kv_cache_fast``
(nanovllm/engine/llava_model_runner.py:712-793): K is scored where it lies in its pages, the kept
indices are selected per (layer, sequence, kv head) and the kept K/V rows are moved to the front
of the same pages in place.  Three launches per pass, nothing leaves the device.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from . import _lib, ops


@dataclass
class PressResult:
    indices: torch.Tensor          # int32 [L, B, Hkv (or 1), n_kept] ascending token positions
    n_kept: int
    scores: Optional[torch.Tensor]  # fp32 [L, B, Hkv, S] (None for index-only presses)


def n_kept_for(seq_len: int, compression_ratio: float) -> int:
    """kvpress ``ScorerPress.compress``: ``int(q_len * (1 - compression_ratio))``, in double."""
    return int(seq_len * (1 - compression_ratio))


def _views(kv_cache: torch.Tensor, block_tables: torch.Tensor, seq_lens: torch.Tensor, max_seq_len: int):
    if kv_cache.dim() != 6 or kv_cache.shape[0] != 2:
        raise _lib.FastcacheError("kv_cache must be [2, L, num_blocks, block_size, Hkv, D]")
    return (_lib.paged_view(kv_cache[0], block_tables, seq_lens, max_seq_len),
            _lib.paged_view(kv_cache[1], block_tables, seq_lens, max_seq_len))


def knorm_compress_paged(kv_cache: torch.Tensor, block_tables: torch.Tensor, seq_lens: torch.Tensor,
                         seq_len: int, compression_ratio: float, compact: bool = True) -> PressResult:
    """KnormPress over sequences that all hold ``seq_len`` tokens."""
    kview, vview = _views(kv_cache, block_tables, seq_lens, seq_len)
    scores = ops.knorm_score(kview, kv_cache.device)
    n = n_kept_for(seq_len, compression_ratio)
    idx = ops.topk_select(scores, n)
    if compact and n > 0:
        ops.compact(kview, vview, kview, vview, idx)
    return PressResult(idx, n, scores)


def snapkv_compress_paged(kv_cache: torch.Tensor, block_tables: torch.Tensor, seq_lens: torch.Tensor,
                          seq_len: int, queries: torch.Tensor, compression_ratio: float, window_size: int = 64,
                          kernel_size: int = 5, causal_window: bool = True, reduction: str = "mean",
                          window_in_budget: bool = True, compact: bool = True) -> PressResult:
    """SnapKVPress over sequences that all hold ``seq_len`` tokens.  ``queries`` are the rotated
    window queries ``[L, B, Hq, W, D]``.  With ``window_in_budget`` (kvpress) the observation window
    counts towards ``n_kept``; otherwise it is kept on top of it."""
    kview, vview = _views(kv_cache, block_tables, seq_lens, seq_len)
    scores = ops.snapkv_score(kview, queries, window_size, kernel_size, causal_window, reduction,
                              seq_lens=seq_lens)
    n = n_kept_for(seq_len, compression_ratio)
    if not window_in_budget:
        n = min(seq_len, n + window_size)
    idx = ops.topk_select(scores, n)
    if compact and n > 0:
        ops.compact(kview, vview, kview, vview, idx)
    return PressResult(idx, n, scores)
