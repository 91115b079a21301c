"""Score -> select -> compact over a paged KV pool, all layers and sequences per launch.

This is the fused counterpart of the reference's per-sequence loop
``_extract_kv_cache_fast`` -> press -> ``_write_compressed_kv_cache_fast``
(nanovllm/engine/llava_model_runner.py:712-793): K is scored where it lies in its pages, the kept
indices are selected per (layer, sequence, kv head) and the kept K/V rows are moved to the front
of the same pages in place.  Three launches per pass, nothing leaves the device.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence

import torch

from . import _lib, ops


@dataclass
class PressResult:
    indices: torch.Tensor          # int32 [L, B, Hkv (or 1), n_kept] ascending token positions (-1 past a row's count)
    n_kept: int                    # kept tokens per sequence (the largest count when the sequences differ)
    scores: Optional[torch.Tensor]  # fp32 [L, B, Hkv, S] (None for index-only presses)
    kept_per_seq: Optional[List[int]] = None    # set when the sequences have different lengths


def n_kept_for(seq_len: int, compression_ratio: float) -> int:
    """kvpress ``ScorerPress.compress``: ``int(q_len * (1 - compression_ratio))``, in double."""
    return int(seq_len * (1 - compression_ratio))


def _views(kv_cache: torch.Tensor, block_tables: torch.Tensor, seq_lens: torch.Tensor, max_seq_len: int):
    if kv_cache.dim() != 6 or kv_cache.shape[0] != 2:
        raise _lib.FastcacheError("kv_cache must be [2, L, num_blocks, block_size, Hkv, D]")
    return (_lib.paged_view(kv_cache[0], block_tables, seq_lens, max_seq_len),
            _lib.paged_view(kv_cache[1], block_tables, seq_lens, max_seq_len))


def _select_and_compact(kview, vview, scores, seq_lens, kept: List[int], compact: bool, heads: int) -> PressResult:
    """Top-k per (layer, sequence, head) row and in-place compaction; one launch each whether or not the
    sequences keep the same number of tokens."""
    width = max(kept)
    one_launch = (compact and width > 0 and ops.press_column_fits(kview.max_seq_len, width) and scores.dim() == 4 and
                  scores.shape[2] == kview.num_kv_heads and scores.is_contiguous())
    if one_launch:       # selection and compaction of a column by one workgroup
        if len(set(kept)) == 1:
            return PressResult(ops.select_compact(kview, vview, scores, width), width, scores)
        n_kept = torch.tensor(kept, dtype=torch.int32, device=scores.device)
        return PressResult(ops.select_compact(kview, vview, scores, width, n_kept=n_kept), width, scores, list(kept))
    if len(set(kept)) == 1:
        idx = ops.topk_select(scores, width)
        if compact and width > 0:
            ops.compact(kview, vview, kview, vview, idx)
        return PressResult(idx, width, scores)
    n_kept = torch.tensor(kept, dtype=torch.int32, device=scores.device)
    idx = ops.topk_select(scores, width, row_lens=seq_lens, n_kept=n_kept, rows_per_len=heads)
    if compact and width > 0:
        ops.compact(kview, vview, kview, vview, idx, n_kept=n_kept)
    return PressResult(idx, width, scores, list(kept))


def knorm_compress_paged(kv_cache: torch.Tensor, block_tables: torch.Tensor, seq_lens: torch.Tensor,
                         seq_len: int, compression_ratio: float, compact: bool = True,
                         host_lens: Optional[Sequence[int]] = None) -> PressResult:
    """KnormPress over sequences that all hold ``seq_len`` tokens, or, with ``host_lens`` (the lengths as
    Python ints, ``seq_len`` their maximum), over sequences of different lengths in the same launches: each keeps
    ``int(its length * (1 - compression_ratio))`` tokens."""
    kview, vview = _views(kv_cache, block_tables, seq_lens, seq_len)
    lens = list(host_lens) if host_lens is not None else [seq_len] * block_tables.shape[0]
    kept = [n_kept_for(n, compression_ratio) for n in lens]
    width = max(kept)
    if compact and 0 < width and ops.press_column_fits(seq_len, width):
        # one launch: every (layer, sequence, head) column is scored, selected and compacted by one workgroup
        if len(set(kept)) == 1:
            scores, idx = ops.knorm_press(kview, vview, width, kv_cache.device)
            return PressResult(idx, width, scores)
        n_kept = torch.tensor(kept, dtype=torch.int32, device=kv_cache.device)
        scores, idx = ops.knorm_press(kview, vview, width, kv_cache.device, n_kept=n_kept)
        return PressResult(idx, width, scores, list(kept))
    scores = ops.knorm_score(kview, kv_cache.device)
    return _select_and_compact(kview, vview, scores, seq_lens, kept, compact, kv_cache.shape[4])


def snapkv_compress_paged(kv_cache: torch.Tensor, block_tables: torch.Tensor, seq_lens: torch.Tensor,
                          seq_len: int, queries: torch.Tensor, compression_ratio: float, window_size: int = 64,
                          kernel_size: int = 5, causal_window: bool = True, reduction: str = "mean",
                          window_in_budget: bool = True, compact: bool = True,
                          host_lens: Optional[Sequence[int]] = None) -> PressResult:
    """SnapKVPress over sequences that all hold ``seq_len`` tokens, or (``host_lens``) of different lengths in
    the same launches.  ``queries`` are the rotated window queries ``[L, B, Hq, W, D]`` (the last W positions of
    every sequence).  With ``window_in_budget`` (kvpress) the observation window counts towards ``n_kept``;
    otherwise it is kept on top of it."""
    kview, vview = _views(kv_cache, block_tables, seq_lens, seq_len)
    lens = list(host_lens) if host_lens is not None else [seq_len] * block_tables.shape[0]
    kept = [n_kept_for(n, compression_ratio) for n in lens]
    if not window_in_budget:
        kept = [min(n, k + window_size) for n, k in zip(lens, kept)]
    width = max(kept)
    # The workgroup that scored a column also selects and compacts it when every row keeps more than the window
    # (sequences no longer than the window keep their first positions either way).  In that launch the window positions
    # rank above every scored key, while after the window fill they TIE with scored keys that equal the layer's largest
    # score; the two selections differ only when more such keys than a row has places outside the window tie exactly,
    # which needs equal scores at the very top: rows with fewer scored keys than the pooling kernel is wide (every pooled
    # score the same) take the separate launches.
    if (compact and all(k > window_size or n <= window_size for n, k in zip(lens, kept)) and width > window_size and
            all(n <= window_size or n - window_size > kernel_size for n in lens) and
            ops.snapkv_press_fits(kview, queries.shape[-3], window_size, width) and
            ops.snapkv_press_preferred(kview, queries.shape[-3], window_size,
                                       torch.cuda.get_device_properties(kv_cache.device).multi_processor_count)):
        same = len(set(kept)) == 1 and len(set(lens)) == 1
        scores, idx = ops.snapkv_press(kview, vview, queries, window_size, kernel_size, width, causal_window,
                                       reduction, seq_lens=seq_lens, n_kept=None if same else kept, host_lens=lens)
        return PressResult(idx, width, scores, None if same else list(kept))
    scores = ops.snapkv_score(kview, queries, window_size, kernel_size, causal_window, reduction,
                              seq_lens=seq_lens)
    return _select_and_compact(kview, vview, scores, seq_lens, kept, compact, kv_cache.shape[4])
