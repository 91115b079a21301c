"""Oracle (test infrastructure): the per-sequence compression driver of the reference, on the CPU.

``compress_batch`` restates ``LlavaModelRunner.compress_kv_cache_batch``
(nanovllm/engine/llava_model_runner.py:712-793): for every sequence, extract its KV from the
pages, run the compressor on the HuggingFace-layout list, write the result back into the leading
pages, and record the compressed length and the blocks that became free.
"""
from __future__ import annotations

from typing import Callable, Dict, List, Sequence, Tuple

import torch

from . import paged, presses

LayerKV = Tuple[torch.Tensor, torch.Tensor]
Compressor = Callable[[List[LayerKV], int, int], List[LayerKV]]   # (hf_kv, seq_index, seq_len) -> hf_kv


def compress_batch(kv_cache: torch.Tensor, block_tables: Sequence[Sequence[int]], seq_lens: Sequence[int],
                   compressor: Compressor) -> Tuple[Dict[int, int], Dict[int, List[int]], float]:
    """Returns ``(compressed_lens, blocks_to_free, ratio)`` keyed by sequence index
    (llava_model_runner.py:745-791)."""
    block_size = kv_cache.shape[3]
    compressed_lens: Dict[int, int] = {}
    to_free: Dict[int, List[int]] = {}
    orig = comp = 0
    for i, (table, n) in enumerate(zip(block_tables, seq_lens)):
        hf = paged.extract_kv(kv_cache, table, n)                       # :751
        orig += sum(k.numel() + v.numel() for k, v in hf)               # :754
        out = compressor(hf, i, n)                                      # :763-766
        comp += sum(k.numel() + v.numel() for k, v in out)              # :769
        c = out[0][0].shape[2]                                          # :770
        paged.write_back(kv_cache, out, table)                          # :774
        compressed_lens[i] = c                                          # :777
        keep = (c + block_size - 1) // block_size                       # :780
        if len(table) > keep:                                           # :782-786
            to_free[i] = list(table[keep:])
    return compressed_lens, to_free, (orig / comp if comp else 1.0)     # :791


def knorm_press_compressor(compression_ratio: float) -> Compressor:
    """Per-layer ``KnormPress.compress`` (kvpress) in the hook order of
    utils_ccm/utils_compress.py:209-270."""
    def run(hf, i, n):
        out = []
        for k, v in hf:
            ck, cv, _ = presses.press_compress(k, v, presses.knorm_score(k), compression_ratio)
            out.append((ck, cv))
        return out
    return run


def snapkv_press_compressor(queries: torch.Tensor, compression_ratio: float, window_size: int,
                            kernel_size: int, causal_window: bool = True, reduction: str = "mean",
                            window_in_budget: bool = True) -> Compressor:
    """Per-layer ``SnapKVPress.compress``; queries ``[L, B, Hq, W, D]`` indexed by layer and sequence.  With
    ``window_in_budget=False`` the window is kept on top of ``int(S * (1 - r))``."""
    def run(hf, i, n):
        out = []
        for layer, (k, v) in enumerate(hf):
            sc = presses.snapkv_score(queries[layer, i:i + 1], k, window_size, kernel_size, causal_window,
                                      reduction)
            ck, cv, _ = presses.press_compress(k, v, sc, compression_ratio,
                                               0 if window_in_budget else window_size)
            out.append((ck, cv))
        return out
    return run


def scored_press_compressor(score_fn, compression_ratio: float) -> Compressor:
    """Any kvpress ``ScorerPress``: ``score_fn(layer, seq_index, keys, values) -> [1, Hkv, S]`` fp32, then
    ``ScorerPress.compress``."""
    def run(hf, i, n):
        out = []
        for layer, (k, v) in enumerate(hf):
            ck, cv, _ = presses.press_compress(k, v, score_fn(layer, i, k, v), compression_ratio)
            out.append((ck, cv))
        return out
    return run
