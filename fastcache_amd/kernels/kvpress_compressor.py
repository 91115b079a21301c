"""``KVPressCompressor`` (nanovllm/kernels/kvpress_compressor.py:48-336): the nano-vllm adapter with
the ``(kv_cache, it_len)`` call shape of the MLP compressors.

Like the reference it scores with its own rules, not with kvpress objects: ``streaming_llm``
(sinks + recent window), ``knorm`` (largest head-averaged key norms), ``random``, and a uniform
stride for every other method name (``snapkv``, ``h2o``, ``tova``, ``observed_attention``,
``expected_attention``).  One index set per batch row is shared by all heads.  The per-head
kvpress presses are in ``fastcache_amd.presses``.

Difference from the reference: the reference builds a kvpress object before it compresses and so
raises ``ImportError`` when the ``kvpress`` package is absent; this class never imports it.
"""
from __future__ import annotations

from typing import Any, List, Optional, Tuple

import torch
import torch.nn as nn

from .. import _lib, ops

LayerKV = Tuple[torch.Tensor, torch.Tensor]


class KVPressCompressor(nn.Module):
    SUPPORTED_METHODS = ["streaming_llm", "snapkv", "h2o", "knorm", "tova", "random", "observed_attention",
                         "expected_attention"]

    def __init__(self, method: str = "streaming_llm", compression_ratio: float = 0.8, config: Optional[Any] = None,
                 **kwargs):
        super().__init__()
        if method not in self.SUPPORTED_METHODS:
            raise ValueError(f"Unknown method: {method}. Supported: {self.SUPPORTED_METHODS}")
        self.method_name = method
        self.compression_ratio = compression_ratio
        self.config = config
        self.kwargs = kwargs
        src = config if config is not None else None
        get = (lambda name, default: getattr(src, name, default)) if src is not None else \
            (lambda name, default: kwargs.get({"num_hidden_layers": "num_layers", "num_attention_heads": "num_heads",
                                               "num_key_value_heads": "num_kv_heads"}.get(name, name), default))
        self.num_layers = get("num_hidden_layers", 32)
        self.num_heads = get("num_attention_heads", 32)
        self.num_kv_heads = get("num_key_value_heads", self.num_heads)
        self.head_dim = get("head_dim", (getattr(src, "hidden_size", 4096) // self.num_heads) if src is not None else 128)
        self._index_cache = {}

    # -- sizes --------------------------------------------------------------------------------------
    def get_compressed_length(self, original_length: int) -> int:
        return max(int(original_length * (1 - self.compression_ratio)), 1)

    @property
    def compression_factor(self) -> float:
        return 1.0 / (1 - self.compression_ratio)

    # -- index rules that need no scores (host arithmetic, cached on the device) ---------------------
    def _static_indices(self, S: int, n: int, device) -> Optional[torch.Tensor]:
        key = (self.method_name, S, n, device)
        if key in self._index_cache:
            return self._index_cache[key]
        if self.method_name == "streaming_llm":
            sink = min(self.kwargs.get("n_sink", 4), n)
            recent = max(0, n - sink)
            if recent > 0 and S > sink + recent:
                idx = list(range(sink)) + list(range(S - recent, S))
            elif recent > 0:
                idx = list(range(n))
            else:
                idx = list(range(sink))
        else:                                   # uniform stride fallback
            n = min(n, S)
            idx = list(range(0, S, max(1, S // n)))[:n]
        t = torch.tensor(idx, dtype=torch.int32, device=device)
        self._index_cache[key] = t
        return t

    def _compress_layer(self, keys: torch.Tensor, values: torch.Tensor, layer_idx: int,
                        attention_weights: Optional[torch.Tensor] = None) -> LayerKV:
        """keys/values ``[B, Hkv, S, D]`` -> ``[B, Hkv, n_kept, D]`` (kvpress_compressor.py:169-251)."""
        _lib.require_gpu(keys, "keys")
        B, H, S, D = keys.shape
        n = self.get_compressed_length(S)
        if n >= S:
            return keys.contiguous(), values.contiguous()
        dev = keys.device
        kview, vview = _lib.dense_view(keys), _lib.dense_view(values)
        if self.method_name == "knorm":
            n = min(n, S)
            score = ops.knorm_mean_score(kview, dev)            # [1, B, S]
            idx = ops.topk_select(score, n).view(1, B, 1, n)    # largest mean norm, ascending positions
        elif self.method_name == "random":
            n = min(n, S)
            idx = torch.randperm(S, device=dev)[:n].sort().values.to(torch.int32)
            idx = idx.view(1, 1, 1, n).expand(1, B, 1, n).contiguous()
        else:
            t = self._static_indices(S, n, dev)
            n = t.numel()
            idx = t.view(1, 1, 1, n).expand(1, B, 1, n).contiguous()
        out_k = torch.empty((B, H, n, D), dtype=keys.dtype, device=dev)
        out_v = torch.empty_like(out_k)
        ops.compact(kview, vview, _lib.dense_view(out_k), _lib.dense_view(out_v), idx)
        return out_k, out_v

    def paged_compressed_len(self, seq_len: int, it_len=None) -> int:
        n = self.get_compressed_length(seq_len)
        if n >= seq_len:
            return seq_len
        if self.method_name in ("knorm", "random"):
            return n
        return int(self._static_indices(seq_len, n, torch.device("cpu")).numel())

    @torch.no_grad()
    def paged_forward(self, kv_cache: torch.Tensor, block_tables: torch.Tensor, seq_lens: torch.Tensor,
                      seq_len: int, it_len=None, layers: Optional[Tuple[int, int]] = None,
                      out: Optional[torch.Tensor] = None, host_lens=None):
        """The same selection and gather on a paged pool ``[2, L, blocks, block_size, Hkv, D]`` for
        sequences that all hold ``seq_len`` tokens: in place, or for the layers ``layers=(l0, l1)`` only, or
        into ``out [2, L, B, Hkv, C, D]`` leaving the pages untouched; returns the kept length.  Sequences of
        different lengths: ``host_lens`` (Python ints; ``seq_len`` is their maximum) -> the list of kept
        lengths, from the same three launches."""
        if host_lens is not None and len(set(host_lens)) > 1:
            return self._paged_forward_ragged(kv_cache, block_tables, seq_lens, seq_len, list(host_lens), layers, out)
        S = seq_len
        n = self.get_compressed_length(S)
        dev = kv_cache.device
        l0, l1 = layers if layers is not None else (0, kv_cache.shape[1])
        L, B = l1 - l0, block_tables.shape[0]
        kview = _lib.paged_view(kv_cache[0][l0:l1], block_tables, seq_lens, S)
        vview = _lib.paged_view(kv_cache[1][l0:l1], block_tables, seq_lens, S)
        if n >= S:
            if out is not None:
                ops.copy_tokens(kview, _lib.dense_view(out[0][l0:l1]), 0, S, 0)
                ops.copy_tokens(vview, _lib.dense_view(out[1][l0:l1]), 0, S, 0)
            return S
        if self.method_name == "knorm":
            idx = ops.topk_select(ops.knorm_mean_score(kview, dev), n).view(L, B, 1, n)
        elif self.method_name == "random":
            rows = [torch.randperm(S, device=dev)[:n].sort().values.to(torch.int32) for _ in range(L)]
            idx = torch.stack(rows).view(L, 1, 1, n).expand(L, B, 1, n).contiguous()
        else:
            t = self._static_indices(S, n, dev)
            n = t.numel()
            idx = t.view(1, 1, 1, n).expand(L, B, 1, n).contiguous()
        if out is None:
            ops.compact(kview, vview, kview, vview, idx)
        else:
            ops.compact(kview, vview, _lib.dense_view(out[0][l0:l1]), _lib.dense_view(out[1][l0:l1]), idx)
        return n

    def _paged_forward_ragged(self, kv_cache, block_tables, seq_lens, max_len, lens, layers, out):
        """Every sequence keeps ``get_compressed_length(its own length)`` tokens; the index rows are padded to the
        longest with -1 and the kernels take the kept counts from a device array.  A sequence that is not
        shortened keeps all its positions (an identity row)."""
        dev = kv_cache.device
        l0, l1 = layers if layers is not None else (0, kv_cache.shape[1])
        L, B = l1 - l0, block_tables.shape[0]
        kview = _lib.paged_view(kv_cache[0][l0:l1], block_tables, seq_lens, max_len)
        vview = _lib.paged_view(kv_cache[1][l0:l1], block_tables, seq_lens, max_len)
        kept = [self.paged_compressed_len(n) for n in lens]
        width = max(kept)
        n_kept = torch.tensor(kept, dtype=torch.int32, device=dev)
        if self.method_name == "knorm" and any(k < n for k, n in zip(kept, lens)):
            score = ops.knorm_mean_score(kview, dev)                                  # [L, B, S], -inf past each length
            idx = ops.topk_select(score, width, row_lens=seq_lens, n_kept=n_kept).view(L, B, 1, width)
        else:
            rows = torch.full((L, B, width), -1, dtype=torch.int32)
            for b, (n, k) in enumerate(zip(lens, kept)):
                if k >= n:
                    rows[:, b, :n] = torch.arange(n, dtype=torch.int32)
                elif self.method_name == "random":
                    for l in range(L):
                        rows[l, b, :k] = torch.randperm(n)[:k].sort().values.to(torch.int32)
                else:
                    rows[:, b, :k] = self._static_indices(n, self.get_compressed_length(n), torch.device("cpu"))
            idx = rows.view(L, B, 1, width).to(dev)
        if out is None:
            ops.compact(kview, vview, kview, vview, idx, n_kept=n_kept)
        else:
            ops.compact(kview, vview, _lib.dense_view(out[0][l0:l1]), _lib.dense_view(out[1][l0:l1]), idx, n_kept=n_kept)
        return kept

    @torch.no_grad()
    def forward(self, kv_cache: List[LayerKV], it_len: Optional[List[int]] = None, **kwargs) -> List[LayerKV]:
        """kvpress_compressor.py:253-289."""
        if len(kv_cache) == 0:
            return kv_cache
        out = []
        for layer_idx, (keys, values) in enumerate(kv_cache):
            if keys is None or values is None:
                out.append((keys, values))
                continue
            out.append(self._compress_layer(keys, values, layer_idx))
        return out

    def __repr__(self):
        return (f"KVPressCompressor(method={self.method_name}, compression_ratio={self.compression_ratio}, "
                f"compression_factor={self.compression_factor:.1f}x)")


def create_kvpress_compressor(method: str = "streaming_llm", compression_factor: int = 5, config: Optional[Any] = None,
                              **kwargs) -> KVPressCompressor:
    """kvpress_compressor.py:310-336: ``compression_ratio = 1 - 1/compression_factor`` in double."""
    return KVPressCompressor(method=method, compression_ratio=1.0 - (1.0 / compression_factor), config=config, **kwargs)
