"""kvpress-style press objects with the call surface the reference uses, computed by HIP kernels.

The reference takes its presses from the third-party ``kvpress`` package
(utils_ccm/utils_compress.py:22-24) and wraps them in ``ScorerPressWithTime``
(utils_compress.py:200-324): dataclass fields ``compression_ratio`` (+ ``window_size``,
``kernel_size``, ``n_sink``), ``score(module, hidden_states, keys, values, attentions, kwargs)``
-> ``[B, Hkv, S]``, ``compress(...)`` -> ``(keys, values)``, ``forward_hook`` registered on every
``layer.self_attn`` by the context manager ``with press(model): ...``, and ``press_select``.
This module provides the same objects.  Scoring, selection and gathering run in
libfastcache_hip; torch only allocates and, for SnapKV inside a live model, projects the window
queries.

Two choices the reference leaves open are fixed here: ties in the selection go to the lowest token
index, and the kept tokens come out in ascending position order (``torch.topk`` guarantees neither).
"""
from __future__ import annotations

import math
import time
from contextlib import contextmanager
from dataclasses import dataclass
from typing import Generator, Optional

import torch
from torch import nn

from . import _lib, ops
from ._lib import FastcacheError


def _cache_layer_kv(cache, layer_idx):
    if hasattr(cache, "key_cache"):                       # transformers 4.x DynamicCache
        return cache.key_cache[layer_idx], cache.value_cache[layer_idx]
    layer = cache.layers[layer_idx]                       # transformers 5.x
    return layer.keys, layer.values


def _set_cache_layer_kv(cache, layer_idx, k, v):
    if hasattr(cache, "key_cache"):
        cache.key_cache[layer_idx], cache.value_cache[layer_idx] = k, v
    else:
        cache.layers[layer_idx].keys, cache.layers[layer_idx].values = k, v


def _seen_tokens(cache, layer_idx):
    if hasattr(cache, "seen_tokens"):
        return cache.seen_tokens
    return cache.get_seq_length(layer_idx)


@dataclass
class ScorerPress:
    """Prune the ``compression_ratio`` fraction of tokens with the lowest ``score`` in every
    (batch, kv head) row, during pre-filling only."""
    compression_ratio: float = 0.0

    def __post_init__(self):
        assert 0 <= self.compression_ratio < 1, "Compression ratio must be between 0 and 1"
        self.totalTime = 0

    def reset_timeCheck(self):
        """utils_compress.py:202-203."""
        self.totalTime = 0

    # -- to be provided by each press -------------------------------------------------------------
    def score(self, module, hidden_states, keys, values, attentions, kwargs) -> torch.Tensor:
        raise NotImplementedError

    # -- selection + gather -------------------------------------------------------------------------
    def n_kept(self, q_len: int) -> int:
        return int(q_len * (1 - self.compression_ratio))

    def select(self, scores: torch.Tensor, n_kept: int) -> torch.Tensor:
        """int32 ``[B, Hkv, n_kept]`` ascending positions of the ``n_kept`` best scores per row."""
        return ops.topk_select(scores.contiguous(), n_kept)

    def compress(self, module, hidden_states, keys, values, attentions, kwargs):
        if self.compression_ratio == 0:
            return keys, values
        scores = self.score(module, hidden_states, keys, values, attentions, kwargs)
        q_len = hidden_states.shape[1] if hidden_states is not None else keys.shape[2]
        n = self.n_kept(q_len)
        B, H, S, D = keys.shape
        idx = self.select(scores, n).view(1, B, H, n)
        out_k = torch.empty((B, H, n, D), dtype=keys.dtype, device=keys.device)
        out_v = torch.empty_like(out_k)
        ops.compact(_lib.dense_view(keys), _lib.dense_view(values), _lib.dense_view(out_k), _lib.dense_view(out_v), idx)
        return out_k, out_v

    # -- nano-vllm runner hook: the press of a paged pool (llava_model_runner.py:745-786) --------------------------
    # ``PagedKVRunner(compressor=press).compress_kv_cache_batch(seqs)`` calls ``paged_forward`` once for the whole
    # batch, in place of the reference's per-sequence extract -> compressor -> write-back loop.
    wants_seq_ids = True          # the runner passes ``seq_ids=``: presses that hold per-sequence inputs look them up

    def paged_compressed_len(self, seq_len: int, it_len=None) -> int:
        n = self.n_kept(seq_len)
        return seq_len if self.compression_ratio == 0 or n >= seq_len else n

    def paged_scores(self, kview, vview, lens, seq_lens, layers, seq_ids, device) -> torch.Tensor:
        """fp32 ``[L, B, Hkv, max_seq_len]`` for the layers ``layers=(l0, l1)`` of the views; entries past a
        sequence's length are never read by the selection."""
        raise FastcacheError(f"{type(self).__name__} cannot score a paged pool")

    @torch.no_grad()
    def paged_forward(self, kv_cache: torch.Tensor, block_tables: torch.Tensor, seq_lens: torch.Tensor,
                      seq_len: int, it_len=None, layers=None, out: Optional[torch.Tensor] = None, host_lens=None,
                      seq_ids=None):
        """Score, select and compact every (layer, sequence, kv head) column of the pool
        ``kv_cache [2, L, blocks, block_size, Hkv, D]``: in place (the kept rows move to the front of the same
        pages, ascending positions), or for ``layers=(l0, l1)`` only, or into ``out [2, L, B, Hkv, C, D]`` with the
        pages left alone.  Sequences all hold ``seq_len`` rows, or ``host_lens`` rows each (Python ints, ``seq_len``
        their maximum; ``seq_lens`` the same numbers on the device).  Returns the kept length, or the list of kept
        lengths when the sequences differ.  ``it_len`` (the MLP compressors' image/text split) is not used."""
        B = block_tables.shape[0]
        lens = list(host_lens) if host_lens is not None else [seq_len] * B
        kept = [self.paged_compressed_len(n) for n in lens]
        l0, l1 = layers if layers is not None else (0, kv_cache.shape[1])
        result = kept if len(set(lens)) > 1 else kept[0]
        if all(k >= n for k, n in zip(kept, lens)):
            if out is not None:
                for p in range(2):
                    ops.copy_tokens(_lib.paged_view(kv_cache[p][l0:l1], block_tables, seq_lens, seq_len),
                                    _lib.dense_view(out[p][l0:l1]), 0, seq_len, 0)
            return result
        self._paged_press(kv_cache[:, l0:l1], block_tables, seq_lens, seq_len, lens, kept, (l0, l1), out, seq_ids)
        return result

    def _paged_press(self, pool, block_tables, seq_lens, seq_len, lens, kept, layers, out, seq_ids):
        """Scores from ``paged_scores``, then one selection + compaction launch (two when a column does not fit LDS)."""
        from . import paged_press
        kview, vview = paged_press._views(pool, block_tables, seq_lens, seq_len)
        scores = self.paged_scores(kview, vview, lens, seq_lens, layers, seq_ids, pool.device)
        if out is None:
            paged_press._select_and_compact(kview, vview, scores, seq_lens, kept, True, pool.shape[4])
            return
        self._compact_into(kview, vview, scores, seq_lens, kept, pool.shape[4], out, layers)

    @staticmethod
    def _compact_into(kview, vview, scores, seq_lens, kept, heads, out, layers):
        l0, l1 = layers
        width = max(kept)
        dk, dv = _lib.dense_view(out[0][l0:l1]), _lib.dense_view(out[1][l0:l1])
        if len(set(kept)) == 1 and seq_lens is None:
            ops.compact(kview, vview, dk, dv, ops.topk_select(scores, width))
            return
        n_kept = torch.tensor(kept, dtype=torch.int32, device=scores.device)
        idx = ops.topk_select(scores, width, row_lens=seq_lens, n_kept=n_kept, rows_per_len=heads)
        ops.compact(kview, vview, dk, dv, idx, n_kept=n_kept)

    # -- HuggingFace hook protocol (utils_compress.py:209-299) ---------------------------------------
    def forward_hook(self, module: nn.Module, input, kwargs: dict, output):
        cache = kwargs.get("past_key_value", kwargs.get("past_key_values"))
        if cache is None:
            cache = output[-1]
        attentions = output[1] if len(output) == 3 else None
        hidden_states = kwargs["hidden_states"]
        q_len = hidden_states.shape[1]
        if _seen_tokens(cache, module.layer_idx) > q_len:      # decoding: leave the cache alone
            return output
        keys, values = _cache_layer_kv(cache, module.layer_idx)
        start = time.time()
        keys, values = self.compress(module, hidden_states, keys, values, attentions, kwargs)
        _set_cache_layer_kv(cache, module.layer_idx, keys, values)
        self.totalTime += time.time() - start
        return output

    @contextmanager
    def __call__(self, model) -> Generator:
        layers = model.model.layers if hasattr(model, "model") and hasattr(model.model, "layers") else model.layers
        hooks = []
        try:
            for layer in layers:
                hooks.append(layer.self_attn.register_forward_hook(self.forward_hook, with_kwargs=True))
            yield
        finally:
            for h in hooks:
                h.remove()


class _PerSequenceInputs:
    """What a prefill hands to a press for the later compression of its sequences on the runner hook: tensors
    ``[L, B, ...]`` (window queries, their log-sum-exp, query statistics), kept whole for the batch they came with
    and, when ``seq_ids`` are given, findable per sequence so that a later batch of other composition (lazy
    compression) can be assembled.  An entry is dropped once it has been used."""

    def __init__(self):
        self._batch = None            # (ids or None, {name: tensor [L, B, ...]})
        self._by_seq = {}             # seq_id -> {name: tensor [L, ...]}

    def put(self, tensors: dict, seq_ids=None) -> None:
        tensors = {k: v for k, v in tensors.items() if v is not None}
        self._batch = (None if seq_ids is None else list(seq_ids), tensors)
        if seq_ids is not None:
            for b, i in enumerate(seq_ids):
                self._by_seq[i] = {k: v[:, b] for k, v in tensors.items()}

    def take(self, batch: int, seq_ids=None) -> dict:
        ids, tensors = self._batch if self._batch is not None else (None, None)
        if tensors is not None and (ids is None or seq_ids is None or ids == list(seq_ids)):
            if next(iter(tensors.values())).shape[1] != batch:
                raise FastcacheError(f"the press holds inputs for {next(iter(tensors.values())).shape[1]} sequences, "
                                     f"the batch has {batch}")
            self._batch = None
            for i in ids or ():
                self._by_seq.pop(i, None)
            return tensors
        missing = [i for i in seq_ids if i not in self._by_seq]
        if missing:
            raise FastcacheError(f"the press holds no inputs for sequences {missing}")
        rows = [self._by_seq.pop(i) for i in seq_ids]
        self._batch = None
        return {k: torch.stack([r[k] for r in rows], dim=1) for k in rows[0]}

    def __bool__(self):
        return self._batch is not None or bool(self._by_seq)


@dataclass
class KnormPress(ScorerPress):
    """``score = -||k||_2``: keys with a small norm are kept."""

    def score(self, module, hidden_states, keys, values, attentions, kwargs) -> torch.Tensor:
        return ops.knorm_score(_lib.dense_view(keys), keys.device)[0]

    def paged_scores(self, kview, vview, lens, seq_lens, layers, seq_ids, device) -> torch.Tensor:
        return ops.knorm_score(kview, device)

    def _paged_press(self, pool, block_tables, seq_lens, seq_len, lens, kept, layers, out, seq_ids):
        if out is not None:
            return super()._paged_press(pool, block_tables, seq_lens, seq_len, lens, kept, layers, out, seq_ids)
        from . import paged_press
        # scoring, selection and compaction of a column by one workgroup, one launch for the batch
        paged_press.knorm_compress_paged(pool, block_tables, seq_lens, seq_len, self.compression_ratio,
                                         host_lens=lens if len(set(lens)) > 1 else None)


@dataclass
class SnapKVPress(ScorerPress):
    """Attention of the last ``window_size`` queries over the prefix, average-pooled.

    ``causal_window`` applies the causal mask among the window positions (kvpress does);
    ``reduction`` is 'mean' (kvpress) or 'sum' over the window queries and over the query heads of a
    group — the two differ by the constant ``window_size * group``;  with ``window_in_budget`` (kvpress)
    the always-kept window counts towards ``n_kept``, otherwise it is kept on top of it.
    Scores stay in fp32 (kvpress rounds the softmax to the query dtype).
    """
    compression_ratio: float = 0.0
    window_size: int = 64
    kernel_size: int = 5
    causal_window: bool = True
    reduction: str = "mean"
    window_in_budget: bool = True

    def __post_init__(self):
        super().__post_init__()
        self._paged_inputs = _PerSequenceInputs()

    def n_kept(self, q_len: int) -> int:
        n = int(q_len * (1 - self.compression_ratio))
        return n if self.window_in_budget else min(q_len, n + self.window_size)

    # -- runner hook ------------------------------------------------------------------------------------------
    def set_window_queries(self, queries: torch.Tensor, seq_ids=None, lse: Optional[torch.Tensor] = None) -> None:
        """What a prefill hands over for the compression of its sequences on the runner hook: the rotated queries of
        the last ``window_size`` positions of every sequence, ``[L, B, Hq, W, D]`` in the cache dtype (sequence order
        = the order of the batch that will be compressed, or named by ``seq_ids`` so that any later batch can be
        assembled), optionally with their log-sum-exp over the keys ``[L, B, Hq, W]`` from the attention kernel."""
        if queries.dim() != 5 or queries.shape[3] != self.window_size:
            raise FastcacheError(f"window queries must be [L, B, Hq, W={self.window_size}, D], got {tuple(queries.shape)}")
        self._paged_inputs.put({"queries": queries, "lse": lse}, seq_ids)

    def paged_scores(self, kview, vview, lens, seq_lens, layers, seq_ids, device) -> torch.Tensor:
        q, lse = self._paged_window(len(lens), layers, seq_ids)
        return ops.snapkv_score(kview, q, self.window_size, self.kernel_size, self.causal_window, self.reduction,
                                seq_lens=seq_lens, lse=lse)

    def _paged_window(self, batch, layers, seq_ids, keep: bool = False):
        if not self._paged_inputs:
            raise FastcacheError("SnapKVPress on the runner hook needs the window queries of the batch: call "
                                 "set_window_queries(q[L, B, Hq, W, D]) after the prefill")
        held = self._paged_inputs
        got = held.take(batch, seq_ids)
        l0, l1 = layers
        if keep or l1 < got["queries"].shape[0]:          # layer chunks (decode overlap) come back for the rest
            held.put(got, seq_ids)
        return got["queries"][l0:l1], (got["lse"][l0:l1] if "lse" in got else None)

    def _paged_press(self, pool, block_tables, seq_lens, seq_len, lens, kept, layers, out, seq_ids):
        if out is not None:
            return super()._paged_press(pool, block_tables, seq_lens, seq_len, lens, kept, layers, out, seq_ids)
        from . import paged_press
        q, lse = self._paged_window(len(lens), layers, seq_ids)
        if lse is not None:          # one sweep over the keys, then selection + compaction
            kview, vview = paged_press._views(pool, block_tables, seq_lens, seq_len)
            scores = ops.snapkv_score(kview, q, self.window_size, self.kernel_size, self.causal_window,
                                      self.reduction, seq_lens=seq_lens, lse=lse)
            paged_press._select_and_compact(kview, vview, scores, seq_lens, kept, True, pool.shape[4])
            return
        paged_press.snapkv_compress_paged(pool, block_tables, seq_lens, seq_len, q, self.compression_ratio,
                                          self.window_size, self.kernel_size, self.causal_window, self.reduction,
                                          self.window_in_budget, host_lens=lens if len(set(lens)) > 1 else None)

    def window_queries(self, module, hidden_states, kwargs) -> torch.Tensor:
        """Rotated queries of the last ``window_size`` positions, ``[B, Hq, W, D]``: given directly as
        ``kwargs['queries']`` (synthetic runs), or projected from ``hidden_states`` with the attention
        module's own ``q_proj`` (+ ``q_norm``) and the rotary ``position_embeddings``."""
        if kwargs is not None and kwargs.get("queries") is not None:
            return kwargs["queries"]
        W = self.window_size
        bsz = hidden_states.shape[0]
        num_heads = module.config.num_attention_heads
        q = module.q_proj(hidden_states[:, -W:]).view(bsz, W, num_heads, module.head_dim)
        if hasattr(module, "q_norm"):
            q = module.q_norm(q)
        q = q.transpose(1, 2)
        cos, sin = kwargs["position_embeddings"]
        cos, sin = cos[:, -W:].unsqueeze(1), sin[:, -W:].unsqueeze(1)
        half = q.shape[-1] // 2
        rot = torch.cat((-q[..., half:], q[..., :half]), dim=-1)
        return (q * cos + rot * sin).contiguous()

    def score(self, module, hidden_states, keys, values, attentions, kwargs) -> torch.Tensor:
        S = keys.shape[2]
        assert S > self.window_size, "Query length should be greater than the window size"
        q = self.window_queries(module, hidden_states, kwargs)
        head_dim = keys.shape[-1]
        lse = kwargs.get("lse") if kwargs is not None else None      # [B, Hq, W] from the prefill's attention kernel
        return ops.snapkv_score(_lib.dense_view(keys), q.to(keys.dtype), self.window_size, self.kernel_size,
                                self.causal_window, self.reduction, 1.0 / math.sqrt(head_dim), lse=lse)[0]


@dataclass
class TOVAPress(ScorerPress):
    """Attention of the last query over the other keys, averaged over all query heads and shared by the kv
    heads; the last token is always kept.  Uses ``attentions`` when the model returns them, otherwise computes the
    last query's softmax (window of one, no pooling) from ``kwargs['queries']`` or the module's ``q_proj``."""
    compression_ratio: float = 0.0

    def score(self, module, hidden_states, keys, values, attentions, kwargs) -> torch.Tensor:
        B, Hkv, S, D = keys.shape
        if attentions is not None:
            per_head = attentions[..., -1, :-1].float()                               # [B, Hq, S-1]
            mean = per_head.mean(1, keepdim=True)
        else:
            snap = SnapKVPress(window_size=1, kernel_size=1)
            q = snap.window_queries(module, hidden_states, kwargs)                     # [B, Hq, 1, D]
            group_sums = ops.snapkv_score(_lib.dense_view(keys), q.to(keys.dtype), 1, 1, True, "sum",
                                          1.0 / math.sqrt(D))[0]                       # [B, Hkv, S]: sums per kv group
            mean = group_sums[..., :S - 1].sum(1, keepdim=True) / q.shape[1]          # mean over all query heads
        scores = torch.empty((B, Hkv, S), dtype=torch.float32, device=keys.device)
        scores[..., :S - 1] = mean
        scores[..., S - 1] = mean.max()
        return scores

    def __post_init__(self):
        super().__post_init__()
        self._paged_inputs = _PerSequenceInputs()

    def set_window_queries(self, queries: torch.Tensor, seq_ids=None) -> None:
        """Runner hook: the rotated query of every sequence's last position, ``[L, B, Hq, 1, D]`` (or a longer
        window, of which the last position is used)."""
        if queries.dim() != 5:
            raise FastcacheError(f"queries must be [L, B, Hq, W, D], got {tuple(queries.shape)}")
        self._paged_inputs.put({"queries": queries[:, :, :, -1:, :]}, seq_ids)

    def paged_scores(self, kview, vview, lens, seq_lens, layers, seq_ids, device) -> torch.Tensor:
        if not self._paged_inputs:
            raise FastcacheError("TOVAPress on the runner hook needs the last queries: call set_window_queries first")
        q = self._paged_inputs.take(len(lens), seq_ids)["queries"][layers[0]:layers[1]].contiguous()
        sums = ops.snapkv_score(kview, q, 1, 1, True, "sum", 1.0 / math.sqrt(kview.head_dim), seq_lens=seq_lens)
        scores = torch.full_like(sums, float("-inf"))
        for b, n in enumerate(lens):                       # per sequence: head mean over its n - 1 other keys
            mean = sums[:, b, :, :n - 1].sum(1, keepdim=True) / q.shape[2]
            scores[:, b, :, :n - 1] = mean
            scores[:, b, :, n - 1] = mean.amax(dim=(1, 2), keepdim=False)[:, None] if n > 1 else 0.0
        return scores


@dataclass
class ObservedAttentionPress(ScorerPress):
    """Attention each key received during prefill (needs the model's attention weights, i.e. eager attention):
    summed over the queries, divided by the number of queries that can see the key, averaged over the group."""
    compression_ratio: float = 0.0
    output_attentions: bool = False

    def score(self, module, hidden_states, keys, values, attentions, kwargs) -> torch.Tensor:
        assert attentions is not None, 'Set output_attentions=True and attn_implementation="eager" to use this hook'
        return ops.observed_attention_score(attentions, keys.shape[1])

    def paged_forward(self, *args, **kwargs):
        raise FastcacheError("ObservedAttentionPress needs the prefill's attention matrices, which a paged runner "
                             "never materialises; use it through the HuggingFace hook")


@dataclass
class ExpectedAttentionPress(ScorerPress):
    """Attention each key can expect from the next ``n_future_positions`` queries, whose distribution is taken
    as Gaussian: its mean and covariance come from the prompt's hidden states through the attention module's
    ``q_proj`` and the average rotary matrix of the future positions; the scores are scaled by the value norms
    and the first ``n_sink`` tokens are always kept.  The statistics (a few matrix products on model tensors)
    are computed with torch; the scoring over the cache runs in libfastcache_hip.  They can also be given
    directly as ``kwargs['mean_query']`` ``[B, Hq, D]`` / ``kwargs['cov_query']`` ``[B, Hq, D, D]``."""
    compression_ratio: float = 0.0
    n_future_positions: int = 512
    n_sink: int = 4
    use_covariance: bool = True
    use_vnorm: bool = True
    epsilon: float = 0.0

    def future_rotary(self, module, q_len: int, head_dim: int, device, kwargs):
        """cos / sin ``[n_future, D]`` of positions ``q_len .. q_len + n_future_positions``: from the module's (or
        ``kwargs['rotary_emb']``'s) rotary embedding when there is one, else plain RoPE with ``config.rope_theta``."""
        pos = torch.arange(q_len, q_len + self.n_future_positions, device=device).unsqueeze(0)
        rotary = getattr(module, "rotary_emb", None) or (kwargs or {}).get("rotary_emb")
        if rotary is not None:
            cos, sin = rotary(torch.zeros(1, 1, head_dim, device=device), pos)
            return cos[0].float(), sin[0].float()
        theta = float(getattr(getattr(module, "config", None), "rope_theta", 10000.0))
        inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, device=device, dtype=torch.float32) / head_dim))
        ang = pos[0].float()[:, None] * inv_freq[None, :]
        emb = torch.cat((ang, ang), dim=-1)
        return emb.cos(), emb.sin()

    @torch.no_grad()
    def get_query_statistics(self, module, hidden_states, kwargs=None):
        bsz, q_len, _ = hidden_states.shape
        n, d = module.config.num_attention_heads, module.head_dim
        h = hidden_states[:, self.n_sink:].float()
        Wq = module.q_proj.weight.float()
        mean_h = h.mean(dim=1, keepdim=True)
        mu = torch.matmul(mean_h, Wq.T).squeeze(1).view(bsz, n, d)
        cov = None
        if self.use_covariance:
            hc = h - mean_h
            cov_h = torch.matmul(hc.transpose(1, 2), hc) / hc.shape[1]
            cov = torch.matmul(Wq, torch.matmul(cov_h, Wq.T)).view(bsz, n, d, n, d)
            cov = cov.diagonal(dim1=1, dim2=3).permute(0, 3, 1, 2)
        cos, sin = self.future_rotary(module, q_len, d, hidden_states.device, kwargs)
        # average over the future positions of R = cos * I + sin * P, P = [[0, -I], [I, 0]] (rotate_half)
        half = d // 2
        R = torch.diag_embed(cos).mean(0)
        sm = sin.mean(0)
        R[half:, :half] += torch.diag(sm[:half])
        R[:half, half:] -= torch.diag(sm[half:])
        mu = torch.matmul(mu, R.T)
        if cov is not None:
            cov = torch.matmul(R, torch.matmul(cov, R.T))
        return mu, cov

    def score(self, module, hidden_states, keys, values, attentions, kwargs) -> torch.Tensor:
        assert keys.size(2) > self.n_sink, f"Input should contain more tokens than n_sink={self.n_sink}"
        if kwargs is not None and kwargs.get("mean_query") is not None:
            mu, cov = kwargs["mean_query"], kwargs.get("cov_query")
        else:
            mu, cov = self.get_query_statistics(module, hidden_states, kwargs)
        if not self.use_covariance:
            cov = None
        return ops.expected_attention_score(_lib.dense_view(keys), _lib.dense_view(values), mu, cov, self.n_sink,
                                            self.use_vnorm, self.epsilon)[0]

    def __post_init__(self):
        super().__post_init__()
        self._paged_inputs = _PerSequenceInputs()

    def set_query_statistics(self, mean_query: torch.Tensor, cov_query: Optional[torch.Tensor] = None,
                             seq_ids=None) -> None:
        """Runner hook: ``mean_query [L, B, Hq, D]`` and ``cov_query [L, B, Hq, D, D]`` of the future queries
        (``get_query_statistics`` per layer of the prefill)."""
        self._paged_inputs.put({"mean": mean_query, "cov": cov_query if self.use_covariance else None}, seq_ids)

    def paged_scores(self, kview, vview, lens, seq_lens, layers, seq_ids, device) -> torch.Tensor:
        if len(set(lens)) > 1:
            raise FastcacheError("ExpectedAttentionPress on the runner hook takes sequences of one length per call")
        if not self._paged_inputs:
            raise FastcacheError("ExpectedAttentionPress on the runner hook needs set_query_statistics first")
        got = self._paged_inputs.take(len(lens), seq_ids)
        l0, l1 = layers
        cov = got["cov"][l0:l1] if "cov" in got else None
        return ops.expected_attention_score(kview, vview, got["mean"][l0:l1], cov, self.n_sink, self.use_vnorm,
                                            self.epsilon)


@dataclass
class StreamingLLMPress(ScorerPress):
    """Keep the first ``n_sink`` tokens and the most recent ones."""
    compression_ratio: float = 0.0
    n_sink: int = 4

    def score(self, module, hidden_states, keys, values, attentions, kwargs) -> torch.Tensor:
        q_len = hidden_states.shape[1] if hidden_states is not None else keys.shape[2]
        assert q_len > self.n_sink, f"Input should contain more tokens than n_sink={self.n_sink}"
        n_pruned = q_len - int(q_len * (1 - self.compression_ratio))
        scores = torch.ones(keys.shape[:3], dtype=torch.float32, device=keys.device)
        scores[:, :, self.n_sink:self.n_sink + n_pruned] = 0
        return scores

    def paged_scores(self, kview, vview, lens, seq_lens, layers, seq_ids, device) -> torch.Tensor:
        rows = torch.full((len(lens), kview.max_seq_len), float("-inf"))
        for b, n in enumerate(lens):
            assert n > self.n_sink, f"Input should contain more tokens than n_sink={self.n_sink}"
            rows[b, :n] = 1.0
            rows[b, self.n_sink:self.n_sink + n - self.paged_compressed_len(n)] = 0.0
        L, H = layers[1] - layers[0], kview.num_kv_heads
        return rows.to(device)[None, :, None, :].expand(L, len(lens), H, -1).contiguous()


@dataclass
class RandomPress(ScorerPress):
    """Uniformly random scores (baseline)."""
    compression_ratio: float = 0.0
    seed: Optional[int] = None

    def score(self, module, hidden_states, keys, values, attentions, kwargs) -> torch.Tensor:
        g = None
        if self.seed is not None:
            g = torch.Generator(device=keys.device).manual_seed(self.seed)
        return torch.rand(keys.shape[:3], dtype=torch.float32, device=keys.device, generator=g)

    def paged_scores(self, kview, vview, lens, seq_lens, layers, seq_ids, device) -> torch.Tensor:
        g = None
        if self.seed is not None:
            g = torch.Generator(device=device).manual_seed(self.seed)
        shape = (layers[1] - layers[0], len(lens), kview.num_kv_heads, kview.max_seq_len)
        scores = torch.rand(shape, dtype=torch.float32, device=device, generator=g)
        for b, n in enumerate(lens):
            scores[:, b, :, n:] = float("-inf")
        return scores


@dataclass
class ThinKPress(ScorerPress):
    """Prune head-dimension channels of the keys instead of tokens (ThinK): the ``key_channel_compression_ratio``
    fraction of channels with the lowest ``mean_window(q^2) * mean_tokens(k^2)`` per (batch, kv head) is set to
    zero for every token, in place; the query statistic is averaged over the query heads of the group.  Values and
    the cache length are unchanged.  The statistics are formed in fp32 (kvpress forms them in the tensor dtype) and
    ties go to the lowest channel index."""
    key_channel_compression_ratio: float = 0.0
    window_size: int = 32

    def __post_init__(self):
        assert 0 <= self.key_channel_compression_ratio < 1, "Compression ratio must be between 0 and 1"
        self.compression_ratio = 0.0
        self.totalTime = 0

    def channel_scores(self, module, hidden_states, keys, kwargs) -> torch.Tensor:
        """fp32 ``[B, Hkv, D]``."""
        B, Hkv, S, D = keys.shape
        q = SnapKVPress(window_size=self.window_size).window_queries(module, hidden_states, kwargs)   # [B, Hq, W, D]
        q_energy = q.float().pow(2).mean(dim=2).view(B, Hkv, q.shape[1] // Hkv, D).mean(dim=2)
        k_energy = ops.key_channel_energy(_lib.dense_view(keys), keys.device)[0] / S
        return q_energy * k_energy

    def compress(self, module, hidden_states, keys, values, attentions, kwargs):
        if self.key_channel_compression_ratio == 0:
            return keys, values
        B, Hkv, S, D = keys.shape
        n_pruned = int(D * self.key_channel_compression_ratio)
        if n_pruned == 0:
            return keys, values
        scores = self.channel_scores(module, hidden_states, keys, kwargs)
        idx = ops.topk_select((-scores).contiguous(), n_pruned).long()             # the lowest scores
        prune = torch.zeros((B, Hkv, D), dtype=torch.uint8, device=keys.device).scatter_(-1, idx, 1)
        ops.key_channel_zero(_lib.dense_view(keys), prune[None])
        return keys, values

    def set_window_queries(self, queries: torch.Tensor, seq_ids=None) -> None:
        """Runner hook: rotated queries of the last ``window_size`` positions, ``[L, B, Hq, W, D]``."""
        if not hasattr(self, "_paged_inputs"):
            self._paged_inputs = _PerSequenceInputs()
        self._paged_inputs.put({"queries": queries}, seq_ids)

    @torch.no_grad()
    def paged_forward(self, kv_cache, block_tables, seq_lens, seq_len, it_len=None, layers=None, out=None,
                      host_lens=None, seq_ids=None):
        """Zero the pruned key channels of every (layer, sequence, kv head) column in the pages; lengths stay."""
        B = block_tables.shape[0]
        lens = list(host_lens) if host_lens is not None else [seq_len] * B
        result = lens if len(set(lens)) > 1 else lens[0]
        if out is not None:
            raise FastcacheError("ThinKPress prunes channels in place; it has no staged output")
        D = kv_cache.shape[-1]
        n_pruned = int(D * self.key_channel_compression_ratio)
        if n_pruned == 0:
            return result
        if not getattr(self, "_paged_inputs", None):
            raise FastcacheError("ThinKPress on the runner hook needs set_window_queries first")
        l0, l1 = layers if layers is not None else (0, kv_cache.shape[1])
        q = self._paged_inputs.take(B, seq_ids)["queries"][l0:l1]                       # [L, B, Hq, W, D]
        kview = _lib.paged_view(kv_cache[0][l0:l1], block_tables, seq_lens, seq_len)
        Hkv = kview.num_kv_heads
        q_energy = q.float().pow(2).mean(dim=3).view(l1 - l0, B, Hkv, q.shape[2] // Hkv, D).mean(dim=3)
        rows = torch.tensor(lens, dtype=torch.float32, device=kv_cache.device).view(1, B, 1, 1)
        scores = q_energy * (ops.key_channel_energy(kview, kv_cache.device) / rows)
        idx = ops.topk_select((-scores).contiguous(), n_pruned).long()
        prune = torch.zeros((l1 - l0, B, Hkv, D), dtype=torch.uint8, device=kv_cache.device).scatter_(-1, idx, 1)
        ops.key_channel_zero(kview, prune)
        return result


@dataclass
class SimLayerKVPress(ScorerPress):
    """Layer-wise pruning (SimLayerKV): a layer is "lazy" when its last ``n_last`` queries put more than
    ``lazy_threshold`` of their attention, averaged over batch, heads and those queries, on the first ``n_initial``
    and the last ``n_recent`` of the other keys; a lazy layer keeps only the first ``n_initial`` tokens and the last
    ``n_recent - n_last`` ones, other layers keep everything.  ``compression_ratios`` records what each call removed."""
    lazy_threshold: float = 1.0
    n_last: int = 1
    n_recent: int = 1024
    n_initial: int = 4

    def __post_init__(self):
        assert 0.0 <= self.lazy_threshold <= 1.0, "lazy_threshold should be in [0, 1]"
        assert self.n_recent > self.n_last, "n_recent must exceed n_last"
        self.compression_ratios = []
        self.totalTime = 0

    @property
    def compression_ratio(self):
        if not self.compression_ratios:
            return 0.0
        return sum(self.compression_ratios) / len(self.compression_ratios)

    @compression_ratio.setter
    def compression_ratio(self, value):
        if isinstance(value, property) or value == 0.0:      # the dataclass default of the base class
            return
        raise AttributeError(f"compression ratio cannot be set for {type(self).__name__}")

    def lazy_score(self, module, hidden_states, keys, kwargs) -> float:
        """Share of the last queries' attention that lands on the initial and the recent keys."""
        B, Hkv, S, D = keys.shape
        q = SnapKVPress(window_size=self.n_last).window_queries(module, hidden_states, kwargs)        # [B, Hq, n_last, D]
        sums = ops.snapkv_score(_lib.dense_view(keys), q.to(keys.dtype), self.n_last, 1, True, "sum",
                                1.0 / math.sqrt(D))[0][..., :S - self.n_last]                          # [B, Hkv, S - n_last]
        per_key = sums.sum(dim=(0, 1)) / (B * q.shape[1] * self.n_last)
        return float(per_key[:self.n_initial].sum() + per_key[-self.n_recent:].sum())

    def compress(self, module, hidden_states, keys, values, attentions, kwargs):
        B, H, S, D = keys.shape
        q_len = hidden_states.shape[1] if hidden_states is not None else S
        if q_len <= self.n_initial + self.n_recent + self.n_last:
            return keys, values
        if self.lazy_score(module, hidden_states, keys, kwargs) <= self.lazy_threshold:
            self.compression_ratios.append(0.0)
            return keys, values
        tail = self.n_recent - self.n_last
        pos = torch.cat([torch.arange(self.n_initial), torch.arange(S - tail, S)]).to(torch.int32)
        n = pos.numel()
        idx = pos.to(keys.device).view(1, 1, 1, n).expand(1, B, 1, n).contiguous()                   # one row for all heads
        out_k = torch.empty((B, H, n, D), dtype=keys.dtype, device=keys.device)
        out_v = torch.empty_like(out_k)
        ops.compact(_lib.dense_view(keys), _lib.dense_view(values), _lib.dense_view(out_k), _lib.dense_view(out_v), idx)
        self.compression_ratios.append((q_len - self.n_initial - self.n_recent + 1) / q_len)
        return out_k, out_v

    def paged_forward(self, *args, **kwargs):
        raise FastcacheError("SimLayerKVPress keeps a different number of tokens per layer, which one block table "
                             "per sequence cannot hold; use it through the HuggingFace hook")


class SimpleKVQuantizer:
    """Symmetric ``nbits`` quantise-dequantise of every K and V tensor of a cache with ONE scale per tensor
    (utils_ccm/utils_compress.py:117-163).  Used as ``with quantizer(model) as q: q.quantize_cache(pkv)``."""

    def __init__(self, nbits: int = 4):
        self.nbits = nbits
        self.totalTime = 0

    def reset_timeCheck(self):
        self.totalTime = 0

    def __call__(self, model):
        return self.QuantizeContext(self)

    def _quantize_tensor(self, x: torch.Tensor) -> torch.Tensor:
        return ops.fake_quantize(x, self.nbits, per_tensor=True)

    def quantize_cache(self, past_key_values):
        return tuple((self._quantize_tensor(k), self._quantize_tensor(v)) for k, v in past_key_values)

    class QuantizeContext:
        def __init__(self, quantizer):
            self.quantizer = quantizer

        def __enter__(self):
            return self.quantizer

        def __exit__(self, exc_type, exc_val, exc_tb):
            pass


class ImprovedKVQuantizer(SimpleKVQuantizer):
    """The same with one scale per row of the last dimension; the scales and row maxima of the last
    ``quantize_cache`` are kept in ``cache['k_<layer>']`` / ``cache['v_<layer>']``
    (utils_ccm/utils_compress.py:27-95)."""

    def __init__(self, nbits: int = 4):
        super().__init__(nbits)
        self.cache = {}

    def _quantize_tensor_with_params(self, x: torch.Tensor, key: str):
        y, scale, max_val = ops.fake_quantize(x, self.nbits, per_tensor=False, return_params=True)
        return y, {"scale": scale, "max_val": max_val}

    def quantize_cache(self, past_key_values):
        quantized = []
        for layer_idx, (k, v) in enumerate(past_key_values):
            k_scaled, self.cache[f"k_{layer_idx}"] = self._quantize_tensor_with_params(k, f"k_{layer_idx}")
            v_scaled, self.cache[f"v_{layer_idx}"] = self._quantize_tensor_with_params(v, f"v_{layer_idx}")
            quantized.append((k_scaled, v_scaled))
        return tuple(quantized)

    def dequantize_cache(self, quantized_cache):
        """``x * scale`` with the stored scales, exactly as the reference does (its input is already
        de-quantised, so this scales a second time)."""
        return tuple((k * self.cache[f"k_{i}"]["scale"], v * self.cache[f"v_{i}"]["scale"])
                     for i, (k, v) in enumerate(quantized_cache))


# names the reference gives its timed subclasses (utils_compress.py:302-324)
TOVAPressWithTime = TOVAPress
ExpectedAttentionPressWithTime = ExpectedAttentionPress
ObservedAttentionPressWithTime = ObservedAttentionPress
KnormPressWithTime = KnormPress
SnapKVPressWithTime = SnapKVPress
StreamingLLMPressWithTime = StreamingLLMPress
RandomPressWithTime = RandomPress


def press_select(compression_method: str = "Knorm", compression_ratio: float = 0.8) -> ScorerPress:
    """utils_compress.py:327-349: 'Quantized' gives the 4-bit ``SimpleKVQuantizer``; any name the reference does
    not list gives the Knorm press, as there."""
    if compression_method == "StreamingLLM":
        press = StreamingLLMPress(compression_ratio=compression_ratio)
    elif compression_method == "RandomPress":
        press = RandomPress(compression_ratio=compression_ratio)
    elif compression_method == "SnapKV":
        press = SnapKVPress(compression_ratio=compression_ratio)
    elif compression_method == "TOVA":
        press = TOVAPress(compression_ratio=compression_ratio)
    elif compression_method == "Quantized":
        return SimpleKVQuantizer(nbits=4)
    elif compression_method == "ExpectedAttention":
        press = ExpectedAttentionPress(compression_ratio=compression_ratio)
    else:
        press = KnormPress(compression_ratio=compression_ratio)
    press.reset_timeCheck()
    return press
