"""Oracle (test infrastructure): token scoring, selection and gathering.

Two families are restated here.

* The in-tree adapter ``KVPressCompressor._compress_layer``
  (nanovllm/kernels/kvpress_compressor.py:169-251): one index set per batch row.
* The kvpress-style presses the reference imports from the third-party ``kvpress`` package
  (requirements.txt:13, ``kvpress>=0.3.0``, no lock file; call sites
  utils_ccm/utils_compress.py:22-24, 200-349; nanovllm/autocompress/methods.py:484-491).  The
  package is not vendored, so its published algorithm is restated: ``ScorerPress.compress`` keeps
  ``n_kept = int(q_len * (1 - compression_ratio))`` tokens per (batch, kv head) by ``topk`` of
  ``score`` and gathers K and V; ``KnormPress.score = -keys.norm(dim=-1)``;
  ``SnapKVPress.score`` is the observation-window attention described at ``snapkv_score``.

Selection order is fixed here (torch.topk leaves ties unspecified): largest score first, ties
to the lowest index, output in ascending token order.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import numpy as np
import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------------------------
# kept-token count
# --------------------------------------------------------------------------------------------
def ratio_from_factor(compression_factor: float) -> float:
    """``compression_ratio = 1.0 - 1.0 / compression_factor`` in double
    (nanovllm/engine/llava_model_runner.py:389, kvpress_compressor.py:328)."""
    return 1.0 - (1.0 / compression_factor)


def n_kept_adapter(seq_len: int, compression_ratio: float) -> int:
    """kvpress_compressor.py:193-194: ``max(int(S * (1 - r)), 1)`` in double arithmetic."""
    return max(int(seq_len * (1 - compression_ratio)), 1)


def n_kept_press(seq_len: int, compression_ratio: float) -> int:
    """kvpress ``ScorerPress.compress``: ``int(q_len * (1 - compression_ratio))``."""
    return int(seq_len * (1 - compression_ratio))


# --------------------------------------------------------------------------------------------
# scores
# --------------------------------------------------------------------------------------------
def knorm_score(keys: torch.Tensor) -> torch.Tensor:
    """kvpress ``KnormPress.score``: ``-keys.norm(dim=-1)``; evaluated in fp32 whatever the
    storage dtype.  keys ``[B, Hkv, S, D]`` -> ``[B, Hkv, S]`` fp32."""
    return -torch.linalg.vector_norm(keys.float(), dim=-1)


def knorm_mean_score(keys: torch.Tensor) -> torch.Tensor:
    """kvpress_compressor.py:222-223: ``keys.norm(dim=-1).mean(dim=1)`` in the input dtype,
    returned as fp32 values (each step rounded to the storage dtype as torch does)."""
    norms = keys.norm(dim=-1)
    return norms.mean(dim=1).float()


def snapkv_score(queries: torch.Tensor, keys: torch.Tensor, window_size: int, kernel_size: int,
                 causal_window: bool = True, reduction: str = "mean",
                 scale: Optional[float] = None) -> torch.Tensor:
    """kvpress ``SnapKVPress.score`` with pre-rotated window queries.

    queries ``[B, Hq, W, D]`` (the last W positions), keys ``[B, Hkv, S, D]``.
    logits = Q K^T / sqrt(D) over all S keys of kv head ``hq // G``; with ``causal_window`` the
    key at position S-W+j is masked for window query i when j > i (the triu mask of
    ``compute_window_attention``); softmax in fp32; the last W columns are dropped; reduce over the
    W queries; ``avg_pool1d(kernel, padding=kernel//2, stride=1)`` (zero padding counted in the
    divisor); reduce over the G query heads of each kv group; the window positions get the global
    maximum of the tensor so that they are never pruned.  ``reduction`` is 'mean' (kvpress) or
    'sum' (both reductions as sums); the two differ by the constant factor W*G.
    Everything after the logits stays in fp32 (kvpress rounds the softmax to the query dtype;
    this build keeps fp32 scores).  Returns ``[B, Hkv, S]`` fp32.
    """
    B, Hq, W, D = queries.shape
    _, Hkv, S, _ = keys.shape
    assert W == window_size and S > W, "sequence must be longer than the window"
    G = Hq // Hkv
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    k_rep = keys.float().repeat_interleave(G, dim=1)                     # repeat_kv
    logits = torch.matmul(queries.float(), k_rep.transpose(2, 3)) * scale  # [B,Hq,W,S]
    if causal_window:
        mask = torch.full((W, S), float("-inf"), device=logits.device)
        mask = torch.triu(mask, diagonal=S - W + 1)
        logits = logits + mask
    attn = F.softmax(logits, dim=-1, dtype=torch.float32)
    attn = attn[..., :-W]
    v = attn.mean(dim=-2) if reduction == "mean" else attn.sum(dim=-2)  # [B,Hq,S-W]
    v = F.avg_pool1d(v, kernel_size=kernel_size, padding=kernel_size // 2, stride=1)
    v = v.view(B, Hkv, G, S - W)
    v = v.mean(2) if reduction == "mean" else v.sum(2)
    return F.pad(v, (0, W), value=v.max().item())


def tova_score(queries: Optional[torch.Tensor], keys: torch.Tensor, attentions: Optional[torch.Tensor] = None,
               scale: Optional[float] = None) -> torch.Tensor:
    """kvpress ``TOVAPress.score`` (third party, restated from its published description; PARITY UNPINNED):
    the attention of the LAST query over the other keys, averaged over ALL query heads, the same row for every
    kv head; the last position gets the maximum so that it is never pruned.  ``attentions [B, Hq, Sq, S]`` is used
    when given, otherwise the softmax is computed from ``queries [B, Hq, 1, D]`` (the last position)."""
    B, Hkv, S, D = keys.shape
    if attentions is not None:
        attn = attentions[..., -1:, :-1].float()
    else:
        G = queries.shape[1] // Hkv
        if scale is None:
            scale = 1.0 / math.sqrt(D)
        logits = torch.matmul(queries.float(), keys.float().repeat_interleave(G, dim=1).transpose(2, 3)) * scale
        attn = F.softmax(logits, dim=-1, dtype=torch.float32)[..., :-1]          # [B, Hq, 1, S-1]
    scores = attn.mean(1)                                                        # [B, 1, S-1]
    scores = scores.repeat(1, Hkv, 1)
    return F.pad(scores, (0, 1), value=scores.max().item())


def expected_attention_query_statistics(hidden_states: torch.Tensor, q_weight: torch.Tensor, num_heads: int,
                                        head_dim: int, cos: torch.Tensor, sin: torch.Tensor, n_sink: int = 4,
                                        use_covariance: bool = True):
    """kvpress ``ExpectedAttentionPress.get_query_statistics`` (third party, restated from its published
    description; PARITY UNPINNED): Gaussian statistics of the queries the next positions will produce.
    ``hidden_states [B, S, hidden]`` (the first ``n_sink`` positions are left out as outliers), ``q_weight``
    ``[num_heads * head_dim, hidden]`` (``q_proj.weight``), ``cos`` / ``sin`` ``[n_future, head_dim]`` of the
    future positions.  mean = W mean(h); covariance = W cov(h) W^T, per-head diagonal blocks, population
    normalisation; both are then rotated by the AVERAGE rotary matrix of the future positions.
    Returns ``(mu [B, H, D], cov [B, H, D, D] or None)`` in fp32."""
    bsz = hidden_states.shape[0]
    n, d = num_heads, head_dim
    h = hidden_states[:, n_sink:].float()
    Wq = q_weight.float()
    mean_h = h.mean(dim=1, keepdim=True)
    mu = torch.matmul(mean_h, Wq.T).squeeze(1).view(bsz, n, d)
    cov = None
    if use_covariance:
        hc = h - mean_h
        cov_h = torch.matmul(hc.transpose(1, 2), hc) / hc.shape[1]
        cov = torch.matmul(Wq, torch.matmul(cov_h, Wq.T))                       # [B, n*d, n*d]
        cov = cov.view(bsz, n, d, n, d).diagonal(dim1=1, dim2=3)                # [B, d, d, n]
        cov = cov.permute(0, 3, 1, 2)
    # rotary matrix of one position: R = cos * I + sin * P with P = [[0, -I], [I, 0]], so that
    # R q = q * cos + rotate_half(q) * sin
    Id = torch.eye(d)
    P = torch.zeros(d, d)
    P[d // 2:, :d // 2], P[:d // 2, d // 2:] = torch.eye(d // 2), -torch.eye(d // 2)
    R = cos.float().unsqueeze(1) * Id + sin.float().unsqueeze(1) * P                # [n_future, d, d]
    R = R.mean(dim=0)
    mu = torch.matmul(mu, R.T)
    if use_covariance:
        cov = torch.matmul(R, torch.matmul(cov, R.T))
    return mu, cov


def expected_attention_score(keys: torch.Tensor, values: torch.Tensor, mean_query: torch.Tensor,
                             cov_query: Optional[torch.Tensor], n_sink: int = 4, use_vnorm: bool = True,
                             epsilon: float = 0.0) -> torch.Tensor:
    """kvpress ``ExpectedAttentionPress.score`` given the query statistics (third party; PARITY UNPINNED):
    keys / values ``[B, Hkv, S, D]``, mean ``[B, Hq, D]``, covariance ``[B, Hq, D, D]`` -> ``[B, Hkv, S]`` fp32."""
    assert keys.size(2) > n_sink
    k = keys[:, :, n_sink:].float()
    v = values[:, :, n_sink:].float()
    bsz, Hkv, q_len, d = k.shape
    G = mean_query.shape[1] // Hkv
    kt = k.repeat_interleave(G, dim=1).transpose(2, 3)                            # [B, Hq, D, n]
    scores = torch.matmul(mean_query.float().unsqueeze(2), kt).squeeze(2) / math.sqrt(d)
    if cov_query is not None:
        scores = scores + torch.einsum("bhin,bhij,bhjn->bhn", kt, cov_query.float(), kt) / d / 2
    scores = F.softmax(scores, dim=-1)
    scores = scores.view(bsz, Hkv, G, q_len).mean(dim=2)
    if use_vnorm:
        scores = (scores + epsilon) * v.norm(dim=-1)
    return F.pad(scores, (n_sink, 0), value=scores.max().item())


def observed_attention_score(attentions: torch.Tensor, num_kv_heads: int) -> torch.Tensor:
    """kvpress ``ObservedAttentionPress.score`` (third party; PARITY UNPINNED): attention received by each key
    summed over the queries, divided by the number of queries that can see the key, averaged over the group."""
    B, Hq, Sq, S = attentions.shape
    scores = attentions.float().sum(2)
    n_tokens_in_sum = torch.arange(S, 0, -1).float()
    scores = scores / n_tokens_in_sum
    return scores.view(B, num_kv_heads, -1, S).mean(2)


# --------------------------------------------------------------------------------------------
# selection
# --------------------------------------------------------------------------------------------
def topk_lowest_index(scores: torch.Tensor, k: int) -> torch.Tensor:
    """The ``k`` largest entries of each row of ``scores[..., S]``; ties to the lowest index;
    indices returned ascending (int64).  NaN ranks above +inf and -0 equals +0, as torch.topk
    orders them."""
    sc = scores.detach().to(torch.float32) + 0.0             # -0 -> +0
    if not torch.isnan(sc).any():
        # stable ascending sort of the negated scores: larger score first, ties keep index order
        order = torch.sort(-sc, dim=-1, stable=True).indices[..., :k]
        return torch.sort(order, dim=-1).values
    s = sc.numpy()
    flat = s.reshape(-1, s.shape[-1])
    out = np.empty((flat.shape[0], k), dtype=np.int64)
    for r in range(flat.shape[0]):
        row = flat[r]
        key = np.where(np.isnan(row), np.inf, row)
        nan_first = np.isnan(row)
        # NaN first, then larger scores, ties keep index order
        order = np.lexsort((np.arange(row.size), -key, ~nan_first))
        out[r] = np.sort(order[:k])
    return torch.from_numpy(out.reshape(*s.shape[:-1], k))


def near_tie_rows(scores: torch.Tensor, k: int, rel: float = 1e-5) -> torch.Tensor:
    """Rows whose k-th and (k+1)-th largest scores differ by less than ``rel`` relative: their kept
    set is not determined at fp32 scoring accuracy and is left out of index comparisons."""
    s = scores.float()
    if k <= 0 or k >= s.shape[-1]:
        return torch.zeros(s.shape[:-1], dtype=torch.bool, device=s.device)
    top = torch.topk(s, k + 1, dim=-1).values
    a, b = top[..., k - 1], top[..., k]
    return (a - b).abs() < rel * a.abs()


def gather_tokens(x: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    """``x.gather(2, idx[..., None].expand(..., D))`` (kvpress_compressor.py:245-249).
    x ``[B, H, S, D]``; idx ``[B, H, k]`` or ``[B, k]`` (shared by all heads)."""
    if idx.dim() == 2:
        idx = idx.unsqueeze(1).expand(-1, x.shape[1], -1)
    return x.gather(2, idx.unsqueeze(-1).expand(-1, -1, -1, x.shape[-1])).contiguous()


# --------------------------------------------------------------------------------------------
# kvpress-style press = score + select + gather
# --------------------------------------------------------------------------------------------
def press_compress(keys: torch.Tensor, values: torch.Tensor, scores: torch.Tensor,
                   compression_ratio: float, extra_kept: int = 0) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """kvpress ``ScorerPress.compress``.  Returns ``(K', V', idx[B, Hkv, n_kept])``.  ``extra_kept`` adds that many
    positions to the budget (the other reading of "keep a quarter plus the window": the SnapKV observation window,
    which always ranks first, kept ON TOP of ``int(S * (1 - r))`` instead of inside it), capped at the length."""
    if compression_ratio == 0:
        S = keys.shape[2]
        idx = torch.arange(S).expand(keys.shape[0], keys.shape[1], S)
        return keys, values, idx
    n = min(keys.shape[2], n_kept_press(keys.shape[2], compression_ratio) + extra_kept)
    idx = topk_lowest_index(scores, n)
    return gather_tokens(keys, idx), gather_tokens(values, idx), idx


# --------------------------------------------------------------------------------------------
# the in-tree adapter
# --------------------------------------------------------------------------------------------
def adapter_indices(method: str, keys: torch.Tensor, compression_ratio: float, n_sink: int = 4,
                    generator: Optional[torch.Generator] = None) -> Optional[torch.Tensor]:
    """Index choice of ``KVPressCompressor._compress_layer`` (kvpress_compressor.py:193-238).
    Returns int64 ``[B, n]`` ascending, or None when nothing is dropped."""
    B, H, S, D = keys.shape
    n = n_kept_adapter(S, compression_ratio)
    if n >= S:                                                        # :197-198
        return None
    if method == "streaming_llm":                                     # :201-218
        sink = min(n_sink, n)
        recent = max(0, n - sink)
        if recent > 0 and S > sink + recent:
            idx = torch.cat([torch.arange(sink), torch.arange(S - recent, S)])
        elif recent > 0:
            idx = torch.arange(n)
        else:
            idx = torch.arange(sink)
    elif method == "knorm":                                           # :220-226
        m = knorm_mean_score(keys)                                    # [B, S]
        return topk_lowest_index(m, min(n, S))
    elif method == "random":                                          # :228-232
        idx = torch.randperm(S, generator=generator)[:min(n, S)].sort().values
    else:                                                             # :234-238
        n = min(n, S)
        step = max(1, S // n)
        idx = torch.arange(0, S, step).long()[:n]
    return idx.unsqueeze(0).expand(B, -1)                             # :241-242


def adapter_compress_layer(method: str, keys: torch.Tensor, values: torch.Tensor,
                           compression_ratio: float, n_sink: int = 4,
                           generator: Optional[torch.Generator] = None
                           ) -> Tuple[torch.Tensor, torch.Tensor]:
    """``KVPressCompressor._compress_layer`` (kvpress_compressor.py:169-251)."""
    idx = adapter_indices(method, keys, compression_ratio, n_sink, generator)
    if idx is None:
        return keys.contiguous(), values.contiguous()
    return gather_tokens(keys, idx), gather_tokens(values, idx)


# --------------------------------------------------------------------------------------------
# quantise -> dequantise of a cache (SimpleKVQuantizer / ImprovedKVQuantizer)
# --------------------------------------------------------------------------------------------
def fake_quantize(x: torch.Tensor, nbits: int, per_tensor: bool):
    """``SimpleKVQuantizer._quantize_tensor`` (utils_ccm/utils_compress.py:144-154, one scale for the whole
    tensor) and ``ImprovedKVQuantizer._quantize_tensor_with_params`` (utils_compress.py:51-70, one scale per row
    of the last dimension): the same eager tensor expression, in the dtype of ``x``.
    Returns ``(x_dequant, scale, max_val)``."""
    if per_tensor:
        max_val = torch.max(torch.abs(x))
    else:
        max_val = torch.max(torch.abs(x), dim=-1, keepdim=True)[0]
    scale = max_val / (2 ** (nbits - 1) - 1)
    x_quant = torch.round(x / scale)
    x_quant = torch.clamp(x_quant, -2 ** (nbits - 1), 2 ** (nbits - 1) - 1)
    return x_quant * scale, scale, max_val


# ---- ThinK and SimLayerKV (kvpress presses the reference registers at nanovllm/autocompress/methods.py:422-423) ----
def think_channel_scores(keys: torch.Tensor, queries: torch.Tensor) -> torch.Tensor:
    """ThinK: ``mean over the window of q^2`` (then over the query heads of a kv group) times ``mean over the tokens of
    k^2`` -> ``[B, Hkv, D]`` (float64).  keys ``[B, Hkv, S, D]``, queries ``[B, Hq, W, D]``."""
    B, Hkv, S, D = keys.shape
    qn = queries.double().pow(2).mean(dim=2).view(B, Hkv, queries.shape[1] // Hkv, D).mean(dim=2)
    kn = keys.double().pow(2).mean(dim=2)
    return qn * kn


def think_prune(keys: torch.Tensor, queries: torch.Tensor, ratio: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """Keys with the ``int(D * ratio)`` lowest-scored channels of every (batch, kv head) zeroed, and the sorted pruned
    channel indices ``[B, Hkv, n]``; ties to the lowest channel."""
    B, Hkv, S, D = keys.shape
    n = int(D * ratio)
    scores = think_channel_scores(keys, queries)
    idx = topk_lowest_index(-scores, n)
    out = keys.clone()
    if n:
        out.scatter_(-1, idx[:, :, None, :].expand(B, Hkv, S, n), 0)
    return out, idx


def simlayer_lazy_score(keys: torch.Tensor, queries: torch.Tensor, n_initial: int, n_recent: int) -> float:
    """SimLayerKV: softmax of the last ``n_last`` queries over all keys (causal among themselves), the window's own
    columns dropped, averaged over batch, heads and queries; sum over the first ``n_initial`` and the last
    ``n_recent`` remaining keys.  keys ``[B, Hkv, S, D]``, queries ``[B, Hq, n_last, D]``."""
    B, Hkv, S, D = keys.shape
    Hq, W = queries.shape[1], queries.shape[2]
    k = keys.double().repeat_interleave(Hq // Hkv, dim=1)
    logits = torch.matmul(queries.double(), k.transpose(2, 3)) / math.sqrt(D)
    logits = logits + torch.triu(torch.full((W, S), float("-inf"), dtype=torch.float64), diagonal=S - W + 1)
    attn = torch.softmax(logits, dim=-1)[..., :S - W].mean(dim=(0, 1, 2))
    return float(attn[:n_initial].sum() + attn[-n_recent:].sum())


def simlayer_keep_positions(S: int, n_initial: int, n_recent: int, n_last: int) -> torch.Tensor:
    """Token positions a lazy layer keeps: the first ``n_initial`` and the last ``n_recent - n_last``."""
    return torch.cat([torch.arange(n_initial), torch.arange(S - (n_recent - n_last), S)])
