"""Oracle (test infrastructure): the CCM learned MLP compressors, eval mode.

Restates ``KVCacheLinearDecoupleCompressor`` (utils_ccm/module_ccm_v11.py:605-729),
``KVCacheHybridCompressor`` (:805-1060), ``MiniCPMKVCompressor``
(nanovllm/kernels/minicpm_compressor.py:16-192) and the batched re-arrangement
``BatchedGEMMCompressor`` (nanovllm/kernels/batched_compress.py:180-495).

Weights are passed in as a ``state_dict``-style mapping with the reference's key names
(``compress_tk.{layer}.{0,3,6}.{weight,bias}`` ...).  ``reference_init_state_dict`` draws them the
way the reference constructors do, so a module of this build constructed after the same
``torch.manual_seed`` holds bit-identical parameters.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

StateDict = Dict[str, torch.Tensor]
LayerKV = Tuple[torch.Tensor, torch.Tensor]


def _mlp(head_dim: int, cf: int) -> nn.Sequential:
    # module_ccm_v11.py:625-633: Linear(cf*D -> D), ReLU, Dropout(0.4), Linear, ReLU, Dropout, Linear
    return nn.Sequential(nn.Linear(head_dim * cf, head_dim), nn.ReLU(), nn.Dropout(p=0.4),
                         nn.Linear(head_dim, head_dim), nn.ReLU(), nn.Dropout(p=0.4),
                         nn.Linear(head_dim, head_dim))


def reference_init_state_dict(kind: str, n_layer: int, head_dim: int, cf: int, seed: int) -> StateDict:
    """Parameters in the creation order of the reference constructors, after ``manual_seed(seed)``.

    kind 'linear_decouple': compress_tk, compress_tv, compress_ik, compress_iv, attention
    (module_ccm_v11.py:625-664); 'hybrid': compress_tk, compress_tv only (:829-851, 877-878);
    'minicpm': tk, tv, ik, iv, attention (nanovllm/kernels/minicpm_compressor.py:42-94).
    """
    torch.manual_seed(seed)
    groups = {"linear_decouple": ["compress_tk", "compress_tv", "compress_ik", "compress_iv"],
              "minicpm": ["compress_tk", "compress_tv", "compress_ik", "compress_iv"],
              "hybrid": ["compress_tk", "compress_tv"]}[kind]
    sd: StateDict = {}
    for g in groups:
        ml = nn.ModuleList([_mlp(head_dim, cf) for _ in range(n_layer)])
        for name, p in ml.state_dict().items():
            sd[f"{g}.{name}"] = p.detach().clone()
    if kind in ("linear_decouple", "minicpm"):
        att = nn.ModuleList([nn.Linear(head_dim, 1) for _ in range(n_layer)])
        for name, p in att.state_dict().items():
            sd[f"attention.{name}"] = p.detach().clone()
    return sd


def mlp3(x: torch.Tensor, sd: StateDict, group: str, layer: int) -> torch.Tensor:
    """Eval-mode ``nn.Sequential`` of the reference: three ``nn.Linear`` with ReLU between
    (dropout is the identity).  Operands in the storage dtype, fp32 accumulation, result rounded to
    the storage dtype after every Linear — the behaviour of torch's half/bfloat16 ``F.linear`` and of
    the Triton kernel's ``tl.store(... .to(dtype))`` (nanovllm/kernels/batched_compress.py:93-122)."""
    dt = x.dtype

    def lin(inp, i):
        w = sd[f"{group}.{layer}.{i}.weight"].to(dt)
        b = sd[f"{group}.{layer}.{i}.bias"].to(dt)
        y = F.linear(inp.float(), w.float(), b.float())       # fp32 accumulate, bias before rounding
        return y.to(dt)

    h = F.relu(lin(x, 0))
    h = F.relu(lin(h, 3))
    return lin(h, 6)


def compress_segment(k: torch.Tensor, v: torch.Tensor, sd: StateDict, group_k: str, group_v: str,
                     layer: int, cf: int, min_seq_len: int) -> LayerKV:
    """``compress_layer`` (module_ccm_v11.py:666-694 / :883-925): rows of ``cf`` consecutive tokens
    go through the layer's MLP, the ``S % cf`` remainder tokens are passed through."""
    B, H, S, D = k.shape
    c = S // cf                                                   # :671
    if c < min_seq_len:                                           # :674-675
        return k, v
    n = c * cf                                                    # :677
    kx = k[:, :, :n, :].reshape(B, H, c, D * cf)                  # :679-680
    vx = v[:, :, :n, :].reshape(B, H, c, D * cf)
    ck = mlp3(kx, sd, group_k, layer)                             # :684
    cv = mlp3(vx, sd, group_v, layer)
    if S > n:                                                     # :688-692
        ck = torch.cat([ck, k[:, :, n:, :]], dim=2)
        cv = torch.cat([cv, v[:, :, n:, :]], dim=2)
    return ck, cv


def linear_decouple_forward(kv_cache: Sequence[LayerKV], it_len: Sequence[int], sd: StateDict,
                            cf: int = 2, min_seq_len: int = 1) -> List[LayerKV]:
    """``KVCacheLinearDecoupleCompressor.forward`` (module_ccm_v11.py:697-729); also
    ``MiniCPMKVCompressor.forward`` for ``it_len[0] > 0``."""
    out = []
    for layer, (k, v) in enumerate(kv_cache):
        ik, iv = k[:, :, :it_len[0], :], v[:, :, :it_len[0], :]   # :706-709
        tk, tv = k[:, :, it_len[0]:, :], v[:, :, it_len[0]:, :]
        cik, civ = compress_segment(ik, iv, sd, "compress_ik", "compress_iv", layer, cf, min_seq_len)
        ctk, ctv = compress_segment(tk, tv, sd, "compress_tk", "compress_tv", layer, cf, min_seq_len)
        out.append((torch.cat([cik, ctk], dim=2).contiguous(),    # :718-720, :729
                    torch.cat([civ, ctv], dim=2).contiguous()))
    return out


def hybrid_forward(kv_cache: Sequence[LayerKV], it_len: Sequence[int], sd: StateDict,
                   cf: int = 2, min_seq_len: int = 1) -> List[LayerKV]:
    """``KVCacheHybridCompressor.forward`` list branch (module_ccm_v11.py:1000-1060).  The class has
    no image MLPs (:877-878): with ``it_len[0] > 0`` the reference indexes ``None`` and raises
    ``TypeError`` as soon as the image segment is long enough to be compressed."""
    out = []
    for layer, (k, v) in enumerate(kv_cache):
        if it_len[0] == 0:                                        # :1006-1019
            ck, cv = compress_segment(k, v, sd, "compress_tk", "compress_tv", layer, cf, min_seq_len)
        else:                                                     # :1020-1046
            ik, iv = k[:, :, :it_len[0], :], v[:, :, :it_len[0], :]
            tk, tv = k[:, :, it_len[0]:, :], v[:, :, it_len[0]:, :]
            if ik.shape[2] // cf >= min_seq_len:
                raise TypeError("'NoneType' object is not subscriptable")
            ctk, ctv = compress_segment(tk, tv, sd, "compress_tk", "compress_tv", layer, cf, min_seq_len)
            ck, cv = torch.cat([ik, ctk], dim=2), torch.cat([iv, ctv], dim=2)
        out.append((ck.contiguous(), cv.contiguous()))
    return out


def minicpm_forward(kv_cache: Sequence[LayerKV], it_len: Sequence[int], sd: StateDict,
                    cf: int = 5, min_seq_len: int = 2) -> List[LayerKV]:
    """``MiniCPMKVCompressor.forward`` (nanovllm/kernels/minicpm_compressor.py:127-192): text MLPs over
    the whole sequence when ``it_len[0] == 0`` (:154-162), otherwise the image/text split."""
    if it_len[0] == 0:
        return [tuple(t.contiguous() for t in
                      compress_segment(k, v, sd, "compress_tk", "compress_tv", layer, cf, min_seq_len))
                for layer, (k, v) in enumerate(kv_cache)]
    return linear_decouple_forward(kv_cache, it_len, sd, cf, min_seq_len)


def compressed_length(seq_len: int, it_len: Sequence[int], cf: int, min_seq_len: int,
                      split: bool = True) -> int:
    """Length after compression: per segment ``c + (n - c*cf)`` when ``c = n // cf >= min_seq_len``
    else ``n``."""
    def seg(n):
        c = n // cf
        return n if c < min_seq_len else c + (n - c * cf)
    if not split or it_len[0] == 0:
        return seg(seq_len)
    return seg(min(it_len[0], seq_len)) + seg(max(0, seq_len - it_len[0]))


def batched_weights_from_state_dict(sd: StateDict, group: str, n_layer: int
                                    ) -> Tuple[torch.Tensor, ...]:
    """``BatchedGEMMCompressor.load_from_original_compressor``
    (nanovllm/kernels/batched_compress.py:260-313): stacked, transposed weights
    ``w[L, in, out] = Linear.weight.T`` and ``b[L, out]``."""
    ws = []
    for i in (0, 3, 6):
        ws.append(torch.stack([sd[f"{group}.{l}.{i}.weight"].T.contiguous() for l in range(n_layer)]))
        ws.append(torch.stack([sd[f"{group}.{l}.{i}.bias"] for l in range(n_layer)]))
    return tuple(ws)


def batched_mlp_forward(x: torch.Tensor, w1, b1, w2, b2, w3, b3) -> torch.Tensor:
    """``_batched_mlp_forward`` bmm branch (batched_compress.py:347-357) with the same rounding as
    ``mlp3``.  x ``[L, M, in]``."""
    dt = x.dtype

    def lin(inp, w, b):
        return (torch.bmm(inp.float(), w.to(dt).float()) + b.to(dt).float().unsqueeze(1)).to(dt)

    h = F.relu(lin(x, w1, b1))
    h = F.relu(lin(h, w2, b2))
    return lin(h, w3, b3)
