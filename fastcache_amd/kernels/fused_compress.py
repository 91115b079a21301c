"""Mirror of the reference's ``nanovllm/kernels/fused_compress.py`` on HIP kernels.

``fused_linear_relu_dropout`` (fused_compress.py:121-178) is one Linear (+bias, +ReLU) launch;
``FusedCompressor`` (:226-377) keeps the text MLP weights of every layer stacked as ``[L, in, out]``
and compresses one layer's K and V.  Here the three Linears of a layer are ONE launch per tensor
(``fc_ccm_mlp``) instead of three.  Dropout exists only in training mode in the reference; this build
is the inference path and refuses ``training=True`` with a positive ``dropout_p``.
"""
from __future__ import annotations

from typing import Tuple

import torch

from .. import _lib, ops
from .._lib import FastcacheError


def fused_linear_relu_dropout(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, dropout_p: float = 0.0,
                              apply_relu: bool = True, training: bool = True) -> torch.Tensor:
    """``Y = ReLU(X @ W + B)`` for ``x [M, K]``, ``weight [K, N]``, ``bias [N]`` (fused_compress.py:121-178)."""
    assert x.is_contiguous()
    assert weight.is_contiguous()
    M, K = x.shape
    K_, N = weight.shape
    assert K == K_
    if training and dropout_p > 0:
        raise FastcacheError("fused_linear_relu_dropout: dropout (training mode) is outside the inference path "
                             "built here; call with training=False")
    return ops.linear_act(x, weight.t().contiguous(), bias, apply_relu)


class FusedCompressor:
    def __init__(self, num_layers: int = 32, num_heads: int = 8, head_dim: int = 128, compression_factor: int = 5,
                 dropout_p: float = 0.4):
        self.num_layers = num_layers
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.compression_factor = compression_factor
        self.dropout_p = dropout_p
        input_dim = head_dim * compression_factor
        hidden_dim = head_dim
        for g in ("k", "v"):                       # [L, in, out] as in the reference (fused_compress.py:252-267)
            setattr(self, f"w1_{g}", torch.empty(num_layers, input_dim, hidden_dim))
            setattr(self, f"b1_{g}", torch.empty(num_layers, hidden_dim))
            setattr(self, f"w2_{g}", torch.empty(num_layers, hidden_dim, hidden_dim))
            setattr(self, f"b2_{g}", torch.empty(num_layers, hidden_dim))
            setattr(self, f"w3_{g}", torch.empty(num_layers, hidden_dim, hidden_dim))
            setattr(self, f"b3_{g}", torch.empty(num_layers, hidden_dim))
        self._packed = None

    def load_from_pytorch_module(self, pytorch_compressor):
        """Copy the text MLPs ``compress_tk / compress_tv`` (fused_compress.py:269-305)."""
        ref = next(pytorch_compressor.parameters())
        with torch.no_grad():
            for g, name in (("k", "compress_tk"), ("v", "compress_tv")):
                mods = getattr(pytorch_compressor, name)
                for i, j in ((1, 0), (2, 3), (3, 6)):
                    w = torch.stack([mods[l][j].weight.detach().T.contiguous() for l in range(self.num_layers)])
                    b = torch.stack([mods[l][j].bias.detach() for l in range(self.num_layers)])
                    setattr(self, f"w{i}_{g}", w.to(ref.device).contiguous())
                    setattr(self, f"b{i}_{g}", b.to(ref.device).contiguous())
        self._packed = None

    def _weights(self, g: str, dtype, device):
        """Kernel layout ``[L, out, in]`` in the KV dtype, cached until the stacked tensors change."""
        ts = [getattr(self, f"{n}{i}_{g}") for i in (1, 2, 3) for n in ("w", "b")]
        key = (g, dtype, device, tuple(t.data_ptr() for t in ts), tuple(t._version for t in ts))
        cache = self._packed or {}
        hit = cache.get(g)
        if hit is None or hit[0] != key:
            packed = tuple((t.transpose(1, 2) if t.dim() == 3 else t).to(device=device, dtype=dtype).contiguous()
                           for t in ts)
            hit = (key, packed)
            cache[g] = hit
            self._packed = cache
        return hit[1]

    def compress_layer_fused(self, k: torch.Tensor, v: torch.Tensor, layer_idx: int,
                             training: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
        """One layer's ``[B, H, S, D]`` K and V -> ``[B, H, S//cf + S%cf, D]`` (fused_compress.py:307-377)."""
        if training and self.dropout_p > 0:
            raise FastcacheError("FusedCompressor: dropout (training mode) is outside the inference path built here")
        B, H, S, D = k.shape
        cf = self.compression_factor
        c = S // cf
        if c < 1:
            return k, v
        out_len = c + (S - c * cf)
        outs = []
        for g, t in (("k", k), ("v", v)):
            _lib.require_gpu(t, g)
            w = tuple(x[layer_idx:layer_idx + 1] for x in self._weights(g, t.dtype, t.device))
            out = torch.empty((B, H, out_len, D), dtype=t.dtype, device=t.device)
            ops.ccm_mlp(_lib.dense_view(t), _lib.dense_view(out), w, cf, 0, S, 0)
            outs.append(out)
        return outs[0], outs[1]
