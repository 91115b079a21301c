"""Decode branch of nano-vllm's ``Attention`` layer over the paged cache
(nanovllm/layers/attention.py:32-79): append the step's K/V rows, then single-query paged
attention.  Prefill attention is outside the compression path and is not provided.
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import nn

from .. import _lib, ops
from .._lib import check, current_stream, fn
from ..utils.context import get_context


def store_kvcache(key: torch.Tensor, value: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                  slot_mapping: torch.Tensor) -> None:
    """``cache.view(-1, Hkv*D)[slot_mapping[i]] = key[i] / value[i]`` (attention.py:32-39).
    key/value ``[N, Hkv, D]``; caches ``[num_blocks, block_size, Hkv, D]``; slot_mapping int32 ``[N]``."""
    N, H, D = key.shape
    row = H * D
    for t, name in ((key, "key"), (value, "value"), (k_cache, "k_cache"), (v_cache, "v_cache")):
        _lib.require_gpu(t, name)
    assert key.stride(-1) == 1 and value.stride(-1) == 1
    assert key.stride(1) == D and value.stride(1) == D
    assert k_cache.stride(1) == row and v_cache.stride(1) == row
    assert slot_mapping.numel() == N and slot_mapping.dtype == torch.int32
    check(fn("fc_store_kv_slots")(key.data_ptr(), key.stride(0), value.data_ptr(), value.stride(0),
                                  k_cache.data_ptr(), v_cache.data_ptr(), slot_mapping.data_ptr(), N, row,
                                  _lib.dtype_code(key.dtype), current_stream()), "fc_store_kv_slots")


_workspaces = {}


def decode_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, cache_seqlens: torch.Tensor,
                     block_table: torch.Tensor, softmax_scale: float, out: Optional[torch.Tensor] = None,
                     workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Stand-in for ``flash_attn_with_kvcache(q, k_cache, v_cache, cache_seqlens=, block_table=,
    softmax_scale=, causal=True)`` with one query token per sequence (attention.py:75-77).
    q ``[B, 1, Hq, D]`` or ``[B, Hq, D]``; caches ``[num_blocks, block_size, Hkv, D]``; returns q's shape."""
    shape = q.shape
    q3 = q.reshape(shape[0], shape[-2], shape[-1])
    if not q3.is_contiguous():
        q3 = q3.contiguous()
    B, Hq, D = q3.shape
    max_len = block_table.shape[1] * k_cache.shape[1]
    kview = _lib.paged_view(k_cache.unsqueeze(0), block_table, None, max_len)
    vview = _lib.paged_view(v_cache.unsqueeze(0), block_table, None, max_len)
    if workspace is None:
        key = (q.device, B, Hq, max_len)
        workspace = _workspaces.get(key)
        if workspace is None:
            workspace = ops.decode_attn_workspace(B, Hq, max_len, q.device)
            _workspaces.clear()          # keep one live workspace
            _workspaces[key] = workspace
    o = ops.decode_attn(kview, vview, 0, q3, cache_seqlens, softmax_scale, workspace, out)
    return o.view(shape)


class Attention(nn.Module):
    """Same constructor and cache attributes as the reference layer; ``forward`` serves decode steps."""

    def __init__(self, num_heads, head_dim, scale, num_kv_heads):
        super().__init__()
        self.num_heads, self.head_dim, self.scale, self.num_kv_heads = num_heads, head_dim, scale, num_kv_heads
        self.k_cache = self.v_cache = torch.tensor([])
        self.workspace: Optional[torch.Tensor] = None   # set by a graph runner that owns the scratch memory

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
        q = q.view(-1, self.num_heads, self.head_dim)
        k = k.view(-1, self.num_kv_heads, self.head_dim)
        v = v.view(-1, self.num_kv_heads, self.head_dim)
        ctx = get_context()
        store_kvcache(k, v, self.k_cache, self.v_cache, ctx.slot_mapping)
        if ctx.is_prefill:
            raise NotImplementedError("prefill attention is outside the KV-cache compression path built here")
        o = decode_attention(q.unsqueeze(1), self.k_cache, self.v_cache, ctx.context_lens, ctx.block_tables, self.scale,
                             workspace=self.workspace)
        return o.view(-1, self.num_heads * self.head_dim)
