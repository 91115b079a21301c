"""Oracle (test infrastructure): decode paged attention and the KV store.

``flash_attn_with_kvcache`` (third-party flash-attn, unpinned in requirements.txt:15; call site
nanovllm/layers/attention.py:75-77) is restated from its definition: for one query token per
sequence, ``softmax(q K^T * scale) V`` over the first ``cache_seqlens[b]`` cached tokens found
through ``block_table``, fp32 softmax and accumulation, output in the input dtype.
"""
from __future__ import annotations

import torch


def store_kv(k_cache: torch.Tensor, v_cache: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor,
             slot_mapping: torch.Tensor) -> None:
    """``store_kvcache`` (nanovllm/layers/attention.py:10-39): ``cache.view(-1, Hkv*D)[slot] = new``.
    caches ``[num_blocks, block_size, Hkv, D]``; new ``[N, Hkv, D]``; slot_mapping ``[N]``."""
    nb, bs, h, d = k_cache.shape
    kf, vf = k_cache.view(nb * bs, h, d), v_cache.view(nb * bs, h, d)
    for i, slot in enumerate(slot_mapping.tolist()):
        kf[slot] = k_new[i]
        vf[slot] = v_new[i]


def decode_slot(block_table, kv_len: int, block_size: int = 256) -> int:
    """Slot of the token appended at position ``kv_len``
    (nanovllm/engine/llava_model_runner.py:655-665)."""
    bi, pos = kv_len // block_size, kv_len % block_size
    if bi < len(block_table):
        return block_table[bi] * block_size + pos
    return block_table[-1] * block_size + pos


def decode_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                     cache_seqlens: torch.Tensor, block_table: torch.Tensor, scale: float) -> torch.Tensor:
    """q ``[B, Hq, D]``; caches ``[num_blocks, block_size, Hkv, D]``; returns ``[B, Hq, D]`` in q's dtype.
    Rows with ``cache_seqlens[b] <= 0`` return zeros."""
    B, Hq, D = q.shape
    nb, bs, Hkv, _ = k_cache.shape
    G = Hq // Hkv
    out = torch.zeros_like(q)
    for b in range(B):
        n = int(cache_seqlens[b])
        if n <= 0:
            continue
        nblk = (n + bs - 1) // bs
        ids = block_table[b, :nblk].long()
        k = k_cache[ids].reshape(nblk * bs, Hkv, D)[:n].float()      # [n, Hkv, D]
        v = v_cache[ids].reshape(nblk * bs, Hkv, D)[:n].float()
        k = k.repeat_interleave(G, dim=1).permute(1, 0, 2)           # [Hq, n, D]
        v = v.repeat_interleave(G, dim=1).permute(1, 0, 2)
        logits = torch.einsum("hd,hnd->hn", q[b].float(), k) * scale
        p = torch.softmax(logits, dim=-1, dtype=torch.float32)
        out[b] = torch.einsum("hn,hnd->hd", p, v).to(q.dtype)
    return out
