"""Seeded synthetic inputs for the five benchmark configurations and their small variants.

Draw order is fixed (K, then V, then Q) from one ``torch.Generator`` on the CPU in fp32; values are
then scaled, cast to the storage dtype and scattered into a paged pool
``[2, L, num_blocks, block_size, Hkv, D]`` through per-sequence block tables taken from a seeded
permutation of the block ids.  ``device_draw=True`` draws on the target device instead (much
faster at full size, same distribution, different values) for throughput runs.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional

import torch

BLOCK_SIZE = 256


@dataclass
class PagedCase:
    """A paged pool holding ``B`` sequences plus everything needed to address it."""
    kv_cache: torch.Tensor                 # [2, L, num_blocks, block_size, Hkv, D]
    block_tables: List[List[int]]          # per sequence
    seq_lens: List[int]
    dense_k: Optional[torch.Tensor] = None  # [L, B, Hkv, S, D] (only when keep_dense)
    dense_v: Optional[torch.Tensor] = None
    queries: Optional[torch.Tensor] = None  # [L, B, Hq, W, D]
    extra: dict = field(default_factory=dict)

    @property
    def block_size(self) -> int:
        return self.kv_cache.shape[3]

    def table_tensor(self, device=None, width: Optional[int] = None) -> torch.Tensor:
        w = max(len(t) for t in self.block_tables) if width is None else width
        rows = [list(t) + [-1] * (w - len(t)) for t in self.block_tables]
        return torch.tensor(rows, dtype=torch.int32, device=device or self.kv_cache.device)

    def lens_tensor(self, device=None) -> torch.Tensor:
        return torch.tensor(self.seq_lens, dtype=torch.int32, device=device or self.kv_cache.device)


def _randn(shape, g: torch.Generator, device, device_draw: bool) -> torch.Tensor:
    if device_draw:
        return torch.randn(shape, generator=g, device=device, dtype=torch.float32)
    return torch.randn(shape, generator=g, dtype=torch.float32)


def make_tables(seq_lens: List[int], num_blocks: int, g: torch.Generator, shuffle: bool,
                block_size: int = BLOCK_SIZE, reserve_tokens: int = 0) -> List[List[int]]:
    """Block tables covering ``len + reserve_tokens`` tokens each, from a seeded permutation
    (``shuffle``) or in allocation order."""
    need = [(n + reserve_tokens + block_size - 1) // block_size for n in seq_lens]
    if sum(need) > num_blocks:
        raise ValueError(f"{sum(need)} blocks needed, pool has {num_blocks}")
    cpu_g = torch.Generator().manual_seed(int(g.initial_seed()) + 7919)
    order = torch.randperm(num_blocks, generator=cpu_g).tolist() if shuffle else list(range(num_blocks))
    tables, at = [], 0
    for n in need:
        tables.append(order[at:at + n])
        at += n
    return tables


def pool_slot_index(tables: List[List[int]], seq_lens: List[int], block_size: int, dense_len: int, device=None):
    """For every token of every sequence, in sequence order: its row in the flattened pool
    (``table[s // block_size] * block_size + s % block_size``) and its row in a dense ``[B, S]`` token grid
    (``b * dense_len + s``), as two int64 tensors."""
    slots, rows = [], []
    for b, (tab, n) in enumerate(zip(tables, seq_lens)):
        pos = torch.arange(n, dtype=torch.int64)
        slots.append(torch.tensor(tab, dtype=torch.int64)[pos // block_size] * block_size + pos % block_size)
        rows.append(pos + b * dense_len)
    slots, rows = torch.cat(slots), torch.cat(rows)
    return (slots.to(device), rows.to(device)) if device is not None else (slots, rows)


def scatter_into_pool(kv_cache: torch.Tensor, plane: int, layer: int, dense: torch.Tensor,
                      tables: List[List[int]], seq_lens: List[int], index=None) -> None:
    """dense ``[B, Hkv, S, D]`` -> pool pages of ``kv_cache[plane, layer]``: one indexed store for the whole
    batch (``index`` = a ``pool_slot_index`` result, to reuse it across layers and planes)."""
    bs = kv_cache.shape[3]
    B, H, S, D = dense.shape
    slots, rows = index if index is not None else pool_slot_index(tables, seq_lens, bs, S, kv_cache.device)
    flat = kv_cache[plane, layer].view(-1, H, D)                                  # [num_blocks * block_size, Hkv, D]
    tokens = dense.permute(0, 2, 1, 3).reshape(B * S, H, D)                       # [B * S, Hkv, D]
    flat.index_copy_(0, slots, tokens.index_select(0, rows.to(tokens.device)).to(flat.device))


def make_paged_case(*, seed: int, num_layers: int, batch: int, num_kv_heads: int, seq_lens: List[int],
                    dtype: torch.dtype, device="cpu", head_dim: int = 128, num_q_heads: int = 0,
                    window: int = 0, outlier_channels: int = 0, outlier_scale: float = 8.0,
                    image_tokens: int = 0, image_scale: float = 1.0, shuffle_tables: bool = True,
                    extra_blocks: int = 2, reserve_tokens: int = 0, keep_dense: bool = False,
                    device_draw: bool = False, block_size: int = BLOCK_SIZE, fill_value: float = 0.0
                    ) -> PagedCase:
    """Generic builder behind the per-config helpers below."""
    assert len(seq_lens) == batch
    dev = torch.device(device)
    g = torch.Generator(device=dev if device_draw else "cpu").manual_seed(seed)
    S = max(seq_lens)
    need = sum((n + reserve_tokens + block_size - 1) // block_size for n in seq_lens)
    num_blocks = need + extra_blocks
    kv_cache = torch.full((2, num_layers, num_blocks, block_size, num_kv_heads, head_dim), fill_value,
                          dtype=dtype, device=dev)
    tables = make_tables(seq_lens, num_blocks, g, shuffle_tables, block_size, reserve_tokens)
    outl = None
    if outlier_channels:
        # channel ids drawn once per head
        og = torch.Generator().manual_seed(seed + 104729)
        outl = torch.stack([torch.randperm(head_dim, generator=og)[:outlier_channels]
                            for _ in range(num_kv_heads)])       # [Hkv, n_out]
    dk = dv = None
    if keep_dense:
        dk = torch.empty((num_layers, batch, num_kv_heads, S, head_dim), dtype=dtype, device=dev)
        dv = torch.empty_like(dk)
    index = pool_slot_index(tables, seq_lens, block_size, S, dev)
    for layer in range(num_layers):
        planes = []
        for _ in range(2):                                        # K then V
            x = _randn((batch, num_kv_heads, S, head_dim), g, dev, device_draw)
            if outl is not None:
                mult = torch.ones((num_kv_heads, head_dim), dtype=torch.float32)
                mult.scatter_(1, outl, outlier_scale)
                x = x * mult.to(x.device)[None, :, None, :]
            if image_tokens and image_scale != 1.0:
                x[:, :, :image_tokens] *= image_scale
            planes.append(x.to(dtype).to(dev))
        for p, x in enumerate(planes):
            scatter_into_pool(kv_cache, p, layer, x, tables, seq_lens, index)
        if keep_dense:
            dk[layer], dv[layer] = planes
    q = None
    if num_q_heads and window:
        q = torch.stack([_randn((batch, num_q_heads, window, head_dim), g, dev, device_draw).to(dtype).to(dev)
                         for _ in range(num_layers)])
    return PagedCase(kv_cache, tables, list(seq_lens), dk, dv, q)


# ---- the five configurations (full size by default; pass smaller numbers for tests) -------------
def knorm_case(seed=0, num_layers=32, num_kv_heads=32, seq_len=1024, batch=1, dtype=torch.float32, **kw):
    """Config 1: LLaMA-7B-shaped fp32 KV, 4 outlier channels per head scaled x8."""
    return make_paged_case(seed=seed, num_layers=num_layers, batch=batch, num_kv_heads=num_kv_heads,
                           seq_lens=[seq_len] * batch, dtype=dtype, outlier_channels=4, **kw)


def snapkv_case(seed=0, num_layers=36, batch=8, num_q_heads=32, num_kv_heads=8, seq_len=4096, window=64,
                dtype=torch.bfloat16, **kw):
    """Config 2: Qwen3-8B-shaped GQA, bf16, window queries for the last 64 positions."""
    return make_paged_case(seed=seed, num_layers=num_layers, batch=batch, num_kv_heads=num_kv_heads,
                           seq_lens=[seq_len] * batch, dtype=dtype, num_q_heads=num_q_heads, window=window, **kw)


def ccm_case(seed=0, num_layers=32, batch=45, num_kv_heads=32, image_tokens=576, text_tokens=64,
             dtype=torch.float16, **kw):
    """Config 3: LLaVA-1.5-7B-shaped fp16 KV, image rows scaled x0.5."""
    return make_paged_case(seed=seed, num_layers=num_layers, batch=batch, num_kv_heads=num_kv_heads,
                           seq_lens=[image_tokens + text_tokens] * batch, dtype=dtype,
                           image_tokens=image_tokens, image_scale=0.5, **kw)


def decode_case(seed=0, num_layers=32, batch=90, num_kv_heads=32, min_len=128, max_len=2048, steps=128,
                dtype=torch.float16, **kw):
    """Config 4: per-sequence lengths uniform in [min_len, max_len], shuffled tables, room for ``steps``
    appended tokens."""
    g = torch.Generator().manual_seed(seed + 15485863)
    lens = torch.randint(min_len, max_len + 1, (batch,), generator=g).tolist()
    return make_paged_case(seed=seed, num_layers=num_layers, batch=batch, num_kv_heads=num_kv_heads,
                           seq_lens=lens, dtype=dtype, reserve_tokens=steps + 1, **kw)


def hybrid_case(seed=0, num_layers=28, batch=16, num_kv_heads=4, seq_len=16384, dtype=torch.bfloat16, **kw):
    """Config 5: MiniCPM-V-2.6 LLM shape (Qwen2-7B), bf16, long prompts."""
    return make_paged_case(seed=seed, num_layers=num_layers, batch=batch, num_kv_heads=num_kv_heads,
                           seq_lens=[seq_len] * batch, dtype=dtype, **kw)
