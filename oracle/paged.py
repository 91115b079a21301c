"""Oracle (test infrastructure): nano-vllm paged KV pool <-> HuggingFace layout.

Pool layout ``kv_cache[2, L, num_blocks, block_size, Hkv, D]``
(nanovllm/engine/llava_model_runner.py:526-529); ``kv_cache[0]`` holds K, ``kv_cache[1]`` V.
"""
from __future__ import annotations

from typing import List, Sequence, Tuple

import torch

BLOCK_SIZE = 256  # nanovllm/engine/sequence.py:15


def num_blocks_for(n_tokens: int, block_size: int = BLOCK_SIZE) -> int:
    """nanovllm/engine/sequence.py:58-59, 96-98."""
    return (n_tokens + block_size - 1) // block_size


def extract_kv(kv_cache: torch.Tensor, block_table: Sequence[int], seq_len: int
               ) -> List[Tuple[torch.Tensor, torch.Tensor]]:
    """LlavaModelRunner._extract_kv_cache_fast (llava_model_runner.py:824-872).

    Returns one ``(K, V)`` pair per layer, each ``[1, Hkv, S, D]`` (a permuted view of a fresh
    copy, as in the reference).
    """
    block_size = kv_cache.shape[3]
    needed = num_blocks_for(seq_len, block_size)
    valid = min(needed, len(block_table))                       # :834-835
    per_block = [block_size] * (valid - 1)                      # :838
    if valid > 0:
        per_block.append(seq_len - (valid - 1) * block_size)    # :839-841
    ids = [block_table[i] for i in range(valid) if block_table[i] >= 0]  # :846
    out = []
    for layer in range(kv_cache.shape[1]):
        k_parts = [kv_cache[0, layer, bid, :n] for bid, n in zip(ids, per_block)]  # :855-857
        v_parts = [kv_cache[1, layer, bid, :n] for bid, n in zip(ids, per_block)]
        if k_parts:
            k = torch.cat(k_parts, dim=0)                       # [S, Hkv, D]  :860-861
            v = torch.cat(v_parts, dim=0)
            out.append((k.permute(1, 0, 2).unsqueeze(0), v.permute(1, 0, 2).unsqueeze(0)))  # :864-865
    return out


def write_back(kv_cache: torch.Tensor, compressed: List[Tuple[torch.Tensor, torch.Tensor]],
               block_table: Sequence[int]) -> None:
    """LlavaModelRunner._write_compressed_kv_cache_fast (llava_model_runner.py:874-912).

    Writes into the leading blocks of the same table; slots past the compressed length and all
    later blocks keep whatever they held.
    """
    block_size = kv_cache.shape[3]
    for layer, (k_hf, v_hf) in enumerate(compressed):
        k_seq = k_hf.squeeze(0).permute(1, 0, 2).contiguous()   # [C, Hkv, D]  :886-887
        v_seq = v_hf.squeeze(0).permute(1, 0, 2).contiguous()
        c = k_seq.shape[0]
        written, i = 0, 0
        while written < c and i < len(block_table):             # :895
            bid = block_table[i]
            if bid < 0:                                         # :897-898
                break
            n = min(block_size, c - written)                    # :900-903
            kv_cache[0, layer, bid, :n] = k_seq[written:written + n]   # :905-908
            kv_cache[1, layer, bid, :n] = v_seq[written:written + n]
            written += n
            i += 1


def scatter_dense_into_pool(kv_cache: torch.Tensor, layer_kv: List[Tuple[torch.Tensor, torch.Tensor]],
                            block_table: Sequence[int]) -> None:
    """Test helper: place a dense ``[1, Hkv, S, D]`` KV into the pool (same addressing as write_back)."""
    write_back(kv_cache, layer_kv, block_table)


def padded_block_tables(tables: Sequence[Sequence[int]]) -> torch.Tensor:
    """LlavaModelRunner.preare_block_tables (llava_model_runner.py:541-549): int32, right-padded with -1."""
    width = max(len(t) for t in tables)
    rows = [list(t) + [-1] * (width - len(t)) for t in tables]
    return torch.tensor(rows, dtype=torch.int32)
