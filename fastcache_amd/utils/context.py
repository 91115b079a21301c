"""What an attention layer needs to know about the step it runs in.

The field names are those of nano-vllm's step context (nanovllm/utils/context.py:7-27), because its attention
layers and model runner read them by name; the holder is one module-level record that is overwritten field by
field, so a reference taken by ``get_context()`` stays valid across steps.
"""
from __future__ import annotations

from typing import Optional

import torch

_FIELDS = {           # name -> value outside any step
    "is_prefill": False,
    "cu_seqlens_q": None,
    "cu_seqlens_k": None,
    "max_seqlen_q": 0,
    "max_seqlen_k": 0,
    "slot_mapping": None,      # int32 [tokens]: flat cache slot of every new K/V row (-1 = skip)
    "context_lens": None,      # int32 [B]: cached tokens each sequence attends (decode)
    "block_tables": None,      # int32 [B, width], -1 padded (decode)
}


class Context:
    __slots__ = tuple(_FIELDS)

    is_prefill: bool
    max_seqlen_q: int
    max_seqlen_k: int
    cu_seqlens_q: Optional[torch.Tensor]
    cu_seqlens_k: Optional[torch.Tensor]
    slot_mapping: Optional[torch.Tensor]
    context_lens: Optional[torch.Tensor]
    block_tables: Optional[torch.Tensor]

    def __init__(self, **values):
        self.assign(**values)

    def assign(self, **values) -> None:
        unknown = set(values) - set(_FIELDS)
        if unknown:
            raise TypeError(f"unknown context fields: {sorted(unknown)}")
        for name, default in _FIELDS.items():
            setattr(self, name, values.get(name, default))

    def __repr__(self):
        return "Context(" + ", ".join(f"{n}={getattr(self, n)!r}" for n in _FIELDS) + ")"


_current = Context()


def get_context() -> Context:
    return _current


def set_context(is_prefill, cu_seqlens_q=None, cu_seqlens_k=None, max_seqlen_q=0, max_seqlen_k=0,
                slot_mapping=None, context_lens=None, block_tables=None) -> None:
    _current.assign(is_prefill=is_prefill, cu_seqlens_q=cu_seqlens_q, cu_seqlens_k=cu_seqlens_k,
                    max_seqlen_q=max_seqlen_q, max_seqlen_k=max_seqlen_k, slot_mapping=slot_mapping,
                    context_lens=context_lens, block_tables=block_tables)


def reset_context() -> None:
    _current.assign()
