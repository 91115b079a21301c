"""Multi-step decode over the paged cache captured once as a HIP graph.

The reference captures one decode step per batch bucket and patches host-filled buffers between
replays (nanovllm/engine/llava_model_runner.py:697-710, 1109-1169).  Here the step's metadata lives
on the device — the append slot is computed from ``context_lens`` and the block table inside the
kernel, and the lengths are advanced by a kernel — so ``steps`` consecutive decode steps of every
layer are recorded into ONE graph and replayed with a single launch.  Blocks for the tokens that
will be appended must already be in the block tables (reserve ``steps`` tokens per sequence).

Per step: append the step's K/V rows of all layers at position ``len``; ``len += 1``; per layer,
attention of the step's query over ``[0, len)``.  (The reference's ``prepare_decode`` attends one
token less: it writes the new row at ``len`` but passes ``len`` as the attended length.)
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import _lib, ops


class DecodeGraph:
    def __init__(self, kv_cache: torch.Tensor, block_tables: torch.Tensor, context_lens: torch.Tensor,
                 q_steps: torch.Tensor, k_steps: torch.Tensor, v_steps: torch.Tensor, scale: float):
        """kv_cache ``[2, L, blocks, block_size, Hkv, D]``; block_tables int32 ``[B, width]``;
        context_lens int32 ``[B]`` (advanced in place by every run); q_steps ``[T, L, B, Hq, D]``;
        k_steps / v_steps ``[T, L, B, Hkv, D]``."""
        self.kv_cache, self.block_tables, self.context_lens = kv_cache, block_tables, context_lens
        self.q_steps, self.k_steps, self.v_steps, self.scale = q_steps, k_steps, v_steps, scale
        self.steps, self.num_layers, self.batch, self.num_q_heads, _ = q_steps.shape
        self.max_len = block_tables.shape[1] * kv_cache.shape[3]
        self.out = torch.empty_like(q_steps)
        self.workspace = ops.decode_attn_workspace(self.batch, self.num_q_heads, self.max_len, kv_cache.device)
        self.kview = _lib.paged_view(kv_cache[0], block_tables, None, self.max_len)
        self.vview = _lib.paged_view(kv_cache[1], block_tables, None, self.max_len)
        self.graph: Optional[torch.cuda.CUDAGraph] = None

    def _enqueue(self) -> None:
        for t in range(self.steps):
            ops.store_kv(self.kview, self.vview, self.k_steps[t], self.v_steps[t], self.context_lens)
            ops.advance_lens(self.context_lens, 1)
            for layer in range(self.num_layers):
                ops.decode_attn(self.kview, self.vview, layer, self.q_steps[t, layer], self.context_lens, self.scale,
                                self.workspace, out=self.out[t, layer])

    def run_eager(self) -> torch.Tensor:
        """The same launches without a graph (reference for the replay check)."""
        self._enqueue()
        return self.out

    def capture(self) -> None:
        """Record all steps.  ``context_lens`` is restored afterwards (capture does not execute)."""
        saved = self.context_lens.clone()
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self._enqueue()
        self.context_lens.copy_(saved)

    def replay(self) -> torch.Tensor:
        if self.graph is None:
            raise RuntimeError("capture() first")
        self.graph.replay()
        return self.out
