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

from typing import Dict, List, Optional, Sequence

import torch

from .. import _lib, ops
from ..utils.context import get_context, reset_context, set_context


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

    def _enqueue(self, steps: Optional[int] = None) -> None:
        for t in range(self.steps if steps is None else steps):
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
        # One step outside the graph first: whatever a kernel's first launch does on the host (loading its code
        # object, raising its LDS limit) happens here and not inside the capture.  It appends the rows the
        # replays will append anyway and its lengths are put back.
        self._enqueue(1)
        torch.cuda.synchronize()
        self.context_lens.copy_(saved)
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


class BucketedDecodeGraphs:
    """One captured decode step per batch bucket, replayed with host-patched static buffers: the
    protocol of ``capture_cudagraph`` / ``reset_graph_vars`` / the decode branch of ``run_model``
    (nanovllm/engine/llava_model_runner.py:1109-1169, 914-921, 697-710), with the attention layers
    standing in for the model.

    ``layers`` are ``fastcache_amd.layers.Attention`` modules whose ``k_cache`` / ``v_cache`` are set.
    A step takes q ``[L, bs, Hq*D]`` and k, v ``[L, bs, Hkv*D]`` and the decode context
    (``set_context(False, slot_mapping=, context_lens=, block_tables=)``) and returns ``[L, bs, Hq*D]``.
    Padded rows of a bucket get ``context_len = 0`` and ``slot = -1`` (skipped by the append kernel); the
    reference zeroes the slot instead, which makes every padded row overwrite slot 0 of block 0.
    """

    def __init__(self, layers: Sequence, max_bs: int, max_num_blocks: int, dtype: torch.dtype, device):
        self.layers = list(layers)
        self.max_bs, self.max_num_blocks = min(max_bs, 256), max_num_blocks
        self.dtype, self.device = dtype, torch.device(device)
        self.graphs: Dict[int, torch.cuda.CUDAGraph] = {}
        self.graph_bs: List[int] = []
        self.graph_vars: Dict[str, torch.Tensor] = {}
        self.graph_pool = None

    def _model(self, q, k, v, out):
        for i, layer in enumerate(self.layers):
            out[i] = layer(q[i], k[i], v[i])

    @torch.inference_mode()
    def capture_cudagraph(self):
        a = self.layers[0]
        L, bsz, dev = len(self.layers), self.max_bs, self.device
        block_size = a.k_cache.shape[1]
        slot_mapping = torch.full((bsz,), -1, dtype=torch.int32, device=dev)
        context_lens = torch.zeros(bsz, dtype=torch.int32, device=dev)
        block_tables = torch.zeros(bsz, self.max_num_blocks, dtype=torch.int32, device=dev)
        q = torch.zeros(L, bsz, a.num_heads * a.head_dim, dtype=self.dtype, device=dev)
        k = torch.zeros(L, bsz, a.num_kv_heads * a.head_dim, dtype=self.dtype, device=dev)
        v = torch.zeros_like(k)
        outputs = torch.zeros_like(q)
        workspace = ops.decode_attn_workspace(bsz, a.num_heads, self.max_num_blocks * block_size, dev)
        for layer in self.layers:
            layer.workspace = workspace
        self.graph_bs = [b for b in [1, 2, 4, 8] + list(range(16, bsz + 1, 16)) if b <= bsz]
        if self.graph_bs[-1] != bsz:
            self.graph_bs.append(bsz)
        for bs in reversed(self.graph_bs):
            graph = torch.cuda.CUDAGraph()
            set_context(False, slot_mapping=slot_mapping[:bs], context_lens=context_lens[:bs],
                        block_tables=block_tables[:bs])
            self._model(q[:, :bs], k[:, :bs], v[:, :bs], outputs[:, :bs])       # warm-up outside the graph
            with torch.cuda.graph(graph, self.graph_pool):
                self._model(q[:, :bs], k[:, :bs], v[:, :bs], outputs[:, :bs])
            if self.graph_pool is None:
                self.graph_pool = graph.pool()
            self.graphs[bs] = graph
            torch.cuda.synchronize()
            reset_context()
        self.graph_vars = dict(slot_mapping=slot_mapping, context_lens=context_lens, block_tables=block_tables,
                               q=q, k=k, v=v, outputs=outputs)

    def reset_graph_vars(self):
        gv = self.graph_vars
        gv["slot_mapping"].fill_(-1)
        gv["context_lens"].zero_()
        gv["block_tables"].zero_()

    @torch.inference_mode()
    def run(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
        """Replay the graph of the smallest bucket that holds the batch, with the current decode context."""
        bs = q.shape[1]
        context = get_context()
        self.reset_graph_vars()
        graph = self.graphs[next(x for x in self.graph_bs if x >= bs)]
        gv = self.graph_vars
        gv["q"][:, :bs] = q
        gv["k"][:, :bs] = k
        gv["v"][:, :bs] = v
        gv["slot_mapping"][:bs] = context.slot_mapping
        gv["context_lens"][:bs] = context.context_lens
        gv["block_tables"][:bs, :context.block_tables.size(1)] = context.block_tables
        graph.replay()
        return gv["outputs"][:, :bs]
