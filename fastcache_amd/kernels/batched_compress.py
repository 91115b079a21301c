"""``BatchedGEMMCompressor`` (nanovllm/kernels/batched_compress.py:180-653): the CCM MLPs with the
weights of all layers stacked, so that one launch per (K|V, segment) covers every layer.

Parameters keep the reference's names and layout (``w{1,2,3}_{tk,tv,ik,iv}[L, in, out]``, i.e.
``nn.Linear.weight.T``, and ``b*[L, out]``); the kernel wants ``[L, out, in]``, so a transposed copy
is cached per group.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch
import torch.nn as nn

from .. import _lib, ops

LayerKV = Tuple[torch.Tensor, torch.Tensor]
_GROUPS = ("tk", "tv", "ik", "iv")


class BatchedGEMMCompressor(nn.Module):
    def __init__(self, num_layers: int = 32, num_heads: int = 8, head_dim: int = 128, compression_factor: int = 5,
                 min_seq_len: int = 1, use_triton: bool = True):
        super().__init__()
        self.num_layers, self.num_heads, self.head_dim = num_layers, num_heads, head_dim
        self.compression_factor, self.min_seq_len = compression_factor, min_seq_len
        self.use_triton = use_triton        # kept for signature compatibility; there is one HIP path
        d_in = head_dim * compression_factor
        for g in _GROUPS:                   # registration order of the reference: per group w1,b1,w2,b2,w3,b3
            for i, k in ((1, d_in), (2, head_dim), (3, head_dim)):
                setattr(self, f"w{i}_{g}", nn.Parameter(torch.empty(num_layers, k, head_dim)))
                setattr(self, f"b{i}_{g}", nn.Parameter(torch.empty(num_layers, head_dim)))
        self._init_weights()
        self._packed = {}

    def _init_weights(self):
        """Xavier-uniform weights, zero biases (batched_compress.py:252-258)."""
        for name, p in self.named_parameters():
            if "w" in name:
                nn.init.xavier_uniform_(p)
            elif "b" in name:
                nn.init.zeros_(p)

    def load_from_original_compressor(self, original_compressor):
        """Copy ``compress_{tk,tv,ik,iv}[layer][{0,3,6}]`` into the stacked layout
        (batched_compress.py:260-313) and follow the original's device and dtype."""
        ref = next(original_compressor.parameters())
        with torch.no_grad():
            for g in _GROUPS:
                mods = getattr(original_compressor, f"compress_{g}")
                for layer in range(self.num_layers):
                    m = mods[layer]
                    for i, j in ((1, 0), (2, 3), (3, 6)):
                        getattr(self, f"w{i}_{g}")[layer] = m[j].weight.T
                        getattr(self, f"b{i}_{g}")[layer] = m[j].bias
        self.to(device=ref.device, dtype=ref.dtype)
        self._packed = {}

    def _apply(self, fn, *a, **kw):
        self._packed = {}
        return super()._apply(fn, *a, **kw)

    def _weights(self, g: str, dtype, device, layers: Optional[Tuple[int, int]] = None):
        ps = [getattr(self, f"{n}{i}_{g}") for i in (1, 2, 3) for n in ("w", "b")]
        key = (dtype, device, tuple(p._version for p in ps), tuple(p.data_ptr() for p in ps))
        hit = self._packed.get(g)
        if hit is None or hit[0] != key:
            with torch.no_grad():
                packed = tuple((p.detach().transpose(1, 2) if p.dim() == 3 else p.detach())
                               .to(device=device, dtype=dtype).contiguous() for p in ps)
            hit = (key, packed)
            self._packed[g] = hit
        w = hit[1]
        return w if layers is None else tuple(t[layers[0]:layers[1]] for t in w)

    # -- segments ---------------------------------------------------------------------------------
    def _seg_len(self, n: int) -> int:
        c = n // self.compression_factor
        return n if c < self.min_seq_len else c + (n - c * self.compression_factor)

    def _run(self, kv_cache: Sequence[LayerKV], it_len, l0: int, l1: int) -> List[LayerKV]:
        """All layers ``[l0, l1)`` of ``kv_cache`` (indexed from 0 = layer l0)."""
        if len(kv_cache) == 0:
            return list(kv_cache)
        k0 = kv_cache[0][0]
        _lib.require_gpu(k0, "kv_cache")
        B, H, S, D = k0.shape
        img = min(int(it_len[0]), S) if it_len[0] > 0 else 0
        C = self._seg_len(img) + self._seg_len(S - img)
        L = len(kv_cache)
        cf = self.compression_factor
        # one stacked copy of the layer list (the reference stacks as well, batched_compress.py:394-395)
        src = [torch.stack([kv[p] for kv in kv_cache]) for p in range(2)]
        out = [torch.empty((L, B, H, C, D), dtype=k0.dtype, device=k0.device) for _ in range(2)]
        for p, kind in ((0, "k"), (1, "v")):
            sv, dv = _lib.dense_view(src[p]), _lib.dense_view(out[p])
            dst = 0
            for seg_start, n, g in ((0, img, "i" + kind), (img, S - img, "t" + kind)):
                if n == 0:
                    continue
                if n // cf < self.min_seq_len:
                    ops.copy_tokens(sv, dv, seg_start, n, dst)
                else:
                    ops.ccm_mlp(sv, dv, self._weights(g, k0.dtype, k0.device, (l0, l1)), cf, seg_start, n, dst)
                dst += self._seg_len(n)
        return [(out[0][i], out[1][i]) for i in range(L)]

    def paged_compressed_len(self, seq_len: int, it_len: Sequence[int]) -> int:
        img = min(int(it_len[0]), seq_len) if it_len[0] > 0 else 0
        return (self._seg_len(img) if img else 0) + (self._seg_len(seq_len - img) if seq_len > img else 0)

    @torch.no_grad()
    def paged_forward(self, kv_cache: torch.Tensor, block_tables: torch.Tensor, seq_lens: torch.Tensor,
                      seq_len: int, it_len: Sequence[int], layers: Optional[Tuple[int, int]] = None,
                      out: Optional[torch.Tensor] = None, host_lens: Optional[Sequence[int]] = None):
        """On a paged pool ``[2, L, blocks, block_size, Hkv, D]`` for sequences that all hold ``seq_len``
        tokens: in place, or for the layers ``layers=(l0, l1)`` only, or into ``out [2, L, B, Hkv, C, D]``
        leaving the pages untouched; returns the compressed length.  Sequences of different lengths:
        ``host_lens`` (Python ints; ``seq_len`` is their maximum) -> the list of compressed lengths, from the
        same number of launches."""
        cf = self.compression_factor
        img = min(int(it_len[0]), seq_len) if it_len[0] > 0 else 0
        l0, l1 = layers if layers is not None else (0, kv_cache.shape[1])
        dst = 0
        views = [_lib.paged_view(kv_cache[p][l0:l1], block_tables, seq_lens, seq_len) for p in range(2)]
        dviews = views if out is None else [_lib.dense_view(out[p][l0:l1]) for p in range(2)]
        if host_lens is not None and len(set(host_lens)) > 1:
            dev = kv_cache.device
            mk = lambda xs: torch.tensor(xs, dtype=torch.int32, device=dev)
            imgs = [min(int(it_len[0]), n) if it_len[0] > 0 else 0 for n in host_lens]
            dsts = [0] * len(imgs)
            for starts, counts, seg in (([0] * len(imgs), imgs, "i"), (imgs, [n - i for n, i in zip(host_lens, imgs)], "t")):
                if max(counts) == 0:
                    continue
                st, ct, dt = mk(starts), mk(counts), mk(dsts)
                for view, dview, kind in ((views[0], dviews[0], "k"), (views[1], dviews[1], "v")):
                    ops.ccm_mlp_ragged(view, dview, self._weights(seg + kind, kv_cache.dtype, dev, (l0, l1)), cf, st, ct,
                                       dt, max(counts), self.min_seq_len)
                dsts = [d + self._seg_len(n) for d, n in zip(dsts, counts)]
            return dsts
        for s0, n, seg in ((0, img, "i"), (img, seq_len - img, "t")):
            if n == 0:
                continue
            for view, dview, kind in ((views[0], dviews[0], "k"), (views[1], dviews[1], "v")):
                if n // cf < self.min_seq_len:
                    if out is not None or dst != s0:
                        ops.copy_tokens(view, dview, s0, n, dst)
                else:
                    ops.ccm_mlp(view, dview, self._weights(seg + kind, kv_cache.dtype, kv_cache.device, (l0, l1)), cf,
                                s0, n, dst)
            dst += self._seg_len(n)
        return dst

    @torch.no_grad()
    def forward(self, kv_cache: List[LayerKV], it_len: List[int] = [0, 1]) -> List[LayerKV]:
        """batched_compress.py:442-495."""
        return self._run(kv_cache, it_len, 0, len(kv_cache))

    @torch.no_grad()
    def compress_layers(self, kv_cache: List[LayerKV], layer_start: int, layer_end: int,
                        it_len: List[int] = [0, 1], stream: Optional[torch.cuda.Stream] = None) -> List[LayerKV]:
        """Layers ``[layer_start, layer_end)`` of the full per-layer list ``kv_cache``, optionally on
        ``stream`` (batched_compress.py:501-570); returns only those layers."""
        if layer_end <= layer_start or len(kv_cache) == 0:
            return []
        layer_kv = kv_cache[layer_start:layer_end]
        if len(layer_kv) == 0:
            return []
        if stream is not None:
            with torch.cuda.stream(stream):
                return self._run(layer_kv, it_len, layer_start, layer_start + len(layer_kv))
        return self._run(layer_kv, it_len, layer_start, layer_start + len(layer_kv))
