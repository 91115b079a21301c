"""CCM learned KV-cache compressors with the reference's call surface, computed by the fused HIP MLP.

Mirrors ``KVCacheLinearDecoupleCompressor`` (utils_ccm/module_ccm_v11.py:605-729) and
``KVCacheHybridCompressor`` (:805-1060): same constructor arguments, same parameter names and
creation order (so ``load_state_dict`` of a reference checkpoint and seeded initialisation give the
same weights), same ``forward(kv_cache, it_len)`` contract.  Inference only: the forward pass is the
eval-mode network (dropout is the identity) and does not build an autograd graph.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch
import torch.nn as nn

from .. import _lib, ops

LayerKV = Tuple[torch.Tensor, torch.Tensor]


def _mlp(head_dim: int, cf: int) -> nn.Sequential:
    return nn.Sequential(
        nn.Linear(head_dim * cf, head_dim), nn.ReLU(), nn.Dropout(p=0.4),
        nn.Linear(head_dim, head_dim), nn.ReLU(), nn.Dropout(p=0.4),
        nn.Linear(head_dim, head_dim))


def _mlp_list(n_layer: int, head_dim: int, cf: int) -> nn.ModuleList:
    return nn.ModuleList([_mlp(head_dim, cf) for _ in range(n_layer)])


class CompressibleCache:
    """What ``KVCacheHybridCompressor.forward`` returns for a cache object (the reference's
    ``CompressibleCache``, utils_ccm/module_ccm_v11.py:93-127): per-layer ``key_cache`` / ``value_cache`` lists
    plus the number of tokens the model has SEEN, which after a compression is larger than the rows the cache
    holds and is what ``get_seq_length`` reports (positions go on from there).  A plain object with the list
    attributes and methods the reference's class has; it does not derive from a ``transformers`` cache class,
    whose storage differs between library versions."""

    def __init__(self):
        self.key_cache: List[torch.Tensor] = []
        self.value_cache: List[torch.Tensor] = []
        self._seen_tokens = -1            # < 0: never set, report the rows held

    @property
    def seen_tokens(self) -> int:
        return self._seen_tokens

    def set_seen_tokens(self, seen_tokens: int) -> None:
        self._seen_tokens = int(seen_tokens)

    def get_actual_seq_length(self, layer_idx: int = 0) -> int:
        if layer_idx >= len(self.key_cache) or self.key_cache[layer_idx].numel() == 0:
            return 0
        return self.key_cache[layer_idx].shape[-2]

    def get_seq_length(self, layer_idx: int = 0) -> int:
        return self._seen_tokens if self._seen_tokens >= 0 else self.get_actual_seq_length(layer_idx)

    def __len__(self) -> int:
        return len(self.key_cache)

    def __getitem__(self, layer_idx: int) -> LayerKV:
        return self.key_cache[layer_idx], self.value_cache[layer_idx]

    def clone(self) -> "CompressibleCache":
        other = CompressibleCache()
        other.key_cache = [k.clone().detach() for k in self.key_cache]
        other.value_cache = [v.clone().detach() for v in self.value_cache]
        other._seen_tokens = self._seen_tokens
        return other


class _CCMBase(nn.Module):
    """Shared machinery: stacked weight cache and the segment compressor."""

    n_layer: int
    head_dim: int
    compression_factor: int
    min_seq_len: int

    def __init__(self):
        super().__init__()
        self._stacked = {}

    # -- weights ------------------------------------------------------------------------------
    def _weights(self, group: str, dtype: torch.dtype, device: torch.device):
        """``(w1, b1, w2, b2, w3, b3)`` stacked over layers in nn.Linear layout ``[L, out, in]``, in
        the KV dtype.  Rebuilt when a parameter changed (version counters) or moved."""
        mods: nn.ModuleList = getattr(self, group)
        params = [p for m in mods for p in (m[0].weight, m[0].bias, m[3].weight, m[3].bias, m[6].weight, m[6].bias)]
        key = (dtype, device, tuple(p._version for p in params), tuple(p.data_ptr() for p in params))
        hit = self._stacked.get(group)
        if hit is not None and hit[0] == key:
            return hit[1]
        with torch.no_grad():
            packed = tuple(
                torch.stack([getattr(m[i], name).detach() for m in mods]).to(device=device, dtype=dtype).contiguous()
                for i in (0, 3, 6) for name in ("weight", "bias"))
        self._stacked[group] = (key, packed)
        return packed

    def _apply(self, fn, *a, **kw):  # .cuda() / .half() invalidate the stacked copies
        self._stacked = {}
        return super()._apply(fn, *a, **kw)

    # -- one segment of one layer ---------------------------------------------------------------
    def _segment_len(self, n: int) -> int:
        c = n // self.compression_factor
        return n if c < self.min_seq_len else c + (n - c * self.compression_factor)

    def _compress_into(self, src: torch.Tensor, out: torch.Tensor, layer: int, group: str, seg_start: int,
                       seg_len: int, dst_start: int) -> int:
        """Compress tokens ``[seg_start, seg_start+seg_len)`` of ``src [B,H,S,D]`` into ``out`` starting
        at token ``dst_start``; returns the number of tokens written."""
        cf = self.compression_factor
        if seg_len == 0:
            return 0
        sv, dv = _lib.dense_view(src), _lib.dense_view(out)
        if seg_len // cf < self.min_seq_len:          # too short: passed through unchanged
            ops.copy_tokens(sv, dv, seg_start, seg_len, dst_start)
            return seg_len
        w = self._weights(group, src.dtype, src.device)
        ops.ccm_mlp(sv, dv, tuple(t[layer:layer + 1] for t in w), cf, seg_start, seg_len, dst_start)
        return self._segment_len(seg_len)

    def compress_layer(self, layer_cache: LayerKV, layer_idx: int, compressor_k, compressor_v) -> LayerKV:
        """Reference-compatible helper (module_ccm_v11.py:666-694): compress one whole ``(k, v)`` pair
        with the given pair of module lists (``self.compress_tk`` ...)."""
        k, v = layer_cache
        names = {id(getattr(self, n)): n for n in ("compress_tk", "compress_tv", "compress_ik", "compress_iv")
                 if getattr(self, n, None) is not None}
        gk, gv = names[id(compressor_k)], names[id(compressor_v)]
        S = k.shape[2]
        if S // self.compression_factor < self.min_seq_len:
            return k, v
        C = self._segment_len(S)
        ok = torch.empty((*k.shape[:2], C, k.shape[3]), dtype=k.dtype, device=k.device)
        ov = torch.empty_like(ok)
        self._compress_into(k, ok, layer_idx, gk, 0, S, 0)
        self._compress_into(v, ov, layer_idx, gv, 0, S, 0)
        return ok, ov

    # -- the same computation in place on a paged pool, every layer and sequence per launch ----------
    def _paged_segments(self, seq_len: int, it_len: Sequence[int]):
        """``[(k group, v group, seg_start, seg_len)]`` in token order for this class's split rule."""
        img = min(int(it_len[0]), seq_len)
        return [("compress_ik", "compress_iv", 0, img), ("compress_tk", "compress_tv", img, seq_len - img)]

    def paged_compressed_len(self, seq_len: int, it_len: Sequence[int]) -> int:
        """Length ``paged_forward`` leaves for a sequence of ``seq_len`` tokens."""
        return sum(self._segment_len(n) for _, _, _, n in self._paged_segments(seq_len, it_len))

    @torch.no_grad()
    def paged_forward(self, kv_cache: torch.Tensor, block_tables: torch.Tensor, seq_lens: torch.Tensor,
                      seq_len: int, it_len: Sequence[int], layers: Optional[Tuple[int, int]] = None,
                      out: Optional[torch.Tensor] = None, host_lens: Optional[Sequence[int]] = None):
        """Compress sequences that all hold ``seq_len`` tokens in the pool
        ``kv_cache [2, L, blocks, block_size, Hkv, D]``.  By default in place: the result occupies the
        leading slots of the same block tables (what extract -> forward -> write-back leaves there).
        ``layers=(l0, l1)`` restricts the work to those layers; ``out [2, L, B, Hkv, C, D]`` receives the
        result instead of the pages (which then stay untouched).  Returns the compressed length.

        Sequences of different lengths go through the same launches: ``host_lens`` gives their lengths as
        Python ints (``seq_lens`` holds the same numbers on the device, ``seq_len`` is their maximum) and the
        result is the list of compressed lengths."""
        cf = self.compression_factor
        l0, l1 = layers if layers is not None else (0, kv_cache.shape[1])
        views = [_lib.paged_view(kv_cache[p][l0:l1], block_tables, seq_lens, seq_len) for p in range(2)]
        dviews = views if out is None else [_lib.dense_view(out[p][l0:l1]) for p in range(2)]
        if host_lens is not None and len(set(host_lens)) > 1:
            return self._paged_forward_ragged(views, dviews, list(host_lens), it_len, (l0, l1), kv_cache)
        dst = 0
        for gk, gv, s0, n in self._paged_segments(seq_len, it_len):
            if n == 0:
                continue
            for view, dview, g in ((views[0], dviews[0], gk), (views[1], dviews[1], gv)):
                if n // cf < self.min_seq_len:
                    if out is not None or dst != s0:
                        ops.copy_tokens(view, dview, s0, n, dst)
                else:
                    w = tuple(t[l0:l1] for t in self._weights(g, kv_cache.dtype, kv_cache.device))
                    ops.ccm_mlp(view, dview, w, cf, s0, n, dst)
            dst += self._segment_len(n)
        return dst

    def _paged_forward_ragged(self, views, dviews, lens: List[int], it_len, layer_range, kv_cache) -> List[int]:
        """One launch set for sequences of different lengths: per segment of the class's split rule, the
        sequences' (start, length, destination) go to the device as three small int32 tensors."""
        cf, (l0, l1) = self.compression_factor, layer_range
        dev = kv_cache.device
        per_seq = [self._paged_segments(n, it_len) for n in lens]
        dst = [0] * len(lens)
        for j in range(max(len(p) for p in per_seq)):
            segs = [p[j] if j < len(p) else (p[-1][0], p[-1][1], 0, 0) for p in per_seq]
            gk, gv = segs[0][0], segs[0][1]
            if any((g[0], g[1]) != (gk, gv) for g in segs):
                raise _lib.FastcacheError("sequences of one batch must take the same split rule")
            n_max = max(g[3] for g in segs)
            if n_max == 0:
                continue
            mk = lambda xs: torch.tensor(xs, dtype=torch.int32, device=dev)
            starts, counts, dsts = mk([g[2] for g in segs]), mk([g[3] for g in segs]), mk(dst)
            for view, dview, g in ((views[0], dviews[0], gk), (views[1], dviews[1], gv)):
                w = tuple(t[l0:l1] for t in self._weights(g, kv_cache.dtype, dev))
                ops.ccm_mlp_ragged(view, dview, w, cf, starts, counts, dsts, n_max, self.min_seq_len)
            dst = [d + self._segment_len(g[3]) for d, g in zip(dst, segs)]
        return dst

    def _forward_split(self, kv_cache: Sequence[LayerKV], it_len: Sequence[int], split: bool) -> List[LayerKV]:
        out: List[LayerKV] = []
        for layer, (k, v) in enumerate(kv_cache):
            _lib.require_gpu(k, "kv_cache")
            S = k.shape[2]
            img = min(int(it_len[0]), S) if split else 0
            C = self._segment_len(img) + self._segment_len(S - img)
            ok = torch.empty((k.shape[0], k.shape[1], C, k.shape[3]), dtype=k.dtype, device=k.device)
            ov = torch.empty_like(ok)
            for src, dst, gi, gt in ((k, ok, "compress_ik", "compress_tk"), (v, ov, "compress_iv", "compress_tv")):
                n = self._compress_into(src, dst, layer, gi, 0, img, 0) if img else 0
                self._compress_into(src, dst, layer, gt, img, S - img, n)
            out.append((ok, ov))
        return out


class KVCacheLinearDecoupleCompressor(_CCMBase):
    """Separate image and text MLPs per layer (module_ccm_v11.py:605-729)."""

    def __init__(self, src_config, compression_factor: int = 2, min_seq_len: int = 1):
        super().__init__()
        tc = src_config.text_config
        self.n_layer = tc.num_hidden_layers
        self.nhead = tc.num_key_value_heads
        self.d_model = tc.hidden_size
        self.head_dim = self.d_model // self.nhead
        self.compression_factor = compression_factor
        self.min_seq_len = min_seq_len
        # creation order fixes the seeded initialisation: tk, tv, ik, iv, attention
        self.compress_tk = _mlp_list(self.n_layer, self.head_dim, compression_factor)
        self.compress_tv = _mlp_list(self.n_layer, self.head_dim, compression_factor)
        self.compress_ik = _mlp_list(self.n_layer, self.head_dim, compression_factor)
        self.compress_iv = _mlp_list(self.n_layer, self.head_dim, compression_factor)
        self.attention = nn.ModuleList([nn.Linear(self.head_dim, 1) for _ in range(self.n_layer)])

    @torch.no_grad()
    def forward(self, kv_cache, it_len=[1, 1], strategy_com="retain"):
        """``kv_cache``: list of ``(k, v)`` per layer, each ``[B, H, S, D]`` (views allowed).  Tokens
        ``[0, it_len[0])`` go through the image MLPs, the rest through the text MLPs; returns
        contiguous ``[B, H, C, D]`` pairs (module_ccm_v11.py:697-729)."""
        return self._forward_split(kv_cache, it_len, split=True)


class KVCacheHybridCompressor(_CCMBase):
    """Text-only variant (module_ccm_v11.py:805-1060): ``compress_ik``/``compress_iv`` are ``None``."""

    def __init__(self, src_config, compression_factor: int = 2, min_seq_len: int = 1):
        super().__init__()
        arch = getattr(src_config, "architectures", None) or [None]
        if type(src_config).__name__ == "LlamaConfig":
            cfg, head_dim = src_config, src_config.head_dim
        elif arch[0] == "MiniCPMV":
            cfg, head_dim = src_config, src_config.hidden_size // src_config.num_attention_heads
        else:
            cfg, head_dim = src_config.text_config, src_config.text_config.head_dim
        self.n_layer = cfg.num_hidden_layers
        self.nhead = cfg.num_key_value_heads
        self.d_model = cfg.hidden_size
        self.head_dim = head_dim
        self.compression_factor = compression_factor
        self.min_seq_len = min_seq_len
        self.compress_tk = _mlp_list(self.n_layer, self.head_dim, compression_factor)
        self.compress_tv = _mlp_list(self.n_layer, self.head_dim, compression_factor)
        self.compress_ik = None
        self.compress_iv = None

    @torch.no_grad()
    def forward(self, kv_cache, it_len=[1, 1], strategy_com="retain", forward_mode="val"):
        """List input -> list output.  An object with ``key_cache`` / ``value_cache`` lists (an HF cache) is left
        as it is and a new ``CompressibleCache`` comes back, holding the compressed layers and, as its seen-token
        count, the input's ``get_seq_length()`` (module_ccm_v11.py:932-999).  ``it_len[0]`` must be 0: with an
        image segment long enough to be compressed the reference subscripts ``None`` (:877-878, 1033-1035) and
        raises ``TypeError``; so does this class."""
        if forward_mode == "train":
            raise NotImplementedError("inference-only build: forward_mode='train' is not supported")
        as_cache = hasattr(kv_cache, "key_cache") and hasattr(kv_cache, "value_cache")
        layers = list(zip(kv_cache.key_cache, kv_cache.value_cache)) if as_cache else \
            [kv_cache[i] for i in range(self.n_layer)]
        if it_len[0] != 0:
            img = min(int(it_len[0]), layers[0][0].shape[2])
            if img // self.compression_factor >= self.min_seq_len:
                raise TypeError("'NoneType' object is not subscriptable")
        out = self._forward_split(layers, [0, 0], split=False) if it_len[0] == 0 else \
            self._forward_passthrough_image(layers, int(it_len[0]))
        if as_cache:
            fresh = CompressibleCache()
            fresh.key_cache = [k for k, _ in out]
            fresh.value_cache = [v for _, v in out]
            seen = kv_cache.get_seq_length() if hasattr(kv_cache, "get_seq_length") else layers[0][0].shape[2]
            fresh.set_seen_tokens(seen)
            return fresh
        return out

    def _paged_segments(self, seq_len: int, it_len: Sequence[int]):
        if it_len[0] == 0:
            return [("compress_tk", "compress_tv", 0, seq_len)]
        img = min(int(it_len[0]), seq_len)
        if img // self.compression_factor >= self.min_seq_len:
            raise TypeError("'NoneType' object is not subscriptable")
        # an image segment too short to compress is passed through; min_seq_len guard of compress_layer
        return [("compress_tk", "compress_tv", 0, img), ("compress_tk", "compress_tv", img, seq_len - img)]

    def _forward_passthrough_image(self, layers, img):
        out = []
        for layer, (k, v) in enumerate(layers):
            S = k.shape[2]
            img_l = min(img, S)
            C = img_l + self._segment_len(S - img_l)
            ok = torch.empty((k.shape[0], k.shape[1], C, k.shape[3]), dtype=k.dtype, device=k.device)
            ov = torch.empty_like(ok)
            for src, dst, g in ((k, ok, "compress_tk"), (v, ov, "compress_tv")):
                ops.copy_tokens(_lib.dense_view(src), _lib.dense_view(dst), 0, img_l, 0)
                self._compress_into(src, dst, layer, g, img_l, S - img_l, img_l)
            out.append((ok, ov))
        return out
