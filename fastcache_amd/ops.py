"""Functional layer over the C ABI: torch tensors in, torch tensors out.

torch is used only for device memory and the current HIP stream; every computation is a call
into libfastcache_hip.so.  All functions enqueue on ``torch.cuda.current_stream()`` and return
without synchronising.
"""
from __future__ import annotations

import ctypes as C
import math
from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import FastcacheError, FcKvView, FcMlpWeights, check, current_stream, fn, ptr


def _i32(t: Optional[torch.Tensor], name: str, device) -> Optional[torch.Tensor]:
    if t is None:
        return None
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise FastcacheError(f"{name} must be a contiguous int32 tensor")
    if t.device != device:
        raise FastcacheError(f"{name} is on {t.device}, expected {device}")
    return t


# ---------------------------------------------------------------------------------------------
# scoring
# ---------------------------------------------------------------------------------------------
def knorm_score(keys: FcKvView, device, score_stride: Optional[int] = None) -> torch.Tensor:
    """``-||k||_2`` per (layer, sequence, kv head, token) -> fp32 ``[L, B, Hkv, stride]``."""
    stride = keys.max_seq_len if score_stride is None else score_stride
    out = torch.empty((keys.num_layers, keys.batch, keys.num_kv_heads, stride), dtype=torch.float32, device=device)
    check(fn("fc_knorm_score")(C.byref(keys), out.data_ptr(), stride, current_stream()), "fc_knorm_score")
    return out


def knorm_mean_score(keys: FcKvView, device, score_stride: Optional[int] = None) -> torch.Tensor:
    """Head-averaged key norm per (layer, sequence, token) -> fp32 ``[L, B, stride]``."""
    stride = keys.max_seq_len if score_stride is None else score_stride
    out = torch.empty((keys.num_layers, keys.batch, stride), dtype=torch.float32, device=device)
    check(fn("fc_knorm_mean_score")(C.byref(keys), out.data_ptr(), stride, current_stream()),
          "fc_knorm_mean_score")
    return out


def key_channel_energy(keys: FcKvView, device) -> torch.Tensor:
    """Sum over each sequence's tokens of ``k^2`` per head-dimension channel -> fp32 ``[L, B, Hkv, 128]``."""
    out = torch.empty((keys.num_layers, keys.batch, keys.num_kv_heads, keys.head_dim), dtype=torch.float32, device=device)
    check(fn("fc_key_channel_energy")(C.byref(keys), out.data_ptr(), current_stream()), "fc_key_channel_energy")
    return out


def key_channel_zero(keys: FcKvView, prune: torch.Tensor) -> None:
    """Zero, in place and for every token, the channels with ``prune[l, b, h, d] != 0`` (uint8 ``[L, B, Hkv, 128]``)."""
    _lib.require_gpu(prune, "prune")
    want = (keys.num_layers, keys.batch, keys.num_kv_heads, keys.head_dim)
    if prune.dtype != torch.uint8 or tuple(prune.shape) != want:
        raise FastcacheError(f"key_channel_zero: prune must be uint8 {want}, got {prune.dtype} {tuple(prune.shape)}")
    pc = prune.contiguous()
    check(fn("fc_key_channel_zero")(C.byref(keys), pc.data_ptr(), current_stream()), "fc_key_channel_zero")


def snapkv_splits(keys: FcKvView, num_q_heads: int, window: int) -> int:
    """Key ranges per column for :func:`snapkv_score`.  Measured on MI355X (window 64, group of 4-7 heads;
    ``python -m fastcache_amd.crossovers splits``, figures in profiles/launch_shape_crossovers.txt): with
    1000 or more (layer, sequence, kv head) columns one workgroup per column is fastest; below that the GPU is not
    filled and cutting the columns pays: 576 columns -13 % with 4 pieces, 288 columns -26 % with 8, 112 columns -39 %.
    A piece keeps at least 8 key tiles of 64.  1 also when the split kernels do not apply (more than 16 query row
    blocks per kv head, pages that are no multiple of 64 tokens)."""
    columns = keys.num_layers * keys.batch * keys.num_kv_heads
    blocks = (num_q_heads // keys.num_kv_heads) * ((window + 31) // 32)
    tiles = (keys.max_seq_len + 63) // 64
    paged_ok = not keys.block_tables or (keys.block_size >= 64 and keys.block_size & (keys.block_size - 1) == 0
                                         and (keys.max_seq_len - 1) // keys.block_size < 1024)
    if columns >= 1000 or blocks > 16 or not paged_ok:
        return 1
    return max(1, min(8, -(-2304 // columns), tiles // 8))


def snapkv_score(keys: FcKvView, queries: torch.Tensor, window: int, kernel_size: int,
                 causal_window: bool = True, reduction: str = "mean", scale: Optional[float] = None,
                 seq_lens: Optional[torch.Tensor] = None, score_stride: Optional[int] = None,
                 lse: Optional[torch.Tensor] = None, splits: Optional[int] = None) -> torch.Tensor:
    """SnapKV observation-window scores -> fp32 ``[L, B, Hkv, stride]`` with the window positions
    set to the per-layer maximum.  queries ``[L, B, Hq, W, D]`` (or ``[B, Hq, W, D]`` for one layer).
    ``lse`` (optional, fp32 ``[L, B, Hq, W]``): natural-log sum of ``exp(scale * q.k)`` over the keys each window
    query sees, as the prefill's attention kernel returns it; with it the keys are read once instead of twice.
    ``splits``: key ranges per (layer, sequence, kv head) column, one workgroup each; default: chosen by
    :func:`snapkv_splits` so that a launch with few columns still fills the GPU."""
    if queries.dim() == 4:
        queries = queries.unsqueeze(0)
        if lse is not None and lse.dim() == 3:
            lse = lse.unsqueeze(0)
    if not queries.is_contiguous():
        queries = queries.contiguous()
    _lib.require_gpu(queries, "queries")
    L, B, Hq, W, D = queries.shape
    if (L, B) != (keys.num_layers, keys.batch) or W != window or D != keys.head_dim:
        raise FastcacheError(f"queries {tuple(queries.shape)} do not match the key view "
                             f"(L={keys.num_layers}, B={keys.batch}, W={window}, D={keys.head_dim})")
    if _lib.dtype_code(queries.dtype) != keys.dtype:
        raise FastcacheError("queries and keys must share a dtype")
    if Hq % keys.num_kv_heads:
        raise FastcacheError("num_q_heads must be a multiple of num_kv_heads")
    G = Hq // keys.num_kv_heads
    if reduction not in ("mean", "sum"):
        raise ValueError("reduction must be 'mean' or 'sum'")
    out_scale = 1.0 / (W * G) if reduction == "mean" else 1.0
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    stride = keys.max_seq_len if score_stride is None else score_stride
    dev = queries.device
    out = torch.empty((L, B, keys.num_kv_heads, stride), dtype=torch.float32, device=dev)
    st = current_stream()
    row_max = torch.empty((L, B, keys.num_kv_heads), dtype=torch.float32, device=dev)
    if lse is not None:
        _lib.require_gpu(lse, "lse")
        if lse.dtype != torch.float32 or tuple(lse.shape) != (L, B, Hq, W):
            raise FastcacheError(f"lse must be fp32 [L={L}, B={B}, Hq={Hq}, W={W}], got {lse.dtype} {tuple(lse.shape)}")
        lse = lse.contiguous()
    nsplit = snapkv_splits(keys, Hq, W) if splits is None else int(splits)
    if nsplit > 1:
        nbytes = int(fn("fc_snapkv_split_workspace_bytes")(L, B, Hq, keys.num_kv_heads, W, stride, nsplit))
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        check(fn("fc_snapkv_score_split")(C.byref(keys), queries.data_ptr(), ptr(lse), Hq, window, kernel_size,
                                          int(causal_window), scale, out_scale, out.data_ptr(), stride,
                                          row_max.data_ptr(), nsplit, ws.data_ptr(), nbytes, st), "fc_snapkv_score_split")
    elif lse is None:
        check(fn("fc_snapkv_score")(C.byref(keys), queries.data_ptr(), Hq, window, kernel_size,
                                    int(causal_window), scale, out_scale, out.data_ptr(), stride, row_max.data_ptr(),
                                    st), "fc_snapkv_score")
    else:
        check(fn("fc_snapkv_score_lse")(C.byref(keys), queries.data_ptr(), lse.data_ptr(), Hq, window, kernel_size,
                                        int(causal_window), scale, out_scale, out.data_ptr(), stride,
                                        row_max.data_ptr(), st), "fc_snapkv_score_lse")
    check(fn("fc_snapkv_fill_window")(out.data_ptr(), stride, L, B, keys.num_kv_heads, ptr(seq_lens),
                                      keys.max_seq_len, window, row_max.data_ptr(), st), "fc_snapkv_fill_window")
    return out


def snapkv_press_fits(keys: FcKvView, num_q_heads: int, window: int, index_stride: int) -> bool:
    """Whether :func:`snapkv_press` takes this shape (otherwise: ``snapkv_score`` + ``select_compact``): at most 16
    blocks of 32 window queries per kv head, pages of 64*2^n tokens or a dense view, and
    the score row plus the kept positions inside the LDS of the key tiles."""
    if num_q_heads % keys.num_kv_heads:
        return False
    blocks = (num_q_heads // keys.num_kv_heads) * ((window + 31) // 32)
    if blocks > 16:
        return False
    waves = 4 if blocks <= 4 else (8 if blocks <= 8 else 16)
    tiles = 4 if waves >= 8 else 3
    room = tiles * 64 * 256 + (4 * waves + 4) * 64 * 4
    paged_ok = (not keys.block_tables) or (keys.block_size >= 64 and keys.block_size & (keys.block_size - 1) == 0
                                           and (keys.max_seq_len - 1) // keys.block_size < 1024)
    return bool(paged_ok and 4 * (keys.max_seq_len + index_stride) + 12288 <= room and
                0 <= keys.stride_token < (1 << 24))


def snapkv_press_preferred(keys: FcKvView, num_q_heads: int, window: int, compute_units: int = 256) -> bool:
    """Whether the one-launch press (whole columns) or split scoring (:func:`snapkv_splits` key ranges per column, then
    ``select_compact``) is the faster form for a shape both take.  Whole columns cost ``rounds x column time`` with
    ``rounds = ceil(columns / workgroups the GPU holds)`` (two per compute unit, one with 16 wavefronts), split scoring
    grows linearly with the columns but pays a merge, a pooling and a compaction launch.  Measured on MI355X (28 x B x 4
    and 36 x B x 8 columns of 4096 to 12000 keys; ``python -m fastcache_amd.crossovers press``, figures in
    profiles/launch_shape_crossovers.txt): whole columns win or tie when the last round is at least 80 % full
    or the columns are short (up to 4096 keys: 0.64 against 0.72 ms at 448 columns, 0.92 against 1.01 at 672, at worst
    2.5 % behind); long columns in poorly filled rounds lose (320 x 12000: 1.64 against 1.37 ms)."""
    if snapkv_splits(keys, num_q_heads, window) == 1:
        return True
    columns = keys.num_layers * keys.batch * keys.num_kv_heads
    blocks = (num_q_heads // keys.num_kv_heads) * ((window + 31) // 32)
    slots = compute_units * (2 if blocks <= 8 else 1)
    rounds = -(-columns // slots)
    return keys.max_seq_len <= 4096 or columns >= 0.8 * rounds * slots


def snapkv_press(keys: FcKvView, values: FcKvView, queries: torch.Tensor, window: int, kernel_size: int, k: int,
                 causal_window: bool = True, reduction: str = "mean", scale: Optional[float] = None,
                 seq_lens: Optional[torch.Tensor] = None, lse: Optional[torch.Tensor] = None,
                 n_kept=None, ragged: bool = False, host_lens=None):
    """SnapKV scores, selection (the window always kept; ``k`` or ``n_kept[b]`` positions per row, window included,
    more than the window) and in-place compaction of both planes, each (layer, sequence, kv head) column by one
    workgroup in one launch; then the window fill of the scores.  Returns ``(scores, indices)`` equal to
    ``snapkv_score`` + ``select_compact``.  Shapes must satisfy :func:`snapkv_press_fits`.

    ``n_kept``: the kept counts per sequence as Python ints (checked here: the kernel leaves a sequence longer than the
    window untouched when its count does not exceed the window, which a caller that then shortens the sequence
    would not notice; ``host_lens`` names the sequences no longer than the window, which are exempt).  A device
    tensor is passed through unchecked for callers that have validated the counts themselves."""
    if n_kept is not None and not isinstance(n_kept, torch.Tensor):
        counts = [int(c) for c in n_kept]
        lens_h = list(host_lens) if host_lens is not None else [keys.max_seq_len] * len(counts)
        bad = [b for b, (c, n) in enumerate(zip(counts, lens_h)) if n > window and not window < c <= min(k, n)]
        if len(counts) != keys.batch or bad:
            raise FastcacheError(f"snapkv_press: kept counts must exceed the window ({window}) and fit the index row "
                                 f"({k}) for every sequence longer than the window; offending sequences: {bad}")
        n_kept = torch.tensor(counts, dtype=torch.int32, device=queries.device)
    if queries.dim() == 4:
        queries = queries.unsqueeze(0)
        if lse is not None and lse.dim() == 3:
            lse = lse.unsqueeze(0)
    if not queries.is_contiguous():
        queries = queries.contiguous()
    _lib.require_gpu(queries, "queries")
    L, B, Hq, W, D = queries.shape
    H = keys.num_kv_heads
    if (L, B) != (keys.num_layers, keys.batch) or W != window or D != keys.head_dim:
        raise FastcacheError(f"queries {tuple(queries.shape)} do not match the key view "
                             f"(L={keys.num_layers}, B={keys.batch}, W={window}, D={keys.head_dim})")
    if _lib.dtype_code(queries.dtype) != keys.dtype:
        raise FastcacheError("queries and keys must share a dtype")
    if reduction not in ("mean", "sum"):
        raise ValueError("reduction must be 'mean' or 'sum'")
    out_scale = 1.0 / (W * (Hq // H)) if reduction == "mean" else 1.0
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    dev = queries.device
    stride = keys.max_seq_len
    scores = torch.empty((L, B, H, stride), dtype=torch.float32, device=dev)
    row_max = torch.empty((L, B, H), dtype=torch.float32, device=dev)
    n_kept = _i32(n_kept, "n_kept", dev)
    if n_kept is not None or ragged:
        idx = torch.full((L, B, H, k), -1, dtype=torch.int32, device=dev)
    else:
        idx = torch.empty((L, B, H, k), dtype=torch.int32, device=dev)
    if lse is not None:
        _lib.require_gpu(lse, "lse")
        if lse.dtype != torch.float32 or tuple(lse.shape) != (L, B, Hq, W):
            raise FastcacheError(f"lse must be fp32 [L={L}, B={B}, Hq={Hq}, W={W}], got {lse.dtype} {tuple(lse.shape)}")
        lse = lse.contiguous()
    st = current_stream()
    check(fn("fc_snapkv_press")(C.byref(keys), C.byref(values), queries.data_ptr(), ptr(lse), Hq, window, kernel_size,
                                int(causal_window), scale, out_scale, scores.data_ptr(), stride, row_max.data_ptr(), k,
                                ptr(n_kept), idx.data_ptr(), k, st), "fc_snapkv_press")
    check(fn("fc_snapkv_fill_window")(scores.data_ptr(), stride, L, B, H, ptr(seq_lens), keys.max_seq_len, window,
                                      row_max.data_ptr(), st), "fc_snapkv_fill_window")
    return scores, idx


# ---------------------------------------------------------------------------------------------
# selection and compaction
# ---------------------------------------------------------------------------------------------
def topk_select(scores: torch.Tensor, k: int, row_lens: Optional[torch.Tensor] = None,
                n_kept: Optional[torch.Tensor] = None, rows_per_len: int = 1) -> torch.Tensor:
    """Indices of the ``k`` largest entries per row of ``scores[..., S]`` (fp32): ties to the lowest
    index, output ascending, int32 ``[..., k]``.  With ``row_lens``/``n_kept`` (int32 ``[B]``) rows
    ordered (..., b, head) take their valid length and kept count from entry ``b``
    (``rows_per_len`` = heads per b); entries past a row's kept count (or valid length) are -1."""
    _lib.require_gpu(scores, "scores")
    if scores.dtype != torch.float32 or scores.stride(-1) != 1:
        raise FastcacheError("scores must be fp32 with a contiguous last axis")
    S = scores.shape[-1]
    flat = scores.reshape(-1, S) if scores.is_contiguous() else None
    if flat is None:
        # rows must be equally spaced: allow a narrowed last axis of a contiguous buffer
        lead = scores.shape[:-1]
        stride = scores.stride(-2) if scores.dim() > 1 else S
        expect = [stride]
        for n in reversed(lead[1:]):
            expect.append(expect[-1] * n)
        if list(scores.stride()[:-1]) != list(reversed(expect)):
            raise FastcacheError("scores rows must be equally spaced in memory")
        rows, score_stride = math.prod(lead), stride
    else:
        rows, score_stride = flat.shape[0], S
    dev = scores.device
    row_lens = _i32(row_lens, "row_lens", dev)
    n_kept = _i32(n_kept, "n_kept", dev)
    per_row = row_lens is not None or n_kept is not None
    mod = (row_lens if row_lens is not None else n_kept).numel() if per_row else 1
    if per_row:
        out = torch.full((*scores.shape[:-1], k), -1, dtype=torch.int32, device=dev)
    else:
        out = torch.empty((*scores.shape[:-1], k), dtype=torch.int32, device=dev)
    check(fn("fc_topk_select")(scores.data_ptr(), score_stride, rows, S, ptr(row_lens), rows_per_len, mod, k,
                               ptr(n_kept), out.data_ptr(), k, current_stream()), "fc_topk_select")
    return out


def compact(src_k: FcKvView, src_v: FcKvView, dst_k: FcKvView, dst_v: FcKvView, indices: torch.Tensor,
            k: Optional[int] = None, n_kept: Optional[torch.Tensor] = None) -> None:
    """dst token j <- src token indices[l, b, h, j]; indices int32 ``[L, B, Hkv or 1, stride]``."""
    if indices.dtype != torch.int32 or indices.dim() != 4 or not indices.is_contiguous():
        raise FastcacheError("indices must be a contiguous int32 [L, B, heads, k] tensor")
    _lib.require_gpu(indices, "indices")
    L, B, Hi, stride = indices.shape
    if (L, B) != (src_k.num_layers, src_k.batch):
        raise FastcacheError("indices do not match the views' layers/batch")
    n_kept = _i32(n_kept, "n_kept", indices.device)
    check(fn("fc_compact")(C.byref(src_k), C.byref(src_v), C.byref(dst_k), C.byref(dst_v), indices.data_ptr(),
                           stride, Hi, stride if k is None else k, ptr(n_kept), current_stream()),
          "fc_compact")


def press_column_fits(max_seq_len: int, k: int) -> bool:
    """Whether :func:`knorm_press` / :func:`select_compact` take sequences of ``max_seq_len`` tokens keeping ``k``: a
    column's scores and kept positions stay in LDS, ``4 * (max_seq_len + k)`` bytes of at most 144 KB."""
    return 4 * (max_seq_len + k) <= 144 * 1024


def knorm_press(keys: FcKvView, values: FcKvView, k: int, device, n_kept: Optional[torch.Tensor] = None,
                ragged: bool = False):
    """Knorm scores, top-``k`` (or ``n_kept[b]``) per (layer, sequence, kv head) row and in-place compaction of
    both planes in one launch; returns ``(scores [L, B, Hkv, max_seq_len] fp32, indices [L, B, Hkv, k] int32)`` equal
    to ``knorm_score`` + ``topk_select`` + ``compact``.  With ``n_kept`` or ``ragged`` (sequences that may hold fewer
    than ``k`` tokens) index entries past a row's kept count are -1."""
    L, B, H, S = keys.num_layers, keys.batch, keys.num_kv_heads, keys.max_seq_len
    scores = torch.empty((L, B, H, S), dtype=torch.float32, device=device)
    n_kept = _i32(n_kept, "n_kept", device)
    if n_kept is not None or ragged:
        idx = torch.full((L, B, H, k), -1, dtype=torch.int32, device=device)
    else:
        idx = torch.empty((L, B, H, k), dtype=torch.int32, device=device)
    check(fn("fc_knorm_press")(C.byref(keys), C.byref(values), scores.data_ptr(), S, k, ptr(n_kept), idx.data_ptr(), k,
                               current_stream()), "fc_knorm_press")
    return scores, idx


def select_compact(keys: FcKvView, values: FcKvView, scores: torch.Tensor, k: int,
                   n_kept: Optional[torch.Tensor] = None, ragged: bool = False) -> torch.Tensor:
    """``topk_select`` over each sequence's own length and ``compact`` of both planes onto themselves in one launch;
    ``scores`` fp32 ``[L, B, Hkv, stride]`` contiguous.  Returns the indices ``[L, B, Hkv, k]`` (-1 past a row's kept
    count with ``n_kept`` or ``ragged``)."""
    _lib.require_gpu(scores, "scores")
    L, B, H = keys.num_layers, keys.batch, keys.num_kv_heads
    if scores.dtype != torch.float32 or scores.dim() != 4 or tuple(scores.shape[:3]) != (L, B, H) or \
            not scores.is_contiguous():
        raise FastcacheError("scores must be a contiguous fp32 [L, B, Hkv, stride] tensor matching the views")
    n_kept = _i32(n_kept, "n_kept", scores.device)
    if n_kept is not None or ragged:
        idx = torch.full((L, B, H, k), -1, dtype=torch.int32, device=scores.device)
    else:
        idx = torch.empty((L, B, H, k), dtype=torch.int32, device=scores.device)
    check(fn("fc_select_compact")(C.byref(keys), C.byref(values), scores.data_ptr(), scores.shape[3], k, ptr(n_kept),
                                  idx.data_ptr(), k, current_stream()), "fc_select_compact")
    return idx


def copy_tokens(src: FcKvView, dst: FcKvView, seg_start: int, count: int, dst_start: int) -> None:
    check(fn("fc_copy_tokens")(C.byref(src), C.byref(dst), seg_start, count, dst_start, current_stream()),
          "fc_copy_tokens")


def copy_tokens_from_layers(layers, dst: FcKvView, count: int, dst_start: int = 0) -> bool:
    """Tokens ``[0, count)`` of a list of per-layer tensors ``[B, Hkv, C, D]`` (one per layer of ``dst``, all of one
    shape, dtype and stride pattern) -> ``dst`` tokens ``[dst_start, dst_start + count)``, in one launch and without
    stacking the list.  Returns False (nothing done) when the tensors do not share one geometry."""
    first = layers[0]
    if len(layers) != dst.num_layers or any(t.shape != first.shape or t.stride() != first.stride() or t.dtype != first.dtype
                                            or t.device != first.device for t in layers):
        return False
    _lib.require_gpu(first, "layer tensor")
    view = _lib.dense_view(first)
    view.num_layers = len(layers)
    table = torch.tensor([t.data_ptr() for t in layers], dtype=torch.int64, pin_memory=True).to(first.device,
                                                                                                 non_blocking=True)
    check(fn("fc_copy_tokens_from_layers")(table.data_ptr(), C.byref(view), C.byref(dst), 0, count, dst_start,
                                           current_stream()), "fc_copy_tokens_from_layers")
    return True


# ---------------------------------------------------------------------------------------------
# CCM MLP
# ---------------------------------------------------------------------------------------------
def ccm_mlp(src: FcKvView, dst: FcKvView, weights: Tuple[torch.Tensor, ...], cf: int, seg_start: int,
            seg_len: int, dst_start: int) -> None:
    """weights = (w1 [L,128,cf*128], b1 [L,128], w2 [L,128,128], b2, w3, b3) in the KV dtype."""
    w1, b1, w2, b2, w3, b3 = weights
    L = src.num_layers
    D = src.head_dim
    shapes = [(L, D, cf * D), (L, D), (L, D, D), (L, D), (L, D, D), (L, D)]
    for t, shp, name in zip(weights, shapes, ("w1", "b1", "w2", "b2", "w3", "b3")):
        _lib.require_gpu(t, name)
        if tuple(t.shape) != shp or not t.is_contiguous() or _lib.dtype_code(t.dtype) != src.dtype:
            raise FastcacheError(f"{name} must be contiguous {shp} in the KV dtype, got {tuple(t.shape)} {t.dtype}")
    w = FcMlpWeights(*(t.data_ptr() for t in weights))
    check(fn("fc_ccm_mlp")(C.byref(src), C.byref(dst), C.byref(w), cf, seg_start, seg_len, dst_start,
                           current_stream()), "fc_ccm_mlp")


def ccm_mlp_ragged(src: FcKvView, dst: FcKvView, weights: Tuple[torch.Tensor, ...], cf: int,
                   seg_start: torch.Tensor, seg_len: torch.Tensor, dst_start: torch.Tensor, max_seg_len: int,
                   min_rows: int) -> None:
    """``ccm_mlp`` with one segment per sequence: int32 device tensors ``[B]``; a sequence whose segment has fewer
    than ``min_rows * cf`` tokens is copied through; ``max_seg_len`` bounds ``seg_len``."""
    L, D = src.num_layers, src.head_dim
    shapes = [(L, D, cf * D), (L, D), (L, D, D), (L, D), (L, D, D), (L, D)]
    for t, shp, name in zip(weights, shapes, ("w1", "b1", "w2", "b2", "w3", "b3")):
        _lib.require_gpu(t, name)
        if tuple(t.shape) != shp or not t.is_contiguous() or _lib.dtype_code(t.dtype) != src.dtype:
            raise FastcacheError(f"{name} must be contiguous {shp} in the KV dtype, got {tuple(t.shape)} {t.dtype}")
    dev = weights[0].device
    arrays = []
    for t, name in ((seg_start, "seg_start"), (seg_len, "seg_len"), (dst_start, "dst_start")):
        t = _i32(t, name, dev)
        if t.numel() != src.batch:
            raise FastcacheError(f"{name} must hold one entry per sequence ({src.batch}), got {t.numel()}")
        arrays.append(t)
    w = FcMlpWeights(*(t.data_ptr() for t in weights))
    check(fn("fc_ccm_mlp_ragged")(C.byref(src), C.byref(dst), C.byref(w), cf, arrays[0].data_ptr(),
                                  arrays[1].data_ptr(), arrays[2].data_ptr(), max_seg_len, min_rows,
                                  current_stream()), "fc_ccm_mlp_ragged")


def expected_attention_score(keys: FcKvView, values: FcKvView, mean_query: torch.Tensor,
                             cov_query: Optional[torch.Tensor], n_sink: int = 4, use_vnorm: bool = True,
                             epsilon: float = 0.0, score_stride: Optional[int] = None) -> torch.Tensor:
    """Expected attention of future queries ~ N(mean_query, cov_query) over the cached keys, scaled by the value
    norms: ``[L, B, Hkv, score_stride]`` fp32.  mean_query ``[L, B, Hq, D]`` (or ``[B, Hq, D]`` for one layer),
    cov_query ``[L, B, Hq, D, D]`` or None; both are converted to contiguous fp32."""
    _lib.require_gpu(mean_query, "mean_query")
    L, B, Hkv, S = keys.num_layers, keys.batch, keys.num_kv_heads, keys.max_seq_len
    mu = mean_query.float().contiguous()
    if mu.dim() == 3:
        mu = mu.unsqueeze(0)
    if mu.dim() != 4 or mu.shape[0] != L or mu.shape[1] != B or mu.shape[3] != keys.head_dim:
        raise FastcacheError(f"mean_query must be [L={L}, B={B}, Hq, {keys.head_dim}], got {tuple(mean_query.shape)}")
    Hq = mu.shape[2]
    cov = None
    if cov_query is not None:
        cov = cov_query.float().contiguous()
        if cov.dim() == 4:
            cov = cov.unsqueeze(0)
        if tuple(cov.shape) != (L, B, Hq, keys.head_dim, keys.head_dim):
            raise FastcacheError(f"cov_query must be [L, B, Hq, D, D], got {tuple(cov_query.shape)}")
    stride = S if score_stride is None else int(score_stride)
    out = torch.empty((L, B, Hkv, stride), dtype=torch.float32, device=mu.device)
    nbytes = int(fn("fc_expected_attention_workspace_bytes")(L, B, Hq, S))
    if nbytes < 0:
        raise FastcacheError("fc_expected_attention_workspace_bytes: bad arguments")
    ws = torch.empty(nbytes, dtype=torch.uint8, device=mu.device)
    check(fn("fc_expected_attention_score")(C.byref(keys), C.byref(values), mu.data_ptr(), _lib.ptr(cov), Hq,
                                            int(n_sink), int(bool(use_vnorm)), float(epsilon), out.data_ptr(), stride,
                                            ws.data_ptr(), nbytes, current_stream()), "fc_expected_attention_score")
    return out


def observed_attention_score(attentions: torch.Tensor, num_kv_heads: int) -> torch.Tensor:
    """fp32 ``[B, Hkv, Sk]`` from a materialised attention matrix ``[B, Hq, Sq, Sk]``: per key, the attention it
    received summed over the queries, divided by the number of queries that could see it, averaged over the group."""
    _lib.require_gpu(attentions, "attentions")
    if attentions.dim() != 4:
        raise FastcacheError(f"attentions must be [B, Hq, Sq, Sk], got {tuple(attentions.shape)}")
    a = attentions.contiguous()
    B, Hq, Sq, Sk = a.shape
    out = torch.empty((B, num_kv_heads, Sk), dtype=torch.float32, device=a.device)
    nbytes = fn("fc_observed_attention_workspace_bytes")(B, num_kv_heads, Sk)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=a.device)
    check(fn("fc_observed_attention_score")(a.data_ptr(), B, Hq, num_kv_heads, Sq, Sk, _lib.dtype_code(a.dtype),
                                            out.data_ptr(), ws.data_ptr(), nbytes, current_stream()),
          "fc_observed_attention_score")
    return out


def quantize_rows(x: torch.Tensor, bits: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-row (last dimension) symmetric quantisation: ``(q int8 like x, scale x.dtype [..., 1])``."""
    _lib.require_gpu(x, "x")
    if x.dim() < 1 or x.numel() == 0:
        raise FastcacheError("quantize_rows: empty input")
    xc = x.contiguous()
    d = xc.shape[-1]
    rows = xc.numel() // d
    q = torch.empty(xc.shape, dtype=torch.int8, device=x.device)
    scale = torch.empty(xc.shape[:-1] + (1,), dtype=x.dtype, device=x.device)
    check(fn("fc_quantize_rows")(xc.data_ptr(), rows, d, _lib.dtype_code(x.dtype), bits, q.data_ptr(),
                                 scale.data_ptr(), current_stream()), "fc_quantize_rows")
    return q, scale


def dequantize_rows(q: torch.Tensor, scale: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """``q.to(dtype) * scale`` with the dtype promotion of that expression."""
    _lib.require_gpu(q, "q")
    _lib.require_gpu(scale, "scale")
    if q.dtype != torch.int8:
        raise FastcacheError(f"dequantize_rows: int8 codes expected, got {q.dtype}")
    d = q.shape[-1]
    rows = q.numel() // d
    if scale.numel() != rows:
        raise FastcacheError("dequantize_rows: one scale per row expected")
    out_dtype = torch.promote_types(dtype, scale.dtype)
    qc, sc = q.contiguous(), scale.contiguous()
    out = torch.empty(qc.shape, dtype=out_dtype, device=q.device)
    check(fn("fc_dequantize_rows")(qc.data_ptr(), sc.data_ptr(), rows, d, _lib.dtype_code(sc.dtype),
                                   _lib.dtype_code(out_dtype), out.data_ptr(), current_stream()), "fc_dequantize_rows")
    return out


def fake_quantize(x: torch.Tensor, bits: int, per_tensor: bool, out: Optional[torch.Tensor] = None,
                  return_params: bool = False):
    """Quantise and dequantise in one pass: ``clamp(round(x / scale), -2^(bits-1), 2^(bits-1)-1) * scale`` with
    ``scale = max|x| / (2^(bits-1)-1)`` over the last dimension, or over the whole tensor when ``per_tensor``.
    With ``return_params`` also ``(scale, max|x|)`` shaped ``[..., 1]`` (or 0-dim for the whole-tensor form)."""
    _lib.require_gpu(x, "x")
    if x.dim() < 1 or x.numel() == 0:
        raise FastcacheError("fake_quantize: empty input")
    xc = x.contiguous()
    d = xc.shape[-1]
    rows = xc.numel() // d
    y = torch.empty_like(xc) if out is None else out
    if y.shape != xc.shape or y.dtype != xc.dtype or not y.is_contiguous():
        raise FastcacheError("fake_quantize: out must be contiguous with the shape and dtype of x")
    pshape = () if per_tensor else xc.shape[:-1] + (1,)
    scale = torch.empty(pshape, dtype=x.dtype, device=x.device) if return_params else None
    amax = torch.empty(pshape, dtype=x.dtype, device=x.device) if return_params else None
    ws, nbytes = None, 0
    if per_tensor:
        nbytes = int(fn("fc_fake_quantize_workspace_bytes")())
        ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    check(fn("fc_fake_quantize")(xc.data_ptr(), y.data_ptr(), rows, d, _lib.dtype_code(x.dtype), bits,
                                 int(bool(per_tensor)), _lib.ptr(scale), _lib.ptr(amax), _lib.ptr(ws), nbytes,
                                 current_stream()), "fc_fake_quantize")
    return (y, scale, amax) if return_params else y


def quantize_rows_asym(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-row asymmetric 8-bit quantisation: ``(q uint8 like x, params x.dtype [..., 2] = (scale, zero point))``."""
    _lib.require_gpu(x, "x")
    if x.dim() < 1 or x.numel() == 0:
        raise FastcacheError("quantize_rows_asym: empty input")
    xc = x.contiguous()
    d = xc.shape[-1]
    rows = xc.numel() // d
    q = torch.empty(xc.shape, dtype=torch.uint8, device=x.device)
    params = torch.empty(xc.shape[:-1] + (2,), dtype=x.dtype, device=x.device)
    check(fn("fc_quantize_rows_asym")(xc.data_ptr(), rows, d, _lib.dtype_code(x.dtype), q.data_ptr(),
                                      params.data_ptr(), current_stream()), "fc_quantize_rows_asym")
    return q, params


def _fp8_dtype(e5m2: bool) -> torch.dtype:
    return torch.float8_e5m2 if e5m2 else torch.float8_e4m3fn


def quantize_fp8(x: torch.Tensor, e5m2: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(x / scale).to(float8)`` with ``scale = clamp(max|x| / 448, 1e-8)`` over the whole tensor:
    ``(codes as a float8 tensor like x, scale 0-dim in x.dtype)``."""
    _lib.require_gpu(x, "x")
    if x.numel() == 0:
        raise FastcacheError("quantize_fp8: empty input")
    xc = x.contiguous()
    q = torch.empty(xc.shape, dtype=torch.uint8, device=x.device)
    scale = torch.empty((), dtype=x.dtype, device=x.device)
    nbytes = int(fn("fc_fake_quantize_workspace_bytes")())
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    check(fn("fc_quantize_fp8")(xc.data_ptr(), xc.numel(), _lib.dtype_code(x.dtype), int(bool(e5m2)), q.data_ptr(),
                                scale.data_ptr(), ws.data_ptr(), nbytes, current_stream()), "fc_quantize_fp8")
    return q.view(_fp8_dtype(e5m2)), scale


def dequantize_fp8(q: torch.Tensor, scale: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """``q.to(dtype) * scale`` for float8 codes and one scale for the tensor, with that expression's dtype promotion."""
    _lib.require_gpu(q, "q")
    _lib.require_gpu(scale, "scale")
    if q.dtype not in (torch.float8_e4m3fn, torch.float8_e5m2):
        raise FastcacheError(f"dequantize_fp8: float8 codes expected, got {q.dtype}")
    # the reference hands the scale out expanded over the leading dimensions: every element is the same number
    sc = scale.reshape(-1)[:1].contiguous()
    out_dtype = torch.promote_types(dtype, sc.dtype)
    qc = q.contiguous()
    out = torch.empty(qc.shape, dtype=out_dtype, device=q.device)
    check(fn("fc_dequantize_fp8")(qc.data_ptr(), sc.data_ptr(), qc.numel(), int(q.dtype == torch.float8_e5m2),
                                  _lib.dtype_code(sc.dtype), _lib.dtype_code(out_dtype), out.data_ptr(),
                                  current_stream()), "fc_dequantize_fp8")
    return out


def quantize_group4(x: torch.Tensor, group_size: int, nf4: bool) -> Tuple[torch.Tensor, torch.Tensor]:
    """Groups of ``group_size`` consecutive elements -> ``(packed uint8 [..., D/2], scale [..., D/group_size])``."""
    _lib.require_gpu(x, "x")
    D = x.shape[-1]
    if x.numel() == 0 or x.numel() % group_size or group_size % 2:
        raise FastcacheError(f"quantize_group4: {tuple(x.shape)} is not a whole number of groups of {group_size}")
    xc = x.contiguous()
    groups = xc.numel() // group_size
    packed = torch.empty(xc.numel() // 2, dtype=torch.uint8, device=x.device)
    scale = torch.empty(groups, dtype=x.dtype, device=x.device)
    check(fn("fc_quantize_group4")(xc.data_ptr(), groups, group_size, _lib.dtype_code(x.dtype), int(bool(nf4)),
                                   packed.data_ptr(), scale.data_ptr(), current_stream()), "fc_quantize_group4")
    return packed.view(*xc.shape[:-1], -1), scale.view(*xc.shape[:-1], -1)


def dequantize_group4(packed: torch.Tensor, scale: torch.Tensor, group_size: int, nf4: bool,
                      dtype: torch.dtype) -> torch.Tensor:
    """Inverse of :func:`quantize_group4`; output ``[..., 2 * packed.shape[-1]]`` in promote(dtype, scale.dtype)."""
    _lib.require_gpu(packed, "packed")
    _lib.require_gpu(scale, "scale")
    if packed.dtype != torch.uint8:
        raise FastcacheError(f"dequantize_group4: uint8 codes expected, got {packed.dtype}")
    n = packed.numel() * 2
    if n % group_size or scale.numel() != n // group_size:
        raise FastcacheError("dequantize_group4: one scale per group expected")
    out_dtype = torch.promote_types(dtype, scale.dtype)
    pc, sc = packed.contiguous(), scale.contiguous()
    out = torch.empty((*pc.shape[:-1], pc.shape[-1] * 2), dtype=out_dtype, device=packed.device)
    check(fn("fc_dequantize_group4")(pc.data_ptr(), sc.data_ptr(), n // group_size, group_size,
                                     _lib.dtype_code(sc.dtype), _lib.dtype_code(dtype), int(bool(nf4)),
                                     out.data_ptr(), current_stream()), "fc_dequantize_group4")
    return out


def linear_act(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], apply_relu: bool) -> torch.Tensor:
    """``act(x @ weight.T + bias)`` for ``x [M, K]`` (unit stride along K) and ``weight [N, K]`` contiguous,
    fp16/bf16, fp32 accumulation, rounded once to the input dtype."""
    _lib.require_gpu(x, "x")
    _lib.require_gpu(weight, "weight")
    if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1]:
        raise FastcacheError(f"linear_act: x {tuple(x.shape)} and weight {tuple(weight.shape)} do not match")
    if x.dtype not in (torch.float16, torch.bfloat16) or weight.dtype != x.dtype:
        raise FastcacheError(f"linear_act: fp16/bf16 operands of one dtype expected, got {x.dtype} and {weight.dtype}")
    if x.stride(1) != 1 or not weight.is_contiguous():
        raise FastcacheError("linear_act: x needs unit stride along K and weight must be contiguous [N, K]")
    if bias is not None:
        _lib.require_gpu(bias, "bias")
        if bias.dtype != x.dtype or tuple(bias.shape) != (weight.shape[0],) or not bias.is_contiguous():
            raise FastcacheError("linear_act: bias must be contiguous [N] in the input dtype")
    M, K = x.shape
    N = weight.shape[0]
    y = torch.empty((M, N), dtype=x.dtype, device=x.device)
    check(fn("fc_linear_act")(x.data_ptr(), x.stride(0) if M > 1 else K, weight.data_ptr(), _lib.ptr(bias),
                              y.data_ptr(), N, M, N, K, _lib.dtype_code(x.dtype), int(bool(apply_relu)),
                              current_stream()), "fc_linear_act")
    return y


# ---------------------------------------------------------------------------------------------
# decode
# ---------------------------------------------------------------------------------------------
def store_kv(k_cache: FcKvView, v_cache: FcKvView, k_new: torch.Tensor, v_new: torch.Tensor,
             context_lens: torch.Tensor) -> None:
    """Append ``k_new/v_new [L, B, Hkv, D]`` at position ``context_lens[b]`` of every sequence."""
    for t, name in ((k_new, "k_new"), (v_new, "v_new")):
        _lib.require_gpu(t, name)
        if tuple(t.shape) != (k_cache.num_layers, k_cache.batch, k_cache.num_kv_heads, k_cache.head_dim) \
                or not t.is_contiguous() or _lib.dtype_code(t.dtype) != k_cache.dtype:
            raise FastcacheError(f"{name} must be contiguous [L, B, Hkv, D] in the cache dtype")
    _i32(context_lens, "context_lens", k_new.device)
    check(fn("fc_store_kv")(C.byref(k_cache), C.byref(v_cache), k_new.data_ptr(), v_new.data_ptr(),
                            context_lens.data_ptr(), current_stream()), "fc_store_kv")


def advance_lens(context_lens: torch.Tensor, delta: int = 1) -> None:
    _i32(context_lens, "context_lens", context_lens.device)
    _lib.require_gpu(context_lens, "context_lens")
    check(fn("fc_advance_lens")(context_lens.data_ptr(), context_lens.numel(), delta, current_stream()),
          "fc_advance_lens")


def decode_attn_workspace(batch: int, num_q_heads: int, max_seq_len: int, device) -> torch.Tensor:
    n = fn("fc_decode_attn_workspace_bytes")(batch, num_q_heads, max_seq_len)
    if n < 0:
        raise FastcacheError("fc_decode_attn_workspace_bytes: bad arguments")
    return torch.empty((max(int(n), 256),), dtype=torch.uint8, device=device)


def decode_attn(k_cache: FcKvView, v_cache: FcKvView, layer: int, q: torch.Tensor, context_lens: torch.Tensor,
                scale: float, workspace: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """q ``[B, Hq, D]`` -> out ``[B, Hq, D]`` for one layer of the cache views."""
    _lib.require_gpu(q, "q")
    if q.dim() != 3 or not q.is_contiguous() or _lib.dtype_code(q.dtype) != k_cache.dtype:
        raise FastcacheError("q must be contiguous [B, Hq, D] in the cache dtype")
    if out is None:
        out = torch.empty_like(q)
    _i32(context_lens, "context_lens", q.device)
    check(fn("fc_decode_attn")(C.byref(k_cache), C.byref(v_cache), layer, q.data_ptr(), out.data_ptr(), q.shape[1],
                               context_lens.data_ptr(), scale, workspace.data_ptr(), workspace.numel(),
                               current_stream()), "fc_decode_attn")
    return out



def decode_attn_static(k_cache: FcKvView, v_cache: FcKvView, layer: int, q: torch.Tensor,
                       context_lens: torch.Tensor, scale: float, out: torch.Tensor) -> torch.Tensor:
    """``decode_attn`` with the chunk partials in the library's built-in device buffer: the call allocates
    nothing (``out`` is the caller's).  Calls that overlap on one GPU share that buffer and race."""
    _lib.require_gpu(q, "q")
    if q.dim() != 3 or not q.is_contiguous() or _lib.dtype_code(q.dtype) != k_cache.dtype:
        raise FastcacheError("q must be contiguous [B, Hq, D] in the cache dtype")
    if out.shape != q.shape or out.dtype != q.dtype or not out.is_contiguous():
        raise FastcacheError("out must be a contiguous tensor shaped and typed like q")
    _lib.require_gpu(out, "out")
    _i32(context_lens, "context_lens", q.device)
    check(fn("fc_decode_attn_static")(C.byref(k_cache), C.byref(v_cache), layer, q.data_ptr(), out.data_ptr(),
                                      q.shape[1], context_lens.data_ptr(), scale, current_stream()),
          "fc_decode_attn_static")
    return out
