"""ctypes binding of libfastcache_hip.so (the C ABI declared in include/fastcache_hip.h).

The library is the only compute path of this package: if it is missing or cannot be loaded the
import of any operator raises, there is no PyTorch or CPU fallback.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path
from typing import Optional

import torch

LIB_PATH = Path(__file__).resolve().parent / "libfastcache_hip.so"

FC_F32, FC_F16, FC_BF16 = 0, 1, 2
_DTYPES = {torch.float32: FC_F32, torch.float16: FC_F16, torch.bfloat16: FC_BF16}

c_i32p = C.POINTER(C.c_int32)


class FcKvView(C.Structure):
    _fields_ = [
        ("base", C.c_void_p),
        ("stride_layer", C.c_int64),
        ("stride_block", C.c_int64),
        ("stride_batch", C.c_int64),
        ("stride_token", C.c_int64),
        ("stride_head", C.c_int64),
        ("block_tables", C.c_void_p),
        ("table_stride", C.c_int32),
        ("block_size", C.c_int32),
        ("dtype", C.c_int32),
        ("num_layers", C.c_int32),
        ("batch", C.c_int32),
        ("num_kv_heads", C.c_int32),
        ("head_dim", C.c_int32),
        ("max_seq_len", C.c_int32),
        ("seq_lens", C.c_void_p),
    ]


class FcMlpWeights(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("w1", "b1", "w2", "b2", "w3", "b3")]


class FastcacheError(RuntimeError):
    pass


_lib: Optional[C.CDLL] = None

_VP = C.c_void_p
_I = C.c_int32
_F = C.c_float
_V = C.POINTER(FcKvView)

# name -> (restype, argtypes); must list every function of include/fastcache_hip.h
SIGNATURES = {
    "fc_abi_version": (C.c_int, []),
    "fc_last_error": (C.c_char_p, []),
    "fc_knorm_score": (C.c_int, [_V, _VP, _I, _VP]),
    "fc_knorm_mean_score": (C.c_int, [_V, _VP, _I, _VP]),
    "fc_snapkv_score": (C.c_int, [_V, _VP, _I, _I, _I, _I, _F, _F, _VP, _I, _VP, _VP]),
    "fc_snapkv_score_lse": (C.c_int, [_V, _VP, _VP, _I, _I, _I, _I, _F, _F, _VP, _I, _VP, _VP]),
    "fc_snapkv_press": (C.c_int, [_V, _V, _VP, _VP, _I, _I, _I, _I, _F, _F, _VP, _I, _VP, _I, _VP, _VP, _I, _VP]),
    "fc_snapkv_split_workspace_bytes": (C.c_int64, [_I, _I, _I, _I, _I, _I, _I]),
    "fc_snapkv_score_split": (C.c_int, [_V, _VP, _VP, _I, _I, _I, _I, _F, _F, _VP, _I, _VP, _I, _VP, C.c_int64, _VP]),
    "fc_snapkv_fill_window": (C.c_int, [_VP, _I, _I, _I, _I, _VP, _I, _I, _VP, _VP]),
    "fc_topk_select": (C.c_int, [_VP, _I, _I, _I, _VP, _I, _I, _I, _VP, _VP, _I, _VP]),
    "fc_compact": (C.c_int, [_V, _V, _V, _V, _VP, _I, _I, _I, _VP, _VP]),
    "fc_knorm_press": (C.c_int, [_V, _V, _VP, _I, _I, _VP, _VP, _I, _VP]),
    "fc_select_compact": (C.c_int, [_V, _V, _VP, _I, _I, _VP, _VP, _I, _VP]),
    "fc_ccm_mlp": (C.c_int, [_V, _V, C.POINTER(FcMlpWeights), _I, _I, _I, _I, _VP]),
    "fc_ccm_mlp_ragged": (C.c_int, [_V, _V, C.POINTER(FcMlpWeights), _I, _VP, _VP, _VP, _I, _I, _VP]),
    "fc_linear_act": (C.c_int, [_VP, C.c_int64, _VP, _VP, _VP, C.c_int64, C.c_int64, _I, _I, _I, _I, _VP]),
    "fc_quantize_rows": (C.c_int, [_VP, C.c_int64, _I, _I, _I, _VP, _VP, _VP]),
    "fc_dequantize_rows": (C.c_int, [_VP, _VP, C.c_int64, _I, _I, _I, _VP, _VP]),
    "fc_fake_quantize_workspace_bytes": (C.c_int64, []),
    "fc_fake_quantize": (C.c_int, [_VP, _VP, C.c_int64, _I, _I, _I, _I, _VP, _VP, _VP, C.c_int64, _VP]),
    "fc_key_channel_energy": (C.c_int, [_V, _VP, _VP]),
    "fc_key_channel_zero": (C.c_int, [_V, _VP, _VP]),
    "fc_quantize_fp8": (C.c_int, [_VP, C.c_int64, _I, _I, _VP, _VP, _VP, C.c_int64, _VP]),
    "fc_dequantize_fp8": (C.c_int, [_VP, _VP, C.c_int64, _I, _I, _I, _VP, _VP]),
    "fc_quantize_rows_asym": (C.c_int, [_VP, C.c_int64, _I, _I, _VP, _VP, _VP]),
    "fc_quantize_group4": (C.c_int, [_VP, C.c_int64, _I, _I, _I, _VP, _VP, _VP]),
    "fc_dequantize_group4": (C.c_int, [_VP, _VP, C.c_int64, _I, _I, _I, _I, _VP, _VP]),
    "fc_expected_attention_workspace_bytes": (C.c_int64, [_I, _I, _I, _I]),
    "fc_expected_attention_score": (C.c_int, [_V, _V, _VP, _VP, _I, _I, _I, _F, _VP, _I, _VP, C.c_int64, _VP]),
    "fc_observed_attention_workspace_bytes": (C.c_int64, [_I, _I, _I]),
    "fc_observed_attention_score": (C.c_int, [_VP, _I, _I, _I, _I, _I, _I, _VP, _VP, C.c_int64, _VP]),
    "fc_copy_tokens": (C.c_int, [_V, _V, _I, _I, _I, _VP]),
    "fc_copy_tokens_from_layers": (C.c_int, [_VP, _V, _V, _I, _I, _I, _VP]),
    "fc_store_kv": (C.c_int, [_V, _V, _VP, _VP, _VP, _VP]),
    "fc_store_kv_slots": (C.c_int, [_VP, C.c_int64, _VP, C.c_int64, _VP, _VP, _VP, _I, _I, _I, _VP]),
    "fc_advance_lens": (C.c_int, [_VP, _I, _I, _VP]),
    "fc_decode_attn_workspace_bytes": (C.c_int64, [_I, _I, _I]),
    "fc_decode_attn": (C.c_int, [_V, _V, _I, _VP, _VP, _I, _VP, _F, _VP, C.c_int64, _VP]),
    "fc_decode_attn_static_capacity": (C.c_int64, []),
    "fc_decode_attn_static": (C.c_int, [_V, _V, _I, _VP, _VP, _I, _VP, _F, _VP]),
}


def load() -> C.CDLL:
    """Open the library once; raise FastcacheError with the reason if that is not possible."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise FastcacheError(
            f"{LIB_PATH} is missing: build it with `python -m fastcache_amd.build` "
            "(hipcc --offload-arch=gfx950); this package has no fallback path")
    try:
        lib = C.CDLL(str(LIB_PATH))
    except OSError as e:  # pragma: no cover - depends on the host
        raise FastcacheError(f"cannot load {LIB_PATH}: {e}") from e
    _lib = lib
    return lib


_bound = {}


def fn(name: str):
    """The entry point `name`, with its ctypes signature set; raises if the library lacks it."""
    f = _bound.get(name)
    if f is None:
        res, args = SIGNATURES[name]
        try:
            f = getattr(load(), name)
        except AttributeError as e:
            raise FastcacheError(f"{LIB_PATH} does not export {name}; rebuild the library") from e
        f.restype = res
        f.argtypes = args
        _bound[name] = f
    return f


_enqueued = 0


def check(rc: int, what: str) -> None:
    global _enqueued
    if rc != 0:
        msg = fn("fc_last_error")().decode("utf-8", "replace")
        raise FastcacheError(f"{what} failed (code {rc}): {msg}")
    _enqueued += 1


def enqueue_count() -> int:
    """Entry-point calls that have returned success so far in this process (each is at least one launch handed to
    a stream).  Callers that rewrite a cache in place compare two readings to tell a failure before any launch
    from one that may have left rows half rewritten."""
    return _enqueued


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _DTYPES[dt]
    except KeyError:
        raise FastcacheError(f"unsupported KV dtype {dt}; expected float32, float16 or bfloat16") from None


def require_gpu(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise FastcacheError(f"{name} must live on the GPU (got device {t.device}); "
                             "libfastcache_hip has no CPU path")


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def current_stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def paged_view(plane: torch.Tensor, block_tables: torch.Tensor, seq_lens: Optional[torch.Tensor],
               max_seq_len: int) -> FcKvView:
    """View of one plane (K or V) of a paged pool.

    plane ``[L, num_blocks, block_size, Hkv, D]`` (``kv_cache[0]`` or ``kv_cache[1]``);
    block_tables int32 ``[B, width]`` on the same device; seq_lens int32 ``[B]`` or None.
    """
    require_gpu(plane, "kv pool")
    if plane.dim() != 5 or plane.stride(-1) != 1:
        raise FastcacheError("paged plane must be [L, blocks, block_size, Hkv, D] with contiguous D")
    if block_tables.dtype != torch.int32 or block_tables.dim() != 2 or not block_tables.is_contiguous():
        raise FastcacheError("block_tables must be a contiguous int32 [B, width] tensor")
    require_gpu(block_tables, "block_tables")
    if seq_lens is not None:
        if seq_lens.dtype != torch.int32 or seq_lens.numel() != block_tables.shape[0]:
            raise FastcacheError("seq_lens must be int32 [B]")
        require_gpu(seq_lens, "seq_lens")
    L, _, bs, H, D = plane.shape
    st = [plane.stride(i) if plane.shape[i] > 1 else 0 for i in range(4)]
    view = FcKvView(
        base=plane.data_ptr(), stride_layer=st[0], stride_block=st[1], stride_batch=0,
        stride_token=st[2], stride_head=st[3],
        block_tables=block_tables.data_ptr(), table_stride=block_tables.shape[1], block_size=bs,
        dtype=dtype_code(plane.dtype), num_layers=L, batch=block_tables.shape[0], num_kv_heads=H,
        head_dim=D, max_seq_len=int(max_seq_len), seq_lens=ptr(seq_lens))
    # the struct carries raw addresses: the view keeps the tensors alive, so that a table or length tensor built in
    # the call expression cannot be handed back to the allocator (and reused) before the kernels have read it
    view._tensors = (plane, block_tables, seq_lens)
    return view


def dense_view(t: torch.Tensor, seq_len: Optional[int] = None) -> FcKvView:
    """View of a HuggingFace-layout tensor ``[B, Hkv, S, D]`` or a stack ``[L, B, Hkv, S, D]``
    (any strides with contiguous D)."""
    require_gpu(t, "kv tensor")
    if t.dim() == 4:
        t = t.unsqueeze(0)
    if t.dim() != 5 or (t.shape[-1] > 1 and t.stride(-1) != 1):
        raise FastcacheError("dense KV must be [B, Hkv, S, D] or [L, B, Hkv, S, D] with contiguous D")
    L, B, H, S, D = t.shape
    st = [t.stride(i) if t.shape[i] > 1 else 0 for i in range(4)]  # strides of size-1 axes are arbitrary
    view = FcKvView(
        base=t.data_ptr(), stride_layer=st[0], stride_block=0, stride_batch=st[1],
        stride_token=st[3], stride_head=st[2], block_tables=None, table_stride=0, block_size=1,
        dtype=dtype_code(t.dtype), num_layers=L, batch=B, num_kv_heads=H, head_dim=D,
        max_seq_len=int(S if seq_len is None else seq_len), seq_lens=None)
    view._tensors = (t,)          # as in paged_view: the view keeps what it points at alive
    return view
