"""The C ABI: the shared library loads and exports every function the header declares, and the
ctypes signatures cover exactly that set.  No compute call is made (runs without a GPU)."""
import ctypes
import re
from pathlib import Path

import pytest

from fastcache_amd import _lib

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "fastcache_hip.h"


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(fc_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_functions():
    names = declared_functions()
    assert "fc_snapkv_score" in names and "fc_decode_attn" in names and len(names) >= 14


def test_library_exports_every_declared_symbol():
    if not _lib.LIB_PATH.exists():
        pytest.fail(f"{_lib.LIB_PATH} missing: run `python -m fastcache_amd.build`")
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    missing = [n for n in declared_functions() if not hasattr(lib, n)]
    assert not missing, f"not exported: {missing}"


def test_signatures_cover_the_header():
    assert sorted(_lib.SIGNATURES) == declared_functions()
    for name in _lib.SIGNATURES:
        _lib.fn(name)          # binds restype/argtypes; raises if the symbol is absent


def test_abi_version_and_error_text():
    assert _lib.fn("fc_abi_version")() == 1
    assert isinstance(_lib.fn("fc_last_error")(), bytes)


def test_argument_validation_without_gpu():
    """Bad arguments are rejected on the host before any launch."""
    rc = _lib.fn("fc_topk_select")(None, 0, 1, 1, None, 1, 1, 1, None, None, 1, None)
    assert rc == -1
    assert b"null" in _lib.fn("fc_last_error")()
    v = _lib.FcKvView()
    rc = _lib.fn("fc_knorm_score")(ctypes.byref(v), None, 0, None)
    assert rc == -1
    v.base = 16
    v.dtype, v.head_dim, v.num_layers, v.batch, v.num_kv_heads = 2, 64, 1, 1, 1
    rc = _lib.fn("fc_knorm_score")(ctypes.byref(v), None, 0, None)
    assert rc == -2 and b"head_dim" in _lib.fn("fc_last_error")()


def _dense_view(seq_len, dtype=2, heads=2):
    """A view of nothing real (base 256): enough for the host-side checks, which never touch the memory."""
    v = _lib.FcKvView()
    v.base, v.dtype, v.head_dim, v.num_layers, v.batch, v.num_kv_heads = 256, dtype, 128, 1, 1, heads
    v.stride_layer = v.stride_batch = heads * seq_len * 128
    v.stride_head, v.stride_token, v.block_size, v.max_seq_len = seq_len * 128, 128, 1, seq_len
    return v


def test_one_launch_presses_validate_on_the_host():
    """fc_knorm_press / fc_select_compact / fc_snapkv_press refuse what they cannot take before any launch: missing
    outputs, kept counts beyond the index row, columns too long for LDS, kept counts inside the window."""
    err = lambda: _lib.fn("fc_last_error")()
    k, v = _dense_view(1024), _dense_view(1024)
    B = ctypes.byref
    assert _lib.fn("fc_knorm_press")(B(k), B(v), None, 1024, 10, None, None, 10, None) == -1 and b"null" in err()
    assert _lib.fn("fc_knorm_press")(B(k), B(v), 16, 1000, 10, None, 16, 10, None) == -1 and b"score_stride" in err()
    assert _lib.fn("fc_select_compact")(B(k), B(v), 16, 1024, 20, None, 16, 10, None) == -1 and b"index_stride" in err()
    other = _dense_view(1024, heads=4)
    assert _lib.fn("fc_select_compact")(B(k), B(other), 16, 1024, 10, None, 16, 10, None) == -1 and b"disagree" in err()
    kl, vl = _dense_view(40000), _dense_view(40000)
    assert _lib.fn("fc_select_compact")(B(kl), B(vl), 16, 40000, 10, None, 16, 10, None) == -2 and b"LDS" in err()
    press = _lib.fn("fc_snapkv_press")
    args = lambda kk, vv, k_keep, stride: (B(kk), B(vv), 16, None, 8, 64, 7, 1, 0.1, 1.0, 16, kk.max_seq_len, 16, k_keep, None,
                                           16, stride, None)
    assert press(*args(k, v, 64, 64)) == -1 and b"exceed the window" in err()
    assert press(*args(kl, vl, 5000, 5000)) == -2 and b"fc_select_compact" in err()
    f32 = _dense_view(1024, dtype=0)
    assert press(*args(f32, f32, 100, 100)) == -2 and b"fp16/bf16" in err()


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "nope.so")
    with pytest.raises(_lib.FastcacheError):
        _lib.load()
