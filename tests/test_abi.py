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


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "nope.so")
    with pytest.raises(_lib.FastcacheError):
        _lib.load()
