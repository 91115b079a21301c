"""GPU: the decode-attention entry point that allocates nothing (chunk partials in a device array built into the
library) gives the bytes of the workspace entry point, on two calls in a row, the second on a smaller input, and
rejects shapes beyond its capacity."""
import ctypes as C

import pytest
import torch

from fastcache_amd import _lib, ops, synth

pytestmark = pytest.mark.gpu


def _case(dev, seed, Hq, Hkv, lens, dtype):
    case = synth.make_paged_case(seed=seed, num_layers=2, batch=len(lens), num_kv_heads=Hkv, seq_lens=lens,
                                 dtype=dtype, reserve_tokens=8)
    q = torch.randn(2, len(lens), Hq, 128, generator=torch.Generator().manual_seed(seed + 1)).to(dtype).to(dev)
    width = max(len(t) for t in case.block_tables) + 1
    tab = case.table_tensor(dev, width)
    pool = case.kv_cache.to(dev)
    max_len = width * 256
    views = tuple(_lib.paged_view(pool[i], tab, None, max_len) for i in range(2))
    return views, q, torch.tensor(lens, dtype=torch.int32, device=dev), max_len, (pool, tab)


def test_static_scratch_entry_matches_workspace_entry(dev):
    scale = 128 ** -0.5
    # first call: 6 sequences up to 9 chunks; second call: a smaller batch, fewer heads, shorter caches
    for seed, Hq, Hkv, lens, dtype in [(3, 16, 4, [2300, 1, 257, 1024, 77, 512], torch.float16),
                                        (4, 14, 2, [300, 40], torch.bfloat16)]:
        (kview, vview), q, lens_d, max_len, keep = _case(dev, seed, Hq, Hkv, lens, dtype)
        ws = ops.decode_attn_workspace(len(lens), Hq, max_len, dev)
        out = torch.empty_like(q)
        for layer in range(2):
            ref = ops.decode_attn(kview, vview, layer, q[layer], lens_d, scale, ws)
            torch.cuda.synchronize()
            before = torch.cuda.memory_allocated(dev)
            ops.decode_attn_static(kview, vview, layer, q[layer], lens_d, scale, out[layer])
            torch.cuda.synchronize()
            assert torch.cuda.memory_allocated(dev) == before
            assert torch.equal(out[layer].view(torch.int16), ref.view(torch.int16)), (seed, layer)


def test_static_scratch_entry_rejects_oversize(dev):
    cap = _lib.fn("fc_decode_attn_static_capacity")()
    assert cap == 16 << 20
    B, Hq, max_len = 64, 32, 8192                     # 64 * 32 * 32 chunks * 520 B = 34 MB of partials
    assert _lib.fn("fc_decode_attn_workspace_bytes")(B, Hq, max_len) > cap
    pool = torch.zeros(2, 1, 4, 256, 8, 128, dtype=torch.float16, device=dev)
    tab = torch.zeros(B, max_len // 256, dtype=torch.int32, device=dev)
    views = [_lib.paged_view(pool[i], tab, None, max_len) for i in range(2)]
    q = torch.zeros(B, Hq, 128, dtype=torch.float16, device=dev)
    lens = torch.ones(B, dtype=torch.int32, device=dev)
    rc = _lib.fn("fc_decode_attn_static")(C.byref(views[0]), C.byref(views[1]), 0, q.data_ptr(), q.data_ptr(), Hq,
                                          lens.data_ptr(), 1.0, None)
    assert rc == -2 and b"built-in" in _lib.fn("fc_last_error")()


_GUARD_CHILD = r"""
import sys, torch
sys.path.insert(0, sys.argv[1])
from fastcache_amd import _lib, ops
dev = torch.device("cuda:0")
pool = torch.randn(2, 1, 8, 256, 2, 128, device=dev).half()
tab = torch.arange(8, dtype=torch.int32, device=dev).view(2, 4)
lens = torch.tensor([700, 300], dtype=torch.int32, device=dev)
views = [_lib.paged_view(pool[i], tab, None, 1024) for i in range(2)]
q = torch.randn(2, 4, 128, device=dev).half()
out = torch.empty_like(q)
side = torch.cuda.Stream()
ops.decode_attn_static(views[0], views[1], 0, q, lens, 0.088, out)          # first call: nothing to compare with
torch.cuda.synchronize()
ref = out.clone()
torch.cuda._sleep(2_000_000_000)                                            # about a second of pending work on the main stream
ops.decode_attn_static(views[0], views[1], 0, q, lens, 0.088, out)
refused = False
with torch.cuda.stream(side):
    try:
        ops.decode_attn_static(views[0], views[1], 0, q, lens, 0.088, out)
    except _lib.FastcacheError as e:
        refused = "another stream" in str(e)
torch.cuda.synchronize()                                                    # the main stream has drained: the side stream may call
with torch.cuda.stream(side):
    ops.decode_attn_static(views[0], views[1], 0, q, lens, 0.088, out)
torch.cuda.synchronize()
print("REFUSED" if refused else "ACCEPTED", "SAME" if torch.equal(out, ref) else "DIFFERENT")
"""


def test_static_scratch_guard_refuses_an_overlapping_stream(dev, tmp_path):
    """FC_STATIC_GUARD=1 (read once per process, hence a child process): a call on another stream while the previous
    call's stream still has work pending is refused before anything is enqueued; once that stream has drained the
    same call goes through and gives the same bytes.  Without the variable the library does not look."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    script = tmp_path / "guard_child.py"
    script.write_text(_GUARD_CHILD)
    for guard, want in (("1", "REFUSED SAME"), ("", "ACCEPTED SAME")):
        env = dict(os.environ, FC_STATIC_GUARD=guard)
        res = subprocess.run([sys.executable, str(script), root], capture_output=True, text=True, env=env, timeout=100)
        assert res.returncode == 0, res.stderr[-2000:]
        assert res.stdout.strip().splitlines()[-1] == want, (guard, res.stdout, res.stderr[-500:])
