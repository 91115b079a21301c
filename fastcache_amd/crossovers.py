"""Measure the crossovers behind the launch-shape rules of this library on the GPU at hand.

``python -m fastcache_amd.crossovers [knorm] [select] [splits] [press]`` times, on random data,

* ``knorm``:  ``fc_knorm_press`` over grids of (columns x rows per column): the rule that gives a column 1024 threads
  instead of 256 is the compile-time constant ``KP_WIDE_BYTES_PRESS`` of csrc/fc_press.hip (bytes of key rows per
  column); build the library with ``FC_EXTRA_HIPCC_FLAGS="-DKP_WIDE_BYTES_PRESS=0 -DKP_WIDE_BYTES_SELECT=0"`` (always
  1024 threads) and with ``=2000000000`` (always 256) and run this on both to see where the two cross;
* ``select``: ``fc_select_compact`` the same way (``KP_WIDE_BYTES_SELECT``);
* ``splits``: ``fc_snapkv_score`` / ``fc_snapkv_score_split`` with 1, 2, 4 and 8 key ranges per column (the rule is
  ``ops.snapkv_splits``);
* ``press``:  the one-launch SnapKV press against split scoring + ``fc_select_compact`` (``ops.snapkv_press_preferred``).

Every figure is the mean of 20 launches after 5, HIP events on the current stream.
"""
from __future__ import annotations

import sys

import torch

from . import _lib, ops


def _time(fn, reps=20, warm=5):
    for _ in range(warm):
        fn()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / reps


def _dense(L, B, H, S, dtype, dev):
    k = torch.randn((L, B, H, S, 128), device=dev, dtype=torch.float32).to(dtype)
    return k, torch.randn((L, B, H, S, 128), device=dev, dtype=torch.float32).to(dtype)


def knorm(dev):
    print("fc_knorm_press, ms per launch (half of each column kept):")
    for dtype, L, B, H, S in ((torch.float32, 32, 1, 32, 1024), (torch.bfloat16, 32, 4, 32, 2048),
                              (torch.bfloat16, 32, 4, 32, 1024), (torch.bfloat16, 32, 16, 32, 512),
                              (torch.bfloat16, 32, 64, 32, 128)):
        k, v = _dense(L, B, H, S, dtype, dev)
        kv, vv = _lib.dense_view(k), _lib.dense_view(v)
        t = _time(lambda: ops.knorm_press(kv, vv, S // 2, dev))
        print(f"  {L * B * H:6d} columns x {S:5d} rows of {k.element_size() * 128} B: {t:.3f}")
        del k, v


def select(dev):
    print("fc_select_compact, ms per launch (a quarter of each column kept):")
    for L, B, H, S in ((36, 8, 8, 4096), (32, 4, 32, 2048), (32, 16, 32, 512)):
        k, v = _dense(L, B, H, S, torch.bfloat16, dev)
        kv, vv = _lib.dense_view(k), _lib.dense_view(v)
        sc = torch.rand((L, B, H, S), device=dev)
        t = _time(lambda: ops.select_compact(kv, vv, sc, S // 4))
        print(f"  {L * B * H:6d} columns x {S:5d} rows of 256 B: {t:.3f}")
        del k, v, sc


def _snap_case(L, B, Hq, Hkv, S, dev, W=64):
    k, v = _dense(L, B, Hkv, S, torch.bfloat16, dev)
    q = torch.randn((L, B, Hq, W, 128), device=dev, dtype=torch.float32).to(torch.bfloat16)
    return k, v, q


def splits(dev):
    print("SnapKV scoring (window 64, kernel 7), ms per launch by key ranges per column (1 = whole columns):")
    for L, B, Hq, Hkv, S in ((36, 8, 32, 8, 4096), (36, 2, 32, 8, 16384), (36, 1, 32, 8, 32768), (28, 1, 28, 4, 32768)):
        k, v, q = _snap_case(L, B, Hq, Hkv, S, dev)
        kv = _lib.dense_view(k)
        row = [f"{_time(lambda: ops.snapkv_score(kv, q, 64, 7, True, 'sum', splits=n)):.3f}" for n in (1, 2, 4, 8)]
        print(f"  {L * B * Hkv:5d} columns x {S:6d} keys, {Hq // Hkv} query heads per kv head: " + " / ".join(row)
              + f"   (ops.snapkv_splits picks {ops.snapkv_splits(kv, Hq, 64)})")
        del k, v, q


def press(dev):
    print("SnapKV press, a quarter kept, ms per pass: one launch / split scoring + fc_select_compact:")
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    for L, B, Hq, Hkv, S in ((28, 4, 28, 4, 4096), (28, 6, 28, 4, 4096), (36, 8, 32, 8, 4096), (20, 4, 28, 4, 12000)):
        k, v, q = _snap_case(L, B, Hq, Hkv, S, dev)
        kv, vv = _lib.dense_view(k), _lib.dense_view(v)
        n = S // 4
        if not ops.snapkv_press_fits(kv, Hq, 64, n):
            print(f"  {L * B * Hkv:5d} columns x {S} keys: the one-launch press does not take this shape")
            continue
        one = _time(lambda: ops.snapkv_press(kv, vv, q, 64, 7, n, True, "sum"))
        ns = max(2, ops.snapkv_splits(kv, Hq, 64))

        def two():
            sc = ops.snapkv_score(kv, q, 64, 7, True, "sum", splits=ns)
            ops.select_compact(kv, vv, sc, n)
        print(f"  {L * B * Hkv:5d} columns x {S:6d} keys: {one:.3f} / {_time(two):.3f} ({ns} ranges)   "
              f"(ops.snapkv_press_preferred: {ops.snapkv_press_preferred(kv, Hq, 64, cus)})")
        del k, v, q


def main(argv):
    if not torch.cuda.is_available():
        raise SystemExit("crossovers: no GPU visible")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    _lib.load()
    todo = argv or ["knorm", "select", "splits", "press"]
    table = {"knorm": knorm, "select": select, "splits": splits, "press": press}
    for name in todo:
        if name not in table:
            raise SystemExit(f"crossovers: unknown group {name!r}; choose from {sorted(table)}")
        table[name](dev)


if __name__ == "__main__":
    main(sys.argv[1:])
