#!/usr/bin/env python3
"""Benchmark of the KV-cache compression path on one MI355X.

``python bench.py --gpus 1 --steps K --warmup W`` prints ONE JSON line.  A step is one pass of the
hot path over one batch of synthetic input that is already resident in HBM.  The default workload
is configuration 2 (SnapKV press over a Qwen3-8B-shaped paged pool: score -> window fill -> top-k
-> in-place compaction, all 36 layers, batch 8, 4096 tokens per sequence).

Extra objects on the line:
  roofline      the dominant kernel of the workload: algorithmic bytes per launch divided by its
                average launch time, measured with HIP events on the launch stream inside the timed
                region, against the published 8 TB/s HBM peak;
  cpu_baseline  the CPU restatement of the reference path (oracle/) timed on this host on a bounded
                sample of the same workload and scaled to the full pass.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_PEAK_TFLOPS = 2500.0      # dense bf16/fp16, published


def _sync_time():
    torch.cuda.synchronize()
    return time.perf_counter()


# ---------------------------------------------------------------------------------------------------
# workload: SnapKV press (configuration 2)
# ---------------------------------------------------------------------------------------------------
class SnapKVWorkload:
    name = "cfg2-snapkv-qwen3-8b"
    dtype_name = "bf16"

    def __init__(self, seed, device, scale=1.0):
        from fastcache_amd import synth
        self.L, self.B, self.Hq, self.Hkv, self.S, self.W, self.ksz = 36, 8, 32, 8, 4096, 64, 7
        if scale != 1.0:                      # reduced shapes for dry runs only (never reported)
            self.L = max(1, int(self.L * scale))
        self.ratio = 0.75
        self.device = device
        self.case = synth.snapkv_case(seed=seed, num_layers=self.L, batch=self.B, num_q_heads=self.Hq,
                                      num_kv_heads=self.Hkv, seq_len=self.S, window=self.W,
                                      dtype=torch.bfloat16, device=device, device_draw=True)
        self.tables = self.case.table_tensor(device)
        self.lens = self.case.lens_tensor(device)
        self.queries = self.case.queries
        self.tokens_per_step = self.B * self.S
        self.n_kept = int(self.S * (1 - self.ratio))
        e = 2
        D = 128
        q_bytes = self.L * self.B * self.Hq * self.W * D * e
        k_bytes = self.L * self.B * self.Hkv * self.S * D * e
        gather_bytes = 4 * self.L * self.B * self.Hkv * self.n_kept * D * e
        score_bytes = self.L * self.B * self.Hkv * self.S * 4
        # dominant kernel = SnapKV scoring: Q window and K read once, fp32 scores written once
        self.kernel_name = "snapkv_kernel"
        self.kernel_bytes = q_bytes + k_bytes + score_bytes
        self.kernel_flops = 2 * self.B * self.L * self.Hq * self.W * self.S * D
        self.pass_bytes = q_bytes + k_bytes + gather_bytes
        self.ev = []

    def config(self):
        return {"workload": self.name, "layers": self.L, "batch": self.B, "q_heads": self.Hq,
                "kv_heads": self.Hkv, "head_dim": 128, "seq_len": self.S, "window": self.W,
                "kernel_size": self.ksz, "keep": self.n_kept, "block_size": 256,
                "reductions": "sum", "causal_window": True, "window_in_budget": True,
                "compaction": "in place"}

    def step(self, record=False):
        """score (bracketed by events when ``record``) -> window fill -> top-k -> in-place compaction."""
        import ctypes as C
        from fastcache_amd import _lib, ops
        from fastcache_amd._lib import check, current_stream, fn
        kv = self.case.kv_cache
        L, B, Hkv, S = self.L, self.B, self.Hkv, self.S
        kview = _lib.paged_view(kv[0], self.tables, self.lens, S)
        vview = _lib.paged_view(kv[1], self.tables, self.lens, S)
        scores = torch.empty((L, B, Hkv, S), dtype=torch.float32, device=self.device)
        st = current_stream()
        if record:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
        check(fn("fc_snapkv_score")(C.byref(kview), self.queries.data_ptr(), self.Hq, self.W, self.ksz, 1,
                                    128 ** -0.5, 1.0, scores.data_ptr(), S, st), "fc_snapkv_score")
        if record:
            e1.record()
            self.ev.append((e0, e1))
        # the window fill needs the whole layer's scores, so it is its own launch
        check(fn("fc_snapkv_fill_window")(scores.data_ptr(), S, L, B, Hkv, self.lens.data_ptr(), S, self.W, st),
              "fc_snapkv_fill_window")
        idx = ops.topk_select(scores, self.n_kept)
        ops.compact(kview, vview, kview, vview, idx)

    def cpu_baseline(self, budget_s=12.0):
        """CPU restatement of the same pass on a sample of layers and sequences, scaled linearly."""
        from oracle import pipeline as opipe
        threads = min(os.cpu_count() or 1, 16)
        torch.set_num_threads(threads)
        bs = min(2, self.B)
        tables = [self.case.block_tables[b] for b in range(bs)]
        lens = [self.S] * bs
        t_total, layers_done = 0.0, 0
        for layer in range(self.L):
            pool = self.case.kv_cache[:, layer:layer + 1].cpu()
            q = self.queries[layer:layer + 1, :bs].cpu()
            comp = opipe.snapkv_press_compressor(q, self.ratio, self.W, self.ksz, True, "sum")
            t0 = time.perf_counter()
            opipe.compress_batch(pool, tables, lens, comp)
            dt = time.perf_counter() - t0
            if layer == 0:          # warm-up layer is not counted
                continue
            t_total += dt
            layers_done += 1
            if t_total > budget_s:
                break
        full_pass_s = t_total / layers_done * self.L * (self.B / bs)
        return {"value": self.tokens_per_step / full_pass_s, "unit": "KV tokens/s", "cores": threads,
                "kind": "port",
                "sample": f"{layers_done} of {self.L} layers x {bs} of {self.B} sequences, "
                          f"{t_total:.2f} s measured, scaled linearly to the full pass"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--scale", type=float, default=1.0, help=argparse.SUPPRESS)
    args = ap.parse_args()

    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (no collectives, no sharding); "
              f"--gpus {args.gpus} is not supported", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from fastcache_amd import _lib
    _lib.load()          # fail loudly when the HIP library is missing
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    w = SnapKVWorkload(args.seed, dev, args.scale)

    for _ in range(args.warmup):
        w.step()
    t0 = _sync_time()
    for _ in range(args.steps):
        w.step(record=True)
    t1 = _sync_time()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    value = w.tokens_per_step / (ms_per_step * 1e-3)

    k_ms = sum(a.elapsed_time(b) for a, b in w.ev) / len(w.ev)
    achieved = w.kernel_bytes / (k_ms * 1e-3) / 1e9
    roofline = {"bound": "hbm", "kernel": w.kernel_name, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                "kernel_ms": round(k_ms, 4), "algorithmic_bytes": w.kernel_bytes,
                "mfma_tflops": round(w.kernel_flops / (k_ms * 1e-3) / 1e12, 1),
                "mfma_frac": round(w.kernel_flops / (k_ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4),
                "pass_gbs": round(w.pass_bytes / (ms_per_step * 1e-3) / 1e9, 1),
                "pass_frac": round(w.pass_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}

    out = {"metric": "KV tokens compressed/sec", "value": round(value, 1), "unit": "KV tokens/s", "n_gpus": 1,
           "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": w.dtype_name,
           "data": "synthetic", "config": w.config(), "roofline": roofline}
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = w.cpu_baseline()
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
