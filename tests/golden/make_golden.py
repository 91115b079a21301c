"""Writes the small golden fixtures of this directory (run from the repository root:
``python tests/golden/make_golden.py``).

The reference's own tests hold no golden vectors for this path, so the fixtures are produced by the CPU oracle on
seeded tiny inputs: they freeze the oracle's outputs (a change in the oracle or in the input generators shows up as
a failing CPU test) and give the GPU tests byte-level expectations that do not depend on the oracle code at test
time.  16-bit tensors are stored as their bit patterns (int16), everything as ``.npz`` without pickling.
"""
import math
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import attention as oattn          # noqa: E402
from oracle import ccm as occm                 # noqa: E402
from oracle import presses as opress           # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def bits(t: torch.Tensor) -> np.ndarray:
    """numpy view of a tensor; fp16 / bf16 as int16 bit patterns."""
    t = t.contiguous()
    return t.view(torch.int16).numpy() if t.dtype in (torch.float16, torch.bfloat16) else t.numpy()


def knorm():
    g = torch.Generator().manual_seed(101)
    keys = torch.randn(1, 2, 40, 128, generator=g)
    keys[:, :, ::7] *= 3.0
    values = torch.randn(1, 2, 40, 128, generator=g)
    scores = opress.knorm_score(keys)
    idx = opress.topk_lowest_index(scores, 10)
    return dict(keys=bits(keys), values=bits(values), scores=bits(scores),
                indices=idx.numpy().astype(np.int32), kept_keys=bits(opress.gather_tokens(keys, idx)),
                kept_values=bits(opress.gather_tokens(values, idx)))


def snapkv():
    g = torch.Generator().manual_seed(202)
    q = torch.randn(1, 4, 16, 128, generator=g).bfloat16()
    keys = torch.randn(1, 2, 96, 128, generator=g).bfloat16()
    out = {"queries": bits(q), "keys": bits(keys)}
    for causal in (True, False):
        for red in ("mean", "sum"):
            sc = opress.snapkv_score(q, keys, 16, 5, causal_window=causal, reduction=red)
            out[f"scores_causal{int(causal)}_{red}"] = bits(sc)
            out[f"indices_causal{int(causal)}_{red}"] = opress.topk_lowest_index(sc, 40).numpy().astype(np.int32)
    return out


def ccm():
    sd = occm.reference_init_state_dict("linear_decouple", n_layer=1, head_dim=128, cf=2, seed=7)
    g = torch.Generator().manual_seed(303)
    k = torch.randn(1, 2, 21, 128, generator=g).half()
    v = torch.randn(1, 2, 21, 128, generator=g).half()
    (ck, cv), = occm.linear_decouple_forward([(k, v)], [12, 9], {n: t.half() for n, t in sd.items()}, cf=2, min_seq_len=1)
    return dict(keys=bits(k), values=bits(v), out_keys=bits(ck), out_values=bits(cv),
                it_len=np.array([12, 9], dtype=np.int32), seed=np.array(7, dtype=np.int32))


def decode():
    g = torch.Generator().manual_seed(404)
    nb, bs, Hkv, Hq, D = 6, 16, 2, 8, 128
    kc = torch.randn(nb, bs, Hkv, D, generator=g).half()
    vc = torch.randn(nb, bs, Hkv, D, generator=g).half()
    q = torch.randn(3, Hq, D, generator=g).half()
    lens = torch.tensor([1, 33, 16], dtype=torch.int32)
    tables = torch.tensor([[4, -1, -1], [2, 0, 5], [3, -1, -1]], dtype=torch.int32)
    out = oattn.decode_attention(q, kc, vc, lens, tables, 1.0 / math.sqrt(D))
    return dict(q=bits(q), k_cache=bits(kc), v_cache=bits(vc), lens=lens.numpy(), tables=tables.numpy(), out=bits(out))


FIXTURES = {"knorm_fp32.npz": knorm, "snapkv_bf16.npz": snapkv, "ccm_linear_decouple_fp16.npz": ccm,
            "decode_attention_fp16.npz": decode}

if __name__ == "__main__":
    for name, make in FIXTURES.items():
        np.savez(os.path.join(HERE, name), **make())
    print("wrote", sorted(FIXTURES))
