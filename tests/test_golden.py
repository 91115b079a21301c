"""The committed golden fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py).

CPU: the oracle still reproduces every stored array (inputs, indices and gathered bytes bit for bit, floating-point
results to the accuracy of the host's summation order: a change of the oracle or of the seeded inputs cannot pass unnoticed).  GPU: the HIP path fed with the stored inputs meets the stored outputs at the parity bar
(indices, tables and copied bytes exact; scores <= 1e-3 relative; MLP outputs within the bound of test_gpu_ccm;
attention <= 2e-2 absolute).
"""
import importlib.util
import os

import numpy as np
import pytest
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _load(name):
    with np.load(os.path.join(GOLDEN, name), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def _t(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    return t.view(dtype) if dtype in (torch.float16, torch.bfloat16) else t


def test_oracle_reproduces_the_fixtures():
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(GOLDEN, "make_golden.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    assert sorted(mod.FIXTURES) == sorted(f for f in os.listdir(GOLDEN) if f.endswith(".npz"))
    # Inputs, indices and gathered bytes are reproduced exactly.  Arrays that come out of a floating-point
    # reduction on the CPU (matmul, softmax, norm) depend on the host's summation order in the last place:
    # fp32 ones must agree to 1e-5 relative, fp16 ones to 1e-3 of the largest value plus 2 units in the last place.
    computed_fp32 = {"scores"} | {f"scores_causal{c}_{r}" for c in (0, 1) for r in ("mean", "sum")}
    computed_fp16 = {"out_keys", "out_values", "out"}
    for name, make in mod.FIXTURES.items():
        stored, fresh = _load(name), make()
        assert sorted(stored) == sorted(fresh), name
        for key in stored:
            a, b = stored[key], fresh[key]
            assert a.dtype == b.dtype and a.shape == b.shape, (name, key)
            if key in computed_fp32:
                assert np.allclose(a, b, rtol=1e-5, atol=0), (name, key)
            elif key in computed_fp16:
                fa, fb = _t(a, torch.float16).float(), _t(b, torch.float16).float()
                scale = float(fa.abs().max())     # a hidden activation may round the other way: bound of test_gpu_ccm
                bound = 1e-3 * scale + 2 * 2.0 ** -10 * fa.abs().clamp_min(scale * 2.0 ** -14)
                assert bool(((fa - fb).abs() <= bound).all()), (name, key)
            else:
                assert np.array_equal(a, b), (name, key)


@pytest.mark.gpu
def test_knorm_fixture(dev):
    from fastcache_amd import _lib, ops
    z = _load("knorm_fp32.npz")
    keys, values = _t(z["keys"]).to(dev), _t(z["values"]).to(dev)
    sc = ops.knorm_score(_lib.dense_view(keys), dev)[0]
    ref = _t(z["scores"])
    assert float(((sc.cpu() - ref).abs() / ref.abs()).max()) <= 1e-3
    idx = ops.topk_select(sc, 10)
    assert torch.equal(idx.cpu(), _t(z["indices"]))
    ok, ov = torch.empty(1, 1, 2, 10, 128, device=dev), torch.empty(1, 1, 2, 10, 128, device=dev)
    ops.compact(_lib.dense_view(keys), _lib.dense_view(values), _lib.dense_view(ok), _lib.dense_view(ov), idx[None])
    assert np.array_equal(ok[0].cpu().numpy(), z["kept_keys"]) and np.array_equal(ov[0].cpu().numpy(), z["kept_values"])


@pytest.mark.gpu
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("reduction", ["mean", "sum"])
def test_snapkv_fixture(dev, causal, reduction):
    from fastcache_amd import _lib, ops
    from oracle import presses as opress
    z = _load("snapkv_bf16.npz")
    q, keys = _t(z["queries"], torch.bfloat16).to(dev), _t(z["keys"], torch.bfloat16).to(dev)
    ref = _t(z[f"scores_causal{int(causal)}_{reduction}"])
    sc = ops.snapkv_score(_lib.dense_view(keys), q[None], 16, 5, causal_window=causal, reduction=reduction)[0]
    torch.testing.assert_close(sc.cpu(), ref, rtol=1e-3, atol=1e-3 * float(ref.abs().mean()))
    idx = ops.topk_select(sc, 40).cpu().long()
    tie = opress.near_tie_rows(ref, 40)
    assert torch.equal(idx[~tie], _t(z[f"indices_causal{int(causal)}_{reduction}"]).long()[~tie])


@pytest.mark.gpu
def test_ccm_fixture(dev):
    """The module built after manual_seed(seed) has the reference's initial weights (same construction order); its
    GPU forward on the stored fp16 cache meets the stored oracle output."""
    from types import SimpleNamespace
    from fastcache_amd.utils_ccm import KVCacheLinearDecoupleCompressor
    z = _load("ccm_linear_decouple_fp16.npz")
    k, v = _t(z["keys"], torch.float16), _t(z["values"], torch.float16)
    torch.manual_seed(int(z["seed"]))
    cfg = SimpleNamespace(text_config=SimpleNamespace(num_hidden_layers=1, num_key_value_heads=2, hidden_size=256))
    m = KVCacheLinearDecoupleCompressor(cfg).to(dev).half().eval()
    (ck, cv), = m([(k.to(dev), v.to(dev))], [int(x) for x in z["it_len"]])
    for got, name in ((ck, "out_keys"), (cv, "out_values")):
        ref = _t(z[name], torch.float16).float()
        assert got.shape == ref.shape
        err = (got.cpu().float() - ref).abs()
        bound = 1e-3 * float(ref.abs().max()) + 2 * 2.0 ** -10 * ref.abs().clamp_min(float(ref.abs().max()) * 2.0 ** -14)
        assert bool((err <= bound).all())


@pytest.mark.gpu
def test_decode_attention_fixture(dev):
    from fastcache_amd import _lib, ops
    z = _load("decode_attention_fp16.npz")
    q = _t(z["q"], torch.float16).to(dev)
    kc, vc = _t(z["k_cache"], torch.float16).to(dev), _t(z["v_cache"], torch.float16).to(dev)
    lens, tables = _t(z["lens"]).to(dev), _t(z["tables"]).to(dev)
    max_len = tables.shape[1] * kc.shape[1]
    kview, vview = _lib.paged_view(kc[None], tables, None, max_len), _lib.paged_view(vc[None], tables, None, max_len)
    ws = ops.decode_attn_workspace(q.shape[0], q.shape[1], max_len, dev)
    out = ops.decode_attn(kview, vview, 0, q, lens, 128 ** -0.5, ws).cpu().float()
    ref = _t(z["out"], torch.float16).float()
    assert float((out - ref).abs().max()) <= 2e-2
