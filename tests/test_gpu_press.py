"""GPU parity: Knorm scoring, top-k selection and in-place paged compaction vs the CPU oracle."""
import pytest
import torch

from fastcache_amd import _lib, ops, synth
from oracle import paged as opaged
from oracle import presses as opress

pytestmark = pytest.mark.gpu


def _oracle_knorm_pool(case, ratio):
    """Reference path on the CPU: extract -> KnormPress (per head) -> write back, per sequence."""
    pool = case.kv_cache.clone()
    all_idx, all_scores = [], []
    for b, (tab, n) in enumerate(zip(case.block_tables, case.seq_lens)):
        kv = opaged.extract_kv(pool, tab, n)
        comp, idxs, scs = [], [], []
        for k, v in kv:
            sc = opress.knorm_score(k)
            ck, cv, idx = opress.press_compress(k, v, sc, ratio)
            comp.append((ck, cv)); idxs.append(idx[0]); scs.append(sc[0])
        opaged.write_back(pool, comp, tab)
        all_idx.append(torch.stack(idxs)); all_scores.append(torch.stack(scs))
    return pool, all_idx, all_scores


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [dict(num_layers=2, num_kv_heads=4, seq_len=700, batch=3),
                                   dict(num_layers=1, num_kv_heads=32, seq_len=1024, batch=1)])
def test_knorm_press_paged_inplace(dev, dtype, shape):
    case = synth.knorm_case(seed=3, dtype=dtype, **shape)
    ratio = 0.5
    ref_pool, ref_idx, ref_scores = _oracle_knorm_pool(case, ratio)

    pool = case.kv_cache.to(dev)
    tables, lens = case.table_tensor(dev), case.lens_tensor(dev)
    S = max(case.seq_lens)
    kview = _lib.paged_view(pool[0], tables, lens, S)
    vview = _lib.paged_view(pool[1], tables, lens, S)
    scores = ops.knorm_score(kview, dev)
    n = opress.n_kept_press(S, ratio)
    idx = ops.topk_select(scores, n)
    ops.compact(kview, vview, kview, vview, idx)
    torch.cuda.synchronize()

    # scores: 1e-3 relative (fp32 accumulation)
    n_tie = 0
    for b in range(len(case.seq_lens)):
        got = scores[:, b].cpu()
        torch.testing.assert_close(got, ref_scores[b], rtol=1e-3, atol=0)
        # indices: bit-exact outside near-ties (score gap below 1e-5 relative)
        tie = opress.near_tie_rows(ref_scores[b], n)
        gi = idx[:, b].cpu().long()
        assert torch.equal(gi[~tie], ref_idx[b][~tie])
        # a near-tie may swap only the two tied tokens
        for a, r in zip(gi[tie], ref_idx[b][tie]):
            assert len(set(a.tolist()) ^ set(r.tolist())) <= 2
        n_tie += int(tie.sum())
    assert n_tie <= 0.2 * idx[..., 0].numel()
    # gathered bytes and untouched slots: the whole pool is bit-identical to extract -> gather with
    # the selected indices -> write back
    exp_pool = case.kv_cache.clone()
    for b, (tab, sl) in enumerate(zip(case.block_tables, case.seq_lens)):
        kv = opaged.extract_kv(exp_pool, tab, sl)
        comp = [(opress.gather_tokens(k, idx[l, b].cpu().long()[None]),
                 opress.gather_tokens(v, idx[l, b].cpu().long()[None])) for l, (k, v) in enumerate(kv)]
        opaged.write_back(exp_pool, comp, tab)
    assert torch.equal(pool.cpu().view(torch.uint8), exp_pool.view(torch.uint8))
    if n_tie == 0:
        assert torch.equal(pool.cpu().view(torch.uint8), ref_pool.view(torch.uint8))


def _oracle_snapkv_scores(case, W, ksz, causal, reduction):
    """[L, B, Hkv, S] fp32 scores from the dense K of every sequence (all sequences share S)."""
    out = []
    for l in range(case.dense_k.shape[0]):
        out.append(opress.snapkv_score(case.queries[l], case.dense_k[l], W, ksz, causal, reduction))
    return torch.stack(out)


@pytest.mark.parametrize("cfg", [
    dict(num_layers=2, batch=2, num_q_heads=8, num_kv_heads=2, seq_len=300, window=64, ksz=7, dtype=torch.bfloat16),
    dict(num_layers=1, batch=1, num_q_heads=4, num_kv_heads=4, seq_len=257, window=32, ksz=5, dtype=torch.float16),
    dict(num_layers=1, batch=2, num_q_heads=14, num_kv_heads=2, seq_len=1000, window=64, ksz=7, dtype=torch.bfloat16),
    dict(num_layers=1, batch=1, num_q_heads=8, num_kv_heads=1, seq_len=100, window=64, ksz=3, dtype=torch.bfloat16),
    dict(num_layers=1, batch=1, num_q_heads=2, num_kv_heads=1, seq_len=520, window=48, ksz=7, dtype=torch.float16),
    # pages smaller than a key tile and pages whose size is no power of two: the per-row addressing path
    dict(num_layers=2, batch=2, num_q_heads=8, num_kv_heads=2, seq_len=333, window=64, ksz=7, dtype=torch.bfloat16,
         block_size=16),
    dict(num_layers=1, batch=2, num_q_heads=4, num_kv_heads=2, seq_len=400, window=32, ksz=5, dtype=torch.float16,
         block_size=48),
    # a group of 16 row blocks (the widest workgroup)
    dict(num_layers=1, batch=1, num_q_heads=8, num_kv_heads=1, seq_len=300, window=64, ksz=7, dtype=torch.bfloat16),
])
@pytest.mark.parametrize("causal,reduction", [(True, "mean"), (False, "sum")])
def test_snapkv_scores_and_selection(dev, cfg, causal, reduction):
    cfg = dict(cfg)
    ksz = cfg.pop("ksz")
    W = cfg["window"]
    case = synth.snapkv_case(seed=11, keep_dense=True, **cfg)
    ref = _oracle_snapkv_scores(case, W, ksz, causal, reduction)

    pool = case.kv_cache.to(dev)
    tables, lens = case.table_tensor(dev), case.lens_tensor(dev)
    S = max(case.seq_lens)
    kview = _lib.paged_view(pool[0], tables, lens, S)
    got = ops.snapkv_score(kview, case.queries.to(dev), W, ksz, causal_window=causal, reduction=reduction,
                           seq_lens=lens)
    torch.cuda.synchronize()
    got = got.cpu()
    # scores within 1e-3 relative (fp32 accumulation); tiny probabilities get an absolute floor
    torch.testing.assert_close(got, ref, rtol=1e-3, atol=1e-3 * float(ref.abs().mean()))

    # the same scores through a dense (HuggingFace-layout) view
    dense_k = case.dense_k.to(dev)          # keep alive: the view only holds its address
    dview = _lib.dense_view(dense_k)
    got_d = ops.snapkv_score(dview, case.queries.to(dev), W, ksz, causal_window=causal, reduction=reduction)
    assert torch.equal(got_d.cpu(), got)

    n = opress.n_kept_press(S, 0.75)
    if n > W:
        idx = ops.topk_select(got.to(dev), n).cpu().long()
        ref_idx = opress.topk_lowest_index(ref, n)
        tie = opress.near_tie_rows(ref[..., :S - W], n - W)
        assert torch.equal(idx[~tie], ref_idx[~tie])
        # the observation window always survives
        assert (idx[..., -W:] == torch.arange(S - W, S)).all()


@pytest.mark.parametrize("boost,where", [(18.0, 130), (30.0, 200), (60.0, 70), (30.0, 10)])
def test_snapkv_extreme_logits(dev, boost, where):
    """Logits that jump far above the running offset: the lazy-offset sweep must rescale (moderate
    jump) or fall back to the general update (jump that overflows fp32) and still match the oracle."""
    L, B, Hq, Hkv, S, W, ksz = 1, 2, 8, 2, 400, 64, 5
    case = synth.snapkv_case(seed=19, num_layers=L, batch=B, num_q_heads=Hq, num_kv_heads=Hkv, seq_len=S,
                             window=W, keep_dense=True)
    case.dense_k[:, :, :, where:where + 10] *= boost
    q = case.queries
    ref = torch.stack([opress.snapkv_score(q[l], case.dense_k[l], W, ksz, True, "sum") for l in range(L)])
    assert torch.isfinite(ref).all()
    dk = case.dense_k.to(dev)
    got = ops.snapkv_score(_lib.dense_view(dk), q.to(dev), W, ksz, causal_window=True, reduction="sum").cpu()
    assert torch.isfinite(got).all()
    torch.testing.assert_close(got, ref, rtol=1e-3, atol=1e-4 * float(ref.max()))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_tova_press(dev, dtype):
    """Last-query attention averaged over all heads (computed from the window query, or taken from given attention
    weights); scores <= 1e-3 relative, kept indices equal outside near-ties, the last token always kept."""
    from fastcache_amd.presses import TOVAPress
    from oracle import presses as opress
    g = torch.Generator().manual_seed(3)
    B, Hq, Hkv, S, D = 2, 8, 2, 700, 128
    q = torch.randn(B, Hq, 1, D, generator=g).to(dtype)
    k = torch.randn(B, Hkv, S, D, generator=g).to(dtype)
    v = torch.randn(B, Hkv, S, D, generator=g).to(dtype)
    press = TOVAPress(compression_ratio=0.6)
    sc = press.score(None, None, k.to(dev), v.to(dev), None, {"queries": q.to(dev)})
    ref = opress.tova_score(q, k)
    assert sc.shape == (B, Hkv, S)
    assert float(((sc.cpu() - ref).abs() / ref.abs().clamp_min(1e-12)).max()) <= 1e-3
    ck, cv = press.compress(None, None, k.to(dev), v.to(dev), None, {"queries": q.to(dev)})
    n = int(S * 0.4)
    assert ck.shape == (B, Hkv, n, D)
    idx = opress.topk_lowest_index(sc.cpu(), n)
    assert bool((idx[..., -1] == S - 1).all())
    assert torch.equal(ck.cpu(), opress.gather_tokens(k, idx)) and torch.equal(cv.cpu(), opress.gather_tokens(v, idx))
    # attention weights handed in by the model
    attn = torch.softmax(torch.randn(B, Hq, 5, S, generator=g), -1)
    sc2 = press.score(None, None, k.to(dev), v.to(dev), attn.to(dev), {})
    assert torch.allclose(sc2.cpu(), opress.tova_score(None, k, attentions=attn), rtol=1e-6, atol=0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,Hq,Hkv,S", [(2, 8, 2, 300), (1, 4, 4, 1025), (1, 2, 1, 64)])
def test_observed_attention_press(dev, dtype, B, Hq, Hkv, S):
    from fastcache_amd.presses import ObservedAttentionPress
    from oracle import presses as opress
    g = torch.Generator().manual_seed(S)
    attn = torch.softmax(torch.randn(B, Hq, S, S, generator=g) + torch.triu(torch.full((S, S), -1e9), 1), -1).to(dtype)
    k = torch.zeros(B, Hkv, S, 128, dtype=torch.float16)
    sc = ObservedAttentionPress(0.5).score(None, None, k.to(dev), k.to(dev), attn.to(dev), {})
    ref = opress.observed_attention_score(attn, Hkv)
    assert sc.shape == (B, Hkv, S) and sc.dtype == torch.float32
    assert float(((sc.cpu() - ref).abs() / ref.abs().clamp_min(1e-12)).max()) <= 1e-3
    with pytest.raises(AssertionError):
        ObservedAttentionPress(0.5).score(None, None, k.to(dev), k.to(dev), None, {})


@pytest.mark.parametrize("S", [17, 33, 64, 65, 127, 128, 129, 192, 193, 255, 256, 257, 320, 321, 449])
@pytest.mark.parametrize("W,ksz", [(16, 5), (1, 1), (33, 31)])
def test_snapkv_short_sequences_and_tile_boundaries(dev, S, W, ksz):
    """Sequence lengths around every key-tile boundary of the first five tiles (prologue, steady state and drain of
    the tile pipeline), windows that are not multiples of 32, widest pooling kernels."""
    if S <= W:
        pytest.skip("needs S > W")
    case = synth.snapkv_case(seed=S + W, num_layers=1, batch=2, num_q_heads=4, num_kv_heads=2, seq_len=S, window=W,
                             keep_dense=True, dtype=torch.bfloat16)
    ref = _oracle_snapkv_scores(case, W, ksz, True, "sum")
    dk = case.dense_k.to(dev)
    got = ops.snapkv_score(_lib.dense_view(dk), case.queries.to(dev), W, ksz, causal_window=True, reduction="sum").cpu()
    torch.testing.assert_close(got, ref, rtol=1e-3, atol=1e-3 * float(ref.abs().mean()))
    pool = case.kv_cache.to(dev)
    tables, lens = case.table_tensor(dev), case.lens_tensor(dev)
    got_p = ops.snapkv_score(_lib.paged_view(pool[0], tables, lens, S), case.queries.to(dev), W, ksz,
                             causal_window=True, reduction="sum", seq_lens=lens).cpu()
    assert torch.equal(got_p, got)
