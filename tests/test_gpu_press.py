"""GPU parity: Knorm scoring, top-k selection and in-place paged compaction vs the CPU oracle."""
import pytest
import torch

from fastcache_amd import _lib, ops, paged_press, synth
from fastcache_amd.presses import SimLayerKVPress, ThinKPress
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


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("lens,block_size,keep", [
    ([700, 512, 1], 256, [350, 256, 0]),          # ragged, a sequence that keeps nothing
    ([1024], 256, [512]),                         # the shape of the first configuration, one sequence
    ([300, 300], 64, [300, 299]),                 # keep everything / all but one
    ([2500, 130, 2049], 128, [1, 129, 700]),      # several pages, a single kept row
    ([193, 77], 48, [100, 33]),                   # pages whose size is not a power of two
    ([20000, 9000], 256, [5000, 2250]),           # long sequences: 100 KB of LDS per column
])
def test_knorm_press_one_launch_equals_three(dev, dtype, lens, block_size, keep):
    """fc_knorm_press against fc_knorm_score + fc_topk_select + fc_compact on the same pool: scores, indices and
    every byte of both planes identical (ties included: both run the same selection)."""
    case = synth.make_paged_case(seed=11, num_layers=2, batch=len(lens), num_kv_heads=3, seq_lens=lens, dtype=dtype,
                                 outlier_channels=4, block_size=block_size)
    # equal rows inside a column: ties that the selection has to break by position
    pool_a = case.kv_cache.to(dev)
    t0 = case.block_tables[0]
    pool_a[0, :, t0[0], 5] = pool_a[0, :, t0[0], 2]
    pool_a[0, :, t0[0], 9] = pool_a[0, :, t0[0], 2]
    pool_b = pool_a.clone()
    tables, lens_d = case.table_tensor(dev), case.lens_tensor(dev)
    S, width = max(lens), max(keep)
    n_kept = torch.tensor(keep, dtype=torch.int32, device=dev)

    ka, va = (_lib.paged_view(pool_a[p], tables, lens_d, S) for p in range(2))
    scores_a = ops.knorm_score(ka, dev)
    idx_a = ops.topk_select(scores_a, width, row_lens=lens_d, n_kept=n_kept, rows_per_len=3)
    ops.compact(ka, va, ka, va, idx_a, n_kept=n_kept)

    kb, vb = (_lib.paged_view(pool_b[p], tables, lens_d, S) for p in range(2))
    scores_b, idx_b = ops.knorm_press(kb, vb, width, dev, n_kept=n_kept)
    torch.cuda.synchronize()
    assert torch.equal(scores_a.view(torch.int32), scores_b.view(torch.int32))
    assert torch.equal(idx_a, idx_b)
    assert torch.equal(pool_a.view(torch.uint8), pool_b.view(torch.uint8))
    # and something did move
    assert not torch.equal(pool_b.view(torch.uint8), case.kv_cache.to(dev).view(torch.uint8)) or width == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("lens,block_size,keep", [
    ([700, 512, 3], 256, [350, 256, 0]),
    ([4096], 256, [1024]),
    ([300, 300], 64, [300, 299]),
    ([2500, 130, 2049], 128, [1, 129, 700]),
    ([193, 77], 48, [100, 33]),
    ([30000, 12345], 256, [4000, 1700]),
])
def test_select_compact_one_launch_equals_two(dev, dtype, lens, block_size, keep):
    """fc_select_compact against fc_topk_select + fc_compact on the same pool and the same scores (random, with
    repeated values and -inf past each sequence's end): indices and every byte of both planes identical."""
    H = 3
    case = synth.make_paged_case(seed=12, num_layers=2, batch=len(lens), num_kv_heads=H, seq_lens=lens, dtype=dtype,
                                 block_size=block_size)
    pool_a = case.kv_cache.to(dev)
    pool_b = pool_a.clone()
    tables, lens_d = case.table_tensor(dev), case.lens_tensor(dev)
    S, width = max(lens), max(keep)
    g = torch.Generator().manual_seed(3)
    scores = torch.randn((2, len(lens), H, S), generator=g)
    scores[..., ::7] = 0.25                                   # many equal scores: the tie-break decides
    for b, n in enumerate(lens):
        scores[:, b, :, n:] = float("-inf")
    scores = scores.to(dev)
    n_kept = torch.tensor(keep, dtype=torch.int32, device=dev)
    ka, va = (_lib.paged_view(pool_a[p], tables, lens_d, S) for p in range(2))
    idx_a = ops.topk_select(scores, width, row_lens=lens_d, n_kept=n_kept, rows_per_len=H)
    ops.compact(ka, va, ka, va, idx_a, n_kept=n_kept)
    kb, vb = (_lib.paged_view(pool_b[p], tables, lens_d, S) for p in range(2))
    idx_b = ops.select_compact(kb, vb, scores, width, n_kept=n_kept)
    torch.cuda.synchronize()
    assert torch.equal(idx_a, idx_b)
    assert torch.equal(pool_a.view(torch.uint8), pool_b.view(torch.uint8))
    if len(set(keep)) == 1 and len(set(lens)) == 1:           # the form without per-sequence counts
        pool_c = case.kv_cache.to(dev)
        kc, vc = (_lib.paged_view(pool_c[p], tables, lens_d, S) for p in range(2))
        idx_c = ops.select_compact(kc, vc, scores, width)
        assert torch.equal(idx_c, ops.topk_select(scores, width))
        assert torch.equal(pool_c.view(torch.uint8), pool_a.view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("lens,Hq,H,W,ksz,keep,given_lse", [
    ([1000, 1000], 8, 2, 64, 7, [250, 250], False),         # 8 query blocks per kv head, equal lengths
    ([700, 512, 20, 300], 8, 2, 32, 5, [175, 128, 5, 75], False),    # ragged, one sequence shorter than the window
    ([2048], 28, 4, 64, 7, [512], False),                   # 14 blocks: 16 wavefronts
    ([900, 333], 4, 1, 32, 1, [225, 83], True),             # 4 blocks, log-sum-exp given, no pooling
    ([4096], 8, 2, 64, 7, [1024], False),                   # the second configuration's column
])
def test_snapkv_press_one_launch_equals_separate(dev, dtype, lens, Hq, H, W, ksz, keep, given_lse):
    """fc_snapkv_press against fc_snapkv_score + fc_snapkv_fill_window + fc_topk_select + fc_compact: the same
    kernel code scores, so scores (window fill included), indices and every cache byte must be identical."""
    L = 2
    case = synth.make_paged_case(seed=21, num_layers=L, batch=len(lens), num_kv_heads=H, seq_lens=lens, dtype=dtype,
                                 num_q_heads=Hq, window=W)
    pool_a = case.kv_cache.to(dev)
    pool_b = pool_a.clone()
    tables, lens_d, q = case.table_tensor(dev), case.lens_tensor(dev), case.queries.to(dev)
    S, width = max(lens), max(keep)
    n_kept = torch.tensor(keep, dtype=torch.int32, device=dev)
    ka, va = (_lib.paged_view(pool_a[p], tables, lens_d, S) for p in range(2))
    lse = None
    if given_lse:
        lse = torch.empty((L, len(lens), Hq, W), dtype=torch.float32, device=dev)
        for l in range(L):
            for b, n in enumerate(lens):
                kd = opaged.extract_kv(case.kv_cache[:, l:l + 1], case.block_tables[b], n)[0][0][0].float()   # [H, n, D]
                logits = torch.matmul(case.queries[l, b].float(), kd.repeat_interleave(Hq // H, 0).transpose(1, 2))
                mask = torch.triu(torch.full((W, n), float("-inf")), diagonal=n - W + 1) if n >= W else torch.zeros(W, n)
                lse[l, b] = torch.logsumexp(logits * 128 ** -0.5 + mask, dim=-1).to(dev)
    assert ops.snapkv_press_fits(ka, Hq, W, width)
    scores_a = ops.snapkv_score(ka, q, W, ksz, True, "sum", seq_lens=lens_d, lse=lse, splits=1)
    idx_a = ops.topk_select(scores_a, width, row_lens=lens_d, n_kept=n_kept, rows_per_len=H)
    ops.compact(ka, va, ka, va, idx_a, n_kept=n_kept)
    kb, vb = (_lib.paged_view(pool_b[p], tables, lens_d, S) for p in range(2))
    scores_b, idx_b = ops.snapkv_press(kb, vb, q, W, ksz, width, True, "sum", seq_lens=lens_d, lse=lse, n_kept=n_kept)
    torch.cuda.synchronize()
    assert torch.equal(scores_a.view(torch.int32), scores_b.view(torch.int32))
    assert torch.equal(idx_a, idx_b)
    assert torch.equal(pool_a.view(torch.uint8), pool_b.view(torch.uint8))
    assert not torch.equal(pool_b.view(torch.uint8), case.kv_cache.to(dev).view(torch.uint8))


@pytest.mark.parametrize("period,keep", [(50, [600, 300]), (7, [1100, 300]), (256, [70, 650])])
def test_snapkv_press_exact_ties_from_periodic_keys(dev, period, keep):
    """Keys that repeat with a period give bit-identical scores period apart (same logits, same exponentials, same
    pooled neighbourhoods), so every row is full of exact ties, among them the threshold's: the one-launch press
    (selection over register-held keys) and the separate launches (the stand-alone top-k kernel) must both keep the
    lowest positions of a tie, and both must equal the stable selection on the kernel's own scores.  (Kept counts are
    chosen so that the threshold does not fall into the group of keys that tie with the row's LARGEST score: there the
    two forms differ by design, the filled window ties with those keys in the separate launches and outranks them in
    the one launch.)"""
    dtype, L, H, G, W, ksz, lens = torch.bfloat16, 2, 2, 2, 32, 5, [1500, 700]
    B, S = len(lens), max(lens)
    g = torch.Generator().manual_seed(period)
    base = torch.randn(L, B, H, period, 128, generator=g)
    reps = -(-S // period)
    dense_k = base.repeat(1, 1, 1, reps, 1)[:, :, :, :S].to(dtype)
    dense_v = torch.randn(L, B, H, S, 128, generator=g).to(dtype)
    q = torch.randn(L, B, H * G, W, 128, generator=g).to(dtype)
    need = [-(-n // 256) for n in lens]
    tables = [list(range(sum(need[:b]), sum(need[:b + 1]))) for b in range(B)]
    pool = torch.zeros(2, L, sum(need), 256, H, 128, dtype=dtype)
    for l in range(L):
        synth.scatter_into_pool(pool, 0, l, dense_k[l], tables, lens)
        synth.scatter_into_pool(pool, 1, l, dense_v[l], tables, lens)
    pa = pool.to(dev)
    pb = pa.clone()
    tt = torch.tensor([t + [-1] * (max(need) - len(t)) for t in tables], dtype=torch.int32, device=dev)
    ll = torch.tensor(lens, dtype=torch.int32, device=dev)
    nk = torch.tensor(keep, dtype=torch.int32, device=dev)
    qd, width = q.to(dev), max(keep)
    ka, va = (_lib.paged_view(pa[p], tt, ll, S) for p in range(2))
    sa = ops.snapkv_score(ka, qd, W, ksz, True, "sum", seq_lens=ll, splits=1)
    ia = ops.topk_select(sa, width, row_lens=ll, n_kept=nk, rows_per_len=H)
    ops.compact(ka, va, ka, va, ia, n_kept=nk)
    kb, vb = (_lib.paged_view(pb[p], tt, ll, S) for p in range(2))
    assert ops.snapkv_press_fits(kb, H * G, W, width)
    sb, ib = ops.snapkv_press(kb, vb, qd, W, ksz, width, True, "sum", seq_lens=ll, n_kept=keep, host_lens=lens)
    torch.cuda.synchronize()
    assert torch.equal(sa.view(torch.int32), sb.view(torch.int32))
    assert torch.equal(ia, ib)
    assert torch.equal(pa.view(torch.uint8), pb.view(torch.uint8))
    for b, n in enumerate(lens):
        row = sb[:, b, :, :n].cpu()
        body = row[..., ksz:n - W - ksz - period]                         # away from the zero-padded borders
        shifted = row[..., ksz + period:n - W - ksz]
        assert bool((body == shifted).all()), "the scores are not periodic: the test lost its ties"
        want = opress.topk_lowest_index(row, keep[b])
        assert torch.equal(ib[:, b, :, :keep[b]].cpu().long(), want)
        kth = row.gather(-1, want).min(-1).values
        assert bool(((row == kth[..., None]).sum(-1) > 1).all()), "no tie at the threshold"


def test_snapkv_paged_press_tiny_scored_part_takes_separate_launches(dev):
    """Six scored keys under a pooling kernel of 13: every pooled score is the same and equals the layer's largest, so
    after the window fill all 38 positions tie and the lowest indices win (position 37, a window position, is the one
    dropped).  The one-launch press ranks the window first and would drop a scored key instead; the host sends such
    rows through the separate launches."""
    L, H, Hq, W, ksz, n = 2, 1, 4, 32, 13, 38
    case = synth.make_paged_case(seed=523480996, num_layers=L, batch=1, num_kv_heads=H, seq_lens=[n], dtype=torch.bfloat16,
                                 num_q_heads=Hq, window=W, block_size=64)
    pool = case.kv_cache.to(dev)
    res = paged_press.snapkv_compress_paged(pool, case.table_tensor(dev), case.lens_tensor(dev), n, case.queries.to(dev),
                                            1.0 - 37.5 / 38, W, ksz, True, "sum")
    torch.cuda.synchronize()
    assert res.n_kept == 37
    scored = res.scores[..., :n - W]
    assert bool((scored == scored[..., :1]).all())                       # the degenerate tie is really there
    assert torch.equal(res.indices[0, 0, 0].cpu(), torch.arange(37, dtype=torch.int32))


def test_snapkv_press_refuses_what_it_cannot_take(dev):
    case = synth.make_paged_case(seed=2, num_layers=1, batch=1, num_kv_heads=1, seq_lens=[512], dtype=torch.bfloat16,
                                 num_q_heads=4, window=64)
    pool = case.kv_cache.to(dev)
    tables, lens_d, q = case.table_tensor(dev), case.lens_tensor(dev), case.queries.to(dev)
    kv, vv = (_lib.paged_view(pool[p], tables, lens_d, 512) for p in range(2))
    with pytest.raises(_lib.FastcacheError, match="exceed the window"):
        ops.snapkv_press(kv, vv, q, 64, 7, 64)                 # a kept count that does not exceed the window
    # ragged counts given as Python ints are checked on the host: one entry at the window is refused before any launch
    two = synth.make_paged_case(seed=3, num_layers=1, batch=2, num_kv_heads=1, seq_lens=[512, 300], dtype=torch.bfloat16,
                                num_q_heads=4, window=64)
    pool2 = two.kv_cache.to(dev)
    tables2, lens2, q2 = two.table_tensor(dev), two.lens_tensor(dev), two.queries.to(dev)
    k2, v2 = (_lib.paged_view(pool2[p], tables2, lens2, 512) for p in range(2))
    with pytest.raises(_lib.FastcacheError, match=r"offending sequences: \[1\]"):
        ops.snapkv_press(k2, v2, q2, 64, 7, 128, seq_lens=lens2, n_kept=[128, 64], host_lens=[512, 300])
    assert torch.equal(pool2, two.kv_cache.to(dev))
    ops.snapkv_press(k2, v2, q2, 64, 7, 128, seq_lens=lens2, n_kept=[128, 75], host_lens=[512, 300])
    torch.cuda.synchronize()
    long = synth.make_paged_case(seed=2, num_layers=1, batch=1, num_kv_heads=1, seq_lens=[20000], dtype=torch.bfloat16,
                                 num_q_heads=4, window=64)
    pool = long.kv_cache.to(dev)
    kv, vv = (_lib.paged_view(pool[p], long.table_tensor(dev), long.lens_tensor(dev), 20000) for p in range(2))
    assert not ops.snapkv_press_fits(kv, 4, 64, 5000)
    with pytest.raises(_lib.FastcacheError, match="fc_select_compact"):
        ops.snapkv_press(kv, vv, long.queries.to(dev), 64, 7, 5000)


def test_knorm_press_one_launch_limits_and_clamps(dev):
    """Sequences beyond 8192 tokens are refused by name; a kept count in device memory larger than the sequence or
    the index row is clamped; a dense view works like a paged one."""
    L, B, H, S = 1, 2, 2, 96
    g = torch.Generator().manual_seed(5)
    k = torch.randn((L, B, H, S, 128), generator=g).to(dev)
    v = torch.randn((L, B, H, S, 128), generator=g).to(dev)
    k2, v2 = k.clone(), v.clone()
    n_kept = torch.tensor([10_000, 40], dtype=torch.int32, device=dev)      # first one far too large
    lens_d = torch.tensor([S, 50], dtype=torch.int32, device=dev)
    def views(kt, vt):
        out = (_lib.dense_view(kt), _lib.dense_view(vt))
        for view in out:
            view.seq_lens = lens_d.data_ptr()
        return out
    ka, va = views(k, v)
    sa = ops.knorm_score(ka, dev)
    ia = ops.topk_select(sa, 64, row_lens=lens_d, n_kept=n_kept, rows_per_len=H)
    ops.compact(ka, va, ka, va, ia, n_kept=n_kept)
    kb, vb = views(k2, v2)
    sb, ib = ops.knorm_press(kb, vb, 64, dev, n_kept=n_kept)
    torch.cuda.synchronize()
    assert torch.equal(sa.view(torch.int32), sb.view(torch.int32)) and torch.equal(ia, ib)
    assert torch.equal(k, k2) and torch.equal(v, v2)
    row = ib[0, 0, 0]                                                        # 10 000 asked for: clamped to the 64 of the row
    assert (row >= 0).all() and (row < S).all() and (row[1:] > row[:-1]).all()
    row = ib[0, 1, 1]
    assert (row[:40] >= 0).all() and (row[:40] < 50).all() and (row[40:] == -1).all()
    big = torch.zeros((1, 1, 1, 40000, 128), device=dev)
    assert not ops.press_column_fits(40000, 10) and ops.press_column_fits(32768, 4096)
    with pytest.raises(_lib.FastcacheError, match="separate launches"):
        ops.knorm_press(_lib.dense_view(big), _lib.dense_view(big.clone()), 10, dev)


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


def _ea_case(seed, B, Hq, Hkv, S, dtype):
    g = torch.Generator().manual_seed(seed)
    k = torch.randn(B, Hkv, S, 128, generator=g).to(dtype)
    v = (torch.randn(B, Hkv, S, 128, generator=g) * torch.rand(B, Hkv, S, 1, generator=g) * 2).to(dtype)
    mu = torch.randn(B, Hq, 128, generator=g) * 0.5
    a = torch.randn(B, Hq, 128, 128, generator=g) / 128 ** 0.5
    cov = a @ a.transpose(-1, -2) * 0.5                      # symmetric positive semi-definite
    return k, v, mu, cov


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,Hq,Hkv,S", [(2, 8, 2, 700), (1, 4, 4, 2500), (1, 14, 2, 100), (2, 2, 2, 37)])
@pytest.mark.parametrize("use_cov,use_vnorm,eps", [(True, True, 0.0), (False, True, 0.02), (True, False, 0.0)])
def test_expected_attention_scores(dev, dtype, B, Hq, Hkv, S, use_cov, use_vnorm, eps):
    """fc_expected_attention_score vs the oracle: scores <= 1e-3 relative (fp32 on both sides; the covariance is
    split into two 16-bit halves on the device), sinks carry the layer maximum."""
    from oracle import presses as opress
    k, v, mu, cov = _ea_case(S + Hq, B, Hq, Hkv, S, dtype)
    ref = opress.expected_attention_score(k, v, mu, cov if use_cov else None, 4, use_vnorm, eps)
    kd, vd = k.to(dev), v.to(dev)                            # the views hold raw pointers: keep the tensors alive
    got = ops.expected_attention_score(_lib.dense_view(kd), _lib.dense_view(vd), mu.to(dev),
                                       cov.to(dev) if use_cov else None, 4, use_vnorm, eps)[0].cpu()
    assert got.shape == (B, Hkv, S)
    assert float(((got - ref).abs() / ref.abs().clamp_min(1e-9)).max()) <= 1e-3
    assert bool((got[..., :4] == got.max()).all())


def test_expected_attention_paged_ragged_and_layers(dev):
    """Paged pool, two layers, ragged lengths: every (layer, sequence) equals the dense single-layer call; entries past
    a sequence's length are -inf; the sink value is the layer's own maximum."""
    dtype, L, Hq, Hkv, lens = torch.bfloat16, 2, 8, 2, [300, 40, 513]
    B, S = len(lens), max(lens)
    case = synth.make_paged_case(seed=9, num_layers=L, batch=B, num_kv_heads=Hkv, seq_lens=lens, dtype=dtype,
                                 keep_dense=True)
    g = torch.Generator().manual_seed(4)
    mu = torch.randn(L, B, Hq, 128, generator=g) * 0.5
    a = torch.randn(L, B, Hq, 128, 128, generator=g) / 128 ** 0.5
    cov = a @ a.transpose(-1, -2) * 0.5
    pool, tab, lens_d = case.kv_cache.to(dev), case.table_tensor(dev), case.lens_tensor(dev)
    kview, vview = (_lib.paged_view(pool[i], tab, lens_d, S) for i in range(2))
    got = ops.expected_attention_score(kview, vview, mu.to(dev), cov.to(dev), 4, True, 0.0).cpu()
    assert got.shape == (L, B, Hkv, S)
    from oracle import presses as opress
    for l in range(L):
        per_seq = [opress.expected_attention_score(case.dense_k[l][b:b + 1, :, :n], case.dense_v[l][b:b + 1, :, :n],
                                                   mu[l, b:b + 1], cov[l, b:b + 1], 4, True, 0.0)[0] for b, n in enumerate(lens)]
        layer_max = max(float(p[:, 4:].max()) for p in per_seq)
        for b, n in enumerate(lens):
            ref = per_seq[b].clone()
            ref[:, :4] = layer_max                       # one batched call shares the sink value across its sequences
            assert float(((got[l, b, :, :n] - ref).abs() / ref.abs().clamp_min(1e-9)).max()) <= 1e-3
            assert bool(torch.isinf(got[l, b, :, n:]).all()) and bool((got[l, b, :, n:] < 0).all())


def test_expected_attention_press_from_module(dev):
    """The press end to end on a stand-in attention module: query statistics from q_proj and the future rotary
    angles (torch on the device) vs the oracle's statistics, then scores and the kept rows."""
    from types import SimpleNamespace
    from fastcache_amd.presses import ExpectedAttentionPress
    from oracle import presses as opress
    g = torch.Generator().manual_seed(8)
    B, S, hidden, Hq, Hkv, D = 2, 260, 256, 4, 2, 128
    q_proj = torch.nn.Linear(hidden, Hq * D, bias=False)
    with torch.no_grad():
        q_proj.weight.copy_(torch.randn(Hq * D, hidden, generator=g) / hidden ** 0.5)
    module = SimpleNamespace(config=SimpleNamespace(num_attention_heads=Hq, rope_theta=10000.0), head_dim=D,
                             q_proj=q_proj.to(dev))
    hs = torch.randn(B, S, hidden, generator=g).bfloat16()
    k = torch.randn(B, Hkv, S, D, generator=g).bfloat16()
    v = torch.randn(B, Hkv, S, D, generator=g).bfloat16()
    press = ExpectedAttentionPress(compression_ratio=0.5, n_future_positions=64)
    mu, cov = press.get_query_statistics(module, hs.to(dev))
    ang = torch.arange(S, S + 64, dtype=torch.float32)[:, None] * (1.0 / (10000.0 ** (torch.arange(0, D, 2).float() / D)))[None]
    cos, sin = torch.cat((ang, ang), -1).cos(), torch.cat((ang, ang), -1).sin()
    rmu, rcov = opress.expected_attention_query_statistics(hs, q_proj.weight.detach().cpu(), Hq, D, cos, sin, 4)
    torch.testing.assert_close(mu.cpu(), rmu, rtol=2e-3, atol=2e-3)
    torch.testing.assert_close(cov.cpu(), rcov, rtol=2e-3, atol=2e-3)
    sc = press.score(module, hs.to(dev), k.to(dev), v.to(dev), None, {})
    ref = opress.expected_attention_score(k, v, mu.cpu(), cov.cpu(), 4, True, 0.0)     # same statistics on both sides
    assert float(((sc.cpu() - ref).abs() / ref.abs().clamp_min(1e-9)).max()) <= 1e-3
    ck, cv = press.compress(module, hs.to(dev), k.to(dev), v.to(dev), None, {})
    idx = opress.topk_lowest_index(sc.cpu(), S // 2)
    assert bool((idx[..., :4] == torch.arange(4)).all())                                # sinks are kept
    assert torch.equal(ck.cpu(), opress.gather_tokens(k, idx)) and torch.equal(cv.cpu(), opress.gather_tokens(v, idx))


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


def test_expected_attention_edge_cases(dev):
    """No sinks; a single scored key; a sequence not longer than the sinks next to a normal one; mean only."""
    from oracle import presses as opress
    k, v, mu, cov = _ea_case(3, 1, 2, 2, 9, torch.float16)
    kd, vd = k.to(dev), v.to(dev)
    for n_sink, use_cov in ((0, True), (8, True), (4, False)):
        ref = opress.expected_attention_score(k, v, mu, cov if use_cov else None, n_sink, True, 0.0)
        got = ops.expected_attention_score(_lib.dense_view(kd), _lib.dense_view(vd), mu.to(dev),
                                           cov.to(dev) if use_cov else None, n_sink, True, 0.0)[0].cpu()
        assert float(((got - ref).abs() / ref.abs().clamp_min(1e-9)).max()) <= 1e-3, (n_sink, use_cov)
    # ragged paged batch: sequence 1 has fewer tokens than sinks -> all its tokens carry the layer maximum
    lens = [40, 3]
    case = synth.make_paged_case(seed=2, num_layers=1, batch=2, num_kv_heads=2, seq_lens=lens, dtype=torch.bfloat16,
                                 keep_dense=True)
    g = torch.Generator().manual_seed(1)
    mu2 = torch.randn(1, 2, 4, 128, generator=g) * 0.3
    pool, tab, lens_d = case.kv_cache.to(dev), case.table_tensor(dev), case.lens_tensor(dev)
    got = ops.expected_attention_score(_lib.paged_view(pool[0], tab, lens_d, 40), _lib.paged_view(pool[1], tab, lens_d, 40),
                                       mu2.to(dev), None, 4, True, 0.0)[0].cpu()
    ref0 = opress.expected_attention_score(case.dense_k[0][0:1], case.dense_v[0][0:1], mu2[0, 0:1], None, 4, True, 0.0)[0]
    assert float(((got[0] - ref0).abs() / ref0.abs().clamp_min(1e-9)).max()) <= 1e-3
    assert bool((got[1, :, :3] == ref0.max()).all()) and bool(torch.isinf(got[1, :, 3:]).all())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("Hq,Hkv,S,W,ksz,causal,bs", [(8, 2, 700, 64, 7, True, 256), (4, 4, 333, 32, 5, False, 256),
                                                       (14, 2, 1000, 48, 3, True, 48), (2, 1, 65, 16, 1, True, 256)])
def test_snapkv_scores_from_given_log_sum_exp(dev, dtype, Hq, Hkv, S, W, ksz, causal, bs):
    """With the log-sum-exp of the window queries handed in (what the prefill's attention kernel returns), the
    single-pass variant gives the scores of the two-pass kernel and of the oracle."""
    L, B = 2, 2
    case = synth.snapkv_case(seed=S, num_layers=L, batch=B, num_q_heads=Hq, num_kv_heads=Hkv, seq_len=S, window=W,
                             keep_dense=True, dtype=dtype, block_size=bs)
    G = Hq // Hkv
    lse = torch.empty(L, B, Hq, W)
    for l in range(L):
        logits = torch.matmul(case.queries[l].float(), case.dense_k[l].float().repeat_interleave(G, 1).transpose(2, 3)) / 128 ** 0.5
        if causal:
            logits = logits + torch.triu(torch.full((W, S), float("-inf")), diagonal=S - W + 1)
        lse[l] = torch.logsumexp(logits, dim=-1)
    pool, tab, lens = case.kv_cache.to(dev), case.table_tensor(dev), case.lens_tensor(dev)
    kview = _lib.paged_view(pool[0], tab, lens, S)
    q = case.queries.to(dev)
    two_pass = ops.snapkv_score(kview, q, W, ksz, causal_window=causal, reduction="sum", seq_lens=lens).cpu()
    one_pass = ops.snapkv_score(kview, q, W, ksz, causal_window=causal, reduction="sum", seq_lens=lens, lse=lse.to(dev)).cpu()
    ref = _oracle_snapkv_scores(case, W, ksz, causal, "sum")
    tol = 1e-3 * float(ref.abs().mean())
    torch.testing.assert_close(one_pass, ref, rtol=1e-3, atol=tol)
    torch.testing.assert_close(one_pass, two_pass, rtol=2e-4, atol=tol)
    with pytest.raises(_lib.FastcacheError):
        ops.snapkv_score(kview, q, W, ksz, lse=lse[..., :-1].to(dev))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("Hq,Hkv,S,W,ksz,causal,splits", [(8, 2, 2000, 64, 7, True, 3), (8, 2, 2000, 64, 7, True, 31),
                                                           (14, 2, 1500, 48, 15, False, 4), (4, 1, 700, 64, 5, True, 2),
                                                           (16, 4, 1100, 32, 63, True, 5)])
def test_snapkv_split_columns(dev, dtype, Hq, Hkv, S, W, ksz, causal, splits):
    """Columns cut into key ranges (one workgroup each, for launches with few columns): same scores as one workgroup
    per column and as the oracle, ragged lengths included; more pieces than tiles leaves some pieces empty."""
    L, lens = 2, [S, S - 517, 65]
    B = len(lens)
    case = synth.make_paged_case(seed=S + splits, num_layers=L, batch=B, num_kv_heads=Hkv, seq_lens=lens, dtype=dtype,
                                 num_q_heads=Hq, window=W, keep_dense=True)
    pool, tab, lens_d = case.kv_cache.to(dev), case.table_tensor(dev), case.lens_tensor(dev)
    kview = _lib.paged_view(pool[0], tab, lens_d, S)
    q = case.queries.to(dev)
    whole = ops.snapkv_score(kview, q, W, ksz, causal_window=causal, reduction="sum", seq_lens=lens_d, splits=1).cpu()
    cut = ops.snapkv_score(kview, q, W, ksz, causal_window=causal, reduction="sum", seq_lens=lens_d, splits=splits).cpu()
    for l in range(L):
        for b, n in enumerate(lens):
            if n <= W:
                continue
            ref = opress.snapkv_score(case.queries[l, b:b + 1], case.dense_k[l][b:b + 1, :, :n], W, ksz, causal, "sum")[0]
            tol = 1e-3 * float(ref[:, :n - W].abs().mean())
            # the window entries hold the layer's maximum over all sequences: compared between the two device paths only
            torch.testing.assert_close(cut[l, b, :, :n - W], ref[:, :n - W], rtol=1e-3, atol=tol)
            torch.testing.assert_close(cut[l, b, :, :n], whole[l, b, :, :n], rtol=2e-4, atol=tol)
            assert bool(torch.isinf(cut[l, b, :, n:]).all())


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,Hq,Hkv,S,W,ratio", [(2, 8, 2, 700, 32, 0.5), (1, 4, 4, 33, 16, 0.25), (3, 6, 3, 1300, 8, 0.9)])
def test_think_press_channel_energy_and_pruning(dev, dtype, B, Hq, Hkv, S, W, ratio):
    """ThinK: channel energies of K within fp32 summation error of the float64 oracle; the pruned channel set equals
    the oracle's wherever the channel scores are not within 1e-5 (relative) of the selection threshold; pruned
    channels are zero for every token, every other element and V are untouched bit for bit."""
    g = torch.Generator().manual_seed(S + W)
    k = (torch.randn(B, Hkv, S, 128, generator=g) * torch.linspace(0.2, 2.0, 128)).to(dtype)
    v = torch.randn(B, Hkv, S, 128, generator=g).to(dtype)
    q = torch.randn(B, Hq, W, 128, generator=g).to(dtype)
    kd, vd = k.to(dev), v.to(dev)
    energy = ops.key_channel_energy(_lib.dense_view(kd), dev)[0].cpu()
    torch.testing.assert_close(energy.double(), k.double().pow(2).sum(2), rtol=1e-5, atol=1e-6)
    press = ThinKPress(key_channel_compression_ratio=ratio, window_size=W)
    ok, ov = press.compress(None, None, kd, vd, None, {"queries": q.to(dev)})
    assert ok.data_ptr() == kd.data_ptr() and torch.equal(ov.cpu(), v)
    ref_k, ref_idx = opress.think_prune(k, q, ratio)
    scores = opress.think_channel_scores(k, q)
    n = int(128 * ratio)
    got = ok.cpu()
    zeroed = (got == 0).all(dim=2)                                   # [B, Hkv, 128]: channels that are zero everywhere
    for b in range(B):
        for h in range(Hkv):
            srt = scores[b, h].sort().values
            thr_lo, thr_hi = srt[n - 1], srt[n]
            near = ((scores[b, h] - thr_lo).abs() <= 1e-5 * thr_lo.abs()) | ((scores[b, h] - thr_hi).abs() <= 1e-5 * thr_hi.abs())
            want = torch.zeros(128, dtype=torch.bool)
            want[ref_idx[b, h]] = True
            assert int(zeroed[b, h].sum()) == n
            assert torch.equal(zeroed[b, h][~near], want[~near])
            kept = ~zeroed[b, h]
            assert torch.equal(got[b, h][:, kept], k[b, h][:, kept])


def test_think_press_paged_ragged_and_no_ops(dev):
    """The two kernels on a paged pool with ragged lengths (energies per sequence, zeroing limited to the sequence's
    own tokens); ratio 0 and a ratio below one channel leave the keys alone."""
    L, H, lens = 2, 2, [300, 17, 129]
    case = synth.make_paged_case(seed=3, num_layers=L, batch=len(lens), num_kv_heads=H, seq_lens=lens, dtype=torch.float16,
                                 keep_dense=True, block_size=64, fill_value=3.0)
    pool, tab, lens_d = case.kv_cache.to(dev), case.table_tensor(dev), case.lens_tensor(dev)
    view = _lib.paged_view(pool[0], tab, lens_d, max(lens))
    energy = ops.key_channel_energy(view, dev).cpu()
    for l in range(L):
        for b, n in enumerate(lens):
            torch.testing.assert_close(energy[l, b].double(), case.dense_k[l][b, :, :n].double().pow(2).sum(1), rtol=1e-5, atol=1e-6)
    prune = torch.zeros(L, len(lens), H, 128, dtype=torch.uint8)
    prune[..., 5] = 1
    prune[1, 2, 1, 64:] = 1
    ops.key_channel_zero(view, prune.to(dev))
    after = pool.cpu()
    used = set()
    for b, n in enumerate(lens):
        used.update(case.block_tables[b])
        for l in range(L):
            rows = torch.cat([after[0, l, blk] for blk in case.block_tables[b]])           # [tokens, H, D]
            want = case.dense_k[l][b, :, :n].clone().permute(1, 0, 2)
            want[..., 5] = 0
            if (l, b) == (1, 2):
                want[:, 1, 64:] = 0
            assert torch.equal(rows[:n], want)
            assert bool((rows[n:] == 3.0).all())                                            # slots past the sequence end
    assert torch.equal(after[1], case.kv_cache[1])
    spare = [i for i in range(after.shape[2]) if i not in used]
    assert bool((after[0][:, spare] == 3.0).all())
    k = torch.randn(1, 2, 40, 128).half().to(dev)
    for ratio in (0.0, 0.005):
        out, _ = ThinKPress(key_channel_compression_ratio=ratio).compress(None, None, k.clone(), k, None, {"queries": k[:, :, :32]})
        assert torch.equal(out, k)
    with pytest.raises(_lib.FastcacheError):
        ops.key_channel_zero(view, prune.to(dev)[..., :64])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n_last,n_recent,n_initial", [(1, 64, 4), (8, 100, 2)])
def test_simlayer_press(dev, dtype, n_last, n_recent, n_initial):
    """SimLayerKV: the lazy score against the float64 oracle (1e-3); below the threshold the layer is left alone,
    above it only the initial and the recent tokens survive, bit for bit; short inputs are never touched."""
    B, Hq, Hkv, S = 2, 8, 2, 900
    g = torch.Generator().manual_seed(n_recent)
    k = torch.randn(B, Hkv, S, 128, generator=g).to(dtype)
    v = torch.randn(B, Hkv, S, 128, generator=g).to(dtype)
    q = (torch.randn(B, Hq, n_last, 128, generator=g) * 0.5).to(dtype)
    kd, vd, kw = k.to(dev), v.to(dev), {"queries": q.to(dev)}
    ref = opress.simlayer_lazy_score(k, q, n_initial, n_recent)
    press = SimLayerKVPress(lazy_threshold=1.0, n_last=n_last, n_recent=n_recent, n_initial=n_initial)
    got = press.lazy_score(None, None, kd, kw)
    assert abs(got - ref) <= 1e-3 * ref and 0.0 < ref < 1.0
    ok, ov = press.compress(None, None, kd, vd, None, kw)                 # threshold 1: never lazy
    assert ok.data_ptr() == kd.data_ptr() and press.compression_ratios == [0.0]
    lazy = SimLayerKVPress(lazy_threshold=ref / 2, n_last=n_last, n_recent=n_recent, n_initial=n_initial)
    ok, ov = lazy.compress(None, None, kd, vd, None, kw)
    pos = opress.simlayer_keep_positions(S, n_initial, n_recent, n_last)
    assert ok.shape == (B, Hkv, pos.numel(), 128)
    assert torch.equal(ok.cpu(), k[:, :, pos]) and torch.equal(ov.cpu(), v[:, :, pos])
    assert lazy.compression_ratios == [(S - n_initial - n_recent + 1) / S] and lazy.compression_ratio == lazy.compression_ratios[0]
    short = kd[:, :, :n_initial + n_recent + n_last]
    ok, _ = lazy.compress(None, None, short, short, None, kw)
    assert ok.data_ptr() == short.data_ptr() and len(lazy.compression_ratios) == 1


@pytest.mark.parametrize("press", ["knorm", "snapkv"])
def test_paged_press_ragged_batch_in_one_launch_set(dev, press):
    """Eight sequences of eight different lengths scored, selected and compacted by one launch each: every
    sequence keeps int(its length * (1 - ratio)) tokens, as the reference's per-sequence press does."""
    dtype, L, Hq, Hkv, W, ksz, ratio = torch.bfloat16, 2, 8, 2, 16, 5, 0.6
    lens = [700, 130, 257, 256, 64, 1000, 511, 90]       # every budget holds the whole window
    B = len(lens)
    case = synth.make_paged_case(seed=41, num_layers=L, batch=B, num_kv_heads=Hkv, seq_lens=lens, dtype=dtype,
                                 keep_dense=True)
    q = torch.randn(L, B, Hq, W, 128, generator=torch.Generator().manual_seed(4)).to(dtype)
    pool = case.kv_cache.to(dev)
    tables, lens_d = case.table_tensor(dev), case.lens_tensor(dev)
    if press == "knorm":
        res = paged_press.knorm_compress_paged(pool, tables, lens_d, max(lens), ratio, host_lens=lens)
    else:
        res = paged_press.snapkv_compress_paged(pool, tables, lens_d, max(lens), q.to(dev), ratio, W, ksz, True, "sum",
                                                host_lens=lens)
    torch.cuda.synchronize()
    assert res.kept_per_seq == [int(n * (1 - ratio)) for n in lens]
    got = pool.cpu()
    for b, n in enumerate(lens):
        k_keep = res.kept_per_seq[b]
        for l in range(L):
            kd, vd = case.dense_k[l][b:b + 1, :, :n], case.dense_v[l][b:b + 1, :, :n]
            if press == "knorm":
                ref = opress.knorm_score(kd)
                scored = n
            else:
                ref = opress.snapkv_score(q[l, b:b + 1], kd, W, ksz, True, "sum")
                scored = n - W
            sc = res.scores[l, b:b + 1, :, :n].cpu()
            torch.testing.assert_close(sc[..., :scored], ref[..., :scored], rtol=1e-3, atol=1e-3 * float(ref[..., :scored].abs().mean()))
            assert bool(torch.isinf(res.scores[l, b, :, n:]).all())
            idx = res.indices[l, b:b + 1, :, :k_keep].cpu().long()
            assert bool((res.indices[l, b, :, k_keep:] == -1).all())
            want = opress.topk_lowest_index(sc, k_keep)                      # the stable selection on the kernel's own scores
            assert torch.equal(idx, want)
            tie = opress.near_tie_rows(ref[..., :scored], k_keep - (0 if press == "knorm" else W))
            ref_full = ref.clone()
            ref_full[..., scored:] = sc[..., scored:]
            assert torch.equal(idx[~tie], opress.topk_lowest_index(ref_full, k_keep)[~tie])
            blocks = case.block_tables[b]
            for p, dense in enumerate((kd, vd)):
                rows = torch.cat([got[p, l, blk] for blk in blocks])[:n].permute(1, 0, 2).unsqueeze(0)   # [1, H, n, D]
                assert torch.equal(rows[:, :, :k_keep], opress.gather_tokens(dense, idx))
                old = torch.cat([case.kv_cache[p, l, blk] for blk in blocks])[:n].permute(1, 0, 2).unsqueeze(0)
                assert torch.equal(rows[:, :, k_keep:], old[:, :, k_keep:])
