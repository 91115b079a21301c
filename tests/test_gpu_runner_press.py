"""The kvpress-style press OBJECTS driven through nano-vllm's runner hook: ``PagedKVRunner(compressor=press)
.compress_kv_cache_batch(seqs)`` against the oracle's restatement of the reference loop
(nanovllm/engine/llava_model_runner.py:745-786: extract -> press -> write back, per sequence), plus the two
readings of "keep a quarter plus the window" and pages shared between sequences."""
import pytest
import torch

from fastcache_amd import _lib, paged_press, synth
from fastcache_amd.engine import BlockManager, Sequence
from fastcache_amd.engine.kv_runner import PagedKVRunner
from fastcache_amd.kernels import KVPressCompressor
from fastcache_amd.presses import (ExpectedAttentionPress, KnormPress, ObservedAttentionPress, RandomPress,
                                   SimLayerKVPress, SnapKVPress, StreamingLLMPress, ThinKPress, TOVAPress)
from oracle import paged as opaged
from oracle import pipeline as opipe
from oracle import presses as opress

pytestmark = pytest.mark.gpu

W, KSZ = 16, 5


def _runner_with_case(dev, case, lens, dtype, compressor, L, H, block_manager=True):
    nb = case.kv_cache.shape[2]
    bm = BlockManager(nb, 256)
    runner = PagedKVRunner(L, H, 128, num_blocks=nb, dtype=dtype, device=dev, image_token_len=0,
                           compressor=compressor, block_manager=bm if block_manager else None)
    seqs = [Sequence(list(range(3000 * i, 3000 * i + n))) for i, n in enumerate(lens)]
    for s in seqs:
        bm.allocate(s)
    for b, s in enumerate(seqs):                                    # "prefill": the rows appear in the sequence's pages
        for i, blk in enumerate(s.block_table):
            runner.kv_cache[:, :, blk] = case.kv_cache[:, :, case.block_tables[b][i]].to(dev)
    return runner, bm, seqs


def _streaming_scores(n, n_kept, n_sink=4):
    sc = torch.ones(n)
    sc[n_sink:n_sink + (n - n_kept)] = 0
    return sc


@pytest.mark.parametrize("kind", ["knorm", "snapkv", "snapkv-window-on-top", "tova", "streaming"])
def test_press_objects_on_the_runner_hook_ragged_batch(dev, kind):
    """Nine sequences of nine lengths, one ``compress_kv_cache_batch`` call with a press object as the runner's
    compressor: compressed lengths, blocks to free and the ratio equal the oracle's per-sequence loop; the pages
    equal the oracle's byte for byte wherever fp32 scoring decides the selection (no score within 1e-5 of a row's
    threshold), and equal the free-function form of the same press everywhere."""
    dtype, L, Hq, Hkv, ratio = torch.bfloat16, 2, 8, 2, 0.6
    lens = [700, 130, 257, 256, 90, 1000, 511, 333, 512]
    B = len(lens)
    case = synth.make_paged_case(seed=91, num_layers=L, batch=B, num_kv_heads=Hkv, seq_lens=lens, dtype=dtype,
                                 shuffle_tables=False, extra_blocks=0, keep_dense=True)
    q = torch.randn(L, B, Hq, W, 128, generator=torch.Generator().manual_seed(12)).to(dtype)
    in_budget = kind != "snapkv-window-on-top"
    if kind == "knorm":
        press = KnormPress(ratio)
        oracle_comp = opipe.knorm_press_compressor(ratio)
        score_of = lambda l, i, k: opress.knorm_score(k)
    elif kind.startswith("snapkv"):
        press = SnapKVPress(ratio, window_size=W, kernel_size=KSZ, window_in_budget=in_budget)
        press.set_window_queries(q.to(dev))
        oracle_comp = opipe.snapkv_press_compressor(q, ratio, W, KSZ, window_in_budget=in_budget)
        score_of = lambda l, i, k: opress.snapkv_score(q[l, i:i + 1], k, W, KSZ)
    elif kind == "tova":
        press = TOVAPress(ratio)
        press.set_window_queries(q.to(dev))
        score_of = lambda l, i, k: opress.tova_score(q[l, i:i + 1, :, -1:], k)
        oracle_comp = opipe.scored_press_compressor(lambda l, i, k, v: score_of(l, i, k), ratio)
    else:
        press = StreamingLLMPress(ratio)
        score_of = lambda l, i, k: _streaming_scores(k.shape[2], int(k.shape[2] * (1 - ratio))).expand(1, Hkv, -1)
        oracle_comp = opipe.scored_press_compressor(lambda l, i, k, v: score_of(l, i, k), ratio)
    runner, bm, seqs = _runner_with_case(dev, case, lens, dtype, press, L, Hkv)
    tables_before = [list(s.block_table) for s in seqs]
    ref_pool = runner.kv_cache.cpu()
    start_pool = ref_pool.clone()
    ref_lens, ref_free, ref_ratio = opipe.compress_batch(ref_pool, tables_before, lens, oracle_comp)

    calls = []
    inner = press.paged_forward
    press.paged_forward = lambda *a, **k: (calls.append(k), inner(*a, **k))[1]
    sec, got_ratio = runner.compress_kv_cache_batch(seqs)
    assert len(calls) == 1 and calls[0]["seq_ids"] == [s.seq_id for s in seqs]
    assert abs(got_ratio - ref_ratio) < 1e-9
    got_pool = runner.kv_cache.cpu()
    exact = 0
    for i, (s, tab, n) in enumerate(zip(seqs, tables_before, lens)):
        C = ref_lens[i]
        want_C = int(n * (1 - ratio)) + (0 if in_budget else W)
        assert runner._compressed_lens[s.seq_id] == C == want_C
        assert runner._blocks_to_free.get(s.seq_id, []) == ref_free.get(i, [])
        undecided = False
        for l, (k, _) in enumerate(opaged.extract_kv(start_pool, tab, n)):
            sc = score_of(l, i, k)
            scored = n - W if kind.startswith("snapkv") else (n - 1 if kind == "tova" else n)
            budget = C - (n - scored)
            if kind != "streaming":
                undecided |= bool(opress.near_tie_rows(sc[..., :scored], budget).any())
        got = opaged.extract_kv(got_pool, tab, n)
        ref = opaged.extract_kv(ref_pool, tab, n)
        for (gk, gv), (rk, rv) in zip(got, ref):
            assert torch.equal(gk[:, :, C:], rk[:, :, C:]) and torch.equal(gv[:, :, C:], rv[:, :, C:])   # stale rows stay
            if not undecided:
                assert torch.equal(gk, rk) and torch.equal(gv, rv)
        exact += not undecided
    assert exact >= B - 2, f"only {exact} of {B} sequences could be compared byte for byte"
    # the same press as free functions on a pool of its own: identical bytes everywhere
    if kind in ("knorm", "snapkv", "snapkv-window-on-top"):
        pool2 = start_pool.to(dev)
        tt, ll = runner._table_and_lens(tables_before, lens)
        if kind == "knorm":
            paged_press.knorm_compress_paged(pool2, tt, ll, max(lens), ratio, host_lens=lens)
        else:
            paged_press.snapkv_compress_paged(pool2, tt, ll, max(lens), q.to(dev), ratio, W, KSZ,
                                              window_in_budget=in_budget, host_lens=lens)
        assert torch.equal(pool2.cpu().view(torch.int16), got_pool.view(torch.int16))


def test_snapkv_press_object_is_config2_through_the_runner(dev):
    """The BASELINE SnapKV configuration (window 64, kernel 7, sums, keep a quarter) at reduced size through the
    runner hook, both readings of the budget: 25 % with the window inside (``fc_snapkv_press`` keeps 256 of 1024)
    and the window on top (320 = 256 + 64, index stride 320)."""
    dtype, L, B, Hq, Hkv, S, Wc, k7, ratio = torch.bfloat16, 3, 4, 8, 2, 1024, 64, 7, 0.75
    case = synth.snapkv_case(seed=5, num_layers=L, batch=B, num_q_heads=Hq, num_kv_heads=Hkv, seq_len=S, window=Wc,
                             shuffle_tables=False, extra_blocks=0)
    for in_budget, C in ((True, 256), (False, 320)):
        press = SnapKVPress(ratio, window_size=Wc, kernel_size=k7, reduction="sum", window_in_budget=in_budget)
        runner, bm, seqs = _runner_with_case(dev, case, [S] * B, dtype, press, L, Hkv)
        press.set_window_queries(case.queries.to(dev), seq_ids=[s.seq_id for s in seqs])
        tables = [list(s.block_table) for s in seqs]
        ref_pool = runner.kv_cache.cpu()
        start = ref_pool.clone()
        ref_lens, ref_free, _ = opipe.compress_batch(
            ref_pool, tables, [S] * B, opipe.snapkv_press_compressor(case.queries, ratio, Wc, k7, True, "sum", in_budget))
        runner.compress_kv_cache_batch(seqs)
        got_pool = runner.kv_cache.cpu()
        assert not press._paged_inputs                                       # the queries were handed back
        for i, s in enumerate(seqs):
            assert runner._compressed_lens[s.seq_id] == ref_lens[i] == C
            assert runner._blocks_to_free[s.seq_id] == ref_free[i] == tables[i][-(-C // 256):]
            tie = False
            for l, (k, _) in enumerate(opaged.extract_kv(start, tables[i], S)):
                sc = opress.snapkv_score(case.queries[l, i:i + 1], k, Wc, k7, True, "sum")
                tie |= bool(opress.near_tie_rows(sc[..., :S - Wc], C - Wc).any())
            if not tie:
                for (gk, gv), (rk, rv) in zip(opaged.extract_kv(got_pool, tables[i], S),
                                              opaged.extract_kv(ref_pool, tables[i], S)):
                    assert torch.equal(gk, rk) and torch.equal(gv, rv)


def test_press_inputs_follow_sequence_ids_into_a_later_batch(dev):
    """Window queries handed over by two prefill batches, named by sequence id, serve one later compression of
    another composition (what the lazy trigger does); a sequence without queries is refused before any launch."""
    dtype, L, Hq, Hkv, S, ratio = torch.float16, 2, 4, 2, 400, 0.5
    lens = [S] * 4
    case = synth.make_paged_case(seed=3, num_layers=L, batch=4, num_kv_heads=Hkv, seq_lens=lens, dtype=dtype,
                                 shuffle_tables=False, extra_blocks=0)
    q = torch.randn(L, 4, Hq, W, 128, generator=torch.Generator().manual_seed(8)).to(dtype)
    press = SnapKVPress(ratio, window_size=W, kernel_size=KSZ)
    runner, bm, seqs = _runner_with_case(dev, case, lens, dtype, press, L, Hkv)
    ids = [s.seq_id for s in seqs]
    press.set_window_queries(q[:, :2].to(dev), seq_ids=ids[:2])          # first prefill batch
    press.set_window_queries(q[:, 2:].to(dev), seq_ids=ids[2:])          # second prefill batch
    order = [3, 0, 2]                                                     # the later batch
    tables = [list(seqs[i].block_table) for i in order]
    ref_pool = runner.kv_cache.cpu()
    ref_lens, _, _ = opipe.compress_batch(ref_pool, tables, [S] * 3,
                                          opipe.snapkv_press_compressor(q[:, order], ratio, W, KSZ))
    pool_before = runner.kv_cache.clone()
    runner.compress_kv_cache_batch([seqs[i] for i in order])
    pool2 = pool_before.clone()
    tt, ll = runner._table_and_lens(tables, [S] * 3)
    paged_press.snapkv_compress_paged(pool2, tt, ll, S, q[:, order].to(dev), ratio, W, KSZ)
    assert torch.equal(pool2, runner.kv_cache)
    assert [runner._compressed_lens[seqs[i].seq_id] for i in order] == [ref_lens[j] for j in range(3)]
    # sequence 1's queries are still held; a sequence nobody handed queries for is refused, cache untouched
    stranger = Sequence(list(range(90000, 90000 + S)))
    stranger.block_table = list(seqs[1].block_table)
    with pytest.raises(_lib.FastcacheError, match="holds no inputs for sequences"):
        runner._compress_enqueue([stranger], 0)
    assert not runner._launch_started
    runner.compress_kv_cache_batch([seqs[1]])
    assert runner._compressed_lens[seqs[1].seq_id] == 200 and not press._paged_inputs


def test_other_press_objects_on_the_runner_hook(dev):
    """ThinK prunes key channels in the pages (lengths stay); ExpectedAttention scores the pages from given query
    statistics; Random keeps the right count; the presses that cannot run on pages say why."""
    dtype, L, Hq, Hkv, S = torch.float16, 2, 4, 2, 300
    case = synth.make_paged_case(seed=6, num_layers=L, batch=2, num_kv_heads=Hkv, seq_lens=[S, S], dtype=dtype,
                                 shuffle_tables=False, extra_blocks=0, keep_dense=True)
    q = torch.randn(L, 2, Hq, 32, 128, generator=torch.Generator().manual_seed(1)).to(dtype)
    # ThinK
    think = ThinKPress(key_channel_compression_ratio=0.25, window_size=32)
    runner, bm, seqs = _runner_with_case(dev, case, [S, S], dtype, think, L, Hkv)
    think.set_window_queries(q.to(dev))
    runner.compress_kv_cache_batch(seqs)
    assert [runner._compressed_lens[s.seq_id] for s in seqs] == [S, S] and not runner._blocks_to_free
    got = runner.kv_cache.cpu()
    for l in range(L):
        for b, s in enumerate(seqs):
            k, v = opaged.extract_kv(case.kv_cache, case.block_tables[b], S)[l]
            want_k, _ = opress.think_prune(k, q[l, b:b + 1], 0.25)
            gk, gv = opaged.extract_kv(got, s.block_table, S)[l]
            assert torch.equal(gk, want_k) and torch.equal(gv, v)
    # ExpectedAttention with given statistics (no covariance): same kept rows as the dense press object
    mu = torch.randn(L, 2, Hq, 128, generator=torch.Generator().manual_seed(2))
    ea = ExpectedAttentionPress(0.5, use_covariance=False)
    runner, bm, seqs = _runner_with_case(dev, case, [S, S], dtype, ea, L, Hkv)
    ea.set_query_statistics(mu.to(dev))
    runner.compress_kv_cache_batch(seqs)
    got = runner.kv_cache.cpu()
    for l in range(L):
        kd, vd = case.dense_k[l].to(dev), case.dense_v[l].to(dev)
        ok, ov = ExpectedAttentionPress(0.5, use_covariance=False).compress(None, None, kd, vd, None,
                                                                            {"mean_query": mu[l].to(dev)})
        for b, s in enumerate(seqs):
            gk, gv = opaged.extract_kv(got, s.block_table, 150)[l]
            assert torch.equal(gk[0], ok[b].cpu()) and torch.equal(gv[0], ov[b].cpu())
    # Random: 150 distinct ascending source rows per column
    rnd = RandomPress(0.5, seed=3)
    runner, bm, seqs = _runner_with_case(dev, case, [S, S], dtype, rnd, L, Hkv)
    runner.compress_kv_cache_batch(seqs)
    assert [runner._compressed_lens[s.seq_id] for s in seqs] == [150, 150]
    gk = opaged.extract_kv(runner.kv_cache.cpu(), seqs[0].block_table, 150)[0][0][0, 0]        # [150, D]
    src = case.dense_k[0][0, 0]                                                              # [S, D]
    pos = [int((src == row).all(-1).nonzero()[0]) for row in gk]
    assert pos == sorted(set(pos)) and len(pos) == 150
    # presses that need what a paged runner does not have
    for press, why in ((ObservedAttentionPress(0.5), "attention matrices"), (SimLayerKVPress(), "per layer")):
        runner, bm, seqs = _runner_with_case(dev, case, [S, S], dtype, press, L, Hkv)
        with pytest.raises(_lib.FastcacheError, match=why):
            runner._compress_enqueue(seqs, 0)
        assert not runner._launch_started


def test_shared_prefix_pages_survive_the_compression_of_one_owner(dev):
    """Two prompts with the same first 512 tokens share two pages.  Compressing one of them in place gives it
    private copies of the shared pages it rewrites first: the other sequence's rows are unchanged, the result equals
    the oracle's, and compressing both in one batch afterwards equals the oracle's per-sequence loop."""
    dtype, L, H = torch.float16, 2, 2
    nb = 12
    comp = KVPressCompressor("knorm", 0.5)
    bm = BlockManager(nb, 256)
    runner = PagedKVRunner(L, H, 128, num_blocks=nb, dtype=dtype, device=dev, image_token_len=0, compressor=comp,
                           block_manager=bm)
    a = Sequence(list(range(600)))
    b = Sequence(list(range(512)) + [7] * 88)
    c = Sequence(list(range(512)) + [8] * 200)
    for s in (a, b, c):
        bm.allocate(s)
    assert a.block_table[:2] == b.block_table[:2] == c.block_table[:2]
    g = torch.Generator().manual_seed(4)
    runner.kv_cache.copy_(torch.randn(runner.kv_cache.shape, generator=g).to(dtype))
    start = runner.kv_cache.cpu()
    rows_b = opaged.extract_kv(start, list(b.block_table), 600)
    tab_a = list(a.block_table)
    ref_pool = start.clone()
    oracle_comp = lambda hf, i, n: [opress.adapter_compress_layer("knorm", k, v, 0.5) for k, v in hf]
    ref_lens, _, _ = opipe.compress_batch(ref_pool, [tab_a], [600], oracle_comp)
    free_before = len(bm.free_block_ids)
    runner.compress_kv_cache_batch([a])                     # 300 rows kept: rewrites pages 0 and 1, both shared
    assert a.block_table[:2] != tab_a[:2] and a.block_table[2] == tab_a[2]
    assert len(bm.free_block_ids) == free_before - 2 and bm.blocks[tab_a[0]].ref_count == 2
    now = runner.kv_cache.cpu()
    for (k0, v0), (k1, v1) in zip(rows_b, opaged.extract_kv(now, list(b.block_table), 600)):
        assert torch.equal(k0, k1) and torch.equal(v0, v1)                     # b reads what it read before
    for (gk, gv), (rk, rv) in zip(opaged.extract_kv(now, list(a.block_table), 300),
                                  opaged.extract_kv(ref_pool, tab_a, 300)):
        assert torch.equal(gk, rk) and torch.equal(gv, rv)
    # b and c still share two pages; one batch compresses both
    tabs = [list(b.block_table), list(c.block_table)]
    ref2 = now.clone()
    # the oracle's loop runs on private copies: give c its own pages first, as the runner will
    ref_lens2, _, _ = opipe.compress_batch(ref2, [tabs[0]], [600], oracle_comp)
    want_b = opaged.extract_kv(ref2, tabs[0], ref_lens2[0])
    ref3 = now.clone()
    ref_lens3, _, _ = opipe.compress_batch(ref3, [tabs[1]], [712], oracle_comp)
    want_c = opaged.extract_kv(ref3, tabs[1], ref_lens3[0])
    runner.compress_kv_cache_batch([b, c])
    assert not set(b.block_table[:2]) & set(c.block_table[:2])
    end = runner.kv_cache.cpu()
    for got, want in ((opaged.extract_kv(end, list(b.block_table), 300), want_b),
                      (opaged.extract_kv(end, list(c.block_table), 356), want_c)):
        for (gk, gv), (rk, rv) in zip(got, want):
            assert torch.equal(gk, rk) and torch.equal(gv, rv)
    # a failure in the host-side checks before any launch leaves the flag clear (state NONE, not FAILED)
    runner.compressor = SnapKVPress(0.5, window_size=W)          # no window queries handed over
    d = Sequence(list(range(40000, 40300)))
    bm.allocate(d)
    with pytest.raises(_lib.FastcacheError, match="needs the window queries"):
        runner._compress_enqueue([d], 0)
    assert not runner._launch_started


def test_rewritten_pages_leave_the_prefix_cache_when_the_compression_starts(dev):
    """With the compression on the side stream the engine shortens the tables only in front of the sequence's next
    decode step; a prefill of the same prompt scheduled in between must not be handed the pages being rewritten."""
    dtype, L, H, nb = torch.float16, 2, 2, 12
    bm = BlockManager(nb, 256)
    runner = PagedKVRunner(L, H, 128, num_blocks=nb, dtype=dtype, device=dev, image_token_len=0,
                           compressor=KVPressCompressor("knorm", 0.5), block_manager=bm)
    a = Sequence(list(range(600)))
    bm.allocate(a)
    runner.kv_cache.copy_(torch.randn(runner.kv_cache.shape, generator=torch.Generator().manual_seed(8)).to(dtype))
    start = runner.kv_cache.cpu()
    tab_a = list(a.block_table)
    done = runner.start_background_compression([a])          # 300 rows kept: pages 0 and 1 are rewritten, page 2 is not
    twin = Sequence(list(range(600)))
    bm.allocate(twin)
    assert twin.num_cached_tokens == 0 and not set(twin.block_table) & set(a.block_table)
    assert all(bm.blocks[p].hash == -1 for p in tab_a[:2])
    runner.wait_compression(done)
    ref_pool = start.clone()
    oracle_comp = lambda hf, i, n: [opress.adapter_compress_layer("knorm", k, v, 0.5) for k, v in hf]
    opipe.compress_batch(ref_pool, [tab_a], [600], oracle_comp)
    for (gk, gv), (rk, rv) in zip(opaged.extract_kv(runner.kv_cache.cpu(), tab_a, 300),
                                  opaged.extract_kv(ref_pool, tab_a, 300)):
        assert torch.equal(gk, rk) and torch.equal(gv, rv)


def test_snapkv_press_object_with_the_prefill_log_sum_exp(dev):
    """``set_window_queries(..., lse=)``: with the window queries' log-sum-exp from the prefill's attention kernel the
    press reads the keys once (single-sweep scoring, then selection + compaction); same kept rows as without it."""
    dtype, L, B, Hq, Hkv, S, ratio = torch.float16, 2, 2, 4, 2, 700, 0.5
    case = synth.make_paged_case(seed=19, num_layers=L, batch=B, num_kv_heads=Hkv, seq_lens=[S] * B, dtype=dtype,
                                 shuffle_tables=False, extra_blocks=0, keep_dense=True)
    q = torch.randn(L, B, Hq, W, 128, generator=torch.Generator().manual_seed(2)).to(dtype)
    G = Hq // Hkv
    mask = torch.triu(torch.full((W, S), float("-inf")), diagonal=S - W + 1)
    lse = torch.empty(L, B, Hq, W)
    for l in range(L):
        k = case.dense_k[l].float().repeat_interleave(G, dim=1)                              # [B, Hq, S, D]
        lse[l] = torch.logsumexp(torch.matmul(q[l].float(), k.transpose(2, 3)) * 128 ** -0.5 + mask, dim=-1)
    pools = []
    for given in (False, True):
        press = SnapKVPress(ratio, window_size=W, kernel_size=KSZ)
        runner, bm, seqs = _runner_with_case(dev, case, [S] * B, dtype, press, L, Hkv)
        press.set_window_queries(q.to(dev), lse=lse.to(dev) if given else None)
        runner.compress_kv_cache_batch(seqs)
        assert [runner._compressed_lens[s.seq_id] for s in seqs] == [350, 350] and not press._paged_inputs
        pools.append((runner.kv_cache.cpu(), [list(s.block_table) for s in seqs]))
    tie = False
    for l in range(L):
        sc = opress.snapkv_score(q[l], case.dense_k[l], W, KSZ)
        tie |= bool(opress.near_tie_rows(sc[..., :S - W], 350 - W).any())
    assert not tie, "a score within 1e-5 of a threshold: pick another seed"
    for b in range(B):
        for (ak, av), (bk, bv) in zip(opaged.extract_kv(pools[0][0], pools[0][1][b], 350),
                                      opaged.extract_kv(pools[1][0], pools[1][1][b], 350)):
            assert torch.equal(ak, bk) and torch.equal(av, bv)
