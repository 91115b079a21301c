"""GPU parity of the reference-surface objects: CCM modules, the kvpress adapter, press objects and
the runner / engine hooks, each against the CPU oracle on the same seeded inputs."""
from types import SimpleNamespace

import pytest
import torch

from fastcache_amd import synth
from fastcache_amd.engine import BlockManager, Sequence
from fastcache_amd.engine.kv_runner import PagedKVRunner
from fastcache_amd.engine.llm_hooks import free_compressed_blocks
from fastcache_amd.kernels import BatchedGEMMCompressor, KVPressCompressor, MiniCPMKVCompressor
from fastcache_amd.presses import KnormPress, RandomPress, SnapKVPress, StreamingLLMPress
from fastcache_amd.utils_ccm import KVCacheHybridCompressor, KVCacheLinearDecoupleCompressor
from oracle import ccm as occm
from oracle import paged as opaged
from oracle import pipeline as opipe
from oracle import presses as opress
from test_gpu_ccm import assert_mlp_close
from test_host_logic import llava_cfg, minicpm_cfg

pytestmark = pytest.mark.gpu


def rand_kv(L, B, H, S, dtype, seed=0, permuted=True):
    """Per-layer (k, v) in the layout the runner hands to compressors: [B, H, S, D] views of [B, S, H, D]."""
    g = torch.Generator().manual_seed(seed)
    out = []
    for _ in range(L):
        k = torch.randn(B, S, H, 128, generator=g).to(dtype)
        v = torch.randn(B, S, H, 128, generator=g).to(dtype)
        out.append((k.permute(0, 2, 1, 3), v.permute(0, 2, 1, 3)) if permuted else
                   (k.permute(0, 2, 1, 3).contiguous(), v.permute(0, 2, 1, 3).contiguous()))
    return out


def to_dev(kv, dev):
    return [(k.to(dev), v.to(dev)) for k, v in kv]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_linear_decouple_module(dev, dtype):
    L, B, H, S, cf = 2, 2, 4, 77, 2
    torch.manual_seed(3)
    m = KVCacheLinearDecoupleCompressor(llava_cfg(L, H), compression_factor=cf).to(dev).to(dtype).eval()
    sd = occm.reference_init_state_dict("linear_decouple", L, 128, cf, seed=3)
    kv = rand_kv(L, B, H, S, dtype)
    ref = occm.linear_decouple_forward(kv, [41, 36], sd, cf, 1)
    out = m(to_dev(kv, dev), it_len=[41, 36])
    assert len(out) == L
    for (ok, ov), (rk, rv) in zip(out, ref):
        assert ok.is_contiguous() and ok.shape == rk.shape and ok.dtype == dtype
        assert_mlp_close(ok.cpu(), rk, dtype)
        assert_mlp_close(ov.cpu(), rv, dtype)
    # a checkpoint in the reference's state-dict layout loads and changes the result accordingly
    sd2 = occm.reference_init_state_dict("linear_decouple", L, 128, cf, seed=4)
    m.load_state_dict(sd2)
    ref2 = occm.linear_decouple_forward(kv, [41, 36], sd2, cf, 1)
    out2 = m(to_dev(kv, dev), it_len=[41, 36])
    assert_mlp_close(out2[1][0].cpu(), ref2[1][0], dtype)


def test_hybrid_and_minicpm_modules(dev):
    dtype, L, B, H, S = torch.bfloat16, 2, 1, 4, 203
    torch.manual_seed(8)
    h = KVCacheHybridCompressor(minicpm_cfg(L), compression_factor=5, min_seq_len=2).to(dev).to(dtype).eval()
    hsd = occm.reference_init_state_dict("hybrid", L, 128, 5, seed=8)
    kv = rand_kv(L, B, H, S, dtype, seed=1)
    ref = occm.hybrid_forward(kv, [0, S], hsd, 5, 2)
    out = h(to_dev(kv, dev), it_len=[0, S])
    for (ok, ov), (rk, rv) in zip(out, ref):
        assert_mlp_close(ok.cpu(), rk, dtype)
        assert_mlp_close(ov.cpu(), rv, dtype)
    with pytest.raises(TypeError):
        h(to_dev(kv, dev), it_len=[64, S - 64])
    # image segment too short to compress is passed through unchanged
    ref_p = occm.hybrid_forward(kv, [7, S - 7], hsd, 5, 2)
    out_p = h(to_dev(kv, dev), it_len=[7, S - 7])
    assert torch.equal(out_p[0][0][:, :, :7].cpu(), kv[0][0][:, :, :7])
    assert_mlp_close(out_p[0][1].cpu(), ref_p[0][1], dtype)
    # a cache object in: a NEW CompressibleCache out, the input untouched, the seen-token count carried over
    from fastcache_amd.utils_ccm import CompressibleCache
    src = CompressibleCache()
    src.key_cache, src.value_cache = [k.to(dev) for k, _ in kv], [v.to(dev) for _, v in kv]
    src.set_seen_tokens(S + 11)                     # the model has seen more tokens than the cache holds rows
    got = h(src, it_len=[0, S])
    assert isinstance(got, CompressibleCache) and got is not src
    assert src.key_cache[0].shape[2] == S and src.get_seq_length() == S + 11
    assert got.get_seq_length() == S + 11 and got.get_actual_seq_length() == ref[0][0].shape[2] == len(got[0][0][0][0])
    for layer in range(L):
        assert torch.equal(got.key_cache[layer], out[layer][0]) and torch.equal(got.value_cache[layer], out[layer][1])
    twin = got.clone()
    assert twin.get_seq_length() == S + 11 and torch.equal(twin.key_cache[1], got.key_cache[1]) \
        and twin.key_cache[1].data_ptr() != got.key_cache[1].data_ptr()
    # short sequences come back unchanged (min_seq_len guard)
    short = rand_kv(L, B, H, 6, dtype, seed=2)
    out_s = h(to_dev(short, dev), it_len=[0, 6])
    assert torch.equal(out_s[0][0].cpu(), short[0][0])

    torch.manual_seed(9)
    mc = MiniCPMKVCompressor(minicpm_cfg(L)).to(dev).to(dtype).eval()
    msd = occm.reference_init_state_dict("minicpm", L, 128, 5, seed=9)
    for it_len in ([0, S], [60, S - 60]):
        ref_m = occm.minicpm_forward(kv, it_len, msd, 5, 2)
        out_m = mc(to_dev(kv, dev), it_len=it_len)
        assert out_m[0][0].shape == ref_m[0][0].shape
        assert_mlp_close(out_m[1][0].cpu(), ref_m[1][0], dtype)


def test_batched_compressor_equals_original(dev):
    dtype, L, B, H, S, cf = torch.float16, 3, 2, 2, 64, 2
    torch.manual_seed(2)
    orig = KVCacheLinearDecoupleCompressor(llava_cfg(L, H), compression_factor=cf).to(dev).to(dtype).eval()
    bat = BatchedGEMMCompressor(num_layers=L, num_heads=H, head_dim=128, compression_factor=cf)
    bat.load_from_original_compressor(orig)
    kv = to_dev(rand_kv(L, B, H, S, dtype, seed=5), dev)
    a = orig(kv, it_len=[40, 24])
    b = bat(kv, it_len=[40, 24])
    for (ak, av), (bk, bv) in zip(a, b):
        assert torch.equal(ak, bk) and torch.equal(av, bv)          # same kernel, same weights: bit-identical
    part = bat.compress_layers(kv, 1, 3, it_len=[40, 24])
    assert len(part) == 2 and torch.equal(part[0][0], a[1][0]) and torch.equal(part[1][1], a[2][1])
    assert bat.compress_layers(kv, 2, 2) == []


@pytest.mark.parametrize("method", ["streaming_llm", "knorm", "snapkv", "h2o", "random"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_kvpress_adapter(dev, method, dtype):
    L, B, H, S = 2, 3, 4, 150
    comp = KVPressCompressor(method=method, compression_ratio=1.0 - 1.0 / 3)
    kv = rand_kv(L, B, H, S, dtype, seed=7)
    out = comp(to_dev(kv, dev), it_len=[10, 140])
    n = comp.get_compressed_length(S)
    for (k, v), (ok, ov) in zip(kv, out):
        assert ok.shape == (B, H, n, 128) and ok.is_contiguous()
        if method == "random":
            # RNG-dependent: kept rows are rows of the input, in ascending position order, same for K and V
            pos = [(k[0, 0] == ok[0, 0, j].cpu()).all(-1).nonzero()[0, 0].item() for j in range(n)]
            assert pos == sorted(set(pos))
            assert torch.equal(ov[0, 0].cpu(), v[0, 0, pos])
            continue
        rk, rv = opress.adapter_compress_layer(method, k, v, comp.compression_ratio)
        if method == "knorm":
            m = opress.knorm_mean_score(k)
            tie = opress.near_tie_rows(m, n)
            if dtype == torch.bfloat16:      # bf16 means collide often; only untied rows are defined
                tie |= (torch.sort(m, -1).values.diff(dim=-1) == 0).any(-1)
            sel = ~tie
            assert torch.equal(ok.cpu()[sel], rk[sel]) and torch.equal(ov.cpu()[sel], rv[sel])
        else:
            assert torch.equal(ok.cpu(), rk) and torch.equal(ov.cpu(), rv)
    # nothing to drop: inputs returned contiguous
    same = KVPressCompressor("knorm", 0.0)(to_dev(kv, dev))
    assert torch.equal(same[0][0].cpu(), kv[0][0])


def test_press_objects_compress(dev):
    dtype, B, Hq, Hkv, S, W = torch.bfloat16, 2, 8, 2, 400, 64
    g = torch.Generator().manual_seed(3)
    k = torch.randn(B, Hkv, S, 128, generator=g).to(dtype)
    v = torch.randn(B, Hkv, S, 128, generator=g).to(dtype)
    q = torch.randn(B, Hq, W, 128, generator=g).to(dtype)
    hidden = torch.zeros(B, S, 1)
    kd, vd = k.to(dev), v.to(dev)
    # Knorm
    ck, cv = KnormPress(0.5).compress(None, hidden, kd, vd, None, {})
    sc = opress.knorm_score(k)
    rk, rv, ridx = opress.press_compress(k, v, sc, 0.5)
    tie = opress.near_tie_rows(sc, 200)
    assert torch.equal(ck.cpu()[~tie], rk[~tie]) and torch.equal(cv.cpu()[~tie], rv[~tie])
    # SnapKV with the rotated window queries handed in
    press = SnapKVPress(compression_ratio=0.75, window_size=W, kernel_size=7)
    ck, cv = press.compress(None, hidden, kd, vd, None, {"queries": q.to(dev)})
    sc = opress.snapkv_score(q, k, W, 7)
    rk, rv, _ = opress.press_compress(k, v, sc, 0.75)
    tie = opress.near_tie_rows(sc[..., :S - W], 100 - W)
    assert ck.shape == (B, Hkv, 100, 128)
    assert torch.equal(ck.cpu()[~tie], rk[~tie]) and torch.equal(cv.cpu()[~tie], rv[~tie])
    got_sc = press.score(None, hidden, kd, vd, None, {"queries": q.to(dev)})
    torch.testing.assert_close(got_sc.cpu(), sc, rtol=1e-3, atol=1e-3 * float(sc.abs().mean()))
    # StreamingLLM: sinks + most recent tokens
    ck, _ = StreamingLLMPress(0.5, n_sink=4).compress(None, hidden, kd, vd, None, {})
    assert torch.equal(ck.cpu(), torch.cat([k[:, :, :4], k[:, :, 204:]], dim=2))
    # Random: seeded, right size, rows of the input
    ck, _ = RandomPress(0.5, seed=1).compress(None, hidden, kd, vd, None, {})
    assert ck.shape == (B, Hkv, 200, 128)


class _FakeAttn(torch.nn.Module):
    """Attention stand-in that appends K/V to a cache object the way HF layers do."""

    def __init__(self, layer_idx):
        super().__init__()
        self.layer_idx = layer_idx

    def forward(self, hidden_states=None, past_key_value=None, k=None, v=None):
        past_key_value.key_cache[self.layer_idx] = k
        past_key_value.value_cache[self.layer_idx] = v
        past_key_value.seen_tokens = k.shape[2]
        return hidden_states, None, past_key_value


def test_press_hook_protocol(dev):
    """``with press(model)`` prunes the cache during pre-fill and leaves decode steps alone."""
    L, B, H, S = 2, 1, 2, 64
    layers = torch.nn.ModuleList([torch.nn.Module() for _ in range(L)])
    for i, lay in enumerate(layers):
        lay.self_attn = _FakeAttn(i)
    model = SimpleNamespace(model=SimpleNamespace(layers=layers))
    cache = SimpleNamespace(key_cache=[None] * L, value_cache=[None] * L, seen_tokens=0)
    kv = to_dev(rand_kv(L, B, H, S, torch.float16, seed=11, permuted=False), dev)
    hidden = torch.zeros(B, S, 8, device=dev)
    press = KnormPress(0.5)
    with press(model):
        for i, lay in enumerate(layers):
            lay.self_attn(hidden_states=hidden, past_key_value=cache, k=kv[i][0], v=kv[i][1])
    assert all(kc.shape[2] == 32 for kc in cache.key_cache) and press.totalTime > 0
    # decode step: cache longer than the query -> untouched
    cache.seen_tokens = 33
    with press(model):
        layers[0].self_attn(hidden_states=hidden[:, :1], past_key_value=cache, k=cache.key_cache[0], v=cache.value_cache[0])
    assert cache.key_cache[0].shape[2] == 32
    assert len(layers[0].self_attn._forward_hooks) == 0             # hooks removed on exit


def _fill_pool_from_case(runner, case, seqs):
    """Copy a synthetic case's pages into the runner's pool following the block manager's tables."""
    for b, s in enumerate(seqs):
        for i, blk in enumerate(case.block_tables[b][:len(s.block_table)]):
            runner.kv_cache[:, :, s.block_table[i]] = case.kv_cache[:, :, blk].to(runner.device)


@pytest.mark.parametrize("backend", ["mlp", "batched", "kvpress", "callable"])
def test_runner_compress_free_and_decode(dev, backend):
    dtype, L, H, img, txt = torch.float16, 2, 4, 300, 213
    S = img + txt
    lens = [S, S, 400]
    case = synth.make_paged_case(seed=31, num_layers=L, batch=3, num_kv_heads=H, seq_lens=lens, dtype=dtype,
                                 shuffle_tables=False, extra_blocks=0)
    torch.manual_seed(12)
    mlp = KVCacheLinearDecoupleCompressor(llava_cfg(L, H), compression_factor=2).to(dev).to(dtype).eval()
    sd = {k: v.detach().cpu().float() for k, v in mlp.state_dict().items()}
    kw = {}
    if backend == "mlp":
        kw["compressor"] = mlp
    elif backend == "batched":
        bat = BatchedGEMMCompressor(L, H, 128, 2)
        bat.load_from_original_compressor(mlp)
        kw["compressor"], kw["batched_compressor"] = mlp, bat
    elif backend == "kvpress":
        kw["compressor"] = KVPressCompressor("streaming_llm", 1.0 - 1.0 / 3)
    else:
        kw["compressor"] = lambda hf, it_len: mlp(hf, it_len=it_len)      # no paged_forward: generic path
    runner = PagedKVRunner(L, H, 128, num_blocks=16, dtype=dtype, device=dev, image_token_len=img, **kw)
    bm = BlockManager(16, 256)
    seqs = [Sequence(list(range(1000 * i, 1000 * i + n))) for i, n in enumerate(lens)]
    for s in seqs:
        bm.allocate(s)
    _fill_pool_from_case(runner, case, seqs)
    tables_before = [list(s.block_table) for s in seqs]
    pool_before = runner.kv_cache.cpu()

    # oracle: the reference's per-sequence loop on the CPU
    ref_pool = pool_before.clone()
    if backend == "kvpress":
        def oracle_comp(hf, i, n):
            return [opress.adapter_compress_layer("streaming_llm", k, v, 1.0 - 1.0 / 3) for k, v in hf]
    else:
        def oracle_comp(hf, i, n):
            return occm.linear_decouple_forward(hf, [img, max(1, n - img)], sd, 2, 1)
    ref_lens, ref_free, ref_ratio = opipe.compress_batch(ref_pool, tables_before, lens, oracle_comp)

    sec, ratio = runner.compress_kv_cache_batch(seqs)
    assert sec > 0 and abs(ratio - ref_ratio) < 1e-9
    for i, s in enumerate(seqs):
        assert runner._compressed_lens[s.seq_id] == ref_lens[i]
        assert runner.get_compressed_block_count(s.seq_id) == -(-ref_lens[i] // 256)
        assert runner._blocks_to_free.get(s.seq_id, []) == ref_free.get(i, [])
    got_pool = runner.kv_cache.cpu()
    for i, (tab, n) in enumerate(zip(tables_before, lens)):
        C = ref_lens[i]
        g = opaged.extract_kv(got_pool, tab, n)
        r = opaged.extract_kv(ref_pool, tab, n)
        for (gk, gv), (rk, rv) in zip(g, r):
            if backend == "kvpress":
                assert torch.equal(gk, rk) and torch.equal(gv, rv)     # gathered bytes and stale tail: bit-exact
            else:
                assert_mlp_close(gk[:, :, :C], rk[:, :, :C], dtype)
                assert torch.equal(gk[:, :, C:], rk[:, :, C:]) and torch.equal(gv[:, :, C:], rv[:, :, C:])

    # block release: tables truncated, tail ids appended to the free deque in table order
    free_before = list(bm.free_block_ids)
    freed = free_compressed_blocks(bm, runner, seqs)
    expect_tail = [b for i in range(3) for b in ref_free.get(i, [])]
    assert freed == len(expect_tail) and list(bm.free_block_ids) == free_before + expect_tail
    for i, s in enumerate(seqs):
        assert s.block_table == tables_before[i][:-(-ref_lens[i] // 256)]
        assert s.kv_cache_len == ref_lens[i] and s.is_compressed
    assert len(bm.free_block_ids) + len(bm.used_block_ids) == 16

    # one decode step's metadata follows the compressed lengths
    for s in seqs:
        s.append_token(7)
        bm.may_append(s)
    ids, pos = runner.prepare_decode(seqs)
    from fastcache_amd.utils.context import get_context
    ctx = get_context()
    assert pos.tolist() == [s.kv_cache_len for s in seqs] == ctx.context_lens.tolist()
    exp_slots = [s.block_table[s.kv_cache_len // 256] * 256 + s.kv_cache_len % 256 for s in seqs]
    assert ctx.slot_mapping.tolist() == exp_slots and ctx.block_tables.shape[0] == 3


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_extract_and_write_back_of_layer_lists(dev, dtype):
    """_extract_kv_cache_fast / _write_compressed_kv_cache_fast against the oracle's paged copies: the write-back takes
    the compressor's list of per-layer tensors as it is (slices of larger tensors: one launch from a table of layer
    addresses) and falls back to stacking when the tensors do not share one geometry; slots past C keep their bytes."""
    L, H, S, C, bs = 3, 2, 300, 117, 64
    case = synth.make_paged_case(seed=4, num_layers=L, batch=2, num_kv_heads=H, seq_lens=[S, 200], dtype=dtype, block_size=bs)
    r = PagedKVRunner(L, H, 128, case.kv_cache.shape[2], dtype, dev, block_size=bs)
    r.kv_cache.copy_(case.kv_cache.to(dev))
    table = case.block_tables[0]
    hf = r._extract_kv_cache_fast(table, S)
    ref = opaged.extract_kv(case.kv_cache, table, S)
    for (k, v), (rk, rv) in zip(hf, ref):
        assert torch.equal(k.cpu(), rk) and torch.equal(v.cpu(), rv)
    g = torch.Generator().manual_seed(9)
    wide = [(torch.randn(1, H, S, 128, generator=g).to(dtype).to(dev), torch.randn(1, H, S, 128, generator=g).to(dtype).to(dev))
            for _ in range(L)]
    for variant in ("slices", "mixed"):
        comp = [(k[:, :, :C], v[:, :, :C]) for k, v in wide]                  # non-contiguous, one geometry
        if variant == "mixed":
            comp[1] = (comp[1][0].contiguous(), comp[1][1].contiguous())       # one layer laid out differently
        pool = case.kv_cache.clone()
        opaged.write_back(pool, [(k.cpu(), v.cpu()) for k, v in comp], table)
        r.kv_cache.copy_(case.kv_cache.to(dev))
        r._write_compressed_kv_cache_fast(comp, table)
        torch.cuda.synchronize()
        assert torch.equal(r.kv_cache.cpu().view(torch.uint8), pool.view(torch.uint8)), variant


def test_background_compression_event_protocol(dev):
    dtype, L, H, S = torch.bfloat16, 2, 2, 600
    case = synth.make_paged_case(seed=4, num_layers=L, batch=2, num_kv_heads=H, seq_lens=[S, S], dtype=dtype,
                                 shuffle_tables=False, extra_blocks=0)
    runner = PagedKVRunner(L, H, 128, num_blocks=8, dtype=dtype, device=dev, image_token_len=0,
                           compressor=KVPressCompressor("knorm", 0.5))
    bm = BlockManager(8, 256)
    seqs = [Sequence(list(range(i * 1000, i * 1000 + S))) for i in range(2)]
    for s in seqs:
        bm.allocate(s)
    _fill_pool_from_case(runner, case, seqs)
    sync_runner = PagedKVRunner(L, H, 128, num_blocks=8, dtype=dtype, device=dev, image_token_len=0,
                                compressor=KVPressCompressor("knorm", 0.5))
    sync_runner.kv_cache.copy_(runner.kv_cache)
    sync_runner.compress_kv_cache_batch(seqs)
    done = runner.start_background_compression(seqs)
    assert done is not None
    runner.wait_compression(done)
    assert done.query()
    assert torch.equal(runner.kv_cache, sync_runner.kv_cache)       # same result as the synchronous path
    assert runner._compressed_lens == sync_runner._compressed_lens
    assert PagedKVRunner(L, H, 128, 2, dtype, dev).start_background_compression(seqs) is None
    runner.clear_compressed_lens([seqs[0].seq_id])
    assert seqs[0].seq_id not in runner._compressed_lens and seqs[1].seq_id in runner._compressed_lens


def test_async_compression_manager_states_and_effective_len(dev):
    """Per-sequence states, events and the effective KV length of the asynchronous manager; the pages end up
    identical to the synchronous path's."""
    from fastcache_amd.engine.async_compress import AsyncCompressionManager, CompressionState
    dtype, L, H, S = torch.float16, 2, 2, 700
    case = synth.make_paged_case(seed=8, num_layers=L, batch=2, num_kv_heads=H, seq_lens=[S, S], dtype=dtype,
                                 shuffle_tables=False, extra_blocks=0)
    mk = lambda: PagedKVRunner(L, H, 128, num_blocks=8, dtype=dtype, device=dev, image_token_len=0,
                               compressor=KVPressCompressor("knorm", 0.5))
    runner, sync_runner = mk(), mk()
    bm = BlockManager(8, 256)
    seqs = [Sequence(list(range(i * 1000, i * 1000 + S))) for i in range(2)]
    for s in seqs:
        bm.allocate(s)
    _fill_pool_from_case(runner, case, seqs)
    sync_runner.kv_cache.copy_(runner.kv_cache)
    sync_runner.compress_kv_cache_batch(seqs)

    mgr = AsyncCompressionManager(runner)
    assert mgr.get_effective_kv_len(seqs[0]) == S and not mgr.is_compression_complete(seqs[0].seq_id)
    mgr.start_async_compression(seqs, image_len=0)
    mgr.wait_for_compression(seqs[0].seq_id)
    mgr.wait_all_compressions()
    for s in seqs:
        assert mgr.seq_states[s.seq_id] == CompressionState.COMPLETED and mgr.is_compression_complete(s.seq_id)
        assert mgr.get_effective_kv_len(s) == 350 == runner._compressed_lens[s.seq_id]
        assert mgr.seq_original_lens[s.seq_id] == S
    assert torch.equal(runner.kv_cache, sync_runner.kv_cache)
    mgr.cleanup_seq(seqs[0].seq_id)
    assert seqs[0].seq_id not in mgr.seq_states and mgr.get_effective_kv_len(seqs[0]) == S
    # a failing compressor leaves the sequence uncompressed instead of raising (the reference's fallback)
    bad = PagedKVRunner(L, H, 128, num_blocks=8, dtype=dtype, device=dev, image_token_len=0,
                        compressor=lambda kv, it_len=None: (_ for _ in ()).throw(RuntimeError("boom")))
    bmgr = AsyncCompressionManager(bad)
    bmgr.start_async_compression(seqs[:1], image_len=0)
    bmgr.wait_all_compressions()
    assert bmgr.seq_states[seqs[0].seq_id] == CompressionState.NONE and bmgr.get_effective_kv_len(seqs[0]) == S
    # a compressor that works in place and fails after it may have launched: the rows are no longer trustworthy,
    # the sequence is marked FAILED and asking for its length raises instead of handing out a stale number
    class Halfway:
        def paged_forward(self, kv_cache, block_tables, seq_lens, seq_len, *a, **k):
            from fastcache_amd import _lib, ops
            ops.knorm_score(_lib.paged_view(kv_cache[0], block_tables, seq_lens, seq_len), kv_cache.device)
            raise RuntimeError("second launch rejected")
    half = PagedKVRunner(L, H, 128, num_blocks=8, dtype=dtype, device=dev, image_token_len=0, compressor=Halfway())
    hmgr = AsyncCompressionManager(half)
    hmgr.start_async_compression(seqs[:1], image_len=0)
    hmgr.wait_all_compressions()
    assert hmgr.seq_states[seqs[0].seq_id] == CompressionState.FAILED
    with pytest.raises(Exception, match="prefill again"):
        hmgr.get_effective_kv_len(seqs[0])
    # the same kind of compressor failing in its host-side checks, before anything was enqueued: the cache is as it was
    class Early:
        def paged_forward(self, *a, **k):
            raise TypeError("image segment cannot be compressed")
    early = PagedKVRunner(L, H, 128, num_blocks=8, dtype=dtype, device=dev, image_token_len=0, compressor=Early())
    emgr = AsyncCompressionManager(early)
    emgr.start_async_compression(seqs[:1], image_len=0)
    emgr.wait_all_compressions()
    assert emgr.seq_states[seqs[0].seq_id] == CompressionState.NONE and emgr.get_effective_kv_len(seqs[0]) == S
    assert AsyncCompressionManager(PagedKVRunner(L, H, 128, 2, dtype, dev)).start_async_compression(seqs) is None


def test_pipeline_async_compressor_round_robin(dev):
    from fastcache_amd.engine.async_compress import CompressionState, PipelineAsyncCompressor
    dtype, L = torch.float16, 2
    comp = KVPressCompressor("streaming_llm", 0.5)
    pipe = PipelineAsyncCompressor(comp, num_streams=2)
    written = {}
    events = []
    kvs = [to_dev(rand_kv(L, 1, 2, 300 + 20 * i, dtype, seed=i), dev) for i in range(3)]
    for i, kv in enumerate(kvs):
        events.append(pipe.submit_compression(i, kv, [i], kv[0][0].shape[2], [0, kv[0][0].shape[2]],
                                              lambda out, table, i=i: written.__setitem__(i, (out, table))))
    assert pipe.current_stream_idx == 1            # three submissions over two streams
    for i, ev in enumerate(events):
        pipe.wait_compression(i)
        assert ev.query() and pipe.is_compression_ready(i)
        assert pipe.seq_states[i] == CompressionState.COMPLETED
        n = (300 + 20 * i) // 2
        assert pipe.get_compressed_len(i) == n and written[i][1] == [i]
        ref = comp(kvs[i], it_len=[0, 300 + 20 * i])
        assert all(torch.equal(a[0], b[0]) and torch.equal(a[1], b[1]) for a, b in zip(written[i][0], ref))
    pipe.cleanup(0)
    assert pipe.get_compressed_len(0) is None and not pipe.is_compression_ready(0)


def test_lazy_compression_engine_on_the_pool(dev):
    """Threshold-triggered batch compression over a real pool: when the free blocks run out the three running
    sequences are compressed in ONE batched pass, their pages equal the oracle's per-sequence loop, the freed
    blocks admit the waiting request, and every block is back in the pool at the end."""
    from fastcache_amd.engine.llm_engine import CompressionEngine, LazyCompressionEngine, SamplingParams
    from fastcache_amd.engine.scheduler import LlavaScheduler
    dtype, L, H, S = torch.float16, 2, 2, 600
    case = synth.make_paged_case(seed=17, num_layers=L, batch=4, num_kv_heads=H, seq_lens=[S] * 4, dtype=dtype,
                                 shuffle_tables=False, extra_blocks=0)
    ratio = 1.0 - 1.0 / 3
    runner = PagedKVRunner(L, H, 128, num_blocks=9, dtype=dtype, device=dev, image_token_len=0,
                           compressor=KVPressCompressor("streaming_llm", ratio))
    sched = LlavaScheduler(max_num_seqs=8, max_num_batched_tokens=600, eos=-1, num_kvcache_blocks=9)
    order = {}

    def model_step(seqs, is_prefill):
        if is_prefill:                         # "prefill": the sequence's KV rows appear in its pages
            for s in seqs:
                b = order.setdefault(s.seq_id, len(order))
                for i, blk in enumerate(s.block_table):
                    runner.kv_cache[:, :, blk] = case.kv_cache[:, :, case.block_tables[b][i]].to(dev)
        return [3] * len(seqs)

    llm = CompressionEngine(sched, runner, model_step)
    eng = LazyCompressionEngine(llm, compression_threshold=0.4)
    seqs = [eng.add_request(list(range(i * 1000, i * 1000 + S)), SamplingParams(max_tokens=4, ignore_eos=True))
            for i in range(4)]
    for _ in range(3):                         # one prefill per step (600 batched tokens)
        eng.step()
    assert len(sched.block_manager.free_block_ids) == 0 and len(sched.waiting) == 1
    tables_before = [list(s.block_table) for s in seqs[:3]]
    ref_pool = runner.kv_cache.cpu()
    lens = [len(s) for s in seqs[:3]]          # 601: the lazy path compresses len(seq) rows, like the reference
    ref_lens, _, _ = opipe.compress_batch(
        ref_pool, tables_before, lens,
        lambda hf, i, n: [opress.adapter_compress_layer("streaming_llm", k, v, ratio) for k, v in hf])
    eng.step()                                 # trigger: compress the three, then prefill the fourth
    assert eng.compression_count == 1 and len(sched.running) == 4 and not sched.waiting
    for s, c, tab in zip(seqs[:3], ref_lens.values(), tables_before):
        assert s.is_compressed and len(s.block_table) == 1 and s.block_table == tab[:1]
        assert s.kv_cache_len == c
        got = runner.kv_cache[:, :, s.block_table[0], :c].cpu()
        assert torch.equal(got, ref_pool[:, :, tab[0], :c])
    steps = 0
    while not eng.is_finished():
        eng.step()
        steps += 1
        assert steps < 50
    bm = sched.block_manager
    assert len(bm.free_block_ids) == 9 and not bm.used_block_ids and llm.total_freed_blocks == 6


@pytest.mark.parametrize("backend", ["mlp", "kvpress", "knorm-press", "snapkv-press"])
def test_decode_overlap_compression_splices_generated_rows(dev, backend):
    """A few layers per decode step on a side stream; at the end the pages hold compress(prefill rows) followed by
    the rows generated meanwhile, and the untouched pages served the steps in between."""
    from fastcache_amd.engine.decode_overlap import DecodeOverlapCompressor
    dtype, L, H, img = torch.float16, 5, 2, 100
    lens = [600, 600, 520]
    case = synth.make_paged_case(seed=41, num_layers=L, batch=3, num_kv_heads=H, seq_lens=lens, dtype=dtype,
                                 shuffle_tables=False, extra_blocks=0, reserve_tokens=8)
    if backend == "mlp":
        torch.manual_seed(2)
        comp = KVCacheLinearDecoupleCompressor(llava_cfg(L, H), compression_factor=2).to(dev).to(dtype).eval()
        sd = {k: v.detach().cpu().float() for k, v in comp.state_dict().items()}
        oracle = lambda hf, n: occm.linear_decouple_forward(hf, [img, max(1, n - img)], sd, 2, 1)
    elif backend == "kvpress":
        comp = KVPressCompressor("knorm", 0.5)
        oracle = lambda hf, n: [opress.adapter_compress_layer("knorm", k, v, 0.5) for k, v in hf]
    elif backend == "knorm-press":
        comp = KnormPress(0.5)
        oracle = lambda hf, n: opipe.knorm_press_compressor(0.5)(hf, 0, n)
    else:
        # the press object with its window queries named by sequence: the two length groups (600, 600 | 520) and the
        # layer chunks of every step find their own slices again
        from fastcache_amd.presses import SnapKVPress
        comp = SnapKVPress(0.5, window_size=16, kernel_size=5)
        wq = torch.randn(L, 3, 2 * H, 16, 128, generator=torch.Generator().manual_seed(5)).to(dtype)
    runner = PagedKVRunner(L, H, 128, num_blocks=16, dtype=dtype, device=dev, image_token_len=img, compressor=comp)
    bm = BlockManager(16, 256)
    seqs = [Sequence(list(range(1000 * i, 1000 * i + n))) for i, n in enumerate(lens)]
    for s in seqs:
        bm.allocate(s)
    _fill_pool_from_case(runner, case, seqs)
    before = runner.kv_cache.cpu()
    if backend == "snapkv-press":
        comp.set_window_queries(wq.to(dev), seq_ids=[s.seq_id for s in seqs])
        index_of = {s.seq_id: i for i, s in enumerate(seqs)}
        oracle = lambda hf, n, _s=None: None      # replaced per sequence below

    ov = DecodeOverlapCompressor(runner, layers_per_step=2)
    ov.start_decode_overlap_compression(seqs)
    assert all(ov.pending(s.seq_id) for s in seqs)
    g = torch.Generator().manual_seed(77)
    appended = {s.seq_id: [] for s in seqs}
    steps = 0
    done = []
    while len(done) < 3:
        # a decode step: one new KV row per sequence at position len(seq), then the sampled token is appended
        for s in seqs:
            row = torch.randn(2, L, H, 128, generator=g).to(dtype)
            pos = len(s)
            blk = s.block_table[pos // 256]
            runner.kv_cache[:, :, blk, pos % 256] = row.to(dev)
            appended[s.seq_id].append(row)
            s.append_token(5)
        steps += 1
        finished = ov.step_decode_overlap_compression(seqs)
        if steps < 3:
            assert finished == []                                   # 5 layers, 2 per step
            # the pages still hold the uncompressed prefix while compression is under way
            assert torch.equal(runner.kv_cache[:, :, seqs[0].block_table[0], :100].cpu(),
                               before[:, :, seqs[0].block_table[0], :100])
        done += finished
    assert steps == 3 and {s.seq_id for s in done} == {s.seq_id for s in seqs}
    torch.cuda.synchronize()
    for s, n in zip(seqs, lens):
        hf = opaged.extract_kv(before, s.block_table, n)
        if backend == "snapkv-press":
            i = index_of[s.seq_id]
            ref = opipe.snapkv_press_compressor(wq[:, i:i + 1], 0.5, 16, 5)(hf, 0, n)
            ties = any(bool(opress.near_tie_rows(opress.snapkv_score(wq[l, i:i + 1], k, 16, 5)[..., :n - 16],
                                                 n // 2 - 16).any()) for l, (k, _) in enumerate(hf))
            assert not ties, "a score within 1e-5 of a threshold: pick another seed"
        else:
            ref = oracle(hf, n)
        C = ref[0][0].shape[2]
        assert runner._compressed_lens[s.seq_id] == C + 3 and not ov.pending(s.seq_id)
        got = opaged.extract_kv(runner.kv_cache.cpu(), s.block_table, C + 3)
        for layer in range(L):
            for p in range(2):
                if backend == "mlp":
                    assert_mlp_close(got[layer][p][:, :, :C], ref[layer][p], dtype)
                else:
                    assert torch.equal(got[layer][p][:, :, :C], ref[layer][p])
                tail = torch.stack([r[p, layer] for r in appended[s.seq_id]], dim=1).unsqueeze(0)   # [1, H, 3, D]
                assert torch.equal(got[layer][p][:, :, C:], tail)
    if backend == "snapkv-press":
        assert not comp._paged_inputs                                   # every slice was used up by the last layer chunk
    freed = free_compressed_blocks(bm, runner, seqs)
    assert freed == sum(-(-(n + 3) // 256) - (-(-(runner_len) // 256)) for n, runner_len in
                        zip(lens, [s.kv_cache_len for s in seqs]))


@pytest.mark.parametrize("backend", ["mlp", "batched", "hybrid", "kvpress-knorm", "kvpress-streaming"])
def test_runner_ragged_batch_in_one_pass(dev, backend):
    """Nine running sequences of nine different lengths (the state a lazy compression trigger finds) compressed by
    ONE paged_forward call, against the reference's per-sequence loop on the CPU."""
    dtype, L, H, img = torch.bfloat16, 2, 2, 100
    lens = [700, 257, 256, 255, 101, 1000, 333, 512, 130]
    case = synth.make_paged_case(seed=77, num_layers=L, batch=len(lens), num_kv_heads=H, seq_lens=lens, dtype=dtype,
                                 shuffle_tables=False, extra_blocks=0)
    torch.manual_seed(2)
    kw, image_len = {}, img
    if backend in ("mlp", "batched"):
        mlp = KVCacheLinearDecoupleCompressor(llava_cfg(L, H), compression_factor=2).to(dev).to(dtype).eval()
        sd = {k: v.detach().cpu().float() for k, v in mlp.state_dict().items()}
        kw["compressor"] = mlp
        if backend == "batched":
            bat = BatchedGEMMCompressor(L, H, 128, 2)
            bat.load_from_original_compressor(mlp)
            kw["batched_compressor"] = bat
        oracle_comp = lambda hf, i, n: occm.linear_decouple_forward(hf, [img, max(1, n - img)], sd, 2, 1)
    elif backend == "hybrid":
        image_len = 0
        cfg = SimpleNamespace(architectures=["MiniCPMV"], num_hidden_layers=L, num_key_value_heads=H,
                              num_attention_heads=H, hidden_size=H * 128)
        hyb = KVCacheHybridCompressor(cfg, compression_factor=5, min_seq_len=30).to(dev).to(dtype).eval()
        sd = {k: v.detach().cpu().float() for k, v in hyb.state_dict().items()}
        kw["compressor"] = hyb
        oracle_comp = lambda hf, i, n: occm.hybrid_forward(hf, [0, n], sd, 5, 30)      # 101 and 130 tokens pass through
    else:
        method = backend.split("-")[1].replace("streaming", "streaming_llm")
        kw["compressor"] = KVPressCompressor(method, 1.0 - 1.0 / 3)
        oracle_comp = lambda hf, i, n: [opress.adapter_compress_layer(method, k, v, 1.0 - 1.0 / 3) for k, v in hf]
    nb = case.kv_cache.shape[2]
    runner = PagedKVRunner(L, H, 128, num_blocks=nb, dtype=dtype, device=dev, image_token_len=image_len, **kw)
    bm = BlockManager(nb, 256)
    seqs = [Sequence(list(range(2000 * i, 2000 * i + n))) for i, n in enumerate(lens)]
    for s in seqs:
        bm.allocate(s)
    _fill_pool_from_case(runner, case, seqs)
    tables_before = [list(s.block_table) for s in seqs]
    ref_pool = runner.kv_cache.cpu()
    ref_lens, ref_free, ref_ratio = opipe.compress_batch(ref_pool, tables_before, lens, oracle_comp)

    comp = runner._active_compressor()
    calls = []
    inner = comp.paged_forward
    comp.paged_forward = lambda *a, **k: (calls.append(1), inner(*a, **k))[1]
    sec, ratio = runner.compress_kv_cache_batch(seqs)
    assert len(calls) == 1 and abs(ratio - ref_ratio) < 1e-9
    got_pool = runner.kv_cache.cpu()
    for i, (s, tab, n) in enumerate(zip(seqs, tables_before, lens)):
        C = ref_lens[i]
        assert runner._compressed_lens[s.seq_id] == C
        assert runner._blocks_to_free.get(s.seq_id, []) == ref_free.get(i, [])
        for (gk, gv), (rk, rv) in zip(opaged.extract_kv(got_pool, tab, n), opaged.extract_kv(ref_pool, tab, n)):
            if backend.startswith("kvpress"):
                assert torch.equal(gk, rk) and torch.equal(gv, rv)
            else:
                assert_mlp_close(gk[:, :, :C], rk[:, :, :C], dtype)
                assert_mlp_close(gv[:, :, :C], rv[:, :, :C], dtype)
                assert torch.equal(gk[:, :, C:], rk[:, :, C:]) and torch.equal(gv[:, :, C:], rv[:, :, C:])
