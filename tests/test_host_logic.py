"""Host-side logic without a GPU: block manager and sequence state against the oracle's restatement,
module construction (parameter names and seeded initialisation), press arithmetic, error paths."""
from types import SimpleNamespace

import pytest
import torch

from fastcache_amd.engine import BlockManager, Sequence
from fastcache_amd.engine.kv_runner import PagedKVRunner
from fastcache_amd.engine.llm_hooks import free_compressed_blocks
from fastcache_amd.kernels import BatchedGEMMCompressor, KVPressCompressor, MiniCPMKVCompressor, create_kvpress_compressor
from fastcache_amd.presses import KnormPress, SnapKVPress, StreamingLLMPress, press_select
from fastcache_amd.utils_ccm import KVCacheHybridCompressor, KVCacheLinearDecoupleCompressor
from oracle import blocks as oblocks
from oracle import ccm as occm


def llava_cfg(L=2, H=4, D=128):
    return SimpleNamespace(text_config=SimpleNamespace(num_hidden_layers=L, num_key_value_heads=H, hidden_size=H * D,
                                                       head_dim=D, num_attention_heads=H))


def minicpm_cfg(L=2, Hq=28, Hkv=4, D=128):
    return SimpleNamespace(architectures=["MiniCPMV"], num_hidden_layers=L, num_key_value_heads=Hkv,
                           num_attention_heads=Hq, hidden_size=Hq * D)


class FakeRunner:
    def __init__(self, lens):
        self._compressed_lens = dict(lens)
        self._blocks_to_free = {}
        self.block_size = 256

    def get_compressed_block_count(self, seq_id):
        if seq_id not in self._compressed_lens:
            return -1
        return -(-self._compressed_lens[seq_id] // self.block_size)


def test_block_manager_matches_oracle_through_compression_and_decode():
    bm = BlockManager(num_blocks=12, block_size=256)
    pool = oblocks.PoolState(num_blocks=12)
    seqs, states = [], []
    base = 0
    for n in (1000, 300, 700):
        s = Sequence(list(range(base, base + n)))       # unique tokens: every block is a cache miss
        base += n
        bm.allocate(s)
        st = oblocks.SeqState(s.seq_id, n)
        oblocks.allocate(pool, st)
        seqs.append(s)
        states.append(st)
        assert s.block_table == st.block_table
    comp = {seqs[0].seq_id: 500, seqs[2].seq_id: 140}    # seqs[1] stays uncompressed
    runner = FakeRunner(comp)
    freed = free_compressed_blocks(bm, runner, seqs)
    ofreed = sum(len(oblocks.free_compressed_blocks(pool, st, comp.get(st.seq_id))) for st in states)
    assert freed == ofreed == 4
    for s, st in zip(seqs, states):
        assert s.block_table == st.block_table and s.kv_cache_len == st.kv_cache_len
        assert s.is_compressed == st.is_compressed
    assert list(bm.free_block_ids) == list(pool.free)
    assert bm.used_block_ids == pool.used
    assert len(bm.free_block_ids) + len(bm.used_block_ids) == 12
    # decode: kv length grows by one per token; a block is taken exactly when kv_len % 256 == 1
    s, st = seqs[0], states[0]
    for step in range(20):
        s.append_token(1)
        st.append_token()
        assert bm.can_append(s) == oblocks.can_append(pool, st)
        bm.may_append(s)
        oblocks.may_append(pool, st)
        assert s.block_table == st.block_table and s.kv_cache_len == st.kv_cache_len == 501 + step
    assert len(s.block_table) == 3 and list(bm.free_block_ids) == list(pool.free)
    # the last kept block lost its prefix-cache hash
    assert bm.blocks[seqs[2].block_table[-1]].hash == -1


def test_block_manager_prefix_cache_and_specific_free():
    bm = BlockManager(8, 256)
    a = Sequence(list(range(600)))
    b = Sequence(list(range(600)))                      # same prefix: the two full blocks are shared
    bm.allocate(a)
    bm.allocate(b)
    assert a.block_table[:2] == b.block_table[:2] and a.block_table[2] != b.block_table[2]
    assert b.num_cached_tokens == 512
    assert bm.blocks[a.block_table[0]].ref_count == 2
    bm.free_specific_blocks([a.block_table[0], 7])      # 7 is not in use: ignored
    assert bm.blocks[a.block_table[0]].ref_count == 1 and a.block_table[0] in bm.used_block_ids
    bm.free_blocks_after_compression(b, 1)
    assert len(b.block_table) == 1
    bm.deallocate(a)
    assert not a.block_table


def test_shared_prefix_pages_get_a_private_copy_before_they_are_rewritten():
    """Two prompts with the same first 512 tokens share two pages.  A compression rewrites leading pages in place:
    the page manager hands the sequence a fresh page for each shared one it will write, forgets the content keys
    of rewritten pages, and a later request with that prefix is served only by pages that still hold prompt rows."""
    bm = BlockManager(10, 256)
    a = Sequence(list(range(600)))
    b = Sequence(list(range(512)) + [9] * 88)
    bm.allocate(a)
    bm.allocate(b)
    assert a.block_table[:2] == b.block_table[:2] and bm.shared_positions(a, 3) == [0, 1]
    assert bm.shared_positions(a, 1) == [0]
    old = a.block_table[0]
    free_before = len(bm.free_block_ids)
    moved = bm.unshare(a, [0])                            # a keeps 100 rows: it rewrites page 0 only
    assert moved == [(old, a.block_table[0])] and a.block_table[0] != b.block_table[0] == old
    assert bm.blocks[old].ref_count == 1 and bm.blocks[a.block_table[0]].ref_count == 1
    assert len(bm.free_block_ids) == free_before - 1 and bm.blocks[a.block_table[0]].hash == -1
    free_compressed_blocks(bm, FakeRunner({a.seq_id: 100}), [a])
    assert len(a.block_table) == 1 and bm.blocks[b.block_table[1]].ref_count == 1      # a let go of shared page 1
    c = Sequence(list(range(600)))                       # same prefix: served by b's untouched pages
    bm.allocate(c)
    assert c.block_table[:2] == b.block_table[:2] and c.num_cached_tokens == 512
    bm.deallocate(c)
    free_compressed_blocks(bm, FakeRunner({b.seq_id: 300}), [b])       # b rewrites both of its pages, keeps both
    assert all(bm.blocks[p].hash == -1 and not bm.blocks[p].token_ids for p in b.block_table[:2])
    d = Sequence(list(range(600)))
    bm.allocate(d)
    assert d.num_cached_tokens == 0 and not set(d.block_table) & set(b.block_table)
    # too few free pages: refused with the tables as they were
    e, f = Sequence(list(range(7000, 7512))), Sequence(list(range(7000, 7512)))
    bm2 = BlockManager(2, 256)
    bm2.allocate(e)
    bm2.allocate(f)
    before = list(e.block_table)
    with pytest.raises(RuntimeError, match="only 0 pages are free"):
        bm2.unshare(e, [0, 1])
    assert e.block_table == before and bm2.blocks[before[0]].ref_count == 2


def test_runner_refuses_a_batch_that_would_rewrite_a_page_twice():
    """Without a page manager the runner cannot copy a shared page; it refuses before any launch."""
    from fastcache_amd._lib import FastcacheError
    runner = PagedKVRunner(1, 1, 128, num_blocks=4, dtype=torch.float16, device="cpu", image_token_len=0,
                           compressor=KVPressCompressor("streaming_llm", 0.5))
    a, b = Sequence(list(range(300))), Sequence(list(range(300)))
    a.block_table, b.block_table = [0, 1], [0, 2]
    with pytest.raises(FastcacheError, match="page 0 belongs to several sequences"):
        runner._compress_enqueue([a, b], 0)
    assert not runner._launch_started and not runner._compressed_lens


def test_synthetic_pool_scatter_is_the_page_formula():
    """``synth.scatter_into_pool`` (one indexed store per plane and layer) against the defining loop
    ``pool[table[s // 256], s % 256] = dense[s]`` on a shuffled, ragged case; untouched slots keep the fill value."""
    from fastcache_amd import synth
    lens = [300, 17, 256, 513]
    case = synth.make_paged_case(seed=5, num_layers=2, batch=4, num_kv_heads=3, seq_lens=lens, dtype=torch.float16,
                                 keep_dense=True, fill_value=7.0, block_size=256)
    want = torch.full_like(case.kv_cache, 7.0)
    for layer in range(2):
        for p, dense in enumerate((case.dense_k, case.dense_v)):
            for b, (tab, n) in enumerate(zip(case.block_tables, lens)):
                for t in range(n):
                    want[p, layer, tab[t // 256], t % 256] = dense[layer, b, :, t]
    assert torch.equal(case.kv_cache.view(torch.int16), want.view(torch.int16))
    assert sorted(sum(case.block_tables, [])) != sum(case.block_tables, [])       # the tables really are shuffled


def test_runner_adopts_an_existing_pool():
    """``PagedKVRunner.adopt``: a runner over the host runner's own pool tensor and ``_compressed_lens`` dictionary."""
    pool = torch.zeros(2, 3, 5, 256, 4, 128, dtype=torch.float16)
    lens = {}
    r = PagedKVRunner.adopt(pool, compressor=KVPressCompressor("knorm", 0.5), image_token_len=0, compressed_lens=lens)
    assert r.kv_cache is pool and r._compressed_lens is lens
    assert (r.num_hidden_layers, r.num_key_value_heads, r.head_dim, r.block_size) == (3, 4, 128, 256)
    assert r.block_manager is None and not r._launch_started and r.get_compressed_block_count(7) == -1
    lens[7] = 300
    assert r.get_compressed_block_count(7) == 2
    with pytest.raises(Exception, match="kv_cache must be"):
        PagedKVRunner.adopt(pool[0])


def test_sequence_state():
    s = Sequence([1, 2, 3])
    assert not s.is_compressed and s.kv_cache_len == 3 and s.kv_num_blocks == 1
    s.append_token(4)
    assert s.kv_cache_len == 4
    s.kv_cache_len = 300
    s.append_token(5)
    assert s.is_compressed and s.kv_cache_len == 301 and s.kv_num_blocks == 2 and len(s) == 5


def test_module_parameter_names_and_seeded_init():
    torch.manual_seed(123)
    m = KVCacheLinearDecoupleCompressor(llava_cfg(), compression_factor=2, min_seq_len=1)
    sd = occm.reference_init_state_dict("linear_decouple", 2, 128, 2, seed=123)
    msd = m.state_dict()
    assert set(msd) == set(sd)
    assert all(torch.equal(msd[k], sd[k]) for k in sd)
    assert list(msd)[0] == "compress_tk.0.0.weight" and "attention.1.bias" in msd
    assert (m.n_layer, m.nhead, m.head_dim, m.compression_factor, m.min_seq_len) == (2, 4, 128, 2, 1)

    torch.manual_seed(5)
    h = KVCacheHybridCompressor(minicpm_cfg(), compression_factor=5, min_seq_len=2)
    hsd = occm.reference_init_state_dict("hybrid", 2, 128, 5, seed=5)
    assert set(h.state_dict()) == set(hsd) and all(torch.equal(h.state_dict()[k], hsd[k]) for k in hsd)
    assert h.compress_ik is None and h.compress_iv is None and h.head_dim == 128

    torch.manual_seed(6)
    mc = MiniCPMKVCompressor(minicpm_cfg())
    csd = occm.reference_init_state_dict("minicpm", 2, 128, 5, seed=6)
    assert all(torch.equal(mc.state_dict()[k], csd[k]) for k in csd)
    assert (mc.compression_factor, mc.min_seq_len) == (5, 2)


def test_batched_compressor_layout_and_loading():
    torch.manual_seed(1)
    orig = KVCacheLinearDecoupleCompressor(llava_cfg(), compression_factor=2)
    b = BatchedGEMMCompressor(num_layers=2, num_heads=4, head_dim=128, compression_factor=2)
    assert b.w1_tk.shape == (2, 256, 128) and b.b3_iv.shape == (2, 128)
    assert float(b.b1_tk.abs().sum()) == 0                     # zero biases, Xavier weights
    b.load_from_original_compressor(orig)
    ow = occm.batched_weights_from_state_dict(orig.state_dict(), "compress_iv", 2)
    for got, want in zip((b.w1_iv, b.b1_iv, b.w2_iv, b.b2_iv, b.w3_iv, b.b3_iv), ow):
        assert torch.equal(got.detach(), want)
    names = [n for n, _ in b.named_parameters()]
    assert names[:6] == ["w1_tk", "b1_tk", "w2_tk", "b2_tk", "w3_tk", "b3_tk"]


def test_kvpress_adapter_surface():
    with pytest.raises(ValueError):
        KVPressCompressor(method="nope")
    c = create_kvpress_compressor("knorm", compression_factor=5)
    assert c.compression_ratio == 1.0 - 1.0 / 5
    assert c.get_compressed_length(1000) == 199               # double-arithmetic truncation kept
    assert c.get_compressed_length(2) == 1
    assert abs(c.compression_factor - 5.0) < 1e-9
    assert "knorm" in repr(c) and len(KVPressCompressor.SUPPORTED_METHODS) == 8
    cfg = SimpleNamespace(num_hidden_layers=3, num_attention_heads=8, num_key_value_heads=2, hidden_size=1024)
    c2 = KVPressCompressor("snapkv", 0.5, config=cfg)
    assert (c2.num_layers, c2.num_kv_heads, c2.head_dim) == (3, 2, 128)
    assert c2.forward([]) == []


def test_press_objects_surface():
    p = press_select("SnapKV", 0.75)
    assert isinstance(p, SnapKVPress) and p.window_size == 64 and p.kernel_size == 5 and p.totalTime == 0
    assert p.n_kept(4096) == 1024
    assert SnapKVPress(0.75, window_in_budget=False).n_kept(4096) == 1088
    assert isinstance(press_select("anything else", 0.5), KnormPress)
    assert isinstance(press_select("StreamingLLM", 0.5), StreamingLLMPress)
    from fastcache_amd.presses import TOVAPress
    assert isinstance(press_select("TOVA", 0.5), TOVAPress)
    from fastcache_amd.presses import ExpectedAttentionPress, SimpleKVQuantizer
    ea = press_select("ExpectedAttention", 0.5)
    assert isinstance(ea, ExpectedAttentionPress) and (ea.n_future_positions, ea.n_sink, ea.use_covariance,
                                                        ea.use_vnorm, ea.epsilon) == (512, 4, True, True, 0.0)
    assert isinstance(press_select("Quantized"), SimpleKVQuantizer)
    with pytest.raises(AssertionError):
        KnormPress(compression_ratio=1.0)
    # ratio 0 returns the inputs untouched without touching the device
    k = torch.zeros(1, 1, 4, 128)
    assert KnormPress(0.0).compress(None, None, k, k, None, {})[0] is k


def test_cpu_tensors_are_rejected_loudly():
    from fastcache_amd._lib import FastcacheError
    m = KVCacheLinearDecoupleCompressor(llava_cfg(L=1, H=1))
    kv = [(torch.zeros(1, 1, 8, 128, dtype=torch.float16), torch.zeros(1, 1, 8, 128, dtype=torch.float16))]
    with pytest.raises(FastcacheError):
        m(kv, it_len=[4, 4])
    with pytest.raises(FastcacheError):
        KnormPress(0.5).compress(None, torch.zeros(1, 8, 1), kv[0][0], kv[0][1], None, {})


def test_hybrid_image_branch_raises_like_reference():
    h = KVCacheHybridCompressor(minicpm_cfg(L=1), compression_factor=2, min_seq_len=1)
    kv = [(torch.zeros(1, 4, 16, 128), torch.zeros(1, 4, 16, 128))]
    with pytest.raises(TypeError):
        h(kv, it_len=[8, 8])
    with pytest.raises(TypeError):
        h._paged_segments(16, [8, 8])
    assert h._paged_segments(16, [0, 16]) == [("compress_tk", "compress_tv", 0, 16)]


class _FakeRunner:
    """Host-side stand-in for PagedKVRunner's bookkeeping (no device work): compression keeps len // cf rows."""

    def __init__(self, cf=4, block_size=256):
        self.cf, self.block_size = cf, block_size
        self._compressed_lens, self._blocks_to_free = {}, {}
        self.batches = []

    def compress_kv_cache_batch(self, seqs, image_len=None):
        self.batches.append([s.seq_id for s in seqs])
        for s in seqs:
            self._compressed_lens[s.seq_id] = len(s) // self.cf
        return 0.0, float(self.cf)

    def get_compressed_block_count(self, seq_id):
        c = self._compressed_lens.get(seq_id)
        return -1 if c is None else -(-c // self.block_size)

    def clear_compressed_lens(self, seq_ids=None):
        for i in (seq_ids or list(self._compressed_lens)):
            self._compressed_lens.pop(i, None)


def _drive(engine, max_steps=200):
    peak, steps, done = 0, 0, {}
    while not engine.is_finished():
        outputs, _ = engine.step()
        llm = getattr(engine, "llm", engine)
        peak = max(peak, len(llm.scheduler.running) + len(outputs))
        bm = llm.scheduler.block_manager
        assert len(bm.free_block_ids) + len(bm.used_block_ids) == len(bm.blocks)
        done.update(dict(outputs))
        steps += 1
        assert steps < max_steps
    return peak, steps, done


def test_scheduler_engine_and_lazy_compression_admit_more_requests():
    """Freed pages turn into admitted requests: with threshold-triggered batch compression all five requests
    run together, without it the pool holds three; every block returns to the pool at the end."""
    from fastcache_amd.engine.llm_engine import CompressionEngine, LazyCompressionEngine, SamplingParams
    from fastcache_amd.engine.scheduler import LlavaScheduler

    def build(lazy):
        sched = LlavaScheduler(max_num_seqs=8, max_num_batched_tokens=4096, eos=-1, num_kvcache_blocks=12)
        runner = _FakeRunner(cf=4)
        llm = CompressionEngine(sched, runner, lambda seqs, is_prefill: [7] * len(seqs))
        eng = LazyCompressionEngine(llm, compression_threshold=0.3) if lazy else llm
        for i in range(5):
            eng.add_request(list(range(i * 5000, i * 5000 + 1000)), SamplingParams(max_tokens=6, ignore_eos=True))
        return eng, llm, runner

    eng, llm, runner = build(lazy=False)
    peak, steps_plain, done = _drive(eng)
    assert peak == 3 and len(done) == 5 and all(len(v) == 6 for v in done.values())
    assert len(llm.scheduler.block_manager.free_block_ids) == 12 and not runner.batches

    eng, llm, runner = build(lazy=True)
    assert eng.threshold_blocks == 3
    peak, steps_lazy, done = _drive(eng)
    assert len(done) == 5 and all(len(v) == 6 for v in done.values())
    assert peak == 5 and steps_lazy < steps_plain
    # the first three prefills exhaust the pool (12 blocks), the next step compresses exactly those three in one batch
    assert len(runner.batches[0]) == 3 and eng.get_stats()["compression_count"] == len(runner.batches) >= 1
    assert llm.total_freed_blocks >= 9
    assert len(llm.scheduler.block_manager.free_block_ids) == 12
    assert not runner._compressed_lens                       # cleared as sequences finish


def test_engine_sync_compression_after_prefill_and_preemption():
    """apply_compression=True shortens every sequence right after its prefill (kv_cache_len, table, freed tail);
    a sequence is shortened once; pre-emption puts a sequence back with its cache dropped."""
    from fastcache_amd.engine.llm_engine import CompressionEngine, SamplingParams
    from fastcache_amd.engine.scheduler import LlavaScheduler
    from fastcache_amd.engine.sequence import SequenceStatus
    sched = LlavaScheduler(max_num_seqs=4, max_num_batched_tokens=8192, eos=-1, num_kvcache_blocks=9)
    runner = _FakeRunner(cf=4)
    llm = CompressionEngine(sched, runner, lambda seqs, is_prefill: [1] * len(seqs))
    a = llm.add_request(list(range(1024)), SamplingParams(max_tokens=3, ignore_eos=True))
    b = llm.add_request(list(range(9000, 9000 + 1100)), SamplingParams(max_tokens=3, ignore_eos=True))
    outputs, n = llm.step(apply_compression=True)             # prefill of both: 4 + 5 blocks
    assert n == 1025 + 1101 and outputs == []                 # counted after the sampled token is appended
    assert a.is_compressed and a.kv_cache_len == 256 + 1 and len(a.block_table) == 1   # 256 rows kept, +1 appended
    assert b.kv_cache_len == 275 + 1 and len(b.block_table) == 2
    assert len(sched.block_manager.free_block_ids) == 9 - 3
    llm.step(apply_compression=True)                          # decode: a crosses into a new block (257 % 256 == 1)
    assert len(a.block_table) == 2 and a.kv_cache_len == 258 and b.kv_cache_len == 277
    # pre-emption drops the cache and the compressed length
    sched.preempt(b)
    sched.running.remove(b)
    assert b.status == SequenceStatus.WAITING and not b.is_compressed and b.block_table == [] and sched.waiting[0] is b


def test_checkpoint_layouts_round_trip(tmp_path):
    """The three file layouts the reference's runner accepts load into a module with the reference's key names;
    a file written by save_checkpoint has the training script's structure."""
    from fastcache_amd.utils_ccm.checkpoint import (load_checkpoint, load_checkpoint_only_model, load_compressor_state,
                                                    save_checkpoint)
    torch.manual_seed(1)
    src = KVCacheLinearDecoupleCompressor(llava_cfg(2, 2), compression_factor=2)
    sd = {k: v.clone() for k, v in src.state_dict().items()}
    assert "compress_tk.1.6.bias" in sd and "attention.0.weight" in sd
    opt = torch.optim.SGD(src.parameters(), lr=0.1)
    path = save_checkpoint(3, src, opt, None, 0.25, True, str(tmp_path), "c.pth")
    assert path.endswith("last_c.pth") and (tmp_path / "best_c.pth").exists()
    raw = torch.load(path, weights_only=True)
    assert set(raw) == {"epoch", "model_state_dict", "optimizer_state_dict", "scheduler_state_dict", "loss"}
    assert set(raw["model_state_dict"]) == {"compressor"}

    def fresh():
        torch.manual_seed(99)
        return KVCacheLinearDecoupleCompressor(llava_cfg(2, 2), compression_factor=2)

    m = fresh()
    assert load_compressor_state(m, path) == ([], [])
    assert all(torch.equal(v, sd[k]) for k, v in m.state_dict().items())
    flat, bare = tmp_path / "flat.pth", tmp_path / "bare.pth"
    partial = {k: v for k, v in sd.items() if not k.startswith("attention")}
    torch.save({"model_state_dict": partial}, flat)
    torch.save(dict(sd, extra=torch.zeros(1)), bare)
    m = fresh()
    missing, unexpected = load_compressor_state(m, str(flat))
    assert sorted(missing) == sorted(k for k in sd if k.startswith("attention")) and unexpected == []
    assert torch.equal(m.state_dict()["compress_iv.0.0.weight"], sd["compress_iv.0.0.weight"])
    m = fresh()
    assert load_compressor_state(m, str(bare)) == ([], ["extra"])
    m = fresh()
    assert load_checkpoint(m, torch.optim.SGD(m.parameters(), lr=0.1), None, path) == (3, 0.25)
    assert load_checkpoint(m, filename=str(tmp_path / "nope.pth")) == (0, float("inf"))
    assert load_checkpoint_only_model(fresh(), path) and not load_checkpoint_only_model(fresh(), str(tmp_path / "no.pth"))


def test_snapkv_split_heuristic():
    """Key ranges per column: none for launches with a thousand columns or more, up to 8 below, never pieces shorter
    than 8 key tiles, never for pages that are no multiple of 64 tokens or groups of more than 16 row blocks."""
    from fastcache_amd import ops
    from fastcache_amd._lib import FcKvView

    def view(L, B, Hkv, S, block_size=256, paged=True):
        return FcKvView(base=0, stride_layer=0, stride_block=0, stride_batch=0, stride_token=0, stride_head=0,
                        block_tables=1 if paged else None, table_stride=0, block_size=block_size, dtype=2,
                        num_layers=L, batch=B, num_kv_heads=Hkv, head_dim=128, max_seq_len=S, seq_lens=None)

    assert ops.snapkv_splits(view(36, 8, 8, 4096), 32, 64) == 1          # 2304 columns
    assert ops.snapkv_splits(view(36, 1, 8, 32768), 32, 64) == 8         # 288 columns
    assert ops.snapkv_splits(view(36, 2, 8, 16384), 32, 64) == 4         # 576 columns
    assert ops.snapkv_splits(view(28, 1, 4, 32768), 28, 64) == 8         # 112 columns, 14 row blocks
    assert ops.snapkv_splits(view(36, 1, 8, 1024), 32, 64) == 2          # 16 tiles: at most 2 pieces
    assert ops.snapkv_splits(view(36, 1, 8, 500), 32, 64) == 1
    assert ops.snapkv_splits(view(36, 1, 8, 32768, block_size=48), 32, 64) == 1
    assert ops.snapkv_splits(view(36, 1, 8, 32768, paged=False), 32, 64) == 8
    assert ops.snapkv_splits(view(4, 1, 1, 32768), 32, 64) == 1          # 64 row blocks per kv head
    # whole columns in one launch, or key ranges: by how full the last round of workgroups is, and the column length
    pref = lambda v, hq: ops.snapkv_press_preferred(v, hq, 64, compute_units=256)
    assert pref(view(36, 8, 8, 4096), 32)                                 # no split in question
    assert pref(view(28, 4, 4, 4096), 28) and pref(view(28, 5, 4, 4096), 28)      # short columns
    assert pref(view(32, 4, 8, 8192), 32)                                 # 1024 columns: two full rounds
    assert pref(view(28, 8, 4, 8192), 28)                                 # 896 columns of 16 wavefronts: 3.5 rounds of 256
    assert not pref(view(36, 1, 8, 8192), 32)                             # 288 long columns in a round of 512
    assert not pref(view(40, 1, 8, 12000), 40)                            # 320 columns of 12000 keys


def test_bench_counter_table_names_real_workloads():
    """The HBM-counter table of bench.py is keyed by workload name: a key that no workload carries would silently
    turn that workload's ``roofline.traffic`` into null.  Also the refusal of more than one GPU."""
    import ast
    import pathlib
    import subprocess
    import sys
    root = pathlib.Path(__file__).resolve().parents[1]
    src = (root / "bench.py").read_text()
    names = {n.value for n in ast.walk(ast.parse(src))
             if isinstance(n, ast.Constant) and isinstance(n.value, str) and n.value.startswith("cfg")}
    names |= {n + "+given-lse" for n in names}
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench_under_test", root / "bench.py")
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    assert set(bench._COUNTER_KIB) <= names
    for key, kib in bench._COUNTER_KIB.items():
        t = bench._measured_traffic(key, kib[2] if len(kib) > 2 else 1)
        assert t is not None and t > 0
    assert bench._measured_traffic("no such workload", 1) is None
    res = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert res.returncode != 0 and "ONE GPU" in (res.stdout + res.stderr)


def test_bench_refuses_graph_workloads_under_the_profiler():
    """The decode-graph workloads exit before any GPU call when the profiler's environment is present, naming the
    eager variant to use; the eager variants and the other workloads are not refused on that ground."""
    import os
    import pathlib
    import subprocess
    import sys
    root = pathlib.Path(__file__).resolve().parents[1]
    env = dict(os.environ, ROCPROF_OUTPUT_PATH="/tmp/x")
    for name, eager in (("decode", "decode-eager"), ("hybrid-decode", "hybrid-decode-eager")):
        res = subprocess.run([sys.executable, str(root / "bench.py"), "--workload", name], capture_output=True,
                             text=True, env=env)
        assert res.returncode == 3 and eager in res.stderr, (res.returncode, res.stderr)
    res = subprocess.run([sys.executable, str(root / "bench.py"), "--workload", "decode-eager"], capture_output=True,
                         text=True, env=env)
    assert res.returncode == 1 and "no GPU" in res.stderr          # passed the fence, stopped at the missing GPU
