"""GPU parity: decode paged attention, KV append and length advance vs the CPU oracle.

Tolerance: attention outputs within 2e-2 absolute in fp16/bf16 (fp32 softmax and accumulation on
both sides; the reference's flash-attn rounds the probabilities to the storage dtype before the PV
product, this kernel keeps them in fp32).
"""
import pytest
import torch

from fastcache_amd import _lib, ops, synth
from oracle import attention as oattn

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("Hq,Hkv,lens", [
    (4, 4, [1, 255, 256, 257, 700]),
    (8, 2, [33, 1024, 513]),
    (14, 2, [300, 17]),
    (16, 1, [129, 0, 600]),
    (6, 2, [77, 260]),          # a group of 3 in a tile of 4
    (10, 2, [513]),             # a group of 5 in a tile of 8
])
def test_decode_attention(dev, dtype, Hq, Hkv, lens):
    L, B = 2, len(lens)
    case = synth.make_paged_case(seed=21, num_layers=L, batch=B, num_kv_heads=Hkv, seq_lens=[max(n, 1) for n in lens],
                                 dtype=dtype, reserve_tokens=8)
    g = torch.Generator().manual_seed(5)
    q = torch.randn(L, B, Hq, 128, generator=g).to(dtype)
    width = max(len(t) for t in case.block_tables) + 2
    tables = case.table_tensor("cpu", width)
    lens_t = torch.tensor(lens, dtype=torch.int32)
    scale = 128 ** -0.5

    pool = case.kv_cache.to(dev)
    tab_d, len_d = tables.to(dev), lens_t.to(dev)
    max_len = width * 256
    kview = _lib.paged_view(pool[0], tab_d, None, max_len)
    vview = _lib.paged_view(pool[1], tab_d, None, max_len)
    ws = ops.decode_attn_workspace(B, Hq, max_len, dev)
    for layer in range(L):
        ref = oattn.decode_attention(q[layer], case.kv_cache[0, layer], case.kv_cache[1, layer], lens_t, tables, scale)
        got = ops.decode_attn(kview, vview, layer, q[layer].to(dev), len_d, scale, ws)
        torch.cuda.synchronize()
        torch.testing.assert_close(got.cpu().float(), ref.float(), atol=2e-2, rtol=0)
        # much tighter in practice: fp32 math on both sides, one rounding at the end
        assert float((got.cpu().float() - ref.float()).abs().max()) < 4e-3


@pytest.mark.parametrize("block_size", [16, 32, 48, 64])
@pytest.mark.parametrize("Hq,Hkv", [(4, 4), (8, 2)])
def test_decode_attention_small_and_odd_pages(dev, block_size, Hq, Hkv):
    """Pages smaller than a 32-token tile or of a size that is no power of two take the per-row
    addressing path; pages of 32 and 64 tokens take the tile path with several pages per chunk."""
    dtype, lens = torch.bfloat16, [1, 31, 32, 33, 255, 256, 257, 530]
    B = len(lens)
    case = synth.make_paged_case(seed=8, num_layers=1, batch=B, num_kv_heads=Hkv, seq_lens=lens, dtype=dtype,
                                 block_size=block_size)
    q = torch.randn(B, Hq, 128, generator=torch.Generator().manual_seed(6)).to(dtype)
    tables, lens_t = case.table_tensor("cpu"), torch.tensor(lens, dtype=torch.int32)
    ref = oattn.decode_attention(q, case.kv_cache[0, 0], case.kv_cache[1, 0], lens_t, tables, 128 ** -0.5)
    pool, tab_d = case.kv_cache.to(dev), tables.to(dev)
    max_len = tables.shape[1] * block_size
    kview, vview = (_lib.paged_view(pool[i], tab_d, None, max_len) for i in range(2))
    ws = ops.decode_attn_workspace(B, Hq, max_len, dev)
    got = ops.decode_attn(kview, vview, 0, q.to(dev), lens_t.to(dev), 128 ** -0.5, ws).cpu()
    assert float((got.float() - ref.float()).abs().max()) < 4e-3


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_decode_attention_dense_view(dev, dtype):
    """A HuggingFace-layout cache [B, Hkv, S, D] gives the same output as the same rows in pages."""
    Hq, Hkv, lens = 8, 4, [700, 64, 385]
    B, S = len(lens), max(lens)
    case = synth.make_paged_case(seed=4, num_layers=1, batch=B, num_kv_heads=Hkv, seq_lens=lens, dtype=dtype,
                                 keep_dense=True)
    q = torch.randn(B, Hq, 128, generator=torch.Generator().manual_seed(7)).to(dtype).to(dev)
    lens_d = torch.tensor(lens, dtype=torch.int32, device=dev)
    dk, dv = case.dense_k[0].to(dev), case.dense_v[0].to(dev)    # rows past a sequence's length hold other data
    ws = ops.decode_attn_workspace(B, Hq, S, dev)
    got = ops.decode_attn(_lib.dense_view(dk), _lib.dense_view(dv), 0, q, lens_d, 128 ** -0.5, ws).cpu()
    pool, tab = case.kv_cache.to(dev), case.table_tensor(dev)
    ws2 = ops.decode_attn_workspace(B, Hq, tab.shape[1] * 256, dev)
    paged = ops.decode_attn(_lib.paged_view(pool[0], tab, None, tab.shape[1] * 256),
                            _lib.paged_view(pool[1], tab, None, tab.shape[1] * 256), 0, q, lens_d, 128 ** -0.5, ws2).cpu()
    assert torch.equal(got, paged)
    ref = oattn.decode_attention(q.cpu(), case.kv_cache[0, 0], case.kv_cache[1, 0], lens_d.cpu(), tab.cpu(), 128 ** -0.5)
    assert float((got.float() - ref.float()).abs().max()) < 4e-3


def test_block_permutation_invariance(dev):
    """Moving the pages around (with the table following) leaves the output bit-identical."""
    dtype, Hq, Hkv, lens = torch.float16, 8, 4, [900, 300, 77]
    case = synth.make_paged_case(seed=2, num_layers=1, batch=3, num_kv_heads=Hkv, seq_lens=lens, dtype=dtype)
    nb = case.kv_cache.shape[2]
    perm = torch.randperm(nb, generator=torch.Generator().manual_seed(1))
    pool2 = torch.empty_like(case.kv_cache)
    pool2[:, :, perm] = case.kv_cache                       # block i moves to perm[i]
    tables1 = case.table_tensor("cpu")
    tables2 = torch.where(tables1 >= 0, perm[tables1.clamp_min(0).long()].int(), tables1)
    q = torch.randn(3, Hq, 128, generator=torch.Generator().manual_seed(3)).to(dtype).to(dev)
    lens_d = torch.tensor(lens, dtype=torch.int32, device=dev)
    outs = []
    for pool, tab in ((case.kv_cache, tables1), (pool2, tables2)):
        p, t = pool.to(dev), tab.to(dev)
        kv = [_lib.paged_view(p[i], t, None, t.shape[1] * 256) for i in range(2)]
        ws = ops.decode_attn_workspace(3, Hq, t.shape[1] * 256, dev)
        outs.append(ops.decode_attn(kv[0], kv[1], 0, q, lens_d, 128 ** -0.5, ws).cpu())
    assert torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_store_kv_and_advance(dev, dtype):
    L, B, Hkv = 3, 4, 2
    lens = [5, 255, 256, 511]
    case = synth.make_paged_case(seed=9, num_layers=L, batch=B, num_kv_heads=Hkv, seq_lens=lens, dtype=dtype,
                                 reserve_tokens=4)
    g = torch.Generator().manual_seed(1)
    k_new = torch.randn(L, B, Hkv, 128, generator=g).to(dtype)
    v_new = torch.randn(L, B, Hkv, 128, generator=g).to(dtype)
    ref = case.kv_cache.clone()
    for layer in range(L):
        slots = torch.tensor([oattn.decode_slot(case.block_tables[b], lens[b]) for b in range(B)])
        oattn.store_kv(ref[0, layer], ref[1, layer], k_new[layer], v_new[layer], slots)

    pool = case.kv_cache.to(dev)
    tab = case.table_tensor(dev)
    len_d = torch.tensor(lens, dtype=torch.int32, device=dev)
    max_len = tab.shape[1] * 256
    kview = _lib.paged_view(pool[0], tab, None, max_len)
    vview = _lib.paged_view(pool[1], tab, None, max_len)
    ops.store_kv(kview, vview, k_new.to(dev), v_new.to(dev), len_d)
    ops.advance_lens(len_d, 1)
    torch.cuda.synchronize()
    assert torch.equal(pool.cpu().view(torch.uint8), ref.view(torch.uint8))
    assert len_d.cpu().tolist() == [n + 1 for n in lens]


def test_multi_step_decode_graph_matches_eager_and_oracle(dev):
    """T steps in one HIP graph: every replay equals the eager launches bit for bit, and both follow
    the oracle (store, advance, attend) across a block boundary."""
    from fastcache_amd.engine.decode_graph import DecodeGraph
    dtype, L, B, Hq, Hkv, T = torch.float16, 2, 3, 4, 2, 6
    lens = [254, 100, 511]                       # two sequences cross a 256-token block boundary
    case = synth.make_paged_case(seed=13, num_layers=L, batch=B, num_kv_heads=Hkv, seq_lens=lens, dtype=dtype,
                                 reserve_tokens=T + 1)
    g = torch.Generator().manual_seed(2)
    q = torch.randn(T, L, B, Hq, 128, generator=g).to(dtype)
    kn = torch.randn(T, L, B, Hkv, 128, generator=g).to(dtype)
    vn = torch.randn(T, L, B, Hkv, 128, generator=g).to(dtype)
    tables = case.table_tensor("cpu")
    scale = 128 ** -0.5

    # oracle
    ref_pool = case.kv_cache.clone()
    ref_out = torch.empty_like(q)
    cur = list(lens)
    for t in range(T):
        for layer in range(L):
            slots = torch.tensor([oattn.decode_slot(case.block_tables[b], cur[b]) for b in range(B)])
            oattn.store_kv(ref_pool[0, layer], ref_pool[1, layer], kn[t, layer], vn[t, layer], slots)
        cur = [n + 1 for n in cur]
        for layer in range(L):
            ref_out[t, layer] = oattn.decode_attention(q[t, layer], ref_pool[0, layer], ref_pool[1, layer],
                                                       torch.tensor(cur, dtype=torch.int32), tables, scale)

    def fresh():
        pool = case.kv_cache.to(dev)
        lens_d = torch.tensor(lens, dtype=torch.int32, device=dev)
        return DecodeGraph(pool, tables.to(dev), lens_d, q.to(dev), kn.to(dev), vn.to(dev), scale), pool, lens_d

    dg, pool, lens_d = fresh()
    eager = dg.run_eager().clone()
    torch.cuda.synchronize()
    assert lens_d.tolist() == [n + T for n in lens]
    assert torch.equal(pool.cpu().view(torch.uint8), ref_pool.view(torch.uint8))
    torch.testing.assert_close(eager.cpu().float(), ref_out.float(), atol=2e-2, rtol=0)

    dg2, pool2, lens2 = fresh()
    dg2.capture()
    assert lens2.tolist() == lens
    for rep in range(3):
        lens2.copy_(torch.tensor(lens, dtype=torch.int32))
        dg2.out.zero_()
        torch.cuda.synchronize()
        out = dg2.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {rep} differs from eager"
        assert lens2.tolist() == [n + T for n in lens]
        _ = (pool2.float().sum()).item()          # unrelated eager work between replays
    assert torch.equal(pool2, pool)


def test_bucketed_decode_graphs_match_eager_layers(dev):
    """One captured step per batch bucket, static buffers patched per step: every replay equals the eager
    Attention layers bit for bit (outputs and pool), for batches that fill a bucket exactly and that do not."""
    from fastcache_amd.engine.decode_graph import BucketedDecodeGraphs
    from fastcache_amd.layers import Attention
    from fastcache_amd.utils.context import reset_context, set_context
    dtype, L, Hq, Hkv, D, steps = torch.float16, 2, 8, 2, 128, 3
    max_bs, scale = 40, 128 ** -0.5
    all_lens = [100 + 37 * i for i in range(21)]
    all_lens[4] = 255                                            # crosses a block boundary during the steps
    case = synth.make_paged_case(seed=21, num_layers=L, batch=21, num_kv_heads=Hkv, seq_lens=all_lens, dtype=dtype,
                                 reserve_tokens=steps + 1)
    tables_all = case.table_tensor("cpu")

    def make_layers(pool):
        layers = []
        for l in range(L):
            a = Attention(Hq, D, scale, Hkv)
            a.k_cache, a.v_cache = pool[0, l], pool[1, l]
            layers.append(a)
        return layers

    pool_g, pool_e = case.kv_cache.to(dev), case.kv_cache.to(dev)
    graphs = BucketedDecodeGraphs(make_layers(pool_g), max_bs, tables_all.shape[1], dtype, dev)
    graphs.capture_cudagraph()
    assert graphs.graph_bs == [1, 2, 4, 8, 16, 32, 40]
    pool_g.copy_(case.kv_cache)                                  # capture warm-ups wrote nothing (slots are -1)
    eager_layers = make_layers(pool_e)
    g = torch.Generator().manual_seed(6)
    for bs in (3, 21, 16):
        lens = list(all_lens[:bs])
        tables = tables_all[:bs].to(dev)
        for t in range(steps):
            q = torch.randn(L, bs, Hq * D, generator=g).to(dtype).to(dev)
            k = torch.randn(L, bs, Hkv * D, generator=g).to(dtype).to(dev)
            v = torch.randn(L, bs, Hkv * D, generator=g).to(dtype).to(dev)
            slots = torch.tensor([oattn.decode_slot(case.block_tables[b], lens[b]) for b in range(bs)],
                                 dtype=torch.int32, device=dev)
            lens = [n + 1 for n in lens]
            ctx_lens = torch.tensor(lens, dtype=torch.int32, device=dev)
            set_context(False, slot_mapping=slots, context_lens=ctx_lens, block_tables=tables)
            out_g = graphs.run(q, k, v).clone()
            out_e = torch.stack([eager_layers[l](q[l], k[l], v[l]) for l in range(L)])
            reset_context()
            torch.cuda.synchronize()
            assert torch.equal(out_g, out_e), f"bs={bs} step={t}"
            assert torch.equal(pool_g, pool_e)
        # restore the prefixes for the next batch size
        pool_g.copy_(case.kv_cache)
        pool_e.copy_(case.kv_cache)


def test_decode_attention_empty_rows(dev):
    """Rows with no cached token give zeros, whatever their table row holds; their neighbours are unaffected."""
    dtype, Hq, Hkv = torch.bfloat16, 8, 2
    case = synth.make_paged_case(seed=3, num_layers=1, batch=3, num_kv_heads=Hkv, seq_lens=[300, 1, 5], dtype=dtype)
    q = torch.randn(3, Hq, 128, generator=torch.Generator().manual_seed(2)).to(dtype).to(dev)
    pool, tab = case.kv_cache.to(dev), case.table_tensor(dev)
    max_len = tab.shape[1] * 256
    kview, vview = _lib.paged_view(pool[0], tab, None, max_len), _lib.paged_view(pool[1], tab, None, max_len)
    ws = ops.decode_attn_workspace(3, Hq, max_len, dev)
    full = ops.decode_attn(kview, vview, 0, q, torch.tensor([300, 1, 5], dtype=torch.int32, device=dev), 128 ** -0.5, ws).cpu()
    some = ops.decode_attn(kview, vview, 0, q, torch.tensor([300, 0, 0], dtype=torch.int32, device=dev), 128 ** -0.5, ws).cpu()
    assert torch.equal(some[0], full[0]) and bool((some[1:] == 0).all())
    none = ops.decode_attn(kview, vview, 0, q, torch.zeros(3, dtype=torch.int32, device=dev), 128 ** -0.5, ws).cpu()
    assert bool((none == 0).all())
