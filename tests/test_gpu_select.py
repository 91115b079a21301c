"""GPU parity: the top-k selection and the gather / compaction kernels on their own, bit-exact.

Indices: identical to the oracle's stable selection (ties to the lowest index, ascending output) on integer-valued
and heavily tied rows, special values, ragged rows, rows longer than the on-chip key buffer.  Compaction: every
output byte equals the gathered source byte, for dense and paged views in either direction, in place, with per-
sequence kept counts and with one index row shared by all heads.
"""
import pytest
import torch

from fastcache_amd import _lib, ops, synth
from oracle import presses as opress

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("S,k", [(1, 1), (7, 3), (64, 64), (65, 1), (1000, 250), (4096, 1024), (15360, 77),
                                 (15361, 5000), (40000, 10000)])
def test_topk_random_and_tied_rows(dev, S, k):
    """Continuous scores, then scores drawn from 5 distinct values so that the k-th value has many ties.  Rows of
    more than 15360 scores do not fit the key buffer in LDS and take the path that re-reads them."""
    g = torch.Generator().manual_seed(S * 7 + k)
    for tied in (False, True):
        sc = torch.randint(0, 5, (3, 4, S), generator=g).float() if tied else torch.randn(3, 4, S, generator=g)
        got = ops.topk_select(sc.to(dev), k).cpu().long()
        assert torch.equal(got, opress.topk_lowest_index(sc, k))
        assert bool((got[..., 1:] > got[..., :-1]).all()) if k > 1 else True


def test_topk_special_values(dev):
    """NaN ranks above +inf, -0 equals +0 (the lower index wins), -inf is taken last."""
    row = torch.tensor([0.0, -0.0, float("inf"), float("nan"), -float("inf"), 1.0, float("nan"), -1.0, 0.0, 1.0])
    for k in range(1, row.numel() + 1):
        got = ops.topk_select(row[None].to(dev), k).cpu().long()
        assert torch.equal(got, opress.topk_lowest_index(row[None], k)), k


def test_topk_ragged_rows_and_kept_counts(dev):
    """Per-sequence valid lengths and kept counts: rows ordered (layer, b, head) use entry b; the tail of a row's
    output stays -1; a kept count above the length keeps the whole row."""
    L, B, H, S, K = 2, 3, 4, 300, 120
    g = torch.Generator().manual_seed(5)
    sc = torch.randn(L, B, H, S, generator=g)
    lens = torch.tensor([300, 17, 150], dtype=torch.int32)
    kept = torch.tensor([120, 40, 33], dtype=torch.int32)
    got = ops.topk_select(sc.to(dev), K, row_lens=lens.to(dev), n_kept=kept.to(dev), rows_per_len=H).cpu().long()
    for b in range(B):
        n, kk = int(lens[b]), min(int(kept[b]), int(lens[b]))
        ref = opress.topk_lowest_index(sc[:, b, :, :n], kk)
        assert torch.equal(got[:, b, :, :kk], ref)
        assert bool((got[:, b, :, kk:] == -1).all())


def test_topk_strided_rows(dev):
    """Rows spaced by a stride larger than their length (a narrowed view of a wider score buffer)."""
    g = torch.Generator().manual_seed(8)
    buf = torch.randn(2, 5, 512, generator=g)
    view = buf.to(dev)[..., :400]
    got = ops.topk_select(view, 100).cpu().long()
    assert torch.equal(got, opress.topk_lowest_index(buf[..., :400], 100))


def _payload(shape, dtype, seed):
    """Values that differ in every (row, column) so that a wrong row or a shifted column shows."""
    g = torch.Generator().manual_seed(seed)
    return (torch.randint(-2000, 2000, shape, generator=g).float() / 8).to(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shared_heads", [False, True])
def test_compact_dense_to_dense(dev, dtype, shared_heads):
    L, B, H, S, K = 2, 2, 3, 333, 100
    k, v = _payload((L, B, H, S, 128), dtype, 1), _payload((L, B, H, S, 128), dtype, 2)
    g = torch.Generator().manual_seed(3)
    hi = 1 if shared_heads else H
    idx = torch.stack([torch.sort(torch.randperm(S, generator=g)[:K]).values for _ in range(L * B * hi)])
    idx = idx.view(L, B, hi, K).int()
    kd, vd = k.to(dev), v.to(dev)
    ok, ov = torch.zeros(L, B, H, K, 128, dtype=dtype, device=dev), torch.zeros(L, B, H, K, 128, dtype=dtype, device=dev)
    ops.compact(_lib.dense_view(kd), _lib.dense_view(vd), _lib.dense_view(ok), _lib.dense_view(ov), idx.to(dev))
    full = idx.long().expand(L, B, H, K)
    for l in range(L):
        assert torch.equal(ok[l].cpu(), opress.gather_tokens(k[l], full[l]))
        assert torch.equal(ov[l].cpu(), opress.gather_tokens(v[l], full[l]))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("block_size", [256, 16, 48])
def test_compact_paged_in_place_with_kept_counts(dev, dtype, block_size):
    """In-place compaction of a paged pool with a different kept count per sequence: the first n_kept[b] tokens of
    every (layer, sequence, head) equal the gathered rows, pages of other sequences and spare pages are untouched."""
    L, H, lens = 2, 4, [700, 64, 301]
    B = len(lens)
    case = synth.make_paged_case(seed=6, num_layers=L, batch=B, num_kv_heads=H, seq_lens=lens, dtype=dtype,
                                 keep_dense=True, block_size=block_size, fill_value=7.0)
    kept = [200, 64, 1]
    K = max(kept)
    g = torch.Generator().manual_seed(11)
    idx = torch.full((L, B, H, K), -1, dtype=torch.int32)
    for l in range(L):
        for b in range(B):
            for h in range(H):
                idx[l, b, h, :kept[b]] = torch.sort(torch.randperm(lens[b], generator=g)[:kept[b]]).values.int()
    pool = case.kv_cache.to(dev)
    tab, lens_d = case.table_tensor(dev), case.lens_tensor(dev)
    S = max(lens)
    views = [_lib.paged_view(pool[p], tab, lens_d, S) for p in range(2)]
    ops.compact(views[0], views[1], views[0], views[1], idx.to(dev), n_kept=torch.tensor(kept, dtype=torch.int32, device=dev))
    after = pool.cpu()
    used = set()
    for b in range(B):
        blocks = case.block_tables[b]
        used.update(blocks)
        for p, dense in enumerate((case.dense_k, case.dense_v)):
            for l in range(L):
                rows = torch.cat([after[p, l, blk] for blk in blocks])[:kept[b]]            # [n, H, D]
                want = opress.gather_tokens(dense[l][b:b + 1, :, :lens[b]], idx[l, b:b + 1, :, :kept[b]].long())[0]
                assert torch.equal(rows.permute(1, 0, 2), want), (b, p, l)
    spare = [i for i in range(after.shape[2]) if i not in used]
    assert bool((after[:, :, spare] == 7.0).all())


@pytest.mark.parametrize("paged", [True, False])
def test_compact_clamps_device_side_kept_counts(dev, paged):
    """A kept count in device memory that exceeds the index row (or the destination) is cut to what the host
    validated: rows past the index stride, other sequences' pages and spare pages keep their bytes."""
    L, H, lens, K = 1, 2, [300, 280], 40
    B = len(lens)
    case = synth.make_paged_case(seed=9, num_layers=L, batch=B, num_kv_heads=H, seq_lens=lens, dtype=torch.bfloat16,
                                 keep_dense=True, fill_value=3.0)
    g = torch.Generator().manual_seed(2)
    idx = torch.stack([torch.sort(torch.randperm(280, generator=g)[:K]).values.int() for _ in range(L * B * H)])
    idx = idx.view(L, B, H, K)
    bogus = torch.tensor([K + 100000, 2 ** 31 - 1], dtype=torch.int32, device=dev)   # far beyond the index rows
    if paged:
        pool = case.kv_cache.to(dev)
        before = pool.cpu().clone()
        tab, lens_d = case.table_tensor(dev), case.lens_tensor(dev)
        views = [_lib.paged_view(pool[p], tab, lens_d, max(lens)) for p in range(2)]
        ops.compact(views[0], views[1], views[0], views[1], idx.to(dev), n_kept=bogus)
        torch.cuda.synchronize()
        after = pool.cpu()
        for b in range(B):
            blocks = case.block_tables[b]
            for p, dense in enumerate((case.dense_k, case.dense_v)):
                rows = torch.cat([after[p, 0, blk] for blk in blocks])                      # [tokens, H, D]
                want = opress.gather_tokens(dense[0][b:b + 1, :, :lens[b]], idx[0, b:b + 1].long())[0]
                assert torch.equal(rows[:K].permute(1, 0, 2), want), (b, p)
                old = torch.cat([before[p, 0, blk] for blk in blocks])
                assert torch.equal(rows[K:], old[K:]), "rows past the index stride were touched"
        used = {blk for t in case.block_tables for blk in t}
        spare = [i for i in range(after.shape[2]) if i not in used]
        assert bool((after[:, :, spare] == 3.0).all())
    else:
        k = case.dense_k[0].to(dev).contiguous()          # [B, H, S, D]
        v = case.dense_v[0].to(dev).contiguous()
        src = [_lib.dense_view(k), _lib.dense_view(v)]
        guard = torch.full((2, B, H, K + 8, 128), 5.0, dtype=torch.bfloat16, device=dev)
        dst = [_lib.dense_view(guard[p, :, :, :K]) for p in range(2)]                       # K rows, 8 guard rows behind
        ops.compact(src[0], src[1], dst[0], dst[1], idx.to(dev), n_kept=bogus)
        torch.cuda.synchronize()
        out = guard.cpu()
        assert bool((out[:, :, :, K:] == 5.0).all()), "rows past the destination were written"
        for p, dense in enumerate((case.dense_k, case.dense_v)):
            want = opress.gather_tokens(dense[0][:, :, :280], idx[0].long())
            assert torch.equal(out[p, :, :, :K], want)


def test_compact_rejects_bad_arguments(dev):
    k = torch.zeros(1, 1, 2, 8, 128, device=dev)
    view = _lib.dense_view(k)
    with pytest.raises(_lib.FastcacheError):
        ops.compact(view, view, view, view, torch.zeros(1, 1, 2, 4, dtype=torch.int64, device=dev))       # not int32
    with pytest.raises(_lib.FastcacheError):
        ops.compact(view, view, view, view, torch.zeros(2, 1, 2, 4, dtype=torch.int32, device=dev))       # layer mismatch


def _copy_reference(src_rows, src_ok, dst_old, dst_ok, lens, seg_start, count, dst_start):
    """Row j of sequence b goes from token seg_start + j to token dst_start + j when j < min(count, len - seg_start),
    the source token's page exists and the destination token's page exists; everything else keeps its bytes.
    src_rows / dst_old [L, B, H, S, D]; src_ok / dst_ok [B, S] bool."""
    out = dst_old.clone()
    for b, n in enumerate(lens):
        for j in range(max(0, min(count, n - seg_start, out.shape[3] - dst_start))):
            if src_ok[b, seg_start + j] and dst_ok[b, dst_start + j]:
                out[:, b, :, dst_start + j] = src_rows[:, b, :, seg_start + j]
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("block_size", [256, 16, 48])
def test_copy_between_a_pool_and_dense_tensors(dev, dtype, block_size):
    """Copies whose source and destination cannot overlap take short-lived workgroups in no particular order: pool ->
    dense, dense -> pool and a list of per-layer tensors -> pool, with sequences of different lengths, offsets on both
    sides, a missing source page and a missing destination page, against a row-by-row restatement."""
    L, H, lens = 3, 4, [700, 64, 301, 0]
    B = len(lens)
    case = synth.make_paged_case(seed=21, num_layers=L, batch=B, num_kv_heads=H, seq_lens=[max(n, 1) for n in lens],
                                 dtype=dtype, keep_dense=True, block_size=block_size, fill_value=7.0)
    S = max(lens)
    pool = case.kv_cache.to(dev)
    tab = case.table_tensor(dev)
    hole = tab.clone()
    hole[0, 1] = -1                                             # sequence 0 lacks its second page
    page_ok = torch.ones(B, S, dtype=torch.bool)
    page_ok[0, block_size:2 * block_size] = False
    all_ok = torch.ones(B, S, dtype=torch.bool)
    lens_d = torch.tensor(lens, dtype=torch.int32, device=dev)
    dense_k = case.dense_k                                      # [L, B, H, S', D] with S' >= S
    for seg_start, count, dst_start in ((0, S, 0), (5, 300, 9), (block_size - 1, 2, 0)):
        # pool -> dense, with and without the hole
        for t, ok in ((tab, all_ok), (hole, page_ok)):
            out = torch.full((L, B, H, S + 16, 128), 3.0, dtype=dtype, device=dev)
            ops.copy_tokens(_lib.paged_view(pool[0], t, lens_d, S), _lib.dense_view(out[:, :, :, :S]), seg_start, count,
                            dst_start)
            want = _copy_reference(dense_k[:, :, :, :S], ok, torch.full((L, B, H, S, 128), 3.0, dtype=dtype), all_ok, lens,
                                   seg_start, count, dst_start)
            got = out.cpu()
            assert torch.equal(got[:, :, :, :S], want), (seg_start, count, dst_start)
            assert bool((got[:, :, :, S:] == 3.0).all())
        # dense -> pool (the V plane of the pool as the destination), destination with and without the hole;
        # a dense source has no lengths of its own, so every sequence gets `count` rows as far as its pages reach
        rows = _payload((L, B, H, S, 128), dtype, 5)
        full = [S] * B
        for t, ok in ((tab, all_ok), (hole, page_ok)):
            dst = pool[1].clone()
            old = torch.stack([torch.stack([_rows_of_table(dst[l].cpu(), case.block_tables[b], S, H) for b in range(B)])
                               for l in range(L)])                                         # [L, B, H, S, D]
            ops.copy_tokens(_lib.dense_view(rows.to(dev)), _lib.paged_view(dst, t, None, S), seg_start, count, dst_start)
            reach = torch.zeros(B, S, dtype=torch.bool)
            for b in range(B):
                reach[b, :len(case.block_tables[b]) * block_size] = True
            want = _copy_reference(rows, all_ok, old, ok & reach, full, seg_start, count, dst_start)
            after = dst.cpu()
            got = torch.stack([torch.stack([_rows_of_table(after[l], case.block_tables[b], S, H) for b in range(B)])
                               for l in range(L)])
            assert torch.equal(got, want), (seg_start, count, dst_start)
            used = {blk for tb in case.block_tables for blk in tb}
            spare = [i for i in range(after.shape[1]) if i not in used]
            assert bool((after[:, spare] == 7.0).all())
    # a list of per-layer tensors as the source
    layers = [_payload((B, H, S, 128), dtype, 30 + l).to(dev) for l in range(L)]
    dst = pool[1].clone()
    assert ops.copy_tokens_from_layers(layers, _lib.paged_view(dst, tab, None, S), 200, 3)
    after = dst.cpu()
    for l in range(L):
        for b in range(B):
            n = min(200, max(0, len(case.block_tables[b]) * block_size - 3))
            got = _rows_of_table(after[l], case.block_tables[b], S, H)
            assert torch.equal(got[:, 3:3 + n], layers[l][b, :, :n].cpu()), (l, b)


def _rows_of_table(plane, table, S, H):
    """[H, S, D] rows of one sequence of one layer's plane [blocks, block_size, H, D]; tokens past its pages are 0."""
    rows = torch.cat([plane[blk] for blk in table])[:S]
    if rows.shape[0] < S:
        rows = torch.cat([rows, torch.zeros(S - rows.shape[0], *rows.shape[1:], dtype=rows.dtype)])
    return rows.permute(1, 0, 2)
