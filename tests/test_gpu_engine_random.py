"""GPU: the page manager, the runner hook and the block-freeing hook under a random sequence of requests, decode
appends, compressions (synchronous and on the side stream, adapter and press objects, batches of one to four) and
retirements on a small pool with a prefix cache, so that prompts share pages, pages are un-shared before they are
rewritten, freed pages are handed out again and cached pages are taken back.  After every operation every live
sequence's rows, read through its block table, must equal a CPU shadow kept with the oracle's selection rules
(position-based selections only: no score ties), and the page accounting must add up.  Follows the life of a request
through nanovllm/engine/llava_engine.py:187-330 and nanovllm/engine/block_manager.py:39-169."""
import random

import pytest
import torch

from fastcache_amd.engine import BlockManager, Sequence
from fastcache_amd.engine.kv_runner import PagedKVRunner
from fastcache_amd.engine.llm_hooks import free_compressed_blocks
from fastcache_amd.kernels import KVPressCompressor
from fastcache_amd.presses import StreamingLLMPress
from oracle import presses as opress

pytestmark = pytest.mark.gpu

L, H, D, NB, BS = 2, 2, 128, 40, 256
VOCAB = 48
dtype = torch.float16


def _drive(dev, seed, n_ops):
    rnd = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    E = torch.randn(2, L, H, VOCAB, D, generator=g)
    P = torch.randn(2, L, H, 4096, D, generator=g) * 0.5

    def rows_of(tokens, pos0):
        t = torch.tensor(tokens)
        p = torch.arange(pos0, pos0 + len(tokens))
        return (E[:, :, :, t] + P[:, :, :, p]).to(dtype)        # [2, L, H, n, D]

    bm = BlockManager(NB, BS)
    runner = PagedKVRunner(L, H, D, num_blocks=NB, dtype=dtype, device=dev, image_token_len=0,
                           compressor=None, block_manager=bm)
    runner.kv_cache.copy_(torch.randn(runner.kv_cache.shape, generator=g).to(dtype))   # garbage everywhere
    bases = [[rnd.randrange(VOCAB) for _ in range(1400)] for _ in range(3)]
    live = {}          # seq_id -> (Sequence, shadow rows [2, L, H, n, D])
    finished_prompts = []
    stats = {"new": 0, "cached": 0, "append": 0, "compress": 0, "finish": 0, "unshared": 0, "refused": 0}

    def write_rows(seq, rows, pos0):
        # rows [2, L, H, n, D] for cache positions pos0 .. pos0+n-1
        n = rows.shape[3]
        pool = runner.kv_cache
        p = pos0
        while p < pos0 + n:
            page, off = divmod(p, BS)
            cnt = min(BS - off, pos0 + n - p)
            blk = seq.block_table[page]
            chunk = rows[:, :, :, p - pos0:p - pos0 + cnt].permute(0, 1, 3, 2, 4)    # [2, L, cnt, H, D]
            pool[:, :, blk, off:off + cnt] = chunk.to(dev)
            p += cnt

    def check(tag):
        pool = runner.kv_cache.cpu()
        for sid, (seq, rows) in live.items():
            n = seq.kv_cache_len
            assert rows.shape[3] == n, (tag, sid, rows.shape, n)
            assert len(seq.block_table) >= -(-n // BS), (tag, sid)
            got = torch.cat([pool[:, :, b] for b in seq.block_table], dim=2)[:, :, :n].permute(0, 1, 3, 2, 4)
            if not torch.equal(got, rows):
                bad = (got != rows).any(-1).any(0).any(0).any(0).nonzero().flatten()
                raise AssertionError(f"{tag}: seq {sid} rows differ at positions {bad[:10].tolist()} (of {n}), "
                                     f"table {seq.block_table}, compressed {seq.is_compressed}")
        owners = {}
        for seq, _ in live.values():
            for b in seq.block_table:
                owners[b] = owners.get(b, 0) + 1
        for b, c in owners.items():
            assert bm.blocks[b].ref_count == c, (tag, b, c, bm.blocks[b].ref_count)
        assert len(bm.free_block_ids) + len(owners) == NB, (tag, len(bm.free_block_ids), len(owners))

    for ops in range(1, n_ops + 1):
        r = rnd.random()
        if r < 0.30 or not live:
            # a new request: a base prompt's prefix, or an earlier request's tokens, plus a random tail
            if finished_prompts and rnd.random() < 0.3:
                src = rnd.choice(finished_prompts)
            else:
                src = rnd.choice(bases)
            m = rnd.choice([0, 256, 512, 768, 100, 300, 700, 1024])
            m = min(m, len(src))
            prompt = src[:m] + [rnd.randrange(VOCAB) for _ in range(rnd.randrange(1, 400))]
            seq = Sequence(prompt)
            if not bm.can_allocate(seq):
                stats["refused"] += 1
                continue
            bm.allocate(seq)
            c = seq.num_cached_tokens
            stats["cached"] += c > 0
            full = rows_of(prompt, 0)
            if c < len(prompt):
                write_rows(seq, full[:, :, :, c:], c)            # the prefill computes only what the cache does not hold
            live[seq.seq_id] = (seq, full)
            stats["new"] += 1
            check(f"op {ops} new len {len(prompt)} cached {c}")
        elif r < 0.55:
            sid = rnd.choice(list(live))
            seq, rows = live[sid]
            k = rnd.choice([1, 1, 3, 40, 260])
            done = 0
            for _ in range(k):
                tok = rnd.randrange(VOCAB)
                seq.append_token(tok)
                if not bm.can_append(seq):
                    seq.token_ids.pop()
                    break
                bm.may_append(seq)
                pos = seq.kv_cache_len - 1
                # an uncompressed sequence's rows are functions of (token, position) so that published pages are honest
                new = rows_of([tok], len(seq) - 1)
                write_rows(seq, new, pos)
                rows = torch.cat([rows, new], dim=3)
                done += 1
            live[sid] = (seq, rows)
            stats["append"] += done
            check(f"op {ops} append {done} to {sid}")
        elif r < 0.85:
            cands = [s for s, _ in live.values() if not s.is_compressed and len(s) >= 8]
            if not cands:
                continue
            group = rnd.sample(cands, rnd.randint(1, min(4, len(cands))))
            ratio = rnd.choice([0.3, 0.5, 0.8])
            kind = rnd.choice(["streaming_llm", "snapkv", "press"])
            if kind == "press":
                runner.compressor = StreamingLLMPress(ratio)
            else:
                runner.compressor = KVPressCompressor(kind, ratio)
            tables_before = {s.seq_id: list(s.block_table) for s in group}
            try:
                if rnd.random() < 0.5:
                    runner.compress_kv_cache_batch(group)
                else:
                    ev = runner.start_background_compression(group)
                    # a request with the same prompt arrives while the compression is in flight
                    twin = Sequence(list(group[0].token_ids))
                    if bm.can_allocate(twin):
                        bm.allocate(twin)
                        c = twin.num_cached_tokens
                        full = rows_of(twin.token_ids, 0)
                        runner.wait_compression(ev)     # (the prefill would run on the main stream; keep it simple)
                        if c < len(twin):
                            write_rows(twin, full[:, :, :, c:], c)
                        live[twin.seq_id] = (twin, full)
                    runner.wait_compression(ev)
            except Exception as e:
                if "pages are free" in str(e):
                    stats["refused"] += 1
                    check(f"op {ops} refused compress")
                    continue
                raise
            stats["unshared"] += sum(tables_before[s.seq_id] != s.block_table for s in group)
            for s in group:
                rows = live[s.seq_id][1]
                n = len(s)
                k4 = [rows[0, l].unsqueeze(0) for l in range(L)]
                v4 = [rows[1, l].unsqueeze(0) for l in range(L)]
                outs = []
                for l in range(L):
                    if kind == "press":
                        nk = int(n * (1 - ratio))
                        sc = torch.ones(n)
                        sc[4:4 + (n - nk)] = 0
                        ck, cv, _ = opress.press_compress(k4[l], v4[l], sc.expand(1, H, -1).contiguous(), ratio)
                    else:
                        ck, cv = opress.adapter_compress_layer(kind, k4[l], v4[l], ratio)
                    outs.append((ck[0], cv[0]))
                new = torch.stack([torch.stack([o[0] for o in outs]), torch.stack([o[1] for o in outs])])
                live[s.seq_id] = (s, new)
            free_compressed_blocks(bm, runner, group)
            stats["compress"] += len(group)
            check(f"op {ops} compress {kind} {ratio} {[s.seq_id for s in group]}")
        else:
            sid = rnd.choice(list(live))
            seq, _ = live.pop(sid)
            if not seq.is_compressed:
                finished_prompts.append(list(seq.token_ids))
            bm.deallocate(seq)
            runner.clear_compressed_lens([sid])
            stats["finish"] += 1
            check(f"op {ops} finish {sid}")
    return stats


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_random_requests_against_a_cpu_shadow(dev, seed):
    stats = _drive(dev, seed, 450)
    assert stats["new"] > 20 and stats["compress"] > 20 and stats["finish"] > 20 and stats["append"] > 1000, stats
    assert stats["cached"] >= 1 and stats["unshared"] >= 1, stats      # the prefix cache and the un-sharing were exercised
