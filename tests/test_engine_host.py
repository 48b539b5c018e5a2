"""Host bookkeeping around the compression path, no GPU: page pool, compression target rule,
scheduler life cycle, and the index tensors of a decode step."""
import random

import numpy as np
import pytest

from oracle import zipage_oracle as O
from zipage_amd.engine.config import EngineConfig
from zipage_amd.engine.inputs import (encode_compress_tables, pack_decode, query_slot_mapping,
                                      unpack_views)
from zipage_amd.engine.pages import PagePool
from zipage_amd.engine.qwen3 import Qwen3Shape
from zipage_amd.engine.scheduler import Scheduler
from zipage_amd.engine.sequence import SamplingParams, Sequence

TINY = Qwen3Shape(2, 64, 4, 2, 16, 128, 100)


def _seq(n, bs=16, max_tokens=8, base=0):
    return Sequence([base + i for i in range(n)], SamplingParams(max_tokens=max_tokens, ignore_eos=True), bs)


def test_prefix_sharing_refcounts_and_release():
    pool = PagePool(32, 16, pages_per_seq=5, enable_prefix_cache=True)
    a, b = _seq(40), _seq(40)
    b.token_ids[35] = 999                      # differs only in the (partial) third page
    pool.admit(a)
    pool.admit(b)
    assert a.block_table[:2] == b.block_table[:2] and a.block_table[2] != b.block_table[2]
    assert b.num_cached_tokens == 32 and a.num_cached_tokens == 0
    assert [pool.refcount[p] for p in a.block_table] == [2, 2, 1]
    pool.release(a)
    assert [pool.refcount[p] for p in b.block_table] == [1, 1, 1]
    pool.release(b)
    assert pool.num_free == 32 and not pool.refcount.any()
    # a prompt that fills a whole table never shares its last page (its window must be captured)
    c, d = _seq(80), _seq(80)
    pool.admit(c)
    pool.admit(d)
    assert c.block_table[:4] == d.block_table[:4] and c.block_table[4] != d.block_table[4]


def test_a_fully_cached_prompt_still_prefills_its_last_page():
    """Two identical prompts of exactly two pages: every page of the second one hits the prefix
    cache, but its last page is taken fresh so that prefill runs the last prompt token (the
    first decode step feeds on it) instead of decoding from a stale token."""
    pool = PagePool(16, 16, pages_per_seq=5, enable_prefix_cache=True)
    a, b = _seq(32), _seq(32)
    pool.admit(a)
    pool.admit(b)
    assert a.block_table[0] == b.block_table[0] and a.block_table[1] != b.block_table[1]
    assert b.num_cached_tokens == 16 < len(b)
    cfg = EngineConfig(shape=TINY, max_concurrency=4, num_kvcache_blocks=16, kvcache_block_size=16,
                       max_cache_blocks_per_seq=4, enable_prefix_cache=True)
    sched = Scheduler(cfg)
    x, y = _seq(32), _seq(32)
    sched.add(x)
    sched.add(y)
    batch, is_prefill = sched.schedule()
    assert is_prefill and batch == [x, y], "both prompts must go through prefill"


@pytest.mark.parametrize("seed", range(6))
def test_plan_compression_follows_the_copy_on_write_rule(seed):
    """Against the oracle's restatement of BlockManager.may_compress on random sharing patterns."""
    rng = random.Random(seed)
    pool = PagePool(64, 16, pages_per_seq=5, enable_prefix_cache=True)
    shared_pages = rng.randint(0, 5)
    n_tokens = 16 * rng.randint(max(5, shared_pages + 1), 7)
    a = _seq(n_tokens)
    b = _seq(n_tokens)
    for i in range(shared_pages * 16, n_tokens):
        b.token_ids[i] = 1000 + i
    pool.admit(a)
    pool.admit(b)
    compressed = rng.random() < 0.3
    b.compressed = compressed
    table = list(b.block_table)
    refs = {p: int(pool.refcount[p]) for p in table}
    free = list(pool.free)
    want = O.target_block_table(table, refs, compressed, 5, free)
    ok = pool.plan_compression(b)
    assert ok and b.require_compress
    assert b.new_block_table == want[0] and b.block_to_release == want[1]
    assert list(pool.free) == want[2]
    pool.commit_compression(b)
    assert b.block_table == want[0] and b.compressed and not b.require_compress
    assert b.num_cached_tokens == 4 * 16 + 1
    # pages of `a` are untouched and still referenced
    assert all(pool.refcount[p] >= 1 for p in a.block_table)
    pool.release(a)
    pool.release(b)
    assert pool.num_free == 64 and not pool.refcount.any()


def test_plan_compression_fails_without_free_pages():
    pool = PagePool(10, 16, pages_per_seq=5, enable_prefix_cache=True)
    a, b = _seq(80), _seq(80)
    b.token_ids[-1] = 7
    pool.admit(a)
    pool.admit(b)          # shares 4 pages, owns 1: 6 pages used
    while pool.num_free > 3:
        pool._take()
    assert pool.plan_compression(b) is False and not b.require_compress


@pytest.mark.parametrize("bs,w", [(16, 4), (256, 32), (256, 16)])
def test_query_slot_mapping_matches_oracle(bs, w):
    for n in list(range(1, 3 * bs + 2, max(1, bs // 8))) + [bs - w, bs - w + 1, bs, bs + 1, 2 * bs]:
        s = _seq(n, bs)
        s.query_id = 3
        got = query_slot_mapping(s, bs, w, True, cu_len=11, seqlen_q=n)
        assert got == O.query_slot_mapping(3, bs, w, is_prefill=True, cu_len=11, seqlen_q=n)
        got = query_slot_mapping(s, bs, w, False, cu_len=5)
        assert got == O.query_slot_mapping(3, bs, w, is_prefill=False, cu_len=5,
                                           last_block_num_tokens=s.last_block_num_tokens)
    s.query_id = -1
    assert query_slot_mapping(s, bs, w, False) == []


def _simulate(cfg, prompts, max_tokens, check):
    """Drive the scheduler without a device: the 'model' only advances lengths."""
    sched = Scheduler(cfg)
    seqs = [Sequence(p, SamplingParams(max_tokens=max_tokens, ignore_eos=True), cfg.kvcache_block_size)
            for p in prompts]
    for s in seqs:
        sched.add(s)
    steps = 0
    while not sched.is_finished():
        batch, is_prefill = sched.schedule()
        assert batch, "scheduler stalled"
        if is_prefill:
            for s in batch:
                s.num_cached_tokens = len(s)          # what prepare_prefill records
        else:
            todo = [s for s in batch if s.require_compress]
            check(sched, batch, todo)
            sched.postprocess(todo)
        sched.postprocess(batch, None, advance=True)
        steps += 1
        assert steps < 100000
    return sched, seqs


def test_scheduler_life_cycle_pages_and_context_lengths():
    BS, budget, W = 16, 4, 4
    cfg = EngineConfig(shape=TINY, max_concurrency=6, num_kvcache_blocks=64, kvcache_block_size=BS,
                       max_cache_blocks_per_seq=budget, query_cache_len=W, max_num_batched_tokens=4096)
    seen = {"compress": 0}

    def check(sched, batch, todo):
        for s in todo:
            seen["compress"] += 1
            # trigger: the token being decoded opens a page and the table is full
            assert len(s.block_table) == budget + 1 and s.num_tokens % BS == 1
            assert len(s.new_block_table) == budget + 1
            enc = encode_compress_tables([s])[0]
            assert enc[-1] == -s.block_table[-1] - 2 and enc[:-1] == s.block_table[:-1]
        for s in batch:
            if s.require_compress:
                continue
            ctx = (len(s.block_table) - 1) * BS + s.last_block_num_tokens
            assert ctx == s.num_cached_tokens, "every cached token is attended exactly once"
            assert len(s.block_table) <= budget + 1

    rng = random.Random(0)
    prompts = [[rng.randrange(100) for _ in range(rng.choice([5, 16, 17, 40, 64, 90]))] for _ in range(10)]
    sched, seqs = _simulate(cfg, prompts, 150, check)
    assert seen["compress"] > 0
    assert all(s.finished and s.num_completion_tokens == 150 for s in seqs)
    assert sched.pool.num_free == 64 and not sched.pool.refcount.any()
    assert sorted(sched.free_rows) == list(range(6))
    # a 90-token prompt decoding 150 tokens crosses the 80-token table 1 + (240-81)//16 times
    for s in seqs:
        total = s.num_prompt_tokens + 150
        first = (budget + 1) * BS + 1                  # length at which the first compression fires
        want = 0 if total - 1 < first else 1 + (total - 1 - first) // BS
        assert s.num_compressions == want, (s.num_prompt_tokens, s.num_compressions, want)


def test_pack_decode_layout_and_padding():
    BS, W, TW = 16, 4, 5
    seqs = []
    for i, n in enumerate([13, 16, 17, 30]):
        s = _seq(n, BS)
        s.query_id = 10 + i
        s.block_table = [100 + 10 * i + j for j in range(s.num_blocks)]
        s.num_tokens += 2                                # two generated tokens
        while len(s.block_table) < s.num_blocks:
            s.block_table.append(200 + i)
        seqs.append(s)
    buf = pack_decode(seqs, 8, BS, W, TW, scratch_row=99)
    head, tables, tri = unpack_views(buf, 8, TW)
    for i, s in enumerate(seqs):
        assert head[0, i] == s.query_id and head[1, i] == len(s) - 1 and head[4, i] == 2
        assert head[2, i] == s.block_table[-1] * BS + s.last_block_num_tokens - 1
        assert head[3, i] == (len(s.block_table) - 1) * BS + s.last_block_num_tokens
        assert tables[i, :len(s.block_table)].tolist() == s.block_table
        assert (tables[i, len(s.block_table):] == -1).all()
        want = query_slot_mapping(s, BS, W, False, cu_len=i)
        got = [tuple(tri[i])] if tri[i, 0] >= 0 else []
        assert got == want
    assert (head[0, 4:] == 99).all() and (head[2, 4:] == -1).all() and (head[3, 4:] == 0).all()
    assert (tables[4:] == -1).all() and (tri[4:] == -1).all()
