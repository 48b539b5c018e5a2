"""GPU tests of the decode engine around the compression path, on a tiny random model."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _tiny():
    from zipage_amd.engine import Qwen3Shape
    return Qwen3Shape(layers=2, hidden=256, heads=4, kv_heads=2, head_dim=64, intermediate=512,
                      vocab=503, max_position=2048)


def _cfg(**kw):
    from zipage_amd.compress import CompressConfig
    from zipage_amd.engine import EngineConfig
    # the scorer needs 256-token pages for 16-bit caches, so the budget is kept to 2 pages
    base = dict(shape=_tiny(), max_concurrency=8, num_kvcache_blocks=40, kvcache_block_size=256,
                max_cache_blocks_per_seq=2, query_cache_len=16, layer_stride=2, seed=5,
                max_model_len=2048, compress=CompressConfig(enable_pooling=True, pooling_size=3))
    base.update(kw)
    return EngineConfig(**base)


def _prompts(n, lens, seed=0):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, 503, (lens[i % len(lens)],), generator=g).tolist() for i in range(n)]


def test_paged_decode_equals_dense_recompute(dev):
    """Prefill a prefix through the paged caches, decode the rest token by token, and compare
    every decode step's hidden state with one dense causal pass over the whole sequence.
    Tolerance: hidden states are RMS-normalised (|x| ~ 1) and pass through 2 bf16 layers; 6e-2
    absolute covers the bf16 rounding of activations (2^-8 relative per op)."""
    from zipage_amd.engine import Qwen3, StepContext
    s = _tiny()
    BS, pages = 16, 24
    model = Qwen3(s, dev, seed=11, init_std=0.05)
    kv = torch.zeros(2, s.layers, pages, BS, s.kv_heads, s.head_dim, device=dev, dtype=torch.bfloat16)
    qc = torch.zeros(s.layers, 2, 4, s.heads, s.head_dim, device=dev, dtype=torch.bfloat16)
    n, n0 = 75, 37
    ids = torch.randint(0, s.vocab, (n,), device=dev)
    pos = torch.arange(n, device=dev)
    dense = model.forward(ids, pos, StepContext(True, None, None, None, None, [n], [n])).float()
    model.attach_caches(kv, qc)
    table = torch.randperm(pages)[:5].int()
    slots = (table.long()[:, None] * BS + torch.arange(BS)[None, :]).flatten().int().to(dev)
    h0 = model.forward(ids[:n0], pos[:n0], StepContext(True, slots[:n0], None, None, None, [n0], [n0]))
    assert (h0.float() - dense[:n0]).abs().max() < 6e-2
    tables = table.view(1, 5).to(dev)
    for t in range(n0, n):
        ctx = StepContext(False, slots[t:t + 1], None,
                          torch.tensor([t + 1], device=dev, dtype=torch.int32), tables)
        h = model.forward(ids[t:t + 1], pos[t:t + 1], ctx)
        assert (h.float() - dense[t:t + 1]).abs().max() < 6e-2, t


def test_cached_prefix_prefill_equals_dense(dev):
    """Prefill in two parts (the second sees the first through the block table, as a prefix
    cache hit does) against one dense pass."""
    from zipage_amd.engine import Qwen3, StepContext
    s = _tiny()
    BS, pages = 16, 12
    model = Qwen3(s, dev, seed=3, init_std=0.05)
    kv = torch.zeros(2, s.layers, pages, BS, s.kv_heads, s.head_dim, device=dev, dtype=torch.bfloat16)
    qc = torch.zeros(s.layers, 2, 4, s.heads, s.head_dim, device=dev, dtype=torch.bfloat16)
    n, n0 = 50, 32
    ids = torch.randint(0, s.vocab, (n,), device=dev)
    pos = torch.arange(n, device=dev)
    dense = model.forward(ids, pos, StepContext(True, None, None, None, None, [n], [n])).float()
    model.attach_caches(kv, qc)
    table = torch.tensor([7, 2, 9, 4], dtype=torch.int32)
    slots = (table.long()[:, None] * BS + torch.arange(BS)[None, :]).flatten().int().to(dev)
    model.forward(ids[:n0], pos[:n0], StepContext(True, slots[:n0], None, None, None, [n0], [n0]))
    h = model.forward(ids[n0:], pos[n0:], StepContext(True, slots[n0:n], None, None,
                                                      table.view(1, 4).to(dev), [n - n0], [n]))
    assert (h.float() - dense[n0:]).abs().max() < 6e-2


def _generate(cfg, prompts, max_tokens):
    from zipage_amd.engine import SamplingParams, ZipageEngine
    eng = ZipageEngine(cfg)
    out = eng.generate(prompts, SamplingParams(max_tokens=max_tokens, ignore_eos=True))
    return eng, out


def test_graph_replay_equals_eager_across_compressions(dev):
    """The same run with the decode step replayed as a HIP graph and launched eagerly: identical
    tokens on every step.  Prompts are ragged, so compressions (eager work on the same stream,
    plus host synchronisations of the pinned ring) fall between replays, and replays cover
    different padded batch sizes as sequences finish."""
    prompts = _prompts(5, [90, 300, 470, 640, 1100])
    e1, a = _generate(_cfg(use_graph=False), prompts, 700)
    e2, b = _generate(_cfg(use_graph=True), prompts, 700)
    assert e1.stats["compress_calls"] > 3
    for x, y in zip(a, b):
        assert len(x["token_ids"]) == 700
        assert x["token_ids"] == y["token_ids"]
        assert x["num_compressions"] == y["num_compressions"] > 0


def test_async_compression_bookkeeping(dev):
    """Side-stream compression: every request still gets all its tokens, each sequence is
    compressed as often as its length dictates, and all pages and rows come back."""
    prompts = _prompts(7, [90, 300, 470, 640, 1100, 256, 257], seed=1)
    cfg = _cfg(enable_async_compress=True, max_compress_blocks=6)
    eng, out = _generate(cfg, prompts, 600)
    BS, cap = 256, 3
    for p, o in zip(prompts, out):
        assert len(o["token_ids"]) == 600
        total = len(p) + 600
        first = max(cap, -(-len(p) // BS)) * BS + 1
        assert o["num_compressions"] == (0 if total - 1 < first else 1 + (total - 1 - first) // BS)
    pool = eng.scheduler.pool
    assert pool.num_free == cfg.num_kvcache_blocks and not pool.refcount.any()
    assert sorted(eng.scheduler.free_rows) == list(range(cfg.max_concurrency))
    assert eng.stats["compress_s"] > 0


def test_engine_compression_moves_the_right_pages(dev):
    """Hook the first compression: per layer and head, the rows the target pages hold afterwards
    are an ordered subset of the rows the sequence's own pages held before (stable gather), and
    the last `query_cache_len` tokens survive."""
    from zipage_amd.engine import SamplingParams, ZipageEngine
    cfg = _cfg(use_graph=False)
    eng = ZipageEngine(cfg)
    r = eng.runner
    seen = {}
    orig = r.compress

    def hooked(seqs, **kw):
        if not seen:
            torch.cuda.synchronize()
            seen["seqs"] = [(list(s.block_table), list(s.new_block_table)) for s in seqs]
            seen["k"] = r.kv_cache[0].clone()
        ev = orig(seqs, **kw)
        if "after" not in seen:
            torch.cuda.synchronize()
            seen["after"] = r.kv_cache[0].clone()
        return ev

    r.compress = hooked
    eng.generate(_prompts(3, [700, 750, 200]), SamplingParams(max_tokens=100, ignore_eos=True))
    assert seen
    BS, budget, W = 256, 2, 16
    for table, target in seen["seqs"]:
        src = seen["k"][:, table].flatten(1, 2)                 # (L, T, Hkv, D)
        dst = seen["after"][:, target[:budget]].flatten(1, 2)   # (L, budget*BS, Hkv, D)
        T = src.shape[1]
        for l in range(src.shape[0]):
            for h in range(src.shape[2]):
                eq = (dst[l, :, h, None, :] == src[l, None, :, h, :]).all(-1)   # (kept, T)
                idx = eq.float().argmax(1)
                assert eq.any(1).all()
                assert (idx[1:] > idx[:-1]).all()
                assert set(range(T - W, T)) <= set(idx.tolist())


def test_eos_stops_a_request_and_frees_its_pages(dev):
    """A request without ignore_eos ends at the first EOS it samples (token values travel to the
    host every step in that case); the others run to max_tokens."""
    from zipage_amd.engine import SamplingParams, ZipageEngine
    prompts = _prompts(3, [40, 300, 90], seed=4)
    ref, out = _generate(_cfg(use_graph=False), prompts, 60)
    eos = out[0]["token_ids"][20]
    first = out[0]["token_ids"].index(eos)
    cfg = _cfg(use_graph=False, eos=eos)
    eng = ZipageEngine(cfg)
    params = [SamplingParams(max_tokens=60, ignore_eos=False)] + [SamplingParams(max_tokens=60, ignore_eos=True)] * 2
    got = eng.generate(prompts, params)
    assert got[0]["token_ids"] == out[0]["token_ids"][:first + 1]
    assert got[1]["token_ids"] == out[1]["token_ids"] and got[2]["token_ids"] == out[2]["token_ids"]
    assert eng.scheduler.pool.num_free == cfg.num_kvcache_blocks


def test_temperature_sampling_runs_eagerly(dev):
    from zipage_amd.engine import SamplingParams, ZipageEngine
    cfg = _cfg(use_graph=True)
    eng = ZipageEngine(cfg)
    torch.manual_seed(0)
    params = [SamplingParams(max_tokens=40, ignore_eos=True, temperature=t) for t in (0.0, 0.8, 1.5)]
    out = eng.generate(_prompts(3, [33, 64, 100], seed=9), params)
    for o in out:
        assert len(o["token_ids"]) == 40 and all(0 <= t < 503 for t in o["token_ids"])
    # greedy request of the mixed batch equals a greedy-only run of the same prompt
    solo, ref = _generate(_cfg(use_graph=False), _prompts(3, [33, 64, 100], seed=9)[:1], 40)
    assert out[0]["token_ids"][:1] == ref[0]["token_ids"][:1]


def test_prefix_cache_shares_pages_between_equal_prompts(dev):
    """Two requests with the same first page: the second prefill reuses the page (refcount 2),
    attends to it through the block table, and everything is released at the end."""
    from zipage_amd.engine import SamplingParams, ZipageEngine
    base = _prompts(1, [300], seed=11)[0]
    other = base[:256] + _prompts(1, [50], seed=12)[0]
    cfg = _cfg(use_graph=False, enable_prefix_cache=True, max_num_batched_tokens=320)
    eng = ZipageEngine(cfg)
    seen = {}
    orig = eng.runner.run_prefill

    def hooked(seqs):
        for s in seqs:
            seen[s.request_id] = (list(s.block_table), s.num_cached_tokens)
        return orig(seqs)

    eng.runner.run_prefill = hooked
    out = eng.generate([base, other], SamplingParams(max_tokens=20, ignore_eos=True))
    (t0, c0), (t1, c1) = [seen[k] for k in sorted(seen)]
    assert c0 == 0 and c1 == 256 and t0[0] == t1[0] and t0[1] != t1[1]
    assert all(len(o["token_ids"]) == 20 for o in out)
    # the shared first page gives the second request the same first token as a run without sharing
    solo, ref = _generate(_cfg(use_graph=False), [other], 20)
    assert out[1]["token_ids"][0] == ref[0]["token_ids"][0]
    pool = eng.scheduler.pool
    assert pool.num_free == cfg.num_kvcache_blocks and not pool.refcount.any()


def test_identical_page_aligned_prompts_with_prefix_cache(dev):
    """Two identical prompts of exactly one page with the prefix cache on: the second one must
    produce the tokens of a run without sharing (a prompt whose every page hit the cache used to
    skip prefill and decode from a stale token, overwriting the shared page)."""
    prompt = _prompts(1, [256], seed=21)[0]
    _, shared = _generate(_cfg(use_graph=False, enable_prefix_cache=True), [prompt, list(prompt)], 12)
    _, solo = _generate(_cfg(use_graph=False), [prompt], 12)
    assert shared[0]["token_ids"] == solo[0]["token_ids"]
    assert shared[1]["token_ids"] == solo[0]["token_ids"]


def test_reference_script_switches_through_the_engine(dev):
    """The switch set of the reference's scripts (global score with decay 0.8 and max-norm,
    lightning redundancy, pooling, attention sink) through the whole engine: the score cache is
    carried and compacted with the K/V pages, every request completes with the compression count
    its length dictates, graph replay and eager launches agree token for token, and all pages and
    rows come back."""
    from zipage_amd.compress import CompressConfig
    sw = CompressConfig(use_global_score=True, decay_factor=0.8, max_norm=True, enable_pooling=True,
                        pooling_size=5, use_redudancy=True, lightning_redudancy=True,
                        use_attention_sink=True, sink_len=4)
    prompts = _prompts(4, [120, 300, 640, 900], seed=3)
    e1, a = _generate(_cfg(use_graph=False, compress=sw), prompts, 650)
    e2, b = _generate(_cfg(use_graph=True, compress=sw), prompts, 650)
    assert e1.runner.score_cache is not None and e1.stats["compress_calls"] > 2
    BS, cap = 256, 3
    for p, x, y in zip(prompts, a, b):
        assert len(x["token_ids"]) == 650 and x["token_ids"] == y["token_ids"]
        total = len(p) + 650
        first = max(cap, -(-len(p) // BS)) * BS + 1
        want = 0 if total - 1 < first else 1 + (total - 1 - first) // BS
        assert x["num_compressions"] == y["num_compressions"] == want
    for eng in (e1, e2):
        pool = eng.scheduler.pool
        assert pool.num_free == eng.cfg.num_kvcache_blocks and not pool.refcount.any()
