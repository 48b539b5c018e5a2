"""BASELINE configs[4] at its own batch and attention shape inside the GPU tests: 256 requests,
32 query / 8 kv heads of 128, pages of 256 tokens, budget 8 pages, compression on the side stream
(zipage/engine/zipage_engine.py:137-186, zipage/engine/block_manager.py:129-169).  The model is
two random layers with a small hidden size, so that the test takes seconds: the compression path
sees exactly the tensors of the benchmark (256 sequences x 9 full pages x 8 heads x 128)."""
import pytest
import torch

pytestmark = pytest.mark.gpu

BS, BUDGET, W, REQ = 256, 8, 16, 256


def _engine(use_graph):
    from zipage_amd.compress import CompressConfig
    from zipage_amd.engine import EngineConfig, Qwen3Shape, ZipageEngine
    shape = Qwen3Shape(layers=2, hidden=512, heads=32, kv_heads=8, head_dim=128, intermediate=1024,
                       vocab=2003, max_position=4096)
    cfg = EngineConfig(shape=shape, max_concurrency=REQ, num_kvcache_blocks=REQ * (BUDGET + 1) + 64,
                       kvcache_block_size=BS, max_cache_blocks_per_seq=BUDGET, query_cache_len=W,
                       layer_stride=2, seed=7, max_model_len=4096, enable_async_compress=True,
                       max_compress_blocks=REQ * 16, use_graph=use_graph,
                       compress=CompressConfig(enable_pooling=True, pooling_size=5))
    return ZipageEngine(cfg)


def _row_hash(pages, seed=0):
    """One int64 per (layer, token, head) row of a (L, n, BS, Hkv, D) page stack."""
    L, n, bs, H, D = pages.shape
    g = torch.Generator(device=pages.device).manual_seed(seed)
    w = torch.randint(1, 1 << 40, (D,), generator=g, device=pages.device, dtype=torch.int64)
    return (pages.view(torch.int16).to(torch.int64) * w).sum(-1).view(L, n * bs, H)


def test_256_requests_compress_once_on_the_side_stream(dev):
    from zipage_amd.engine import SamplingParams
    g = torch.Generator().manual_seed(0)
    prompts = [torch.randint(0, 2003, (2040,), generator=g).tolist() for _ in range(REQ)]
    out_tokens = 300      # every sequence reaches 2305 tokens once: one compression each
    runs = []
    for use_graph in (False, True):
        eng = _engine(use_graph)
        r = eng.runner
        seen = []
        orig = r.compress

        def hooked(seqs, **kw):
            torch.cuda.synchronize()
            rec = dict(tables=[list(s.block_table) for s in seqs],
                       targets=[list(s.new_block_table) for s in seqs],
                       release=[list(s.block_to_release) for s in seqs],
                       compressed=[s.compressed for s in seqs], on_side_stream="stream" in kw,
                       k=r.kv_cache[0].clone() if not seen else None)
            ev = orig(seqs, **kw)
            if not seen:
                torch.cuda.synchronize()
                rec["after"] = r.kv_cache[0].clone()
            seen.append(rec)
            return ev

        r.compress = hooked
        out = eng.generate(prompts, SamplingParams(max_tokens=out_tokens, ignore_eos=True))
        runs.append((eng, out, seen))

    (e1, a, seen), (e2, b, seen2) = runs
    # graph replay and eager launches: the same tokens for every request
    for x, y in zip(a, b):
        assert len(x["token_ids"]) == out_tokens and x["token_ids"] == y["token_ids"]
        assert x["num_compressions"] == y["num_compressions"] == 1
    for eng, calls in ((e1, seen), (e2, seen2)):
        assert sum(len(c["tables"]) for c in calls) == REQ and all(c["on_side_stream"] for c in calls)
        assert eng.stats["compress_seqs"] == REQ
        pool = eng.scheduler.pool
        assert pool.num_free == eng.cfg.num_kvcache_blocks and not pool.refcount.any()
    # lock-step prompts: all 256 sequences reach the budget on the same step and go as one call
    first = seen[0]
    assert len(first["tables"]) == REQ
    # page moves follow the copy-on-write rule: nothing shared, never compressed before, so each
    # sequence compacts into its own first nine pages and releases nothing
    for table, target, release, was in zip(first["tables"], first["targets"], first["release"],
                                           first["compressed"]):
        assert len(table) == BUDGET + 1 and not was
        assert target == table[:BUDGET + 1] and release == []
    # stable in-place gather, both layers, every head: the rows of the first eight target pages are
    # an ordered subset of the rows the sequence held, and the last W tokens (the window) survive
    before, after = first["k"], first["after"]
    for table, target in zip(first["tables"], first["targets"]):
        src = _row_hash(before[:, table])                    # (L, T, Hkv)
        dst = _row_hash(after[:, target[:BUDGET]])           # (L, keep, Hkv)
        L, T, H = src.shape
        s = src.permute(0, 2, 1).reshape(L * H, T)
        d = dst.permute(0, 2, 1).reshape(L * H, BUDGET * BS)
        order = torch.argsort(s, dim=1)
        pos = torch.searchsorted(torch.gather(s, 1, order), d)
        idx = torch.gather(order, 1, pos.clamp_max(T - 1))   # source token of every kept row
        assert torch.equal(torch.gather(s, 1, idx), d)
        assert (idx[:, 1:] > idx[:, :-1]).all()
        assert (idx[:, -W:] == torch.arange(T - W, T, device=idx.device)).all()
