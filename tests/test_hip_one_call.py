"""zp_compress_layers (one host call per layer chunk, caller-passed workspace) against the same
stages issued one entry point at a time: keep flags, K, V and the score cache must be the same
bits, for every switch set the runner has (zipage/engine/model_runner.py:466-622)."""
import pytest
import torch

from tests import cases

pytestmark = pytest.mark.gpu

SWITCHES = {
    "pooling": dict(enable_pooling=True, pooling_size=7),
    "plain": dict(),
    "scripts": dict(use_global_score=True, decay_factor=0.8, enable_pooling=True,
                    use_redudancy=True, lightning_redudancy=True),
    "raw+sink+maxnorm": dict(use_global_score=True, max_norm=True, use_redudancy=True,
                             lightning_redudancy=False, use_attention_sink=True, sink_len=4,
                             enable_pooling=True, continues_pooling=True, pooling_mode="avg",
                             activate_method="sum", decay_factor=0.9, redudancy_lambda=0.5),
    "max-reduced": dict(reduced="max", enable_pooling=True),
}


def _inputs(dtype, seed=91, L=2, B=4, Hkv=2, Hq=8, W=16, budget=2):
    tables, enc, target = cases.random_tables(seed, B, 40, [3, 4], budget)
    k, v, q, sc = cases.make_caches(seed, L, 40, 256, Hkv, Hq, 128, W, B + 1, dtype,
                                    touched=cases.touched_pages(enc), with_score_cache=True)
    base = torch.randn((1, 1, 1, Hkv, 128), generator=torch.Generator().manual_seed(seed + 1))
    k = (k.float() * 0.8 + 0.6 * base).to(dtype)
    qid = torch.arange(B, dtype=torch.int32)
    comp = torch.tensor([False, True, False, True][:B])
    return k, v, q, sc, qid, enc, comp, target


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("name", list(SWITCHES))
@pytest.mark.parametrize("deterministic_carry", [True, False])
def test_one_call_equals_separate_stages(dev, dtype, name, deterministic_carry):
    from zipage_amd.compress import CompressConfig, StageTimer, compress_layers
    kw = SWITCHES[name]
    if not kw.get("use_global_score") and not deterministic_carry:
        pytest.skip("the carried-score mode only matters with the global score on")
    k, v, q, sc, qid, enc, comp, target = _inputs(dtype)
    cfg = CompressConfig(budget_blocks=2, query_cache_len=16, **kw)
    outs = []
    for one_call in (True, False):
        gk, gv, gsc = k.clone().to(dev), v.clone().to(dev), sc.clone().to(dev)
        timer = StageTimer(True)
        res = compress_layers(gk, gv, q.to(dev), gsc, qid.to(dev), enc.to(dev), comp.to(dev),
                              target.to(dev), cfg, timer=timer, return_intermediates=not one_call,
                              deterministic_carry=deterministic_carry)
        torch.cuda.synchronize()
        flag = res if one_call else res[0]
        secs = timer.seconds()
        want = {"attention_score", "pooling+window_mask+topk_mask", "compress_kv"}
        if kw.get("use_global_score"):
            want |= {"global_score", "compress_global_score"}
        if kw.get("use_redudancy"):
            want.add("redudancy_score")
        assert set(secs) == want and all(0 < s < 1 for s in secs.values()), secs
        outs.append((flag.cpu(), gk.cpu(), gv.cpu(), gsc.cpu()))
    for a, b in zip(*outs):
        assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))
    assert (outs[0][0].flatten(3).sum(-1) == 2 * 256).all()


@pytest.mark.parametrize("deterministic_carry", [True, False])
def test_one_call_equals_separate_stages_on_many_rows(dev, deterministic_carry):
    """More than 1 024 (layer, sequence, head) rows with a carried score cache: the compaction
    launch is then the one-workgroup-per-row kernel with the scores' rounds behind the K/V rounds
    (every other test here stays below and gets keys and values in workgroups of their own)."""
    from zipage_amd.compress import CompressConfig, StageTimer, compress_layers
    dtype, L, B, Hkv, Hq, D, BS, W, P = torch.bfloat16, 2, 66, 8, 8, 64, 128, 16, 420
    assert L * B * Hkv > 1024
    tables, enc, target = cases.random_tables(93, B, P, [3, 4], 2)
    k, v, q, sc = cases.make_caches(93, L, P, BS, Hkv, Hq, D, W, B + 1, dtype,
                                    touched=cases.touched_pages(enc), with_score_cache=True)
    base = torch.randn((1, 1, 1, Hkv, D), generator=torch.Generator().manual_seed(94))
    k = (k.float() * 0.8 + 0.6 * base).to(dtype)
    qid = torch.arange(B, dtype=torch.int32)
    comp = torch.tensor([b % 2 == 1 for b in range(B)])
    cfg = CompressConfig(budget_blocks=2, query_cache_len=W, **SWITCHES["scripts"])
    outs = []
    for one_call in (True, False):
        gk, gv, gsc = k.clone().to(dev), v.clone().to(dev), sc.clone().to(dev)
        res = compress_layers(gk, gv, q.to(dev), gsc, qid.to(dev), enc.to(dev), comp.to(dev),
                              target.to(dev), cfg, timer=StageTimer(False),
                              return_intermediates=not one_call,
                              deterministic_carry=deterministic_carry)
        torch.cuda.synchronize()
        flag = res if one_call else res[0]
        outs.append((flag.cpu(), gk.cpu(), gv.cpu(), gsc.cpu()))
    for a, b in zip(*outs):
        assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))
    assert (outs[0][0].flatten(3).sum(-1) == 2 * BS).all()


def test_one_call_rejects_a_short_workspace(dev):
    import ctypes
    from zipage_amd import _lib
    from zipage_amd.compress import CompressConfig, c_config, layer_chunk_args
    k, v, q, sc, qid, enc, comp, target = (t.to(dev) for t in _inputs(torch.bfloat16))
    dims, strides = layer_chunk_args(k, v, q, sc, qid, enc, comp, target)
    cc = c_config(CompressConfig(budget_blocks=2, query_cache_len=16))
    lib = _lib.load()
    need = lib.zp_compress_layers_workspace(*dims[:6], dims[7], 0, ctypes.byref(cc), 1)
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    with pytest.raises(RuntimeError, match="workspace of"):
        _lib.call("zp_compress_layers", k.data_ptr(), v.data_ptr(), q.data_ptr(), 0, qid.data_ptr(),
                  enc.data_ptr(), comp.data_ptr(), target.data_ptr(), 0, *dims, strides, 0,
                  ctypes.byref(cc), ws.data_ptr(), need - 256, None, 0)


@pytest.mark.parametrize("kw", [dict(enable_pooling=True, pooling_size=5),
                                dict(use_global_score=True, decay_factor=0.8)],
                         ids=["pooling", "global-score"])
def test_one_call_on_rows_too_long_for_the_one_launch_selection(dev, kw):
    """A sequence of 80 pages (20 480 tokens) does not fit the one-launch selection's LDS row:
    zp_compress_layers then runs pooling, the mask epilogue and top-k as separate launches on
    copies inside its workspace (the carried scores still come from the untouched scores).  Same
    bits as the separate entry points called from Python."""
    from zipage_amd.compress import CompressConfig, StageTimer, _compress_layers_one_call, compress_layers
    from oracle.zipage_oracle import encode_block_table
    dtype, L, Hkv, Hq, W, budget, NB = torch.bfloat16, 1, 1, 2, 16, 8, 80
    tables = [list(range(NB)), list(range(NB, NB + 12))]
    enc = encode_block_table(tables)
    target = torch.tensor([t[:budget + 1] for t in tables], dtype=torch.int32)
    k, v, q, sc = cases.make_caches(5, L, NB + 12, 256, Hkv, Hq, 128, W, 2, dtype, with_score_cache=True)
    qid = torch.arange(2, dtype=torch.int32)
    comp = torch.tensor([True, False])
    cfg = CompressConfig(budget_blocks=budget, query_cache_len=W, **kw)
    outs = []
    for one_call in (True, False):
        gk, gv, gsc = k.clone().to(dev), v.clone().to(dev), sc.clone().to(dev)
        args = (gk, gv, q.to(dev), gsc, qid.to(dev), enc.to(dev), comp.to(dev), target.to(dev), cfg)
        if one_call:
            flag = _compress_layers_one_call(*args, StageTimer(False), True)
        else:
            flag = compress_layers(*args, fused_select=False)
        torch.cuda.synchronize()
        outs.append((flag.cpu(), gk.cpu(), gv.cpu(), gsc.cpu()))
    for a, b in zip(*outs):
        assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))
    assert (outs[0][0].flatten(3).sum(-1) == budget * 256).all()
