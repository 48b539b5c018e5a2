"""GPU parity of the whole compression pipeline (stage order of
zipage/engine/model_runner.py:466-622) against the CPU oracle.

Contract checked here:
  (i)   the final scores agree with the oracle's within the per-dtype bar;
  (ii)  the keep flag is exactly what the oracle's selector picks from the GPU's own scores
        (lowest index wins ties), with exactly k survivors per row;
  (iii) a flag that differs from the oracle's own end-to-end flag sits at a score within the
        tolerance of the row's k-th score (a near-tie, not a selection error);
  (iv)  K, V and the score cache after compaction are bit-identical to the oracle's
        compaction driven by the same flag.
"""
import pytest
import torch

from oracle import zipage_oracle as O
from tests import cases

pytestmark = pytest.mark.gpu


def _run(dev, dtype, cfg_kwargs, seed=61, L=2, B=4, Hkv=2, Hq=8, W=32, budget=2,
         nb_choices=(3, 4), num_pages=40, compressed=(False, True, False, True)):
    from zipage_amd.compress import CompressConfig, compress_layers
    tables, enc, target = cases.random_tables(seed, B, num_pages, list(nb_choices), budget)
    k, v, q, sc = cases.make_caches(seed, L, num_pages, 256, Hkv, Hq, 128, W, B + 1, dtype,
                                    touched=cases.touched_pages(enc), with_score_cache=True)
    # correlated keys so the redundancy threshold matters
    base = torch.randn((1, 1, 1, Hkv, 128), generator=torch.Generator().manual_seed(seed + 1))
    k = (k.float() * 0.8 + 0.6 * base).to(dtype)
    qid = torch.arange(B, dtype=torch.int32)
    comp = torch.tensor(compressed[:B])
    cfg = CompressConfig(budget_blocks=budget, query_cache_len=W, **cfg_kwargs)

    ok, ov, osc = k.clone(), v.clone(), sc.clone()
    oflag, oscores = O.compress_pipeline(
        ok, ov, q, osc, qid, enc, comp, target, budget_blocks=budget, query_cache_len=W,
        return_intermediates=True, **cfg_kwargs)

    gk, gv, gsc = k.clone().to(dev), v.clone().to(dev), sc.clone().to(dev)
    gflag, gscores = compress_layers(gk, gv, q.to(dev), gsc, qid.to(dev), enc.to(dev),
                                     comp.to(dev), target.to(dev), cfg, return_intermediates=True)
    gflag, gscores = gflag.cpu(), gscores.cpu()
    BS = 256
    NB = enc.shape[1]
    kk = BS * budget

    # (i) scores
    gs, os_ = gscores.float(), oscores.float()
    assert torch.equal(torch.isinf(gs), torch.isinf(os_))
    fin = torch.isfinite(os_)
    rel = 1e-3 if dtype == torch.float32 else 2.0 ** -6
    err = (gs[fin] - os_[fin]).abs()
    tol = rel * os_[fin].abs() + 1e-9
    frac_bad = (err > tol).float().mean().item()
    assert frac_bad <= (0.0 if dtype == torch.float32 else 2e-3), f"{frac_bad} of scores off"

    # (ii) selector on the GPU's own scores
    want_flag = O.topk_mask(gscores.view(L, B, Hkv, NB * BS), kk).view_as(gflag)
    assert torch.equal(gflag, want_flag)
    assert (gflag.view(L, B, Hkv, -1).sum(-1) == kk).all()

    # (iii) differences from the oracle's end-to-end flag are near-ties
    diff = gflag != oflag
    if diff.any():
        flat = os_.view(L, B, Hkv, NB * BS)
        kth = flat.topk(kk, dim=-1).values[..., -1:].expand_as(flat).reshape_as(os_)
        gap = (os_ - kth).abs()[diff]
        assert (gap <= 4 * rel * kth[diff].abs() + 1e-9).all(), "flag differs away from the k-th score"
    mism = diff.float().mean().item()
    assert mism <= (1e-4 if dtype == torch.float32 else 2e-2)

    # (iv) compaction driven by the GPU flag
    ck, cv, csc = k.clone(), v.clone(), sc.clone()
    if cfg.use_global_score:
        # the score cache the compaction reads is the one global_score wrote
        s2 = O.attention_score(k, q, qid, enc, None, cfg.reduced)
        if cfg.max_norm:
            s2 = O.max_normalise(s2)
        O.global_score(s2, csc, enc, comp, cfg.decay_factor, cfg.activate_method)
    O.compress_kv(ck, cv, gflag, enc, target)
    assert torch.equal(gk.cpu().view(torch.uint8), ck.view(torch.uint8))
    assert torch.equal(gv.cpu().view(torch.uint8), cv.view(torch.uint8))
    if cfg.use_global_score:
        # carried scores: same walk; values agree to the score tolerance
        O.compress_score(csc, gflag, enc, target)
        touched = sorted(cases.touched_pages(enc))
        a, b_ = gsc.cpu().float()[:, touched], csc.float()[:, touched]
        bad = ((a - b_).abs() > rel * b_.abs() + 1e-9).float().mean().item()
        assert bad <= (0.0 if dtype == torch.float32 else 2e-3), f"{bad} of carried scores off"
    return dict(mismatch=mism)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_pipeline_score_pool_topk_compact(dev, dtype):
    """BASELINE config 1/2 pipeline: score, max-pool 7, top-k, compact."""
    _run(dev, dtype, dict(enable_pooling=True, pooling_size=7))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("lightning", [True, False])
def test_pipeline_global_and_redundancy(dev, dtype, lightning):
    """BASELINE config 3 pipeline: global score (decay 0.9), redundancy, combine, pooling."""
    _run(dev, dtype, dict(use_global_score=True, decay_factor=0.9, enable_pooling=True,
                          pooling_size=7, use_redudancy=True, lightning_redudancy=lightning,
                          redudancy_lambda=0.5))


def test_pipeline_shipping_defaults(dev):
    """The reference scripts' switches (scripts/mathbench.sh:18-32): W=16, lightning
    redundancy lambda 0.2 T 0.4, global score decay 0.8, pooling 5, plus max-norm and sink."""
    _run(dev, torch.bfloat16,
         dict(use_global_score=True, decay_factor=0.8, max_norm=True, enable_pooling=True,
              use_redudancy=True, lightning_redudancy=True, use_attention_sink=True, sink_len=4),
         W=16)
