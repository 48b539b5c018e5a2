"""GPU parity of the one-launch selection (pooling + combine + masks + top-k): bit-exact
against the oracle's separate stages and against the library's own separate entry points."""
import pytest
import torch

from oracle import zipage_oracle as O
from tests import cases

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def _tables(B, NB, seed):
    """Ragged tables with a last page each and trailing pads."""
    g = torch.Generator().manual_seed(seed)
    rows, nxt = [], 0
    for b in range(B):
        nb = NB if b == 0 else int(torch.randint(1, NB + 1, (1,), generator=g))
        ids = list(range(nxt, nxt + nb))
        nxt += nb
        rows.append(ids[:-1] + [-ids[-1] - 2] + [-1] * (NB - nb))
    return torch.tensor(rows, dtype=torch.int32)


def _oracle(scores, enc, compressed, k, pool, continues, mode, red, norm_r, lam, sink, window):
    w = scores
    if pool > 1:
        w = O.pool_scores(w, compressed, pool, continues, mode=mode)
    w = w.clone()
    if red is not None:
        r = O.max_normalise(red.clone()) if norm_r else red
        w = O.combine_scores(w, r, lam)
    if sink:
        w = O.attention_sink(w.contiguous(), sink)
    if window:
        w = O.window_mask(w.contiguous(), enc, window)
    w = O.pad_mask(w.contiguous(), enc)
    L, B, Hkv, NB, BS = w.shape
    return O.topk_mask(w.view(L, B, Hkv, NB * BS), k).view(w.shape), w


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("NB,BS", [(9, 256), (3, 16), (12, 256)])
def test_select_topk_matches_separate_stages(dev, dtype, NB, BS):
    from zipage_amd.kernel import pool_scores, score_epilogue, select_topk, topk_mask
    L, B, Hkv = 2, 4, 2
    g = torch.Generator().manual_seed(41 + NB)
    enc = _tables(B, NB, 43)
    # coarse values: many exact ties, so the lowest-index rule decides a large share of rows
    scores = (torch.randint(0, 50, (L, B, Hkv, NB, BS), generator=g).float() / 256.0).to(dtype)
    red = torch.rand((L, B, Hkv, NB, BS), generator=g).to(dtype)
    compressed = torch.tensor([False, True, False, True])
    d = lambda x: x.to(dev)
    cases_ = [
        dict(pool=7, continues=False, mode="max", red=None, norm_r=False, lam=0.0, sink=0, window=BS // 8),
        dict(pool=5, continues=True, mode="max", red=None, norm_r=False, lam=0.0, sink=4, window=BS // 16),
        dict(pool=0, continues=False, mode="max", red=red, norm_r=True, lam=0.2, sink=0, window=BS // 8),
        dict(pool=3, continues=False, mode="max", red=red, norm_r=False, lam=0.7, sink=2, window=0),
        dict(pool=9, continues=False, mode="max", red=None, norm_r=False, lam=0.0, sink=0, window=BS // 8),
        dict(pool=5, continues=False, mode="avg", red=red, norm_r=True, lam=0.3, sink=1, window=BS // 4),
    ]
    for c in cases_:
        for k in (BS * (NB - 1), 1, 0, NB * BS):
            want_flag, want_scores = _oracle(scores, enc, compressed, k, c["pool"], c["continues"],
                                             c["mode"], c["red"], c["norm_r"], c["lam"], c["sink"],
                                             c["window"])
            flag, out = select_topk(d(scores), d(enc), d(compressed), k, pooling_size=c["pool"],
                                    continues_pooling=c["continues"], pooling_mode=c["mode"],
                                    redundancy=None if c["red"] is None else d(c["red"]),
                                    max_norm_red=c["norm_r"], redudancy_lambda=c["lam"],
                                    sink_len=c["sink"], window=c["window"], mask_pad=True,
                                    return_scores=True)
            assert flag.dtype == torch.bool and (flag.sum((-1, -2)) == k).all()
            if c["mode"] == "max":  # average pooling (an extension) matches the oracle to an ulp only
                assert torch.equal(out.cpu(), want_scores), (c, k)
                assert torch.equal(flag.cpu(), want_flag), (c, k)
            # and the library's separate entry points
            s2 = d(scores)
            if c["pool"] > 1:
                s2 = pool_scores(s2, d(compressed), c["pool"], c["continues"], c["mode"])
            else:
                s2 = s2.clone()
            score_epilogue(s2, d(enc), None if c["red"] is None else d(c["red"]),
                           max_norm_red=c["norm_r"], redudancy_lambda=c["lam"], sink_len=c["sink"],
                           window=c["window"], mask_pad=True)
            f2 = topk_mask(s2.view(L, B, Hkv, NB * BS), k).view(flag.shape)
            assert torch.equal(flag, f2) and torch.equal(out, s2), (c, k)
            # without the scores output the flag is the same
            f3 = select_topk(d(scores), d(enc), d(compressed), k, pooling_size=c["pool"],
                             continues_pooling=c["continues"], pooling_mode=c["mode"],
                             redundancy=None if c["red"] is None else d(c["red"]),
                             max_norm_red=c["norm_r"], redudancy_lambda=c["lam"],
                             sink_len=c["sink"], window=c["window"], mask_pad=True)
            assert torch.equal(f3, flag)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_select_topk_avg_pool_and_special_values(dev, dtype):
    from zipage_amd.kernel import pool_scores, score_epilogue, select_topk, topk_mask
    L, B, Hkv, NB, BS = 1, 3, 2, 4, 256
    g = torch.Generator().manual_seed(47)
    enc = _tables(B, NB, 53)
    scores = torch.rand((L, B, Hkv, NB, BS), generator=g).to(dtype)
    scores[0, 0, 0, 0, :40] = float("inf")
    scores[0, 1, 1, 0, 7:90] = 0.0
    scores[0, 2, 0, 0, ::3] = -0.0
    compressed = torch.zeros(B, dtype=torch.bool)
    d = lambda x: x.to(dev)
    k = BS * 2
    flag, out = select_topk(d(scores), d(enc), d(compressed), k, pooling_size=7, pooling_mode="avg",
                            window=32, return_scores=True)
    s2 = pool_scores(d(scores), d(compressed), 7, False, "avg")
    score_epilogue(s2, d(enc), window=32, mask_pad=True)
    assert torch.equal(out, s2)
    assert torch.equal(flag, topk_mask(s2.view(L, B, Hkv, NB * BS), k).view(flag.shape))


def test_select_topk_rejects_bad_arguments(dev):
    from zipage_amd.kernel import select_topk
    enc = _tables(2, 3, 59).to(dev)
    scores = torch.zeros((1, 2, 2, 3, 256), dtype=torch.bfloat16, device=dev)
    comp = torch.zeros(2, dtype=torch.bool, device=dev)
    with pytest.raises(RuntimeError, match="out of range"):
        select_topk(scores, enc, comp, 3 * 256 + 1)
    with pytest.raises(RuntimeError, match="must be odd"):
        select_topk(scores, enc, comp, 256, pooling_size=4)
    with pytest.raises(RuntimeError, match="window"):
        select_topk(scores, enc, comp, 256, window=257)


def test_select_topk_random_shapes(dev):
    """Thirty random small shapes (rows shorter than the workgroup, pages of 8 to 64 slots, chunk
    boundaries that split pages, k anywhere in [0, T]) against the oracle's separate stages."""
    from zipage_amd.kernel import select_topk
    g = torch.Generator().manual_seed(71)
    ri = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    for trial in range(30):
        dtype = [torch.float32, torch.bfloat16, torch.float16][trial % 3]
        L, B, Hkv = ri(1, 2), ri(1, 3), ri(1, 3)
        BS, NB = [8, 16, 24, 32, 64][ri(0, 4)], ri(1, 12)
        enc = _tables(B, NB, 100 + trial)
        scores = (torch.randint(0, 30, (L, B, Hkv, NB, BS), generator=g).float() / 64.0).to(dtype)
        compressed = torch.rand(B, generator=g) < 0.5
        pool = [0, 3, 5, 7, 9][ri(0, 4)]
        k = ri(0, NB * BS)
        window, sink = ri(0, BS), ri(0, 5)
        want_flag, want_scores = _oracle(scores, enc, compressed, k, pool, bool(trial & 1), "max",
                                         None, False, 0.0, sink, window)
        flag, out = select_topk(scores.to(dev), enc.to(dev), compressed.to(dev), k,
                                pooling_size=pool, continues_pooling=bool(trial & 1), sink_len=sink,
                                window=window, mask_pad=True, return_scores=True)
        case = dict(trial=trial, dtype=dtype, shape=(L, B, Hkv, NB, BS), pool=pool, k=k,
                    window=window, sink=sink)
        assert torch.equal(out.cpu(), want_scores), case
        assert torch.equal(flag.cpu(), want_flag), case
