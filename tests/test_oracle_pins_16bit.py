"""Pins for the oracle's 16-bit branches: where it places the cache-dtype roundings.

The reference finishes several stages with ordinary torch ops applied to cache-dtype tensors
(zipage/kernel/attention_score.py:217-247, zipage/kernel/lightning_redudancy_score.py:248-252,
zipage/kernel/raw_redudancy_score.py:226-229, zipage/engine/model_runner.py:482-487,505-530,
551-559).  What such an op rounds, and when, is a property of the library, so the same op
sequence run here on bf16 / fp16 CPU tensors is an independent statement of the result: the
oracle writes the roundings out by hand on fp32 values (``_rnd``), the library applies them by
itself.  Every check below demands bit equality and is accompanied by a mutation check: with
any single one of the oracle's hand-placed roundings left out the comparison fails, so a
misplaced or missing rounding cannot pass.

Also pinned here, on the CPU: this build's race-free handling of the carried scores
(``global_score(write_cache=False)`` + ``compress_score(scores_src=)``) equals the reference's
store-then-read-back mode bit for bit whenever no page is shared.
"""
import pytest
import torch
import torch.nn.functional as F

from oracle import zipage_oracle as O
from tests import cases

DTYPES = [torch.bfloat16, torch.float16]


def _inputs(seed, dtype, L=2, P=12, BS=32, Hkv=2, Hq=8, D=16, W=8, S=3):
    g = torch.Generator().manual_seed(seed)
    k = torch.randn((L, P, BS, Hkv, D), generator=g).to(dtype)
    q = torch.randn((L, S, W, Hq, D), generator=g).to(dtype)
    enc = torch.tensor([[3, 0, 7, -11], [5, -4, -1, -1], [10, 6, -3, -1]], dtype=torch.int32)
    sidx = torch.tensor([2, 0, 1], dtype=torch.int32)
    return k, q, enc, sidx


def _skip_nth_rounding(monkeypatch, n):
    """Make the n-th call of the oracle's ``_rnd`` (counting from 0) the identity."""
    real = O._rnd
    count = {"i": -1}

    def patched(x, dtype, rounding):
        count["i"] += 1
        return x if count["i"] == n else real(x, dtype, rounding)

    monkeypatch.setattr(O, "_rnd", patched)
    return count


# ------------------------------------------------------------------ a2 epilogue
def _attention_epilogue_library(logits, L, B, Hkv, G, W, NB, BS, reduced):
    """The op sequence of attention_score.py:217-247 on the cache-dtype logits tensor."""
    buf = logits.reshape(L, B, Hkv * G, W, -1)
    buf = buf - buf.max(dim=-1, keepdim=True).values
    score = torch.softmax(buf, dim=-1)
    score = score.view(L, B, Hkv, G, W, -1)
    red = torch.max(score, dim=3).values
    red = red.reshape(L, B, Hkv, W, NB, BS)
    if reduced == "mean":
        return red.mean(dim=3)
    return red.max(dim=3).values


@pytest.mark.parametrize("reduced", ["mean", "max"])
@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_epilogue_rounds_where_the_library_does(dtype, reduced, monkeypatch):
    k, q, enc, sidx = _inputs(21, dtype)
    L, _, BS, Hkv, _ = k.shape
    W, Hq = q.shape[2], q.shape[3]
    B, NB = enc.shape
    scores, logits = O.attention_score(k, q, sidx, enc, reduced=reduced, return_logits=True)
    assert scores.dtype == dtype and logits.dtype == dtype
    want = _attention_epilogue_library(logits, L, B, Hkv, Hq // Hkv, W, NB, BS, reduced)
    assert want.dtype == dtype
    assert torch.equal(scores.view(torch.int16), want.view(torch.int16))
    # the data discriminates: leave out any one rounding and the bits change.  The calls are,
    # in order: logits, logit - max, softmax output, window mean (mean only).  Whatever is
    # rounded last is followed only by exact maxima and the cast of the returned tensor, so
    # leaving that one out cannot show.
    n_calls = 4 if reduced == "mean" else 3
    for n in range(n_calls - 1):
        with monkeypatch.context() as m:
            cnt = _skip_nth_rounding(m, n)
            mutated = O.attention_score(k, q, sidx, enc, reduced=reduced)
            assert cnt["i"] == n_calls - 1
        assert not torch.equal(mutated.view(torch.int16), want.view(torch.int16)), n


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_logits_round_once_from_fp32(dtype):
    """attention_score.py:96-129: fp32 dot, fp32 scale, ONE cast to the cache dtype."""
    k, q, enc, sidx = _inputs(22, dtype)
    _, logits = O.attention_score(k, q, sidx, enc, return_logits=True)
    D = k.shape[-1]
    scale = torch.tensor(D ** -0.5, dtype=torch.float32)
    for b in range(enc.shape[0]):
        for j, code in enumerate(enc[b].tolist()):
            pad, last, pid = O.decode_page(code)
            if pad or last:
                continue
            qf = q[:, int(sidx[b])].float()                      # (L, W, Hq, D)
            kf = k[:, pid].float().repeat_interleave(q.shape[3] // k.shape[3], dim=2)
            want = (torch.einsum("lwhd,lshd->lhws", qf, kf) * scale).to(dtype)
            got = logits.view(k.shape[0], enc.shape[0], q.shape[3], q.shape[2],
                              enc.shape[1], k.shape[2])[:, b, :, :, j]
            # fp32 summation order may differ between einsum and matmul by one fp32 ulp;
            # after the single rounding that is at most one unit of the cache dtype, rarely
            same = (got.view(torch.int16) == want.view(torch.int16)).float().mean()
            assert same > 0.99
            assert (got.float() - want.float()).abs().max() <= \
                2.0 ** (-7 if dtype == torch.bfloat16 else -10) * want.float().abs().max()


# ------------------------------------------------------------------ a6 / a7 wrapper epilogue
@pytest.mark.parametrize("dtype", DTYPES)
def test_lightning_wrapper_epilogue_rounds_where_the_library_does(dtype, monkeypatch):
    """lightning_redudancy_score.py:246-252: ``div_(temperature * BS)``, ``x - max``, softmax."""
    k, _, enc, _ = _inputs(23, dtype)
    L, _, BS, Hkv, _ = k.shape
    B, NB = enc.shape
    temperature = 0.4
    logits, red = O.lightning_redudancy_score(k, enc, threshold=0.2, temperature=temperature,
                                              return_logits=True)
    assert logits.dtype == dtype and red.dtype == dtype
    x = logits.clone().view(L, B, Hkv, -1)
    x = x.div_(temperature * BS)
    x = x - x.max(dim=-1, keepdim=True).values
    x = x.softmax(dim=-1).reshape(L, B, Hkv, NB, BS)
    assert torch.equal(red.view(torch.int16), x.view(torch.int16))
    for n in range(2):  # the third rounding is the cast of the returned tensor itself
        with monkeypatch.context() as m:
            _skip_nth_rounding(m, n)
            mutated = O.lightning_redudancy_score(k, enc, threshold=0.2, temperature=temperature)
        assert not torch.equal(mutated.view(torch.int16), x.view(torch.int16)), n


@pytest.mark.parametrize("dtype", DTYPES)
def test_raw_wrapper_epilogue_rounds_where_the_library_does(dtype, monkeypatch):
    """raw_redudancy_score.py:218-229: pad pages -inf, ``div_(temperature * valid_len)`` with a
    per-sequence length tensor, ``x - max``, softmax."""
    k, _, enc, _ = _inputs(24, dtype)
    L, _, BS, Hkv, _ = k.shape
    B, NB = enc.shape
    temperature = 0.7
    logits, red = O.raw_redudancy_score(k, enc, threshold=0.2, temperature=temperature,
                                        return_logits=True)
    x = logits.clone().view(L, B, Hkv, -1)
    seq_length = (enc != -1).sum(dim=-1) * BS
    x = x.div_(temperature * seq_length.unsqueeze(-1).unsqueeze(-1))
    x = x - x.max(dim=-1, keepdim=True).values
    x = x.softmax(dim=-1).reshape(L, B, Hkv, NB, BS)
    assert torch.equal(red.view(torch.int16), x.view(torch.int16))
    # pad pages: -inf logits, exactly zero redundancy
    pad = (enc == -1).view(1, B, 1, NB, 1).expand_as(red)
    assert (red[pad] == 0).all() and torch.isinf(logits.view_as(red)[pad]).all()
    # the partial-sum chain inside raw_redudancy_logits rounds first; the wrapper's three
    # roundings are the last three calls
    with monkeypatch.context() as m:
        cnt = _skip_nth_rounding(m, -1)
        O.raw_redudancy_score(k, enc, threshold=0.2, temperature=temperature)
    total = cnt["i"] + 1
    for n in range(2):
        with monkeypatch.context() as m:
            _skip_nth_rounding(m, total - 3 + n)
            mutated = O.raw_redudancy_score(k, enc, threshold=0.2, temperature=temperature)
        assert not torch.equal(mutated.view(torch.int16), x.view(torch.int16)), n


# ------------------------------------------------------------------ a4 / a8 on 16-bit scores
@pytest.mark.parametrize("dtype", DTYPES)
def test_runner_torch_ops_on_16bit_scores(dtype):
    """max-norm (model_runner.py:482-487), pooling (:505-530) and the redundancy combine
    (:557-559) are torch ops on cache-dtype tensors in the reference.  Each result is compared
    with the same arithmetic spelled out in fp32 with an explicit rounding after every op."""
    g = torch.Generator().manual_seed(25)
    L, B, H, NB, BS = 2, 3, 2, 3, 16
    s = torch.rand((L, B, H, NB, BS), generator=g).to(dtype)
    r = torch.rand((L, B, H, NB, BS), generator=g).to(dtype)
    lam = 0.2

    def rnd(x):
        return x.to(dtype).float()

    # combine: two products and a difference, each rounded; the scalars are used at the
    # precision torch gives a python float next to a 16-bit tensor (fp32 arithmetic)
    got = O.combine_scores(s, r, lam)
    assert got.dtype == dtype
    lam32 = torch.tensor(lam, dtype=torch.float32)
    one_minus = torch.tensor(1 - lam, dtype=torch.float32)
    want = rnd(rnd(s.float() * lam32) - rnd(r.float() * one_minus))
    assert torch.equal(got.float(), want)
    fused = rnd(s.float() * lam32 - r.float() * one_minus)  # one rounding: must differ
    assert not torch.equal(got.float(), fused)

    # max-norm: a quotient of two cache-dtype values, rounded once
    m = O.max_normalise(s)
    flat = s.float().reshape(L, B, H, -1)
    want = rnd(flat / flat.max(dim=-1, keepdim=True).values).reshape(s.shape)
    assert m.dtype == dtype and torch.equal(m.float(), want)
    lib = s.clone().view(L, B, H, -1)
    lib = lib.div_(lib.max(dim=-1, keepdim=True).values).view(s.shape)
    assert torch.equal(m.view(torch.int16), lib.view(torch.int16))

    # pooling: a max of cache-dtype values is exact, no rounding; library op on the 16-bit tensor
    comp = torch.tensor([False, True, False])
    p = O.pool_scores(s.clone(), comp, 5)
    flat = s.view(L * B, H, -1)
    lib = F.max_pool1d(flat, kernel_size=5, stride=1, padding=2)
    mask = comp.unsqueeze(0).expand(L, B).unsqueeze(-1).unsqueeze(-1).reshape(L * B, 1, 1)
    lib = torch.where(mask, flat, lib).view(s.shape)
    assert torch.equal(p.view(torch.int16), lib.view(torch.int16))


@pytest.mark.parametrize("method", ["max", "sum"])
@pytest.mark.parametrize("dtype", DTYPES)
def test_global_score_16bit_rounds_once(dtype, method):
    """global_score.py:60-70: cache and new score are widened to fp32, combined there, and the
    result is cast once to the scores' dtype."""
    g = torch.Generator().manual_seed(26)
    enc = torch.tensor(cases.REF_TABLES["global"], dtype=torch.int32)
    L, P, BS, Hkv = 2, 10, 16, 3
    scores = torch.rand((L, 2, Hkv, 3, BS), generator=g).to(dtype)
    cache = torch.rand((L, P, BS, Hkv), generator=g).to(dtype)
    comp = torch.tensor([False, True])
    s, c = scores.clone(), cache.clone()
    O.global_score(s, c, enc, comp, 0.9, method)
    old = cache[:, 8].permute(0, 2, 1).float() * torch.tensor(0.9, dtype=torch.float32)
    new = scores[:, 1, :, 0].float()
    want = (torch.maximum(new, old) if method == "max" else new + old).to(dtype)
    assert torch.equal(s[:, 1, :, 0].view(torch.int16), want.view(torch.int16))
    assert torch.equal(c[:, 8].view(torch.int16), want.permute(0, 2, 1).contiguous().view(torch.int16))
    if method == "sum":  # rounding the decayed value first would differ somewhere
        twice = (new + old.to(dtype).float()).to(dtype)
        assert not torch.equal(twice.view(torch.int16), want.view(torch.int16))


# ------------------------------------------------------------------ race-free carry
def _carry_case(seed, dtype, shared):
    L, P, BS, Hkv, Hq, D, W, budget = 2, 24, 8, 2, 4, 8, 4, 2
    g = torch.Generator().manual_seed(seed)
    k = torch.randn((L, P, BS, Hkv, D), generator=g).to(dtype)
    v = torch.randn((L, P, BS, Hkv, D), generator=g).to(dtype)
    q = torch.randn((L, 3, W, Hq, D), generator=g).to(dtype)
    sc = torch.rand((L, P, BS, Hkv), generator=g).to(dtype)
    if shared:   # sequences 0 and 2 share their first page, copy-on-write targets
        tables = [[0, 1, 2, 3], [4, 5, 6], [0, 7, 8, 9]]
        targets = [[20, 1, 2], [4, 5, 6], [21, 7, 8]]
        comp = [False, True, False]
    else:
        tables = [[0, 1, 2, 3], [4, 5, 6], [10, 7, 8, 9]]
        targets = [[0, 1, 2], [4, 5, 6], [10, 7, 8]]
        comp = [True, True, False]
    enc = O.encode_block_table(tables)
    return (k, v, q, sc, torch.arange(3, dtype=torch.int32), enc, torch.tensor(comp),
            torch.tensor(targets, dtype=torch.int32), budget, W)


@pytest.mark.parametrize("method", ["max", "sum"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_race_free_carry_equals_reference_mode_without_sharing(dtype, method):
    k, v, q, sc, qid, enc, comp, tgt, budget, W = _carry_case(31, dtype, shared=False)
    kw = dict(budget_blocks=budget, query_cache_len=W, use_global_score=True,
              activate_method=method, decay_factor=0.8, enable_pooling=True, pooling_size=3)
    k1, v1, s1 = k.clone(), v.clone(), sc.clone()
    f1 = O.compress_pipeline(k1, v1, q, s1, qid, enc, comp, tgt, deterministic_carry=False, **kw)
    k2, v2, s2 = k.clone(), v.clone(), sc.clone()
    f2 = O.compress_pipeline(k2, v2, q, s2, qid, enc, comp, tgt, deterministic_carry=True, **kw)
    assert torch.equal(f1, f2) and torch.equal(k1, k2) and torch.equal(v1, v2)
    # the written target pages hold the same carried scores; pages the race-free mode never
    # writes (sources that are not targets) keep their old contents there
    BS = k.shape[2]
    for b in range(enc.shape[0]):
        for j in range(budget):
            pid = int(tgt[b, j])
            assert torch.equal(s1[:, pid], s2[:, pid]), (b, j)
    written = {int(p) for p in tgt[:, :budget].flatten()}
    for pid in range(sc.shape[1]):
        if pid not in written:
            assert torch.equal(s2[:, pid], sc[:, pid]), pid
    assert BS * budget == int(f1[0, 0, 0].sum())


def test_race_free_carry_stages_equal_reference_stages():
    """Stage level: ``global_score(write_cache=False)`` returns the same scores as the
    reference mode and leaves the cache alone; ``compress_score(scores_src=)`` then moves the
    values the reference mode would have stored and read back."""
    g = torch.Generator().manual_seed(32)
    L, P, BS, Hkv, B, NB, budget = 2, 12, 8, 2, 2, 3, 2
    enc = O.encode_block_table([[0, 1, 2], [5, 6, 7]])
    tgt = torch.tensor([[0, 1, 2], [5, 6, 7]], dtype=torch.int32)
    comp = torch.tensor([True, False])
    scores = torch.rand((L, B, Hkv, NB, BS), generator=g)
    cache = torch.rand((L, P, BS, Hkv), generator=g)
    flag = O.topk_mask(torch.rand((L, B, Hkv, NB * BS), generator=g), BS * budget)
    flag = flag.view(L, B, Hkv, NB, BS)
    s1, c1 = scores.clone(), cache.clone()
    O.global_score(s1, c1, enc, comp, 0.8, "max")
    O.compress_score(c1, flag, enc, tgt)
    s2, c2 = scores.clone(), cache.clone()
    O.global_score(s2, c2, enc, comp, 0.8, "max", write_cache=False)
    assert torch.equal(c2, cache) and torch.equal(s1, s2)
    O.compress_score(c2, flag, enc, tgt, scores_src=s2)
    for b in range(B):
        for j in range(budget):
            assert torch.equal(c1[:, int(tgt[b, j])], c2[:, int(tgt[b, j])])


def test_race_free_carry_is_order_independent_under_sharing():
    """With a shared source page the reference mode depends on which sequence stored last; the
    race-free mode does not: permuting the batch permutes its results and nothing else."""
    k, v, q, sc, qid, enc, comp, tgt, budget, W = _carry_case(33, torch.float32, shared=True)
    kw = dict(budget_blocks=budget, query_cache_len=W, use_global_score=True,
              deterministic_carry=True)
    k1, v1, s1 = k.clone(), v.clone(), sc.clone()
    f1 = O.compress_pipeline(k1, v1, q, s1, qid, enc, comp, tgt, **kw)
    perm = torch.tensor([2, 1, 0])
    k2, v2, s2 = k.clone(), v.clone(), sc.clone()
    f2 = O.compress_pipeline(k2, v2, q, s2, qid[perm], enc[perm], comp[perm], tgt[perm], **kw)
    assert torch.equal(f1[:, perm], f2)
    assert torch.equal(k1, k2) and torch.equal(v1, v2) and torch.equal(s1, s2)
    assert torch.equal(s1[:, 0], sc[:, 0])  # the shared (read-only) page is never written
