"""16-bit redundancy kernels at a resolution where ONE wrong claim shows.

Keys are near-orthogonal N(0,1) vectors (cosines ~ N(0, 1/128), row sums about +-1.5, one bf16
unit in the last place there is 2^-7) with a few dozen PLANTED pairs at cosine 0.51-1.0 at known
positions: pairs inside a page, pairs across pages (which only the all-pairs variant may claim),
chains of duplicates of duplicates, bit-identical copies and a pair either side of the threshold.
A claimed entry changes its row sum by its cosine, i.e. by 65-128 units in the last place, so a
missing, doubled or misplaced claim cannot hide in the tolerance (1 unit).

Rule under test: diagonal zeroed, then for every column the LAST row over the threshold zeroed,
row sums (zipage/kernel/lightning_redudancy_score.py:136-154,
zipage/kernel/raw_redudancy_score.py:113-131).

The CPU half pins the oracle on the same data against a float64 scalar walk of that rule.
"""
import numpy as np
import pytest
import torch

from oracle import zipage_oracle as O
from tests import cases

BS, D, HKV = 256, 128, 2
THR = 0.5


def planted_case(seed, dtype, nb_choices=(3, 4), B=2, L=1):
    """Returns (k_cache, encoded tables, plan) where plan[(l, b, h)] lists the planted
    (source logical index, destination logical index, cosine) triples."""
    num_pages = 12
    tables, enc, _ = cases.random_tables(seed, B, num_pages, list(nb_choices), 2)
    g = torch.Generator().manual_seed(seed)
    k = torch.zeros((L, num_pages, BS, HKV, D), dtype=torch.float32)
    for p in sorted(cases.touched_pages(enc)):
        k[:, p] = torch.randn((L, BS, HKV, D), generator=g)
    plan = {}
    for l in range(L):
        for b, table in enumerate(tables):
            T = len(table) * BS
            for h in range(HKV):
                def vec(i):
                    return k[l, table[i // BS], i % BS, h]

                def plant(src, dst, c):
                    """key[dst] := cosine c with key[src], same norm as before, the rest of it
                    orthogonal to key[src]."""
                    s = vec(src).double()
                    s = s / s.norm()
                    r = vec(dst).double()
                    n = r.norm()
                    r = r - (r @ s) * s
                    r = r / r.norm()
                    vec(dst).copy_(((c * s + (1 - c * c) ** 0.5 * r) * n).float())

                used, triples = set(), []
                def fresh(lo, hi):
                    while True:
                        i = int(torch.randint(lo, hi, (1,), generator=g))
                        if i not in used:
                            used.add(i)
                            return i

                # pairs inside one page
                for c in (0.6, 0.7, 0.8, 0.9, 0.95, 0.65, 0.75, 0.85):
                    pg = int(torch.randint(0, len(table), (1,), generator=g))
                    a, d = fresh(pg * BS, (pg + 1) * BS), fresh(pg * BS, (pg + 1) * BS)
                    triples.append((a, d, c))
                # pairs across pages (first page <-> last page, neighbours)
                n = len(table)
                for c, (pa, pb) in zip((0.62, 0.78, 0.93, 0.7),
                                       ((0, n - 1), (n - 1, 0), (0, 1), (1, 2 % n))):
                    a, d = fresh(pa * BS, (pa + 1) * BS), fresh(pb * BS, (pb + 1) * BS)
                    triples.append((a, d, c))
                # a chain inside a page and one across pages: duplicate of a duplicate
                a, d, e = fresh(0, BS), fresh(0, BS), fresh(0, BS)
                triples += [(a, d, 0.9), (d, e, 0.9)]
                a, d, e = fresh(0, BS), fresh(BS, 2 * BS), fresh(T - BS, T)
                triples += [(a, d, 0.92), (d, e, 0.92)]
                # bit-identical copies (a survivor copied by an earlier compaction stays behind)
                a, d = fresh(BS, 2 * BS), fresh(BS, 2 * BS)
                triples.append((a, d, 1.0))
                a, d = fresh(0, BS), fresh(T - BS, T)
                triples.append((a, d, 1.0))
                # either side of the threshold
                a, d = fresh(0, BS), fresh(0, BS)
                triples.append((a, d, THR + 0.01))
                a, d = fresh(0, BS), fresh(0, BS)
                triples.append((a, d, THR - 0.01))
                for a, d, c in triples:
                    if c == 1.0:
                        vec(d).copy_(vec(a))
                    else:
                        plant(a, d, c)
                plan[(l, b, h)] = triples
    if dtype == torch.float32:     # fp32 norms are not rounded to a coarser type
        return k, enc, tables, plan
    return _clear_of_norm_boundaries(k.to(dtype)), enc, tables, plan


def _clear_of_norm_boundaries(k, margin=3e-5):
    """The kernels and the oracle both divide a key by its norm ROUNDED to the cache dtype
    (zipage/kernel/key_norm.py:54-56).  A norm whose exact value lies on a rounding boundary of
    that dtype rounds either way depending on the order of the fp32 sum of squares, and the
    other rounding moves every cosine of that key by 2^-11 (fp16) or 2^-8 (bf16) of itself: a
    property of the data, not of the code under test.  Keys whose exact norm lies within
    ``margin`` (relative) of such a boundary get their largest element moved up by one unit in
    the last place until it does not."""
    mant = {torch.bfloat16: 7, torch.float16: 10}[k.dtype]
    flat = k.view(-1, k.shape[-1])
    bits = flat.view(torch.int16)
    for _ in range(64):
        n = flat.double().pow(2).sum(-1).sqrt()
        live = n > 0
        ulp = torch.exp2(torch.floor(torch.log2(n.clamp(min=1e-30))) - mant)
        x = n / ulp
        near = live & (((x - torch.floor(x)) - 0.5).abs() < margin * x)
        if not near.any():
            return k
        rows = torch.nonzero(near).flatten()
        cols = flat[rows].abs().float().argmax(dim=-1)
        bits[rows, cols] += 1          # one ulp further from zero, whatever the sign
    raise AssertionError("could not move every key norm off the rounding boundaries")


def _walk_float64(keys, norms, page_of, thr, same_page_only):
    """Scalar walk of the rule on one head's keys (float64): returns the row sums and the set of
    (row, column) entries that were claimed."""
    e = keys / norms[:, None]
    S = e @ e.T
    n = S.shape[0]
    np.fill_diagonal(S, 0.0)
    if same_page_only:
        S = np.where(page_of[:, None] == page_of[None, :], S, 0.0)
    claimed = set()
    for j in range(n):
        over = np.nonzero(S[:, j] > thr)[0]
        if same_page_only:
            over = over[page_of[over] == page_of[j]]
        if len(over):
            claimed.add((int(over[-1]), j))
    for i, j in claimed:
        S[i, j] = 0.0
    return S.sum(axis=1), claimed


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("variant", ["lightning", "raw"])
def test_oracle_claims_the_planted_pairs(dtype, variant):
    """CPU: on the planted data the oracle's row sums are the float64 walk's, and the walk claims
    what was planted (so the GPU comparison below really exercises claims)."""
    k, enc, tables, plan = planted_case(101, dtype, nb_choices=(2, 3), B=1)
    if variant == "lightning":
        logits = O.lightning_redudancy_logits(k, enc, THR).float()
    else:
        logits = O.raw_redudancy_logits(k, enc, THR, rounding="fp32").float().view(1, 1, HKV, -1, BS)
    norm = O.key_norm(k, enc).double()
    table = tables[0]
    T = len(table) * BS
    for h in range(HKV):
        keys = torch.stack([k[0, table[i // BS], i % BS, h] for i in range(T)]).double().numpy()
        norms = norm[0, 0, h, :len(table)].reshape(-1).numpy()
        page_of = np.arange(T) // BS
        want, claimed = _walk_float64(keys, norms, page_of, THR, variant == "lightning")
        got = logits[0, 0, h, :len(table)].reshape(-1).double().numpy()
        ulp = 2.0 ** (-7 if dtype == torch.bfloat16 else -10)
        assert np.abs(got - want).max() <= ulp * max(1.0, np.abs(want).max()), "oracle row sums"
        pairs = {(a, d) for a, d, c in plan[(0, 0, h)] if c > THR}
        if variant == "lightning":
            pairs = {(a, d) for a, d in pairs if a // BS == d // BS}
        undirected = {frozenset(x) for x in claimed}
        missing = [p for p in pairs if frozenset(p) not in undirected]
        # a pair is only left unclaimed when a later key over the threshold exists in both of its
        # columns (chains); at least 3 in 4 planted pairs must be claimed entries
        assert len(missing) * 4 <= len(pairs), f"planted pairs not claimed: {missing}"
        assert len(claimed) >= len(pairs)


def _close_in_ulps(got, want, dtype, ulps, frac_exact, chain_scale=None):
    g, w = got.float().cpu(), want.float().cpu()
    assert torch.equal(torch.isinf(g), torch.isinf(w))
    fin = torch.isfinite(w)
    g, w = g[fin], w[fin]
    eps = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[dtype]
    # sums near zero are the remainder of cancelling terms: fp32 order noise floor
    tol = ulps * 2 * eps * torch.maximum(w.abs(), g.abs()) + 2e-5
    if chain_scale is not None:
        # the all-pairs variant rounds a running partial sum after every chunk: an fp32 sum on a
        # rounding boundary there moves the result by one unit in the last place of the PARTIAL
        # sum, which can be larger than the result; allow two such flips per row
        tol = tol + 2 * 2 * eps * chain_scale.reshape(-1)[fin.reshape(-1)]
    err = (g - w).abs()
    worst = float((err / tol).max())
    same = float((g == w).float().mean())
    print(f"  worst error {worst:.2f} x tolerance ({ulps} ulp), bit-identical {same:.4f}")
    assert worst <= 1.0, f"{int((err > tol).sum())} of {err.numel()} values beyond {ulps} ulp"
    assert same >= frac_exact, f"only {same:.4f} bit-identical"


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("variant", ["lightning", "raw"])
@pytest.mark.parametrize("thr", [THR, -0.1])
def test_planted_pairs_against_oracle(dev, dtype, variant, thr):
    from zipage_amd import kernel as K
    k, enc, tables, plan = planted_case(103, dtype)
    kw = dict(threshold=thr, temperature=0.4, return_logits=True)
    chain_scale = None
    if variant == "lightning":
        wl, wr = O.lightning_redudancy_score(k, enc, **kw)
        noclaim = O.lightning_redudancy_logits(k, enc, 2.0)
        gl, gr = K.lightning_redudancy_score(k.to(dev), enc.to(dev), **kw)
    else:
        wl, wr = O.raw_redudancy_score(k, enc, rounding=RAW_ORACLE_ROUNDING, **kw)
        noclaim = O.raw_redudancy_logits(k, enc, 2.0, rounding=RAW_ORACLE_ROUNDING)
        chain_scale = O.raw_redudancy_logits(k, enc, thr, rounding=RAW_ORACLE_ROUNDING,
                                             return_partial_max=True)[1]
        gl, gr = K.raw_redudancy_score(k.to(dev), enc.to(dev), **kw)
    if thr > 0:
        # the comparison is only worth something if claims moved many rows by far more than a ulp
        moved = ((noclaim.float().reshape(-1) - wl.float().reshape(-1)).abs() > 0.4)
        moved = moved & torch.isfinite(wl.float().reshape(-1))
        assert int(moved.sum()) >= 2 * 12 * HKV, f"only {int(moved.sum())} rows carry a claim"
    _close_in_ulps(gl, wl, dtype, ulps=1, frac_exact=0.97,
                   chain_scale=chain_scale if variant == "raw" else None)
    _close_in_ulps(gr, wr, dtype, ulps=4, frac_exact=0.5)


@pytest.mark.gpu
@pytest.mark.parametrize("variant", ["lightning", "raw"])
@pytest.mark.parametrize("thr", [THR, -0.1])
def test_planted_pairs_fp32(dev, variant, thr):
    """fp32 caches on the same data: most 32 x 32 tiles hold no entry over the threshold and take
    the kernels' short path, the planted ones take the claim path; a claim moves its row by its
    cosine (>= 0.51), the comparison allows 1e-3."""
    from zipage_amd import kernel as K
    k, enc, tables, plan = planted_case(107, torch.float32)
    kw = dict(threshold=thr, temperature=0.4, return_logits=True)
    if variant == "lightning":
        wl, wr = O.lightning_redudancy_score(k, enc, **kw)
        noclaim = O.lightning_redudancy_logits(k, enc, 2.0)
        gl, gr = K.lightning_redudancy_score(k.to(dev), enc.to(dev), **kw)
    else:
        wl, wr = O.raw_redudancy_score(k, enc, **kw)
        noclaim = O.raw_redudancy_logits(k, enc, 2.0)
        gl, gr = K.raw_redudancy_score(k.to(dev), enc.to(dev), **kw)
    fin = torch.isfinite(wl)
    if thr > 0:
        moved = ((noclaim.reshape(-1) - wl.reshape(-1)).abs() > 0.4) & fin.reshape(-1)
        assert int(moved.sum()) >= 2 * 12 * HKV, f"only {int(moved.sum())} rows carry a claim"
    gl, gr = gl.cpu(), gr.cpu()
    assert torch.equal(torch.isfinite(gl), fin)
    err = (gl[fin] - wl[fin]).abs().max().item()
    assert err < 1e-3, f"row sums off by {err}"
    assert torch.allclose(gr, wr, rtol=1e-3, atol=1e-9)


# rounding chain of the all-pairs variant the GPU kernel is held to: the reference's partial sums
# in the cache dtype (zipage/kernel/raw_redudancy_score.py:146-155,218)
RAW_ORACLE_ROUNDING = "reference"
