"""Pins for the CPU oracle: every function is checked against something that does not share
its formula -- a scalar brute-force walk of the reference's loops on tiny shapes, a dense
textbook/library routine, a closed form or an invariant -- chosen so that a dropped term, a
wrong sign or index, or a transposed operand fails at least one check.  The reference holds
no golden vectors for this path (its tests print differences); the table shapes below are the
ones its scripts use.  Runs on the CPU in seconds.
"""
import math

import pytest
import torch
import torch.nn.functional as F
from hypothesis import given, settings, strategies as st

from oracle import zipage_oracle as O
from tests import cases


def _tiny(seed=0, L=2, P=6, BS=4, Hkv=2, Hq=4, D=8, W=2, S=3, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    k = torch.randn((L, P, BS, Hkv, D), generator=g).to(dtype)
    v = torch.randn((L, P, BS, Hkv, D), generator=g).to(dtype)
    q = torch.randn((L, S, W, Hq, D), generator=g).to(dtype)
    return k, v, q


# ------------------------------------------------------------------ a1 store_query
def test_store_query_arange_scatter():
    """arange-valued Q, triples as in the reference's tests/test_store_query.py:24-65."""
    Ntok, Hq, D, W, S = 10, 2, 4, 3, 4
    q = torch.arange(Ntok * Hq * D, dtype=torch.float32).view(Ntok, Hq, D)
    qc = torch.full((S, W, Hq, D), -1.0)
    sm = torch.tensor([[0, 0, 0], [1, 0, 1], [5, 2, 2], [9, 3, 0]], dtype=torch.int32)
    O.store_query_cache(q, qc, sm)
    for pos, s, slot in sm.tolist():
        assert torch.equal(qc[s, slot], q[pos])
    untouched = torch.ones((S, W), dtype=torch.bool)
    for _, s, slot in sm.tolist():
        untouched[s, slot] = False
    assert (qc[untouched] == -1).all()
    O.store_query_cache(q, qc[:0], sm)  # empty cache: no-op, no error


# ------------------------------------------------------------------ a2 attention score
def _attention_bruteforce(k, q, seq_idx, enc, scale, reduced):
    """Scalar loops over (layer, seq, kv head, token): absolute-position causal rule."""
    L, _, BS, Hkv, D = k.shape
    _, _, W, Hq, _ = q.shape
    B, NB = enc.shape
    G = Hq // Hkv
    out = torch.zeros((L, B, Hkv, NB, BS), dtype=torch.float64)
    for l in range(L):
        for b in range(B):
            pages = [(j, O.decode_page(int(c))) for j, c in enumerate(enc[b].tolist())]
            valid = [(j, p[2]) for j, p in pages if not p[0]]
            T = len(valid) * BS
            for hk in range(Hkv):
                probs = torch.zeros((G, W, T), dtype=torch.float64)
                for g in range(G):
                    for w in range(W):
                        qv = q[l, int(seq_idx[b]), w, hk * G + g].double()
                        logit = torch.full((T,), -math.inf, dtype=torch.float64)
                        q_pos = T - W + w  # window row w sits at this absolute position
                        for n, (j, pid) in enumerate(valid):
                            for s in range(BS):
                                t = n * BS + s
                                last_page = n == len(valid) - 1
                                if last_page and t > q_pos:
                                    continue
                                logit[t] = float((qv * k[l, pid, s, hk].double()).sum()) * scale
                        probs[g, w] = torch.softmax(logit, dim=0)
                r = probs.max(dim=0).values
                r = r.mean(dim=0) if reduced == "mean" else r.max(dim=0).values
                for n, (j, pid) in enumerate(valid):
                    out[l, b, hk, j] = r[n * BS:(n + 1) * BS]
    return out


@pytest.mark.parametrize("reduced", ["mean", "max"])
def test_attention_score_bruteforce(reduced):
    k, _, q = _tiny(seed=1)
    enc = torch.tensor([[0, 2, -7], [4, -3, -1]], dtype=torch.int32)  # last pages 5 and 1
    seq_idx = torch.tensor([2, 0], dtype=torch.int32)
    want = _attention_bruteforce(k, q, seq_idx, enc, 8 ** -0.5, reduced)
    got = O.attention_score(k, q, seq_idx, enc, reduced=reduced).double()
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-7)
    assert (got[:, 1, :, 2] == 0).all()  # pad page scores exactly 0


def test_attention_only_last_page_is_masked():
    """Earlier pages are fully visible even to the first window row; a transposed mask or a
    mask applied to every page would change these numbers."""
    k, _, q = _tiny(seed=2, W=3)
    enc = torch.tensor([[1, -2]], dtype=torch.int32)  # pages 1 then 0 (last)
    logits = O.attention_logits(k, q, torch.tensor([0], dtype=torch.int32), enc)
    BS, W = 4, 3
    assert torch.isfinite(logits[:, 0, :, :, 0, :]).all()
    for w in range(W):
        vis = torch.isfinite(logits[0, 0, 0, w, 1])
        assert vis.tolist() == [s <= BS - W + w for s in range(BS)]


def test_attention_reduces_to_plain_softmax():
    """G=1, W=1: the score is the ordinary attention weight of the single query."""
    k, _, q = _tiny(seed=3, Hq=2, Hkv=2, W=1)
    enc = torch.tensor([[3, 0, -3]], dtype=torch.int32)
    s = O.attention_score(k, q, torch.tensor([1], dtype=torch.int32), enc)
    keys = torch.cat([k[:, 3], k[:, 0], k[:, 1]], dim=1)  # (L, T, Hkv, D)
    logits = torch.einsum("lhd,lthd->lht", q[:, 1, 0], keys) * 8 ** -0.5
    want = torch.softmax(logits, dim=-1)
    assert torch.allclose(s.reshape(2, 2, -1), want, rtol=1e-5, atol=1e-7)
    assert torch.allclose(s.reshape(2, 2, -1).sum(-1), torch.ones(2, 2), atol=1e-5)


def test_attention_reference_rounding_points_are_representable():
    """In reference-rounding mode every returned logit and score is a cache-dtype value and
    the logits equal the fp32 logits rounded once."""
    k, _, q = _tiny(seed=4, dtype=torch.bfloat16)
    enc = torch.tensor([[0, 1, -4], [5, -6, -1]], dtype=torch.int32)
    sidx = torch.tensor([0, 1], dtype=torch.int32)
    s, lg = O.attention_score(k, q, sidx, enc, return_logits=True)
    assert s.dtype == torch.bfloat16 and lg.dtype == torch.bfloat16
    exact = O.attention_logits(k, q, sidx, enc, rounding="fp32").reshape(lg.shape)
    assert torch.equal(lg.float(), exact.to(torch.bfloat16).float())
    with pytest.raises(ValueError):
        O.attention_score(k, q, sidx, enc, reduced="sum")


# ------------------------------------------------------------------ a3 global score
def test_global_score_closed_forms():
    g = torch.Generator().manual_seed(5)
    enc = torch.tensor(cases.REF_TABLES["global"], dtype=torch.int32)  # [[0,1,-4],[8,-9,-1]]
    L, P, BS, Hkv = 2, 10, 4, 3
    scores = torch.rand((L, 2, Hkv, 3, BS), generator=g)
    cache = torch.rand((L, P, BS, Hkv), generator=g)
    comp = torch.tensor([False, True])
    s, c = scores.clone(), cache.clone()
    out = O.global_score(s, c, enc, comp, 0.9, "max")
    assert out is s
    # uncompressed sequence: scores unchanged, cache pages 0,1,2 hold them (slot-major)
    assert torch.equal(s[:, 0], scores[:, 0])
    for j, pid in enumerate([0, 1, 2]):
        assert torch.equal(c[:, pid], scores[:, 0, :, j].permute(0, 2, 1))
    # compressed sequence: page 8 carries max(new, old*0.9); its last page (7) never reads
    want = torch.maximum(scores[:, 1, :, 0], cache[:, 8].permute(0, 2, 1) * 0.9)
    assert torch.allclose(s[:, 1, :, 0], want)
    assert torch.equal(s[:, 1, :, 1], scores[:, 1, :, 1])
    assert torch.equal(c[:, 7], scores[:, 1, :, 1].permute(0, 2, 1))
    # pad page and unrelated cache pages untouched
    assert torch.equal(s[:, 1, :, 2], scores[:, 1, :, 2])
    for pid in (3, 4, 5, 6, 9):
        assert torch.equal(c[:, pid], cache[:, pid])
    # sum variant and decay 0
    s2, c2 = scores.clone(), cache.clone()
    O.global_score(s2, c2, enc, comp, 0.5, "sum")
    assert torch.allclose(s2[:, 1, :, 0], scores[:, 1, :, 0] + 0.5 * cache[:, 8].permute(0, 2, 1))
    s3, c3 = scores.clone(), cache.clone()
    O.global_score(s3, c3, enc, comp, 0.0, "max")
    assert torch.equal(s3, scores)
    with pytest.raises(AssertionError):
        O.global_score(s3, c3, enc, comp, 1.5)
    with pytest.raises(AssertionError):
        O.global_score(s3, c3, enc, comp, 0.5, "mean")


# ------------------------------------------------------------------ a4 pooling
def test_pooling_bruteforce_and_where():
    g = torch.Generator().manual_seed(6)
    L, B, H, NB, BS = 2, 3, 2, 2, 4
    x = torch.rand((L, B, H, NB, BS), generator=g)
    comp = torch.tensor([False, True, False])
    got = O.pool_scores(x, comp, 5)
    flat = x.view(L, B, H, -1)
    T = NB * BS
    for b in range(B):
        for t in range(T):
            lo, hi = max(0, t - 2), min(T, t + 3)
            want = flat[:, b, :, t] if comp[b] else flat[:, b, :, lo:hi].max(-1).values
            assert torch.equal(got.view(L, B, H, -1)[:, b, :, t], want)
    assert torch.equal(O.pool_scores(x, comp, 5, continues_pooling=True).view(L * B, H, T),
                       F.max_pool1d(flat.reshape(L * B, H, T), 5, 1, 2))
    allc = torch.tensor([True, True, True])
    assert O.pool_scores(x, allc, 5) is x  # skipped entirely
    avg = O.pool_scores(x, comp, 3, continues_pooling=True, mode="avg").view(L, B, H, T)
    assert torch.allclose(avg[..., 0], (flat[..., 0] + flat[..., 1]) / 3)


# ------------------------------------------------------------------ a5 key norm
def test_key_norm_library_and_clamp():
    k, _, _ = _tiny(seed=7)
    k[0, 2, 1, 0] = 0
    enc = torch.tensor([[2, -2, -1]], dtype=torch.int32)
    n = O.key_norm(k, enc)
    want = torch.linalg.vector_norm(k[:, 2], dim=-1).permute(0, 2, 1)
    assert torch.allclose(n[:, 0, :, 0], want.clamp(min=1e-6), rtol=1e-6)
    assert n[0, 0, 0, 0, 1] == pytest.approx(1e-6)
    assert torch.allclose(n[:, 0, :, 2], torch.full_like(n[:, 0, :, 2], 1e-6))  # pad page
    nb = O.key_norm(k.to(torch.bfloat16), enc)
    assert nb.dtype == torch.bfloat16


# ------------------------------------------------------------------ a6/a7 redundancy
def _redundancy_bruteforce(keys, thr):
    """keys (T, D) fp64-normalised; the reference's rule, columns claimed last-row-first."""
    T = keys.shape[0]
    sim = [[float((keys[i] * keys[j]).sum()) if i != j else 0.0 for j in range(T)] for i in range(T)]
    claimed = [False] * T
    for i in range(T - 1, -1, -1):          # rows from the end
        for j in range(T):
            if sim[i][j] > thr and not claimed[j]:
                claimed[j] = True
                sim[i][j] = 0.0
    return torch.tensor([sum(row) for row in sim], dtype=torch.float64)


@pytest.mark.parametrize("thr", [0.5, 0.0, 0.2])
def test_lightning_bruteforce(thr):
    g = torch.Generator().manual_seed(8)
    L, P, BS, Hkv, D = 1, 4, 8, 2, 6
    base = torch.randn((1, 1, 1, Hkv, D), generator=g)
    k = torch.randn((L, P, BS, Hkv, D), generator=g) * 0.7 + base
    enc = torch.tensor([[0, 1, -4], [3, -1, -1]], dtype=torch.int32)
    logits = O.lightning_redudancy_logits(k, enc, threshold=thr)
    for b, j, pid in [(0, 0, 0), (0, 1, 1), (0, 2, 2), (1, 0, 3)]:
        for h in range(Hkv):
            kk = k[0, pid, :, h].double()
            kk = kk / kk.norm(dim=-1, keepdim=True)
            want = _redundancy_bruteforce(kk, thr)
            assert torch.allclose(logits[0, b, h, j].double(), want, atol=1e-5)
    assert torch.isinf(logits[0, 1, :, 1:]).all()
    red = O.lightning_redudancy_score(k, enc, threshold=thr, temperature=0.4)
    x = logits.view(1, 2, Hkv, -1) / (0.4 * BS)
    assert torch.allclose(red.view(1, 2, Hkv, -1), torch.softmax(x, -1), atol=1e-6)
    assert torch.allclose(red.view(1, 2, Hkv, -1).sum(-1), torch.ones(1, 2, Hkv), atol=1e-5)


def test_redundancy_special_cases():
    """thr >= 1: nothing is claimed -> plain off-diagonal row sum; orthonormal keys -> all
    similarities 0 -> uniform softmax over the valid tokens."""
    g = torch.Generator().manual_seed(9)
    k = torch.randn((1, 2, 8, 1, 8), generator=g)
    enc = torch.tensor([[0, -3]], dtype=torch.int32)
    lg = O.lightning_redudancy_logits(k, enc, threshold=1.5)
    kh = k[0, 0, :, 0] / k[0, 0, :, 0].norm(dim=-1, keepdim=True)
    sim = kh @ kh.T
    assert torch.allclose(lg[0, 0, 0, 0], sim.sum(-1) - sim.diag(), atol=1e-5)
    eye = torch.eye(8).view(1, 1, 8, 1, 8).repeat(1, 2, 1, 1, 1) * 3.0
    red = O.lightning_redudancy_score(eye, enc)
    assert torch.allclose(red, torch.full_like(red, 1 / 16), atol=1e-6)
    raw = O.raw_redudancy_score(eye, torch.tensor([[0, -1]], dtype=torch.int32))
    assert torch.allclose(raw[0, 0, 0, 0], torch.full((8,), 1 / 8), atol=1e-6)
    assert (raw[0, 0, 0, 1] == 0).all()


def test_raw_bruteforce_and_single_page_equals_lightning():
    g = torch.Generator().manual_seed(10)
    L, P, BS, Hkv, D = 1, 4, 8, 2, 6
    base = torch.randn((1, 1, 1, Hkv, D), generator=g)
    k = torch.randn((L, P, BS, Hkv, D), generator=g) * 0.7 + base
    enc = torch.tensor([[2, 0, -3], [3, -1, -1]], dtype=torch.int32)  # seq0: pages 2,0,1
    lg = O.raw_redudancy_logits(k, enc, threshold=0.5)
    for h in range(Hkv):
        kk = torch.cat([k[0, 2, :, h], k[0, 0, :, h], k[0, 1, :, h]]).double()
        kk = kk / kk.norm(dim=-1, keepdim=True)
        want = _redundancy_bruteforce(kk, 0.5)
        assert torch.allclose(lg[0, 0, h].double(), want, atol=1e-5)
    # one valid page: the whole-sequence variant is the per-page variant
    light = O.lightning_redudancy_logits(k, enc, threshold=0.5)
    assert torch.allclose(lg[0, 1, :, :BS], light[0, 1, :, 0], atol=1e-6)
    # the symmetric restatement used by the reference's own test
    # (tests/test_redudancy_paged.py:17-94): last COLUMN over the threshold per row, then
    # column sums
    for h in range(Hkv):
        kk = torch.cat([k[0, 2, :, h], k[0, 0, :, h], k[0, 1, :, h]]).double()
        kk = kk / kk.norm(dim=-1, keepdim=True)
        sim = kk @ kk.T
        sim.fill_diagonal_(0)
        T = sim.shape[0]
        for i in range(T):
            over = (sim[i] > 0.5).nonzero().flatten()
            if len(over):
                sim[i, over[-1]] = 0
        assert torch.allclose(lg[0, 0, h].double(), sim.sum(0), atol=1e-5)
    red = O.raw_redudancy_score(k, enc, temperature=0.4)
    x = lg[0, 0] / (0.4 * 3 * BS)
    assert torch.allclose(red[0, 0].reshape(Hkv, -1), torch.softmax(x, -1), atol=1e-6)


def _raw_program_walk(e_pages, thr, dtype, block_m=64, block_n=16):
    """The all-pairs kernel's own loop nest, one program per column page
    (zipage/kernel/raw_redudancy_score.py:50-155), on normalised keys ``e_pages[page] (BS, D)``
    fp32: columns in chunks of 16, row pages last to first, rows in blocks of 64 from the end; a
    column is claimed by the first block row that exceeds the threshold in this order (:113-131);
    the block's row sums are added to the column page's partial sums, which are kept in the
    cache dtype (:133-155).  Then the partial sums of the column pages are added in fp32 and
    rounded once (:218)."""
    n_pages, BS = len(e_pages), e_pages[0].shape[0]
    partial = torch.zeros((n_pages, n_pages, BS), dtype=dtype)       # [column page][row page]
    ar = torch.arange(block_m).view(-1, 1)
    for n in range(n_pages):
        for n_off in range(0, BS, block_n):
            cols = e_pages[n][n_off:n_off + block_n]
            zo = torch.zeros((1, block_n), dtype=torch.bool)
            for m in range(n_pages - 1, -1, -1):
                for m_off in range(BS - block_m, -1, -block_m):
                    sim = e_pages[m][m_off:m_off + block_m] @ cols.T
                    if m == n:
                        same = (m_off + ar) == (n_off + torch.arange(block_n).view(1, -1))
                        sim = torch.where(same, torch.zeros_like(sim), sim)
                    tm = (sim > thr) & ~zo
                    last_idx = torch.where(tm, ar.expand_as(sim), torch.full_like(sim, -1, dtype=torch.long)).max(0, keepdim=True).values
                    last = ar == last_idx
                    sim = torch.where(last, torch.zeros_like(sim), sim)
                    zo = zo | last.any(0, keepdim=True)
                    cur = partial[n, m, m_off:m_off + block_m].float()
                    partial[n, m, m_off:m_off + block_m] = (sim.sum(1) + cur).to(dtype)
    return partial.float().sum(0).to(dtype)      # (row page, BS)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_raw_reference_rounding_chain(dtype):
    """The oracle's restatement of the partial-sum chain (16-bit caches) against a literal walk
    of the reference kernel's loop nest: same claims, same chain of cache-dtype roundings.  The
    two add a chunk's 16 similarities in a different fp32 order, so a sum that lands on a rounding
    boundary may differ by one unit in the last place; nothing else may."""
    g = torch.Generator().manual_seed(12)
    L, P, BS, Hkv, D = 1, 5, 64, 2, 8
    base = torch.randn((1, 1, 1, Hkv, D), generator=g)
    k = (torch.randn((L, P, BS, Hkv, D), generator=g) * 0.8 + 0.5 * base).to(dtype)
    enc = torch.tensor([[3, 0, -6, -1], [1, -4, -1, -1]], dtype=torch.int32)   # pages 3,0,4 / 1,2
    thr = 0.5
    got = O.raw_redudancy_logits(k, enc, threshold=thr).view(L, 2, Hkv, 4, BS)
    plain = O.raw_redudancy_logits(k, enc, threshold=thr, rounding="fp32").view(L, 2, Hkv, 4, BS)
    norm = O.key_norm(k, enc)
    tables = [[3, 0, 4], [1, 2]]
    differs_from_plain = 0
    for b, table in enumerate(tables):
        for h in range(Hkv):
            e = [k[0, pid, :, h].float() / norm[0, b, h, j].float().unsqueeze(-1)
                 for j, pid in enumerate(table)]
            want = _raw_program_walk(e, thr, dtype)
            g_ = got[0, b, h, :len(table)].float()
            w_ = want.float()
            eps = 2.0 ** (-8 if dtype == torch.bfloat16 else -11)
            assert ((g_ - w_).abs() <= 2 * eps * w_.abs() + 1e-6).all()
            assert (g_ == w_).float().mean() >= 0.97
            differs_from_plain += int((plain[0, b, h, :len(table)].float() != w_).sum())
        assert torch.isinf(got[0, b, :, len(table):]).all()
    # the chain is not a no-op: rounding once at the end gives other bits on many rows
    assert differs_from_plain > 20


# ------------------------------------------------------------------ a8/a9 closed forms
def test_combine_sink_window_pad():
    g = torch.Generator().manual_seed(11)
    enc = torch.tensor(cases.REF_TABLES["attention"], dtype=torch.int32)
    s = torch.rand((1, 2, 2, 4, 8), generator=g)
    r = torch.rand((1, 2, 2, 4, 8), generator=g)
    c = O.combine_scores(s, r, 0.2)
    assert torch.allclose(c, 0.2 * s - 0.8 * r)
    m = O.max_normalise(s)
    assert torch.allclose(m.reshape(1, 2, 2, -1).max(-1).values, torch.ones(1, 2, 2))
    w = O.window_mask(s.clone(), enc, 3)
    assert torch.isinf(w[0, 0, :, 3, 5:]).all() and torch.isfinite(w[0, 0, :, 3, :5]).all()
    assert torch.isinf(w[0, 1, :, 2, 5:]).all() and torch.isfinite(w[0, 1, :, 3]).all()
    assert torch.equal(w[0, 0, :, :3], s[0, 0, :, :3])
    p = O.pad_mask(s.clone(), enc)
    assert (p[0, 1, :, 3] == -math.inf).all() and torch.equal(p[0, 0], s[0, 0])
    k = O.attention_sink(s.clone(), 10)
    assert torch.isinf(k[0, :, :, 0]).all() and torch.isinf(k[0, :, :, 1, :2]).all()
    assert torch.equal(k[0, :, :, 1, 2:], s[0, :, :, 1, 2:])


# ------------------------------------------------------------------ a10 top-k
@settings(max_examples=150, deadline=None)
@given(st.lists(st.sampled_from([0.0, -0.0, 0.25, 0.5, 1.0, -1.0, math.inf, -math.inf, 3.5]),
                min_size=1, max_size=40), st.data())
def test_topk_properties(vals, data):
    k = data.draw(st.integers(0, len(vals)))
    x = torch.tensor([vals])
    m = O.topk_mask(x, k)[0]
    assert int(m.sum()) == k
    kept, dropped = x[0][m], x[0][~m]
    if k and len(dropped):
        assert kept.min() >= dropped.max()
        # among equals the lower index is kept
        thr = kept.min()
        eq = (x[0] == thr).nonzero().flatten()
        flags = m[eq].tolist()
        assert flags == sorted(flags, reverse=True)
    # brute force: stable order by (-value, index)
    order = sorted(range(len(vals)), key=lambda i: (-vals[i], i))
    want = torch.zeros(len(vals), dtype=torch.bool)
    want[order[:k]] = True
    assert torch.equal(m, want)


# ------------------------------------------------------------------ a11/a12 compaction
@pytest.mark.parametrize("style", ["aliased", "cow"])
def test_compaction_arange_invariants(style):
    """Token id encoded in the value (idea of the reference's tests/test_compress.py:51-58)."""
    L, P, BS, Hkv, D = 1, 12, 4, 2, 3
    k = torch.arange(P * BS, dtype=torch.float32).view(1, P, BS, 1, 1).expand(L, P, BS, Hkv, D).clone()
    k = k + torch.arange(Hkv).view(1, 1, 1, Hkv, 1) * 1000
    v = -k.clone()
    sc = k[..., 0].clone()
    tables = [[5, 2, 7, 1], [9, 3, 0]]
    enc = O.encode_block_table(tables)
    budget = 2
    if style == "aliased":
        target = torch.tensor([[5, 2, 7], [9, 3, 0]], dtype=torch.int32)
    else:
        target = torch.tensor([[10, 11, 7], [4, 6, 0]], dtype=torch.int32)
    g = torch.Generator().manual_seed(12)
    scores = O.pad_mask(torch.rand((L, 2, Hkv, 4, BS), generator=g), enc)
    flag = O.topk_mask(scores.view(L, 2, Hkv, -1), budget * BS).view(L, 2, Hkv, 4, BS)
    k0 = k.clone()
    ka, va = k.clone(), v.clone()
    O.compress_kv_loop(ka, va, flag, enc, target)
    kb, vb = k.clone(), v.clone()
    O.compress_kv(kb, vb, flag, enc, target)
    assert torch.equal(ka, kb) and torch.equal(va, vb)
    assert torch.equal(va, -ka)
    sca = O.compress_score(sc.clone(), flag, enc, target)
    for b, table in enumerate(tables):
        for h in range(Hkv):
            src = [k0[0, pid, s, h, 0].item() for j, pid in enumerate(table) for s in range(BS)
                   if flag[0, b, h, j, s]]
            got = [ka[0, int(target[b, n // BS]), n % BS, h, 0].item() for n in range(budget * BS)]
            assert got == src and src == sorted(src, key=lambda x: src.index(x))
            got_sc = [sca[0, int(target[b, n // BS]), n % BS, h].item() for n in range(budget * BS)]
            assert got_sc == src
    # pages outside every target are untouched
    written = set(target[:, :budget].flatten().tolist())
    for pid in range(P):
        if pid not in written:
            assert torch.equal(ka[:, pid], k0[:, pid])


# ------------------------------------------------------------------ a13 pipeline order
def test_pipeline_order_against_per_token_walk():
    """Tiny end-to-end run against an independent per-row walk that applies the stages in the
    runner's order (zipage/engine/model_runner.py:466-622)."""
    g = torch.Generator().manual_seed(13)
    L, P, BS, Hkv, Hq, D, W, budget = 1, 8, 4, 1, 2, 8, 2, 2
    k = torch.randn((L, P, BS, Hkv, D), generator=g)
    v = torch.randn((L, P, BS, Hkv, D), generator=g)
    q = torch.randn((L, 2, W, Hq, D), generator=g)
    sc = torch.rand((L, P, BS, Hkv), generator=g)
    tables = [[0, 1, 2], [3, 4, 5, 6]]
    enc = O.encode_block_table(tables)
    target = torch.tensor([[0, 1, 2], [3, 4, 5]], dtype=torch.int32)
    comp = torch.tensor([True, False])
    qid = torch.tensor([1, 0], dtype=torch.int32)
    kk, vv, ss = k.clone(), v.clone(), sc.clone()
    flag, final = O.compress_pipeline(
        kk, vv, q, ss, qid, enc, comp, target, budget_blocks=budget, query_cache_len=W,
        use_global_score=True, decay_factor=0.9, enable_pooling=True, pooling_size=3,
        use_redudancy=True, lightning_redudancy=True, redudancy_lambda=0.3,
        redudancy_temperature=0.4, use_attention_sink=True, sink_len=1, return_intermediates=True)
    att = _attention_bruteforce(k, q, qid, enc, D ** -0.5, "mean").float()
    red = O.lightning_redudancy_score(k, enc, temperature=0.4)
    for b, table in enumerate(tables):
        T = len(table) * BS
        a = att[0, b, 0].reshape(-1)[:T].clone()
        if comp[b]:  # carry: every page but the last
            old = torch.cat([sc[0, pid, :, 0] for pid in table])
            carry = torch.maximum(a, old * 0.9)
            a[:T - BS] = carry[:T - BS]
        pooled = a.clone()
        if not comp[b]:
            for t in range(T):
                pooled[t] = a[max(0, t - 1):t + 2].max()
        r = red[0, b, 0].reshape(-1)[:T]
        s = pooled * 0.3 - r * 0.7
        s[:1] = math.inf
        s[T - W:] = math.inf
        assert torch.allclose(final[0, b, 0].reshape(-1)[:T], s, atol=1e-6)
        keep = sorted(sorted(range(T), key=lambda i: (-s[i].item(), i))[:budget * BS])
        assert flag[0, b, 0].reshape(-1)[:T].nonzero().flatten().tolist() == keep
        assert not flag[0, b, 0].reshape(-1)[T:].any()
        for n, t in enumerate(keep):
            assert torch.equal(kk[0, int(target[b, n // BS]), n % BS, 0], k[0, table[t // BS], t % BS, 0])
            assert torch.equal(vv[0, int(target[b, n // BS]), n % BS, 0], v[0, table[t // BS], t % BS, 0])


# ------------------------------------------------------------------ host bookkeeping
def test_query_slot_mapping_rule():
    """model_runner.py:319-350 with BS=256, W=16."""
    qs = O.query_slot_mapping
    assert qs(-1, 256, 16, is_prefill=False, last_block_num_tokens=250) == []
    assert qs(3, 256, 16, is_prefill=False, cu_len=7, last_block_num_tokens=240) == []
    assert qs(3, 256, 16, is_prefill=False, cu_len=7, last_block_num_tokens=241) == [(7, 3, 0)]
    assert qs(3, 256, 16, is_prefill=False, cu_len=7, last_block_num_tokens=256) == [(7, 3, 15)]
    # prefill of 500 tokens: last page holds 244 > 240 -> positions 496..499 at slots 0..3
    assert qs(5, 256, 16, is_prefill=True, cu_len=100, seqlen_q=500) == [
        (100 + 496 + i, 5, i) for i in range(4)]
    assert qs(5, 256, 16, is_prefill=True, seqlen_q=400) == []
    assert qs(5, 256, 16, is_prefill=True, seqlen_q=0) == []


def test_target_block_table_rule():
    """block_manager.py:129-169 with budget+1 = 4."""
    tb = O.target_block_table
    assert tb([7, 8, 9, 10, 11], {}, True, 4, [1, 2]) == ([7, 8, 9, 10], [11], [1, 2])
    new, rel, free = tb([7, 8, 9, 10, 11], {7: 3, 8: 2}, False, 4, [1, 2, 3])
    assert new == [1, 2, 9, 10] and rel == [7, 8, 11] and free == [3]
    assert tb([7, 8, 9, 10, 11], {7: 3, 8: 2}, False, 4, [1]) is None
    new, rel, _ = tb([7, 8, 9, 10, 11], {7: 2, 8: 2, 9: 2, 10: 2}, False, 4, [1, 2, 3])
    assert new == [1, 2, 3, 11] and rel == [7, 8, 9, 10]
    new, rel, _ = tb([7, 8, 9, 10], {}, False, 4, [])
    assert new == [7, 8, 9, 10] and rel == []
    enc = O.encode_block_table([[3, 4, 5], [6, 7]])
    assert enc.tolist() == [[3, 4, -7], [6, -9, -1]]
