"""GPU parity: every HIP entry point against the CPU oracle on the same seeded inputs.

Bars: bit-exact for copies, masks and indices; for floating-point scores 1e-3 relative
(plus a small absolute floor) with fp32 caches, and at most one unit in the last place of
the cache dtype with bf16/fp16 caches (the reference rounds its intermediates to the cache
dtype, so 1e-3 is below the output's own resolution there).
"""
import pytest
import torch

from oracle import zipage_oracle as O
from tests import cases

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def _ulp_close(got, want, dtype, ulps=1, frac_exact=0.0, abs_floor=1e-30):
    """got/want: tensors in `dtype`.  Every element within `ulps` units in the last place
    (or within `abs_floor`, for values that are the small remainder of a cancelling sum)."""
    g, w = got.float().cpu(), want.float().cpu()
    assert torch.equal(torch.isinf(g), torch.isinf(w))
    fin = torch.isfinite(w)
    g, w = g[fin], w[fin]
    eps = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2.0 ** -24}[dtype]
    tol = ulps * 2 * eps * torch.maximum(w.abs(), g.abs()) + abs_floor
    bad = (g - w).abs() > tol
    if bad.any():
        i = int(((g - w).abs() / tol).argmax())
        raise AssertionError(f"{int(bad.sum())} of {bad.numel()} beyond {ulps} ulp; worst got {g[i].item()!r} "
                             f"want {w[i].item()!r}")
    if frac_exact:
        same = (g == w).float().mean().item()
        assert same >= frac_exact, f"only {same:.4f} bit-identical"


def _rel_close(got, want, rel=1e-3, abs_floor=1e-7):
    g, w = got.float().cpu(), want.float().cpu()
    assert torch.equal(torch.isinf(g), torch.isinf(w))
    fin = torch.isfinite(w)
    err = (g[fin] - w[fin]).abs()
    tol = rel * w[fin].abs() + abs_floor
    assert (err <= tol).all(), f"max rel err {(err / (w[fin].abs() + abs_floor)).max()}"


def _setup(seed, dtype, L=2, B=3, Hkv=2, Hq=8, D=128, W=32, BS=256, nb_choices=(3, 4), budget=2,
           num_pages=24, score_cache=False):
    tables, enc, target = cases.random_tables(seed, B, num_pages, list(nb_choices), budget)
    k, v, q, sc = cases.make_caches(seed, L, num_pages, BS, Hkv, Hq, D, W, B + 2, dtype,
                                    touched=cases.touched_pages(enc), with_score_cache=score_cache)
    seq_idx = torch.tensor([(b * 2 + 1) % (B + 2) for b in range(B)], dtype=torch.int32)
    return dict(k=k, v=v, q=q, sc=sc, enc=enc, target=target, seq_idx=seq_idx, tables=tables)


# ------------------------------------------------------------------ copies / masks
@pytest.mark.parametrize("dtype", DTYPES)
def test_store_query_cache(dev, dtype):
    from zipage_amd.kernel import store_query_cache
    g = torch.Generator().manual_seed(3)
    Ntok, Hq, D, W, S = 37, 8, 128, 16, 5
    q = torch.randn((Ntok, Hq, D), generator=g).to(dtype)
    qc = torch.randn((S, W, Hq, D), generator=g).to(dtype)
    sm = torch.tensor([[0, 1, 3], [36, 4, 15], [7, 0, 0], [8, 0, 1], [20, 2, 9]], dtype=torch.int32)
    want = qc.clone()
    O.store_query_cache(q, want, sm)
    got = qc.clone().to(dev)
    store_query_cache(q.to(dev), got, sm.to(dev))
    assert torch.equal(got.cpu(), want)
    # empty slot mapping and empty cache are no-ops
    store_query_cache(q.to(dev), got, sm[:0].to(dev))
    store_query_cache(q.to(dev), got[:0], sm.to(dev))
    assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("style", ["aliased", "cow"])
def test_compress_kv_bit_exact(dev, dtype, style):
    from zipage_amd.kernel import compress_kv
    s = _setup(11, dtype, L=2, B=4, Hkv=3, Hq=3, nb_choices=(3, 4, 5), budget=2, num_pages=40)
    k, v, enc = s["k"], s["v"], s["enc"]
    L, _, BS, Hkv, D = k.shape
    B, NB = enc.shape
    g = torch.Generator().manual_seed(5)
    scores = torch.rand((L, B, Hkv, NB * BS), generator=g)
    scores = O.pad_mask(scores.view(L, B, Hkv, NB, BS), enc).view(L, B, Hkv, NB * BS)
    flag = O.topk_mask(scores, 2 * BS).view(L, B, Hkv, NB, BS)
    if style == "aliased":   # already-compressed sequences: target = own first pages
        target = s["target"]
    else:                    # copy-on-write: two fresh pages then own pages
        used = cases.touched_pages(enc)
        fresh = [p for p in range(40) if p not in used]
        target = torch.tensor([[fresh[2 * b], fresh[2 * b + 1], t[2]] for b, t in enumerate(s["tables"])],
                              dtype=torch.int32)
    wk, wv = k.clone(), v.clone()
    O.compress_kv_loop(wk, wv, flag, enc, target)
    gk, gv = k.clone().to(dev), v.clone().to(dev)
    compress_kv(gk, gv, flag.to(dev), enc.to(dev), target.to(dev))
    assert torch.equal(gk.cpu().view(torch.uint8), wk.view(torch.uint8))
    assert torch.equal(gv.cpu().view(torch.uint8), wv.view(torch.uint8))


@pytest.mark.parametrize("style", ["aliased", "cow"])
def test_compress_kv_many_rows(dev, style):
    """More than 1 024 (layer, sequence, head) rows: one workgroup per row moves keys and values
    (with fewer rows, as in every other small test, keys and values get workgroups of their own)."""
    from zipage_amd.kernel import compress_kv
    dtype = torch.bfloat16
    L, B, Hkv, BS, D, P = 3, 44, 8, 64, 32, 300
    assert L * B * Hkv > 1024
    s = _setup(17, dtype, L=L, B=B, Hkv=Hkv, Hq=Hkv, D=D, BS=BS, W=16, nb_choices=(3, 4, 5), budget=2,
               num_pages=P)
    k, v, enc = s["k"], s["v"], s["enc"]
    NB = enc.shape[1]
    g = torch.Generator().manual_seed(19)
    scores = O.pad_mask(torch.rand((L, B, Hkv, NB, BS), generator=g), enc).view(L, B, Hkv, NB * BS)
    flag = O.topk_mask(scores, 2 * BS).view(L, B, Hkv, NB, BS)
    if style == "aliased":
        target = s["target"]
    else:
        used = cases.touched_pages(enc)
        fresh = [p for p in range(P) if p not in used]
        assert len(fresh) >= 2 * B
        target = torch.tensor([[fresh[2 * b], fresh[2 * b + 1], t[2]] for b, t in enumerate(s["tables"])],
                              dtype=torch.int32)
    wk, wv = k.clone(), v.clone()
    O.compress_kv_loop(wk, wv, flag, enc, target)
    gk, gv = k.clone().to(dev), v.clone().to(dev)
    compress_kv(gk, gv, flag.to(dev), enc.to(dev), target.to(dev))
    assert torch.equal(gk.cpu().view(torch.uint8), wk.view(torch.uint8))
    assert torch.equal(gv.cpu().view(torch.uint8), wv.view(torch.uint8))


def test_compress_kv_strided_views(dev):
    """key/value as slices of one (2, L, pages, BS, Hkv, D) allocation, layer-sliced."""
    from zipage_amd.kernel import compress_kv
    dtype = torch.bfloat16
    s = _setup(12, dtype, L=3, B=2, Hkv=2, Hq=2, nb_choices=(3,), budget=2, num_pages=10)
    kv = torch.stack([s["k"], s["v"]])
    enc, target = s["enc"], s["target"]
    L, BS, Hkv = 2, 256, 2
    g = torch.Generator().manual_seed(6)
    flag = O.topk_mask(torch.rand((L, 2, Hkv, 3 * BS), generator=g), 2 * BS).view(L, 2, Hkv, 3, BS)
    want = kv.clone()
    O.compress_kv_loop(want[0, 1:3], want[1, 1:3], flag, enc, target)
    got = kv.clone().to(dev)
    compress_kv(got[0, 1:3], got[1, 1:3], flag.to(dev), enc.to(dev), target.to(dev))
    assert torch.equal(got.cpu().view(torch.uint8), want.view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_compress_score_bit_exact(dev, dtype):
    from zipage_amd.kernel import compress_score
    s = _setup(13, dtype, L=2, B=3, Hkv=4, Hq=4, nb_choices=(3, 4), budget=2, num_pages=30,
               score_cache=True)
    enc, target, sc = s["enc"], s["target"], s["sc"]
    L, _, BS, Hkv = sc.shape
    B, NB = enc.shape
    g = torch.Generator().manual_seed(7)
    scores = O.pad_mask(torch.rand((L, B, Hkv, NB, BS), generator=g), enc)
    flag = O.topk_mask(scores.view(L, B, Hkv, NB * BS), 2 * BS).view(L, B, Hkv, NB, BS)
    want = O.compress_score(sc.clone(), flag, enc, target)
    got = compress_score(sc.clone().to(dev), flag.to(dev), enc.to(dev), target.to(dev))
    assert torch.equal(got.cpu().view(torch.uint8), want.view(torch.uint8))


@pytest.mark.parametrize("dtype", DTYPES)
def test_topk_mask_ties_lowest_index(dev, dtype):
    from zipage_amd.kernel import topk_mask
    g = torch.Generator().manual_seed(17)
    rows, T = 24, 2304
    # few distinct values -> massive ties; sprinkle +-inf, zeros of both signs
    x = (torch.randint(0, 40, (rows, T), generator=g).float() / 64.0 - 0.25).to(dtype)
    x[0, :100] = float("inf")
    x[1, 5:300] = float("-inf")
    x[2, ::2] = 0.0
    x[2, 1::2] = -0.0
    x[3] = 0.125
    for k in (2048, 1, T, 0, 777):
        want = O.topk_mask(x, k)
        got = topk_mask(x.to(dev), k).cpu()
        assert got.dtype == torch.bool
        assert torch.equal(got, want), f"k={k}"
        assert (got.sum(-1) == k).all()
    y = torch.randn((3, 2, 5, 1280), generator=g).to(dtype)
    assert torch.equal(topk_mask(y.to(dev), 1024).cpu(), O.topk_mask(y, 1024))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("method", ["max", "sum"])
def test_global_score(dev, dtype, method):
    from zipage_amd.kernel import global_score
    s = _setup(19, dtype, L=2, B=3, Hkv=4, Hq=4, nb_choices=(2, 3), budget=2, num_pages=16,
               score_cache=True)
    enc, sc = s["enc"], s["sc"]
    L, _, BS, Hkv = sc.shape
    B, NB = enc.shape
    g = torch.Generator().manual_seed(23)
    scores = torch.rand((L, B, Hkv, NB, BS), generator=g).to(dtype)
    compressed = torch.tensor([True, False, True])
    ws, wc = scores.clone(), sc.clone()
    O.global_score(ws, wc, enc, compressed, 0.9, method)
    gs, gc = scores.clone().to(dev), sc.clone().to(dev)
    out = global_score(gs, gc, enc.to(dev), compressed.to(dev), 0.9, method)
    assert out.data_ptr() == gs.data_ptr()
    if method == "max" or dtype == torch.float32:
        assert torch.equal(gs.cpu(), ws) and torch.equal(gc.cpu(), wc)
    else:
        _ulp_close(gs, ws, dtype)
        _ulp_close(gc, wc, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("continues", [False, True])
def test_pool_scores(dev, dtype, continues):
    from zipage_amd.kernel import pool_scores
    g = torch.Generator().manual_seed(29)
    L, B, Hkv, NB, BS = 2, 3, 2, 3, 256
    scores = torch.rand((L, B, Hkv, NB, BS), generator=g).to(dtype)
    compressed = torch.tensor([False, True, False])
    for ksz in (5, 7, 1):
        want = O.pool_scores(scores, compressed, ksz, continues)
        got = pool_scores(scores.to(dev), compressed.to(dev), ksz, continues)
        assert torch.equal(got.cpu(), want)
    want = O.pool_scores(scores, compressed, 7, continues, mode="avg")
    got = pool_scores(scores.to(dev), compressed.to(dev), 7, continues, mode="avg")
    _ulp_close(got, want, dtype)
    # all compressed and not continues -> untouched
    allc = torch.tensor([True, True, True])
    assert torch.equal(pool_scores(scores.to(dev), allc.to(dev), 5, False).cpu(),
                       O.pool_scores(scores, allc, 5, False))


@pytest.mark.parametrize("dtype", DTYPES)
def test_window_mask_and_epilogue(dev, dtype):
    from zipage_amd.kernel import window_mask, score_epilogue
    enc = torch.tensor(cases.REF_TABLES["attention"], dtype=torch.int32)
    g = torch.Generator().manual_seed(31)
    L, B, Hkv, NB, BS = 2, 2, 3, 4, 256
    scores = torch.rand((L, B, Hkv, NB, BS), generator=g).to(dtype)
    red = torch.rand((L, B, Hkv, NB, BS), generator=g).to(dtype)
    want = O.window_mask(scores.clone(), enc, 24)
    got = window_mask(scores.clone().to(dev), enc.to(dev), 24)
    assert torch.equal(got.cpu(), want)
    # full epilogue in the runner's order
    w = O.max_normalise(scores.clone())
    w = O.combine_scores(w, O.max_normalise(red.clone()), 0.2)
    w = O.attention_sink(w.contiguous(), 4)
    w = O.window_mask(w, enc, 16)
    w = O.pad_mask(w, enc)
    g2 = score_epilogue(scores.clone().to(dev), enc.to(dev), red.to(dev), max_norm_scores=True,
                        max_norm_red=True, redudancy_lambda=0.2, sink_len=4, window=16,
                        mask_pad=True)
    assert torch.equal(g2.cpu(), w)


@pytest.mark.parametrize("dtype", DTYPES)
def test_key_norm(dev, dtype):
    from zipage_amd.kernel import key_norm
    s = _setup(37, dtype, L=2, B=2, Hkv=3, Hq=3, nb_choices=(2, 3), budget=2, num_pages=12)
    s["k"][0, s["tables"][0][0], 5, 1] = 0  # a zero key clamps to eps
    want = O.key_norm(s["k"], s["enc"])
    got = key_norm(s["k"].to(dev), s["enc"].to(dev))
    if dtype == torch.float32:
        _rel_close(got, want, rel=1e-6)
    else:
        _ulp_close(got, want, dtype, frac_exact=0.999)


# ------------------------------------------------------------------ scorer
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cfg", [dict(Hkv=2, Hq=8, W=32), dict(Hkv=2, Hq=4, W=32),
                                 dict(Hkv=2, Hq=16, W=24), dict(Hkv=3, Hq=3, W=16),
                                 dict(Hkv=1, Hq=7, W=16)])
@pytest.mark.parametrize("reduced", ["mean", "max"])
def test_attention_score(dev, dtype, cfg, reduced):
    from zipage_amd.kernel import attention_score
    s = _setup(41, dtype, L=2, B=3, nb_choices=(2, 3, 4), num_pages=20, **cfg)
    args = (s["k"], s["q"], s["seq_idx"], s["enc"])
    want, wlog = O.attention_score(*args, reduced=reduced, return_logits=True)
    got, glog = attention_score(*(a.to(dev) for a in args), reduced=reduced, return_logits=True)
    assert got.shape == want.shape and got.dtype == dtype
    assert glog.shape == wlog.shape
    if dtype == torch.float32:
        _rel_close(glog, wlog, rel=1e-4, abs_floor=1e-5)
        _rel_close(got, want, rel=1e-3, abs_floor=1e-9)
    else:
        # near-zero logits are the remainder of a cancelling 128-term sum: fp32 order noise
        _ulp_close(glog, wlog, dtype, ulps=1, frac_exact=0.995, abs_floor=2e-6)
        # one logit that rounds the other way moves its probability by exp(ulp(logit)), a
        # few output ulps; the window mean dilutes that, the window max does not
        _ulp_close(got, want, dtype, ulps=2 if reduced == "mean" else 16, frac_exact=0.9)
    # without logits another kernel runs: fp32 caches take the row maximum and the row sum in one
    # sweep (the same to 1e-5); 16-bit caches keep the rounded logits in registers and sweep K
    # once -- the same rounding points, another fp32 summation order of the row sums
    got2 = attention_score(*(a.to(dev) for a in args), reduced=reduced)
    if dtype == torch.float32:
        _rel_close(got2, got, rel=1e-5, abs_floor=1e-12)
        _rel_close(got2, want, rel=1e-3, abs_floor=1e-9)
    else:
        _ulp_close(got2, want, dtype, ulps=2 if reduced == "mean" else 16, frac_exact=0.9)
        _ulp_close(got2, got.cpu(), dtype, ulps=2 if reduced == "mean" else 16, frac_exact=0.97)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("BS,D", [(128, 128), (512, 128), (256, 64), (128, 32), (384, 96)])
def test_attention_score_head_dims_and_page_sizes(dev, dtype, BS, D):
    """Head dims below 128 (part of every staged key row stays zero) and pages of one, two, three
    and four 128-token tiles (the tile -> page mapping is a shift or a division)."""
    from zipage_amd.kernel import attention_score
    s = _setup(59, dtype, L=1, B=3, Hkv=2, Hq=8, D=D, W=32, BS=BS, nb_choices=(2, 3, 4), num_pages=20)
    args = (s["k"], s["q"], s["seq_idx"], s["enc"])
    want = O.attention_score(*args)
    got = attention_score(*(a.to(dev) for a in args))
    assert got.shape == want.shape and got.dtype == dtype
    if dtype == torch.float32:
        _rel_close(got, want, rel=1e-3, abs_floor=1e-9)
    else:
        _ulp_close(got, want, dtype, ulps=2, frac_exact=0.9)


@pytest.mark.parametrize("boost", [1.0, 40.0, 400.0])
def test_attention_score_fp32_logit_range(dev, boost):
    """fp32 caches take the row maximum and the row sum in one sweep, every lane against its own
    reference logit, and fall back to two sweeps when a logit lies far above a reference.  Keys
    of the later pages are scaled up so that the logits' spread is small (merged sweep), near
    the switch-over, and far beyond it (fallback); all three must match the oracle."""
    from zipage_amd.kernel import attention_score
    s = _setup(97, torch.float32, L=1, B=3, nb_choices=(2, 3, 4), num_pages=20, Hkv=2, Hq=8, W=32)
    k = s["k"].clone()
    for t in s["tables"]:
        for pid in t[1:]:
            k[:, pid] *= boost
    args = (k, s["q"], s["seq_idx"], s["enc"])
    want = O.attention_score(*args)
    got = attention_score(*(a.to(dev) for a in args))
    _rel_close(got, want, rel=1e-3, abs_floor=1e-30)
    assert torch.isfinite(got.float()).all()


def _score_three_sweeps(k, q, seq_idx, enc, reduced="mean"):
    """zp_attention_score without the scratch for the window partials: the library then takes
    the kernel that sweeps K three times."""
    from zipage_amd import _lib
    L, P, BS, Hkv, D = k.shape
    _, S, W, Hq, _ = q.shape
    B, NB = enc.shape
    lib = _lib.load()
    out = torch.empty((L, B, Hkv, NB, BS), device=k.device, dtype=k.dtype)
    full = lib.zp_attention_score_workspace(L, B, NB, BS, Hkv, Hq, W)
    assert full > 0
    # more than 128 window x group rows: the three-sweep kernel keeps fp32 partial sums of its
    # own (one row of the scores), still less than the one-sweep kernel asks for
    gp = 1
    while gp < Hq // Hkv:
        gp *= 2
    floor = L * B * Hkv * NB * BS * 4 if (W * gp + 31) // 32 > 4 else 0
    assert floor < full
    ws = torch.empty(max(floor, 1), device=k.device, dtype=torch.uint8)
    _lib.call("zp_attention_score", _lib.dev_ptr(k), _lib.dev_ptr(q), _lib.dev_ptr(seq_idx),
              _lib.dev_ptr(enc), _lib.dev_ptr(out), 0, L, B, NB, BS, Hkv, Hq, D, W, P, S,
              k.stride(0), k.stride(1), q.stride(0), q.stride(1), float(D ** -0.5),
              {"mean": 0, "max": 1}[reduced], _lib.dtype_tag(k), _lib.dev_ptr(ws) if floor else 0,
              floor, _lib.stream_ptr(k))
    return out


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [
    dict(Hkv=2, Hq=8, W=32, nb_choices=(9, 10)),            # four row blocks, 18-20 tiles
    dict(Hkv=2, Hq=8, W=16, nb_choices=(2, 5, 9)),          # two row blocks
    dict(Hkv=1, Hq=7, W=24, nb_choices=(3, 4)),             # group 7 padded to 8: six row blocks
    dict(Hkv=3, Hq=3, W=8, nb_choices=(1, 2)),              # no group, a quarter of a row block
    dict(Hkv=2, Hq=4, W=32, D=64, BS=128, nb_choices=(7, 20)),   # one tile per page, 64-wide heads
    dict(Hkv=2, Hq=8, W=32, BS=384, nb_choices=(2, 6)),     # three tiles per page
])
@pytest.mark.parametrize("reduced", ["mean", "max"])
def test_attention_score_one_sweep_matches_three_sweeps(dev, dtype, shape, reduced):
    """16-bit caches, sequences of at most 2560 tokens: the kernel that keeps the rounded logits
    in registers (one sweep over K) against the three-sweep kernel and against the oracle.  Same
    rounding points; the row sums are added in another order, which moves a few values across a
    rounding boundary."""
    from zipage_amd.kernel import attention_score
    shape = dict(shape)
    nb = shape.pop("nb_choices")
    s = _setup(71, dtype, L=2, B=4, nb_choices=nb, num_pages=48, **shape)
    args = tuple(a.to(dev) for a in (s["k"], s["q"], s["seq_idx"], s["enc"]))
    one = attention_score(*args, reduced=reduced)
    three = _score_three_sweeps(*args, reduced=reduced)
    ulps = 2 if reduced == "mean" else 16
    _ulp_close(one, three.cpu(), dtype, ulps=ulps, frac_exact=0.98)
    want = O.attention_score(s["k"], s["q"], s["seq_idx"], s["enc"], reduced=reduced)
    _ulp_close(one, want, dtype, ulps=ulps, frac_exact=0.9)
    pad = (s["enc"] == -1).view(1, -1, 1, s["enc"].shape[1], 1).expand_as(want)
    assert (one.cpu()[pad] == 0).all()     # pad pages score exactly 0


@pytest.mark.parametrize("shape", [
    dict(Hkv=8, Hq=16, W=32, nb_choices=(9, 10)),           # group 2 (configs[2]): four blocks of 16 rows, 36-40 tiles
    dict(Hkv=2, Hq=8, W=16, nb_choices=(2, 5, 9)),          # group 4
    dict(Hkv=1, Hq=7, W=24, nb_choices=(3, 4)),             # group 7 padded to 8: a window spans two lane groups
    dict(Hkv=1, Hq=16, W=5, nb_choices=(2, 3)),             # group 16: a block is one window
    dict(Hkv=3, Hq=3, W=8, nb_choices=(1, 2)),              # no group, half a block of rows
    dict(Hkv=2, Hq=4, W=32, D=64, BS=128, nb_choices=(7, 20)),   # two tiles per page, 64-wide heads
    dict(Hkv=2, Hq=8, W=32, BS=192, nb_choices=(2, 6)),     # three tiles per page
    dict(Hkv=2, Hq=4, W=12, D=32, BS=64, nb_choices=(5, 33)),    # one tile per page, 32-wide heads
])
@pytest.mark.parametrize("reduced", ["mean", "max"])
def test_attention_score_fp32_one_sweep_matches_two_sweeps(dev, shape, reduced):
    """fp32 caches, sequences of at most 2560 tokens: the kernel that keeps the logits in registers
    (one sweep over K, blocks of 16 query rows) against the kernel that recomputes them and against
    the oracle, to the fp32 tolerance."""
    from zipage_amd import _lib
    from zipage_amd.kernel import attention_score
    shape = dict(shape)
    nb = shape.pop("nb_choices")
    s = _setup(79, torch.float32, L=2, B=4, nb_choices=nb, num_pages=140, **shape)
    args = tuple(a.to(dev) for a in (s["k"], s["q"], s["seq_idx"], s["enc"]))
    L, _, BS, Hkv, _ = s["k"].shape
    B, NB = s["enc"].shape
    Hq, W = s["q"].shape[3], s["q"].shape[2]
    lib = _lib.load()
    need = lib.zp_attention_score_workspace_for(L, B, NB, BS, Hkv, Hq, W, 2)
    assert need == L * B * Hkv * -(-W * max(1, 1 << (Hq // Hkv - 1).bit_length()) // 16) * NB * BS * 4
    assert need <= lib.zp_attention_score_workspace(L, B, NB, BS, Hkv, Hq, W)
    one = attention_score(*args, reduced=reduced)
    two = _score_three_sweeps(*args, reduced=reduced)
    _rel_close(one, two.cpu(), rel=1e-4, abs_floor=1e-9)
    want = O.attention_score(s["k"], s["q"], s["seq_idx"], s["enc"], reduced=reduced)
    _rel_close(one, want, rel=1e-3, abs_floor=1e-9)
    pad = (s["enc"] == -1).view(1, -1, 1, s["enc"].shape[1], 1).expand_as(want)
    assert (one.cpu()[pad] == 0).all()     # pad pages score exactly 0


def test_attention_score_long_rows_take_three_sweeps(dev):
    """More than 2560 tokens do not fit the registers: same entry point, three sweeps."""
    from zipage_amd.kernel import attention_score
    dtype = torch.bfloat16
    s = _setup(73, dtype, L=1, B=2, Hkv=2, Hq=8, W=32, nb_choices=(11, 12), num_pages=32)
    args = (s["k"], s["q"], s["seq_idx"], s["enc"])
    got = attention_score(*(a.to(dev) for a in args))
    _ulp_close(got, O.attention_score(*args), dtype, ulps=2, frac_exact=0.9)


def test_attention_score_reference_script_shape(dev):
    """Shape of the reference's own script: 2 seqs, tables [[0,1,2,-5],[5,6,-9,-1]], W=24,
    Hq=16, Hkv=2, D=128, fp16 (tests/test_attention_score.py:314-358)."""
    from zipage_amd.kernel import attention_score
    dtype = torch.float16
    enc = torch.tensor(cases.REF_TABLES["attention"], dtype=torch.int32)
    k, _, q, _ = cases.make_caches(43, 4, 16, 256, 2, 16, 128, 24, 8, dtype, with_v=False)
    seq_idx = torch.tensor([3, 6], dtype=torch.int32)
    want = O.attention_score(k, q, seq_idx, enc)
    got = attention_score(k.to(dev), q.to(dev), seq_idx.to(dev), enc.to(dev))
    _ulp_close(got, want, dtype, ulps=2, frac_exact=0.9)
    assert (got.cpu()[1, 1, :, 3] == 0).all()  # pad page scores exactly 0


# ------------------------------------------------------------------ redundancy
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("thr", [0.5, 0.0, 0.1])
def test_lightning_redundancy(dev, dtype, thr):
    from zipage_amd.kernel import lightning_redudancy_score
    s = _setup(47, dtype, L=2, B=2, Hkv=2, Hq=2, nb_choices=(2, 3), num_pages=12)
    k = s["k"]
    # correlated keys so that similarities exceed the threshold
    base = torch.randn((1, 1, 1, 2, 128), generator=torch.Generator().manual_seed(1))
    k = (k.float() * 0.6 + base).to(dtype)
    wl, wr = O.lightning_redudancy_score(k, s["enc"], threshold=thr, temperature=0.4,
                                         return_logits=True)
    gl, gr = lightning_redudancy_score(k.to(dev), s["enc"].to(dev), threshold=thr, temperature=0.4,
                                       return_logits=True)
    if dtype == torch.float32:
        _rel_close(gl, wl, rel=1e-4, abs_floor=1e-3)
        _rel_close(gr, wr, rel=1e-3, abs_floor=1e-9)
    else:
        # a fully claimed row sums to exactly 0 in the oracle and to fp32 noise of a
        # ~200-large cancelling sum here: absolute floor
        _ulp_close(gl, wl, dtype, ulps=1, frac_exact=0.97, abs_floor=1e-2)
        _ulp_close(gr, wr, dtype, ulps=2, frac_exact=0.9)


@pytest.mark.parametrize("dtype,scale", [(torch.float16, 2e-5), (torch.float16, 40.0),
                                         (torch.bfloat16, 1e-12), (torch.bfloat16, 1e12)])
@pytest.mark.parametrize("variant", ["lightning", "raw"])
def test_redundancy_key_magnitudes(dev, dtype, scale, variant):
    """The kernels multiply the keys as stored and scale afterwards: keys far from unit norm
    (fp16 subnormal elements included) must give the same cosines as normalising first."""
    from zipage_amd import kernel as K
    s = _setup(71, dtype, L=1, B=2, Hkv=2, Hq=2, BS=64, nb_choices=(2, 3), budget=1, num_pages=12)
    base = torch.randn((1, 1, 1, 2, 128), generator=torch.Generator().manual_seed(9))
    k = ((s["k"].float() * 0.7 + base) * scale).to(dtype)
    if variant == "lightning":
        wl, wr = O.lightning_redudancy_score(k, s["enc"], threshold=0.45, temperature=0.4,
                                             return_logits=True)
        gl, gr = K.lightning_redudancy_score(k.to(dev), s["enc"].to(dev), threshold=0.45,
                                             temperature=0.4, return_logits=True)
    else:
        wl, wr = O.raw_redudancy_score(k, s["enc"], threshold=0.45, temperature=0.4,
                                       return_logits=True)
        gl, gr = K.raw_redudancy_score(k.to(dev), s["enc"].to(dev), threshold=0.45,
                                       temperature=0.4, return_logits=True)
    _ulp_close(gl, wl, dtype, ulps=1, abs_floor=1e-2)
    _ulp_close(gr, wr, dtype, ulps=4)


@pytest.mark.parametrize("dtype,span", [(torch.float16, 6), (torch.bfloat16, 14)])
def test_lightning_redundancy_mixed_key_magnitudes(dev, dtype, span):
    """Every key of a page scaled by its own power of two: the cosines do not change, and the page
    kernel, which sums the keys weighted by 1 / norm on the matrix cores (fp16: in pieces scaled
    per block of 32 keys), must not lose the small weights beside the large ones."""
    from zipage_amd import kernel as K
    s = _setup(97, dtype, L=1, B=2, Hkv=2, Hq=2, BS=256, nb_choices=(2, 3), budget=1, num_pages=10)
    g = torch.Generator().manual_seed(13)
    base = torch.randn((1, 1, 1, 2, 128), generator=g)
    k0 = s["k"].float() * 0.7 + base
    expo = torch.randint(-span, span + 1, k0.shape[:-1] + (1,), generator=g).float()
    kw = dict(threshold=0.45, temperature=0.4, return_logits=True)
    # the unscaled keys rounded first, so that scaling by a power of two is exact in both dtypes
    k = (k0.to(dtype).float() * torch.exp2(expo)).to(dtype)
    wl, wr = O.lightning_redudancy_score(k, s["enc"], **kw)
    gl, gr = K.lightning_redudancy_score(k.to(dev), s["enc"].to(dev), **kw)
    _ulp_close(gl, wl, dtype, ulps=1, abs_floor=1e-2)
    _ulp_close(gr, wr, dtype, ulps=4)
    # and the same scores as the unscaled keys give (the oracle's own invariance, then ours)
    ul, _ = K.lightning_redudancy_score(k0.to(dtype).to(dev), s["enc"].to(dev), **kw)
    _ulp_close(gl, ul.cpu(), dtype, ulps=2, abs_floor=1e-2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("BS,D", [(128, 128), (512, 128), (256, 64), (64, 32), (192, 128)])
@pytest.mark.parametrize("variant", ["lightning", "raw"])
def test_redundancy_page_and_head_sizes(dev, dtype, BS, D, variant):
    """Page sizes on both sides of the 256-key page kernel (and one that is no multiple of 128)
    and head dims below 128, which leave part of every staged key row at zero."""
    from zipage_amd import kernel as K
    s = _setup(83, dtype, L=1, B=2, Hkv=2, Hq=2, D=D, BS=BS, nb_choices=(2, 3), budget=1,
               num_pages=10)
    base = torch.randn((1, 1, 1, 2, D), generator=torch.Generator().manual_seed(11))
    k = (s["k"].float() * 0.7 + base).to(dtype)
    kw = dict(threshold=0.45, temperature=0.4, return_logits=True)
    if variant == "lightning":
        wl, wr = O.lightning_redudancy_score(k, s["enc"], **kw)
        gl, gr = K.lightning_redudancy_score(k.to(dev), s["enc"].to(dev), **kw)
    else:
        wl, wr = O.raw_redudancy_score(k, s["enc"], **kw)
        gl, gr = K.raw_redudancy_score(k.to(dev), s["enc"].to(dev), **kw)
    if dtype == torch.float32:
        _rel_close(gl, wl, rel=1e-4, abs_floor=1e-2)
        _rel_close(gr, wr, rel=1e-3, abs_floor=1e-9)
    else:
        _ulp_close(gl, wl, dtype, ulps=1, abs_floor=1e-2)
        _ulp_close(gr, wr, dtype, ulps=4)


@pytest.mark.parametrize("dtype,BS", [(torch.bfloat16, 64), (torch.float16, 128), (torch.float16, 256)])
def test_lightning_redundancy_long_ragged_tables(dev, dtype, BS):
    """Rows of 1 to 70 pages in one padded table (more entries than a wave has lanes): the page
    kernel walks a row's pages one after the other and skips the padding."""
    from zipage_amd.kernel import lightning_redudancy_score
    perm = torch.randperm(120, generator=torch.Generator().manual_seed(101)).tolist()
    tables, pos = [], 0
    for nb in (9, 70, 1, 33):
        tables.append(perm[pos:pos + nb])
        pos += nb
    enc = O.encode_block_table(tables)
    assert enc.shape == (4, 70) and (enc == -1).any()
    k = cases.make_caches(101, 1, 120, BS, 2, 2, 128, 32, 4, dtype, touched=cases.touched_pages(enc))[0]
    base = torch.randn((1, 1, 1, 2, 128), generator=torch.Generator().manual_seed(3))
    k = (k.float() * 0.7 + base).to(dtype)
    kw = dict(threshold=0.45, temperature=0.4, return_logits=True)
    wl, wr = O.lightning_redudancy_score(k, enc, **kw)
    gl, gr = lightning_redudancy_score(k.to(dev), enc.to(dev), **kw)
    _ulp_close(gl, wl, dtype, ulps=1, abs_floor=1e-2)
    _ulp_close(gr, wr, dtype, ulps=4)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("nb_choices", [(1, 2), (3, 4), (5, 6), (7,)])
def test_raw_redundancy_page_counts(dev, dtype, nb_choices):
    """Sequences of 1..7 pages in one padded table: every assignment of page pairs to
    workgroups (odd and even page counts, wrapped pairs) against the oracle."""
    from zipage_amd.kernel import raw_redudancy_score
    s = _setup(59 + nb_choices[0], dtype, L=1, B=3, Hkv=2, Hq=2, BS=64, nb_choices=nb_choices,
               budget=1, num_pages=30)
    base = torch.randn((1, 1, 1, 2, 128), generator=torch.Generator().manual_seed(7))
    k = (s["k"].float() * 0.7 + base).to(dtype)
    for thr in (0.35, 0.6):
        wl, wr = O.raw_redudancy_score(k, s["enc"], threshold=thr, temperature=0.4,
                                       return_logits=True)
        gl, gr = raw_redudancy_score(k.to(dev), s["enc"].to(dev), threshold=thr, temperature=0.4,
                                     return_logits=True)
        if dtype == torch.float32:
            _rel_close(gl, wl, rel=1e-4, abs_floor=1e-2)
            _rel_close(gr, wr, rel=1e-3, abs_floor=1e-9)
        else:
            _ulp_close(gl, wl, dtype, ulps=1, abs_floor=1e-2)
            _ulp_close(gr, wr, dtype, ulps=4)


@pytest.mark.parametrize("variant", ["lightning", "raw"])
def test_fp32_redundancy_products_are_fp32_grade(dev, variant):
    """fp32 caches: the key products run as two fp16 planes per operand on the 16-bit matrix
    instructions.  With no claims (threshold 2) the logits are plain sums of cosines, which a
    float64 evaluation gives to 1e-15: the distance to it must be what fp32 arithmetic leaves.
    Measured: mean 1.1e-6 / 2.4e-6 (lightning / raw), max 4.9e-6 / 9.5e-6, against 0.9e-6 / 1.5e-6
    and 4.1e-6 / 9.6e-6 with fp32 matrix instructions; a two-plane bf16 split would be 16-64
    times further away, TF32 a thousand times.  Elements of very different sizes inside a key
    (1e-5 .. 1) and keys of very different norms exercise the planes' scale."""
    from zipage_amd import kernel as K
    s = _setup(97, torch.float32, L=1, B=2, Hkv=2, Hq=2, nb_choices=(2, 3), num_pages=12)
    g = torch.Generator().manual_seed(31)
    k = s["k"].float()
    k = k * torch.logspace(-5, 0, 128).view(1, 1, 1, 1, 128)[..., torch.randperm(128, generator=g)]
    k = (k * torch.logspace(-3, 3, k.shape[2]).view(1, 1, -1, 1, 1)).contiguous()
    fn = K.lightning_redudancy_score if variant == "lightning" else K.raw_redudancy_score
    gl, _ = fn(k.to(dev), s["enc"].to(dev), threshold=2.0, temperature=0.4, return_logits=True)
    L, _, BS, Hkv, D = k.shape
    gl = gl.cpu().double().view(L, len(s["tables"]), Hkv, -1, BS)
    worst, total, count = 0.0, 0.0, 0
    for b, table in enumerate(s["tables"]):
        pages = [(j, pid) for j, pid in enumerate(table) if pid >= 0]
        for h in range(Hkv):
            x = torch.cat([k[0, pid, :, h].double() for _, pid in pages])
            x = x / x.norm(dim=-1, keepdim=True).clamp_min(1e-6)
            sim = x @ x.T
            sim.fill_diagonal_(0.0)
            if variant == "lightning":     # only pairs inside a page
                blk = torch.block_diag(*[torch.ones(BS, BS, dtype=torch.float64)] * len(pages))
                sim = sim * blk
            want = sim.sum(1)
            got = torch.cat([gl[0, b, h, j] for j, _ in pages])
            err = (got - want).abs()
            worst = max(worst, err.max().item())
            total += err.sum().item()
            count += err.numel()
    print(f"fp32 {variant}: row sums against float64: max {worst:.2e}, mean {total / count:.2e}")
    max_bound, mean_bound = (1.5e-5, 3e-6) if variant == "lightning" else (3e-5, 7e-6)
    assert worst < max_bound and total / count < mean_bound


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_raw_redundancy(dev, dtype):
    from zipage_amd.kernel import raw_redudancy_score
    s = _setup(53, dtype, L=1, B=2, Hkv=2, Hq=2, nb_choices=(2, 3), num_pages=12)
    base = torch.randn((1, 1, 1, 2, 128), generator=torch.Generator().manual_seed(2))
    k = (s["k"].float() * 0.6 + base).to(dtype)
    wl, wr = O.raw_redudancy_score(k, s["enc"], threshold=0.5, temperature=0.4,
                                   return_logits=True)
    gl, gr = raw_redudancy_score(k.to(dev), s["enc"].to(dev), threshold=0.5, temperature=0.4,
                                 return_logits=True)
    if dtype == torch.float32:
        _rel_close(gl, wl, rel=1e-4, abs_floor=1e-2)
        _rel_close(gr, wr, rel=1e-3, abs_floor=1e-9)
    else:
        _ulp_close(gl, wl, dtype, ulps=1, abs_floor=1e-2)
        _ulp_close(gr, wr, dtype, ulps=4)
