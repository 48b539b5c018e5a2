"""GPU edge cases of the drop-in functions: empty batches, a sequence that is one page long,
tables that are mostly padding, and the row-length fallback of the one-launch selection."""
import pytest
import torch

from oracle import zipage_oracle as O
from tests import cases

pytestmark = pytest.mark.gpu


def test_empty_batch_is_a_noop(dev):
    import zipage_amd.kernel as K
    L, P, BS, Hkv, Hq, D, W = 2, 4, 256, 2, 4, 128, 16
    dt = torch.bfloat16
    k = torch.randn(L, P, BS, Hkv, D, device=dev).to(dt)
    v = k.clone()
    q = torch.randn(L, 3, W, Hq, D, device=dev).to(dt)
    sc = torch.rand(L, P, BS, Hkv, device=dev).to(dt)
    k0, v0, sc0 = k.clone(), v.clone(), sc.clone()
    seq = torch.zeros(0, dtype=torch.int32, device=dev)
    enc = torch.zeros((0, 3), dtype=torch.int32, device=dev)
    tgt = torch.zeros((0, 3), dtype=torch.int32, device=dev)
    comp = torch.zeros(0, dtype=torch.bool, device=dev)
    scores = K.attention_score(k, q, seq, enc)
    assert scores.shape == (L, 0, Hkv, 3, BS)
    s2, lg = K.attention_score(k, q, seq, enc, return_logits=True)
    assert lg.shape == (L, 0, Hq, W, 3 * BS)
    assert K.global_score(scores, sc, enc, comp).shape == scores.shape
    assert K.pool_scores(scores, comp, 5).shape == scores.shape
    assert K.window_mask(scores, enc, W).shape == scores.shape
    assert K.key_norm(k, enc).shape == scores.shape
    assert K.lightning_redudancy_score(k, enc).shape == scores.shape
    assert K.raw_redudancy_score(k, enc).shape == scores.shape
    flag = K.select_topk(scores, enc, comp, 2 * BS, pooling_size=5, window=W)
    assert flag.shape == scores.shape and flag.dtype == torch.bool
    assert K.topk_mask(scores.view(L, 0, Hkv, 3 * BS), 2 * BS).shape == (L, 0, Hkv, 3 * BS)
    assert K.compress_kv(k, v, flag, enc, tgt) is None
    assert K.compress_score(sc, flag, enc, tgt) is sc
    K.store_query_cache(torch.zeros(0, Hq, D, device=dev, dtype=dt), q[0],
                        torch.zeros((0, 3), dtype=torch.int32, device=dev))
    torch.cuda.synchronize()
    assert torch.equal(k, k0) and torch.equal(v, v0) and torch.equal(sc, sc0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_single_page_sequences_and_wide_padding(dev, dtype):
    """One sequence is a single (last) page, the other has two pages; both sit in a table six
    wide, so most entries are padding.  Budget 1 page: the short one keeps everything the window
    mask and the top-k leave, the other drops a page's worth."""
    from zipage_amd.compress import CompressConfig, compress_layers
    L, P, BS, Hkv, Hq, D, W = 1, 8, 256, 2, 4, 128, 16
    k, v, q, _ = cases.make_caches(61, L, P, BS, Hkv, Hq, D, W, 2, dtype)
    tables = [[5], [2, 7]]
    enc = O.encode_block_table(tables, pad_to=6)
    target = torch.tensor([[5, 6], [2, 7]], dtype=torch.int32)
    seq_idx = torch.tensor([0, 1], dtype=torch.int32)
    comp = torch.tensor([False, False])
    cfg = CompressConfig(budget_blocks=1, query_cache_len=W, enable_pooling=True, pooling_size=5)
    wk, wv = k.clone(), v.clone()
    want_flag = O.compress_pipeline(wk, wv, q, None, seq_idx, enc, comp, target, budget_blocks=1,
                                    query_cache_len=W, enable_pooling=True, pooling_size=5)
    gk, gv = k.clone().to(dev), v.clone().to(dev)
    d = lambda x: x.to(dev)
    flag, scores = compress_layers(gk, gv, d(q), None, d(seq_idx), d(enc), d(comp), d(target), cfg,
                                   return_intermediates=True)
    assert (flag.sum((-1, -2)) == BS).all()
    assert not flag[:, :, :, 2:].any() and not flag[:, 0, :, 1:].any()     # never a pad token
    # the selector applied to the GPU's own scores, then the compaction driven by those flags
    assert torch.equal(flag.cpu(), O.topk_mask(scores.cpu().view(L, 2, Hkv, -1), BS).view(flag.shape))
    ok, ov = k.clone(), v.clone()
    O.compress_kv(ok, ov, flag.cpu(), enc, target)
    assert torch.equal(gk.cpu(), ok) and torch.equal(gv.cpu(), ov)
    if isinstance(want_flag, tuple):
        want_flag = want_flag[0]
    agree = (flag.cpu() == want_flag).float().mean().item()
    assert agree > 0.995, agree


def test_rows_too_long_for_one_launch_selection_fall_back(dev):
    """A table of 80 pages (20 480 tokens) is beyond what the one-launch selection stages in LDS;
    compress_layers then runs the separate stages and gives the same kind of result."""
    from zipage_amd.compress import CompressConfig, compress_layers
    from zipage_amd.kernel.select import MAX_ROW_TOKENS, select_topk
    L, BS, Hkv, Hq, D, W, NB = 1, 256, 1, 1, 128, 16, 80
    assert NB * BS > MAX_ROW_TOKENS
    P = NB + 2
    g = torch.Generator().manual_seed(67)
    k = torch.randn((L, P, BS, Hkv, D), generator=g).to(torch.bfloat16)
    v = torch.randn((L, P, BS, Hkv, D), generator=g).to(torch.bfloat16)
    q = torch.randn((L, 1, W, Hq, D), generator=g).to(torch.bfloat16)
    enc = O.encode_block_table([list(range(NB))])
    target = torch.tensor([list(range(9))], dtype=torch.int32)
    d = lambda x: x.to(dev)
    cfg = CompressConfig(budget_blocks=8, query_cache_len=W, enable_pooling=True, pooling_size=5)
    gk, gv = d(k.clone()), d(v.clone())
    flag, scores = compress_layers(gk, gv, d(q), None, d(torch.zeros(1, dtype=torch.int32)), d(enc),
                                   d(torch.zeros(1, dtype=torch.bool)), d(target), cfg,
                                   return_intermediates=True)
    assert (flag.sum((-1, -2)) == 8 * BS).all()
    assert torch.equal(flag.cpu(), O.topk_mask(scores.cpu().view(L, 1, Hkv, -1), 8 * BS).view(flag.shape))
    ok, ov = k.clone(), v.clone()
    O.compress_kv(ok, ov, flag.cpu(), enc, target)
    assert torch.equal(gk.cpu(), ok) and torch.equal(gv.cpu(), ov)
    with pytest.raises(RuntimeError, match="exceeds LDS"):
        select_topk(scores, d(enc), d(torch.zeros(1, dtype=torch.bool)), 8 * BS)
