"""The benchmark's workload builder: the parts that need no GPU."""
import torch

from zipage_amd.bench.workload import fresh_last_pages, ragged_batch


def _decode(row):
    return [(-c - 2) if c < -1 else c for c in row if c != -1]


def test_fresh_last_pages_only_change_the_last_page():
    wl = ragged_batch(4, L=2, pool_pages=64, budget=8, W=32, seed=5, lengths=(2049, 2304),
                      with_score_cache=True, device="cpu")
    k_before = wl.k.clone()
    own = {p for t in wl.tables for p in t}
    tables, targets = fresh_last_pages(wl, 5)
    assert tables.shape == (5,) + tuple(wl.block_tables.shape) and tables.dtype == torch.int32
    assert targets.shape == (5,) + tuple(wl.targets.shape)
    assert torch.equal(tables[0], wl.block_tables) and torch.equal(targets[0], wl.targets)
    seen = set()
    for i in range(1, 5):
        for b in range(4):
            row, base = _decode(tables[i, b].tolist()), wl.tables[b]
            assert row[:-1] == base[:-1] and tables[i, b, len(base) - 1] < -1   # last page flagged
            new = row[-1]
            assert new not in own and new not in seen
            seen.add(new)
            want = [new if p == base[-1] else p for p in wl.targets[b].tolist()]
            assert targets[i, b].tolist() == want
    new_ids = torch.tensor(sorted(seen))
    old_ids = torch.tensor(sorted(own))
    assert torch.equal(wl.k[:, old_ids], k_before[:, old_ids])         # the workload's pages untouched
    assert torch.isfinite(wl.k[:, new_ids].float()).all() and wl.k[:, new_ids].float().std() > 0.5
    assert torch.isfinite(wl.score_cache[:, new_ids].float()).all()


def test_fresh_last_pages_need_spare_pages():
    wl = ragged_batch(4, pool_pages=40, budget=8, W=32, seed=5, lengths=(2049, 2304), device="cpu")
    assert fresh_last_pages(wl, 3) is None      # 36 pages used, 4 spare, 8 needed
    assert fresh_last_pages(wl, 2) is not None
