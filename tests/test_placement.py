"""Pool placement: the choice logic on the CPU, the timed gather on the GPU."""
import pytest
import torch

from zipage_amd.bench.placement import place_kv_pools, place_pools


def test_place_pools_keeps_fastest_and_releases_the_rest():
    alive, peak, made = set(), [0], [0]

    class Pool:
        def __init__(self):
            self.i = made[0]
            made[0] += 1
            alive.add(self.i)
            peak[0] = max(peak[0], len(alive))

        def __del__(self):
            alive.discard(self.i)

    times = [200.0, 190.0, 205.0, 175.0, 150.0]
    best, rep = place_pools(Pool, lambda p: times[p.i], tries=4)
    assert best.i == 3 and rep == {"tries": 4, "probe_us": [200.0, 190.0, 205.0, 175.0], "kept": 3}
    assert peak[0] == 4 and alive == {3}  # all candidates alive while probing, then only the winner


def test_place_pools_stops_early_and_single_try():
    times = [200.0, 176.0, 150.0]
    made = []

    def alloc():
        made.append(len(made))
        return made[-1]

    best, rep = place_pools(alloc, lambda i: times[i], tries=3, good_enough=175.0)
    assert best == 1 and rep["tries"] == 2 and rep["kept"] == 1
    best, rep = place_pools(lambda: 7, lambda i: 1.0, tries=0)
    assert best == 7 and rep["tries"] == 1


def test_place_kv_pools_stops_at_the_first_pair_in_different_zones():
    # slabs 0-3 in one zone, 4.. in another: the first pair across the boundary ends the search
    zone = [0, 0, 0, 0, 1, 1, 1, 1]
    alive, made = set(), [0]

    class Pool:
        def __init__(self):
            self.i = made[0]
            made[0] += 1
            alive.add(self.i)

        def __del__(self):
            alive.discard(self.i)

    (k, v), rep = place_kv_pools(Pool, lambda a, b: 170.0 if zone[a.i] != zone[b.i] else 196.0 + b.i, 8)
    assert (k.i, v.i) == (0, 4) and rep["slabs"] == 5 and rep["kept"] == [0, 4]
    assert rep["probe_us"] == {"0-1": 197.0, "0-2": 198.0, "0-3": 199.0, "0-4": 170.0}
    assert alive == {0, 4}


def test_place_kv_pools_limits():
    made = []

    def alloc():
        made.append(len(made))
        return made[-1]

    (k, v), rep = place_kv_pools(alloc, lambda a, b: 200.0 - b, 3)       # slab limit, no fast pair
    assert (k, v) == (0, 2) and rep["slabs"] == 3
    made.clear()
    (k, v), rep = place_kv_pools(alloc, lambda a, b: 200.0, 16, span_bytes=50e9, pool_bytes=10e9)
    assert rep["slabs"] == 5 and (k, v) == (0, 1)                        # 5 x 10 GB is the span
    made.clear()
    (k, v), rep = place_kv_pools(alloc, lambda a, b: 200.0, 16, span_bytes=50e9, pool_bytes=40e9)
    assert rep["slabs"] == 2                                             # always at least two pools
    made.clear()
    padded = []
    (k, v), rep = place_kv_pools(alloc, lambda a, b: 200.0, 4, span_bytes=40e9, pool_bytes=1e9,
                                 spacer=lambda n: padded.append(n))
    assert rep["slabs"] == 4 and padded == [9e9] * 3                     # small pools step by span / slabs


@pytest.mark.gpu
def test_placed_workload_runs_the_pipeline():
    from zipage_amd.compress import CompressConfig, compress_layers
    from zipage_amd.bench.workload import ragged_batch
    wl = ragged_batch(4, L=1, pool_pages=64, budget=8, W=32, seed=5, lengths=(2049, 2304),
                      place_tries=2)
    assert wl.placement["slabs"] == 2 and set(wl.placement["probe_us"]) == {"0-1"}
    assert all(t > 0 for t in wl.placement["probe_us"].values())
    assert torch.isfinite(wl.k[0, wl.tables[0][0]].float()).all()  # data written after the probe
    cfg = CompressConfig(budget_blocks=8, query_cache_len=32, enable_pooling=True, pooling_size=7)
    compress_layers(wl.k, wl.v, wl.q, wl.score_cache, wl.query_ids, wl.block_tables,
                    wl.compressed, wl.targets, cfg)
    torch.cuda.synchronize()
