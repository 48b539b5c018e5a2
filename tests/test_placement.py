"""Pool placement: the choice logic on the CPU, the timed gather on the GPU."""
import pytest
import torch

from zipage_amd.placement import place_pools


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


@pytest.mark.gpu
def test_placed_workload_runs_the_pipeline():
    from zipage_amd.compress import CompressConfig, compress_layers
    from zipage_amd.workload import ragged_batch
    wl = ragged_batch(4, L=1, pool_pages=64, budget=8, W=32, seed=5, lengths=(2049, 2304),
                      place_tries=2)
    assert wl.placement["tries"] == 2 and len(wl.placement["probe_us"]) == 2
    assert all(t > 0 for t in wl.placement["probe_us"])
    assert torch.isfinite(wl.k[0, wl.tables[0][0]].float()).all()  # data written after the probe
    cfg = CompressConfig(budget_blocks=8, query_cache_len=32, enable_pooling=True, pooling_size=7)
    compress_layers(wl.k, wl.v, wl.q, wl.score_cache, wl.query_ids, wl.block_tables,
                    wl.compressed, wl.targets, cfg)
    torch.cuda.synchronize()
