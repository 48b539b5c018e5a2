"""Choosing where the KV pools land in device memory.

The in-place compaction (and every other gather through the page table) runs 10-15 % faster or
slower depending on which physical region the driver gave the pool allocation; inside one
allocation the figure never changes, and neither the page set a batch touches nor the distance
between the K and V pools matters.  An engine allocates its pools once, so it can afford to
time a small gather on a fresh allocation and try another region when the first one is slow.
``place_pools`` does that; the candidates stay allocated until the choice is made, because a
candidate allocated after another was released would land in the released region again (on a
fresh device, 20 GB allocations made one after the other and all kept alive gave 202, 202, 203,
180, 170, 196, 194, 197, 173 and 199 microseconds for the same gather, the same in every
process).
"""
from __future__ import annotations

import torch


def probe_gather_us(k, v, block_tables, compressed, targets, keep, reps=8):
    """Microseconds per in-place compaction of a random selection of ``keep`` tokens per head
    through ``block_tables`` into ``targets``.  Overwrites pool contents (call it before the
    pools hold data)."""
    from zipage_amd.kernel import compress_kv, select_topk
    L, _, BS, Hkv, _ = k.shape
    B, NB = block_tables.shape
    scores = torch.rand((L, B, Hkv, NB, BS), device=k.device, dtype=torch.float32).to(k.dtype)
    flag = select_topk(scores, block_tables, compressed, keep)
    for _ in range(2):
        compress_kv(k, v, flag, block_tables, targets)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        compress_kv(k, v, flag, block_tables, targets)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps * 1e3


def place_pools(alloc, probe, tries=6, good_enough=None):
    """``alloc() -> pools`` (any object holding the tensors), ``probe(pools) -> microseconds``.
    Allocates up to ``tries`` candidates and keeps every one alive until the last has been
    probed, so that each lands in a different region of device memory (a candidate allocated
    after another was released would take over the released region); returns
    ``(pools, report)`` for the fastest; ``report`` lists every probe figure and the index that
    was kept.  Stops early when a candidate is within 3 % of ``good_enough`` microseconds, or
    when the next candidate does not fit in memory.  The losers are released before returning."""
    cands, times = [], []
    for _ in range(max(1, tries)):
        try:
            cands.append(alloc())
        except torch.cuda.OutOfMemoryError:
            break
        times.append(round(probe(cands[-1]), 1))
        if good_enough is not None and times[-1] <= good_enough * 1.03:
            break
    kept = min(range(len(times)), key=times.__getitem__)
    best = cands[kept]
    del cands
    if torch.cuda.is_available():
        torch.cuda.empty_cache()
    return best, {"tries": len(times), "probe_us": times, "kept": kept}
