"""Choosing where the KV pools land in device memory.

The in-place compaction (and every other gather through the page table) runs 10-15 % faster or
slower depending on which physical region the driver gave the pool allocation; inside one
allocation the figure never changes, and neither the page set a batch touches nor the distance
between the K and V pools matters.  An engine allocates its pools once, so it can afford to
time a small gather on a fresh allocation and try another region when the first one is slow.
``place_pools`` does that while holding at most two candidates at a time.
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


def place_pools(alloc, probe, tries=4, good_enough=None):
    """``alloc() -> pools`` (any object holding the tensors), ``probe(pools) -> microseconds``.
    Allocates up to ``tries`` candidates one after the other, keeping the fastest so far alive
    while the next one is allocated (so the next one lands elsewhere), and returns
    ``(pools, report)``; ``report`` lists every probe figure and the index that was kept.
    Stops early when a candidate is within 3 % of ``good_enough`` microseconds, or when a
    second candidate does not fit in memory."""
    best, best_us, times, kept = None, None, [], 0
    for i in range(max(1, tries)):
        try:
            cand = alloc()
        except torch.cuda.OutOfMemoryError:
            break
        us = probe(cand)
        times.append(round(us, 1))
        if best is None or us < best_us:
            best, best_us, kept = cand, us, i   # the previous best is released here
        del cand
        torch.cuda.empty_cache()
        if good_enough is not None and best_us <= good_enough * 1.03:
            break
    return best, {"tries": len(times), "probe_us": times, "kept": kept}
