"""Choosing where the KV pools land in device memory.

Measured on MI355X: device memory behaves as a few large physical zones (about 70, 100 and
100+ GB in allocation order on a fresh device).  A kernel that reads and writes K and V at
once -- the in-place compaction -- runs ~15 % faster when the K pool and the V pool lie in
DIFFERENT zones (169 us against 194-197 us for 64 sequences), whatever the virtual addresses,
alignment or physical chunking; striping either pool over zones gives the same 169 us.  A
read-only kernel (decode attention) prefers K and V in the SAME zone by ~4 %.  Inside one
allocation the figure never changes, and neither the page set a batch touches nor a small
shift between the pools matters.  The driver gives no way to ask for a zone, but an engine
allocates its pools once, so it can allocate a few pool-sized slabs side by side, time a small
gather on pairs of them, keep the best pair and release the rest: ``place_kv_pools``.
``place_pools`` is the simpler form for candidates that hold both pools.
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


def place_kv_pools(alloc_one, probe_pair, slabs=16, gain=0.93, span_bytes=160e9, pool_bytes=None,
                   spacer=None):
    """``alloc_one() -> pool`` allocates ONE pool-sized tensor; ``probe_pair(k, v) ->
    microseconds``.  Allocates pools side by side (all stay alive, so they cover consecutive
    regions of device memory) and probes the first one as the K pool against each new one as
    the V pool, until a pair runs in ``gain`` x the slowest pair's time or less (the new pool
    reached another zone), ``slabs`` pools exist, their span passes ``span_bytes`` (needs
    ``pool_bytes``) or memory runs out.  Pools much smaller than ``span_bytes / slabs`` would
    never leave the first zone, so ``spacer(nbytes)`` (default: a byte tensor on the pool's
    device) pads each step to that size; spacers are released with the losing pools.  Returns
    ``((k, v), report)`` for the fastest pair."""
    pools, times, pads = [alloc_one()], {}, []
    step = pool_bytes
    if pool_bytes is not None and pool_bytes * max(2, slabs) < span_bytes:
        step = span_bytes / max(2, slabs)
        if spacer is None and isinstance(pools[0], torch.Tensor):
            dev = pools[0].device
            spacer = lambda n: torch.empty(int(n), dtype=torch.uint8, device=dev)
        if spacer is None:
            step = pool_bytes
    while len(pools) < max(2, slabs):
        if step is not None and len(pools) >= 2 and (len(pools) + 1) * step > span_bytes:
            break
        try:
            if step is not None and step > pool_bytes:
                pads.append(spacer(step - pool_bytes))
            pools.append(alloc_one())
        except torch.cuda.OutOfMemoryError:
            break
        j = len(pools) - 1
        times[(0, j)] = round(probe_pair(pools[0], pools[j]), 1)
        if min(times.values()) <= gain * max(times.values()):
            break
    if len(pools) < 2:
        raise RuntimeError("place_kv_pools: fewer than two pools fit in device memory")
    (ki, vi) = min(times, key=times.get)
    k, v = pools[ki], pools[vi]
    n = len(pools)
    del pools, pads
    if torch.cuda.is_available():
        torch.cuda.empty_cache()
    return (k, v), {"slabs": n, "probe_us": {f"{i}-{j}": t for (i, j), t in times.items()},
                    "kept": [ki, vi]}
