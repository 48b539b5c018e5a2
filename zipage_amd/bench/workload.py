"""Synthetic compression workloads at the benchmark shapes, built directly on the device.

Host bookkeeping follows the reference engine: page tables are encoded as in
zipage/engine/model_runner.py:437-463, target tables follow ``BlockManager.may_compress``
(zipage/engine/block_manager.py:129-169): an already-compressed sequence compacts in place
into its own first ``budget+1`` pages; a first compression behind a shared prefix of ``p``
pages writes into ``min(p, budget)`` fresh pages followed by its own pages.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

QWEN3_8B = dict(Hq=32, Hkv=8, D=128)
QWEN3_0_6B = dict(Hq=16, Hkv=8, D=128)


@dataclass
class Workload:
    name: str
    k: torch.Tensor            # (L, pages, BS, Hkv, D)
    v: torch.Tensor
    q: torch.Tensor            # (L, B, W, Hq, D)
    score_cache: torch.Tensor | None
    query_ids: torch.Tensor    # (B,) int32
    block_tables: torch.Tensor  # (B, NB) int32, encoded
    compressed: torch.Tensor   # (B,) bool
    targets: torch.Tensor      # (B, budget+1) int32
    budget: int
    W: int
    tables: list
    placement: dict | None = None  # report of placement.place_pools, when it chose the pools

    @property
    def B(self):
        return self.block_tables.shape[0]

    @property
    def L(self):
        return self.k.shape[0]


def encode_tables(tables, device):
    width = max(len(t) for t in tables)
    rows = [list(t[:-1]) + [-t[-1] - 2] + [-1] * (width - len(t)) for t in tables]
    return torch.tensor(rows, dtype=torch.int32, device=device)


def ragged_batch(B, *, L=1, pool_pages=20000, budget=8, W=32, BS=256, dtype=torch.bfloat16,
                 seed=1, lengths=(2049, 2304), shared_prefix_group=0, shared_prefix_pages=2,
                 with_score_cache=False, compressed=False, shape=QWEN3_8B, device="cuda:0",
                 name="ragged", place_tries=1, one_allocation=False):
    """B sequences with token counts uniform in ``lengths`` (rounded up to whole pages, since
    compression fires only on a full last page), pages drawn without replacement from a pool
    of ``pool_pages`` ids.  With ``shared_prefix_group = n`` every group of n sequences shares
    its first ``shared_prefix_pages`` pages (copy-on-write targets).  With ``place_tries > 1``
    the K and V pools are chosen by ``placement.place_kv_pools`` among that many pool-sized
    allocations made side by side (a timed gather on pairs of them, before any data is
    written); the report is kept in ``placement``.  With ``one_allocation`` K and V are the two
    halves of ONE ``(2, L, pool_pages, BS, Hkv, D)`` tensor, which is how the engine and the
    reference allocate their cache (zipage/engine/model_runner.py:219-307)."""
    g = torch.Generator().manual_seed(seed)
    Hq, Hkv, D = shape["Hq"], shape["Hkv"], shape["D"]
    lens = torch.randint(lengths[0], lengths[1] + 1, (B,), generator=g)
    nbs = ((lens + BS - 1) // BS).tolist()
    perm = torch.randperm(pool_pages, generator=g).tolist()
    pos = 0

    def take(n):
        nonlocal pos
        out = perm[pos:pos + n]
        pos += n
        assert len(out) == n, "page pool exhausted"
        return out

    tables, targets = [], []
    shared = None
    for b in range(B):
        if shared_prefix_group and b % shared_prefix_group == 0:
            shared = take(shared_prefix_pages)
        if shared_prefix_group:
            own = take(nbs[b] - shared_prefix_pages)
            table = shared + own
            n_new = min(shared_prefix_pages, budget)
            fresh = take(n_new)
            target = fresh + table[shared_prefix_pages:shared_prefix_pages + budget + 1 - n_new]
        else:
            table = take(nbs[b])
            target = table[:budget + 1]
        tables.append(table)
        targets.append(target)
    used = sorted({p for t in tables for p in t})
    dev = torch.device(device)
    block_tables = encode_tables(tables, dev)
    compressed_t = torch.full((B,), bool(compressed), dtype=torch.bool, device=dev)
    targets_t = torch.tensor(targets, dtype=torch.int32, device=dev)

    def alloc_one():
        return torch.empty((L, pool_pages, BS, Hkv, D), dtype=dtype, device=dev)

    placement = None
    if one_allocation:
        kv = torch.empty((2, L, pool_pages, BS, Hkv, D), dtype=dtype, device=dev)
        k, v = kv[0], kv[1]
    elif place_tries > 1:
        from zipage_amd.bench.placement import place_kv_pools, probe_gather_us
        (k, v), placement = place_kv_pools(
            alloc_one, lambda kp, vp: probe_gather_us(kp, vp, block_tables, compressed_t, targets_t,
                                                      budget * BS), place_tries,
            pool_bytes=L * pool_pages * BS * Hkv * D * torch.empty((), dtype=dtype).element_size())
    else:
        k, v = alloc_one(), alloc_one()
    gg = torch.Generator(device=dev).manual_seed(seed)
    idx = torch.tensor(used, device=dev)
    for l in range(L):
        k[l, idx] = torch.randn((len(used), BS, Hkv, D), generator=gg, device=dev,
                                dtype=torch.float32).to(dtype)
        v[l, idx] = torch.randn((len(used), BS, Hkv, D), generator=gg, device=dev,
                                dtype=torch.float32).to(dtype)
    q = torch.randn((L, B, W, Hq, D), generator=gg, device=dev, dtype=torch.float32).to(dtype)
    sc = None
    if with_score_cache:
        sc = torch.empty((L, pool_pages, BS, Hkv), dtype=dtype, device=dev)
        for l in range(L):
            sc[l, idx] = torch.rand((len(used), BS, Hkv), generator=gg, device=dev).to(dtype)
    return Workload(
        name=name, k=k, v=v, q=q, score_cache=sc,
        query_ids=torch.arange(B, dtype=torch.int32, device=dev),
        block_tables=block_tables, compressed=compressed_t, targets=targets_t,
        budget=budget, W=W, tables=tables, placement=placement)


def fresh_last_pages(wl: Workload, n: int, seed: int = 7):
    """``n`` block tables (and target tables) for ``wl`` that differ in every sequence's LAST page:
    table 0 is the workload's own, the others name pool pages nobody uses, filled with fresh
    random keys, values and cached scores.  A benchmark that compresses the same sequences step
    after step takes them in turn, as a decode would have refilled the last page between two
    compressions; with one table the survivors copied out of the last page would also still sit in
    it, and the redundancy kernels would meet more and more duplicated keys.
    Returns ``(tables (n, B, NB) int32, targets (n, B, budget+1) int32)`` on the device, or ``None``
    when the pool has fewer than ``(n - 1) * B`` spare pages."""
    L, pool_pages = wl.k.shape[0], wl.k.shape[1]
    dev = wl.k.device
    used = {p for t in wl.tables for p in t} | set(wl.targets.flatten().tolist())
    spare = [p for p in range(pool_pages) if p not in used]
    B = wl.B
    if n < 2 or len(spare) < (n - 1) * B:
        return None
    g = torch.Generator().manual_seed(seed)
    order = torch.randperm(len(spare), generator=g)[:(n - 1) * B].tolist()
    alt = [spare[i] for i in order]
    idx = torch.tensor(alt, device=dev)
    gg = torch.Generator(device=dev).manual_seed(seed)
    for l in range(L):
        for pool in (wl.k, wl.v):
            pool[l, idx] = torch.randn((len(alt),) + tuple(pool.shape[2:]), generator=gg, device=dev,
                                       dtype=torch.float32).to(pool.dtype)
        if wl.score_cache is not None:
            wl.score_cache[l, idx] = torch.rand((len(alt),) + tuple(wl.score_cache.shape[2:]),
                                                generator=gg, device=dev).to(wl.score_cache.dtype)
    targets0 = wl.targets.tolist()
    tabs, tgts = [wl.block_tables], [wl.targets]
    for i in range(n - 1):
        tables, targets = [], []
        for b in range(B):
            last, new = wl.tables[b][-1], alt[i * B + b]
            tables.append(list(wl.tables[b][:-1]) + [new])
            targets.append([new if p == last else p for p in targets0[b]])
        tabs.append(encode_tables(tables, dev))
        tgts.append(torch.tensor(targets, dtype=torch.int32, device=dev))
    return torch.stack(tabs), torch.stack(tgts)


def algorithmic_bytes(wl: Workload, cfg, layers=None) -> dict:
    """HBM bytes each stage has to move for this workload (per launch over ``layers`` layers, all
    of the workload's by default):
    K once + Q + score out for the scorer; score-cache read+write for the global score;
    K and V survivors read+written for the compaction."""
    L, _, BS, Hkv, D = wl.k.shape
    L = L if layers is None else layers
    Hq = wl.q.shape[3]
    es = wl.k.element_size()
    valid_pages = sum(len(t) for t in wl.tables)
    keep = cfg.budget_blocks * BS
    B = wl.B
    out = {
        "attention_score": L * (valid_pages * BS * Hkv * D * es + B * wl.W * Hq * D * es
                                + valid_pages * BS * Hkv * es),
        "compress_kv": L * B * 2 * 2 * keep * Hkv * D * es,
    }
    if cfg.use_global_score:
        out["global_score"] = L * 2 * valid_pages * BS * Hkv * es
        out["compress_global_score"] = L * B * 2 * keep * Hkv * es
    if cfg.use_redudancy:
        out["redudancy_score"] = L * valid_pages * BS * Hkv * D * es
    out["pipeline"] = sum(out.values())
    return out


def cpu_subset(wl: Workload, seq_ids, layer=None):
    """Host copy of the sequences ``seq_ids`` (all layers, or the one given) with their pages
    renumbered densely, for checking or timing against a CPU implementation.  Returns a dict of
    CPU tensors with the same meaning as the Workload fields (block tables already encoded)."""
    seq_ids = list(seq_ids)
    lsel = slice(None) if layer is None else slice(layer, layer + 1)   # a view, never a pool copy
    tables = [wl.tables[b] for b in seq_ids]
    targets = wl.targets[seq_ids].tolist()
    used = sorted({p for t in tables for p in t} | {int(p) for row in targets for p in row})
    remap = {p: i for i, p in enumerate(used)}
    idx = torch.tensor(used, device=wl.k.device)
    width = wl.block_tables.shape[1]
    rows = [[remap[p] for p in t] for t in tables]
    enc = torch.tensor([r[:-1] + [-r[-1] - 2] + [-1] * (width - len(r)) for r in rows],
                       dtype=torch.int32)
    return dict(
        k=wl.k[lsel][:, idx].cpu(), v=wl.v[lsel][:, idx].cpu(), q=wl.q[lsel][:, seq_ids].cpu(),
        score_cache=None if wl.score_cache is None else wl.score_cache[lsel][:, idx].cpu(),
        query_ids=torch.arange(len(seq_ids), dtype=torch.int32), block_tables=enc,
        compressed=wl.compressed[seq_ids].cpu(),
        targets=torch.tensor([[remap[int(p)] for p in row] for row in targets], dtype=torch.int32),
        pages=used)
