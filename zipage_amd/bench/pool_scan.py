"""Where in device memory do the K and V pools of a layer lie, and what does that do to the
in-place compaction?

    python -m zipage_amd.bench.pool_scan [--layers 36] [--pages 6600] [--batch 256]

Allocates ONE cache tensor (2, layers, pages, 256, 8, 128) in bf16 -- the engine's allocation --
and times `compress_kv` of one ragged batch (random keep flags, 2048 survivors per head) on
(K slot, V slot) pairs of its 2 x layers pool-sized slots: every layer's own pair, and one slot
against every other.  On MI355X the time has two levels ~15 % apart; which one a pair gets depends
on where its two slots lie (the classes repeat in 32 GiB steps of the allocation), not on the
kernel's access pattern, and a plain device copy between the same slots does not show it.
"""
from __future__ import annotations

import argparse
import json

import torch


def _time_us(fn, reps=6):
    for _ in range(2):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps * 1e3


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--layers", type=int, default=36)
    ap.add_argument("--pages", type=int, default=6600)
    ap.add_argument("--batch", type=int, default=256)
    args = ap.parse_args()
    from zipage_amd.bench.workload import encode_tables
    from zipage_amd.kernel import compress_kv, topk_mask

    L, P, B = args.layers, args.pages, args.batch
    dev = torch.device("cuda:0")
    kv = torch.empty((2, L, P, 256, 8, 128), dtype=torch.bfloat16, device=dev)
    slots = kv.view(2 * L, 1, P, 256, 8, 128)      # slot l is K of layer l, slot L + l its V
    g = torch.Generator().manual_seed(3)
    perm = torch.randperm(P, generator=g).tolist()
    nbs = torch.randint(9, 11, (B,), generator=g).tolist()
    tables, pos = [], 0
    for n in nbs:
        tables.append(perm[pos:pos + n])
        pos += n
    enc = encode_tables(tables, dev)
    tgt = torch.tensor([t[:9] for t in tables], dtype=torch.int32, device=dev)
    NB = enc.shape[1]
    sc = torch.rand((1, B, 8, NB, 256), device=dev)
    sc[(enc == -1)[None, :, None, :, None].expand_as(sc)] = -1e30
    flag = topk_mask(sc.view(1, B, 8, NB * 256), 2048).view(1, B, 8, NB, 256)
    alg = B * 2 * 2 * 2048 * 8 * 128 * 2
    slot_gb = P * 524288 / 1e9

    def pair(i, j):
        return round(_time_us(lambda: compress_kv(slots[i], slots[j], flag, enc, tgt)), 1)

    own = [pair(l, L + l) for l in range(L)]
    fast = min(own)
    out = {
        "allocation_GB": round(2 * L * slot_gb, 1), "slot_GB": round(slot_gb, 2),
        "algorithmic_bytes": alg,
        "own_pairs_us": own,
        "own_pairs_frac_of_8TBs": [round(alg / t / 1e3 / 8000, 3) for t in own],
        "mean_frac": round(alg / (sum(own) / L) / 1e3 / 8000, 4),
        "slow_layers": [l for l in range(L) if own[l] > 1.08 * fast],
        "slot0_against_odd_slots_us": [pair(0, j) for j in range(1, 2 * L, 2)],
        "last_K_slot_against_even_slots_us": [pair(L - 1, j) for j in range(0, 2 * L, 2) if j != L - 1],
    }
    n = slots[0].numel()
    out["plain_copy_TBs"] = {f"{i}->{j}": round(2 * n * 2 / _time_us(lambda: slots[j].copy_(slots[i]), 3) / 1e6, 2)
                             for i, j in ((0, 1), (0, L // 2), (0, L), (0, 2 * L - 1), (L - 1, L))}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
