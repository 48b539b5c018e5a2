"""Per-phase cycle counts of the register-resident scorer (`score_resident_kernel`).

Needs a library built with the measurement macro, which makes wave 0 of every workgroup record
the core-clock counter at the phase boundaries and the constant-rate (100 MHz) counter at both
ends, behind the window partials in the workspace:

    ZP_EXTRA_HIPCC_FLAGS=-DZP_RES_STAMP python -m zipage_amd.build
    python -m zipage_amd.bench.scorer_stamps [--batch 256] [--hot]
    python -m zipage_amd.build            # back to the product build

`--hot` points every sequence at the first sequence's pages, so that all key blocks are L2 hits.
A build with `-DZP_RES_STAMP -DZP_RES_HALFDMA` fetches only half of every key block (wrong results,
half the bytes through the load path).  The core clock is cycles / wall time per workgroup.
"""
from __future__ import annotations

import argparse
import json

import torch


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--batch", type=int, default=256)
    ap.add_argument("--hot", action="store_true")
    args = ap.parse_args()
    from zipage_amd import _lib
    from zipage_amd.bench.workload import ragged_batch

    B = args.batch
    wl = ragged_batch(B, L=1, pool_pages=20000, seed=3, lengths=(2049, 2560) if B > 64 else (2049, 2304))
    k, q, qid, enc = wl.k, wl.q, wl.query_ids, wl.block_tables
    tables = wl.tables
    if args.hot:
        enc = enc.clone()
        enc[:] = enc[0]
        tables = [tables[0]] * B
    L, P, BS, Hkv, D = k.shape
    _, S, W, Hq, _ = q.shape
    NB = enc.shape[1]
    lib = _lib.load()
    need = lib.zp_attention_score_workspace_for(L, B, NB, BS, Hkv, Hq, W, _lib.dtype_tag(k))
    RB = (W * (Hq // Hkv) + 31) // 32
    units = L * B * Hkv * RB
    ws = torch.zeros(need + units * 64, dtype=torch.uint8, device=k.device)
    out = torch.empty((L, B, Hkv, NB, BS), dtype=k.dtype, device=k.device)

    def run():
        _lib.call("zp_attention_score", k.data_ptr(), q.data_ptr(), qid.data_ptr(), enc.data_ptr(),
                  out.data_ptr(), 0, L, B, NB, BS, Hkv, Hq, D, W, P, S, k.stride(0), k.stride(1),
                  q.stride(0), q.stride(1), float(D ** -0.5), 0, 0, ws.data_ptr(), need + units * 64,
                  torch.cuda.current_stream().cuda_stream)

    for _ in range(3):
        run()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    run()
    e1.record()
    torch.cuda.synchronize()
    st = ws[need:].view(torch.int64).view(units, 8).cpu().double()
    if not st.any():
        raise SystemExit("no stamps: build the library with ZP_EXTRA_HIPCC_FLAGS=-DZP_RES_STAMP")
    d = st[:, 1:7] - st[:, 0:6]
    names = ["prologue + query rows", "sweep", "row-maximum exchange", "x and exp sums",
             "row-sum exchange", "output"]
    tot = st[:, 6] - st[:, 0]
    tiles = torch.tensor([len(t) for t in tables]).repeat_interleave(Hkv * RB).double() * (BS // 128)
    rep = {
        "kernels_us": round(e0.elapsed_time(e1) * 1e3, 1), "workgroups": units,
        "phases_cycles_mean_min_max_share": {
            n: [round(d[:, i].mean().item()), int(d[:, i].min()), int(d[:, i].max()),
                round((d[:, i].sum() / tot.sum()).item(), 3)] for i, n in enumerate(names)},
        "workgroup_cycles_mean": round(tot.mean().item()),
        "workgroup_wall_us_mean": round(st[:, 7].mean().item() / 100, 2),
        "core_clock_GHz": round((tot.sum() / (st[:, 7].sum() / 100e6) / 1e9).item(), 3),
        "cycles_per_128_token_tile": {"sweep": round((d[:, 1] / tiles).mean().item()),
                                      "x and exp sums": round((d[:, 3] / tiles).mean().item()),
                                      "output": round((d[:, 5] / tiles).mean().item())},
    }
    print(json.dumps(rep))


if __name__ == "__main__":
    main()
