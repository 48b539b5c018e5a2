"""Per-phase cycle counts of the 16-bit redundancy kernels (`gram_page_kernel`, `raw_chain_kernel`).

Needs a library built with the measurement macro, which makes thread 0 of every workgroup record
the core-clock counter at the phase boundaries (and the constant-rate 100 MHz counter at both ends)
into a device array that `zp_debug_page_stamps` / `zp_debug_chain_stamps` copy out:

    ZP_EXTRA_HIPCC_FLAGS=-DZP_PAGE_STAMP python -m zipage_amd.build
    python -m zipage_amd.bench.redundancy_stamps [--batch 64] [--raw]
    python -m zipage_amd.build            # back to the product build

The keys are random, so no key has a claim; the times printed first are the whole stage (Gram
kernel(s) + softmax) by HIP events.
"""
from __future__ import annotations

import argparse
import ctypes

import numpy as np
import torch

PAGE_PHASES = ["row set-up (first page only), claim slots cleared",
               "own rows landed, diagonal tile, norms",
               "barrier: all rows and norms",
               "summed key (thread 0's wave has none: waves 4-7)",
               "Gram tiles of wave 0",
               "barrier behind the tiles",
               "next page requested, summed-key tile, claim values",
               "barrier",
               "store"]
CHAIN_PHASES = ["table lookup, page list, key loads",
                "claims of the round gathered",
                "first planes",
                "corrections cleared (all tiles)",
                "corrections added",
                "products and epilogue",
                "next planes stored, serial chain",
                "barrier behind the chain"]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--raw", action="store_true", help="the all-pairs variant (raw_chain_kernel)")
    args = ap.parse_args()
    from zipage_amd import _lib
    from zipage_amd.bench.workload import ragged_batch
    from zipage_amd.kernel import lightning_redudancy_score, raw_redudancy_score

    B = args.batch
    wl = ragged_batch(B, L=1, pool_pages=20000, seed=3, lengths=(2049, 2560) if B > 64 else (2049, 2304))
    k, enc = wl.k, wl.block_tables
    lib = _lib.load()
    name = "zp_debug_chain_stamps" if args.raw else "zp_debug_page_stamps"
    if not hasattr(lib, name):
        raise SystemExit("this library has no phase stamps: build it with ZP_EXTRA_HIPCC_FLAGS=-DZP_PAGE_STAMP")
    fn = raw_redudancy_score if args.raw else lightning_redudancy_score

    def run():
        return fn(k, enc, 0.5, 1.0)

    for _ in range(3):
        run()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(10):
        run()
    e1.record()
    torch.cuda.synchronize()
    print(f"{'raw' if args.raw else 'lightning'} redundancy, {B} sequences: {e0.elapsed_time(e1) * 100:.1f} us per call")
    L, _, _, Hkv, _ = k.shape
    n = L * B * Hkv * enc.shape[1]
    buf = np.zeros((n, 12), dtype=np.int64)
    rc = getattr(lib, name)(ctypes.c_void_p(buf.ctypes.data), n)
    assert rc == 0, rc
    st = buf[buf[:, 11] > 0].astype(np.float64)
    if args.raw:     # accumulated cycles per phase
        d, names = st[:, :8], CHAIN_PHASES
    else:            # stamps at the phase boundaries of one page
        d, names = st[:, 1:10] - st[:, 0:9], PAGE_PHASES
    tot = d.sum(1)
    print(f"{len(st)} pages")
    for i, nm in enumerate(names):
        print(f"  {nm:52s} mean {d[:, i].mean():8.0f} cycles  min {d[:, i].min():7.0f}  max {d[:, i].max():8.0f}  "
              f"share {d[:, i].sum() / tot.sum():.3f}")
    wall_us = st[:, 11] / 100
    print(f"  total {tot.mean():.0f} cycles per page; {wall_us.mean():.2f} us -> core clock "
          f"{tot.sum() / (wall_us.sum() * 1e-6) / 1e9:.2f} GHz")


if __name__ == "__main__":
    main()
