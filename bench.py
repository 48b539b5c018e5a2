#!/usr/bin/env python3
"""Benchmark of the KV-compression hot path on one MI355X.

A step is one pass of the compression pipeline (score -> max-pool 7 -> window mask ->
top-2048 per kv head -> in-place compaction to 8 pages) over one batch of synthetic ragged
sequences at Qwen3-8B attention shape (32 q heads, 8 kv heads, head_dim 128, bf16, page 256,
window 32), inputs resident in HBM.  The default workload is the one the metric is quoted on,
BASELINE configs[3]: 256 ragged sequences of 9-10 pages, groups of 16 sharing two prefix pages
(copy-on-write targets), all 36 layers per step, one layer per call.  The cache is ONE allocation
(2, 4, 60000 pages, 256, 8, 128) with K and V as its halves -- the way the engine and the reference
allocate theirs -- and the 36 layers take its four layer slices in turn, so that no layer finds the
previous layer's pages in a cache.  Prints ONE JSON line.

After it, unless --no-extra-legs, the same process adds the 64-sequence single-layer workload
(BASELINE configs[1]) as `configs1_b64`, and, unless --no-e2e, BASELINE's end-to-end case
(random-init Qwen3-8B, 256 requests x 512-token prompts x 4096 greedy tokens, budget 8 pages)
through the decode engine as `end_to_end` (decode tokens/s and the compression share).

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--no-cpu-baseline] [--no-e2e]
  python bench.py --config 5 [--requests R] [--prompt P] [--out-tokens T] [--sync-compress]
"""
from __future__ import annotations

import argparse
import dataclasses
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes one compaction launch moves, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this
# program on the named workload, scaled by a plain copy kernel of known size (--calibrate-copy).
# Counters cannot be read from inside the benchmark, so these are figures of earlier profiled runs
# of the same workload (keyed by config and batch); --traffic overrides them, and a workload
# without a counter run reports null.
COMPACT_TRAFFIC = {
    (4, 256): (4_012_038_557, "profiles/pipeline_cfg4_b256.md"),
    (2, 64): (1_075_347_047, "profiles/pipeline_cfg2_b64.md"),
}


def cpu_baseline(wl, cfg, sample_seqs, layers=1, budget_s=30.0):
    """The CPU oracle (a PyTorch port of the reference algorithm) on the first
    ``sample_seqs`` sequences of the same workload, one layer, on the host cores; a workload of
    ``layers`` layers is reported as that time x ``layers``."""
    import torch
    from oracle import zipage_oracle as O
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    from zipage_amd.bench.workload import cpu_subset
    b = min(sample_seqs, wl.B)
    sub = cpu_subset(wl, range(b), layer=0)
    k, v, q = sub["k"], sub["v"], sub["q"]
    enc, tgt, comp, qid = sub["block_tables"], sub["targets"], sub["compressed"], sub["query_ids"]
    times = []
    t_all = time.perf_counter()
    for it in range(4):
        kk, vv = k.clone(), v.clone()
        t0 = time.perf_counter()
        sc = None if sub["score_cache"] is None else sub["score_cache"].clone()
        O.compress_pipeline(kk, vv, q, sc, qid, enc, comp, tgt, **dataclasses.asdict(cfg))
        dt = time.perf_counter() - t0
        if it > 0:
            times.append(dt)
        if time.perf_counter() - t_all > budget_s and times:
            break
    times.sort()
    med = times[len(times) // 2]
    unit = "sequences/s (one layer)" if layers == 1 else f"sequences/s ({layers} layers)"
    return {"value": b / (med * layers), "unit": unit, "cores": cores, "kind": "port",
            "sample": f"first {b} sequences of the same batch, 1 layer, median of {len(times)} runs "
                      f"after 1 warm-up ({med * 1e3:.0f} ms per run)"
                      + ("" if layers == 1 else f"; the figure is that time x {layers} layers")}


def end_to_end(requests=256, prompt=512, out_tokens=4096, async_compress=True, ragged=False,
               script_switches=False, attention_probe=True):
    """BASELINE configs[4]: offline decode of a random-init Qwen3-8B with the KV budget on.
    Returns decode tokens/s (decode steps only, first decode step to the last, device-complete),
    the share of that time the compression kernels were running, and the bandwidth of the
    decode-attention kernel at the steady-state shape."""
    import torch
    from zipage_amd.compress import CompressConfig
    from zipage_amd.engine import QWEN3_8B, EngineConfig, SamplingParams, ZipageEngine
    from zipage_amd.layers import paged_decode_attention

    cfg = EngineConfig(shape=QWEN3_8B, max_concurrency=requests,
                       num_kvcache_blocks=requests * 9 + 64, query_cache_len=16,
                       max_model_len=prompt + out_tokens + 1, enable_async_compress=async_compress,
                       max_compress_blocks=requests * 16,
                       compress=(CompressConfig(use_global_score=True, decay_factor=0.8, enable_pooling=True,
                                                pooling_size=5, use_redudancy=True, lightning_redudancy=True)
                                 if script_switches else CompressConfig(enable_pooling=True, pooling_size=5)))
    eng = ZipageEngine(cfg)
    g = torch.Generator().manual_seed(0)
    if ragged:
        lens = torch.randint(prompt // 2, prompt + prompt // 2 + 1, (requests,), generator=g).tolist()
    else:
        lens = [prompt] * requests
    prompts = [torch.randint(0, QWEN3_8B.vocab, (n,), generator=g).tolist() for n in lens]
    outs = eng.generate(prompts, SamplingParams(max_tokens=out_tokens, ignore_eos=True))
    st = eng.stats
    assert all(len(o["token_ids"]) == out_tokens for o in outs)
    out = {
        "workload": (f"configs[4]: random-init Qwen3-8B bf16, {requests} requests, "
                     f"{'ragged ' if ragged else ''}{prompt}-token prompts"
                     + (f" (uniform in [{prompt // 2}, {prompt + prompt // 2}])" if ragged else "")
                     + f", {out_tokens} greedy tokens "
                     "each, budget 8 pages x 256 tokens, window 16, "
                     + ("global score (decay 0.8) + lightning redundancy + max-pool 5" if script_switches
                        else "max-pool 5") + ", compression "
                     + ("on a side stream" if async_compress else "in line with the decode steps")),
        "decode_tok_per_s": round(st["decode_tokens"] / st["decode_s"], 1),
        "ms_per_decode_step": round(st["decode_s"] / st["decode_steps"] * 1e3, 3),
        "decode_steps": st["decode_steps"],
        "prefill_tok_per_s": round(st["prefill_tokens"] / st["prefill_s"], 1),
        "compress_calls": st["compress_calls"], "sequences_compressed": st["compress_seqs"],
        "compress_share_of_decode_time": round(st["compress_s"] / st["decode_s"], 5),
    }
    if not attention_probe:
        del eng
        torch.cuda.empty_cache()
        return out
    # decode attention alone, at the steady-state shape of this run (8 full pages + half a page)
    r = eng.runner
    B, BS = requests, cfg.kvcache_block_size
    ctx_len = min(8 * BS + BS // 2, prompt + out_tokens)
    tables = torch.arange(B * 9, device=r.device, dtype=torch.int32).view(B, 9)
    ctx = torch.full((B,), ctx_len, device=r.device, dtype=torch.int32)
    q = torch.randn(B, QWEN3_8B.heads, QWEN3_8B.head_dim, device=r.device).to(torch.bfloat16)
    kc, vc = r.kv_cache[0, 0], r.kv_cache[1, 0]
    for _ in range(3):
        paged_decode_attention(q, kc, vc, ctx, tables, 128 ** -0.5)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(20):
        paged_decode_attention(q, kc, vc, ctx, tables, 128 ** -0.5)
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) / 20 * 1e3
    alg = B * ctx_len * QWEN3_8B.kv_heads * QWEN3_8B.head_dim * 2 * 2   # K and V rows, read once
    out.update({
        "decode_attention": {"bound": "hbm", "kernel": "paged_decode_kernel",
                             "avg_launch_us": round(us, 1), "algorithmic_bytes": alg,
                             "achieved": round(alg / us / 1e3, 1), "peak": HBM_PEAK_GBS,
                             "unit": "GB/s", "frac": round(alg / us / 1e3 / HBM_PEAK_GBS, 4)},
    })
    del eng
    torch.cuda.empty_cache()
    return out


def run_pipeline(config, args, sw="pooling", batch=None, steps=None, warmup=None):
    """One compression workload (numbered from 1 as in BASELINE.json): build it in HBM, run
    ``warmup`` untimed and ``steps`` timed steps, then a second pass with events around every
    stage.  Returns the JSON-ready dict of the run (without the contract's fixed keys)."""
    import torch
    from zipage_amd.compress import CompressConfig, StageTimer, compress_layers
    from zipage_amd.bench.workload import algorithmic_bytes, ragged_batch

    steps = args.steps if steps is None else steps
    warmup = args.warmup if warmup is None else warmup
    if config == 2:
        batch, layers = batch or 64, 1
        wl = ragged_batch(batch, L=1, pool_pages=20000, budget=8, W=16 if sw == "scripts" else 32,
                          seed=1, lengths=(2049, 2304), name="cfg2",
                          with_score_cache=sw == "scripts", compressed=sw == "scripts",
                          place_tries=args.place_tries, one_allocation=args.place_tries <= 1)
        desc = (f"configs[1]: {batch} ragged sequences, 1 layer, Qwen3-8B attention shape (32q/8kv "
                "heads, head_dim 128), bf16, 9 pages x 256 tokens, window 32, 20k-page pool, score "
                "-> max-pool 7 -> top-2048/head -> compact to 8 pages")
    elif config == 3:
        from zipage_amd.bench.workload import QWEN3_0_6B
        batch, layers = batch or 128, 1
        wl = ragged_batch(batch, L=1, pool_pages=20000, budget=8, W=32, seed=0, lengths=(2304, 2304),
                          dtype=torch.float32, shape=QWEN3_0_6B, name="cfg3", with_score_cache=True,
                          compressed=True, place_tries=args.place_tries,
                          one_allocation=args.place_tries <= 1)
        desc = (f"configs[2]: {batch} sequences, 1 layer, Qwen3-0.6B attention shape (16q/8kv heads, "
                "head_dim 128), fp32, 9 pages x 256 tokens, window 32, 20k-page pool, score -> global "
                "score (U(0,1) carried, decay 0.9, added) -> avg-pool 7 -> minus 0.5 x "
                + ("raw all-pairs" if sw == "raw" else "lightning (same-page)")
                + " redundancy (lambda 2/3) -> top-2048/head -> compact to 8 pages")
    else:
        batch, layers = batch or 256, 36
        # ONE cache tensor (2, slices, 60000 pages, ...), K and V its two halves, as the engine and
        # the reference allocate theirs; the 36 layers of a step take its layer slices in turn, so
        # no launch finds the previous layer's pages in a cache.  Placed pools (--place-tries > 1)
        # are separate allocations and an extra report, never the headline.
        wl, pool_slices = None, args.pool_slices
        while wl is None:
            try:
                wl = ragged_batch(batch, L=pool_slices, pool_pages=60000, budget=8, W=32, seed=3,
                                  lengths=(2049, 2560), shared_prefix_group=16, shared_prefix_pages=2,
                                  name="cfg4", one_allocation=True)
            except torch.cuda.OutOfMemoryError:
                if pool_slices == 1:
                    raise
                pool_slices //= 2
                torch.cuda.empty_cache()
        desc = (f"configs[3]: {batch} ragged sequences (9-10 pages x 256 tokens), groups of 16 share "
                "2 prefix pages (copy-on-write targets), Qwen3-8B attention shape (32q/8kv heads, "
                "head_dim 128), bf16, window 32, score -> max-pool 7 -> top-2048/head -> compact to 8 "
                f"pages; one cache allocation (2, {pool_slices}, 60000 pages, 256, 8, 128) = "
                f"{2 * pool_slices * 60000 * 524288 / 1e9:.0f} GB with K and V as its halves; a step "
                f"is 36 layers, one layer per call, over the {pool_slices} layer slices in turn")
    cfg = CompressConfig(budget_blocks=8, query_cache_len=32, enable_pooling=True, pooling_size=7)
    if config == 3:
        if sw == "scripts":
            sys.exit("bench.py: --config 3 takes --pipeline-switches pooling (lightning) or raw")
        cfg = CompressConfig(budget_blocks=8, query_cache_len=32, use_global_score=True,
                             decay_factor=0.9, activate_method="sum", use_redudancy=True,
                             lightning_redudancy=sw != "raw", redudancy_lambda=2.0 / 3.0,
                             enable_pooling=True, continues_pooling=True, pooling_size=7,
                             pooling_mode="avg")
    elif sw != "pooling":
        if config != 2:
            sys.exit("bench.py: --pipeline-switches applies to --config 2 and 3")
        if sw == "scripts":
            cfg = CompressConfig(budget_blocks=8, query_cache_len=16, use_global_score=True,
                                 decay_factor=0.8, use_redudancy=True, lightning_redudancy=True,
                                 enable_pooling=True)
            desc += (" [NOT the headline switches: window 16, global score (decay 0.8), lightning "
                     "redundancy, max-pool 5, sequences already compressed once]")
        else:
            cfg = CompressConfig(budget_blocks=8, query_cache_len=32, use_redudancy=True,
                                 lightning_redudancy=False, enable_pooling=True, pooling_size=7)
            desc += " [NOT the headline switches: raw all-pairs redundancy added]"

    slices = wl.L if layers > 1 else 1
    sc = wl.score_cache
    # Redundancy scores depend on the keys: a step that found the survivors of the last page still
    # in that page would meet more duplicated keys with every step.  The one-layer workloads with
    # a redundancy stage therefore take a fresh last page per step, as a decode refills it.
    rot = None
    if layers == 1 and cfg.use_redudancy:
        from zipage_amd.bench.workload import fresh_last_pages
        rot = fresh_last_pages(wl, 64)
        desc += (" [every step finds fresh keys in each sequence's last page: 64 tables in turn]"
                 if rot is not None else
                 " [the pool has no spare pages for fresh last pages: the steps re-compress the "
                 "same pages and meet keys duplicated by earlier steps]")
    calls = [0]

    def step(timer=None):
        tables, targets = wl.block_tables, wl.targets
        if rot is not None:
            tables, targets = rot[0][calls[0] % 64], rot[1][calls[0] % 64]
            calls[0] += 1
        for i in range(layers):
            l = i % slices
            compress_layers(wl.k[l:l + 1] if layers > 1 else wl.k, wl.v[l:l + 1] if layers > 1 else wl.v,
                            wl.q[l:l + 1] if layers > 1 else wl.q,
                            sc if sc is None or layers == 1 else sc[l:l + 1], wl.query_ids,
                            tables, wl.compressed, targets, cfg, timer=timer,
                            fused_select=not args.separate_select_stages)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    # timed region: only the roofline kernel carries events (each event pair costs the stream a
    # few microseconds, 8 % of a step when every stage has one)
    kv_timer = StageTimer(True, only=("compress_kv",))
    t0 = time.perf_counter()
    for _ in range(steps):
        step(kv_timer)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    # the per-stage breakdown comes from a second, untimed pass with events around every stage
    timer = StageTimer(True)
    for _ in range(min(steps, max(1, 200 // layers))):
        step(timer)
    torch.cuda.synchronize()
    stage_steps = min(steps, max(1, 200 // layers))

    stage_s = timer.seconds()
    ms_per_step = elapsed / steps * 1e3
    seqs_per_s = wl.B / (elapsed / steps)
    alg = algorithmic_bytes(wl, cfg, layers=1)  # one layer
    kv_s = kv_timer.seconds()["compress_kv"] / (steps * layers)
    # with a carried score cache the launch also moves the survivors' scores (one call pipeline)
    kv_bytes = alg["compress_kv"] + alg.get("compress_global_score", 0)
    achieved = kv_bytes / kv_s / 1e9
    stages_ms = {k: round(v / (stage_steps * layers) * 1e3, 4) for k, v in stage_s.items()}
    gpu_ms = sum(stage_s.values()) / (stage_steps * layers) * 1e3  # per layer
    if args.traffic is not None:
        traffic, traffic_src = args.traffic, "--traffic"
    elif (config, wl.B) in COMPACT_TRAFFIC and sw == "pooling" and wl.placement is None:
        traffic, traffic_src = COMPACT_TRAFFIC[(config, wl.B)]
        traffic_src = ("rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE per compact_kernel dispatch of this "
                       "command in a counter run (counters cannot be read from inside a timed "
                       "run), scaled by the calibration copy: " + traffic_src)
    else:
        traffic, traffic_src = None, "no counter run of this workload"
    roof = {"bound": "hbm", "kernel": "compact_kernel (compress_kv)",
            "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": traffic, "traffic_source": traffic_src,
            "algorithmic_bytes": kv_bytes,
            "avg_launch_us": round(kv_s * 1e6, 2),
            "pools": ("K and V are the halves of one cache allocation, as the engine allocates"
                      if wl.placement is None else
                      "K and V are separate allocations picked by a timed probe (bench only)")}
    if slices > 1:
        # the launches of the timed steps by the layer slice they worked on: where a slice's K
        # and V lie in device memory moves this kernel by up to 15 %
        per = [[] for _ in range(slices)]
        for i, (_, st, ed) in enumerate(kv_timer.spans):
            per[(i % layers) % slices].append(st.elapsed_time(ed) * 1e3)
        roof["avg_launch_us_by_layer_slice"] = [round(sum(p) / len(p), 1) for p in per]
    out = {
        "value": round(seqs_per_s, 1),
        "unit": "sequences/s (one layer)" if layers == 1 else f"sequences/s ({layers} layers)",
        "steps": steps, "warmup": warmup, "ms_per_step": round(ms_per_step, 4),
        "dtype": "f32" if config == 3 else "bf16",
        "config": {"workload": desc, "batch": wl.B, "layers": layers},
        "roofline": roof,
        "pipeline": {"algorithmic_bytes": alg["pipeline"],
                     "gpu_ms_sum_of_stages_per_layer": round(gpu_ms, 4),
                     "wall_ms_per_layer": round(ms_per_step / layers, 4),
                     "hbm_frac_of_stage_time": round(alg["pipeline"] / (gpu_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "stages_ms": stages_ms},
    }
    if wl.placement is not None:
        # the K / V pools were chosen among pool-sized allocations by a timed compaction of this
        # batch (random keep flags); pair 0-1 is what the first two allocations give, and the
        # engine's single cache allocation does not run this search: bench-only
        out["placement"] = dict(wl.placement, scope="bench-only: the engine makes one cache allocation")
        first = wl.placement["probe_us"].get("0-1")
        if first:
            roof["first_two_allocations"] = {
                "avg_launch_us": first, "achieved": round(alg["compress_kv"] / first / 1e3, 1),
                "frac": round(alg["compress_kv"] / first / 1e3 / HBM_PEAK_GBS, 4),
                "note": "same kernel and batch with K and V in the first two pool allocations "
                        "(probe before any data is written, 8 launches)"}
        roof["placed"] = {"pools": wl.placement["kept"], "frac": roof["frac"]}
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(wl, cfg, min(args.cpu_sample, 16) if config == 3
                                           else args.cpu_sample, layers)
    del wl
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--batch", type=int, default=None)
    ap.add_argument("--config", type=int, default=4, choices=[2, 3, 4, 5],
                    help="workload, numbered from 1 as in BASELINE.json: 4 (default, the headline "
                         "line) = 256 ragged sequences with shared prefixes and copy-on-write "
                         "targets, 36 layers per step run one layer at a time over one page pool; "
                         "2 = 64 ragged sequences, one layer; 3 = 128 sequences at Qwen3-0.6B "
                         "shape in fp32 with the global-score and redundancy terms (lightning; "
                         "--pipeline-switches raw for all pairs); 5 = the end-to-end decode case "
                         "alone")
    ap.add_argument("--no-e2e", action="store_true",
                    help="skip the end-to-end decode leg that follows the default run")
    ap.add_argument("--no-extra-legs", action="store_true",
                    help="skip the 64-sequence leg and the end-to-end leg that follow the default run")
    ap.add_argument("--no-e2e-variants", action="store_true",
                    help="skip the shorter end-to-end runs that follow the end-to-end leg (ragged "
                         "prompts with side-stream and with in-line compression)")
    ap.add_argument("--all-e2e-variants", action="store_true",
                    help="also run the pair with the reference scripts' switch set (side stream and "
                         "in line; ~90 s more)")
    ap.add_argument("--variant-tokens", type=int, default=2560,
                    help="greedy tokens per request in the end-to-end variants")
    ap.add_argument("--requests", type=int, default=256)
    ap.add_argument("--prompt", type=int, default=512)
    ap.add_argument("--out-tokens", type=int, default=4096)
    ap.add_argument("--sync-compress", action="store_true",
                    help="end-to-end leg: compress in line with the decode steps instead of on "
                         "the side stream")
    ap.add_argument("--script-switches", action="store_true",
                    help="end-to-end leg: compress with the switch set of the reference's scripts "
                         "(global score, lightning redundancy, pooling) instead of pooling alone")
    ap.add_argument("--pipeline-switches", choices=["pooling", "scripts", "raw"], default="pooling",
                    help="compression switches of --config 2 / 3: pooling alone (default), the "
                         "reference scripts' set (window 16, global score, lightning redundancy, "
                         "pooling 5) or raw all-pairs redundancy with pooling 7; the non-default "
                         "sets say so in config.workload")
    ap.add_argument("--ragged-prompts", action="store_true",
                    help="end-to-end leg: prompt lengths uniform in [P/2, 3P/2] so sequences reach "
                         "their budget on different steps")
    ap.add_argument("--separate-select-stages", action="store_true",
                    help="run pooling, the mask epilogue and top-k as three launches (timed under "
                         "the reference's stage names) instead of the one-launch selection")
    ap.add_argument("--pool-slices", type=int, default=4,
                    help="layer slices of the headline workload's cache allocation "
                         "(2 x slices x 60000 pages x 512 KB; halved until it fits)")
    ap.add_argument("--place-tries", type=int, default=1,
                    help="--config 2 / 3 only, not the headline: above 1, K and V are separate "
                         "allocations chosen among that many pool-sized ones made side by side "
                         "before any data is written, by a timed compaction on pairs of them (the "
                         "in-place compaction is ~15 %% faster when the two lie in different regions "
                         "of device memory); every probe figure is reported in 'placement'.  1 "
                         "(default) = one cache allocation with K and V as its halves, as the "
                         "engine allocates")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-sample", type=int, default=64)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy (read 1 GiB, write 1 GiB) so that a "
                         "rocprofv3 --pmc run of this command has a kernel of known traffic to "
                         "scale FETCH_SIZE / WRITE_SIZE by")
    ap.add_argument("--traffic", type=float, default=None,
                    help="HBM bytes per compaction launch measured with rocprofv3 --pmc "
                         "(reported as roofline.traffic)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures the single-GPU hot path only; run with --gpus 1 "
              "(every (sequence, kv head, layer) is independent, so more GPUs shard sequences "
              "with no exchange step).", file=sys.stderr)
        sys.exit(2)

    import torch
    from zipage_amd import _lib

    _lib.load()  # fail loudly if the HIP library is missing
    torch.cuda.set_device(0)
    if args.config == 5:
        e2e = end_to_end(args.requests, args.prompt, args.out_tokens, not args.sync_compress,
                         args.ragged_prompts, args.script_switches)
        print(json.dumps({
            "metric": "decode tokens/sec", "value": e2e["decode_tok_per_s"], "unit": "tokens/s",
            "n_gpus": 1, "steps": e2e["decode_steps"], "warmup": 0,
            "ms_per_step": e2e["ms_per_decode_step"], "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": e2e["workload"]}, "roofline": e2e["decode_attention"],
            "cpu_baseline": None, "end_to_end": e2e}))
        return

    if args.calibrate_copy:
        src = torch.ones(1 << 28, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.mul(src, 1.0, out=dst)  # one streaming kernel: reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    run = run_pipeline(args.config, args, args.pipeline_switches, args.batch)
    out = {"metric": "sequences compressed/sec", "value": run.pop("value"), "unit": run.pop("unit"),
           "n_gpus": 1, "steps": run.pop("steps"), "warmup": run.pop("warmup"),
           "ms_per_step": run.pop("ms_per_step"), "higher_is_better": True, "scaling": "weak",
           "vs_baseline": None, "dtype": run.pop("dtype"), "data": "synthetic"}
    out.update(run)
    headline = args.config == 4 and args.batch is None
    if headline and not args.no_extra_legs:
        # the smaller single-layer workload of BASELINE configs[1], more steps (a step is 0.4 ms)
        out["configs1_b64"] = run_pipeline(2, args, steps=max(args.steps, 100), warmup=10)
        if not args.no_e2e:
            out["end_to_end"] = end_to_end(args.requests, args.prompt, args.out_tokens,
                                           not args.sync_compress, args.ragged_prompts,
                                           args.script_switches)
            if not args.no_e2e_variants:
                # where overlap can exist: ragged prompts, on the side stream and in line, from this
                # same process (shorter runs: every sequence still compresses 2-4 times); with
                # --all-e2e-variants also where the compression does more work (the reference
                # scripts' switch set)
                n = min(args.out_tokens, args.variant_tokens)
                pairs = ((True, False), (False, True)) if args.all_e2e_variants else ((False, True),)
                out["end_to_end"]["variants"] = [
                    end_to_end(args.requests, args.prompt, n, a, ragged, scripts, attention_probe=False)
                    for scripts, ragged in pairs for a in (True, False)]
    print(json.dumps(out))


if __name__ == "__main__":
    main()
