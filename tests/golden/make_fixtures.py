#!/usr/bin/env python3
"""Writes tests/golden/compress_cases.json: known-answer vectors of the compression pipeline.

The vectors come from THIS repository's CPU oracle (oracle/zipage_oracle.py) on seeded inputs.
They are not outputs of the reference implementation: its kernels could not be executed in the
build environment, and its own tests hold no stored vectors.  What the file pins is therefore
(1) that the oracle does not drift (CPU test), and (2) that the HIP path reproduces the same
vectors on a GPU box where only this file, not the oracle's history, is the authority.

Inputs are regenerated from the seed by tests/cases.py and verified against the stored SHA-256, so
the file stays a few KB; outputs are stored in full (scores as raw 16/32-bit words, keep flags as
packed bits) together with the SHA-256 of the compacted K/V target pages.

  python tests/golden/make_fixtures.py        # rewrite the file
"""
from __future__ import annotations

import base64
import hashlib
import json
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from cases import make_caches, random_tables, touched_pages  # noqa: E402
from oracle import zipage_oracle as O  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "compress_cases.json")
DTYPES = {"bfloat16": torch.bfloat16, "float16": torch.float16, "float32": torch.float32}

CASES = [
    dict(name="bf16_pool", seed=101, dtype="bfloat16", L=1, B=3, Hkv=2, G=4, D=64, BS=256, W=16,
         pages=12, nb=[2, 3], budget=1, kw=dict(enable_pooling=True, pooling_size=7)),
    dict(name="fp16_max_sink", seed=202, dtype="float16", L=2, B=2, Hkv=2, G=2, D=32, BS=256, W=8,
         pages=8, nb=[3], budget=2, kw=dict(reduced="max", use_attention_sink=True, sink_len=4)),
    dict(name="fp32_global_lightning", seed=303, dtype="float32", L=1, B=2, Hkv=2, G=2, D=32, BS=128,
         W=8, pages=10, nb=[3, 4], budget=2, score_cache=True,
         kw=dict(use_global_score=True, decay_factor=0.9, use_redudancy=True, lightning_redudancy=True,
                 redudancy_lambda=0.5, enable_pooling=True, pooling_size=5, continues_pooling=True)),
]


def raw_bytes(t: torch.Tensor) -> bytes:
    t = t.contiguous()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().tobytes()
    if t.dtype == torch.bool:
        return np.packbits(t.numpy().astype(np.uint8).ravel()).tobytes()
    return t.numpy().tobytes()


def sha(*tensors) -> str:
    h = hashlib.sha256()
    for t in tensors:
        if t is not None:
            h.update(raw_bytes(t))
    return h.hexdigest()


def build_inputs(c):
    dtype = DTYPES[c["dtype"]]
    tables, enc, target = random_tables(c["seed"], c["B"], c["pages"], c["nb"], c["budget"])
    k, v, q, sc = make_caches(c["seed"] + 1, c["L"], c["pages"], c["BS"], c["Hkv"], c["Hkv"] * c["G"],
                              c["D"], c["W"], c["B"], dtype, touched=touched_pages(enc),
                              with_score_cache=c.get("score_cache", False))
    query_ids = torch.arange(c["B"], dtype=torch.int32).flip(0).contiguous()
    compressed = torch.tensor([i % 2 == 1 for i in range(c["B"])])
    return dict(k=k, v=v, q=q, sc=sc, query_ids=query_ids, enc=enc, target=target, compressed=compressed)


def run_oracle(c, inp):
    k, v = inp["k"].clone(), inp["v"].clone()
    sc = None if inp["sc"] is None else inp["sc"].clone()
    flag, scores = O.compress_pipeline(k, v, inp["q"], sc, inp["query_ids"], inp["enc"],
                                       inp["compressed"], inp["target"], budget_blocks=c["budget"],
                                       query_cache_len=c["W"], return_intermediates=True, **c["kw"])
    tgt = inp["target"][:, :c["budget"]].flatten().long()
    return dict(flag=flag, scores=scores, k_after=k[:, tgt], v_after=v[:, tgt],
                sc_after=None if sc is None else sc[:, tgt])


def main():
    out = []
    for c in CASES:
        inp = build_inputs(c)
        res = run_oracle(c, inp)
        out.append(dict(
            case=c,
            inputs_sha256=sha(inp["k"], inp["v"], inp["q"], inp["sc"], inp["enc"], inp["target"]),
            scores_shape=list(res["scores"].shape),
            scores_b64=base64.b64encode(raw_bytes(res["scores"])).decode(),
            flag_shape=list(res["flag"].shape),
            flag_bits_b64=base64.b64encode(raw_bytes(res["flag"])).decode(),
            kept_per_row=int(res["flag"].flatten(3).sum(-1).unique().item()),
            compacted_sha256=sha(res["k_after"], res["v_after"], res["sc_after"]),
        ))
    with open(OUT, "w") as f:
        json.dump(out, f, indent=1)
    print(f"wrote {OUT} ({os.path.getsize(OUT)} bytes)")


if __name__ == "__main__":
    main()
