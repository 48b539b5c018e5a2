"""Seeded synthetic inputs shared by the oracle and the GPU parity tests.

Block tables follow the page-table encoding of zipage/engine/model_runner.py:437-463.
The small tables are the shapes used by the reference's own print-scripts
(tests/test_attention_score.py:342-344, tests/test_global_score.py:76-80,
tests/test_lightning_redudancy.py:111-115).
"""
from __future__ import annotations

import torch

REF_TABLES = {
    "attention": [[0, 1, 2, -5], [5, 6, -9, -1]],
    "global": [[0, 1, -4], [8, -9, -1]],
    "lightning": [[0, 1, 2, -9], [8, 9, -16, -1]],
}


def make_caches(seed, L, num_pages, BS, Hkv, Hq, D, W, max_seqs, dtype, touched=None,
                with_v=True, with_score_cache=False):
    """K/V ~ N(0,1) (only the touched pages get data, the rest stay zero), Q ~ N(0,1)."""
    g = torch.Generator().manual_seed(seed)
    k = torch.zeros((L, num_pages, BS, Hkv, D), dtype=dtype)
    v = torch.zeros((L, num_pages, BS, Hkv, D), dtype=dtype) if with_v else None
    pages = list(range(num_pages)) if touched is None else sorted(set(touched))
    for p in pages:
        k[:, p] = torch.randn((L, BS, Hkv, D), generator=g).to(dtype)
        if with_v:
            v[:, p] = torch.randn((L, BS, Hkv, D), generator=g).to(dtype)
    q = torch.randn((L, max_seqs, W, Hq, D), generator=g).to(dtype)
    sc = None
    if with_score_cache:
        sc = torch.rand((L, num_pages, BS, Hkv), generator=g).to(dtype)
    return k, v, q, sc


def random_tables(seed, B, num_pages, nb_choices, budget):
    """Per-sequence page lists drawn without replacement, ragged in page count; returns
    (python tables, encoded (B,NB) int32 tensor, compressed-style target (B,budget+1))."""
    from oracle.zipage_oracle import encode_block_table
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(num_pages, generator=g).tolist()
    tables, pos = [], 0
    for b in range(B):
        nb = nb_choices[int(torch.randint(len(nb_choices), (1,), generator=g))]
        tables.append(perm[pos:pos + nb])
        pos += nb
    enc = encode_block_table(tables)
    target = torch.tensor([(t[:budget + 1] + [-1] * (budget + 1))[:budget + 1] for t in tables],
                          dtype=torch.int32)
    return tables, enc, target


def touched_pages(enc):
    out = set()
    for code in enc.flatten().tolist():
        if code == -1:
            continue
        out.add(-code - 2 if code < 0 else code)
    return out
