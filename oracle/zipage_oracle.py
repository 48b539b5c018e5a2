"""CPU oracle for the compressed-PagedAttention KV-compression path.

TEST INFRASTRUCTURE ONLY.  This module is a plain PyTorch-on-CPU restatement of the
algorithm in the reference's ``zipage/kernel/*.py`` and of the glue in
``zipage/engine/model_runner.py:424-631``.  It is imported only by ``tests/``, by
``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py``, always as
the checker and never as a product path.  The product (``zipage_amd``) never imports it
and raises if its HIP library is missing.

Every function cites the reference lines it follows.  The reference rounds several
intermediates to the cache dtype (bf16/fp16).  ``rounding="reference"`` (the default)
rounds at exactly those points; ``rounding="fp32"`` keeps every intermediate in fp32 and
rounds only the returned tensor.  With fp32 caches both modes are identical.

Pinning status (which independent check fixes each function) lives in the tests:
``tests/test_oracle_pins.py`` (fp32: brute force, library routines, closed forms) and
``tests/test_oracle_pins_16bit.py`` (bf16/fp16: the torch-op epilogues of the reference run as
library ops on cache-dtype CPU tensors, bit for bit, with a mutation check per rounding).
Parity unpinned -- only an execution of the reference on its own GPU stack could pin these, so
this file *defines* them: ``torch.topk``'s tie order (here: lowest index first); the
arithmetic of Triton's ``tl.dot`` on fp32 operands (TF32 on NVIDIA; here IEEE fp32); whether
Triton rounds ``cache * decay_factor`` to the cache dtype before the max / add of
``global_score`` (here: the product stays fp32); and that torch's GPU kernel for
``tensor.div_(python_scalar)`` may multiply by the reciprocal (here: a true division).

Page-table encoding (``zipage/engine/model_runner.py:437-463``): an int32 row per
sequence; ``id >= 0`` is a full page, ``-1`` is padding, ``x < -1`` marks the sequence's
last page with ``id = -x - 2``.
"""

from __future__ import annotations

import math

import torch
import torch.nn.functional as F

NEG_INF = float("-inf")
POS_INF = float("inf")


# ----------------------------------------------------------------------------- helpers
def _rnd(x: torch.Tensor, dtype: torch.dtype, rounding: str) -> torch.Tensor:
    """Round an fp32 tensor to ``dtype`` and come back to fp32 (identity in fp32 mode)."""
    if rounding == "fp32" or dtype == torch.float32:
        return x
    return x.to(dtype).to(torch.float32)


def decode_page(code: int):
    """(is_pad, is_last, page_id) of one block-table entry (attention_score.py:80-86)."""
    if code == -1:
        return True, False, -1
    if code < 0:
        return False, True, -code - 2
    return False, False, code


def encode_block_table(tables, pad_to=None) -> torch.Tensor:
    """Host glue of ``ModelRunner.compress`` (model_runner.py:437-463): mark each
    sequence's last page as ``-(id)-2`` and right-pad with ``-1``."""
    width = max(len(t) for t in tables) if pad_to is None else pad_to
    rows = []
    for t in tables:
        row = list(t[:-1]) + [-t[-1] - 2]
        rows.append(row + [-1] * (width - len(row)))
    return torch.tensor(rows, dtype=torch.int32)


# -------------------------------------------------------------------- a1 store_query
def store_query_cache(query, query_cache, slot_mapping) -> None:
    """``q_cache[seq_id, slot] = q[pos]`` for every int32 triple ``(pos, seq_id, slot)``
    (store_query_cache.py:7-32,35-68).  No-op on an empty cache (:50-51)."""
    if query_cache.numel() == 0:
        return
    assert query.stride(-1) == 1
    assert query.stride(1) == query.shape[-1]
    for pos, seq_id, slot in slot_mapping.tolist():
        query_cache[seq_id, slot] = query[pos]


# -------------------------------------------------------------------- a2 attention score
def attention_logits(k_cache, query_cache, seq_idx, block_table, softmax_scale=None,
                     rounding="reference") -> torch.Tensor:
    """Scaled, masked logits ``(L,B,Hq,W,NB,BS)`` as fp32 values that are representable
    in the cache dtype (attention_score.py:44-130): fp32 dot, ``* scale``, causal mask on
    the last page (``slot > BS-W+w`` -> -inf, :112-120), cast to the input dtype (:129);
    pad pages stay -inf (:174-186)."""
    L, _, BS, Hkv, D = k_cache.shape
    _, _, W, Hq, _ = query_cache.shape
    B, NB = block_table.shape
    G = Hq // Hkv
    scale = D ** (-0.5) if softmax_scale is None else softmax_scale
    scale = float(torch.tensor(scale, dtype=torch.float32))
    out = torch.full((L, B, Hq, W, NB, BS), NEG_INF, dtype=torch.float32)
    slots = torch.arange(BS)[None, :]
    rows = (BS - W + torch.arange(W))[:, None]
    causal = slots > rows  # (W, BS)
    for b in range(B):
        q = query_cache[:, int(seq_idx[b])].to(torch.float32)  # (L, W, Hq, D)
        q = q.permute(0, 2, 1, 3)  # (L, Hq, W, D)
        for j in range(NB):
            pad, last, pid = decode_page(int(block_table[b, j]))
            if pad:
                continue
            k = k_cache[:, pid].to(torch.float32)  # (L, BS, Hkv, D)
            k = k.permute(0, 2, 3, 1).repeat_interleave(G, dim=1)  # (L, Hq, D, BS)
            s = torch.matmul(q, k) * scale  # (L, Hq, W, BS)
            if last:
                s = s.masked_fill(causal, NEG_INF)
            out[:, b, :, :, j, :] = s
    return _rnd(out, k_cache.dtype, rounding)


def attention_score(k_cache, query_cache, seq_idx, block_table, softmax_scale=None,
                    reduced="mean", return_logits=False, rounding="reference"):
    """Per-token importance ``(L,B,Hkv,NB,BS)`` in the cache dtype
    (attention_score.py:133-250): logits as above; ``x = logits - rowmax`` (:222);
    ``P = softmax_T(x)`` (:223); max over the GQA group (:225-229); mean or max over the
    window (:242-247).  Each torch op in the reference runs on cache-dtype tensors, so
    each of those four results is rounded to the cache dtype."""
    if reduced not in ("mean", "max"):
        raise ValueError(f"Invalid reduction method: {reduced}")
    dt = k_cache.dtype
    L, _, BS, Hkv, D = k_cache.shape
    _, _, W, Hq, _ = query_cache.shape
    B, NB = block_table.shape
    G = Hq // Hkv
    logits = attention_logits(k_cache, query_cache, seq_idx, block_table, softmax_scale,
                              rounding)
    flat = logits.reshape(L, B, Hq, W, NB * BS)
    x = _rnd(flat - flat.max(dim=-1, keepdim=True).values, dt, rounding)
    p = _rnd(torch.softmax(x, dim=-1), dt, rounding)
    p = p.view(L, B, Hkv, G, W, NB * BS).max(dim=3).values
    if reduced == "mean":
        r = _rnd(p.mean(dim=3), dt, rounding)
    else:
        r = p.max(dim=3).values
    r = r.reshape(L, B, Hkv, NB, BS).to(dt)
    if return_logits:
        return r, flat.to(dt)
    return r


# -------------------------------------------------------------------- a3 global score
def global_score(reduced_scores, score_cache, block_table, compressed, decay_factor=0.9,
                 activate_method="max", write_cache=True):
    """Carry scores over from the previous compression (global_score.py:8-74,77-120).
    For a non-pad page of a sequence that is ``compressed`` and is not its last page:
    ``out = max(new, old*decay)`` or ``new + old*decay`` in fp32, cast to the scores'
    dtype (:60-70); otherwise ``out = new``.  ``out`` goes to the scores in place and to
    ``score_cache[l, page, slot, head]`` (:73-74).  The loop visits sequences in order, so a
    page several sequences share ends up with the LAST sequence's scores (on a GPU the
    reference's stores race).  ``write_cache=False`` is this build's race-free mode: the cache
    is only read (see :func:`compress_score`, ``scores_src``)."""
    assert 0 <= decay_factor <= 1
    assert activate_method in ("max", "sum")
    decay = float(torch.tensor(decay_factor, dtype=torch.float32))
    B, NB = block_table.shape
    for b in range(B):
        for j in range(NB):
            pad, last, pid = decode_page(int(block_table[b, j]))
            if pad:
                continue
            new = reduced_scores[:, b, :, j, :]  # (L, Hkv, BS) view
            if bool(compressed[b]) and not last:
                old = score_cache[:, pid].permute(0, 2, 1).to(torch.float32)  # (L,Hkv,BS)
                if activate_method == "max":
                    out = torch.maximum(new.to(torch.float32), old * decay)
                else:
                    out = new.to(torch.float32) + old * decay
                out = out.to(reduced_scores.dtype)
            else:
                out = new.clone()
            reduced_scores[:, b, :, j, :] = out
            if write_cache:
                score_cache[:, pid] = out.permute(0, 2, 1).to(score_cache.dtype)
    return reduced_scores


# -------------------------------------------------------------------- a4 pooling
def pool_scores(scores, compressed, kernel_size=5, continues_pooling=False, mode="max"):
    """Sequence-axis pooling as the runner does it (model_runner.py:499-530):
    ``max_pool1d(kernel, stride 1, pad kernel//2)`` over the flattened ``NB*BS`` axis;
    sequences already ``compressed`` keep their raw scores unless ``continues_pooling``;
    nothing happens when every sequence is compressed.  ``mode="avg"`` is an extension
    of this build (``avg_pool1d``, zero padding counted) with no counterpart in the
    reference."""
    L, B, Hkv, NB, BS = scores.shape
    if not continues_pooling and bool(torch.all(compressed)):
        return scores
    flat = scores.reshape(L * B, Hkv, NB * BS)
    if mode == "max":
        pooled = F.max_pool1d(flat.to(torch.float32), kernel_size, 1, kernel_size // 2)
    elif mode == "avg":
        pooled = F.avg_pool1d(flat.to(torch.float32), kernel_size, 1, kernel_size // 2)
    else:
        raise ValueError(mode)
    pooled = pooled.to(scores.dtype)
    if not continues_pooling:
        keep_raw = compressed.view(1, B).expand(L, B).reshape(L * B, 1, 1)
        pooled = torch.where(keep_raw, flat, pooled)
    return pooled.reshape(L, B, Hkv, NB, BS)


# -------------------------------------------------------------------- a5 key norm
def key_norm(key_cache, block_table, norm_epsilon=1e-6, rounding="reference"):
    """``max(||k||_2, eps)`` per cached key, ``(L,B,Hkv,NB,BS)`` in the cache dtype
    (key_norm.py:8-69,72-113): fp32 sum of squares and sqrt, cast to the cache dtype
    (:54-56), pad pages 0, then ``clamp(min=eps)`` (:112)."""
    L, _, BS, Hkv, D = key_cache.shape
    B, NB = block_table.shape
    out = torch.zeros((L, B, Hkv, NB, BS), dtype=torch.float32)
    for b in range(B):
        for j in range(NB):
            pad, _, pid = decode_page(int(block_table[b, j]))
            if pad:
                continue
            k = key_cache[:, pid].to(torch.float32)  # (L, BS, Hkv, D)
            out[:, b, :, j, :] = torch.sqrt((k * k).sum(dim=-1)).permute(0, 2, 1)
    out = out.to(key_cache.dtype)  # the kernel stores in the cache dtype in both modes
    return torch.clamp(out, min=norm_epsilon)


# -------------------------------------------------------------------- a6/a7 redundancy
def _claim_last_over_threshold(sim: torch.Tensor, threshold: float) -> torch.Tensor:
    """For every column j of ``sim (..., R, C)`` zero the entry of the LAST row i with
    ``sim[i, j] > threshold`` (lightning_redudancy_score.py:136-154,
    raw_redudancy_score.py:113-131: rows are visited from the end and a column is
    claimed once)."""
    R = sim.shape[-2]
    over = sim > threshold
    idx = torch.arange(R).view(R, 1).expand_as(sim)
    last = torch.where(over, idx, torch.full_like(idx, -1)).max(dim=-2, keepdim=True).values
    return torch.where(idx == last, torch.zeros_like(sim), sim)


def _normalised_keys(key_cache, norm, b, j, pid):
    k = key_cache[:, pid].to(torch.float32).permute(0, 2, 1, 3)  # (L, Hkv, BS, D)
    n = norm[:, b, :, j, :].to(torch.float32).unsqueeze(-1)  # (L, Hkv, BS, 1)
    return k / n


def lightning_redudancy_logits(key_cache, block_table, threshold=0.5,
                               rounding="reference"):
    """Per-page redundancy row sums ``(L,B,Hkv,NB,BS)`` in the cache dtype
    (lightning_redudancy_score.py:10-169): within one page, cosine similarity of every
    key pair (keys divided by the cache-dtype norm in fp32, :73-75,108-109, fp32 dot),
    diagonal zeroed (:111-113), last row over the threshold zeroed per column
    (:136-154), row sum stored in the cache dtype (:155-169); pad pages -inf (:198-209).
    """
    L, _, BS, Hkv, D = key_cache.shape
    B, NB = block_table.shape
    norm = key_norm(key_cache, block_table)
    out = torch.full((L, B, Hkv, NB, BS), NEG_INF, dtype=torch.float32)
    eye = torch.eye(BS, dtype=torch.bool)
    for b in range(B):
        for j in range(NB):
            pad, _, pid = decode_page(int(block_table[b, j]))
            if pad:
                continue
            kh = _normalised_keys(key_cache, norm, b, j, pid)
            sim = torch.matmul(kh, kh.transpose(-1, -2))  # (L, Hkv, BS, BS)
            sim = sim.masked_fill(eye, 0.0)
            sim = _claim_last_over_threshold(sim, threshold)
            out[:, b, :, j, :] = sim.sum(dim=-1)
    return out.to(key_cache.dtype)


def _redundancy_softmax(logits, divisor, dt, rounding):
    """Wrapper epilogue shared by both variants (lightning_redudancy_score.py:248-252,
    raw_redudancy_score.py:226-229): in-place divide, subtract the row max, softmax over
    the flattened sequence; each op rounds to the cache dtype."""
    x = _rnd(logits.to(torch.float32) / divisor, dt, rounding)
    x = _rnd(x - x.max(dim=-1, keepdim=True).values, dt, rounding)
    return _rnd(torch.softmax(x, dim=-1), dt, rounding)


def lightning_redudancy_score(key_cache, block_table, threshold=0.5, temperature=1.0,
                              return_logits=False, rounding="reference"):
    """Softmax-normalised per-page key redundancy (lightning_redudancy_score.py:172-261).
    """
    L, _, BS, Hkv, _ = key_cache.shape
    B, NB = block_table.shape
    dt = key_cache.dtype
    logits = lightning_redudancy_logits(key_cache, block_table, threshold, rounding)
    flat = logits.view(L, B, Hkv, NB * BS)
    div = torch.tensor(temperature * BS, dtype=torch.float32)
    red = _redundancy_softmax(flat, div, dt, rounding).to(dt).reshape(L, B, Hkv, NB, BS)
    if return_logits:
        return logits, red
    return red


def raw_redudancy_logits(key_cache, block_table, threshold=0.5, rounding="reference",
                         col_chunk=16, return_partial_max=False):
    """Whole-sequence redundancy row sums ``(L,B,Hkv,NB*BS)`` (raw_redudancy_score.py:
    10-155,218-222).  Same rule as the lightning variant but the similarity matrix spans
    every cached key of the sequence; the diagonal is the global one (:107-111) and "last
    row" is by logical position because row pages are visited last to first (:84).
    The reference keeps one partial row sum per column page, accumulated in the cache
    dtype over that page's 16-column chunks (:146-155), then sums the partials over
    column pages (:218); ``rounding="reference"`` follows that chain.
    ``return_partial_max`` also returns, per key, the largest magnitude any of its partial sums
    reached along the chain (tests size their tolerance by it: one fp32-order rounding flip
    inside the chain moves the result by one unit in the last place of a PARTIAL sum)."""
    L, _, BS, Hkv, D = key_cache.shape
    B, NB = block_table.shape
    dt = key_cache.dtype
    norm = key_norm(key_cache, block_table)
    out = torch.full((L, B, Hkv, NB * BS), NEG_INF, dtype=torch.float32)
    pmax = torch.zeros((L, B, Hkv, NB * BS), dtype=torch.float32)
    for b in range(B):
        valid = [j for j in range(NB) if int(block_table[b, j]) != -1]
        kh = torch.cat([
            _normalised_keys(key_cache, norm, b, j, decode_page(int(block_table[b, j]))[2])
            for j in valid], dim=2)  # (L, Hkv, Tv, D)
        Tv = kh.shape[2]
        sim = torch.matmul(kh, kh.transpose(-1, -2))  # (L, Hkv, Tv, Tv)
        sim = sim.masked_fill(torch.eye(Tv, dtype=torch.bool), 0.0)
        sim = _claim_last_over_threshold(sim, threshold)
        if rounding == "fp32" or dt == torch.float32:
            rows = sim.sum(dim=-1)
            big = rows.abs()
        else:
            chunks = sim.view(L, Hkv, Tv, len(valid), BS // col_chunk, col_chunk).sum(-1)
            part = torch.zeros((L, Hkv, Tv, len(valid)), dtype=torch.float32)
            big = torch.zeros((L, Hkv, Tv), dtype=torch.float32)
            for c in range(BS // col_chunk):
                part = _rnd(part + chunks[..., c], dt, rounding)
                big = torch.maximum(big, part.abs().amax(dim=-1))
            rows = _rnd(part.sum(dim=-1), dt, rounding)
        for n, j in enumerate(valid):
            out[:, b, :, j * BS:(j + 1) * BS] = rows[:, :, n * BS:(n + 1) * BS]
            pmax[:, b, :, j * BS:(j + 1) * BS] = big[:, :, n * BS:(n + 1) * BS]
    if return_partial_max:
        return out.to(dt), pmax
    return out.to(dt)


def raw_redudancy_score(key_cache, block_table, threshold=0.5, temperature=1.0,
                        return_logits=False, rounding="reference"):
    """Softmax-normalised whole-sequence key redundancy (raw_redudancy_score.py:158-238):
    divide by ``temperature * (#non-pad pages * BS)`` (:226-227)."""
    L, _, BS, Hkv, _ = key_cache.shape
    B, NB = block_table.shape
    dt = key_cache.dtype
    logits = raw_redudancy_logits(key_cache, block_table, threshold, rounding)
    seq_len = ((block_table != -1).sum(dim=-1) * BS).to(torch.float32)
    div = (temperature * seq_len).view(1, B, 1, 1)
    red = _redundancy_softmax(logits, div, dt, rounding).to(dt).reshape(L, B, Hkv, NB, BS)
    if return_logits:
        return logits, red
    return red


# -------------------------------------------------------------------- a8 combine / sink
def max_normalise(x):
    """``x / max_T(x)`` over the flattened sequence axis (model_runner.py:482-487,
    551-556)."""
    L, B, H, NB, BS = x.shape
    flat = x.reshape(L, B, H, NB * BS)
    return (flat / flat.max(dim=-1, keepdim=True).values).reshape(L, B, H, NB, BS)


def combine_scores(scores, redundancy, redudancy_lambda):
    """``scores*lambda - redundancy*(1-lambda)`` with the torch semantics of the runner
    (model_runner.py:557-559): each product and the difference round to the dtype."""
    return scores * redudancy_lambda - redundancy * (1 - redudancy_lambda)


def attention_sink(scores, sink_len):
    """First ``sink_len`` logical tokens get +inf (model_runner.py:565-578)."""
    L, B, H, NB, BS = scores.shape
    flat = scores.view(L, B, H, NB * BS)
    flat[..., :sink_len] = POS_INF
    return scores


# -------------------------------------------------------------------- a9 window mask
def window_mask(scores, block_table, query_cache_len):
    """Slots ``[BS-W, BS)`` of each sequence's last page get +inf, in place
    (window_mask.py:8-44,47-72)."""
    B, NB = block_table.shape
    BS = scores.shape[-1]
    for b in range(B):
        for j in range(NB):
            pad, last, _ = decode_page(int(block_table[b, j]))
            if last:
                scores[:, b, :, j, BS - query_cache_len:] = POS_INF
    return scores


# -------------------------------------------------------------------- a10 top-k mask
def pad_mask(scores, block_table):
    """Pad pages get -inf before selection (model_runner.py:592-593)."""
    mask = (block_table == -1).view(1, block_table.shape[0], 1, block_table.shape[1], 1)
    return scores.masked_fill_(mask, NEG_INF)


def topk_mask(scores, k):
    """Bool mask, True on the ``k`` largest entries of the last axis
    (zipage/kernel/utils.py:21-36).  ``torch.topk`` leaves the order among equal values
    unspecified; this build defines it: among equals the lowest index wins, i.e. a stable
    descending sort followed by taking the first ``k``."""
    order = torch.sort(scores.to(torch.float32), dim=-1, descending=True, stable=True).indices
    mask = torch.zeros_like(scores, dtype=torch.bool)
    mask.scatter_(-1, order[..., :k], True)
    return mask


# -------------------------------------------------------------------- a11/a12 compaction
def _compaction_plan(flag_row, table_row, target_row, BS):
    """Source and destination (page, slot) lists of one (layer, sequence, head) walk
    (compress_kv.py:53-100): pages in table order, slots ascending, the n-th kept token
    goes to ``target[n // BS]``, slot ``n % BS``."""
    src_page, src_slot = [], []
    for j, code in enumerate(table_row):
        pad, _, pid = decode_page(int(code))
        if pad:
            continue
        kept = torch.nonzero(flag_row[j]).flatten().tolist()
        src_page += [pid] * len(kept)
        src_slot += kept
    n = len(src_page)
    dst_page = [int(target_row[i // BS]) for i in range(n)]
    dst_slot = [i % BS for i in range(n)]
    return src_page, src_slot, dst_page, dst_slot


def compress_kv_loop(key, value, flag, block_table, target_block_table) -> None:
    """Literal token-by-token restatement of compress_kv.py:39-100 (in place, serial, so
    aliasing source/target pages behave exactly as in the reference).  Slow: tests only.
    """
    L, _, BS, Hkv, _ = key.shape
    _, B, _, NB, _ = flag.shape
    for l in range(L):
        for b in range(B):
            for h in range(Hkv):
                sp, ss, dp, ds = _compaction_plan(flag[l, b, h], block_table[b],
                                                  target_block_table[b], BS)
                for a, s, c, d in zip(sp, ss, dp, ds):
                    key[l, c, d, h] = key[l, a, s, h]
                    value[l, c, d, h] = value[l, a, s, h]


def compress_kv(key, value, flag, block_table, target_block_table) -> None:
    """Vectorised equivalent of :func:`compress_kv_loop` for tables the engine produces
    (a target page aliases a source page only at the same logical index, so reading all
    sources before writing gives the serial result; checked against the loop in tests).
    """
    L, _, BS, Hkv, _ = key.shape
    _, B, _, NB, _ = flag.shape
    for l in range(L):
        for b in range(B):
            for h in range(Hkv):
                sp, ss, dp, ds = _compaction_plan(flag[l, b, h], block_table[b],
                                                  target_block_table[b], BS)
                if not sp:
                    continue
                sp, ss = torch.tensor(sp), torch.tensor(ss)
                dp, ds = torch.tensor(dp), torch.tensor(ds)
                kk = key[l, sp, ss, h].clone()
                vv = value[l, sp, ss, h].clone()
                key[l, dp, ds, h] = kk
                value[l, dp, ds, h] = vv


def compress_score(score_cache, flag, block_table, target_block_table, scores_src=None):
    """Same walk moving one ``score_cache[l, page, slot, head]`` scalar per kept token
    (compress_score.py:8-63,66-99).  With ``scores_src`` ``(L,B,Hkv,NB,BS)`` (this build's
    race-free mode, no counterpart in the reference) the scalar of a kept token is taken from
    there: it is what ``global_score`` would have stored for THIS sequence, so the result
    equals the reference's whenever no source page is shared with another sequence of the
    batch, and does not depend on the order of the sequences when one is."""
    L, _, BS, Hkv = score_cache.shape
    _, B, _, NB, _ = flag.shape
    for l in range(L):
        for b in range(B):
            for h in range(Hkv):
                sp, ss, dp, ds = _compaction_plan(flag[l, b, h], block_table[b],
                                                  target_block_table[b], BS)
                if not sp:
                    continue
                if scores_src is not None:
                    # logical (page index, slot) of every kept token, in the walk's order
                    kept = [(j, s) for j, code in enumerate(block_table[b].tolist()) if code != -1
                            for s in torch.nonzero(flag[l, b, h, j]).flatten().tolist()]
                    vals = torch.stack([scores_src[l, b, h, j, s] for j, s in kept])
                    score_cache[l, torch.tensor(dp), torch.tensor(ds), h] = vals.to(score_cache.dtype)
                    continue
                vals = score_cache[l, torch.tensor(sp), torch.tensor(ss), h].clone()
                score_cache[l, torch.tensor(dp), torch.tensor(ds), h] = vals
    return score_cache


# -------------------------------------------------------------------- a13 pipeline glue
def compress_pipeline(k_cache, v_cache, query_cache, score_cache, query_ids, block_table,
                      compressed, target_block_table, *, budget_blocks, query_cache_len,
                      softmax_scale=None, reduced="mean", use_global_score=False,
                      max_norm=False, decay_factor=0.8, activate_method="max",
                      enable_pooling=False, continues_pooling=False, pooling_size=5,
                      pooling_mode="max", use_redudancy=False, lightning_redudancy=False,
                      redudancy_lambda=0.2, redudancy_temperature=0.4,
                      redudancy_threshold=0.5, use_attention_sink=False, sink_len=4,
                      rounding="reference", return_intermediates=False,
                      deterministic_carry=False):
    """One layer chunk of ``ModelRunner.compress`` (model_runner.py:466-622), same stage
    order: attention_score -> [max-norm] global_score -> pooling -> redundancy + combine
    -> sink -> window_mask -> pad mask -> top-k (k = BS*budget) -> compress_kv ->
    compress_score.  Mutates ``k_cache``, ``v_cache`` and ``score_cache`` in place and
    returns the keep flag (and the final scores when asked).  ``deterministic_carry`` is this
    build's race-free handling of the score cache: ``global_score`` only reads it and the
    carried scores of the survivors are compacted from the scores it returned.  It is off by
    default here (this function restates the reference) and on by default in the product's
    ``compress_layers``: pass it explicitly to both when comparing them."""
    BS = k_cache.shape[2]
    scores = attention_score(k_cache, query_cache, query_ids, block_table, softmax_scale,
                             reduced, rounding=rounding)
    if use_global_score:
        if max_norm:
            scores = max_normalise(scores)
        scores = global_score(scores, score_cache, block_table, compressed, decay_factor,
                              activate_method, write_cache=not deterministic_carry)
        carried = scores.clone() if deterministic_carry else None
    if enable_pooling:
        scores = pool_scores(scores, compressed, pooling_size, continues_pooling,
                             pooling_mode)
    if use_redudancy:
        fn = lightning_redudancy_score if lightning_redudancy else raw_redudancy_score
        red = fn(k_cache, block_table, threshold=redudancy_threshold,
                 temperature=redudancy_temperature, rounding=rounding)
        if use_global_score and max_norm:
            red = max_normalise(red)
        scores = combine_scores(scores, red, redudancy_lambda)
    if use_attention_sink:
        scores = attention_sink(scores, sink_len)
    scores = window_mask(scores, block_table, query_cache_len)
    scores = pad_mask(scores, block_table)
    L, B, Hkv, NB, _ = scores.shape
    flag = topk_mask(scores.view(L, B, Hkv, NB * BS), BS * budget_blocks)
    flag = flag.view(L, B, Hkv, NB, BS)
    compress_kv(k_cache, v_cache, flag, block_table, target_block_table)
    if use_global_score:
        compress_score(score_cache, flag, block_table, target_block_table, scores_src=carried)
    if return_intermediates:
        return flag, scores
    return flag


# -------------------------------------------------------------------- host bookkeeping
def query_slot_mapping(query_id, block_size, query_cache_len, *, is_prefill, cu_len=0,
                       seqlen_q=0, last_block_num_tokens=0):
    """Which of this step's query rows enter the window ring and where
    (model_runner.py:319-350).  Returns ``(row, query_id, slot)`` triples."""
    out = []
    if query_id == -1:
        return out
    if is_prefill:
        nb = (seqlen_q + block_size - 1) // block_size
        if nb == 0:
            return out
        last = seqlen_q - (nb - 1) * block_size
        if last > block_size - query_cache_len:
            start = nb * block_size - query_cache_len
            for idx, pos in enumerate(range(start, seqlen_q)):
                out.append((cu_len + pos, query_id, idx))
    elif last_block_num_tokens > block_size - query_cache_len:
        out.append((cu_len, query_id,
                    last_block_num_tokens - (block_size - query_cache_len) - 1))
    return out


def target_block_table(block_table, ref_counts, is_compressed, max_blocks, free_ids):
    """Copy-on-write target table of ``BlockManager.may_compress``
    (block_manager.py:129-169).  ``max_blocks`` is budget+1.  Returns
    ``(new_table, to_release, remaining_free)`` or ``None`` when there are not enough
    free pages."""
    if is_compressed:
        return list(block_table[:max_blocks]), list(block_table[max_blocks:]), list(free_ids)
    p = 0
    for pid in block_table:
        if ref_counts.get(pid, 1) > 1:
            p += 1
        else:
            break
    assert len(block_table) - p >= 1
    n_new = min(p, max_blocks - 1)
    if n_new > len(free_ids):
        return None
    new = list(free_ids[:n_new]) + list(block_table[p:p + max_blocks - n_new])
    assert len(new) == max_blocks
    release = list(block_table[:p]) + list(block_table[p + max_blocks - n_new:])
    return new, release, list(free_ids[n_new:])
