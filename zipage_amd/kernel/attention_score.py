"""Drop-in for zipage/kernel/attention_score.py:133-250."""
import torch

from zipage_amd import _lib

_REDUCE = {"mean": 0, "max": 1}


def attention_score(k_cache: torch.Tensor, query_cache: torch.Tensor, seq_idx: torch.Tensor,
                    block_table: torch.Tensor, softmax_scale=None, reduced="mean",
                    return_logits=False) -> torch.Tensor:
    """Importance of every cached token under the stored window queries.

    softmax over the sequence of (window query x key) logits, max over the GQA group, mean
    (or max) over the window.

    k_cache: (L, num_pages, BS, Hkv, D); query_cache: (L, max_num_seqs, W, Hq, D);
    seq_idx: (B,) int32 row of the query cache per sequence; block_table: (B, NB) int32,
    -1 is padding, x < -1 marks the last page (id = -x-2).
    Returns scores (L, B, Hkv, NB, BS) in the cache dtype, plus the raw logits
    (L, B, Hq, W, NB*BS) when ``return_logits``.
    """
    L, num_pages, BS, Hkv, D = k_cache.shape
    _, max_seqs, W, Hq, _ = query_cache.shape
    B, NB = block_table.shape
    if softmax_scale is None:
        softmax_scale = query_cache.shape[-1] ** (-0.5)
    assert k_cache.is_contiguous()
    assert query_cache.is_contiguous()
    assert seq_idx.is_contiguous()
    assert block_table.is_contiguous()
    assert seq_idx.dtype == torch.int32 and block_table.dtype == torch.int32
    assert query_cache.dtype == k_cache.dtype and query_cache.shape[0] == L
    if reduced not in _REDUCE:
        raise ValueError(f"Invalid reduction method: {reduced}")
    dev, dt = k_cache.device, k_cache.dtype
    scores = torch.empty((L, B, Hkv, NB, BS), device=dev, dtype=dt)
    logits = None
    if return_logits:
        logits = torch.full((L, B, Hq, W, NB * BS), -float("inf"), device=dev, dtype=dt)
    if L == 0 or B == 0:  # nothing to score: empty outputs, as the torch ops would give
        return (scores, logits) if return_logits else scores
    lib = _lib.load()
    ws_bytes = lib.zp_attention_score_workspace_for(L, B, NB, BS, Hkv, Hq, W, _lib.dtype_tag(k_cache))
    ws = torch.empty(ws_bytes, device=dev, dtype=torch.uint8) if ws_bytes else None
    _lib.call("zp_attention_score", _lib.dev_ptr(k_cache), _lib.dev_ptr(query_cache),
              _lib.dev_ptr(seq_idx), _lib.dev_ptr(block_table), _lib.dev_ptr(scores),
              _lib.dev_ptr(logits), L, B, NB, BS, Hkv, Hq, D, W, num_pages, max_seqs,
              k_cache.stride(0), k_cache.stride(1), query_cache.stride(0), query_cache.stride(1),
              float(softmax_scale), _REDUCE[reduced], _lib.dtype_tag(k_cache), _lib.dev_ptr(ws),
              ws_bytes, _lib.stream_ptr(k_cache))
    if return_logits:
        return scores, logits
    return scores
