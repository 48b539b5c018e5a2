"""Drop-in for zipage/kernel/global_score.py:77-120."""
import torch

from zipage_amd import _lib

_METHODS = {"max": 0, "sum": 1}


def global_score(reduced_scores: torch.Tensor, score_cache: torch.Tensor,
                 block_table: torch.Tensor, compressed: torch.Tensor,
                 decay_factor: float = 0.9, activate_method: str = "max", *,
                 write_cache: bool = True) -> torch.Tensor:
    """max(new, old*decay) (or the sum) against the carried score cache.

    ``write_cache=False`` (not in the reference) leaves the score cache untouched: the reference
    stores every sequence's result into its pages (global_score.py:73-74), which races when
    sequences of one batch share prefix pages; the carried values are then compacted from the
    returned scores (``compress_score(..., scores_src=...)``).

    reduced_scores: (L, B, Hkv, NB, BS), updated in place and returned; score_cache:
    (L, num_pages, BS, Hkv), updated in place; block_table: (B, NB) int32; compressed:
    (B,) bool.
    """
    assert decay_factor >= 0 and decay_factor <= 1
    assert activate_method in ["max", "sum"]
    L, num_pages, BS, Hkv = score_cache.shape
    B, NB = block_table.shape
    assert reduced_scores.shape == (L, B, Hkv, NB, BS)
    assert reduced_scores.is_contiguous() and block_table.is_contiguous()
    assert score_cache.stride(3) == 1 and score_cache.stride(2) == Hkv
    assert reduced_scores.dtype == score_cache.dtype
    assert block_table.dtype == torch.int32 and compressed.dtype == torch.bool
    compressed = compressed.contiguous()
    if reduced_scores.numel() == 0:
        return reduced_scores
    _lib.call("zp_global_score", _lib.dev_ptr(reduced_scores), _lib.dev_ptr(score_cache),
              _lib.dev_ptr(block_table), _lib.dev_ptr(compressed), L, B, NB, BS, Hkv, num_pages,
              score_cache.stride(0), score_cache.stride(1), float(decay_factor),
              _METHODS[activate_method], int(write_cache), _lib.dtype_tag(reduced_scores),
              _lib.stream_ptr(reduced_scores))
    return reduced_scores
