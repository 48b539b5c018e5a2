"""Drop-in for zipage/kernel/window_mask.py:47-72."""
import torch

from zipage_amd import _lib


def score_epilogue(scores, block_table, redundancy=None, *, max_norm_scores=False,
                   max_norm_red=False, redudancy_lambda=0.0, sink_len=0, window=0,
                   mask_pad=False):
    """Fused in-place post-processing of (L, B, Hkv, NB, BS) scores; see
    zp_score_epilogue in include/zipage_hip.h for the reference lines each switch covers."""
    L, B, Hkv, NB, BS = scores.shape
    assert scores.is_contiguous() and block_table.is_contiguous()
    assert block_table.shape == (B, NB) and block_table.dtype == torch.int32
    if redundancy is not None:
        assert redundancy.shape == scores.shape and redundancy.dtype == scores.dtype
        assert redundancy.is_contiguous()
    if scores.numel() == 0:
        return scores
    _lib.call("zp_score_epilogue", _lib.dev_ptr(scores), _lib.dev_ptr(redundancy),
              _lib.dev_ptr(block_table), L, B, NB, BS, Hkv, int(max_norm_scores),
              int(max_norm_red), float(redudancy_lambda), int(sink_len), int(window),
              int(mask_pad), _lib.dtype_tag(scores), _lib.stream_ptr(scores))
    return scores


def window_mask(scores: torch.Tensor, block_table: torch.Tensor, query_cache_len: int):
    """Set the scores of the last ``query_cache_len`` slots of each sequence's last page to
    +inf, in place.  scores: (L, B, Hkv, NB, BS); block_table: (B, NB)."""
    return score_epilogue(scores, block_table, window=query_cache_len)
