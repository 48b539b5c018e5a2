"""Drop-in for zipage/kernel/compress_score.py:66-99."""
import torch

from zipage_amd import _lib


def compress_score(score_cache: torch.Tensor, flag: torch.Tensor, block_table: torch.Tensor,
                   target_block_table: torch.Tensor, *, scores_src: torch.Tensor | None = None):
    """Same walk as compress_kv, moving one carried score per kept token.

    score_cache: (L, num_pages, BS, Hkv), compacted in place and returned.  With ``scores_src``
    (L, B, Hkv, NB, BS; not in the reference) the value of a kept token is read from there
    instead of from its source page of the cache: no page another sequence shares is read.
    """
    L, B, Hkv, NB, BS = flag.shape
    assert score_cache.shape[0] == L and score_cache.shape[2:] == (BS, Hkv)
    assert flag.dtype == torch.bool and flag.is_contiguous()
    assert block_table.shape == (B, NB) and block_table.is_contiguous()
    assert target_block_table.shape[0] == B and target_block_table.is_contiguous()
    assert block_table.dtype == torch.int32 and target_block_table.dtype == torch.int32
    if flag.numel() == 0:
        return score_cache
    if scores_src is not None:
        assert scores_src.shape == flag.shape and scores_src.is_contiguous()
        assert scores_src.dtype == score_cache.dtype
    _lib.call("zp_compress_score", _lib.dev_ptr(score_cache), _lib.dev_ptr(scores_src),
              _lib.dev_ptr(flag),
              _lib.dev_ptr(block_table), _lib.dev_ptr(target_block_table), L, B, NB, BS, Hkv,
              score_cache.shape[1], target_block_table.shape[1], score_cache.stride(0),
              score_cache.stride(1), score_cache.stride(2), score_cache.stride(3),
              _lib.dtype_tag(score_cache), _lib.stream_ptr(score_cache))
    return score_cache
