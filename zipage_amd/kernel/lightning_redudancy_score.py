"""Drop-in for zipage/kernel/lightning_redudancy_score.py:172-261."""
import torch

from zipage_amd import _lib
from zipage_amd.kernel.key_norm import _check_cache


def lightning_redudancy_score(key_cache: torch.Tensor, block_table: torch.Tensor,
                              threshold: float = 0.5, temperature: float = 1.0,
                              return_logits: bool = False):
    """Per-page key redundancy: cosine similarity of every key pair inside a page, diagonal
    and (per column) the last row above ``threshold`` zeroed, row sums divided by
    ``temperature * BS`` and softmax-normalised over the sequence.

    key_cache: (L, num_pages, BS, Hkv, D); block_table: (B, NB) -> (L, B, Hkv, NB, BS) in the
    cache dtype; with ``return_logits`` returns ``(row_sums, redundancy)``.
    """
    L, num_pages, BS, Hkv, D = _check_cache(key_cache)
    B, NB = block_table.shape
    assert block_table.is_contiguous() and block_table.dtype == torch.int32
    dev, dt = key_cache.device, key_cache.dtype
    red = torch.empty((L, B, Hkv, NB, BS), device=dev, dtype=dt)
    logits = torch.empty_like(red) if return_logits else None
    if red.numel() == 0:
        return (logits, red) if return_logits else red
    _lib.call("zp_redundancy_lightning", _lib.dev_ptr(key_cache), _lib.dev_ptr(block_table),
              _lib.dev_ptr(red), _lib.dev_ptr(logits), L, B, NB, BS, Hkv, D, num_pages,
              key_cache.stride(0), key_cache.stride(1), float(threshold), float(temperature),
              _lib.dtype_tag(key_cache), _lib.stream_ptr(key_cache))
    if return_logits:
        return logits, red
    return red
