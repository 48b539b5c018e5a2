"""Drop-in for zipage/kernel/raw_redudancy_score.py:158-238."""
import torch

from zipage_amd import _lib
from zipage_amd.kernel.key_norm import _check_cache


def raw_redudancy_score(key_cache: torch.Tensor, block_table: torch.Tensor,
                        threshold: float = 0.5, temperature: float = 1.0,
                        return_logits: bool = False):
    """Whole-sequence key redundancy: as the lightning variant but the similarity matrix
    spans every cached key of the sequence; row sums are divided by
    ``temperature * (#pages * BS)`` before the softmax.

    With ``return_logits`` returns ``(row_sums (L,B,Hkv,NB*BS), redundancy)``.
    """
    L, num_pages, BS, Hkv, D = _check_cache(key_cache)
    B, NB = block_table.shape
    assert block_table.is_contiguous() and block_table.dtype == torch.int32
    dev, dt = key_cache.device, key_cache.dtype
    red = torch.empty((L, B, Hkv, NB, BS), device=dev, dtype=dt)
    logits = torch.empty((L, B, Hkv, NB * BS), device=dev, dtype=dt) if return_logits else None
    if red.numel() == 0:
        return (logits, red) if return_logits else red
    lib = _lib.load()
    ws_bytes = lib.zp_redundancy_raw_workspace(L, B, NB, BS, Hkv)
    ws = torch.empty(ws_bytes, device=dev, dtype=torch.uint8) if ws_bytes else None
    _lib.call("zp_redundancy_raw", _lib.dev_ptr(key_cache), _lib.dev_ptr(block_table),
              _lib.dev_ptr(red), _lib.dev_ptr(logits), L, B, NB, BS, Hkv, D, num_pages,
              key_cache.stride(0), key_cache.stride(1), float(threshold), float(temperature),
              _lib.dtype_tag(key_cache), _lib.dev_ptr(ws), ws_bytes, _lib.stream_ptr(key_cache))
    if return_logits:
        return logits, red
    return red
