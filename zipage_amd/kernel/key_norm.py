"""Drop-in for zipage/kernel/key_norm.py:72-113."""
import torch

from zipage_amd import _lib


def _check_cache(key_cache):
    L, num_pages, BS, Hkv, D = key_cache.shape
    assert key_cache.stride(4) == 1 and key_cache.stride(3) == D and key_cache.stride(2) == Hkv * D, \
        "key cache must be contiguous in its (slot, head, dim) axes"
    return L, num_pages, BS, Hkv, D


def key_norm(key_cache: torch.Tensor, block_table: torch.Tensor, norm_epsilon: float = 1e-6):
    """L2 norm of every cached key, clamped to ``norm_epsilon``.

    key_cache: (L, num_pages, BS, Hkv, D); block_table: (B, NB) -> (L, B, Hkv, NB, BS) in the
    cache dtype.
    """
    L, num_pages, BS, Hkv, D = _check_cache(key_cache)
    B, NB = block_table.shape
    assert block_table.is_contiguous() and block_table.dtype == torch.int32
    out = torch.empty((L, B, Hkv, NB, BS), device=key_cache.device, dtype=key_cache.dtype)
    if out.numel() == 0:
        return out
    _lib.call("zp_key_norm", _lib.dev_ptr(key_cache), _lib.dev_ptr(block_table), _lib.dev_ptr(out),
              L, B, NB, BS, Hkv, D, num_pages, key_cache.stride(0), key_cache.stride(1),
              float(norm_epsilon), _lib.dtype_tag(key_cache), _lib.stream_ptr(key_cache))
    return out
