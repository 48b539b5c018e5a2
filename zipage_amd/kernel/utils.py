"""Drop-in for zipage/kernel/utils.py (topk_mask :21-36)."""
import torch

from zipage_amd import _lib


def topk_mask(scores: torch.Tensor, k: int):
    """Bool mask with the same shape as ``scores``: True on the k largest entries of the last
    axis.  Among equal scores the lowest index wins (the reference's torch.topk leaves the
    order of ties unspecified)."""
    assert scores.is_contiguous()
    Tn = scores.shape[-1]
    rows = scores.numel() // Tn if Tn else 0
    mask = torch.empty(scores.shape, device=scores.device, dtype=torch.bool)
    if rows == 0:
        return mask
    if not 0 <= k <= Tn:
        raise RuntimeError(f"selected index k out of range: k={k}, row length {Tn}")
    _lib.call("zp_topk_mask", _lib.dev_ptr(scores), _lib.dev_ptr(mask), rows, Tn, int(k),
              _lib.dtype_tag(scores), _lib.stream_ptr(scores))
    return mask
