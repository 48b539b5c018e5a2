"""Sequence-axis pooling the reference runner does inline
(zipage/engine/model_runner.py:499-530)."""
import torch

from zipage_amd import _lib

_MODES = {"max": 0, "avg": 1}


def pool_scores(scores: torch.Tensor, compressed: torch.Tensor, kernel_size: int = 5,
                continues_pooling: bool = False, mode: str = "max") -> torch.Tensor:
    """max_pool1d(kernel, stride 1, pad kernel//2) over the flattened NB*BS axis of
    (L, B, Hkv, NB, BS) scores.  Sequences already ``compressed`` keep their raw scores unless
    ``continues_pooling`` -- decided per sequence on the device, so the reference's
    ``torch.all(compressed)`` host sync is not needed (it only skips work whose result is
    the input).  ``mode="avg"`` is an extension with no counterpart in the reference."""
    L, B, Hkv, NB, BS = scores.shape
    assert scores.is_contiguous() and compressed.dtype == torch.bool
    out = torch.empty_like(scores)
    if out.numel() == 0:
        return out
    _lib.call("zp_pool_scores", _lib.dev_ptr(scores), _lib.dev_ptr(out),
              _lib.dev_ptr(compressed.contiguous()), L, B, Hkv, NB * BS, int(kernel_size),
              int(continues_pooling), _MODES[mode], _lib.dtype_tag(scores),
              _lib.stream_ptr(scores))
    return out
