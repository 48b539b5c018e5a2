"""The selection stages the reference runner does inline between scoring and compaction
(zipage/engine/model_runner.py:499-530 pooling, :551-600 combine, sink, window mask, pad
mask and top-k), as one launch."""
import torch

from zipage_amd import _lib

_MODES = {"max": 0, "avg": 1}
MAX_ROW_TOKENS = 150 * 1024 // 8  # one row is staged twice in LDS as 32-bit words


def select_topk(scores: torch.Tensor, block_table: torch.Tensor, compressed: torch.Tensor, k: int,
                *, pooling_size: int = 0, continues_pooling: bool = False,
                pooling_mode: str = "max", redundancy: torch.Tensor | None = None,
                max_norm_red: bool = False, redudancy_lambda: float = 0.0, sink_len: int = 0,
                window: int = 0, mask_pad: bool = True, return_scores: bool = False):
    """Keep flag (L, B, Hkv, NB, BS) bool with exactly ``k`` True per (layer, sequence, head):
    the result of ``pool_scores`` (when ``pooling_size > 1``), ``score_epilogue`` and
    ``topk_mask`` applied in that order, bit for bit.  ``scores`` is left untouched;
    ``return_scores=True`` also returns the post-processed scores."""
    L, B, Hkv, NB, BS = scores.shape
    assert scores.is_contiguous() and block_table.is_contiguous()
    assert block_table.shape == (B, NB) and block_table.dtype == torch.int32
    assert compressed.dtype == torch.bool and compressed.shape == (B,)
    if redundancy is not None:
        assert redundancy.shape == scores.shape and redundancy.dtype == scores.dtype
        assert redundancy.is_contiguous()
    if not 0 <= k <= NB * BS:
        raise RuntimeError(f"selected index k out of range: k={k}, row length {NB * BS}")
    flag = torch.empty(scores.shape, device=scores.device, dtype=torch.bool)
    out = torch.empty_like(scores) if return_scores else None
    if flag.numel() == 0:
        return (flag, out) if return_scores else flag
    _lib.call("zp_select_topk", _lib.dev_ptr(scores), _lib.dev_ptr(out), _lib.dev_ptr(redundancy),
              _lib.dev_ptr(flag), _lib.dev_ptr(block_table), _lib.dev_ptr(compressed.contiguous()),
              L, B, NB, BS, Hkv, int(pooling_size), int(continues_pooling), _MODES[pooling_mode],
              int(max_norm_red), float(redudancy_lambda), int(sink_len), int(window),
              int(mask_pad), int(k), _lib.dtype_tag(scores), _lib.stream_ptr(scores))
    return (flag, out) if return_scores else flag
