"""Drop-in for zipage/kernel/compress_kv.py:103-141."""
import torch

from zipage_amd import _lib


def compress_kv(key: torch.Tensor, value: torch.Tensor, flag: torch.Tensor,
                block_table: torch.Tensor, target_block_table: torch.Tensor):
    """Stable in-place compaction of the flagged tokens' K and V into the target pages.

    key/value: (L, num_pages, BS, Hkv, D) (any layer/page/slot/head strides, unit head_dim
    stride); flag: (L, B, Hkv, NB, BS) bool; block_table: (B, NB) int32;
    target_block_table: (B, budget+1) int32.  Returns None.
    """
    L, num_pages, BS, Hkv, D = key.shape
    _, B, _, NB, _ = flag.shape
    assert value.shape == key.shape and value.dtype == key.dtype
    assert key.stride(4) == 1 and value.stride(4) == 1
    assert flag.shape == (L, B, Hkv, NB, BS) and flag.dtype == torch.bool and flag.is_contiguous()
    assert block_table.shape == (B, NB) and block_table.is_contiguous()
    assert target_block_table.shape[0] == B and target_block_table.is_contiguous()
    assert block_table.dtype == torch.int32 and target_block_table.dtype == torch.int32
    if flag.numel() == 0:
        return None
    _lib.call("zp_compress_kv", _lib.dev_ptr(key), _lib.dev_ptr(value), _lib.dev_ptr(flag),
              _lib.dev_ptr(block_table), _lib.dev_ptr(target_block_table), L, B, NB, BS, Hkv, D,
              num_pages, target_block_table.shape[1],
              key.stride(0), key.stride(1), key.stride(2), key.stride(3),
              value.stride(0), value.stride(1), value.stride(2), value.stride(3),
              _lib.dtype_tag(key), _lib.stream_ptr(key))
