"""Cache-side pieces of the attention layer around the compression path
(zipage/layers/attention.py): the K/V scatter and the decode-time attention over pages."""
import torch

from zipage_amd import _lib


def store_kvcache(key: torch.Tensor, value: torch.Tensor, k_cache: torch.Tensor,
                  v_cache: torch.Tensor, slot_mapping: torch.Tensor):
    """Drop-in for zipage/layers/attention.py:33-50.

    key, value: (N, num_kv_heads, head_dim); k_cache, v_cache: one layer's
    (num_pages, block_size, num_kv_heads, head_dim); slot_mapping: (N,) int32 flat slot
    (page * block_size + offset), -1 skips the token.  Same asserts as the reference.
    """
    N, num_heads, head_dim = key.shape
    D = num_heads * head_dim
    assert key.stride(-1) == 1 and value.stride(-1) == 1
    assert key.stride(1) == head_dim and value.stride(1) == head_dim
    assert k_cache.stride(1) == D and v_cache.stride(1) == D
    assert slot_mapping.numel() == N
    assert slot_mapping.dtype == torch.int32
    assert key.dtype == k_cache.dtype == value.dtype == v_cache.dtype
    _lib.call("zp_store_kvcache", _lib.dev_ptr(key), _lib.dev_ptr(value), _lib.dev_ptr(k_cache),
              _lib.dev_ptr(v_cache), _lib.dev_ptr(slot_mapping), N, D, key.stride(0),
              value.stride(0), k_cache.shape[0] * k_cache.shape[1], _lib.dtype_tag(key),
              _lib.stream_ptr(key))


def paged_decode_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                           context_lens: torch.Tensor, block_tables: torch.Tensor,
                           softmax_scale: float) -> torch.Tensor:
    """What the decode branch of Attention.forward asks of flash_attn_with_kvcache
    (zipage/layers/attention.py:95-103): for every sequence one query token attends to the
    first context_lens[b] tokens of the pages block_tables[b] lists.

    q: (B, num_heads, head_dim); caches (num_pages, block_size, num_kv_heads, head_dim);
    context_lens (B,) int32; block_tables (B, NB) int32, -1 padded.  Returns (B, num_heads,
    head_dim) in q's dtype.
    """
    B, Hq, D = q.shape
    num_pages, BS, Hkv, _ = k_cache.shape
    assert q.is_contiguous() and k_cache.stride(-1) == 1 and v_cache.stride(-1) == 1
    assert k_cache.stride(2) == D and k_cache.stride(1) == Hkv * D
    assert v_cache.stride(2) == D and v_cache.stride(1) == Hkv * D
    assert block_tables.dtype == torch.int32 and context_lens.dtype == torch.int32
    assert block_tables.is_contiguous() and context_lens.is_contiguous()
    assert q.dtype == k_cache.dtype == v_cache.dtype
    out = torch.empty_like(q)
    _lib.call("zp_paged_decode_attention", _lib.dev_ptr(q), _lib.dev_ptr(k_cache),
              _lib.dev_ptr(v_cache), _lib.dev_ptr(block_tables), _lib.dev_ptr(context_lens),
              _lib.dev_ptr(out), B, Hq, Hkv, D, BS, block_tables.shape[1], num_pages,
              k_cache.stride(0), v_cache.stride(0), float(softmax_scale), _lib.dtype_tag(q),
              _lib.stream_ptr(q))
    return out
