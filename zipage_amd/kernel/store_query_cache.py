"""Drop-in for zipage/kernel/store_query_cache.py:35-68."""
import torch

from zipage_amd import _lib


def store_query_cache(query: torch.Tensor, query_cache: torch.Tensor, slot_mapping: torch.Tensor):
    """Store query rows into the per-sequence window ring.

    query: (L, num_heads, head_dim); query_cache: (max_num_seqs, query_cache_len, num_heads,
    head_dim); slot_mapping: (N, 3) int32 triples (row of query, sequence slot, ring slot).
    Same contract as the reference: no-op on an empty cache (warm-up), the same three
    stride asserts, mutates ``query_cache`` in place, returns None.
    """
    N = slot_mapping.shape[0]
    _, num_heads, head_dim = query.shape
    D = num_heads * head_dim
    if query_cache.numel() == 0 or N == 0:  # warmup, or nothing to store
        return
    assert query.stride(-1) == 1
    assert query.stride(1) == head_dim
    assert query_cache.stride(1) == D
    assert slot_mapping.dtype == torch.int32
    assert query.dtype == query_cache.dtype
    _lib.call("zp_store_query", _lib.dev_ptr(query), _lib.dev_ptr(query_cache),
              _lib.dev_ptr(slot_mapping), N, D, query.shape[0], query_cache.shape[0],
              query_cache.shape[1], query.stride(0), query_cache.stride(0),
              query_cache.stride(1), slot_mapping.stride(0), slot_mapping.stride(1),
              _lib.dtype_tag(query), _lib.stream_ptr(query))
