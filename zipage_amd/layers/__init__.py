from .attention import paged_decode_attention, store_kvcache  # noqa: F401
