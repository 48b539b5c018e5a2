from .attention import paged_decode_attention, store_kvcache  # noqa: F401
from .fused import qk_norm_rope_store, rms_norm, silu_and_mul  # noqa: F401
