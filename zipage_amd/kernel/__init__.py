"""MI355X kernels behind the call signatures of the reference's ``zipage/kernel`` package
(imported at zipage/engine/model_runner.py:19-26 and zipage/layers/attention.py:8)."""
from zipage_amd.kernel.store_query_cache import store_query_cache
from zipage_amd.kernel.attention_score import attention_score
from zipage_amd.kernel.global_score import global_score
from zipage_amd.kernel.window_mask import window_mask, score_epilogue
from zipage_amd.kernel.key_norm import key_norm
from zipage_amd.kernel.lightning_redudancy_score import lightning_redudancy_score
from zipage_amd.kernel.raw_redudancy_score import raw_redudancy_score
from zipage_amd.kernel.utils import topk_mask
from zipage_amd.kernel.compress_kv import compress_kv
from zipage_amd.kernel.compress_score import compress_score
from zipage_amd.kernel.pooling import pool_scores
from zipage_amd.kernel.select import select_topk

__all__ = [
    "store_query_cache", "attention_score", "global_score", "window_mask", "score_epilogue",
    "key_norm", "lightning_redudancy_score", "raw_redudancy_score", "topk_mask", "compress_kv",
    "compress_score", "pool_scores", "select_topk",
]
