"""Engine switches (zipage/config.py) without the Hugging Face lookup: the model shape is
given directly because weights are random-initialised."""
from __future__ import annotations

from dataclasses import dataclass, field

from zipage_amd.compress import CompressConfig

from .qwen3 import QWEN3_8B, Qwen3Shape


@dataclass
class EngineConfig:
    shape: Qwen3Shape = QWEN3_8B
    max_num_batched_tokens: int = 32768
    max_num_seqs: int = 512
    max_concurrency: int = 256          # query-cache rows = sequences resident at once
    max_model_len: int = 8192
    eos: int = -1
    kvcache_block_size: int = 256
    num_kvcache_blocks: int = 2560
    max_cache_blocks_per_seq: int = 8   # the budget; tables hold one page more
    query_cache_len: int = 16
    layer_stride: int = 8               # layers per compression launch (model_runner.py:466)
    enable_async_compress: bool = False
    max_compress_blocks: int = 4096     # pages one asynchronous compression may cover
    enable_prefix_cache: bool = False
    use_graph: bool = True              # replay the decode step as a HIP graph
    seed: int = 0
    compress: CompressConfig = field(default_factory=CompressConfig)

    def __post_init__(self):
        assert self.kvcache_block_size % 256 == 0 or self.kvcache_block_size in (16, 32, 64, 128)
        assert self.max_cache_blocks_per_seq >= 1
        self.compress.budget_blocks = self.max_cache_blocks_per_seq
        self.compress.query_cache_len = self.query_cache_len
