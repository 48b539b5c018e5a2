"""Per-request state the scheduler and the runner share (zipage/engine/sequence.py)."""
from __future__ import annotations

import itertools
import time
from dataclasses import dataclass, field

_ids = itertools.count()


@dataclass
class SamplingParams:
    temperature: float = 0.0       # 0 = greedy
    max_tokens: int = 64
    ignore_eos: bool = False


@dataclass
class Sequence:
    """One request.  Lengths follow the reference: `num_tokens` counts prompt + generated
    tokens, `num_cached_tokens` the tokens whose K/V sit in the pages of `block_table` (after a
    compression: budget pages + the token being decoded)."""
    token_ids: list[int]
    params: SamplingParams = field(default_factory=SamplingParams)
    block_size: int = 256

    def __post_init__(self):
        self.request_id = next(_ids)
        self.token_ids = list(self.token_ids)
        self.num_prompt_tokens = len(self.token_ids)
        self.num_tokens = len(self.token_ids)
        self.num_cached_tokens = 0
        self.block_table: list[int] = []
        self.new_block_table: list[int] = []       # target table of a pending compression
        self.block_to_release: list[int] = []
        self.require_compress = False
        self.compressed = False
        self.num_compressions = 0
        self.query_id = -1
        self.finished = False
        self.device_row = -1                       # row of the runner's device-side token log
        self.time_prefilled = 0.0
        self.time_finished = 0.0

    def __len__(self):
        return self.num_tokens

    @property
    def num_completion_tokens(self) -> int:
        return self.num_tokens - self.num_prompt_tokens

    @property
    def num_blocks(self) -> int:
        return -(-self.num_tokens // self.block_size)

    @property
    def last_block_num_tokens(self) -> int:
        return self.num_tokens - (self.num_blocks - 1) * self.block_size

    @property
    def completion_token_ids(self) -> list[int]:
        return self.token_ids[self.num_prompt_tokens:]

    def block(self, i: int) -> list[int]:
        return self.token_ids[i * self.block_size:(i + 1) * self.block_size]

    def advance(self, token_id: int | None):
        """One decoded token.  `token_id` is None when the value stays on the device (greedy
        fixed-length generation never needs it on the host before the end)."""
        if token_id is not None:
            self.token_ids.append(token_id)
        self.num_tokens += 1
        self.num_cached_tokens += 1
        if self.num_completion_tokens == 1:
            self.time_prefilled = time.time()
