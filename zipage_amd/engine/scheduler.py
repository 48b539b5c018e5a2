"""Admission, decode scheduling and the hand-back after a step (zipage/engine/scheduler.py).

Two simplifications against the reference, both outside the compression path: every resident
sequence owns a query-cache row (no hybrid mode with row-less sequences), and a sequence that
cannot get a page is suspended or, with prefix caching on, makes room by preempting the
youngest uncompressed one.
"""
from __future__ import annotations

import time
from collections import deque

from .config import EngineConfig
from .pages import PagePool
from .sequence import Sequence


class Scheduler:
    def __init__(self, cfg: EngineConfig):
        self.cfg = cfg
        self.pool = PagePool(cfg.num_kvcache_blocks, cfg.kvcache_block_size,
                             cfg.max_cache_blocks_per_seq + 1, cfg.enable_prefix_cache)
        self.waiting: deque[Sequence] = deque()
        self.running: deque[Sequence] = deque()
        self.free_rows: deque[int] = deque(range(cfg.max_concurrency))

    def add(self, seq: Sequence):
        self.waiting.append(seq)

    def is_finished(self) -> bool:
        return not self.waiting and not self.running

    # ------------------------------------------------------------------ schedule
    def schedule(self) -> tuple[list[Sequence], bool]:
        cfg = self.cfg
        prefill, budget = [], 0
        while self.waiting and len(prefill) < cfg.max_num_seqs and self.free_rows:
            seq = self.waiting[0]
            if budget + len(seq) > cfg.max_num_batched_tokens or not self.pool.can_admit(seq):
                break
            seq.query_id = self.free_rows.popleft()
            self.pool.admit(seq)
            self.waiting.popleft()
            self.running.append(seq)
            if seq.num_cached_tokens != len(seq):
                budget += len(seq) - seq.num_cached_tokens
                prefill.append(seq)
        if prefill:
            return prefill, True

        kept, batch = [], []
        while self.running and len(batch) < cfg.max_num_seqs:
            seq = self.running.popleft()
            rejoin = []
            ok = True
            while not self.pool.can_append_or_compress(seq):
                if self.running and cfg.enable_prefix_cache:
                    victim = self.running.pop()
                    if victim.compressed or victim.require_compress:
                        rejoin.append(victim)
                    else:
                        self.preempt(victim)
                else:
                    ok = False          # suspended for this step
                    break
            kept.append(seq)
            if ok:
                self.pool.append(seq)
                batch.append(seq)
            self.running.extend(reversed(rejoin))
        self.running.extendleft(reversed(kept))
        return batch, False

    def preempt(self, seq: Sequence):
        assert not seq.compressed and not seq.require_compress
        self.free_rows.append(seq.query_id)
        seq.query_id = -1
        self.pool.release(seq)
        self.waiting.appendleft(seq)

    # ------------------------------------------------------------------ hand-back
    def postprocess(self, seqs: list[Sequence], token_ids: list[int] | None = None,
                    advance: bool = False):
        """After a compression (`token_ids` None, `advance` False): swap tables.  After a model
        step: append the token (its value may stay on the device: `advance` without ids) and
        retire finished sequences (scheduler.py:141-167)."""
        for i, seq in enumerate(seqs):
            if seq.require_compress:
                self.pool.commit_compression(seq)
            if token_ids is None and not advance:
                continue
            tok = token_ids[i] if token_ids is not None else None
            seq.advance(tok)
            hit_eos = tok is not None and not seq.params.ignore_eos and tok == self.cfg.eos
            if hit_eos or seq.num_completion_tokens >= seq.params.max_tokens:
                seq.finished = True
                seq.time_finished = time.time()
                self.pool.release(seq)
                self.running.remove(seq)
                self.free_rows.append(seq.query_id)
