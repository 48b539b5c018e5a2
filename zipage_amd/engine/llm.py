"""The generation loop (zipage/engine/zipage_engine.py): schedule, compress what reached its
budget, run the model step, hand tokens back.

`step` compresses in line with the decode steps (zipage_engine.py:99-135).  `async_step`
(zipage_engine.py:137-185) launches the compression on a side stream and lets the sequences
under compression sit the step out; instead of a worker thread blocking on the stream, two
events order the streams: the compression waits for the decode steps already queued (they may
still write the pages it reads), and the first decode step that includes the compressed
sequences again waits for the compression's end event.
"""
from __future__ import annotations

from time import perf_counter

import torch

from .config import EngineConfig
from .model_runner import ModelRunner
from .scheduler import Scheduler
from .sequence import SamplingParams, Sequence


class ZipageEngine:
    def __init__(self, cfg: EngineConfig, device="cuda:0"):
        self.cfg = cfg
        self.runner = ModelRunner(cfg, device)
        self.scheduler = Scheduler(cfg)
        self.stats = dict(prefill_s=0.0, decode_s=0.0, decode_tokens=0, decode_steps=0,
                          prefill_tokens=0, compress_calls=0, compress_seqs=0)
        self._inflight: tuple[torch.cuda.Event, list[Sequence]] | None = None
        self._pending_fetch: list[tuple[Sequence, torch.Tensor]] = []

    # ------------------------------------------------------------------ requests
    def add_request(self, token_ids: list[int], params: SamplingParams | None = None) -> Sequence:
        seq = Sequence(token_ids, params or SamplingParams(), self.cfg.kvcache_block_size)
        cfg = self.cfg
        if not 0 < len(seq) <= min(cfg.max_num_batched_tokens, cfg.max_model_len):
            raise ValueError(f"prompt of {len(seq)} tokens: need 1..{min(cfg.max_num_batched_tokens, cfg.max_model_len)}")
        if seq.num_blocks > cfg.num_kvcache_blocks:
            raise ValueError(f"prompt needs {seq.num_blocks} pages, the pool has {cfg.num_kvcache_blocks}")
        self.runner.reserve_token_log(seq.params.max_tokens + 1)
        self.scheduler.add(seq)
        return seq

    def is_finished(self) -> bool:
        return self.scheduler.is_finished()

    # ------------------------------------------------------------------ steps
    def _needs_host_tokens(self, seqs: list[Sequence]) -> bool:
        return any(not s.params.ignore_eos for s in seqs)

    def _finish_step(self, seqs: list[Sequence], tok: torch.Tensor):
        ids = tok.tolist() if self._needs_host_tokens(seqs) else None
        self.scheduler.postprocess(seqs, ids, advance=True)
        for s in seqs:
            if s.finished:
                self._pending_fetch.append((s, self.runner.fetch_tokens(s)))

    def step(self) -> int:
        """One scheduler round; returns +prefilled tokens or -decoded tokens."""
        seqs, is_prefill = self.scheduler.schedule()
        if not seqs:
            return 0
        if is_prefill:
            self._finish_step(seqs, self.runner.run_prefill(seqs))
            n = sum(len(s) for s in seqs)
            self.stats["prefill_tokens"] += n
            return n
        todo = [s for s in seqs if s.require_compress]
        if todo:
            self.runner.compress(todo)
            self.scheduler.postprocess(todo)
            self.stats["compress_calls"] += 1
            self.stats["compress_seqs"] += len(todo)
        self._finish_step(seqs, self.runner.run_decode(seqs))
        self.stats["decode_tokens"] += len(seqs)
        self.stats["decode_steps"] += 1
        return -len(seqs)

    def async_step(self) -> int:
        r = self.runner
        if self._inflight is not None and self._inflight[0].query():
            ev, done = self._inflight
            r.run_stream.wait_event(ev)           # their next decode step reads the new pages
            self.scheduler.postprocess(done)
            self._inflight = None
        seqs, is_prefill = self.scheduler.schedule()
        if not seqs:
            if self._inflight is not None:        # everything left is under compression
                self._inflight[0].synchronize()
            return 0
        if is_prefill:
            self._finish_step(seqs, r.run_prefill(seqs))
            n = sum(len(s) for s in seqs)
            self.stats["prefill_tokens"] += n
            return n
        busy = set(id(s) for s in self._inflight[1]) if self._inflight else set()
        todo = [s for s in seqs if s.require_compress and id(s) not in busy]
        run = [s for s in seqs if not s.require_compress]
        if todo and self._inflight is None:
            widest = max(len(s.block_table) for s in todo)
            todo = todo[:max(self.cfg.max_compress_blocks // widest, 1)]
            gate = torch.cuda.Event()
            gate.record(r.run_stream)             # decode steps queued so far wrote these pages
            r.compress_stream.wait_event(gate)
            ev = r.compress(todo, stream=r.compress_stream)
            self._inflight = (ev, todo)
            self.stats["compress_calls"] += 1
            self.stats["compress_seqs"] += len(todo)
        if run:
            self._finish_step(run, r.run_decode(run))
            self.stats["decode_tokens"] += len(run)
            self.stats["decode_steps"] += 1
        elif self._inflight is not None:
            self._inflight[0].synchronize()
        return -len(run)

    # ------------------------------------------------------------------ generate
    def generate(self, prompts: list[list[int]], params: SamplingParams | list[SamplingParams]):
        """Run all prompts to completion; returns one dict per prompt with `token_ids`, and
        fills `self.stats` (decode tokens/s counts decode steps only, as the reference's
        progress line does: zipage_engine.py:247-262)."""
        if not isinstance(params, list):
            params = [params] * len(prompts)
        seqs = [self.add_request(p, sp) for p, sp in zip(prompts, params)]
        step = self.async_step if self.cfg.enable_async_compress else self.step
        dev = self.runner.device
        idle = 0
        while not self.is_finished():
            t0 = perf_counter()
            n = step()
            idle = idle + 1 if n == 0 else 0
            if idle > 10000:
                raise RuntimeError("scheduler stalled: no sequence can get a page or a query row "
                                   f"({self.scheduler.pool.num_free} pages free)")
            if n > 0:
                torch.cuda.synchronize(dev)       # prefill is timed on its own
                self.stats["prefill_s"] += perf_counter() - t0
            elif self.stats["decode_steps"] == 1 and n < 0:
                self._t_decode0 = t0
        torch.cuda.synchronize(dev)
        if self.stats["decode_steps"]:
            self.stats["decode_s"] = perf_counter() - self._t_decode0
        self.stats["compress_s"] = self.runner.compress_seconds()
        for seq, host in self._pending_fetch:
            seq.token_ids = seq.token_ids[:seq.num_prompt_tokens] + host.tolist()
        self._pending_fetch.clear()
        return [dict(token_ids=s.completion_token_ids, request_id=s.request_id,
                     num_compressions=s.num_compressions) for s in seqs]
