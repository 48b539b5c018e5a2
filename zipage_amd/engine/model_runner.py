"""Device side of the engine: caches, step inputs, the model step, and the compression call
(zipage/engine/model_runner.py).

What differs from the reference by design:
  * sampled tokens stay on the device (`last_token`, `token_log` indexed by query row), so a
    fixed-length greedy run never synchronises with the host inside the decode loop;
  * step inputs travel as ONE packed int32 buffer (pinned ring -> device), and the decode step
    itself is replayed as a HIP graph over static buffers;
  * compression is launched on a side stream with event hand-off in both directions instead of a
    worker thread that blocks on a stream synchronise.
"""
from __future__ import annotations

import numpy as np
import torch

from zipage_amd.compress import StageTimer, compress_layers

from .config import EngineConfig
from .inputs import encode_compress_tables, pack_decode, packed_words, query_slot_mapping, unpack_views
from .qwen3 import Qwen3, StepContext
from .sequence import Sequence


class _PinnedRing:
    """Pinned staging buffers reused round-robin; a slot is rewritten only after the copy that
    read it has completed."""

    def __init__(self, words: int, depth: int = 8):
        self.bufs = [torch.empty(words, dtype=torch.int32, pin_memory=True) for _ in range(depth)]
        self.events: list[torch.cuda.Event | None] = [None] * depth
        self.i = 0

    def next(self) -> tuple[torch.Tensor, int]:
        i = self.i
        self.i = (i + 1) % len(self.bufs)
        if self.events[i] is not None:
            self.events[i].synchronize()
        return self.bufs[i], i

    def sent(self, i: int, stream):
        ev = torch.cuda.Event()
        ev.record(stream)
        self.events[i] = ev


class ModelRunner:
    def __init__(self, cfg: EngineConfig, device="cuda:0"):
        self.cfg, self.device = cfg, torch.device(device)
        torch.cuda.set_device(self.device)
        s = cfg.shape
        self.block_size = cfg.kvcache_block_size
        self.table_width = cfg.max_cache_blocks_per_seq + 1
        self.model = Qwen3(s, self.device, seed=cfg.seed)
        self.allocate_kv_cache()
        self.run_stream = torch.cuda.Stream(self.device)
        self.compress_stream = torch.cuda.Stream(self.device)
        R = cfg.max_concurrency
        # row R is a scratch row: the inert entries that pad a batch read and write it
        self.last_token = torch.zeros(R + 1, dtype=torch.int64, device=self.device)
        self.token_log = torch.zeros(R + 1, 1, dtype=torch.int32, device=self.device)
        self.time_record: dict[str, float] = {}
        self._compress_spans: list[tuple[torch.cuda.Event, torch.cuda.Event]] = []
        self._graphs: dict[tuple[int, int], tuple] = {}
        # packed decode inputs: 5 header rows, tables, query triples
        widest = max(self.table_width, -(-cfg.max_model_len // self.block_size) + 1)
        self.ring = _PinnedRing(packed_words(self._graph_batch(R) + 16, widest))

    # ------------------------------------------------------------------ memory
    def allocate_kv_cache(self):
        """model_runner.py:219-307, with the page count given by the configuration."""
        cfg, s = self.cfg, self.cfg.shape
        dt = self.model.dtype
        self.kv_cache = torch.zeros(2, s.layers, cfg.num_kvcache_blocks, self.block_size, s.kv_heads,
                                    s.head_dim, dtype=dt, device=self.device)
        self.query_cache = torch.zeros(s.layers, cfg.max_concurrency, cfg.query_cache_len, s.heads,
                                       s.head_dim, dtype=dt, device=self.device)
        self.score_cache = None
        if cfg.compress.use_global_score:
            self.score_cache = torch.zeros(s.layers, cfg.num_kvcache_blocks, self.block_size,
                                           s.kv_heads, dtype=dt, device=self.device)
        self.model.attach_caches(self.kv_cache, self.query_cache)

    def reserve_token_log(self, max_tokens: int):
        if self.token_log.shape[1] < max_tokens:
            old = self.token_log
            with torch.cuda.stream(self.run_stream):   # ordered after the steps that wrote `old`
                self.token_log = torch.zeros(self.cfg.max_concurrency + 1, max_tokens,
                                             dtype=torch.int32, device=self.device)
                self.token_log[:, :old.shape[1]] = old
            self._graphs.clear()

    # ------------------------------------------------------------------ step inputs
    def get_query_slot_mapping(self, seq: Sequence, is_prefill=False, cu_len=0, seqlen_q=0):
        return query_slot_mapping(seq, self.block_size, self.cfg.query_cache_len, is_prefill,
                                  cu_len, seqlen_q)

    def prepare_prefill(self, seqs: list[Sequence]):
        """model_runner.py:352-422."""
        BS = self.block_size
        ids, pos, slots, qmap, lens_q, lens_k = [], [], [], [], [], []
        cu = 0
        for seq in seqs:
            n, cached = len(seq), seq.num_cached_tokens
            ids.extend(seq.token_ids[cached:n])
            pos.extend(range(cached, n))
            qmap.extend(self.get_query_slot_mapping(seq, True, cu_len=cu, seqlen_q=n - cached))
            lens_q.append(n - cached)
            lens_k.append(n)
            cu += n - cached
            for i in range(cached // BS, seq.num_blocks):
                start = seq.block_table[i] * BS
                count = BS if i != seq.num_blocks - 1 else seq.last_block_num_tokens
                slots.extend(range(start, start + count))
            seq.num_cached_tokens = n
        dev = self.device
        t = lambda a, dt: torch.tensor(a, dtype=dt, pin_memory=True).to(dev, non_blocking=True)
        tables = None
        if lens_q != lens_k:
            width = max(len(s.block_table) for s in seqs)
            tables = t([s.block_table + [-1] * (width - len(s.block_table)) for s in seqs], torch.int32)
        ctx = StepContext(True, t(slots, torch.int32),
                          t(qmap, torch.int32) if qmap else None, None, tables, lens_q, lens_k)
        return t(ids, torch.int64), t(pos, torch.int64), ctx

    def _pack_decode(self, seqs: list[Sequence], Bp: int, TW: int) -> np.ndarray:
        return pack_decode(seqs, Bp, self.block_size, self.cfg.query_cache_len, TW,
                           self.cfg.max_concurrency)

    # ------------------------------------------------------------------ model step
    def _sample(self, logits: torch.Tensor, temperatures: torch.Tensor | None) -> torch.Tensor:
        """Greedy where the temperature is 0, else the exponential-race draw of
        zipage/layers/sampler.py:17-33."""
        greedy = logits.argmax(dim=-1)
        if temperatures is None:
            return greedy
        t = temperatures.clamp_min(1e-6).unsqueeze(1)
        probs = torch.softmax(logits.float() / t, dim=-1)
        drawn = probs.div_(torch.empty_like(probs).exponential_(1).clamp_min_(1e-10)).argmax(dim=-1)
        return torch.where(temperatures > 0, drawn, greedy)

    def _decode_hidden(self, buf: torch.Tensor, Bp: int, TW: int) -> torch.Tensor:
        """The part of the step a graph replays: embedding to final norm."""
        head, tables, triples = unpack_views(buf, Bp, TW)
        ctx = StepContext(False, head[2], triples, head[3], tables)
        return self.model.forward(self.last_token[head[0].long()], head[1].long(), ctx)

    def _decode_tail(self, buf: torch.Tensor, Bp: int, TW: int, hidden: torch.Tensor,
                     temperatures=None):
        """Vocabulary projection, sampling and the device-side token hand-over.  Kept out of the
        graph: wide reductions of the tensor library may record memset nodes."""
        head, _, _ = unpack_views(buf, Bp, TW)
        rows, cols = head[0].long(), head[4].long()
        tok = self._sample(self.model.compute_logits(hidden), temperatures)
        self.last_token.index_put_((rows,), tok)
        self.token_log.index_put_((rows, cols), tok.int())
        return tok

    @torch.inference_mode()
    def run_prefill(self, seqs: list[Sequence]) -> torch.Tensor:
        with torch.cuda.stream(self.run_stream):
            ids, pos, ctx = self.prepare_prefill(seqs)
            hidden = self.model.forward(ids, pos, ctx)
            ends = torch.tensor(np.cumsum(ctx.seq_lens_q) - 1, device=self.device)
            temps = [s.params.temperature for s in seqs]
            temps = torch.tensor(temps, device=self.device) if any(temps) else None
            tok = self._sample(self.model.compute_logits(hidden[ends]), temps)
            rows = torch.tensor([s.query_id for s in seqs], device=self.device)
            cols = torch.tensor([s.num_completion_tokens for s in seqs], device=self.device)
            self.last_token[rows] = tok
            self.token_log[rows, cols] = tok.int()
        return tok

    @torch.inference_mode()
    def run_decode(self, seqs: list[Sequence]) -> torch.Tensor:
        """One decode step for `seqs`; returns the device tensor of the sampled ids."""
        B = len(seqs)
        temps = [s.params.temperature for s in seqs]
        graph = self.cfg.use_graph and not any(temps)
        Bp = self._graph_batch(B)      # eager steps pad the same way, so both paths run the same kernels
        # a prompt longer than the table keeps its pages until its first compression
        TW = max(self.table_width, max(len(s.block_table) for s in seqs))
        packed = self._pack_decode(seqs, Bp, TW)
        words = packed.shape[0]
        pinned, slot = self.ring.next()
        pinned[:words].numpy()[:] = packed
        with torch.cuda.stream(self.run_stream):
            t = torch.tensor(temps + [0.0] * (Bp - B), device=self.device) if any(temps) else None
            if graph:
                g, sbuf, hidden = self._graph(Bp, TW)
                sbuf.copy_(pinned[:words], non_blocking=True)
                self.ring.sent(slot, self.run_stream)
                g.replay()
                return self._decode_tail(sbuf, Bp, TW, hidden)[:B]
            buf = pinned[:words].to(self.device, non_blocking=True)
            self.ring.sent(slot, self.run_stream)
            return self._decode_tail(buf, Bp, TW, self._decode_hidden(buf, Bp, TW), t)[:B]

    # ------------------------------------------------------------------ HIP graph
    def _graph_batch(self, B: int) -> int:
        for cap in (1, 2, 4, 8):
            if B <= cap:
                return cap
        return -(-B // 16) * 16

    def _graph(self, Bp: int, TW: int):
        """Capture the decode step for a padded batch of Bp (tables TW wide) once; later steps
        replay it."""
        if (Bp, TW) in self._graphs:
            return self._graphs[(Bp, TW)]
        sbuf = torch.zeros(packed_words(Bp, TW), dtype=torch.int32, device=self.device)
        sbuf[:Bp] = self.cfg.max_concurrency          # all entries inert for the warm-up runs
        sbuf[2 * Bp:3 * Bp] = -1
        sbuf[5 * Bp:] = -1                          # tables and triples
        for _ in range(2):                            # lazy initialisations happen outside capture
            self._decode_hidden(sbuf, Bp, TW)
        torch.cuda.current_stream().synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=torch.cuda.current_stream()):
            out = self._decode_hidden(sbuf, Bp, TW)
        self._graphs[(Bp, TW)] = (g, sbuf, out)
        return self._graphs[(Bp, TW)]

    # ------------------------------------------------------------------ compression
    @torch.inference_mode()
    def compress(self, seqs: list[Sequence], stream: torch.cuda.Stream | None = None,
                 timer: StageTimer | None = None) -> torch.cuda.Event:
        """Score, select and compact `seqs` in place, `layer_stride` layers per launch
        (model_runner.py:424-631).  Runs on `stream` (default: the run stream, i.e. in line
        with the decode steps) and returns the event that marks its end; nothing blocks."""
        stream = stream or self.run_stream
        cfg = self.cfg
        enc = encode_compress_tables(seqs)
        t = lambda a, dt: torch.tensor(a, dtype=dt, pin_memory=True).to(self.device, non_blocking=True)
        with torch.cuda.stream(stream):
            st = torch.cuda.Event(enable_timing=True)
            ed = torch.cuda.Event(enable_timing=True)
            st.record(stream)
            query_ids = t([s.query_id for s in seqs], torch.int32)
            compressed = t([s.compressed for s in seqs], torch.bool)
            targets = t([s.new_block_table for s in seqs], torch.int32)
            tables = t(enc, torch.int32)
            L = cfg.shape.layers
            for l0 in range(0, L, cfg.layer_stride):
                l1 = min(L, l0 + cfg.layer_stride)
                compress_layers(self.kv_cache[0, l0:l1], self.kv_cache[1, l0:l1],
                                self.query_cache[l0:l1],
                                None if self.score_cache is None else self.score_cache[l0:l1],
                                query_ids, tables, compressed, targets, cfg.compress, timer=timer)
            ed.record(stream)
        self._compress_spans.append((st, ed))
        return ed

    def compress_seconds(self) -> float:
        """Device time spent in compression so far; call after a synchronise."""
        return sum(st.elapsed_time(ed) for st, ed in self._compress_spans) / 1000.0

    def fetch_tokens(self, seq: Sequence) -> torch.Tensor:
        """Queue the copy of a finished sequence's generated ids to pinned host memory."""
        n = seq.num_completion_tokens
        host = torch.empty(n, dtype=torch.int32, pin_memory=True)
        with torch.cuda.stream(self.run_stream):
            host.copy_(self.token_log[seq.query_id, :n], non_blocking=True)
        return host
