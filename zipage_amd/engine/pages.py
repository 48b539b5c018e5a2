"""Refcounted page allocator with prefix sharing and the compression target rule
(zipage/engine/block_manager.py).

State is kept in flat arrays (refcount, chain hash per page) plus a free deque, so the GPU-side
tables and this bookkeeping index pages the same way.  Sharing is by a chained xxh64 of each full
page of prompt tokens; a page that more than one table holds is read-only, which is what makes
the copy-on-write rule of `plan_compression` necessary.
"""
from __future__ import annotations

import threading
from collections import deque

import numpy as np
import xxhash

from .sequence import Sequence


class PagePool:
    def __init__(self, num_pages: int, page_size: int, pages_per_seq: int,
                 enable_prefix_cache: bool = False):
        """`pages_per_seq` = budget pages + 1 (the page new tokens are written to)."""
        self.num_pages, self.page_size, self.pages_per_seq = num_pages, page_size, pages_per_seq
        self.enable_prefix_cache = enable_prefix_cache
        self.refcount = np.zeros(num_pages, dtype=np.int32)
        self.page_hash: list[int] = [-1] * num_pages
        self.page_tokens: list[list[int] | None] = [None] * num_pages
        self.by_hash: dict[int, int] = {}
        self.free: deque[int] = deque(range(num_pages))
        self.lock = threading.Lock()     # compression hand-back may run on a worker thread

    # ------------------------------------------------------------------ primitives
    @staticmethod
    def chain_hash(token_ids: list[int], prefix: int = -1) -> int:
        """zipage/engine/block_manager.py:45-51: xxh64 over the parent hash and the page's ids."""
        h = xxhash.xxh64()
        if prefix != -1:
            h.update(prefix.to_bytes(8, "little"))
        h.update(np.array(token_ids).tobytes())
        return h.intdigest()

    @property
    def num_free(self) -> int:
        return len(self.free)

    @property
    def occupancy(self) -> float:
        return 1.0 - len(self.free) / self.num_pages

    def _take(self, page: int | None = None) -> int:
        with self.lock:
            if page is None:
                page = self.free.popleft()
            else:
                self.free.remove(page)
            assert self.refcount[page] == 0
            self.refcount[page] = 1
            self.page_hash[page] = -1
            self.page_tokens[page] = None
        return page

    def _drop(self, page: int):
        with self.lock:
            self.refcount[page] -= 1
            assert self.refcount[page] >= 0
            if self.refcount[page] == 0:
                self.free.append(page)

    def _own(self, page: int):
        """A page that is about to be rewritten loses its shareable identity."""
        self.refcount[page] = 1
        self.page_hash[page] = -1
        self.page_tokens[page] = None

    # ------------------------------------------------------------------ prompt admission
    def can_admit(self, seq: Sequence) -> bool:
        return self.num_free >= seq.num_blocks

    def admit(self, seq: Sequence):
        """Pages for a prompt; leading full pages already cached under the same chain hash are
        shared (block_manager.py:78-112).  The last page of a prompt is never shared: a prompt
        whose every page hits would skip prefill altogether, and the first decode step needs the
        last prompt token run through the model (and, when the prompt fills a whole table, the
        window queries of that page captured)."""
        assert not seq.block_table
        h, miss = -1, False
        for i in range(seq.num_blocks):
            toks = seq.block(i)
            full = len(toks) == self.page_size and self.enable_prefix_cache
            h = self.chain_hash(toks, h) if full else -1
            page = self.by_hash.get(h, -1)
            if page == -1 or self.page_tokens[page] != toks or i == seq.num_blocks - 1:
                miss = True
            if miss:
                page = self._take()
            else:
                seq.num_cached_tokens += self.page_size
                if self.refcount[page] > 0:
                    self.refcount[page] += 1
                else:
                    self._take(page)
            if h != -1:
                self.page_hash[page], self.page_tokens[page] = h, toks
                self.by_hash[h] = page
            seq.block_table.append(page)

    def release(self, seq: Sequence):
        for page in reversed(seq.block_table):
            self._drop(page)
        seq.block_table.clear()
        seq.num_cached_tokens = 0

    # ------------------------------------------------------------------ decode growth
    def wants_page(self, seq: Sequence) -> bool:
        """True on the step whose token opens a new page."""
        return (seq.num_tokens % self.page_size == 1
                and seq.num_cached_tokens > self.page_size * len(seq.block_table))

    def can_append_or_compress(self, seq: Sequence) -> bool:
        """block_manager.py:158-171."""
        if seq.require_compress:
            return True              # compression in flight: this step is skipped for it
        if self.wants_page(seq):
            if len(seq.block_table) < self.pages_per_seq:
                return self.num_free > 0
            return self.plan_compression(seq)
        return True

    def append(self, seq: Sequence):
        """block_manager.py:176-210."""
        if seq.require_compress:
            return
        if self.wants_page(seq):
            seq.block_table.append(self._take())
        elif seq.num_tokens % self.page_size == 0 and not seq.compressed and self.enable_prefix_cache \
                and len(seq.token_ids) == seq.num_tokens:
            last = seq.block_table[-1]
            toks = seq.block(seq.num_blocks - 1)
            parent = self.page_hash[seq.block_table[-2]] if len(seq.block_table) > 1 else -1
            h = self.chain_hash(toks, parent)
            self.page_hash[last], self.page_tokens[last] = h, toks
            self.by_hash[h] = last

    # ------------------------------------------------------------------ compression
    def plan_compression(self, seq: Sequence) -> bool:
        """Choose the pages the survivors are written to (block_manager.py:125-156).

        A sequence compressed before owns all its pages: it keeps its table.  Otherwise the
        leading pages other tables also hold are read-only sources: as many fresh pages as there
        are shared ones (at most the budget) head the target, the sequence's own pages follow,
        and everything that is not in the target is released after the kernel ran.
        """
        cap = self.pages_per_seq
        table = seq.block_table
        if seq.compressed:
            seq.new_block_table = table[:cap]
            seq.block_to_release = table[cap:]
        else:
            shared = 0
            for page in table:
                if self.refcount[page] > 1:
                    shared += 1
                else:
                    break
            assert len(table) - shared >= 1
            fresh = min(shared, cap - 1)
            if fresh > self.num_free:
                return False
            own = table[shared:shared + cap - fresh]
            seq.new_block_table = [self._take() for _ in range(fresh)] + own
            assert len(seq.new_block_table) == cap
            seq.block_to_release = table[:shared] + table[shared + cap - fresh:]
            for page in own:
                self._own(page)
        seq.require_compress = True
        return True

    def commit_compression(self, seq: Sequence):
        """After the kernels ran: release the sources, swap the table
        (scheduler.py:149-156)."""
        for page in reversed(seq.block_to_release):
            self._drop(page)
        seq.block_to_release = []
        seq.block_table, seq.new_block_table = seq.new_block_table, []
        seq.num_cached_tokens = (len(seq.block_table) - 1) * self.page_size + 1
        seq.compressed = True
        seq.require_compress = False
        seq.num_compressions += 1
