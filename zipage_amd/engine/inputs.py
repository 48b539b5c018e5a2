"""Host-side construction of a step's index tensors (numpy only, no device needed)."""
from __future__ import annotations

import numpy as np

from .sequence import Sequence

HEADER_ROWS = 5   # query row, position, flat K/V slot, context length, token-log column


def query_slot_mapping(seq: Sequence, block_size: int, query_cache_len: int, is_prefill=False,
                       cu_len=0, seqlen_q=0) -> list[tuple[int, int, int]]:
    """(row of q, query row, ring slot) triples for the tokens that fall into the last
    `query_cache_len` positions of a page (zipage/engine/model_runner.py:319-350)."""
    BS, W = block_size, query_cache_len
    if seq.query_id == -1:
        return []
    if is_prefill:
        pages = -(-seqlen_q // BS)
        if pages == 0:
            return []
        tail = seqlen_q - (pages - 1) * BS
        if tail <= BS - W:
            return []
        first = pages * BS - W
        return [(cu_len + pos, seq.query_id, i) for i, pos in enumerate(range(first, seqlen_q))]
    if seq.last_block_num_tokens > BS - W:
        return [(cu_len, seq.query_id, seq.last_block_num_tokens - (BS - W) - 1)]
    return []


def packed_words(batch: int, table_width: int) -> int:
    return batch * (HEADER_ROWS + table_width + 3)


def pack_decode(seqs: list[Sequence], padded: int, block_size: int, query_cache_len: int,
                table_width: int, scratch_row: int) -> np.ndarray:
    """All int32 inputs of one decode step in one buffer: the header rows (each `padded` long),
    then the block tables (padded x table_width, -1 filled) and the query triples (padded x 3).

    For the live entries this is zipage/engine/model_runner.py:633-675: position = len - 1,
    slot = last page * BS + tokens in the last page - 1, context = (pages - 1) * BS + tokens in
    the last page.  Entries past len(seqs) are inert: scratch row, slot -1, context 0, triple
    row -1, so a padded batch can replay a graph captured for a larger one.
    """
    BS, W, TW = block_size, query_cache_len, table_width
    B = len(seqs)
    n = np.fromiter((s.num_tokens for s in seqs), np.int64, B)
    npg = np.fromiter((len(s.block_table) for s in seqs), np.int64, B)
    last = np.fromiter((s.block_table[-1] for s in seqs), np.int64, B)
    rows = np.fromiter((s.query_id for s in seqs), np.int64, B)
    done = np.fromiter((s.num_completion_tokens for s in seqs), np.int64, B)
    tail = n - ((n + BS - 1) // BS - 1) * BS
    out = np.empty(packed_words(padded, TW), dtype=np.int32)
    head = out[:HEADER_ROWS * padded].reshape(HEADER_ROWS, padded)
    head[0].fill(scratch_row)
    head[1].fill(0)
    head[2].fill(-1)
    head[3].fill(0)
    head[4].fill(0)
    head[0, :B], head[1, :B] = rows, n - 1
    head[2, :B] = last * BS + tail - 1
    head[3, :B] = (npg - 1) * BS + tail
    head[4, :B] = done
    tab = out[HEADER_ROWS * padded:HEADER_ROWS * padded + padded * TW].reshape(padded, TW)
    tab.fill(-1)
    for i, s in enumerate(seqs):
        tab[i, :len(s.block_table)] = s.block_table
    tri = out[HEADER_ROWS * padded + padded * TW:].reshape(padded, 3)
    tri.fill(-1)
    hit = tail > BS - W
    tri[:B, 0] = np.where(hit, np.arange(B), -1)
    tri[:B, 1] = rows
    tri[:B, 2] = np.where(hit, tail - (BS - W) - 1, -1)
    return out


def unpack_views(buf, padded: int, table_width: int):
    """Views of a packed buffer (numpy array or torch tensor): header, tables, triples."""
    h = HEADER_ROWS * padded
    t = h + padded * table_width
    return (buf[:h].reshape(HEADER_ROWS, padded), buf[h:t].reshape(padded, table_width),
            buf[t:t + 3 * padded].reshape(padded, 3))


def encode_compress_tables(seqs: list[Sequence]) -> list[list[int]]:
    """Block tables as the compression kernels read them: last page as -id-2, -1 padding
    (zipage/engine/model_runner.py:437-463)."""
    width = max(len(s.block_table) for s in seqs)
    return [s.block_table[:-1] + [-s.block_table[-1] - 2] + [-1] * (width - len(s.block_table))
            for s in seqs]
