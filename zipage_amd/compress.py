"""One layer chunk of the compression pipeline on the GPU.

Host-side mirror of the body of ``ModelRunner.compress``
(zipage/engine/model_runner.py:466-622): the same stages with the same switches, each
dispatched to its HIP entry point.  The redundancy score only reads the key cache, so it is
launched before the selection stages, which then run as one launch (pooling, combine, sink /
window / pad masks, top-k); ``fused_select=False`` keeps them as the reference's separate
stages, in its order.  Nothing here synchronises with the host: the
reference's ``torch.all(compressed)`` test before pooling (model_runner.py:501) only skips
work whose result equals its input, so pooling is decided per sequence on the device.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass

import torch

from zipage_amd import _lib

from zipage_amd.kernel.attention_score import attention_score
from zipage_amd.kernel.compress_kv import compress_kv
from zipage_amd.kernel.compress_score import compress_score
from zipage_amd.kernel.global_score import global_score
from zipage_amd.kernel.lightning_redudancy_score import lightning_redudancy_score
from zipage_amd.kernel.pooling import pool_scores
from zipage_amd.kernel.raw_redudancy_score import raw_redudancy_score
from zipage_amd.kernel.select import MAX_ROW_TOKENS, select_topk
from zipage_amd.kernel.utils import topk_mask
from zipage_amd.kernel.window_mask import score_epilogue

# stage names as the reference records them (model_runner.py:424-429,624-630)
STAGES = ("attention_score", "global_score", "pooling", "redudancy_score", "attention_sink",
          "window_mask", "topk_mask", "compress_kv", "compress_global_score")
# pooling, combine, sink / window / pad masks and top-k run as one launch unless a caller asks
# for the separate stages; the timer then books them under this one name
FUSED_SELECT_STAGE = "pooling+window_mask+topk_mask"


@dataclass
class CompressConfig:
    """The switches of zipage/config.py:22-46 that the compression path reads."""
    budget_blocks: int = 8            # max_cache_blocks_per_seq
    query_cache_len: int = 16
    softmax_scale: float | None = None
    reduced: str = "mean"
    use_global_score: bool = False
    decay_factor: float = 0.8
    activate_method: str = "max"
    max_norm: bool = False
    use_redudancy: bool = False
    lightning_redudancy: bool = False
    redudancy_lambda: float = 0.2
    redudancy_temperature: float = 0.4
    redudancy_threshold: float = 0.5
    enable_pooling: bool = False
    continues_pooling: bool = False
    pooling_size: int = 5             # the reference runner hard-codes 5 (model_runner.py:71)
    pooling_mode: str = "max"
    use_attention_sink: bool = False
    sink_len: int = 4


class StageTimer:
    """Optional per-stage device timing with the reference's stage names."""

    def __init__(self, enabled: bool, only: tuple[str, ...] | None = None):
        self.enabled = enabled
        self.only = only      # time just these stages (every event pair costs a few microseconds)
        self.spans = []

    def start(self, name):
        if not self.enabled or (self.only is not None and name not in self.only):
            return None
        st, ed = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        st.record()
        self.spans.append((name, st, ed))
        return ed

    @staticmethod
    def stop(ed):
        if ed is not None:
            ed.record()

    def event_array(self, stages):
        """Start / stop event handles for ``zp_compress_layers`` (a host array of
        2 * ZP_NUM_STAGES hipEvent_t; stages that are not timed stay NULL), or None."""
        if not self.enabled:
            return None
        arr = (ctypes.c_void_p * (2 * len(_lib.STAGE_NAMES)))()
        for i, name in enumerate(_lib.STAGE_NAMES):
            if name not in stages or (self.only is not None and name not in self.only):
                continue
            st, ed = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            st.record()   # torch creates the HIP event on its first record
            ed.record()
            arr[2 * i], arr[2 * i + 1] = st.cuda_event, ed.cuda_event
            self.spans.append((name, st, ed))
        return arr

    def seconds(self):
        """Per-stage totals; call after the stream has been synchronised."""
        out = {}
        for name, st, ed in self.spans:
            out[name] = out.get(name, 0.0) + st.elapsed_time(ed) / 1000.0
        return out


def compress_layers(k_cache, v_cache, query_cache, score_cache, query_ids, block_tables,
                    compressed, target_block_tables, cfg: CompressConfig, timer=None,
                    return_intermediates=False, fused_select=True, deterministic_carry=True):
    """Score, select and compact one chunk of layers in place.

    k_cache/v_cache: (L, num_pages, BS, Hkv, D); query_cache: (L, max_seqs, W, Hq, D);
    score_cache: (L, num_pages, BS, Hkv) or None; query_ids: (B,) int32; block_tables:
    (B, NB) int32 encoded as in model_runner.py:437-463; compressed: (B,) bool;
    target_block_tables: (B, budget+1) int32.  Returns the keep flag (L, B, Hkv, NB, BS).

    ``deterministic_carry`` (default): the reference's global_score stores every sequence's
    scores into its pages of the score cache (global_score.py:73-74) and compress_score reads
    them back (compress_score.py:50-53); when sequences of the batch share prefix pages those
    stores race and the carried scores depend on the order the GPU ran them in.  Here the
    score cache is only read by global_score and the survivors' carried scores are compacted
    straight from the scores it returned: the same values as the reference whenever no page is
    shared, independent of scheduling when one is, and no shared (read-only) page is written.
    ``False`` runs the reference's two stores.  (The CPU oracle's ``compress_pipeline`` is the
    reference restated, so ITS default is ``deterministic_carry=False``: a comparison of the two
    on a batch with shared pages passes the switch explicitly to both.)
    """
    t = timer or StageTimer(False)
    BS = k_cache.shape[2]
    if fused_select and not return_intermediates and block_tables.shape[1] * BS <= MAX_ROW_TOKENS:
        return _compress_layers_one_call(k_cache, v_cache, query_cache, score_cache, query_ids,
                                         block_tables, compressed, target_block_tables, cfg, t,
                                         deterministic_carry)

    ev = t.start("attention_score")
    scores = attention_score(k_cache, query_cache, query_ids, block_tables, cfg.softmax_scale,
                             cfg.reduced)
    t.stop(ev)

    if cfg.use_global_score:
        ev = t.start("global_score")
        if cfg.max_norm:
            score_epilogue(scores, block_tables, max_norm_scores=True)
        scores = global_score(scores, score_cache, block_tables, compressed, cfg.decay_factor,
                              cfg.activate_method, write_cache=not deterministic_carry)
        t.stop(ev)
    carried = scores if (cfg.use_global_score and deterministic_carry) else None

    red = None
    if cfg.use_redudancy:
        ev = t.start("redudancy_score")
        fn = lightning_redudancy_score if cfg.lightning_redudancy else raw_redudancy_score
        red = fn(k_cache, block_tables, threshold=cfg.redudancy_threshold,
                 temperature=cfg.redudancy_temperature)
        t.stop(ev)

    L, B, Hkv, NB, _ = scores.shape
    if fused_select and NB * BS <= MAX_ROW_TOKENS:
        ev = t.start(FUSED_SELECT_STAGE)
        out = select_topk(scores, block_tables, compressed, BS * cfg.budget_blocks,
                          pooling_size=cfg.pooling_size if cfg.enable_pooling else 0,
                          continues_pooling=cfg.continues_pooling, pooling_mode=cfg.pooling_mode,
                          redundancy=red,
                          max_norm_red=cfg.use_redudancy and cfg.use_global_score and cfg.max_norm,
                          redudancy_lambda=cfg.redudancy_lambda,
                          sink_len=cfg.sink_len if cfg.use_attention_sink else 0,
                          window=cfg.query_cache_len, mask_pad=True,
                          return_scores=return_intermediates)
        flag, scores = out if return_intermediates else (out, scores)
        t.stop(ev)
    else:
        if carried is not None and not cfg.enable_pooling:
            carried = scores.clone()   # the mask epilogue below works in place on `scores`
        if cfg.enable_pooling:
            ev = t.start("pooling")
            scores = pool_scores(scores, compressed, cfg.pooling_size, cfg.continues_pooling,
                                 cfg.pooling_mode)
            t.stop(ev)

        # combine + sink + window mask + pad mask: one fused pass (window_mask stage)
        ev = t.start("window_mask")
        score_epilogue(scores, block_tables, red,
                       max_norm_red=cfg.use_redudancy and cfg.use_global_score and cfg.max_norm,
                       redudancy_lambda=cfg.redudancy_lambda,
                       sink_len=cfg.sink_len if cfg.use_attention_sink else 0,
                       window=cfg.query_cache_len, mask_pad=True)
        t.stop(ev)

        ev = t.start("topk_mask")
        flag = topk_mask(scores.view(L, B, Hkv, NB * BS), BS * cfg.budget_blocks)
        flag = flag.view(L, B, Hkv, NB, BS)
        t.stop(ev)

    ev = t.start("compress_kv")
    compress_kv(k_cache, v_cache, flag, block_tables, target_block_tables)
    t.stop(ev)

    if cfg.use_global_score:
        ev = t.start("compress_global_score")
        compress_score(score_cache, flag, block_tables, target_block_tables, scores_src=carried)
        t.stop(ev)
    if return_intermediates:
        return flag, scores
    return flag


_REDUCE = {"mean": 0, "max": 1}
_ACTIVATE = {"max": 0, "sum": 1}
_POOL = {"max": 0, "avg": 1}


def c_config(cfg: CompressConfig, deterministic_carry=True) -> "_lib.CompressConfigC":
    if cfg.reduced not in _REDUCE:
        raise ValueError(f"Invalid reduction method: {cfg.reduced}")
    assert cfg.activate_method in _ACTIVATE and cfg.pooling_mode in _POOL
    assert 0 <= cfg.decay_factor <= 1
    return _lib.CompressConfigC(
        budget_blocks=cfg.budget_blocks, query_cache_len=cfg.query_cache_len,
        softmax_scale=-1.0 if cfg.softmax_scale is None else float(cfg.softmax_scale),
        reduced=_REDUCE[cfg.reduced], use_global_score=int(cfg.use_global_score),
        decay_factor=float(cfg.decay_factor), activate_method=_ACTIVATE[cfg.activate_method],
        max_norm=int(cfg.max_norm), use_redundancy=int(cfg.use_redudancy),
        lightning=int(cfg.lightning_redudancy), redundancy_lambda=float(cfg.redudancy_lambda),
        redundancy_temperature=float(cfg.redudancy_temperature),
        redundancy_threshold=float(cfg.redudancy_threshold),
        pooling_size=cfg.pooling_size if cfg.enable_pooling else 0,
        continues_pooling=int(cfg.continues_pooling), pooling_mode=_POOL[cfg.pooling_mode],
        sink_len=cfg.sink_len if cfg.use_attention_sink else 0,
        deterministic_carry=int(deterministic_carry))


def layer_chunk_args(k_cache, v_cache, query_cache, score_cache, query_ids, block_tables,
                     compressed, target_block_tables):
    """Shape checks and the dims / strides block shared by the one-call entry points."""
    L, num_pages, BS, Hkv, D = k_cache.shape
    _, max_seqs, W, Hq, _ = query_cache.shape
    B, NB = block_tables.shape
    assert v_cache.shape == k_cache.shape and v_cache.dtype == k_cache.dtype
    assert query_cache.shape[0] == L and query_cache.dtype == k_cache.dtype
    assert query_cache.is_contiguous() and k_cache.stride(4) == 1 and v_cache.stride(4) == 1
    assert query_ids.shape == (B,) and query_ids.dtype == torch.int32 and query_ids.is_contiguous()
    assert block_tables.dtype == torch.int32 and block_tables.is_contiguous()
    assert compressed.shape == (B,) and compressed.dtype == torch.bool
    assert target_block_tables.shape[0] == B and target_block_tables.dtype == torch.int32
    assert target_block_tables.is_contiguous()
    strides = list(k_cache.stride()[:4]) + list(v_cache.stride()[:4]) + list(query_cache.stride()[:2])
    if score_cache is not None:
        assert score_cache.shape == (L, num_pages, BS, Hkv) and score_cache.dtype == k_cache.dtype
        strides += list(score_cache.stride())
    else:
        strides += [0, 0, 0, 0]
    dims = (L, B, NB, BS, Hkv, Hq, D, W, num_pages, max_seqs, target_block_tables.shape[1])
    return dims, (ctypes.c_int64 * 14)(*strides)


def _compress_layers_one_call(k_cache, v_cache, query_cache, score_cache, query_ids, block_tables,
                              compressed, target_block_tables, cfg, timer, deterministic_carry):
    """The whole chunk through ``zp_compress_layers``: one host call enqueues every stage; the
    only allocations are the keep flags and the workspace (torch's caching allocator)."""
    dims, strides = layer_chunk_args(k_cache, v_cache, query_cache, score_cache, query_ids,
                                     block_tables, compressed, target_block_tables)
    L, B, NB, BS, Hkv, Hq, D, W = dims[:8]
    if cfg.use_global_score:
        assert score_cache is not None
    flag = torch.empty((L, B, Hkv, NB, BS), device=k_cache.device, dtype=torch.bool)
    if flag.numel() == 0:
        return flag
    cc = c_config(cfg, deterministic_carry)
    lib = _lib.load()
    tag = _lib.dtype_tag(k_cache)
    ws_bytes = lib.zp_compress_layers_workspace(L, B, NB, BS, Hkv, Hq, W, tag, ctypes.byref(cc), 0)
    ws = torch.empty(ws_bytes, device=k_cache.device, dtype=torch.uint8)
    running = {"attention_score", FUSED_SELECT_STAGE, "compress_kv"}
    if cfg.use_global_score:
        running |= {"global_score", "compress_global_score"}
    if cfg.use_redudancy:
        running.add("redudancy_score")
    events = timer.event_array(running)
    compressed = compressed.contiguous()
    _lib.call("zp_compress_layers", _lib.dev_ptr(k_cache), _lib.dev_ptr(v_cache),
              _lib.dev_ptr(query_cache), _lib.dev_ptr(score_cache), _lib.dev_ptr(query_ids),
              _lib.dev_ptr(block_tables), _lib.dev_ptr(compressed),
              _lib.dev_ptr(target_block_tables), _lib.dev_ptr(flag), *dims, strides, tag,
              ctypes.byref(cc), _lib.dev_ptr(ws), ws_bytes, events, _lib.stream_ptr(k_cache))
    return flag
