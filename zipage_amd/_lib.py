"""ctypes binding of ``libzipage_hip.so`` (the C ABI in ``include/zipage_hip.h``).

The product path has no CPU fallback: if the shared object is missing or a symbol cannot
be resolved, importing a kernel wrapper raises.  ctypes releases the GIL for the duration
of every call, so the wrappers can be driven from a worker thread while another thread
runs the model forward (the reference calls this path from a ThreadPoolExecutor worker,
zipage/engine/zipage_engine.py:153-166).
"""
from __future__ import annotations

import ctypes as C
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libzipage_hip.so")

ZP_BF16, ZP_F16, ZP_F32 = 0, 1, 2
_DTYPES = {torch.bfloat16: ZP_BF16, torch.float16: ZP_F16, torch.float32: ZP_F32}

i32, i64, f32, f64, ptr = C.c_int32, C.c_int64, C.c_float, C.c_double, C.c_void_p

# name -> argument types, in the order of include/zipage_hip.h
SIGNATURES = {
    "zp_store_query": [ptr, ptr, ptr, i32, i32, i32, i32, i32, i64, i64, i64, i64, i64, i32, ptr],
    "zp_attention_score": [ptr, ptr, ptr, ptr, ptr, ptr, i32, i32, i32, i32, i32, i32, i32, i32,
                           i32, i32, i64, i64, i64, i64, f32, i32, i32, ptr, i64, ptr],
    "zp_global_score": [ptr, ptr, ptr, ptr, i32, i32, i32, i32, i32, i32, i64, i64, f32, i32, i32,
                        i32, ptr],
    "zp_pool_scores": [ptr, ptr, ptr, i32, i32, i32, i32, i32, i32, i32, i32, ptr],
    "zp_key_norm": [ptr, ptr, ptr, i32, i32, i32, i32, i32, i32, i32, i64, i64, f32, i32, ptr],
    "zp_redundancy_lightning": [ptr, ptr, ptr, ptr, i32, i32, i32, i32, i32, i32, i32, i64, i64,
                                f32, f64, i32, ptr],
    "zp_redundancy_raw": [ptr, ptr, ptr, ptr, i32, i32, i32, i32, i32, i32, i32, i64, i64, f32,
                          f64, i32, ptr, i64, ptr],
    "zp_score_epilogue": [ptr, ptr, ptr, i32, i32, i32, i32, i32, i32, i32, f64, i32, i32, i32,
                          i32, ptr],
    "zp_topk_mask": [ptr, ptr, i32, i32, i32, i32, ptr],
    "zp_select_topk": [ptr, ptr, ptr, ptr, ptr, ptr, i32, i32, i32, i32, i32, i32, i32, i32, i32,
                       f64, i32, i32, i32, i32, i32, ptr],
    "zp_compress_kv": [ptr, ptr, ptr, ptr, ptr, i32, i32, i32, i32, i32, i32, i32, i32,
                       i64, i64, i64, i64, i64, i64, i64, i64, i32, ptr],
    "zp_compress_score": [ptr, ptr, ptr, ptr, ptr, i32, i32, i32, i32, i32, i32, i32, i64, i64, i64,
                          i64, i32, ptr],
    "zp_store_kvcache": [ptr, ptr, ptr, ptr, ptr, i32, i32, i64, i64, i64, i32, ptr],
    "zp_paged_decode_attention": [ptr, ptr, ptr, ptr, ptr, ptr, i32, i32, i32, i32, i32, i32, i32,
                                  i64, i64, f32, i32, ptr],
    "zp_add_rms_norm": [ptr, ptr, ptr, ptr, i32, i32, i64, i64, i64, f32, i32, ptr],
    "zp_silu_and_mul": [ptr, ptr, i32, i32, i64, i64, i32, ptr],
    "zp_qk_norm_rope_store": [ptr, ptr, ptr, ptr, ptr, ptr, ptr, ptr, ptr, ptr, ptr, ptr, ptr, i32, i32,
                              i32, i32, i32, i64, i64, i32, i32, i64, i64, f32, i32, ptr],
}


class CompressConfigC(C.Structure):
    """zp_compress_config of include/zipage_hip.h."""
    _fields_ = [("budget_blocks", i32), ("query_cache_len", i32), ("softmax_scale", f32),
                ("reduced", i32), ("use_global_score", i32), ("decay_factor", f32),
                ("activate_method", i32), ("max_norm", i32), ("use_redundancy", i32),
                ("lightning", i32), ("redundancy_lambda", f64), ("redundancy_temperature", f64),
                ("redundancy_threshold", f32), ("pooling_size", i32), ("continues_pooling", i32),
                ("pooling_mode", i32), ("sink_len", i32), ("deterministic_carry", i32)]


# stage order of the ZP_STAGE_* enum, under the names the reference's timers use
# (zipage/engine/model_runner.py:424-429); the one-launch selection has its own name
STAGE_NAMES = ("attention_score", "global_score", "pooling", "redudancy_score", "window_mask",
               "topk_mask", "pooling+window_mask+topk_mask", "compress_kv", "compress_global_score")

SIGNATURES["zp_compress_layers"] = (
    [ptr] * 9 + [i32] * 11 + [C.POINTER(i64), i32, C.POINTER(CompressConfigC), ptr, i64,
                              C.POINTER(ptr), ptr])
SIGNATURES["zp_compress_layers_static"] = (
    [ptr] * 9 + [i32] * 11 + [C.POINTER(i64), i32, C.POINTER(CompressConfigC), ptr])
SIGNATURES["zp_static_scratch_init"] = []
STATIC_SCRATCH_BYTES = 32 << 20
I64_RETURNING = {
    "zp_compress_layers_workspace": [i32, i32, i32, i32, i32, i32, i32, i32,
                                     C.POINTER(CompressConfigC), i32],
    "zp_attention_score_workspace": [i32, i32, i32, i32, i32, i32, i32],
    "zp_attention_score_workspace_for": [i32, i32, i32, i32, i32, i32, i32, i32],
    "zp_redundancy_raw_workspace": [i32, i32, i32, i32, i32],
}
EXPORTS = sorted(list(SIGNATURES) + list(I64_RETURNING) + ["zp_abi_version", "zp_last_error"])

_lib = None


def load() -> C.CDLL:
    """Load the shared object once and type every entry point.  Raises if absent."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m zipage_amd.build` "
            "(there is no CPU fallback for the compression kernels)")
    lib = C.CDLL(LIB_PATH)
    for name, args in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes, fn.restype = args, i32
    for name, args in I64_RETURNING.items():
        fn = getattr(lib, name)
        fn.argtypes, fn.restype = args, i64
    lib.zp_abi_version.argtypes, lib.zp_abi_version.restype = [], i32
    lib.zp_last_error.argtypes, lib.zp_last_error.restype = [], C.c_char_p
    _lib = lib
    return lib


def call(name: str, *args) -> None:
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise RuntimeError(f"{name} failed ({rc}): {lib.zp_last_error().decode()}")


def dtype_tag(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported cache dtype {t.dtype}; use bfloat16, float16 or float32")


def dev_ptr(t) -> int:
    if t is None:
        return 0
    if not t.is_cuda:
        raise RuntimeError("the compression kernels need device tensors (no CPU fallback)")
    return t.data_ptr()


def stream_ptr(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream
