"""Fused elementwise steps of the decoder layer (one HIP launch each)."""
import torch

from zipage_amd import _lib


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, residual: torch.Tensor | None = None):
    """RMSNorm.forward(x, residual) of the reference's nanovllm dependency
    (used at zipage/models/qwen3.py:139-150): without a residual returns norm(x) * weight; with
    one, `residual` becomes x + residual (rounded, in place) and the norm is taken of the fp32
    sum.  x: (N, hidden), 16-bit."""
    N, H = x.shape
    assert x.stride(1) == 1 and weight.is_contiguous() and weight.numel() == H
    out = torch.empty((N, H), dtype=x.dtype, device=x.device)
    if residual is not None:
        assert residual.shape == x.shape and residual.stride(1) == 1 and residual.dtype == x.dtype
    _lib.call("zp_add_rms_norm", _lib.dev_ptr(x), _lib.dev_ptr(residual), _lib.dev_ptr(weight),
              _lib.dev_ptr(out), N, H, x.stride(0), residual.stride(0) if residual is not None else 0,
              out.stride(0), float(eps), _lib.dtype_tag(x), _lib.stream_ptr(x))
    return out if residual is None else (out, residual)


def silu_and_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """SiluAndMul of the dependency (zipage/models/qwen3.py:108-111): silu(x[:, :I]) * x[:, I:]."""
    N, two_i = gate_up.shape
    I = two_i // 2
    assert gate_up.stride(1) == 1
    out = torch.empty((N, I), dtype=gate_up.dtype, device=gate_up.device)
    _lib.call("zp_silu_and_mul", _lib.dev_ptr(gate_up), _lib.dev_ptr(out), N, I, gate_up.stride(0),
              out.stride(0), _lib.dtype_tag(gate_up), _lib.stream_ptr(gate_up))
    return out


def qk_norm_rope_store(qkv: torch.Tensor, positions: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                       q_norm_weight: torch.Tensor, k_norm_weight: torch.Tensor, num_heads: int,
                       num_kv_heads: int, head_dim: int, eps: float,
                       k_cache: torch.Tensor | None = None, v_cache: torch.Tensor | None = None,
                       slot_mapping: torch.Tensor | None = None,
                       query_cache: torch.Tensor | None = None,
                       query_triples: torch.Tensor | None = None, return_k: bool = False):
    """q_norm, k_norm, rotary embedding, store_kvcache and (for decode steps) store_query_cache of
    one attention layer in one launch (zipage/models/qwen3.py:72-88 with
    zipage/layers/attention.py:69-92).  qkv: (N, (Hq + 2 Hkv) * D); positions: (N,) int32;
    cos/sin: (max_position, D/2) fp32; caches of one layer; slot_mapping (N,) int32;
    query_triples (N, 3) int32 with row i naming token i or -1.  Returns q (N, Hq, D), and with
    `return_k` also the rotated k (N, Hkv, D)."""
    N = qkv.shape[0]
    assert qkv.stride(1) == 1 and qkv.shape[1] == (num_heads + 2 * num_kv_heads) * head_dim
    assert positions.dtype == torch.int32 and positions.is_contiguous()
    assert cos.dtype == torch.float32 and cos.is_contiguous() and sin.is_contiguous()
    assert cos.shape[1] == head_dim // 2
    q = torch.empty((N, num_heads, head_dim), dtype=qkv.dtype, device=qkv.device)
    k = torch.empty((N, num_kv_heads, head_dim), dtype=qkv.dtype, device=qkv.device) if return_k else None
    num_slots = 0
    if slot_mapping is not None:
        assert slot_mapping.dtype == torch.int32 and slot_mapping.is_contiguous()
        assert k_cache.stride(1) == num_kv_heads * head_dim and v_cache.stride(1) == num_kv_heads * head_dim
        num_slots = k_cache.shape[0] * k_cache.shape[1]
    qc = (0, 0, 0, 0)
    if query_triples is not None:
        assert query_triples.dtype == torch.int32 and query_triples.is_contiguous()
        assert query_triples.shape == (N, 3)
        qc = (query_cache.shape[0], query_cache.shape[1], query_cache.stride(0), query_cache.stride(1))
    _lib.call("zp_qk_norm_rope_store", _lib.dev_ptr(qkv), _lib.dev_ptr(q), _lib.dev_ptr(k), _lib.dev_ptr(k_cache),
              _lib.dev_ptr(v_cache), _lib.dev_ptr(query_cache if query_triples is not None else None),
              _lib.dev_ptr(q_norm_weight), _lib.dev_ptr(k_norm_weight), _lib.dev_ptr(cos),
              _lib.dev_ptr(sin), _lib.dev_ptr(positions), _lib.dev_ptr(slot_mapping),
              _lib.dev_ptr(query_triples), N, num_heads, num_kv_heads, head_dim, cos.shape[0],
              qkv.stride(0), num_slots, qc[0], qc[1], qc[2], qc[3], float(eps), _lib.dtype_tag(qkv),
              _lib.stream_ptr(qkv))
    return (q, k) if return_k else q
