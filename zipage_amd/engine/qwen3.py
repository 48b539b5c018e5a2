"""Random-initialised Qwen3 decoder (zipage/models/qwen3.py) wired to the paged caches.

Only what the decode benchmark needs: bf16 weights drawn on the device and the fused qkv and
gate/up projections through torch's GEMMs; everything between the GEMMs is this package's HIP
kernels (residual add + RMSNorm, per-head q/k norm + rotary embedding + K/V scatter + window-query
capture, paged decode attention, SiLU gate).  Prefill attention is torch's
scaled_dot_product_attention.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch
import torch.nn.functional as F

from zipage_amd.kernel import store_query_cache
from zipage_amd.layers import paged_decode_attention, qk_norm_rope_store, rms_norm, silu_and_mul


@dataclass(frozen=True)
class Qwen3Shape:
    layers: int
    hidden: int
    heads: int
    kv_heads: int
    head_dim: int
    intermediate: int
    vocab: int
    eps: float = 1e-6
    rope_theta: float = 1e6
    max_position: int = 40960


QWEN3_8B = Qwen3Shape(36, 4096, 32, 8, 128, 12288, 151936)
QWEN3_0_6B = Qwen3Shape(28, 1024, 16, 8, 128, 3072, 151936)


@dataclass
class StepContext:
    """Per-step attention metadata (the reference keeps it in a module-global context,
    zipage/utils/context.py; here it is passed explicitly so a captured graph can own one)."""
    is_prefill: bool
    slot_mapping: torch.Tensor                      # (N,) int32
    query_slot_mapping: torch.Tensor | None = None  # (M, 3) int32
    context_lens: torch.Tensor | None = None        # (B,) int32, decode
    block_tables: torch.Tensor | None = None        # (B, NB) int32, decode / cached prefill
    seq_lens_q: list[int] | None = None             # prefill: new tokens per sequence
    seq_lens_k: list[int] | None = None             # prefill: total tokens per sequence


class Qwen3:
    def __init__(self, shape: Qwen3Shape, device, dtype=torch.bfloat16, seed: int = 0,
                 init_std: float = 0.02):
        self.shape, self.device, self.dtype = shape, torch.device(device), dtype
        s = shape
        g = torch.Generator(device=self.device).manual_seed(seed)

        def w(*dims):
            return torch.empty(*dims, device=self.device, dtype=dtype).normal_(0.0, init_std, generator=g)

        def ones(n):
            return torch.ones(n, device=self.device, dtype=dtype)

        self.embed = w(s.vocab, s.hidden)
        self.lm_head = w(s.vocab, s.hidden)
        self.final_norm = ones(s.hidden)
        qkv_out = (s.heads + 2 * s.kv_heads) * s.head_dim
        self.layers = []
        for _ in range(s.layers):
            self.layers.append(dict(
                ln1=ones(s.hidden), wqkv=w(qkv_out, s.hidden), qn=ones(s.head_dim), kn=ones(s.head_dim),
                wo=w(s.hidden, s.heads * s.head_dim), ln2=ones(s.hidden),
                wgu=w(2 * s.intermediate, s.hidden), wd=w(s.hidden, s.intermediate)))
        inv = 1.0 / (s.rope_theta ** (torch.arange(0, s.head_dim, 2, dtype=torch.float32) / s.head_dim))
        ang = torch.arange(s.max_position, dtype=torch.float32)[:, None] * inv[None, :]
        self.cos = ang.cos().to(self.device)     # (max_position, D/2) fp32
        self.sin = ang.sin().to(self.device)
        self.scale = s.head_dim ** -0.5
        self.k_cache = self.v_cache = self.q_cache = None   # (L, ...) views set by the runner

    def attach_caches(self, kv_cache: torch.Tensor, query_cache: torch.Tensor):
        self.k_cache, self.v_cache, self.q_cache = kv_cache[0], kv_cache[1], query_cache

    # ------------------------------------------------------------------ pieces
    def _prefill_attention(self, li, q, k, v, ctx: StepContext) -> torch.Tensor:
        s = self.shape
        lens_q, lens_k = ctx.seq_lens_q, ctx.seq_lens_k
        if lens_q == lens_k and len(set(lens_q)) == 1:
            B, n = len(lens_q), lens_q[0]
            o = F.scaled_dot_product_attention(
                q.view(B, n, s.heads, s.head_dim).transpose(1, 2),
                k.view(B, n, s.kv_heads, s.head_dim).transpose(1, 2),
                v.view(B, n, s.kv_heads, s.head_dim).transpose(1, 2),
                is_causal=True, scale=self.scale, enable_gqa=True)
            return o.transpose(1, 2).reshape(B * n, s.heads * s.head_dim)
        out = torch.empty_like(q)
        BS = self.k_cache.shape[2]
        off = 0
        for b, (nq, nk) in enumerate(zip(lens_q, lens_k)):
            qq = q[off:off + nq].transpose(0, 1).unsqueeze(0)
            if nq == nk:
                kk, vv = k[off:off + nq], v[off:off + nq]
            else:  # cached prefix: read the whole context back through the table
                pages = ctx.block_tables[b, : (nk + BS - 1) // BS].long()
                kk = self.k_cache[li][pages].reshape(-1, s.kv_heads, s.head_dim)[:nk]
                vv = self.v_cache[li][pages].reshape(-1, s.kv_heads, s.head_dim)[:nk]
            mask = torch.ones(nq, nk, dtype=torch.bool, device=q.device).tril(diagonal=nk - nq)
            o = F.scaled_dot_product_attention(qq, kk.transpose(0, 1).unsqueeze(0),
                                               vv.transpose(0, 1).unsqueeze(0), attn_mask=mask,
                                               scale=self.scale, enable_gqa=True)
            out[off:off + nq] = o[0].transpose(0, 1)
            off += nq
        return out.view(-1, s.heads * s.head_dim)

    def _attention(self, li, p, x, pos32, ctx: StepContext) -> torch.Tensor:
        """zipage/models/qwen3.py:72-88 + zipage/layers/attention.py:69-104."""
        s = self.shape
        N = x.shape[0]
        qkv = F.linear(x, p["wqkv"])
        q_sz, kv_sz = s.heads * s.head_dim, s.kv_heads * s.head_dim
        cached = self.k_cache is not None and self.k_cache.numel() > 0 and ctx.slot_mapping is not None
        kc = self.k_cache[li] if cached else None
        vc = self.v_cache[li] if cached else None
        if ctx.is_prefill:
            q, k = qk_norm_rope_store(qkv, pos32, self.cos, self.sin, p["qn"], p["kn"], s.heads,
                                      s.kv_heads, s.head_dim, s.eps, kc, vc,
                                      ctx.slot_mapping if cached else None, return_k=True)
            if ctx.query_slot_mapping is not None:
                store_query_cache(q, self.q_cache[li], ctx.query_slot_mapping)
            v = qkv[:, q_sz + kv_sz:].view(N, s.kv_heads, s.head_dim)
            o = self._prefill_attention(li, q, k, v, ctx)
        else:
            q = qk_norm_rope_store(qkv, pos32, self.cos, self.sin, p["qn"], p["kn"], s.heads,
                                   s.kv_heads, s.head_dim, s.eps, kc, vc, ctx.slot_mapping,
                                   self.q_cache[li] if ctx.query_slot_mapping is not None else None,
                                   ctx.query_slot_mapping)
            o = paged_decode_attention(q, kc, vc, ctx.context_lens, ctx.block_tables,
                                       self.scale).view(N, q_sz)
        return F.linear(o, p["wo"])

    # ------------------------------------------------------------------ forward
    @torch.inference_mode()
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        """Hidden states (N, hidden) after the final norm (zipage/models/qwen3.py:169-181).  In a
        decode step `ctx.query_slot_mapping` holds one triple per token (row -1 = none)."""
        s = self.shape
        pos32 = positions.to(torch.int32)
        hidden = F.embedding(input_ids, self.embed)
        resid = None
        for li, p in enumerate(self.layers):
            if resid is None:
                resid, h = hidden, rms_norm(hidden, p["ln1"], s.eps)
            else:
                h, resid = rms_norm(hidden, p["ln1"], s.eps, resid)
            hidden = self._attention(li, p, h, pos32, ctx)
            h, resid = rms_norm(hidden, p["ln2"], s.eps, resid)
            hidden = F.linear(silu_and_mul(F.linear(h, p["wgu"])), p["wd"])
        h, _ = rms_norm(hidden, self.final_norm, s.eps, resid)
        return h

    @torch.inference_mode()
    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden, self.lm_head)
