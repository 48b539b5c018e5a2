"""GPU parity of the decode-step cache kernels against plain PyTorch.

store_kvcache is a copy: bit-exact.  Decode attention is floating point: compared with an
fp32 PyTorch softmax(q K^T scale) V over the same gathered pages; the kernel accumulates in
fp32 and rounds the output once to the cache dtype, so the bound is one output ulp of the cache
dtype plus fp32 accumulation noise (2^-8 relative to the row's largest |value| for bf16,
2^-11 for fp16).
"""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _ref_decode(q, k_cache, v_cache, ctx, tables, scale):
    B, Hq, D = q.shape
    _, BS, Hkv, _ = k_cache.shape
    G = Hq // Hkv
    out = torch.zeros(B, Hq, D, dtype=torch.float32, device=q.device)
    for b in range(B):
        n = int(ctx[b])
        if n == 0:
            continue
        pages = tables[b][: (n + BS - 1) // BS].long()
        k = k_cache[pages].reshape(-1, Hkv, D)[:n].float()      # (n, Hkv, D)
        v = v_cache[pages].reshape(-1, Hkv, D)[:n].float()
        qq = q[b].float().view(Hkv, G, D)
        logit = torch.einsum("hgd,nhd->hgn", qq, k) * scale
        p = torch.softmax(logit, dim=-1)
        out[b] = torch.einsum("hgn,nhd->hgd", p, v).reshape(Hq, D)
    return out


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("Hq,Hkv,D,BS,NB,B", [
    (32, 8, 128, 256, 9, 5),      # Qwen3-8B decode shape
    (16, 8, 128, 256, 9, 3),      # Qwen3-0.6B
    (8, 8, 64, 16, 7, 4),         # no GQA, small pages
    (16, 2, 128, 32, 5, 2),       # group of 8
    (32, 8, 128, 256, 40, 3),     # 10 240-token table: walked in slices with rescaled accumulators
    (16, 2, 64, 256, 24, 2),      # sliced, group of 8
])
def test_paged_decode_attention(dev, dtype, Hq, Hkv, D, BS, NB, B):
    from zipage_amd.layers import paged_decode_attention
    g = torch.Generator(device="cpu").manual_seed(Hq * 131 + BS)
    pages = 3 * B * NB + 2
    k_cache = torch.randn(pages, BS, Hkv, D, generator=g).to(dtype).to(dev)
    v_cache = torch.randn(pages, BS, Hkv, D, generator=g).to(dtype).to(dev)
    q = torch.randn(B, Hq, D, generator=g).to(dtype).to(dev)
    perm = torch.randperm(pages, generator=g)[: B * NB].view(B, NB).int()
    ctx = torch.randint(1, NB * BS + 1, (B,), generator=g).int()
    ctx[0] = NB * BS            # full table
    ctx[-1] = 1                 # a single token
    tables = perm.clone()
    for b in range(B):
        used = (int(ctx[b]) + BS - 1) // BS
        tables[b, used:] = -1
    tables, ctx = tables.to(dev), ctx.to(dev)
    scale = D ** -0.5
    got = paged_decode_attention(q, k_cache, v_cache, ctx, tables, scale)
    want = _ref_decode(q, k_cache, v_cache, ctx.cpu(), tables, scale)
    assert got.dtype == dtype and got.shape == q.shape
    eps = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    tol = eps * want.abs().amax(dim=-1, keepdim=True).clamp(min=1e-3) + eps * want.abs()
    assert ((got.float() - want).abs() <= tol).all()


def test_paged_decode_attention_per_head_compacted_cache(dev):
    """After compression every kv head keeps its own survivors at the same positions of the
    same pages; attention over such a cache must treat each head's rows independently: permuting
    one head's token rows inside the context leaves the output unchanged up to summation order."""
    from zipage_amd.layers import paged_decode_attention
    torch.manual_seed(7)
    Hq, Hkv, D, BS, NB = 32, 8, 128, 256, 9
    k = torch.randn(NB, BS, Hkv, D, device=dev).bfloat16()
    v = torch.randn(NB, BS, Hkv, D, device=dev).bfloat16()
    q = torch.randn(1, Hq, D, device=dev).bfloat16()
    tables = torch.arange(NB, device=dev, dtype=torch.int32).view(1, NB)
    ctx = torch.tensor([8 * BS + 17], device=dev, dtype=torch.int32)
    a = paged_decode_attention(q, k, v, ctx, tables, D ** -0.5)
    n = int(ctx[0])
    perm = torch.randperm(n, device=dev)
    k2, v2 = k.clone().view(-1, Hkv, D), v.clone().view(-1, Hkv, D)
    k2[:n, 3] = k.view(-1, Hkv, D)[perm, 3]
    v2[:n, 3] = v.view(-1, Hkv, D)[perm, 3]
    b = paged_decode_attention(q, k2.view_as(k), v2.view_as(v), ctx, tables, D ** -0.5)
    assert torch.equal(a[:, :12], b[:, :12]) and torch.equal(a[:, 16:], b[:, 16:])
    assert (a[:, 12:16].float() - b[:, 12:16].float()).abs().max() <= 2.0 ** -8


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_store_kvcache(dev, dtype):
    from zipage_amd.layers import store_kvcache
    torch.manual_seed(3)
    N, Hkv, D, pages, BS = 300, 8, 128, 12, 64
    qkv = torch.randn(N, (16 + 2 * Hkv) * D, device=dev).to(dtype)
    key = qkv[:, 16 * D:(16 + Hkv) * D].view(N, Hkv, D)      # strided rows, as out of a fused qkv
    value = qkv[:, (16 + Hkv) * D:].view(N, Hkv, D)
    k_cache = torch.randn(pages, BS, Hkv, D, device=dev).to(dtype)
    v_cache = torch.randn(pages, BS, Hkv, D, device=dev).to(dtype)
    slots = torch.randperm(pages * BS, device=dev)[:N].int()
    slots[::7] = -1
    wk, wv = k_cache.clone(), v_cache.clone()
    keep = slots >= 0
    wk.view(-1, Hkv, D)[slots[keep].long()] = key[keep]
    wv.view(-1, Hkv, D)[slots[keep].long()] = value[keep]
    store_kvcache(key, value, k_cache, v_cache, slots)
    assert torch.equal(k_cache, wk) and torch.equal(v_cache, wv)


def test_store_kvcache_empty(dev):
    from zipage_amd.layers import store_kvcache
    k_cache = torch.zeros(2, 16, 2, 64, device=dev, dtype=torch.bfloat16)
    v_cache = torch.zeros_like(k_cache)
    key = torch.zeros(0, 2, 64, device=dev, dtype=torch.bfloat16)
    store_kvcache(key, key.clone(), k_cache, v_cache, torch.zeros(0, device=dev, dtype=torch.int32))
    assert not k_cache.any()
