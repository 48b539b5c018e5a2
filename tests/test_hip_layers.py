"""GPU parity of the fused decoder-layer kernels against the unfused PyTorch module sequence
(fp32 math, rounding to the 16-bit dtype where the modules round).  Bound: results are 16-bit
values produced from fp32 intermediates that can differ in the last fp32 bits (rsqrt, exp), so
almost every element is identical; where two roundings are chained (normalise, then scale; silu,
then multiply) a one-ulp difference in the first can become two in the result, so the bound is two
16-bit ulps."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _ulps(got, want):
    """Largest distance in units in the last place of the 16-bit dtype, and fraction identical."""
    mant, emin = (7, -126) if want.dtype == torch.bfloat16 else (10, -14)
    g, w = got.float(), want.float()
    mag = torch.maximum(w.abs(), g.abs()).clamp(min=2.0 ** emin)
    ulp = torch.exp2(torch.floor(torch.log2(mag)) - mant)
    return ((g - w).abs() / ulp).max().item(), (got == want).float().mean().item()


def _rope_ulps(got, want):
    """As _ulps, but in ulps at the magnitude of the rotated pair: a rotation can cancel, so a
    one-ulp difference of its inputs is not small against a small output."""
    mant, emin = (7, -126) if want.dtype == torch.bfloat16 else (10, -14)
    g, w = got.float(), want.float()
    w1, w2 = w.chunk(2, dim=-1)
    mag = (w1 * w1 + w2 * w2).sqrt().clamp(min=2.0 ** emin)
    ulp = torch.exp2(torch.floor(torch.log2(mag)) - mant)
    ulp = torch.cat((ulp, ulp), dim=-1)
    return ((g - w).abs() / ulp).max().item(), (got == want).float().mean().item()


def _rms_ref(x, w, eps, residual=None):
    orig = x.dtype
    x = x.float()
    if residual is not None:
        x = x + residual.float()
        residual = x.to(orig)
    var = x.pow(2).mean(-1, keepdim=True)
    x = x * torch.rsqrt(var + eps)
    out = x.to(orig) * w
    return out if residual is None else (out, residual)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("N,H", [(256, 4096), (3, 1024), (17, 8192), (5, 64)])
def test_rms_norm_with_and_without_residual(dev, dtype, N, H):
    from zipage_amd.layers import rms_norm
    torch.manual_seed(N + H)
    x = torch.randn(N, H, device=dev).to(dtype)
    r = torch.randn(N, H, device=dev).to(dtype)
    w = (1 + 0.1 * torch.randn(H, device=dev)).to(dtype)
    worst, same = _ulps(rms_norm(x, w, 1e-6), _rms_ref(x, w, 1e-6))
    assert worst <= 2.0 and same > 0.995
    want_out, want_res = _rms_ref(x, w, 1e-6, r)
    r2 = r.clone()
    out, res = rms_norm(x, w, 1e-6, r2)
    assert res is r2 and torch.equal(res, want_res)
    worst, same = _ulps(out, want_out)
    assert worst <= 2.0 and same > 0.995


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_rms_norm_strided_rows(dev, dtype):
    from zipage_amd.layers import rms_norm
    torch.manual_seed(0)
    big = torch.randn(9, 3 * 256, device=dev).to(dtype)
    x = big[:, 256:512]
    w = torch.ones(256, device=dev, dtype=dtype)
    worst, same = _ulps(rms_norm(x, w, 1e-6), _rms_ref(x, w, 1e-6))
    assert worst <= 2.0 and same > 0.995


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("N,I", [(256, 12288), (7, 3072), (1, 8)])
def test_silu_and_mul(dev, dtype, N, I):
    from zipage_amd.layers import silu_and_mul
    torch.manual_seed(I)
    gu = (2 * torch.randn(N, 2 * I, device=dev)).to(dtype)
    g, u = gu.chunk(2, dim=-1)
    want = torch.nn.functional.silu(g) * u
    worst, same = _ulps(silu_and_mul(gu), want)
    assert worst <= 2.0 and same > 0.99


def _rope_ref(x, cos, sin):
    x1, x2 = torch.chunk(x.float(), 2, dim=-1)
    return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1).to(x.dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("Hq,Hkv,D", [(32, 8, 128), (16, 8, 128), (4, 2, 64)])
def test_qk_norm_rope_store(dev, dtype, Hq, Hkv, D):
    from zipage_amd.layers import qk_norm_rope_store
    torch.manual_seed(Hq + D)
    N, pages, BS, max_pos, W, rows = 37, 6, 16, 500, 4, 5
    qkv = torch.randn(N, (Hq + 2 * Hkv) * D, device=dev).to(dtype)
    qn = (1 + 0.1 * torch.randn(D, device=dev)).to(dtype)
    kn = (1 + 0.1 * torch.randn(D, device=dev)).to(dtype)
    inv = 1.0 / (1e6 ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    ang = torch.arange(max_pos, dtype=torch.float32)[:, None] * inv[None, :]
    cos, sin = ang.cos().to(dev), ang.sin().to(dev)
    pos = torch.randint(0, max_pos, (N,), device=dev, dtype=torch.int32)
    slots = torch.randperm(pages * BS, device=dev)[:N].int()
    slots[::5] = -1
    tri = torch.full((N, 3), -1, device=dev, dtype=torch.int32)
    for i in range(0, N, 3):
        tri[i] = torch.tensor([i, i % rows, (i // 3) % W])
    k_cache = torch.randn(pages, BS, Hkv, D, device=dev).to(dtype)
    v_cache = torch.randn(pages, BS, Hkv, D, device=dev).to(dtype)
    q_cache = torch.randn(rows, W, Hq, D, device=dev).to(dtype)
    # unfused module sequence
    q = qkv[:, :Hq * D].view(N, Hq, D)
    k = qkv[:, Hq * D:(Hq + Hkv) * D].view(N, Hkv, D)
    v = qkv[:, (Hq + Hkv) * D:].view(N, Hkv, D)
    c, s = cos[pos.long()].unsqueeze(1), sin[pos.long()].unsqueeze(1)
    wq = _rope_ref(_rms_ref(q, qn, 1e-6), c, s)
    wk = _rope_ref(_rms_ref(k, kn, 1e-6), c, s)
    wkc, wvc, wqc = k_cache.clone(), v_cache.clone(), q_cache.clone()
    keep = slots >= 0
    wkc.view(-1, Hkv, D)[slots[keep].long()] = wk[keep]
    wvc.view(-1, Hkv, D)[slots[keep].long()] = v[keep]
    for i in range(0, N, 3):
        wqc[i % rows, (i // 3) % W] = wq[i]
    got = qk_norm_rope_store(qkv, pos, cos, sin, qn, kn, Hq, Hkv, D, 1e-6, k_cache, v_cache, slots,
                             q_cache, tri)
    worst, same = _rope_ulps(got, wq)
    assert worst <= 2.0 and same > 0.99
    assert torch.equal(v_cache, wvc)
    worst, same = _rope_ulps(k_cache, wkc)
    assert worst <= 2.0 and same > 0.99
    touched = torch.zeros(pages * BS, dtype=torch.bool, device=dev)
    touched[slots[keep].long()] = True
    assert torch.equal(k_cache.view(-1, Hkv, D)[~touched], wkc.view(-1, Hkv, D)[~touched])
    # the ring holds exactly the q rows the kernel returned
    for i in range(0, N, 3):
        assert torch.equal(q_cache[i % rows, (i // 3) % W], got[i])
    # without caches: prefill-style call on a model that has none attached
    got2, k2 = qk_norm_rope_store(qkv, pos, cos, sin, qn, kn, Hq, Hkv, D, 1e-6, return_k=True)
    assert torch.equal(got2, got)
    assert torch.equal(k2[keep], k_cache.view(-1, Hkv, D)[slots[keep].long()])
    worst, same = _rope_ulps(k2, wk)
    assert worst <= 2.0 and same > 0.99
