"""zp_compress_layers_static -- the entry point that allocates nothing (its scratch is a fixed
array in device memory owned by the library) -- against zp_compress_layers with a caller-passed
workspace: keep flags, K, V and the score cache bit for bit, on two calls in a row, the second
with a smaller input (the array keeps the first call's contents), and a clear refusal of a chunk
that does not fit.  Both entries are called through the C ABI."""
import ctypes

import pytest
import torch

from tests import cases

pytestmark = pytest.mark.gpu


def _case(dev, dtype, seed, L, B, kw, budget=2, W=16, Hkv=2, Hq=8, nb=(3, 4)):
    from zipage_amd.compress import CompressConfig
    tables, enc, target = cases.random_tables(seed, B, 48, list(nb), budget)
    k, v, q, sc = cases.make_caches(seed, L, 48, 256, Hkv, Hq, 128, W, B + 1, dtype,
                                    touched=cases.touched_pages(enc), with_score_cache=True)
    base = torch.randn((1, 1, 1, Hkv, 128), generator=torch.Generator().manual_seed(seed + 1))
    k = (k.float() * 0.8 + 0.6 * base).to(dtype)
    qid = torch.arange(B, dtype=torch.int32)
    comp = torch.tensor([i % 2 == 1 for i in range(B)])
    cfg = CompressConfig(budget_blocks=budget, query_cache_len=W, **kw)
    return [t.to(dev) for t in (k, v, q, sc, qid, enc, comp, target)], cfg


def _call(entry, tensors, cfg, flag_in_scratch=False, deterministic_carry=True, check_memory=False):
    """Runs `entry` on clones of the caches; returns (flag or None, k, v, score cache).  With
    ``check_memory`` the free device memory is read right before and right after the call."""
    from zipage_amd import _lib
    from zipage_amd.compress import c_config, layer_chunk_args
    k, v, q, sc, qid, enc, comp, target = tensors
    k, v, sc = k.clone(), v.clone(), sc.clone()
    dims, strides = layer_chunk_args(k, v, q, sc, qid, enc, comp, target)
    L, B, NB, BS, Hkv, Hq, D, W = dims[:8]
    cc = c_config(cfg, deterministic_carry=deterministic_carry)
    tag = _lib.dtype_tag(k)
    flag = None if flag_in_scratch else torch.zeros((L, B, Hkv, NB, BS), dtype=torch.bool, device=k.device)
    head = (k.data_ptr(), v.data_ptr(), q.data_ptr(), sc.data_ptr(), qid.data_ptr(), enc.data_ptr(),
            comp.data_ptr(), target.data_ptr(), 0 if flag is None else flag.data_ptr(), *dims,
            strides, tag, ctypes.byref(cc))
    stream = torch.cuda.current_stream().cuda_stream
    if entry == "static":
        torch.cuda.synchronize()
        free0 = torch.cuda.mem_get_info(k.device)[0]
        _lib.call("zp_compress_layers_static", *head, stream)
        torch.cuda.synchronize()
        if check_memory:   # nothing was allocated or released on the device, by anyone
            assert torch.cuda.mem_get_info(k.device)[0] == free0
    else:
        lib = _lib.load()
        need = lib.zp_compress_layers_workspace(L, B, NB, BS, Hkv, Hq, W, tag, ctypes.byref(cc),
                                                int(flag is None))
        ws = torch.empty(need, dtype=torch.uint8, device=k.device)
        _lib.call("zp_compress_layers", *head, ws.data_ptr(), need, None, stream)
    torch.cuda.synchronize()
    return flag, k, v, sc


SCRIPTS = dict(use_global_score=True, decay_factor=0.8, enable_pooling=True, use_redudancy=True,
               lightning_redudancy=True)
RAW = dict(use_global_score=True, use_redudancy=True, lightning_redudancy=False, enable_pooling=True,
           pooling_size=7, use_attention_sink=True)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_static_scratch_entry_matches_the_workspace_entry(dev, dtype):
    # first call: the larger input; second call: fewer, shorter sequences and other switches
    big, cfg_big = _case(dev, dtype, 5, L=2, B=6, kw=SCRIPTS)
    small, cfg_small = _case(dev, dtype, 6, L=1, B=2, kw=RAW, nb=(3,))
    from zipage_amd import _lib
    _lib.call("zp_static_scratch_init")     # the address look-up, outside any capture
    for tensors, cfg in ((big, cfg_big), (small, cfg_small)):
        want = _call("workspace", tensors, cfg)
        got = _call("static", tensors, cfg, check_memory=True)
        for name, a, b in zip(("flag", "k", "v", "score cache"), got, want):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), name
        assert (got[0].flatten(3).sum(-1) == 2 * 256).all()
        # flags kept inside the library's array: the caches still come out the same
        got2 = _call("static", tensors, cfg, flag_in_scratch=True)
        for name, a, b in zip(("k", "v", "score cache"), got2[1:], want[1:]):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), name


def test_static_scratch_entry_with_the_reference_carry(dev):
    """deterministic_carry off (the reference's store-then-read-back of the score cache, no page
    shared in this batch): the same bits as the workspace entry, twice in a row."""
    tensors, cfg = _case(dev, torch.bfloat16, 8, L=2, B=5, kw=SCRIPTS)
    for _ in range(2):
        want = _call("workspace", tensors, cfg, deterministic_carry=False)
        got = _call("static", tensors, cfg, deterministic_carry=False, check_memory=True)
        for name, a, b in zip(("flag", "k", "v", "score cache"), got, want):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), name


def test_static_scratch_entry_refuses_what_does_not_fit(dev):
    from zipage_amd import _lib
    from zipage_amd.compress import CompressConfig, c_config
    cc = c_config(CompressConfig(budget_blocks=8, query_cache_len=32, use_redudancy=True))
    lib = _lib.load()
    # 256 sequences x 10 pages with the all-pairs redundancy needs more than the array holds
    need = lib.zp_compress_layers_workspace(1, 256, 10, 256, 8, 32, 32, 0, ctypes.byref(cc), 1)
    assert need > _lib.STATIC_SCRATCH_BYTES
    one = torch.zeros(1, dtype=torch.int32, device=dev)
    strides = (ctypes.c_int64 * 14)(256 * 8 * 128 * 4, 256 * 8 * 128, 8 * 128, 128,
                                    256 * 8 * 128 * 4, 256 * 8 * 128, 8 * 128, 128,
                                    32 * 32 * 128, 32 * 32 * 128, 0, 0, 0, 0)
    p = one.data_ptr()
    rc = lib.zp_compress_layers_static(p, p, p, 0, p, p, p, p, 0, 1, 256, 10, 256, 8, 32, 128, 32,
                                       4, 1, 9, strides, 0, ctypes.byref(cc), 0)
    assert rc == 1 and b"bytes of scratch" in lib.zp_last_error()
