"""The C-ABI library loads and exports every symbol include/zipage_hip.h declares.
No compute calls: this runs without a GPU."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "zipage_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(zp_[a-z_0-9]+)\s*\(", text)))


def test_header_declares_expected_entry_points():
    names = _declared()
    for n in ["zp_store_query", "zp_attention_score", "zp_global_score", "zp_pool_scores",
              "zp_key_norm", "zp_redundancy_lightning", "zp_redundancy_raw", "zp_score_epilogue",
              "zp_topk_mask", "zp_compress_kv", "zp_compress_score", "zp_last_error",
              "zp_abi_version"]:
        assert n in names


def test_library_exports_every_declared_symbol():
    from zipage_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.fail(f"{_lib.LIB_PATH} not built (python -m zipage_amd.build)")
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in _declared():
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert sorted(_lib.EXPORTS) == _declared()


def test_version_and_error_string():
    from zipage_amd import _lib
    lib = _lib.load()
    assert lib.zp_abi_version() >= 2
    assert isinstance(lib.zp_last_error(), bytes)


def test_argument_validation_needs_no_gpu():
    """Bad arguments are rejected on the host before any launch."""
    from zipage_amd import _lib
    lib = _lib.load()
    rc = lib.zp_topk_mask(None, None, 4, 16, 17, 0, None)
    assert rc == 1 and b"k=17" in lib.zp_last_error()
    rc = lib.zp_global_score(1, 1, 1, 1, 1, 1, 1, 256, 8, 4, 0, 0, 1.5, 0, 1, 0, None)
    assert rc == 1 and b"decay_factor" in lib.zp_last_error()


def test_product_has_no_cpu_fallback():
    import torch
    from zipage_amd.kernel import topk_mask
    with pytest.raises(RuntimeError, match="device tensors"):
        topk_mask(torch.zeros(2, 8), 3)
