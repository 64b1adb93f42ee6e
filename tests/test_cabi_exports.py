"""The C-ABI library loads without a GPU and exports every symbol the header declares."""
import ctypes
import os
import re

from matchattention_amd import _cabi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "matchattn_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(matchattn_[a-z_0-9]+)\s*\(", text)))


def test_header_and_binding_list_the_same_symbols():
    assert _declared_symbols() == sorted(_cabi.SIGNATURES)


def test_library_exports_every_declared_symbol():
    assert os.path.exists(_cabi.LIB_PATH), "build first: python -m matchattention_amd.build"
    lib = ctypes.CDLL(_cabi.LIB_PATH)
    for name in _declared_symbols():
        assert hasattr(lib, name), name


def test_host_only_entry_points_work_without_a_gpu():
    lib = _cabi.load()
    assert lib.matchattn_abi_version() == _cabi.ABI_VERSION
    # fp32 needs no staging; 16-bit types stage dK and dV in fp32
    # head size without a tiled kernel: atomic mode only (fp32 accumulates in place; 16-bit types stage in fp32)
    assert lib.matchattn_backward_workspace_bytes(1, 8, 8, 48, 4, 1, 1, _cabi.F32) == 0
    assert lib.matchattn_backward_workspace_bytes(1, 8, 8, 48, 4, 1, 1, _cabi.F16) == 2 * 8 * 8 * 48 * 4
    # tiled shapes: per-tap scratch (nhq x M pairs: two floats in fp32, two halves otherwise) and the inverse index on top
    assert lib.matchattn_backward_workspace_bytes(1, 8, 8, 32, 4, 1, 1, _cabi.F16) > 8 * 8 * 4 * 16 * 4
    assert lib.matchattn_backward_workspace_bytes(1, 8, 8, 32, 4, 1, 1, _cabi.F32) > 8 * 8 * 4 * 16 * 8
    assert lib.matchattn_set_option(b"no_such_option", 1) == 1
    assert b"unknown option" in lib.matchattn_last_error()
    assert lib.matchattn_set_option(b"forward_variant", 3) == 1
    assert lib.matchattn_set_option(b"forward_variant", -1) == 0
    # argument validation happens before any GPU call
    assert lib.matchattn_forward(None, None, None, None, None, None, 1, 8, 8, 32, 4, 1, 1, 1.0, 0, None) == 1
    assert b"null" in lib.matchattn_last_error()
    assert lib.matchattn_forward(None, None, None, None, None, None, 1, 8, 8, 30, 4, 1, 1, 1.0, 0, None) == 1
    assert b"multiple" in lib.matchattn_last_error()


def test_python_boundary_rejects_what_the_library_cannot_do():
    import pytest
    import torch
    from matchattention_amd import MF_FusedForwardOps
    op = MF_FusedForwardOps()
    q = torch.zeros(1, 64, 8)
    mo = torch.zeros(1, 64, 1, 2)
    with pytest.raises(ValueError, match="GPU tensor"):
        op(mo, q, q, q, 8, 8, [1, 1], 16, "l1_norm", 1.0)
    with pytest.raises(ValueError, match="l1_norm"):
        op(mo, q, q, q, 8, 8, [1, 1], 16, "dot_product", 1.0)


def test_fused_entry_validates_before_any_gpu_call():
    import pytest
    import torch
    from matchattention_amd import fused_module_forward
    lib = _cabi.load()
    # maps below the LDS-tile path's sizes need no scratch (the kernel adds the pixel grid and clamps itself); on that
    # path the workspace covers the sampling positions (2 values per head-query) plus the forward's own
    assert lib.matchattn_forward_fused_workspace_bytes(1, 8, 8, 32, 4, 1, 1, _cabi.F16) == 0
    big = (1, 544, 960, 256, 8, 2, 2, _cabi.F16)
    assert lib.matchattn_forward_fused_workspace_bytes(*big) == 544 * 960 * 8 * 2 * 2 + lib.matchattn_forward_workspace_bytes(*big) > 0
    assert lib.matchattn_forward_fused(None, 4, None, None, None, None, None, 0, None, 0, None, 0, 1, 8, 8, 32, 4, 1, 1, 1.0, 1, None) == 1
    assert b"null" in lib.matchattn_last_error()
    import ctypes
    host = (ctypes.c_char * 16)()                    # any non-null address: these calls fail before touching it
    p = ctypes.addressof(host)
    assert lib.matchattn_forward_fused(p, 3, p, p, p, None, p, 0, p, 0, None, 0, 1, 8, 8, 32, 4, 1, 1, 1.0, 1, None) == 1
    assert b"position_heads" in lib.matchattn_last_error()
    assert lib.matchattn_forward_fused(p, 8, p, p, p, None, p, 0, p, 0, p, 16, 1, 544, 960, 256, 8, 2, 2, 1.0, 1, None) == 2
    assert b"workspace" in lib.matchattn_last_error()
    assert lib.matchattn_forward_fused(p, 0, p, p, p, None, p, -1, p, 0, None, 0, 1, 8, 8, 32, 4, 1, 1, 1.0, 1, None) == 1
    assert b"stride" in lib.matchattn_last_error()
    # host side: shapes and devices are checked in Python
    q = torch.zeros(1, 64, 32)
    with pytest.raises(ValueError, match="position must be"):
        fused_module_forward(torch.zeros(1, 64, 3, 2), q, q, q, 8, 8, [1, 1], 4, 1.0)
    with pytest.raises(ValueError, match="GPU tensor"):
        fused_module_forward(torch.zeros(1, 64, 1, 2), q, q, q, 8, 8, [1, 1], 4, 1.0)
