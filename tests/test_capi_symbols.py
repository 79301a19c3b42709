"""The C-ABI library must load and export every symbol include/gdn_mi355x.h declares, with the binding's
signature table covering exactly that set (no compute calls here: no GPU needed)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "gdn_mi355x.h")


def declared():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(gdn_[a-z0-9_]+)\s*\(", src)))


def test_header_declares_the_operator_entry_points():
    names = declared()
    for n in ("gdn_chunk_fwd", "gdn_chunk_bwd", "gdn_recurrent_fwd", "gdn_conv1d_fwd", "gdn_conv1d_bwd",
              "gdn_conv1d_update", "gdn_chunk_workspace_bytes", "gdn_rmsnorm_gated_fwd", "gdn_rmsnorm_gated_bwd"):
        assert n in names


def test_binding_matches_header():
    from mindspeed_mm_amd._lib import SIGNATURES
    assert sorted(SIGNATURES) == declared()


def test_library_exports_every_symbol():
    from mindspeed_mm_amd._lib import LIB_PATH
    if not os.path.exists(LIB_PATH):
        pytest.fail(f"{LIB_PATH} is not built (run __graft_entry__.build())")
    lib = ctypes.CDLL(LIB_PATH)
    for n in declared():
        assert hasattr(lib, n), n
    lib.gdn_profile_kernel_count.restype = ctypes.c_int
    assert lib.gdn_profile_kernel_count() > 0
    lib.gdn_chunk_workspace_bytes.restype = ctypes.c_int64
    lib.gdn_chunk_workspace_bytes.argtypes = [ctypes.c_int] * 9
    fwd = lib.gdn_chunk_workspace_bytes(2, 8192, 2, 16, 32, 128, 128, 1, 0)
    both = lib.gdn_chunk_workspace_bytes(2, 8192, 2, 16, 32, 128, 128, 1, 1)
    assert 0 < fwd < both


def test_ops_refuse_host_tensors():
    """There is no CPU fallback: the shipped entry points reject tensors that are not on the GPU."""
    import torch
    from mindspeed_mm_amd._lib import LIB_PATH
    if not os.path.exists(LIB_PATH):
        pytest.fail("library not built")
    import mindspeed_mm_amd as M
    q = torch.randn(1, 64, 1, 64)
    with pytest.raises(RuntimeError, match="no host fallback"):
        M.chunk_gated_delta_rule(q, q, q, torch.zeros(1, 64, 1), torch.ones(1, 64, 1))
    with pytest.raises(RuntimeError, match="no host fallback"):
        M.causal_conv1d(torch.randn(1, 8, 8), torch.randn(4, 8))


def test_validation_errors_match_reference():
    """ValueError set of chunk_gated_delta_rule.py:379-414."""
    import torch
    import mindspeed_mm_amd as M
    q = torch.randn(1, 64, 1, 64, dtype=torch.bfloat16)
    g, b = torch.zeros(1, 64, 1), torch.ones(1, 64, 1)
    with pytest.raises(ValueError):
        M.chunk_gated_delta_rule(q, q.float(), q, g, b)
    with pytest.raises(ValueError):
        M.chunk_gated_delta_rule(q, q, q, g, b[..., None])
    q2 = torch.randn(2, 64, 1, 64, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        M.chunk_gated_delta_rule(q2, q2, q2, torch.zeros(2, 64, 1), torch.ones(2, 64, 1),
                                 cu_seqlens=torch.tensor([0, 64, 128]))
    with pytest.raises(ValueError):
        M.chunk_gated_delta_rule(q, q, q, g, b, cu_seqlens=torch.tensor([0, 30, 64]),
                                 initial_state=torch.zeros(3, 1, 64, 64))
    with pytest.raises(ValueError):
        M.causal_conv1d(torch.randn(1, 8, 8), torch.randn(4, 16))
