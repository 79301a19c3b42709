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


def test_packed_lengths_are_checked_on_the_host():
    """A cu_seqlens list or host tensor must start at 0, not decrease and stay within the packed tokens (no device
    synchronisation needed for the check); one that stops short of the packed length is a padded batch and passes:
    the kernels clear the rows behind it."""
    import torch
    import mindspeed_mm_amd as M
    q = torch.randn(1, 100, 1, 64, dtype=torch.bfloat16)
    g, b = torch.zeros(1, 100, 1), torch.ones(1, 100, 1)
    for bad in ([5, 30, 100], [0, 60, 30, 100], [0, 30, 101]):
        with pytest.raises(ValueError, match="cu_seqlens must start at 0, not decrease and end at or before"):
            M.chunk_gated_delta_rule(q, q, q, g, b, cu_seqlens=bad)
    with pytest.raises(ValueError, match="cu_seqlens must start at 0"):
        M.chunk_gated_delta_rule(q, q, q, g, b, cu_seqlens=torch.tensor([0, 30, 120]))
    for good in ([0, 30, 100], torch.tensor([0, 30, 90])):
        with pytest.raises(RuntimeError, match="no host fallback"):      # passes the check, then needs the GPU
            M.chunk_gated_delta_rule(q, q, q, g, b, cu_seqlens=good)


def test_autograd_functions_carry_the_guards():
    """Every autograd function runs with its tensors' device current and keeps the forward's autocast state in the
    backward pass (the reference's input_guard and custom_fwd / custom_bwd)."""
    from mindspeed_mm_amd import ops
    for cls in (ops._ChunkGatedDeltaRule, ops._ChunkGatedDeltaRuleNorm, ops._ChunkGatedDeltaRuleQKV, ops._GdnGates,
                ops._CausalConv1d, ops._RMSNormGated):
        for fn in (cls.forward, cls.backward):
            assert hasattr(fn, "__wrapped__"), (cls.__name__, fn.__name__)


def test_validation_of_the_layer_level_entry_points():
    """Shape and dtype errors of the operators around the rule are raised before anything touches a device."""
    import torch
    import mindspeed_mm_amd as M
    BF = torch.bfloat16
    mixed = torch.randn(1, 64, 2 * 64 + 64, dtype=BF)
    g, b = torch.zeros(1, 64, 1), torch.ones(1, 64, 1)
    with pytest.raises(ValueError):          # too narrow for q | k | v
        M.chunk_gated_delta_rule_qkv(mixed[..., :100], g, b, 1, 1, 64, 64)
    with pytest.raises(ValueError):          # g, beta of the wrong head count
        M.chunk_gated_delta_rule_qkv(mixed, torch.zeros(1, 64, 2), torch.ones(1, 64, 2), 1, 1, 64, 64)
    with pytest.raises(ValueError):          # packed input needs batch 1
        M.chunk_gated_delta_rule_qkv(torch.cat([mixed, mixed]), torch.zeros(2, 64, 1), torch.ones(2, 64, 1), 1, 1, 64, 64,
                                     cu_seqlens=torch.tensor([0, 64, 128]))
    with pytest.raises(RuntimeError, match="no host fallback"):
        M.chunk_gated_delta_rule_qkv(mixed, g, b, 1, 1, 64, 64)
    a = torch.randn(2, 5, 4, dtype=BF)
    with pytest.raises(ValueError):          # parameters of the wrong length
        M.gdn_gates(a, a, torch.zeros(3), torch.zeros(4))
    with pytest.raises(ValueError):          # a, b of different dtypes
        M.gdn_gates(a, a.float(), torch.zeros(4), torch.zeros(4))
    with pytest.raises(RuntimeError, match="no host fallback"):
        M.gdn_gates(a, a, torch.zeros(4), torch.zeros(4))
    with pytest.raises(ValueError):          # projections of the wrong shape for the decode step
        M.fused_recurrent_gated_delta_rule_qkv(mixed[:, :1], a[:1, :1], a[:1, :1], torch.zeros(4), torch.zeros(4),
                                               1, 1, 64, 64)


def test_decode_cache_bookkeeping():
    import torch
    from mindspeed_mm_amd import GdnDecodeCache
    c = GdnDecodeCache(3)
    assert len(c) == 3 and not c.has_previous_state(1)
    conv, rec = torch.arange(2 * 4 * 3.).reshape(2, 4, 3), torch.arange(2 * 1 * 2 * 2.).reshape(2, 1, 2, 2)
    c.set_prefill(1, conv, rec.to(torch.bfloat16))
    assert c.has_previous_state(1) and c.recurrent_states[1].dtype == torch.float32
    c.reorder_cache(torch.tensor([1, 1, 0]))
    assert torch.equal(c.conv_states[1], conv[[1, 1, 0]]) and torch.equal(c.recurrent_states[1], rec[[1, 1, 0]])
    assert c.conv_states[0] is None and c.recurrent_states[2] is None


def test_short_convolution_module_host_side():
    """Constructor, parameters and argument checks of the KDA layer's convolution module (short_conv.py:46-81,
    137-143), none of which touches a device; a host tensor then meets the operator's refusal."""
    import torch
    import mindspeed_mm_amd as M
    conv = M.ShortConvolution(32, 4, bias=True, activation="silu", backend="cuda", dtype=torch.bfloat16)
    assert isinstance(conv, torch.nn.Conv1d) and conv.groups == 32 and conv.padding == (3,)
    assert tuple(conv.weight.shape) == (32, 1, 4) and conv.weight.dtype == torch.bfloat16 and tuple(conv.bias.shape) == (32,)
    assert M.ShortConvolution(8, 2).bias is None and M.ShortConvolution(8, 2, activation=None).activation is None
    assert conv.state_size == 32 * 4 and "activation=silu" in repr(conv)
    with pytest.raises(AssertionError):
        M.ShortConvolution(8, 4, activation="relu")
    x = torch.randn(1, 10, 32, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="cannot be provided at the same time"):
        conv(x, mask=torch.ones(1, 10), cu_seqlens=torch.tensor([0, 4, 10]))
    with pytest.raises(RuntimeError, match="no host fallback"):
        conv(x)
    with pytest.raises(RuntimeError, match="no host fallback"):
        conv(x[:, :1])     # one token per sequence: the decoding call

