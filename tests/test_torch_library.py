"""The torch.library operators exist with tensor-only schemas and their fake implementations give the shapes and
dtypes of the real ones (checked on the meta device: no GPU, no kernel call)."""
import torch

import mindspeed_mm_amd  # noqa: F401  (registers the operators)


def _meta(*shape, dtype=torch.bfloat16):
    return torch.empty(*shape, dtype=dtype, device="meta")


def test_operators_are_registered_with_tensor_schemas():
    ns = torch.ops.mindspeed_mm_amd
    for name in ("chunk_gated_delta_rule_fwd", "chunk_gated_delta_rule_bwd", "fused_recurrent_gated_delta_rule",
                 "causal_conv1d_fwd", "causal_conv1d_bwd", "causal_conv1d_update"):
        schema = str(getattr(ns, name).default._schema)
        assert schema.startswith(f"mindspeed_mm_amd::{name}("), schema
    assert "Tensor(a1!) conv_state" in str(ns.causal_conv1d_update.default._schema)   # the state is declared as mutated


def test_fake_implementations_give_shapes_and_dtypes():
    ns = torch.ops.mindspeed_mm_amd
    q, v = _meta(2, 128, 2, 128), _meta(2, 128, 4, 128)
    g, beta = _meta(2, 128, 4, dtype=torch.float32), _meta(2, 128, 4)
    o, ht, ws = ns.chunk_gated_delta_rule_fwd(q, q, v, g, beta, 0.1, None, True, None, True, True)
    assert o.shape == v.shape and o.dtype == torch.bfloat16
    assert ht.shape == (2, 4, 128, 128) and ht.dtype == torch.float32
    assert ws.dtype == torch.uint8 and ws.numel() > 0      # the part of the workspace a backward call reuses
    cu = torch.empty(4, dtype=torch.int64, device="meta")
    o, ht, ws = ns.chunk_gated_delta_rule_fwd(q[:1], q[:1], v[:1], g[:1], beta[:1], 0.1, None, False, cu, True, False)
    assert ht.numel() == 0 and ws.numel() == 0
    h0 = _meta(2, 4, 128, 128, dtype=torch.float32)
    outs = ns.chunk_gated_delta_rule_bwd(q, q, v, g, beta, 0.1, h0, None, True, ws, v, None)
    assert [t.shape for t in outs] == [q.shape, q.shape, v.shape, g.shape, beta.shape, h0.shape]
    assert outs[3].dtype == torch.float32 and outs[4].dtype == torch.bfloat16
    o, s = ns.fused_recurrent_gated_delta_rule(q[:1, :5], q[:1, :5], v[:1, :5], g[:1, :5], beta[:1, :5], 0.1, None, True, cu, True)
    assert o.shape == (1, 5, 4, 128) and s.shape == (3, 4, 128, 128)
    x, w = _meta(1, 50, 64), _meta(4, 64)
    y, fs = ns.causal_conv1d_fwd(x, w, None, None, None, True, cu, True)
    assert y.shape == x.shape and fs.shape == (3, 64, 4)
    dx, dw, db, dh0 = ns.causal_conv1d_bwd(x, w, None, None, True, cu, x, None)
    assert dx.shape == x.shape and dw.shape == w.shape and db.numel() == 0 and dh0.numel() == 0
