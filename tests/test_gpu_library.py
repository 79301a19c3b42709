"""The torch.library operators (torch.ops.mindspeed_mm_amd.*) against the autograd functions of the same package:
identical bits forward and backward, fake-tensor propagation, and a traced (torch.compile, aot_eager) run."""
import pytest
import torch

import mindspeed_mm_amd as M
from mindspeed_mm_amd import library as L
from tests import parity as P

pytestmark = pytest.mark.gpu
BF, F32 = torch.bfloat16, torch.float32


def _chunk_case(dtype, B, T, Hqk, Hv, K, V, cu, seed):
    N = (len(cu) - 1) if cu is not None else B
    x = P.gdn_inputs(B, T, Hqk, Hv, K, V, dtype, seed=seed, N=N)
    return {n: t.cuda() for n, t in x.items()}


def _run_chunk(fn, d, cu, with_h0):
    leaves = {n: d[n].clone().requires_grad_(True) for n in ("q", "k", "v", "g", "beta", "h0")}
    o, ht = fn(leaves["q"], leaves["k"], leaves["v"], leaves["g"], leaves["beta"],
               initial_state=leaves["h0"] if with_h0 else None, output_final_state=True, cu_seqlens=cu,
               use_qk_l2norm_in_kernel=True)
    ((o.float() * d["do"].float()).sum() + (ht * d["dht"]).sum()).backward()
    grads = {n: leaves[n].grad for n in leaves if not (n == "h0" and not with_h0)}
    return o, ht, grads


@pytest.mark.parametrize("dtype,B,T,Hqk,Hv,K,V,cu,with_h0", [
    (BF, 2, 300, 2, 4, 128, 128, None, True),
    (BF, 1, 200, 1, 2, 64, 128, [0, 70, 200], False),
    (F32, 1, 130, 1, 2, 128, 64, None, True),
])
def test_chunk_operator_equals_the_autograd_function(dtype, B, T, Hqk, Hv, K, V, cu, with_h0):
    d = _chunk_case(dtype, B, T, Hqk, Hv, K, V, cu, seed=31)
    o1, h1, g1 = _run_chunk(M.chunk_gated_delta_rule, d, cu, with_h0)
    o2, h2, g2 = _run_chunk(L.chunk_gated_delta_rule, d, cu, with_h0)
    assert torch.equal(o1, o2) and torch.equal(h1, h2)
    assert set(g1) == set(g2)
    for n in g1:
        assert g1[n].dtype == g2[n].dtype and torch.equal(g1[n], g2[n]), n
    with torch.no_grad():
        o3, h3 = L.chunk_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], use_qk_l2norm_in_kernel=True,
                                          cu_seqlens=cu)
    assert h3 is None and o3.shape == o1.shape


def test_chunk_operator_traces():
    """torch.compile carries the operator as one node (full graph, no break) and gives the eager bits, gradients
    included; the fake implementation is what shapes the trace."""
    d = _chunk_case(BF, 1, 256, 2, 4, 128, 128, None, seed=32)

    def f(q, k, v, g, beta):
        o, ht = L.chunk_gated_delta_rule(q * 1.0, k, v, g, beta, output_final_state=True, use_qk_l2norm_in_kernel=True)
        return o.float().sum() + ht.sum()

    args = [d[n].clone().requires_grad_(True) for n in ("q", "k", "v", "g", "beta")]
    want = f(*args)
    want.backward()
    grads = [a.grad.clone() for a in args]
    for a in args:
        a.grad = None
    got = torch.compile(f, backend="aot_eager", fullgraph=True)(*args)
    got.backward()
    assert torch.equal(want, got)
    for a, w in zip(args, grads):
        assert torch.equal(a.grad, w)


def test_operator_registrations_pass_opcheck():
    d = _chunk_case(BF, 1, 128, 1, 2, 64, 64, None, seed=33)
    args = (d["q"].requires_grad_(True), d["k"], d["v"], d["g"], d["beta"], 0.125, d["h0"], True, None, True, True)
    torch.library.opcheck(torch.ops.mindspeed_mm_amd.chunk_gated_delta_rule_fwd.default, args,
                          test_utils=("test_schema", "test_autograd_registration", "test_faketensor"))
    x = torch.randn(1, 64, 32, device="cuda", dtype=BF)
    w = torch.randn(4, 32, device="cuda", dtype=BF)
    torch.library.opcheck(torch.ops.mindspeed_mm_amd.causal_conv1d_fwd.default,
                          (x.requires_grad_(True), w, None, None, None, True, None, True),
                          test_utils=("test_schema", "test_autograd_registration", "test_faketensor"))
    state = torch.zeros(2, 32, 4, device="cuda", dtype=BF)
    torch.library.opcheck(torch.ops.mindspeed_mm_amd.causal_conv1d_update.default,
                          (torch.randn(2, 1, 32, device="cuda", dtype=BF), state, w.t().contiguous(), None, True),
                          test_utils=("test_schema", "test_faketensor"))


def test_decode_operator_equals_the_entry_point():
    x = P.gdn_inputs(1, 12, 1, 2, 128, 128, BF, seed=34, N=2)
    d = {n: t.cuda() for n, t in x.items()}
    cu = [0, 5, 12]
    o1, s1 = M.fused_recurrent_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], initial_state=d["h0"],
                                                output_final_state=True, use_qk_l2norm_in_kernel=True, cu_seqlens=cu)
    o2, s2 = L.fused_recurrent_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"], initial_state=d["h0"],
                                                output_final_state=True, use_qk_l2norm_in_kernel=True, cu_seqlens=cu)
    assert torch.equal(o1, o2) and torch.equal(s1, s2)
    o3, s3 = L.fused_recurrent_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"])
    assert s3 is None and o3.shape == o1.shape


@pytest.mark.parametrize("cu", [None, [0, 30, 100]])
def test_conv_operators_equal_the_entry_points(cu):
    gen = torch.Generator().manual_seed(35)
    B, T, D, W = (2, 100, 64, 4) if cu is None else (1, 100, 64, 4)
    N = B if cu is None else len(cu) - 1
    mk = lambda *s: torch.randn(*s, generator=gen).to(BF).cuda()
    x, w, b, res, h0, dy, dfs = mk(B, T, D), mk(W, D) / 2, mk(D), mk(B, T, D), mk(N, D, W), mk(B, T, D), mk(N, D, W)

    def run(fn):
        leaves = [t.clone().requires_grad_(True) for t in (x, w, b, res, h0)]
        y, fs = fn(leaves[0], leaves[1], leaves[2], leaves[3], leaves[4], "silu", cu, True)
        ((y.float() * dy.float()).sum() + (fs.float() * dfs.float()).sum()).backward()
        return y, fs, [t.grad for t in leaves]
    y1, f1, g1 = run(M.causal_conv1d)
    y2, f2, g2 = run(L.causal_conv1d)
    assert torch.equal(y1, y2) and torch.equal(f1, f2)
    for a, c in zip(g1, g2):
        assert a.dtype == c.dtype and torch.equal(a, c)
    # decode update: the state is rolled in place by both
    s1, s2 = h0.clone(), h0.clone()
    xt = mk(N, 1, D)
    u1 = M.causal_conv1d_update(xt, s1, w.t().contiguous(), b, "silu")
    u2 = L.causal_conv1d_update(xt, s2, w.t().contiguous(), b, "silu")
    assert torch.equal(u1, u2) and torch.equal(s1, s2) and not torch.equal(s1, h0)
