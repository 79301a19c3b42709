"""The benchmark configurations at their full sizes, on the GPU, through the C ABI.

The CPU oracle cannot run these shapes whole in test time, so each configuration is checked through properties that
do not depend on the size, plus the oracle on a slice that is cheap because heads and sequences are independent:
  * split-run continuity: a sequence processed in two calls with the state handed over equals the single call
    (the split lies on a chunk boundary, so every chunk sees the same operands: bit-exact);
  * linearity: with q, k, g, beta fixed the operator is linear in (v, h0) and its backward in (dO, dht); a factor of
    two is exact in binary floating point, so outputs and gradients must double bit for bit;
  * packed == separate: a packed batch equals its sequences run one by one;
  * head / batch slices against the fp32 oracle with the tolerances of the small-shape parity tests.
"""
import pytest
import torch

from mindspeed_mm_amd.inputs import gdn_inputs, packed_lengths
from oracle import gdn_oracle as O
from parity import BF16_ABS_GRAD, BF16_ABS_O, _err

pytestmark = pytest.mark.gpu
BF = torch.bfloat16
NAMES = ("q", "k", "v", "g", "beta")


@pytest.fixture(scope="module")
def ops():
    from mindspeed_mm_amd.ops import _default_ops
    return _default_ops()


def _run(ops, d, h0, cu=None, backward=False, do=None, dht=None):
    leaves = {n: d[n].clone().requires_grad_(backward) for n in NAMES}
    h = h0.clone().requires_grad_(backward) if h0 is not None else None
    o, ht = ops.chunk_gated_delta_rule(leaves["q"], leaves["k"], leaves["v"], leaves["g"], leaves["beta"],
                                       initial_state=h, output_final_state=True, use_qk_l2norm_in_kernel=True,
                                       cu_seqlens=cu)
    if not backward:
        return o, ht
    outs, gouts = [o], [do]
    if dht is not None:
        outs.append(ht)
        gouts.append(dht)
    grads = torch.autograd.grad(outs, [leaves[n] for n in NAMES] + [h], gouts)
    return o, ht, dict(zip(NAMES + ("h0",), grads))


def _oracle_slice(x, b, hq, grp, cu=None, n_sel=None):
    """fp32 oracle on batch row b, q/k head hq and its grp value heads (heads and rows are independent)."""
    hs = slice(hq * grp, (hq + 1) * grp)
    L = {"q": x["q"][b:b + 1, :, hq:hq + 1], "k": x["k"][b:b + 1, :, hq:hq + 1], "v": x["v"][b:b + 1, :, hs],
         "g": x["g"][b:b + 1, :, hs], "beta": x["beta"][b:b + 1, :, hs]}
    L = {n: t.float().clone().requires_grad_(True) for n, t in L.items()}
    rows = slice(b, b + 1) if n_sel is None else n_sel
    h0 = x["h0"][rows, hs].clone().requires_grad_(True)
    o, ht = O.chunk_gated_delta_rule_ref(L["q"], L["k"], L["v"], L["g"], L["beta"], initial_state=h0,
                                         output_final_state=True, use_qk_l2norm_in_kernel=True, cu_seqlens=cu)
    return L, h0, o, ht


def test_config1_chunk_fwd_bwd_full_size(ops):
    """BASELINE configs[1]: B=2, T=8192, H_qk=16, H_v=32, d=128, bf16, fwd+bwd."""
    B, T, Hqk, Hv, K, V = 2, 8192, 16, 32, 128, 128
    x = gdn_inputs(B, T, Hqk, Hv, K, V, BF, seed=0)
    d = {n: t.cuda() for n, t in x.items()}
    o, ht, gr = _run(ops, d, d["h0"], backward=True, do=d["do"], dht=d["dht"])
    assert torch.isfinite(o.float()).all() and torch.isfinite(ht).all()

    # split-run continuity at a chunk boundary
    half = {n: d[n][:, :T // 2].contiguous() for n in NAMES}
    rest = {n: d[n][:, T // 2:].contiguous() for n in NAMES}
    o1, s1 = _run(ops, half, d["h0"])
    o2, s2 = _run(ops, rest, s1)
    assert torch.equal(torch.cat([o1, o2], 1), o) and torch.equal(s2, ht)

    # linearity in (v, h0) forward and in (dO, dht) backward: exact doubling
    d2 = dict(d, v=d["v"] * 2)
    o_2, ht_2 = _run(ops, d2, d["h0"] * 2)
    assert torch.equal(o_2, o * 2) and torch.equal(ht_2, ht * 2)
    _, _, gr2 = _run(ops, d, d["h0"], backward=True, do=d["do"] * 2, dht=d["dht"] * 2)
    for n in gr:
        assert torch.equal(gr2[n], gr[n] * 2), n

    # oracle on one batch row and one q/k group (2 value heads), all 128 chunks
    b, hq, grp = 1, 5, Hv // Hqk
    L, h0, ro, rht = _oracle_slice(x, b, hq, grp)
    hs = slice(hq * grp, (hq + 1) * grp)
    rg = torch.autograd.grad([ro, rht], list(L.values()) + [h0], [x["do"][b:b + 1, :, hs].float(), x["dht"][b:b + 1, hs]])
    rg = dict(zip(NAMES + ("h0",), rg))
    _err("o", o[b:b + 1, :, hs], ro, BF, BF16_ABS_O)
    _err("final_state", ht[b:b + 1, hs], rht, BF, BF16_ABS_O)
    _err("dq", gr["q"][b:b + 1, :, hq:hq + 1], rg["q"], BF, BF16_ABS_GRAD)
    _err("dk", gr["k"][b:b + 1, :, hq:hq + 1], rg["k"], BF, BF16_ABS_GRAD)
    for n in ("v", "g", "beta"):
        _err("d" + n, gr[n][b:b + 1, :, hs], rg[n], BF, BF16_ABS_GRAD)
    _err("dh0", gr["h0"][b:b + 1, hs], rg["h0"], BF, BF16_ABS_GRAD)


def test_config2_packed_sequences_full_size(ops):
    """BASELINE configs[2]: 32768 packed tokens in 24 sequences of ragged lengths, H_qk=16, H_v=32, d=128, bf16."""
    cu = packed_lengths()
    N, total, Hqk, Hv, K, V = len(cu) - 1, cu[-1], 16, 32, 128, 128
    x = gdn_inputs(1, total, Hqk, Hv, K, V, BF, seed=2, N=N)
    d = {n: t.cuda() for n, t in x.items()}
    cu_t = torch.tensor(cu, dtype=torch.int64, device="cuda")
    o, ht, gr = _run(ops, d, d["h0"], cu=cu_t, backward=True, do=d["do"], dht=d["dht"])

    # packed == every sequence on its own (same chunking inside a sequence: bit-exact)
    for n in range(N):
        a, b = cu[n], cu[n + 1]
        one = {m: d[m][:, a:b].contiguous() for m in NAMES}
        o_n, ht_n, gr_n = _run(ops, one, d["h0"][n:n + 1], backward=True, do=d["do"][:, a:b].contiguous(),
                               dht=d["dht"][n:n + 1])
        assert torch.equal(o_n, o[:, a:b]) and torch.equal(ht_n, ht[n:n + 1]), n
        for m in NAMES:
            assert torch.equal(gr_n[m], gr[m][:, a:b]), (n, m)
        assert torch.equal(gr_n["h0"], gr["h0"][n:n + 1]), n

    # oracle on the two shortest sequences, one q/k group
    lens = [cu[n + 1] - cu[n] for n in range(N)]
    for n in sorted(range(N), key=lambda i: lens[i])[:2]:
        a, b = cu[n], cu[n + 1]
        hq, grp = 7, Hv // Hqk
        hs = slice(hq * grp, (hq + 1) * grp)
        xs = {m: x[m][:, a:b] for m in NAMES}
        xs["h0"] = x["h0"]
        L, h0, ro, rht = _oracle_slice(xs, 0, hq, grp, n_sel=slice(n, n + 1))
        rg = torch.autograd.grad([ro, rht], list(L.values()) + [h0],
                                 [x["do"][:, a:b, hs].float(), x["dht"][n:n + 1, hs]])
        rg = dict(zip(NAMES + ("h0",), rg))
        _err("o", o[:, a:b, hs], ro, BF, BF16_ABS_O)
        _err("final_state", ht[n:n + 1, hs], rht, BF, BF16_ABS_O)
        _err("dq", gr["q"][:, a:b, hq:hq + 1], rg["q"], BF, BF16_ABS_GRAD)
        _err("dk", gr["k"][:, a:b, hq:hq + 1], rg["k"], BF, BF16_ABS_GRAD)
        for m in ("v", "g", "beta"):
            _err("d" + m, gr[m][:, a:b, hs], rg[m], BF, BF16_ABS_GRAD)


def test_config2_conv1d_packed_full_size(ops):
    """BASELINE configs[2], conv part: packed [1, 32768, 8192], W=4, SiLU, fwd+bwd; packed == sequences one by one."""
    cu = packed_lengths()
    D, W = 8192, 4
    gen = torch.Generator().manual_seed(2)
    xx = torch.randn(1, cu[-1], D, generator=gen).to("cuda", BF).requires_grad_(True)
    ww = (torch.randn(W, D, generator=gen) / 2).to("cuda", BF).requires_grad_(True)
    dy = torch.randn(1, cu[-1], D, generator=gen).to("cuda", BF)
    cu_t = torch.tensor(cu, dtype=torch.int64, device="cuda")
    y, _ = ops.causal_conv1d(xx, ww, None, None, None, "silu", cu_t, False)
    dx, dw = torch.autograd.grad([y], [xx, ww], [dy])
    for n in (0, 5, len(cu) - 2):
        a, b = cu[n], cu[n + 1]
        xs = xx.detach()[:, a:b].contiguous().requires_grad_(True)
        ys, _ = ops.causal_conv1d(xs, ww, None, None, None, "silu", None, False)
        dxs, _ = torch.autograd.grad([ys], [xs, ww], [dy[:, a:b].contiguous()])
        assert torch.equal(ys, y[:, a:b]) and torch.equal(dxs, dx[:, a:b]), n
    # dw over the packed batch against the eager definition on a channel slice (fp32)
    ch = slice(0, 64)
    xr = xx.detach()[0, :, ch].float().cpu().requires_grad_(True)
    wr = ww.detach()[:, ch].float().cpu().requires_grad_(True)
    yr = O.causal_conv1d_ref(xr[None], wr, None, None, None, "silu", cu, False)[0]
    dxr, dwr = torch.autograd.grad([yr], [xr, wr], [dy[:, :, ch].float().cpu()])
    _err("y", y[0, :, ch], yr[0], BF, 1e-2, rtol=1e-2)
    _err("dx", dx[0, :, ch], dxr, BF, 2e-2, rtol=1e-2)
    _err("dw", dw[:, ch], dwr, BF, 1e-2 * dwr.abs().max().item(), rtol=1e-2)


def test_config3_decode_batch256_64_steps(ops):
    """BASELINE configs[3]: batch 256, one token per sequence per step, 64 steps, state updated in place."""
    B, S, Hqk, Hv, K, V = 256, 64, 16, 32, 128, 128
    x = gdn_inputs(B, S, Hqk, Hv, K, V, BF, seed=3)
    d = {n: t.cuda() for n, t in x.items()}
    state = d["h0"].clone()
    outs = []
    for t in range(S):
        tok = {n: d[n][:, t:t + 1].contiguous() for n in NAMES}
        o, s = ops.fused_recurrent_gated_delta_rule(tok["q"], tok["k"], tok["v"], tok["g"], tok["beta"],
                                                    initial_state=state, output_final_state=True,
                                                    use_qk_l2norm_in_kernel=True, inplace_state=True)
        assert s.data_ptr() == state.data_ptr()
        outs.append(o)
    o_steps = torch.cat(outs, 1)
    # 64 single-token calls == one 64-token call (same arithmetic per token: bit-exact)
    o_all, s_all = ops.fused_recurrent_gated_delta_rule(d["q"], d["k"], d["v"], d["g"], d["beta"],
                                                        initial_state=d["h0"], output_final_state=True,
                                                        use_qk_l2norm_in_kernel=True)
    assert torch.equal(o_steps, o_all) and torch.equal(state, s_all)
    # oracle on a batch slice
    bs = slice(100, 104)
    ro, rs = O.recurrent_gated_delta_rule_ref(x["q"][bs].float(), x["k"][bs].float(), x["v"][bs].float(), x["g"][bs],
                                              x["beta"][bs].float(), x["h0"][bs], True, True)
    _err("o", o_steps[bs], ro, BF, BF16_ABS_O)
    _err("state", state[bs], rs, torch.float32, 0)


def test_config4_long_sequence_wide_heads(ops):
    """BASELINE configs[4]: B=1, T=65536, H_qk=16, H_v=64, d_k=128, d_v=256, bf16, fwd+bwd (1024 chunks)."""
    B, T, Hqk, Hv, K, V = 1, 65536, 16, 64, 128, 256
    x = gdn_inputs(B, T, Hqk, Hv, K, V, BF, seed=4, a_log=(0.5, 2.0), dt_bias=(-6.0, -4.0))
    d = {n: t.cuda() for n, t in x.items()}
    o, ht, gr = _run(ops, d, d["h0"], backward=True, do=d["do"], dht=d["dht"])
    assert torch.isfinite(o.float()).all() and torch.isfinite(ht).all()
    for n in gr:
        assert torch.isfinite(gr[n].float()).all(), n

    quarter = T // 4   # four calls with the state handed over == one call
    s, parts = d["h0"], []
    for i in range(4):
        part = {n: d[n][:, i * quarter:(i + 1) * quarter].contiguous() for n in NAMES}
        oi, s = _run(ops, part, s)
        parts.append(oi)
    assert torch.equal(torch.cat(parts, 1), o) and torch.equal(s, ht)

    _, _, gr2 = _run(ops, d, d["h0"], backward=True, do=d["do"] * 2, dht=d["dht"] * 2)
    for n in gr:
        assert torch.equal(gr2[n], gr[n] * 2), n

    # backward continuity: the second half's gradient w.r.t. its initial state is the first half's dht
    half = T // 2
    first = {n: d[n][:, :half].contiguous() for n in NAMES}
    second = {n: d[n][:, half:].contiguous() for n in NAMES}
    _, s_mid = _run(ops, first, d["h0"])
    _, _, g2 = _run(ops, second, s_mid, backward=True, do=d["do"][:, half:].contiguous(), dht=d["dht"])
    _, _, g1 = _run(ops, first, d["h0"], backward=True, do=d["do"][:, :half].contiguous(), dht=g2["h0"])
    for n in NAMES:
        assert torch.equal(torch.cat([g1[n], g2[n]], 1), gr[n]), n
    assert torch.equal(g1["h0"], gr["h0"])

    # oracle (forward; its autograd over 1024 chunks takes minutes) on one q/k group of 4 value heads:
    # o and the final state after 1024 chunks
    hq, grp = 9, Hv // Hqk
    hs = slice(hq * grp, (hq + 1) * grp)
    with torch.no_grad():
        ro, rht = O.chunk_gated_delta_rule_ref(x["q"][:, :, hq:hq + 1].float(), x["k"][:, :, hq:hq + 1].float(),
                                               x["v"][:, :, hs].float(), x["g"][:, :, hs], x["beta"][:, :, hs].float(),
                                               initial_state=x["h0"][:, hs], output_final_state=True,
                                               use_qk_l2norm_in_kernel=True)
    _err("o", o[:, :, hs], ro, BF, BF16_ABS_O)
    _err("final_state", ht[:, hs], rht, BF, BF16_ABS_O)


def test_kda_full_size(ops):
    """The KDA benchmark shape (B=2, T=8192, H=32, d=128, bf16, the layer's options) forward and backward: split-run
    continuity, exact linearity, and the oracle on one head (heads are independent; the gradients of A_log and dt_bias of
    a head sum over the batch rows, which the slice keeps both of)."""
    from mindspeed_mm_amd.inputs import kda_inputs
    from oracle import kda_oracle as KO
    from parity import kda_param_tol
    B, T, H, K, V = 2, 8192, 32, 128, 128
    x = kda_inputs(B, T, H, K, V, BF, seed=11)
    x["h0"], x["dht"] = (x[n].transpose(-1, -2).contiguous() for n in ("h0", "dht"))     # [N,H,V,K] as the layer keeps them
    d = {n: t.cuda() for n, t in x.items()}
    names = ("q", "k", "v", "g", "beta", "A_log", "dt_bias", "h0")
    kw = dict(output_final_state=True, use_qk_l2norm_in_kernel=True, use_gate_in_kernel=True,
              use_beta_sigmoid_in_kernel=True, transpose_state_layout=True)

    def run(t, h0, backward=False, do=None, dht=None):
        L = {n: t[n].clone().requires_grad_(backward) for n in names[:-1]}
        h = h0.clone().requires_grad_(backward)
        with torch.set_grad_enabled(backward):
            o, ht = ops.chunk_kda(L["q"], L["k"], L["v"], L["g"], L["beta"], initial_state=h, A_log=L["A_log"],
                                  dt_bias=L["dt_bias"], **kw)
        if not backward:
            return o, ht
        grads = torch.autograd.grad([o, ht], [L[n] for n in names[:-1]] + [h], [do, dht])
        return o, ht, dict(zip(names, grads))

    o, ht, gr = run(d, d["h0"], True, d["do"], d["dht"])
    assert torch.isfinite(o.float()).all() and torch.isfinite(ht).all()
    assert all(torch.isfinite(g.float()).all() for g in gr.values())

    # split-run continuity at a chunk boundary: every chunk sees the same operands
    tok = ("q", "k", "v", "g", "beta")
    half = dict(d, **{n: d[n][:, :T // 2].contiguous() for n in tok})
    rest = dict(d, **{n: d[n][:, T // 2:].contiguous() for n in tok})
    o1, s1 = run(half, d["h0"])
    o2, s2 = run(rest, s1)
    assert torch.equal(torch.cat([o1, o2], 1), o) and torch.equal(s2, ht)

    # linear in (v, h0) forward and in (dO, dht) backward: a factor of two is exact
    o_2, ht_2 = run(dict(d, v=d["v"] * 2), d["h0"] * 2)
    assert torch.equal(o_2, o * 2) and torch.equal(ht_2, ht * 2)
    _, _, gr2 = run(d, d["h0"], True, d["do"] * 2, d["dht"] * 2)
    for n in gr:
        assert torch.equal(gr2[n], gr[n] * 2), n

    # the oracle on head hs of both batch rows, all 128 chunks
    hs = 7
    R = {n: x[n][:, :, hs:hs + 1].clone().requires_grad_(True) for n in tok}
    R["A_log"] = x["A_log"][hs:hs + 1].clone().requires_grad_(True)
    R["dt_bias"] = x["dt_bias"][hs * K:(hs + 1) * K].clone().requires_grad_(True)
    R["h0"] = x["h0"][:, hs:hs + 1].clone().requires_grad_(True)
    ro, rht = KO.chunk_kda_ref(R["q"], R["k"], R["v"], R["g"], R["beta"], initial_state=R["h0"], A_log=R["A_log"],
                               dt_bias=R["dt_bias"], round_output=False, **kw)
    rg = torch.autograd.grad([ro, rht], [R[n] for n in names], [x["do"][:, :, hs:hs + 1].float(), x["dht"][:, hs:hs + 1]])
    rg = dict(zip(names, rg))
    _err("o", o[:, :, hs:hs + 1], ro, BF, BF16_ABS_O)
    _err("final_state", ht[:, hs:hs + 1], rht, BF, BF16_ABS_O)
    for n in tok:
        _err("d" + n, gr[n][:, :, hs:hs + 1], rg[n], BF, BF16_ABS_GRAD)
    _err("dh0", gr["h0"][:, hs:hs + 1], rg["h0"], BF, BF16_ABS_GRAD)
    _err("dA_log", gr["A_log"][hs:hs + 1], rg["A_log"], BF, kda_param_tol(rg["A_log"], B * T))
    _err("ddt_bias", gr["dt_bias"][hs * K:(hs + 1) * K], rg["dt_bias"], BF, kda_param_tol(rg["dt_bias"], B * T))


def test_config4_shape_backward_against_the_oracle(ops):
    """The long-context shape's head geometry and decay (one q/k group of BASELINE configs[4]: H_qk=1, H_v=4, d_k=128,
    d_v=256, A_log ~ U(log 0.5, log 2), dt_bias ~ U(-6, -4)) at T=8192, forward and backward against the oracle and
    autograd through it: at the full T=65536 the gradients are held to linearity and continuity only, which a term
    that is wrong but linear and consistent across splits would pass; 128 slowly decaying chunks are where such a term
    would show."""
    from parity import check_chunk
    # with this slow decay dg reaches 15 and more: the absolute bound alone would ask for more than the 8 bits of the
    # operands give, so the gradients are held to 5e-2 + 1e-2 |ref| (the relative part is the reference test's own,
    # tests/ut_fsdp/models/qwen3_5/test_chunk_gated_delta_rule.py:236-247)
    errs = check_chunk(ops, "cuda", 1, 8192, 1, 4, 128, 256, BF, l2=True, backward=True, seed=14, grad_rtol=1e-2,
                       a_log=(0.5, 2.0), dt_bias=(-6.0, -4.0))
    print({n: f"{e:.2e}" for n, e in errs.items()})


def test_kda_gate_parameter_gradients_fp32_full_length(ops):
    """dA_log and d(dt_bias) sum terms of both signs over every token; in bf16 they are held to a calibrated bound that
    grows with the number of chunks.  The float32 kernels run the same reductions (per-chunk partial sums, then the
    sum over the chunks) and are held to 1e-4 here at the benchmark's length, T=8192, on one head."""
    from parity import check_kda
    errs = check_kda(ops, "cuda", 1, 8192, 1, 128, 128, torch.float32, backward=True, seed=12)
    print({n: f"{e:.2e}" for n, e in errs.items()})

