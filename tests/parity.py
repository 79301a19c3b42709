"""Parity checks shared by the GPU tests (HIP library on cuda:0) and the CPU kernel-emulation tests.

Each check runs one operator of the package through the C ABI on seeded inputs and compares it with the
CPU oracle (oracle/gdn_oracle.py, oracle/kda_oracle.py).  Tolerances are the ones the task states:
    fp32: "max relative error <= 1e-4", checked in two readings at once:
          normalised   max|x - ref| <= 1e-4 max|ref|
          elementwise  |x - ref| <= 1e-4 |ref| + 1e-5 max|ref|   (the floor stands for entries that are themselves the
                       rounding residue of sums of terms of size max|ref|; an entry a hundred times smaller than the
                       largest is thereby held to 1e-3 of its own size, one ten thousand times smaller to 1e-1)
    bf16 vs the fp32 oracle on the same (bf16-valued) inputs: max abs error <= 2e-2 on o and on the final state,
          <= 5e-2 on dq/dk/dv/dg/dbeta (and on the gradient of the initial state).
"""
import torch

from mindspeed_mm_amd.inputs import gdn_inputs, kda_inputs
from oracle import gdn_oracle as O
from oracle import kda_oracle as KO

FP32_REL = 1e-4
FP32_FLOOR = 1e-5
BF16_ABS_O = 2e-2
BF16_ABS_GRAD = 5e-2
# dA_log and d(dt_bias) are sums over every token of the batch (dA_log over the channels too) of terms of both signs,
# each within the bound above: the error of the sum grows like a random walk, with the square root of the number of
# chunks, while the sum itself may cancel; 2 % on top, of the largest entry of the reference (the heads and channels
# draw their terms from one distribution, so the largest sum stands for the size of the terms also where an entry's own
# sum has cancelled)
KDA_PARAM_RTOL = 2e-2


def kda_param_tol(ref_grad, tokens):
    """Absolute bound for an entry of dA_log or d(dt_bias) in half precision.  Twice the per-entry bound per square root
    of the number of chunks: the oracle itself, evaluated in bf16 instead of fp32 on the seeded random cases of
    test_kda_random_shapes, moves dA_log by up to 0.2 at 400 tokens (the kernels by 0.02-0.2 on the same cases)."""
    return 2.0 * BF16_ABS_GRAD * max(1.0, tokens / 64.0) ** 0.5 + KDA_PARAM_RTOL * ref_grad.abs().max().item()


def _err(name, got, ref, dtype, abs_tol, rtol=0.0):
    """fp32: max|x-ref| <= 1e-4 max|ref| and |x-ref| <= 1e-4 |ref| + 1e-5 max|ref| elementwise.  Half precision:
    |x-ref| <= abs_tol + rtol |ref| elementwise."""
    got, ref = got.detach().float().cpu(), ref.detach().float().cpu()
    assert got.shape == ref.shape, f"{name}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(got).all(), f"{name}: non-finite values"
    diff = (got - ref).abs().max().item() if got.numel() else 0.0
    scale = ref.abs().max().item() if got.numel() else 0.0
    if dtype == torch.float32:
        assert diff <= FP32_REL * max(scale, 1e-30), f"{name}: max rel err {diff / max(scale, 1e-30):.3e} > {FP32_REL}"
        if got.numel():
            over = ((got - ref).abs() - FP32_REL * ref.abs()).max().item()
            assert over <= FP32_FLOOR * scale, (f"{name}: an entry is off by {over / max(scale, 1e-30):.3e} max|ref| beyond "
                                                f"{FP32_REL} of its own size (floor {FP32_FLOOR})")
    else:
        excess = ((got - ref).abs() - rtol * ref.abs()).max().item() if got.numel() else 0.0
        assert excess <= abs_tol, f"{name}: max abs err {diff:.3e} > {abs_tol} + {rtol}|ref| (ref max {scale:.3f})"
    return diff


def check_chunk(ops, device, B, T, Hqk, Hv, K, V, dtype, l2=True, cu=None, backward=False, seed=0, with_h0=True,
                scale=None, wrap=lambda t: t, skip_recompute=False, grad_rtol=0.0, **recipe):
    """grad_rtol: half precision only: the gradients are held to 5e-2 + grad_rtol |ref| instead of 5e-2 (for recipes whose
    gradients grow far beyond 1, where 5e-2 is below the resolution of the 16-bit operands)."""
    N = (len(cu) - 1) if cu is not None else B
    x = gdn_inputs(B, T, Hqk, Hv, K, V, dtype, seed=seed, N=N, l2norm_in_kernel=l2, **recipe)
    dev = {n: wrap(t.to(device)) for n, t in x.items()}
    leaves = {n: dev[n].clone().requires_grad_(backward) for n in ("q", "k", "v", "g", "beta")}
    h0 = dev["h0"].clone().requires_grad_(backward) if with_h0 else None
    cu_t = torch.tensor(cu, dtype=torch.int64, device=device) if cu is not None else None
    o, ht = ops.chunk_gated_delta_rule(leaves["q"], leaves["k"], leaves["v"], leaves["g"], leaves["beta"],
                                       scale=scale, initial_state=h0, output_final_state=True,
                                       use_qk_l2norm_in_kernel=l2, cu_seqlens=cu_t, skip_recompute=skip_recompute)
    ref_leaves = {n: x[n].float().clone().requires_grad_(backward) for n in ("q", "k", "v", "g", "beta")}
    rh0 = x["h0"].clone().requires_grad_(backward) if with_h0 else None
    ro, rht = O.chunk_gated_delta_rule_ref(ref_leaves["q"], ref_leaves["k"], ref_leaves["v"], ref_leaves["g"],
                                           ref_leaves["beta"], scale=scale, initial_state=rh0,
                                           output_final_state=True, use_qk_l2norm_in_kernel=l2, cu_seqlens=cu)
    assert o.dtype == dtype and ht.dtype == torch.float32
    errs = {"o": _err("o", o, ro, dtype, BF16_ABS_O), "ht": _err("final_state", ht, rht, dtype, BF16_ABS_O)}
    if backward:
        ((o.float() * dev["do"].float()).sum() + (ht * dev["dht"]).sum()).backward()
        ((ro * x["do"].float()).sum() + (rht * x["dht"]).sum()).backward()
        for n in ("q", "k", "v", "g", "beta"):
            assert leaves[n].grad.dtype == leaves[n].dtype
            errs["d" + n] = _err("d" + n, leaves[n].grad, ref_leaves[n].grad, dtype, BF16_ABS_GRAD, grad_rtol)
        if with_h0:
            errs["dh0"] = _err("dh0", h0.grad, rh0.grad, dtype, BF16_ABS_GRAD, grad_rtol)
    return errs


def check_chunk_reference_recipe(ops, device, B, T, H, K, V, l2, cu=None, oracle_heads=2, seed=42):
    """The reference's own test of the operator (tests/ut_fsdp/models/qwen3_5/test_chunk_gated_delta_rule.py:158-247):
    bf16, q, k, v ~ N(0,1) (q, k l2-normalised beforehand when the kernel is not asked to), beta = sigmoid(U(0,1)),
    g = logsigmoid(U(0,1)) in bf16, no initial state, loss = sum(o * do), seed 42.  All heads run on the device; the
    oracle runs on the first `oracle_heads` heads (heads are independent), which keeps its CPU time bounded.
    Checked against the task's bounds (2e-2 on o, 5e-2 on gradients, absolute) and against the reference test's own
    allclose(rtol=1e-2, atol=1e-2)."""
    dtype = torch.bfloat16
    gen = torch.Generator().manual_seed(seed)
    q, k = torch.randn(B, T, H, K, generator=gen), torch.randn(B, T, H, K, generator=gen)
    if not l2:
        q = q * torch.rsqrt((q * q).sum(-1, keepdim=True) + 1e-6)
        k = k * torch.rsqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    v = torch.randn(B, T, H, V, generator=gen)
    beta = torch.rand(B, T, H, generator=gen).to(dtype).sigmoid()
    g = torch.nn.functional.logsigmoid(torch.rand(B, T, H, generator=gen).to(dtype))
    do = torch.randn(B, T, H, V, generator=gen).to(dtype)
    x = dict(q=q.to(dtype), k=k.to(dtype), v=v.to(dtype), g=g, beta=beta)
    leaves = {n: t.to(device).requires_grad_(True) for n, t in x.items()}
    cu_t = torch.tensor(cu, dtype=torch.int64, device=device) if cu is not None else None
    o, _ = ops.chunk_gated_delta_rule(leaves["q"], leaves["k"], leaves["v"], leaves["g"], leaves["beta"],
                                      use_qk_l2norm_in_kernel=l2, cu_seqlens=cu_t)
    (o.float() * do.to(device).float()).sum().backward()
    hs = min(oracle_heads, H)
    ref = {n: t[:, :, :hs].float().clone().requires_grad_(True) for n, t in x.items()}
    ro, _ = O.chunk_gated_delta_rule_ref(ref["q"], ref["k"], ref["v"], ref["g"], ref["beta"],
                                         use_qk_l2norm_in_kernel=l2, cu_seqlens=cu)
    (ro * do[:, :, :hs].float()).sum().backward()
    assert o.dtype == dtype
    errs = {"o": _err("o", o[:, :, :hs], ro, dtype, BF16_ABS_O)}
    _err("o (reference test's allclose)", o[:, :, :hs], ro, dtype, 1e-2, 1e-2)
    for n in ("q", "k", "v", "g", "beta"):
        assert leaves[n].grad.dtype == leaves[n].dtype
        errs["d" + n] = _err("d" + n, leaves[n].grad[:, :, :hs], ref[n].grad, dtype, BF16_ABS_GRAD)
    return errs


def check_chunk_recompute_equals_stored(ops, device, B, T, Hqk, Hv, K, V, dtype, l2=True, cu=None, seed=0,
                                        wrap=lambda t: t, **recipe):
    """skip_recompute=False (nothing kept, the backward pass refills a workspace) against skip_recompute=True (the
    forward pass's workspace is kept): outputs and every gradient bit for bit."""
    N = (len(cu) - 1) if cu is not None else B
    x = gdn_inputs(B, T, Hqk, Hv, K, V, dtype, seed=seed, N=N, l2norm_in_kernel=l2, **recipe)
    dev = {n: wrap(t.to(device)) for n, t in x.items()}
    cu_t = torch.tensor(cu, dtype=torch.int64, device=device) if cu is not None else None
    res = []
    for skip in (False, True):
        L = {n: dev[n].clone().requires_grad_(True) for n in ("q", "k", "v", "g", "beta", "h0")}
        o, ht = ops.chunk_gated_delta_rule(L["q"], L["k"], L["v"], L["g"], L["beta"], initial_state=L["h0"],
                                           output_final_state=True, use_qk_l2norm_in_kernel=l2, cu_seqlens=cu_t,
                                           skip_recompute=skip)
        ((o.float() * dev["do"].float()).sum() + (ht * dev["dht"]).sum()).backward()
        res.append((o, ht, L))
    (o1, h1, L1), (o2, h2, L2) = res
    assert torch.equal(o1, o2) and torch.equal(h1, h2)
    for n in L1:
        assert torch.equal(L1[n].grad, L2[n].grad), f"gradient of {n} differs between the two modes"


def check_recurrent(ops, device, B, T, Hqk, Hv, K, V, dtype, l2=True, seed=0, with_state=True, wrap=lambda t: t):
    x = gdn_inputs(B, T, Hqk, Hv, K, V, dtype, seed=seed, l2norm_in_kernel=l2)
    dev = {n: wrap(t.to(device)) for n, t in x.items()}
    s0 = dev["h0"] if with_state else None
    o, s = ops.fused_recurrent_gated_delta_rule(dev["q"], dev["k"], dev["v"], dev["g"], dev["beta"], initial_state=s0,
                                                output_final_state=True, use_qk_l2norm_in_kernel=l2)
    ro, rs = O.recurrent_gated_delta_rule_ref(x["q"].float(), x["k"].float(), x["v"].float(), x["g"],
                                              x["beta"].float(), x["h0"] if with_state else None, True, l2)
    return {"o": _err("o", o, ro, dtype, BF16_ABS_O), "state": _err("state", s, rs, torch.float32, 0)}


def check_recurrent_packed(ops, device, T, cu, Hqk, Hv, K, V, dtype, l2=True, seed=0, with_state=True, wrap=lambda t: t):
    """The decode rule on one row of packed sequences against the oracle run sequence by sequence, each from its own
    state; tokens outside every listed sequence come back as zeros."""
    N = len(cu) - 1
    x = gdn_inputs(1, T, Hqk, Hv, K, V, dtype, seed=seed, N=N, l2norm_in_kernel=l2)
    dev = {n: wrap(t.to(device)) for n, t in x.items()}
    o, s = ops.fused_recurrent_gated_delta_rule(dev["q"], dev["k"], dev["v"], dev["g"], dev["beta"],
                                                initial_state=dev["h0"] if with_state else None, output_final_state=True,
                                                use_qk_l2norm_in_kernel=l2,
                                                cu_seqlens=torch.tensor(cu, dtype=torch.int64, device=device))
    ro = torch.zeros(1, T, Hv, V)
    rs = torch.zeros(N, Hv, K, V)
    for n in range(N):
        a, b = cu[n], cu[n + 1]
        h0 = x["h0"][n:n + 1] if with_state else None
        if b > a:
            ro[:, a:b], rs[n:n + 1] = O.recurrent_gated_delta_rule_ref(
                x["q"][:, a:b].float(), x["k"][:, a:b].float(), x["v"][:, a:b].float(), x["g"][:, a:b],
                x["beta"][:, a:b].float(), h0, True, l2)
        elif with_state:
            rs[n] = x["h0"][n]
    assert s.shape == rs.shape
    return {"o": _err("o", o, ro, dtype, BF16_ABS_O), "state": _err("state", s, rs, torch.float32, 0)}


def check_conv(ops, device, B, T, D, W, dtype, activation="silu", cu=None, bias=True, residual=False, state=True,
               backward=True, seed=0, wrap=lambda t: t):
    gen = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=gen)
    N = (len(cu) - 1) if cu is not None else B
    x = dict(x=r(B, T, D), w=r(W, D) / 2, b=r(D) if bias else None, res=r(B, T, D) if residual else None,
             h0=r(N, D, W) if state else None, dy=r(B, T, D), dfs=r(N, D, W))
    x = {n: (None if t is None else t.to(dtype)) for n, t in x.items()}
    cu_t = torch.tensor(cu, dtype=torch.int64, device=device) if cu is not None else None
    mk = lambda t, grad: None if t is None else wrap(t.to(device)).clone().requires_grad_(grad)
    dv = dict(x=mk(x["x"], backward), w=mk(x["w"], backward), b=mk(x["b"], backward), res=mk(x["res"], backward),
              h0=mk(x["h0"], backward))
    y, fs = ops.causal_conv1d(dv["x"], dv["w"], dv["b"], dv["res"], dv["h0"], activation, cu_t, True)
    rf = {n: (None if t is None else t.float().clone().requires_grad_(backward)) for n, t in x.items()
          if n in ("x", "w", "b", "res", "h0")}
    ry, rfs = O.causal_conv1d_ref(rf["x"], rf["w"], rf["b"], rf["res"], rf["h0"], activation, cu, True)
    # half precision: the reference's own bounds (test_forward.py:299-305, test_backward.py:88-89), applied as
    # allclose(atol, rtol) because outputs here reach |y| ~ 6 where one bf16 ulp is already 3e-2
    tol_f, tol_b, rt = 1e-2, 5e-2, 1e-2
    errs = {"y": _err("y", y, ry, dtype, tol_f, rt), "final_state": _err("final_state", fs, rfs, dtype, tol_f, rt)}
    if backward:
        ((y.float() * x["dy"].to(device).float()).sum() + (fs.float() * x["dfs"].to(device).float()).sum()).backward()
        ((ry * x["dy"].float()).sum() + (rfs * x["dfs"].float()).sum()).backward()
        for n in ("x", "w", "b", "res", "h0"):
            if dv[n] is not None:
                tol = tol_b * (max(1.0, B * T / 256) if n in ("w", "b") else 1.0)   # test_large_shape.py:156-158
                errs["d" + n] = _err("d" + n, dv[n].grad, rf[n].grad, dtype, tol, rt)
    return errs


def check_conv_update(ops, device, B, T, D, W, dtype, seed=0, wrap=lambda t: t, S=None):
    """S: length of the state rows (default W, the layer's; a longer state takes the kernel's general path)."""
    gen = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=gen)
    x, st, w, b = r(B, T, D).to(dtype), r(B, D, S or W).to(dtype), (r(D, W) / 2).to(dtype), r(D).to(dtype)
    st_dev = wrap(st.to(device)).clone()
    y = ops.causal_conv1d_update(wrap(x.to(device)), st_dev, wrap(w.to(device)), wrap(b.to(device)), "silu")
    st_ref = st.float().clone()
    ry = O.causal_conv1d_update_ref(x.float(), st_ref, w.float(), b.float(), "silu")
    return {"y": _err("y", y, ry, dtype, 1e-2, 1e-2), "state": _err("state", st_dev, st_ref, dtype, 1e-2, 1e-2)}


def check_rms_norm_gated(ops, device, rows_shape, N, dtype, weight_dtype=None, seed=0, backward=True, wrap=lambda t: t,
                         activation="silu"):
    """Gated RMSNorm against the oracle on the same (dtype-valued) inputs.  Half precision: the outputs are O(1)
    products of values rounded to bf16 several times on both sides, compared with |err| <= atol + rtol |ref|."""
    gen = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=gen)
    weight_dtype = weight_dtype or dtype
    x = dict(x=(2.0 * r(*rows_shape, N)).to(dtype), g=(1.5 * r(*rows_shape, N)).to(dtype),
             w=(1.0 + 0.2 * r(N)).to(weight_dtype), dy=r(*rows_shape, N).to(dtype))
    dev = {n: wrap(t.to(device)) for n, t in x.items()}
    L = {n: dev[n].clone().requires_grad_(backward) for n in ("x", "g", "w")}
    ref = O.rms_norm_gated_ref if activation == "silu" else O.rms_norm_sigmoid_gated_ref
    y = ops.rms_norm_gated(L["x"], L["g"], L["w"], 1e-6, activation)
    R = {n: x[n].clone().requires_grad_(backward) for n in ("x", "g", "w")}
    ry = ref(R["x"], R["g"], R["w"], 1e-6)
    assert y.shape == ry.shape and y.dtype == dtype
    errs = {"y": _err("y", y, ry, dtype, 2e-2, rtol=1e-2)}
    if backward:
        y.backward(dev["dy"])
        # the oracle's own autograd in half precision rounds every intermediate; differentiate its fp32 form instead
        R32 = {n: x[n].float().clone().requires_grad_(True) for n in ("x", "g", "w")}
        ref(R32["x"], R32["g"], R32["w"], 1e-6).backward(x["dy"].float())
        for n, m in (("x", "dx"), ("g", "dgate")):
            assert L[n].grad.dtype == dtype
            errs[m] = _err(m, L[n].grad, R32[n].grad, dtype, 5e-2, rtol=2e-2)
        scale = max(R32["w"].grad.abs().max().item(), 1.0)
        errs["dw"] = _err("dweight", L["w"].grad, R32["w"].grad, dtype, 1e-2 * scale, rtol=1e-2)
    return errs


def check_chunk_qkv(ops, device, B, T, Hqk, Hv, K, V, dtype, l2=True, cu=None, backward=True, seed=0, pad=0,
                    wrap=lambda t: t, **recipe):
    """The rule on the unsplit [B,T,D] tensor (q | k | v | `pad` unused columns) against the oracle on the split
    tensors, and bit for bit against the operator on contiguous q, k, v (same kernels, other strides)."""
    N = (len(cu) - 1) if cu is not None else B
    x = gdn_inputs(B, T, Hqk, Hv, K, V, dtype, seed=seed, N=N, l2norm_in_kernel=l2, **recipe)
    nq, nv = Hqk * K, Hv * V
    mixed = torch.cat([x["q"].reshape(B, T, nq), x["k"].reshape(B, T, nq), x["v"].reshape(B, T, nv),
                       torch.zeros(B, T, pad, dtype=dtype)], dim=-1)
    dev = {n: wrap(t.to(device)) for n, t in x.items()}
    mx = wrap(mixed.to(device)).clone().requires_grad_(backward)
    g, beta = (dev[n].clone().requires_grad_(backward) for n in ("g", "beta"))
    h0 = dev["h0"].clone().requires_grad_(backward)
    cu_t = torch.tensor(cu, dtype=torch.int64, device=device) if cu is not None else None
    o, ht = ops.chunk_gated_delta_rule_qkv(mx, g, beta, Hqk, Hv, K, V, initial_state=h0, output_final_state=True,
                                           use_qk_l2norm_in_kernel=l2, cu_seqlens=cu_t)
    # the same through column slices of the wide tensor (views: read in place) and through contiguous copies
    mx2 = mx.detach().clone().requires_grad_(backward)
    q2, k2, v2 = torch.split(mx2, [nq, nq, nv, pad][:3 + (pad > 0)], dim=-1)[:3]
    leaves2 = [t.clone().requires_grad_(backward) for t in (dev["g"], dev["beta"], dev["h0"])]
    o2, ht2 = ops.chunk_gated_delta_rule(q2.reshape(B, T, Hqk, K), k2.reshape(B, T, Hqk, K), v2.reshape(B, T, Hv, V),
                                         leaves2[0], leaves2[1], initial_state=leaves2[2], output_final_state=True,
                                         use_qk_l2norm_in_kernel=l2, cu_seqlens=cu_t)
    assert torch.equal(o, o2) and torch.equal(ht, ht2)
    ref = {n: x[n].float().clone().requires_grad_(backward) for n in ("q", "k", "v", "g", "beta")}
    rh0 = x["h0"].clone().requires_grad_(backward)
    ro, rht = O.chunk_gated_delta_rule_ref(ref["q"], ref["k"], ref["v"], ref["g"], ref["beta"], initial_state=rh0,
                                           output_final_state=True, use_qk_l2norm_in_kernel=l2, cu_seqlens=cu)
    errs = {"o": _err("o", o, ro, dtype, BF16_ABS_O), "ht": _err("final_state", ht, rht, dtype, BF16_ABS_O)}
    if backward:
        ((o.float() * dev["do"].float()).sum() + (ht * dev["dht"]).sum()).backward()
        ((o2.float() * dev["do"].float()).sum() + (ht2 * dev["dht"]).sum()).backward()
        ((ro * x["do"].float()).sum() + (rht * x["dht"]).sum()).backward()
        assert mx.grad.shape == mx.shape and mx.grad.dtype == dtype
        assert torch.equal(mx.grad, mx2.grad), "packed gradient differs from the gradient through the split views"
        assert torch.equal(g.grad, leaves2[0].grad) and torch.equal(beta.grad, leaves2[1].grad)
        assert torch.equal(h0.grad, leaves2[2].grad)
        dq, dk, dv = mx.grad[..., :nq], mx.grad[..., nq:2 * nq], mx.grad[..., 2 * nq:2 * nq + nv]
        errs["dq"] = _err("dq", dq.reshape(B, T, Hqk, K), ref["q"].grad, dtype, BF16_ABS_GRAD)
        errs["dk"] = _err("dk", dk.reshape(B, T, Hqk, K), ref["k"].grad, dtype, BF16_ABS_GRAD)
        errs["dv"] = _err("dv", dv.reshape(B, T, Hv, V), ref["v"].grad, dtype, BF16_ABS_GRAD)
        if pad:
            assert not mx.grad[..., 2 * nq + nv:].any()
        errs["dg"] = _err("dg", g.grad, ref["g"].grad, dtype, BF16_ABS_GRAD)
        errs["dbeta"] = _err("dbeta", beta.grad, ref["beta"].grad, dtype, BF16_ABS_GRAD)
        errs["dh0"] = _err("dh0", h0.grad, rh0.grad, dtype, BF16_ABS_GRAD)
    return errs


def check_chunk_norm(ops, device, B, T, Hqk, Hv, K, V, dtype, l2=True, cu=None, backward=True, weight_dtype=None,
                     seed=0, wrap=lambda t: t, **recipe):
    """Rule + gated RMSNorm in one pass: bit for bit against the two operators in sequence (outputs and every
    gradient), and against the oracle's rule followed by the oracle's norm.  The norm divides by the row's rms, so an
    absolute error e on o becomes e / rms on y: the bar on y is the bar on o over the smallest rms of the reference
    rows (times the largest |weight silu(gate)|), plus the norm's own rounding."""
    N = (len(cu) - 1) if cu is not None else B
    x = gdn_inputs(B, T, Hqk, Hv, K, V, dtype, seed=seed, N=N, l2norm_in_kernel=l2, **recipe)
    gen = torch.Generator().manual_seed(seed + 77)
    weight_dtype = weight_dtype or dtype
    z = (1.5 * torch.randn(B, T, Hv * V, generator=gen)).to(dtype)        # the layer's z: [B, T, Hv * V]
    w = (1.0 + 0.2 * torch.randn(V, generator=gen)).to(weight_dtype)
    dy = torch.randn(B, T, Hv, V, generator=gen).to(dtype)
    dev = {n: wrap(t.to(device)) for n, t in x.items()}
    cu_t = torch.tensor(cu, dtype=torch.int64, device=device) if cu is not None else None
    names = ("q", "k", "v", "g", "beta", "h0")

    def leaves():
        L = {n: dev[n].clone().requires_grad_(backward) for n in names}
        L["z"] = wrap(z.to(device)).clone().requires_grad_(backward)
        L["w"] = wrap(w.to(device)).clone().requires_grad_(backward)
        return L
    A, Bc = leaves(), leaves()
    y, ht = ops.chunk_gated_delta_rule_norm(A["q"], A["k"], A["v"], A["g"], A["beta"], A["z"], A["w"], eps=1e-6,
                                            initial_state=A["h0"], output_final_state=True,
                                            use_qk_l2norm_in_kernel=l2, cu_seqlens=cu_t, in_output_kernel=True)
    o2, ht2 = ops.chunk_gated_delta_rule(Bc["q"], Bc["k"], Bc["v"], Bc["g"], Bc["beta"], initial_state=Bc["h0"],
                                         output_final_state=True, use_qk_l2norm_in_kernel=l2, cu_seqlens=cu_t)
    y2 = ops.rms_norm_gated(o2.reshape(-1, V), Bc["z"].reshape(-1, V), Bc["w"], 1e-6).view(B, T, Hv, V)
    assert y.shape == (B, T, Hv, V) and y.dtype == dtype
    assert torch.equal(y, y2), "fused norm differs from the two operators in sequence"
    assert torch.equal(ht, ht2)
    if not backward:    # without gradients the fused pass writes no o: check that path too
        with torch.no_grad():
            y3, _ = ops.chunk_gated_delta_rule_norm(dev["q"], dev["k"], dev["v"], dev["g"], dev["beta"],
                                                    wrap(z.to(device)), wrap(w.to(device)), initial_state=dev["h0"],
                                                    use_qk_l2norm_in_kernel=l2, cu_seqlens=cu_t, in_output_kernel=True)
        assert torch.equal(y3, y)
    ro, rht = O.chunk_gated_delta_rule_ref(x["q"].float(), x["k"].float(), x["v"].float(), x["g"], x["beta"],
                                           initial_state=x["h0"], output_final_state=True,
                                           use_qk_l2norm_in_kernel=l2, cu_seqlens=cu)
    ry = O.rms_norm_gated_ref(ro.reshape(-1, V), z.float().reshape(-1, V), w.float(), 1e-6).view(B, T, Hv, V)
    rms = ro.pow(2).mean(-1).add(1e-6).sqrt().min().item()
    amp = (w.float().abs().max() * (z.float() * torch.sigmoid(z.float())).abs().max()).item() / rms
    o_bar = BF16_ABS_O if dtype == torch.bfloat16 else 1e-4 * ro.abs().max().item()
    half = dtype == torch.bfloat16
    # elementwise |err| <= abs_tol + rtol |ref| in both precisions (torch.bfloat16 selects that form of the check)
    errs = {"y": _err("y", y, ry, torch.bfloat16, o_bar * amp + (2e-2 if half else 1e-5), rtol=1e-2 if half else 1e-4)}
    if backward:
        ((y.float() * wrap(dy.to(device)).float()).sum() + (ht * dev["dht"]).sum()).backward()
        ((y2.float() * wrap(dy.to(device)).float()).sum() + (ht2 * dev["dht"]).sum()).backward()
        for n in names + ("z", "w"):
            assert A[n].grad is not None and A[n].grad.dtype == A[n].dtype, n
            assert torch.equal(A[n].grad, Bc[n].grad), f"gradient of {n} differs from the two operators in sequence"
    return errs


def check_chunk_qkv_norm(ops, device, B, T, Hqk, Hv, K, V, dtype, l2=True, cu=None, backward=True, seed=0,
                         wrap=lambda t: t, **recipe):
    """The layer's sequence convolution output -> rule -> gated norm in one call on the unsplit tensor, bit for bit
    against the rule on the unsplit tensor followed by the norm operator (each checked against the oracle on its own)."""
    N = (len(cu) - 1) if cu is not None else B
    x = gdn_inputs(B, T, Hqk, Hv, K, V, dtype, seed=seed, N=N, l2norm_in_kernel=l2, **recipe)
    gen = torch.Generator().manual_seed(seed + 5)
    nq, nv = Hqk * K, Hv * V
    mixed = torch.cat([x["q"].reshape(B, T, nq), x["k"].reshape(B, T, nq), x["v"].reshape(B, T, nv)], dim=-1)
    z = (1.5 * torch.randn(B, T, nv, generator=gen)).to(dtype)
    w = (1.0 + 0.2 * torch.randn(V, generator=gen)).to(dtype)
    dy = torch.randn(B, T, Hv, V, generator=gen).to(dtype)
    cu_t = torch.tensor(cu, dtype=torch.int64, device=device) if cu is not None else None

    def leaves():
        L = dict(mx=wrap(mixed.to(device)).clone(), z=wrap(z.to(device)).clone(), w=wrap(w.to(device)).clone(),
                 g=wrap(x["g"].to(device)).clone(), beta=wrap(x["beta"].to(device)).clone(),
                 h0=wrap(x["h0"].to(device)).clone())
        return {n: t.requires_grad_(backward) for n, t in L.items()}
    A, Bc = leaves(), leaves()
    y, ht = ops.chunk_gated_delta_rule_qkv(A["mx"], A["g"], A["beta"], Hqk, Hv, K, V, initial_state=A["h0"],
                                           output_final_state=True, use_qk_l2norm_in_kernel=l2, cu_seqlens=cu_t,
                                           gate=A["z"], norm_weight=A["w"])
    o2, ht2 = ops.chunk_gated_delta_rule_qkv(Bc["mx"], Bc["g"], Bc["beta"], Hqk, Hv, K, V, initial_state=Bc["h0"],
                                             output_final_state=True, use_qk_l2norm_in_kernel=l2, cu_seqlens=cu_t)
    y2 = ops.rms_norm_gated(o2.reshape(-1, V), Bc["z"].reshape(-1, V), Bc["w"], 1e-6).view(B, T, Hv, V)
    assert y.shape == (B, T, Hv, V) and torch.equal(y, y2) and torch.equal(ht, ht2)
    if backward:
        dyd = wrap(dy.to(device)).float()
        (y.float() * dyd).sum().backward()
        (y2.float() * dyd).sum().backward()
        for n in A:
            assert A[n].grad is not None and A[n].grad.shape == A[n].shape and A[n].grad.dtype == A[n].dtype, n
            assert torch.equal(A[n].grad, Bc[n].grad), f"gradient of {n} differs from the two operators in sequence"
    return {"y_max": y.detach().float().abs().max().item()}


def check_gdn_gates(ops, device, shape, Hv, dtype, param_dtype=None, seed=0, backward=True, wrap=lambda t: t):
    """Gate recipe against the oracle on the same (dtype-valued) inputs.  g is fp32 on both sides (relative 1e-4 of
    the largest value, the fp32 bar); beta and the gradients in half precision carry one rounding to bf16."""
    gen = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=gen)
    param_dtype = param_dtype or dtype
    x = dict(a=(2.0 * r(*shape, Hv)).to(dtype), b=(2.0 * r(*shape, Hv)).to(dtype),
             A=torch.empty(Hv).uniform_(0.0, 2.77, generator=gen).to(param_dtype),
             d=torch.empty(Hv).uniform_(-4.0, -2.0, generator=gen).to(param_dtype),
             dg=r(*shape, Hv), dbeta=r(*shape, Hv).to(dtype))
    x["a"].view(-1)[:3] = torch.tensor([30.0, 24.5, -30.0]).to(dtype)    # both softplus branches and the far left
    dev = {n: wrap(t.to(device)) for n, t in x.items()}
    L = {n: dev[n].clone().requires_grad_(backward) for n in ("a", "b", "A", "d")}
    g, beta = ops.gdn_gates(L["a"], L["b"], L["A"], L["d"])
    R = {n: x[n].float().clone().requires_grad_(backward) for n in ("a", "b", "A", "d")}
    rg, rbeta = O.gdn_gates_ref(R["a"], R["b"], R["A"], R["d"])
    assert g.dtype == torch.float32 and beta.dtype == dtype and g.shape == rg.shape
    errs = {"g": _err("g", g, rg, torch.float32, 0), "beta": _err("beta", beta, rbeta, dtype, 4e-3)}
    if backward:
        ((g * dev["dg"]).sum() + (beta.float() * dev["dbeta"].float()).sum()).backward()
        ((rg * x["dg"]).sum() + (rbeta * x["dbeta"].float()).sum()).backward()
        for n, m in (("a", "da"), ("b", "db")):
            assert L[n].grad.dtype == dtype
            errs[m] = _err(m, L[n].grad, R[n].grad, dtype, 5e-2, rtol=1e-2)
        for n, m in (("A", "dA_log"), ("d", "ddt_bias")):
            assert L[n].grad.dtype == param_dtype
            scale = max(R[n].grad.abs().max().item(), 1.0)
            errs[m] = _err(m, L[n].grad, R[n].grad, param_dtype, 1e-2 * scale, rtol=1e-2)
    return errs


def check_decode_step(ops, device, B, steps, Hqk, Hv, K, V, W, dtype, param_dtype=None, seed=0, wrap=lambda t: t):
    """`steps` consecutive decode tokens through decode_step (convolution update + rule on its unsplit output with the
    gates formed in the kernel, both states in place) against the oracle's chain conv update -> split -> gate recipe
    -> recurrent rule, and bit for bit against this package's own unfused operators."""
    gen = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=gen)
    param_dtype = param_dtype or dtype
    nq, nv = Hqk * K, Hv * V
    D = 2 * nq + nv
    x = dict(mixed=r(B, steps, D).to(dtype), a=r(B, steps, Hv).to(dtype), b=r(B, steps, Hv).to(dtype),
             cw=(r(D, W) / 2).to(dtype), cb=(r(D) / 4).to(dtype),
             A=torch.empty(Hv).uniform_(0.0, 2.77, generator=gen).to(param_dtype),
             d=torch.empty(Hv).uniform_(-4.0, -2.0, generator=gen).to(param_dtype),
             conv=r(B, D, W).to(dtype), S=0.1 * r(B, Hv, K, V))
    dev = {n: wrap(t.to(device)) for n, t in x.items()}
    conv1, S1 = dev["conv"].clone(), dev["S"].clone()
    conv2, S2 = dev["conv"].clone(), dev["S"].clone()
    rconv, rS = x["conv"].float().clone(), x["S"].clone()
    errs = {}
    for t in range(steps):
        sl = slice(t, t + 1)
        o = ops.decode_step(dev["mixed"][:, sl], dev["a"][:, sl], dev["b"][:, sl], conv1, S1, dev["cw"], dev["cb"],
                            dev["A"], dev["d"], Hqk, Hv, K, V)
        # the same with this package's separate operators
        y2 = ops.causal_conv1d_update(dev["mixed"][:, sl], conv2, dev["cw"], dev["cb"], "silu")
        q2, k2, v2 = torch.split(y2, [nq, nq, nv], dim=-1)
        g2, beta2 = ops.gdn_gates(dev["a"][:, sl], dev["b"][:, sl], dev["A"], dev["d"])
        o2, _ = ops.fused_recurrent_gated_delta_rule(
            q2.reshape(B, 1, Hqk, K), k2.reshape(B, 1, Hqk, K), v2.reshape(B, 1, Hv, V), g2, beta2, initial_state=S2,
            output_final_state=True, use_qk_l2norm_in_kernel=True, inplace_state=True)
        assert torch.equal(o, o2), f"step {t}: fused decode step differs from the separate operators"
        # oracle chain, with the layer's dtype flow (the convolution's output is in the activations' dtype)
        ry = O.causal_conv1d_update_ref(x["mixed"][:, sl].float(), rconv, x["cw"].float(), x["cb"].float(), "silu")
        ry = ry.to(dtype).float()
        rq, rk, rv = torch.split(ry, [nq, nq, nv], dim=-1)
        rg, rbeta = O.gdn_gates_ref(x["a"][:, sl], x["b"][:, sl], x["A"], x["d"])
        ro, rS = O.recurrent_gated_delta_rule_ref(rq.reshape(B, 1, Hqk, K), rk.reshape(B, 1, Hqk, K),
                                                  rv.reshape(B, 1, Hv, V), rg, rbeta.float(), rS, True, True)
        errs["o"] = max(errs.get("o", 0.0), _err(f"o[{t}]", o, ro, dtype, BF16_ABS_O))
    assert torch.equal(conv1, conv2) and torch.equal(S1, S2)
    errs["conv_state"] = _err("conv_state", conv1, rconv, dtype, 1e-2, 1e-2)
    errs["state"] = _err("recurrent_state", S1, rS, dtype, BF16_ABS_GRAD)
    return errs


def check_kda(ops, device, B, T, H, K, V, dtype, cu=None, seed=0, with_h0=True, gate_in_kernel=True, lower_bound=None,
              beta_sigmoid=True, allow_neg=False, l2=True, transpose_state=True, g_dtype=None, scale=None, backward=False,
              wrap=lambda t: t, states=False, **recipe):
    """chunk_kda against the oracle's statement of chunk_kda_naive, with the options of the layer's call
    (modeling_kimi_linear.py:681-699: raw gate and beta, l2 norm in the kernel, [N,H,V,K] states) or without them.
    backward: every gradient against autograd through the oracle (loss = <o, do> + <final state, dht>).
    states: also return_intermediate_states=True, the state at every chunk entry against the oracle's."""
    N = (len(cu) - 1) if cu is not None else B
    x = kda_inputs(B, T, H, K, V, dtype, seed=seed, N=N, **recipe)
    if not gate_in_kernel:   # the caller hands over the log decay itself
        x["g"] = KO.kda_gate_ref(x["g"], x["A_log"], x["dt_bias"], lower_bound)
    if g_dtype is not None:
        x["g"] = x["g"].to(g_dtype)
    if not beta_sigmoid:
        x["beta"] = torch.sigmoid(x["beta"].float()).to(x["beta"].dtype)
    if not l2:
        x["q"], x["k"] = (KO._l2norm_rounded(t) for t in (x["q"], x["k"]))
    if transpose_state:
        x["h0"], x["dht"] = (x[n].transpose(-1, -2).contiguous() for n in ("h0", "dht"))
    names = ("q", "k", "v", "g", "beta", "h0", "A_log", "dt_bias")
    dev = {n: wrap(t.to(device)) for n, t in x.items()}
    leaves = {n: dev[n].clone().requires_grad_(backward) for n in names}
    ref = {n: x[n].clone().requires_grad_(backward) for n in names}
    cu_t = torch.tensor(cu, dtype=torch.int64, device=device) if cu is not None else None
    kw = dict(scale=scale, output_final_state=True, use_qk_l2norm_in_kernel=l2, use_gate_in_kernel=gate_in_kernel,
              use_beta_sigmoid_in_kernel=beta_sigmoid, allow_neg_eigval=allow_neg, lower_bound=lower_bound if gate_in_kernel else None,
              transpose_state_layout=transpose_state, return_intermediate_states=states)
    with torch.set_grad_enabled(backward):
        o, ht, *hs = ops.chunk_kda(leaves["q"], leaves["k"], leaves["v"], leaves["g"], leaves["beta"],
                              initial_state=leaves["h0"] if with_h0 else None, cu_seqlens=cu_t,
                              safe_gate=lower_bound is not None, A_log=leaves["A_log"], dt_bias=leaves["dt_bias"], **kw)
        ro, rht, *rhs = KO.chunk_kda_ref(ref["q"], ref["k"], ref["v"], ref["g"], ref["beta"], initial_state=ref["h0"] if with_h0 else None,
                                   cu_seqlens=cu, A_log=ref["A_log"], dt_bias=ref["dt_bias"], round_output=False, **kw)
    assert o.dtype == dtype and ht.dtype == torch.float32 and ht.shape == rht.shape
    errs = {"o": _err("o", o, ro, dtype, BF16_ABS_O), "ht": _err("final_state", ht, rht, dtype, BF16_ABS_O)}
    if states:
        assert len(hs) == 1 and hs[0].dtype == dtype and not hs[0].requires_grad
        errs["h"] = _err("intermediate states", hs[0], rhs[0], dtype, BF16_ABS_O)
    if backward:
        ((o.float() * dev["do"].float()).sum() + (ht * dev["dht"]).sum()).backward()
        ((ro * x["do"].float()).sum() + (rht * x["dht"]).sum()).backward()
        for n in names:
            if (n == "h0" and not with_h0) or (n in ("A_log", "dt_bias") and not gate_in_kernel):
                continue
            assert leaves[n].grad is not None, n
            assert leaves[n].grad.dtype == leaves[n].dtype and leaves[n].grad.shape == leaves[n].shape
            param = n in ("A_log", "dt_bias")
            errs["d" + n] = _err("d" + n, leaves[n].grad, ref[n].grad, dtype,
                                 kda_param_tol(ref[n].grad, B * T) if param else BF16_ABS_GRAD)
    return errs
