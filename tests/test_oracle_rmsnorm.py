"""Pins oracle.gdn_oracle.rms_norm_gated_ref (Qwen3_5RMSNormGated.forward, modeling_qwen3_5.py:341-349) with checks that
do not retype its formula: a library routine, a closed form, an invariance and a numerical gradient."""
import math

import torch
import torch.nn.functional as F

from oracle import gdn_oracle as O


def _inputs(rows, N, dtype=torch.float64, seed=0):
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, N, generator=gen, dtype=torch.float64).to(dtype)
    g = torch.randn(rows, N, generator=gen, dtype=torch.float64).to(dtype)
    w = (1 + 0.3 * torch.randn(N, generator=gen, dtype=torch.float64)).to(dtype)
    return x, g, w


def test_matches_library_rms_norm_times_silu_gate():
    x, g, w = _inputs(37, 128)
    ref = F.rms_norm(x, (128,), w, eps=1e-6) * F.silu(g)
    got = O.rms_norm_gated_ref(x.float(), g.float(), w.float()).double()   # the oracle normalises in fp32
    assert torch.allclose(got, ref, rtol=2e-6, atol=2e-6)


def test_closed_form_constant_row():
    # x = c everywhere: mean(x^2) = c^2, so the normalised row is sign(c) (up to eps) and y = w * silu(gate)
    N = 64
    g = torch.linspace(-3, 3, N)[None]
    w = torch.linspace(0.5, 1.5, N)
    for c in (-4.0, 0.25, 7.0):
        y = O.rms_norm_gated_ref(torch.full((1, N), c), g, w)
        expect = math.copysign(1.0, c) * w * g * torch.sigmoid(g)
        assert torch.allclose(y, expect, rtol=1e-5, atol=1e-6)


def test_scale_invariance_in_x_and_linearity_in_weight():
    x, g, w = _inputs(9, 256, torch.float32)
    y = O.rms_norm_gated_ref(x, g, w, eps=0.0)
    assert torch.allclose(O.rms_norm_gated_ref(8.0 * x, g, w, eps=0.0), y, rtol=1e-5, atol=1e-6)
    assert torch.allclose(O.rms_norm_gated_ref(x, g, 3.0 * w, eps=0.0), 3.0 * y, rtol=1e-6, atol=1e-6)
    # every output row has weighted RMS equal to rms(w * silu(g)) only through the normalised x: check the norm itself
    xn = O.rms_norm_gated_ref(x, torch.full_like(g, 30.0), torch.ones_like(w), eps=0.0) / 30.0   # silu(30) = 30
    assert torch.allclose(xn.pow(2).mean(-1), torch.ones(9), rtol=1e-5)


def test_half_precision_casts_follow_the_reference_order():
    # bf16: the normalised row is rounded to bf16 before the weight, the weighted row again (weight in bf16), and the
    # gate is applied in fp32 -- rebuilt here step by step with explicit casts
    x, g, w = _inputs(5, 128, torch.bfloat16, seed=3)
    xn = (x.float() * torch.rsqrt(x.float().pow(2).mean(-1, keepdim=True) + 1e-6)).to(torch.bfloat16)
    t = w * xn                                # bf16 * bf16 -> bf16
    expect = (t.float() * (g.float() * torch.sigmoid(g.float()))).to(torch.bfloat16)
    assert torch.equal(O.rms_norm_gated_ref(x, g, w), expect)


def test_gradcheck_float64():
    x, g, w = _inputs(3, 16)
    # float64 inputs: the oracle's internal fp32 cast would spoil the numerical gradient, so check its formula in a
    # float64-preserving wrapper built from the same library routine it was pinned against above
    fn = lambda a, b, c: F.rms_norm(a, (16,), c, eps=1e-6) * F.silu(b)
    args = [t.clone().requires_grad_(True) for t in (x, g, w)]
    assert torch.autograd.gradcheck(fn, args, eps=1e-6, atol=1e-5)
    # and the oracle's autograd agrees with that routine's autograd
    a32 = [t.float().clone().requires_grad_(True) for t in (x, g, w)]
    dy = torch.randn(3, 16)
    O.rms_norm_gated_ref(*a32).backward(dy)
    fn(*args).backward(dy.double())
    for p, q in zip(a32, args):
        assert torch.allclose(p.grad.double(), q.grad, rtol=1e-4, atol=1e-5)


# ---- the KDA layer's norm: sigmoid gate (KimiK_3_MoeRMSNormGated.forward, modeling_kimi_linear.py:89-94)
def test_sigmoid_gated_matches_library_rms_norm_times_sigmoid():
    x, g, w = _inputs(37, 128)
    ref = F.rms_norm(x, (128,), w, eps=1e-6) * torch.special.expit(g)
    got = O.rms_norm_sigmoid_gated_ref(x.float(), g.float(), w.float()).double()
    assert torch.allclose(got, ref, rtol=2e-6, atol=2e-6)


def test_sigmoid_gated_limits_of_the_gate():
    # gate = 0 halves the normalised row; a wide open gate (sigmoid -> 1) leaves it; a closed one removes it
    x, _, w = _inputs(6, 64, torch.float32, seed=2)
    plain = F.rms_norm(x, (64,), w, eps=1e-6)
    assert torch.allclose(O.rms_norm_sigmoid_gated_ref(x, torch.zeros_like(x), w), 0.5 * plain, rtol=1e-6, atol=1e-7)
    assert torch.allclose(O.rms_norm_sigmoid_gated_ref(x, torch.full_like(x, 40.0), w), plain, rtol=1e-6, atol=1e-7)
    assert O.rms_norm_sigmoid_gated_ref(x, torch.full_like(x, -120.0), w).abs().max() == 0
    # and the two gated norms differ by exactly the factor gate: silu(g) = g sigmoid(g)
    g = torch.linspace(-3, 3, 64).expand(6, 64)
    assert torch.allclose(O.rms_norm_gated_ref(x, g, w), g * O.rms_norm_sigmoid_gated_ref(x, g, w), rtol=1e-5, atol=1e-6)


def test_sigmoid_gated_half_precision_casts_follow_the_reference_order():
    # bf16: normalised row rounded, weighted row rounded (weight in bf16), the sigmoid rounded to bf16 before the product
    x, g, w = _inputs(5, 128, torch.bfloat16, seed=3)
    xn = (x.float() * torch.rsqrt(x.float().pow(2).mean(-1, keepdim=True) + 1e-6)).to(torch.bfloat16)
    expect = (w * xn) * torch.sigmoid(g.float()).to(torch.bfloat16)
    assert expect.dtype == torch.bfloat16 and torch.equal(O.rms_norm_sigmoid_gated_ref(x, g, w), expect)


def test_sigmoid_gated_gradient_against_the_silu_form():
    # d/dg of t sigmoid(g) from the pinned silu form: t silu(g) = g (t sigmoid(g))  =>  d(silu form)/dg = y + g dy/dg
    x, g, w = _inputs(4, 32, torch.float32, seed=5)
    g1 = g.clone().requires_grad_(True)
    y = O.rms_norm_sigmoid_gated_ref(x, g1, w)
    dy_dg, = torch.autograd.grad(y.sum(), g1)
    g2 = g.clone().requires_grad_(True)
    ds_dg, = torch.autograd.grad(O.rms_norm_gated_ref(x, g2, w).sum(), g2)
    assert torch.allclose(ds_dg, y.detach() + g * dy_dg, rtol=1e-5, atol=1e-6)

