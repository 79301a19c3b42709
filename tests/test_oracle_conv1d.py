"""Pins the conv1d oracle against the library routine F.conv1d(groups=D) (the reference's own eager
branch, modeling_qwen3_5.py:803-806), state continuity and the final-state definition."""
import pytest
import torch
import torch.nn.functional as F

from oracle import gdn_oracle as O


def _rand(*s, seed=0):
    return torch.randn(*s, generator=torch.Generator().manual_seed(seed), dtype=torch.float64)


@pytest.mark.parametrize("T,W,act", [(37, 4, "silu"), (3, 4, None), (1, 4, "swish"), (20, 1, "silu"), (9, 3, None)])
def test_matches_library_conv(T, W, act):
    B, D = 2, 10
    x, w, b = _rand(B, T, D, seed=1), _rand(W, D, seed=2), _rand(D, seed=3)
    y, _ = O.causal_conv1d_ref(x, w, b, activation=act, dtype=torch.float64)
    lib = F.conv1d(x.transpose(1, 2), w.t().unsqueeze(1), b, padding=W - 1, groups=D)[:, :, :T]
    if act:
        lib = F.silu(lib)
    torch.testing.assert_close(y, lib.transpose(1, 2), rtol=1e-12, atol=1e-13)


def test_initial_state_is_left_context():
    """initial_state[n,d,j] is the input at step j-W: conv over (context ++ x) equals conv with state."""
    B, T, D, W = 2, 11, 6, 4
    ctx, x, w = _rand(B, W, D, seed=4), _rand(B, T, D, seed=5), _rand(W, D, seed=6)
    y_full, _ = O.causal_conv1d_ref(torch.cat([ctx, x], 1), w, activation="silu", dtype=torch.float64)
    y, fs = O.causal_conv1d_ref(x, w, initial_state=ctx.transpose(1, 2), activation="silu",
                                output_final_state=True, dtype=torch.float64)
    torch.testing.assert_close(y, y_full[:, W:], rtol=1e-12, atol=1e-13)
    torch.testing.assert_close(fs, x[:, T - W:].transpose(1, 2))


@pytest.mark.parametrize("T", [1, 2, 3])
def test_final_state_short_sequence(T):
    """T < W: the final state keeps the tail of the initial state (reference_impl.py:81-102)."""
    B, D, W = 2, 5, 4
    x, h0 = _rand(B, T, D, seed=7), _rand(B, D, W, seed=8)
    _, fs = O.causal_conv1d_ref(x, _rand(W, D, seed=9), initial_state=h0, output_final_state=True,
                                dtype=torch.float64)
    want = torch.cat([h0[:, :, T:], x.transpose(1, 2)], dim=-1)
    torch.testing.assert_close(fs, want)
    _, fs0 = O.causal_conv1d_ref(x, _rand(W, D, seed=9), output_final_state=True, dtype=torch.float64)
    torch.testing.assert_close(fs0, torch.cat([torch.zeros(B, D, W - T, dtype=torch.float64), x.transpose(1, 2)], -1))


def test_state_continuity_and_varlen():
    D, W = 8, 4
    cu = [0, 1, 3, 20, 21, 50]
    x, w, b = _rand(1, 50, D, seed=10), _rand(W, D, seed=11), _rand(D, seed=12)
    h0 = _rand(5, D, W, seed=13)
    y, fs = O.causal_conv1d_ref(x, w, b, initial_state=h0, activation="silu", cu_seqlens=cu,
                                output_final_state=True, dtype=torch.float64)
    for n in range(5):
        s, e = cu[n], cu[n + 1]
        yn, fn = O.causal_conv1d_ref(x[:, s:e], w, b, initial_state=h0[n:n + 1], activation="silu",
                                     output_final_state=True, dtype=torch.float64)
        torch.testing.assert_close(y[:, s:e], yn)
        torch.testing.assert_close(fs[n:n + 1], fn)
    # split + chain == full
    ya, fa = O.causal_conv1d_ref(x[:, :17], w, b, activation="silu", output_final_state=True, dtype=torch.float64)
    yb, fb = O.causal_conv1d_ref(x[:, 17:], w, b, initial_state=fa, activation="silu", output_final_state=True,
                                 dtype=torch.float64)
    yf, ff = O.causal_conv1d_ref(x, w, b, activation="silu", output_final_state=True, dtype=torch.float64)
    torch.testing.assert_close(torch.cat([ya, yb], 1), yf)
    torch.testing.assert_close(fb, ff)


def test_residual_and_bias():
    x, w, b, r = _rand(1, 9, 4, seed=14), _rand(4, 4, seed=15), _rand(4, seed=16), _rand(1, 9, 4, seed=17)
    y0, _ = O.causal_conv1d_ref(x, w, dtype=torch.float64)
    y1, _ = O.causal_conv1d_ref(x, w, b, residual=r, dtype=torch.float64)
    torch.testing.assert_close(y1, y0 + b + r)


def test_update_matches_full_conv():
    """Token-by-token decode update reproduces the full conv; conv_state ends as the final state."""
    B, T, D, W = 2, 13, 6, 4
    x, w, b = _rand(B, T, D, seed=18), _rand(W, D, seed=19), _rand(D, seed=20)
    y_full, fs = O.causal_conv1d_ref(x, w, b, activation="silu", output_final_state=True, dtype=torch.float64)
    state = torch.zeros(B, D, W, dtype=torch.float64)
    outs = [O.causal_conv1d_update_ref(x[:, t:t + 1], state, w.t().contiguous(), b, "silu") for t in range(T)]
    torch.testing.assert_close(torch.cat(outs, 1), y_full, rtol=1e-12, atol=1e-13)
    torch.testing.assert_close(state, fs)
    # multi-token update
    state2 = torch.zeros(B, D, W, dtype=torch.float64)
    y2 = O.causal_conv1d_update_ref(x, state2, w.t().contiguous(), b, "silu")
    torch.testing.assert_close(y2, y_full, rtol=1e-12, atol=1e-13)
    torch.testing.assert_close(state2, fs)


def test_gradcheck():
    x, w, b = _rand(1, 7, 3, seed=21), _rand(4, 3, seed=22), _rand(3, seed=23)
    h0 = _rand(2, 3, 4, seed=24)
    args = [t.requires_grad_(True) for t in (x, w, b, h0)]
    f = lambda x, w, b, h0: O.causal_conv1d_ref(x, w, b, initial_state=h0, activation="silu", cu_seqlens=[0, 2, 7],
                                                output_final_state=True, dtype=torch.float64)
    assert torch.autograd.gradcheck(f, args, eps=1e-6, atol=1e-6)
