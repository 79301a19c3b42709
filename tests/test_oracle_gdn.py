"""Pins the CPU oracle of the gated delta rule (oracle/gdn_oracle.py) against
independent facts: the textbook recurrence, closed forms, invariants, a library
triangular solve, autograd/gradcheck and committed golden vectors."""
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import gdn_oracle as O

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def make_inputs(B, T, Hqk, Hv, K, V, seed=0, dtype=torch.float64, normalize=True, N=None):
    gen = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float64)
    q, k, v = r(B, T, Hqk, K), r(B, T, Hqk, K), r(B, T, Hv, V)
    if normalize:
        q, k = O.l2norm(q), O.l2norm(k)
    beta = torch.sigmoid(r(B, T, Hv))
    A_log = torch.empty(Hv, dtype=torch.float64).uniform_(0.0, math.log(16.0), generator=gen)
    dt_bias = torch.empty(Hv, dtype=torch.float64).uniform_(-4.0, -2.0, generator=gen)
    g = -A_log.exp() * F.softplus(r(B, T, Hv) + dt_bias)
    h0 = 0.5 * r(N if N is not None else B, Hv, K, V)
    return [x.to(dtype) for x in (q, k, v, g, beta, h0)]


# ---- chunked == textbook recurrence -------------------------------------------------

@pytest.mark.parametrize("B,T,Hqk,Hv,K,V,l2", [
    (1, 64, 2, 2, 16, 16, False),
    (2, 100, 2, 4, 16, 24, True),      # GQA, ragged T, l2norm in kernel
    (1, 193, 1, 3, 8, 12, True),
    (1, 1, 2, 2, 16, 16, False),
])
def test_chunk_equals_recurrence(B, T, Hqk, Hv, K, V, l2):
    q, k, v, g, beta, h0 = make_inputs(B, T, Hqk, Hv, K, V, seed=1, normalize=not l2)
    o1, s1 = O.naive_gated_delta_rule(q, k, v, g, beta, initial_state=h0, output_final_state=True,
                                      use_qk_l2norm_in_kernel=l2)
    o2, s2 = O.chunk_gated_delta_rule_ref(q, k, v, g, beta, initial_state=h0, output_final_state=True,
                                          use_qk_l2norm_in_kernel=l2, dtype=torch.float64)
    o3, s3 = O.recurrent_gated_delta_rule_ref(q, k, v, g, beta, initial_state=h0, output_final_state=True,
                                              use_qk_l2norm_in_kernel=l2, dtype=torch.float64)
    torch.testing.assert_close(o2, o1, rtol=1e-10, atol=1e-11)
    torch.testing.assert_close(s2, s1, rtol=1e-10, atol=1e-11)
    torch.testing.assert_close(o3, o1, rtol=1e-12, atol=1e-13)
    torch.testing.assert_close(s3, s1, rtol=1e-12, atol=1e-13)


def test_chunk_fp32_close_to_fp64():
    q, k, v, g, beta, h0 = make_inputs(1, 256, 2, 2, 32, 32, seed=2)
    o1, s1 = O.naive_gated_delta_rule(q, k, v, g, beta, initial_state=h0, output_final_state=True)
    o2, s2 = O.chunk_gated_delta_rule_ref(q, k, v, g, beta, initial_state=h0, output_final_state=True)
    assert o2.dtype == torch.float32
    assert (o2.double() - o1).abs().max() / o1.abs().max() < 1e-5
    assert (s2.double() - s1).abs().max() / s1.abs().max() < 1e-5


@pytest.mark.parametrize("C", [16, 32, 64])
def test_chunk_size_invariance(C):
    q, k, v, g, beta, h0 = make_inputs(1, 150, 2, 2, 16, 16, seed=3)
    o64, s64 = O.chunk_gated_delta_rule_ref(q, k, v, g, beta, initial_state=h0, output_final_state=True,
                                            dtype=torch.float64)
    oc, sc = O.chunk_gated_delta_rule_ref(q, k, v, g, beta, initial_state=h0, output_final_state=True,
                                          chunk_size=C, dtype=torch.float64)
    torch.testing.assert_close(oc, o64, rtol=1e-10, atol=1e-11)
    torch.testing.assert_close(sc, s64, rtol=1e-10, atol=1e-11)


def test_zero_padding_invariance():
    """Appending tokens with k=0, beta=0, g=0 changes nothing (modeling_qwen3_5.py:419-425)."""
    q, k, v, g, beta, h0 = make_inputs(1, 70, 2, 2, 16, 16, seed=4)
    o, s = O.chunk_gated_delta_rule_ref(q, k, v, g, beta, initial_state=h0, output_final_state=True,
                                        dtype=torch.float64)
    pad = lambda x: F.pad(x, (0, 0) * (x.dim() - 2) + (0, 30))
    o2, s2 = O.chunk_gated_delta_rule_ref(pad(q), pad(k), pad(v), pad(g), pad(beta), initial_state=h0,
                                          output_final_state=True, dtype=torch.float64)
    torch.testing.assert_close(o2[:, :70], o, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(s2, s, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("split", [1, 63, 64, 65, 100])
def test_state_continuity(split):
    q, k, v, g, beta, h0 = make_inputs(2, 130, 2, 2, 16, 16, seed=5)
    o, s = O.chunk_gated_delta_rule_ref(q, k, v, g, beta, initial_state=h0, output_final_state=True,
                                        dtype=torch.float64)
    a = [x[:, :split] for x in (q, k, v, g, beta)]
    b = [x[:, split:] for x in (q, k, v, g, beta)]
    oa, sa = O.chunk_gated_delta_rule_ref(*a, initial_state=h0, output_final_state=True, dtype=torch.float64)
    ob, sb = O.chunk_gated_delta_rule_ref(*b, initial_state=sa, output_final_state=True, dtype=torch.float64)
    torch.testing.assert_close(torch.cat([oa, ob], 1), o, rtol=1e-10, atol=1e-11)
    torch.testing.assert_close(sb, s, rtol=1e-10, atol=1e-11)


def test_scale_linearity_and_default():
    q, k, v, g, beta, h0 = make_inputs(1, 80, 2, 2, 16, 16, seed=6)
    o1, _ = O.chunk_gated_delta_rule_ref(q, k, v, g, beta, dtype=torch.float64)
    o2, _ = O.chunk_gated_delta_rule_ref(q, k, v, g, beta, scale=16 ** -0.5, dtype=torch.float64)
    o3, _ = O.chunk_gated_delta_rule_ref(q, k, v, g, beta, scale=1.0, dtype=torch.float64)
    torch.testing.assert_close(o1, o2)
    torch.testing.assert_close(o3 * 16 ** -0.5, o1, rtol=1e-12, atol=1e-13)


def test_gqa_equals_repeat_interleave():
    q, k, v, g, beta, h0 = make_inputs(1, 90, 2, 6, 16, 16, seed=7)
    o1, s1 = O.chunk_gated_delta_rule_ref(q, k, v, g, beta, initial_state=h0, output_final_state=True,
                                          dtype=torch.float64)
    qe, ke = q.repeat_interleave(3, 2), k.repeat_interleave(3, 2)
    o2, s2 = O.chunk_gated_delta_rule_ref(qe, ke, v, g, beta, initial_state=h0, output_final_state=True,
                                          dtype=torch.float64)
    torch.testing.assert_close(o1, o2)
    torch.testing.assert_close(s1, s2)


def test_head_permutation_equivariance():
    q, k, v, g, beta, h0 = make_inputs(1, 70, 3, 3, 8, 8, seed=8)
    perm = torch.tensor([2, 0, 1])
    o1, s1 = O.chunk_gated_delta_rule_ref(q, k, v, g, beta, initial_state=h0, output_final_state=True,
                                          dtype=torch.float64)
    o2, s2 = O.chunk_gated_delta_rule_ref(q[:, :, perm], k[:, :, perm], v[:, :, perm], g[:, :, perm],
                                          beta[:, :, perm], initial_state=h0[:, perm],
                                          output_final_state=True, dtype=torch.float64)
    torch.testing.assert_close(o2, o1[:, :, perm])
    torch.testing.assert_close(s2, s1[:, perm])


# ---- closed forms ----------------------------------------------------------------

def test_closed_form_beta_zero():
    """beta == 0: S_t = e^{sum g} S_0 and o_t = scale e^{G_t} S_0^T q_t."""
    q, k, v, g, beta, h0 = make_inputs(1, 100, 2, 2, 16, 16, seed=9)
    beta = torch.zeros_like(beta)
    o, s = O.chunk_gated_delta_rule_ref(q, k, v, g, beta, initial_state=h0, output_final_state=True,
                                        dtype=torch.float64)
    G = g.cumsum(1)                                                   # [B,T,H]
    want_s = h0 * G[:, -1].exp()[..., None, None]
    want_o = 16 ** -0.5 * torch.einsum("bhkv,bthk->bthv", h0, q) * G.exp()[..., None]
    torch.testing.assert_close(s, want_s, rtol=1e-10, atol=1e-12)
    torch.testing.assert_close(o, want_o, rtol=1e-10, atol=1e-12)


def test_closed_form_orthonormal_keys():
    """g=0, beta=1, S_0=0, orthonormal keys: S_T = sum k_t v_t^T, o_t = scale sum_{s<=t} (k_s.q_t) v_s."""
    T = K = 16
    gen = torch.Generator().manual_seed(10)
    Qm, _ = torch.linalg.qr(torch.randn(K, K, generator=gen, dtype=torch.float64))
    k = Qm[None, :, None, :]                                          # [1,T,1,K] rows orthonormal
    q = torch.randn(1, T, 1, K, generator=gen, dtype=torch.float64)
    v = torch.randn(1, T, 1, 8, generator=gen, dtype=torch.float64)
    g = torch.zeros(1, T, 1, dtype=torch.float64)
    beta = torch.ones(1, T, 1, dtype=torch.float64)
    o, s = O.chunk_gated_delta_rule_ref(q, k, v, g, beta, output_final_state=True, dtype=torch.float64)
    want_s = torch.einsum("tk,tv->kv", k[0, :, 0], v[0, :, 0])
    torch.testing.assert_close(s[0, 0], want_s, rtol=1e-10, atol=1e-12)
    kq = torch.einsum("sk,tk->ts", k[0, :, 0], q[0, :, 0]).tril()
    want_o = K ** -0.5 * kq @ v[0, :, 0]
    torch.testing.assert_close(o[0, :, 0], want_o, rtol=1e-10, atol=1e-12)


def test_closed_form_overwrite_property():
    """Writing the same unit key twice with beta=1, g=0 leaves k v2^T on that direction."""
    K, V = 8, 4
    kvec = F.normalize(torch.arange(1.0, K + 1, dtype=torch.float64), dim=0)
    k = kvec.expand(1, 2, 1, K).contiguous()
    v = torch.tensor([[1.0, 2, 3, 4], [-5.0, 6, -7, 8]], dtype=torch.float64)[None, :, None, :]
    q = k.clone()
    g = torch.zeros(1, 2, 1, dtype=torch.float64)
    beta = torch.ones(1, 2, 1, dtype=torch.float64)
    _, s = O.chunk_gated_delta_rule_ref(q, k, v, g, beta, output_final_state=True, dtype=torch.float64)
    torch.testing.assert_close(s[0, 0], torch.outer(kvec, v[0, 1, 0]), rtol=1e-12, atol=1e-13)


def test_closed_form_single_token():
    q, k, v, g, beta, h0 = make_inputs(1, 1, 1, 1, 8, 8, seed=11)
    o, s = O.chunk_gated_delta_rule_ref(q, k, v, g, beta, initial_state=h0, output_final_state=True,
                                        dtype=torch.float64)
    S0 = h0[0, 0] * g[0, 0, 0].exp()
    kk, qq, vv = k[0, 0, 0], q[0, 0, 0], v[0, 0, 0]
    S1 = S0 + beta[0, 0, 0] * torch.outer(kk, vv - S0.T @ kk)
    torch.testing.assert_close(s[0, 0], S1, rtol=1e-12, atol=1e-13)
    torch.testing.assert_close(o[0, 0, 0], 8 ** -0.5 * S1.T @ qq, rtol=1e-12, atol=1e-13)


def test_wy_solve_is_library_triangular_inverse():
    """With S_0 = 0 and one chunk, v_new = (I + L)^{-1} (beta v) with
    L = strict_tril(beta_i k_i.k_j e^{G_i-G_j}); so o = scale tril(QK^T Gamma) v_new and the final
    state follow from torch.linalg.solve_triangular."""
    T = 64
    q, k, v, g, beta, _ = make_inputs(1, T, 1, 1, 16, 16, seed=12)
    o, s = O.chunk_gated_delta_rule_ref(q, k, v, g, beta, output_final_state=True, dtype=torch.float64)
    kk, qq, vv, gg, bb = k[0, :, 0], q[0, :, 0], v[0, :, 0], g[0, :, 0], beta[0, :, 0]
    G = gg.cumsum(0)
    Gam = (G[:, None] - G[None, :]).tril().exp().tril()
    L = (bb[:, None] * (kk @ kk.T) * Gam).tril(-1)
    vnew = torch.linalg.solve_triangular(torch.eye(T, dtype=torch.float64) + L, bb[:, None] * vv, upper=False)
    want_o = 16 ** -0.5 * ((qq @ kk.T) * Gam) @ vnew
    want_s = (kk * (G[-1] - G).exp()[:, None]).T @ vnew
    torch.testing.assert_close(o[0, :, 0], want_o, rtol=1e-9, atol=1e-11)
    torch.testing.assert_close(s[0, 0], want_s, rtol=1e-9, atol=1e-11)


# ---- packed sequences -----------------------------------------------------------------

REF_CU = [
    [0, 112, 209, 240, 281, 489, 523, 566, 689, 721, 785, 837, 985] + list(range(986, 1025)),
    [0, 112, 209, 240, 281, 489, 523, 566, 689, 721, 785, 837, 985, 1071, 1121],
    [0] + list(range(804, 809)),
]


@pytest.mark.parametrize("cu", REF_CU, ids=["T1024-1tok", "T1121", "T808-1tok"])
def test_varlen_equals_pad_and_batch(cu):
    """cu_seqlens lists of the reference's own test table
    (test_chunk_gated_delta_rule.py:123-129,138), incl. 1-token sequences."""
    T, N = cu[-1], len(cu) - 1
    q, k, v, g, beta, h0 = make_inputs(1, T, 1, 2, 8, 8, seed=13, N=N)
    o, s = O.chunk_gated_delta_rule_ref(q, k, v, g, beta, initial_state=h0, output_final_state=True,
                                        cu_seqlens=cu, dtype=torch.float64)
    qb, kb, vb, gb, bb = O.pad_and_batch(cu, q, k, v, g, beta)
    ob, sb = O.chunk_gated_delta_rule_ref(qb, kb, vb, gb, bb, initial_state=h0, output_final_state=True,
                                          dtype=torch.float64)
    (o_b,) = O.pad_and_batch(cu, o)
    lens = torch.tensor([cu[i + 1] - cu[i] for i in range(N)])
    mask = (torch.arange(ob.shape[1])[None] < lens[:, None])[..., None, None]
    torch.testing.assert_close(o_b, ob * mask, rtol=1e-10, atol=1e-11)
    torch.testing.assert_close(s, sb, rtol=1e-10, atol=1e-11)
    on, sn = O.naive_gated_delta_rule(q, k, v, g, beta, initial_state=h0, output_final_state=True, cu_seqlens=cu)
    torch.testing.assert_close(o, on, rtol=1e-10, atol=1e-11)
    torch.testing.assert_close(s, sn, rtol=1e-10, atol=1e-11)


# ---- backward ----------------------------------------------------------------------------

def _grads(fn, args, h0, l2, cu=None, seed=0):
    args = [a.detach().clone().requires_grad_(True) for a in args]
    h0 = h0.detach().clone().requires_grad_(True)
    o, s = fn(*args, initial_state=h0, output_final_state=True, use_qk_l2norm_in_kernel=l2, cu_seqlens=cu)
    gen = torch.Generator().manual_seed(100 + seed)
    do = torch.randn(o.shape, generator=gen, dtype=o.dtype)
    ds = torch.randn(s.shape, generator=gen, dtype=s.dtype)
    ((o * do).sum() + (s * ds).sum()).backward()
    return [a.grad for a in args] + [h0.grad]


@pytest.mark.parametrize("l2,cu", [(False, None), (True, None), (True, [0, 5, 70, 71, 140])])
def test_backward_chunk_equals_recurrence(l2, cu):
    T = 140 if cu else 100
    B = 1 if cu else 2
    q, k, v, g, beta, h0 = make_inputs(B, T, 2, 4, 8, 8, seed=14, normalize=not l2, N=(4 if cu else B))
    chunk = lambda *a, **kw: O.chunk_gated_delta_rule_ref(*a, dtype=torch.float64, **kw)
    g1 = _grads(O.naive_gated_delta_rule, (q, k, v, g, beta), h0, l2, cu)
    g2 = _grads(chunk, (q, k, v, g, beta), h0, l2, cu)
    for a, b, name in zip(g2, g1, "dq dk dv dg dbeta dh0".split()):
        torch.testing.assert_close(a, b, rtol=1e-8, atol=1e-10, msg=lambda m, n=name: f"{n}: {m}")


def test_gradcheck_recurrence_tiny():
    q, k, v, g, beta, h0 = make_inputs(1, 5, 1, 2, 3, 2, seed=15, normalize=False)
    args = [a.requires_grad_(True) for a in (q, k, v, g, beta, h0)]

    def f(q, k, v, g, beta, h0):
        o, s = O.naive_gated_delta_rule(q, k, v, g, beta, initial_state=h0, output_final_state=True,
                                        use_qk_l2norm_in_kernel=True)
        return o, s

    assert torch.autograd.gradcheck(f, args, eps=1e-6, atol=1e-6)


# ---- golden vectors ------------------------------------------------------------------------

@pytest.mark.parametrize("name", ["gdn_T128_H2_d16", "gdn_varlen_T96_H2_d16"])
def test_golden_vectors(name):
    z = np.load(os.path.join(GOLD, name + ".npz"))
    t = {k_: torch.from_numpy(z[k_]) for k_ in z.files}
    cu = t["cu_seqlens"].tolist() if "cu_seqlens" in t else None
    args = [t[n].clone().requires_grad_(True) for n in ("q", "k", "v", "g", "beta")]
    h0 = t["h0"].clone().requires_grad_(True)
    o, s = O.chunk_gated_delta_rule_ref(*args, initial_state=h0, output_final_state=True,
                                        use_qk_l2norm_in_kernel=True, cu_seqlens=cu, dtype=torch.float64)
    torch.testing.assert_close(o, t["o"], rtol=1e-9, atol=1e-11)
    torch.testing.assert_close(s, t["ht"], rtol=1e-9, atol=1e-11)
    ((o * t["do"]).sum() + (s * t["dht"]).sum()).backward()
    for a, n in zip(args + [h0], ("dq", "dk", "dv", "dg", "dbeta", "dh0")):
        torch.testing.assert_close(a.grad, t[n], rtol=1e-8, atol=1e-10)
    # fp32 chunked oracle, the one GPU parity tests use, stays within 1e-4 of the fp64 truth
    o32, s32 = O.chunk_gated_delta_rule_ref(*[a.detach().float() for a in args], initial_state=h0.detach().float(),
                                            output_final_state=True, use_qk_l2norm_in_kernel=True, cu_seqlens=cu)
    assert (o32.double() - t["o"]).abs().max() / t["o"].abs().max() < 1e-5
    assert (s32.double() - t["ht"]).abs().max() / t["ht"].abs().max() < 1e-5
