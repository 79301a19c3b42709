"""Pins the CPU oracle of KDA (oracle/kda_oracle.py) against independent facts: the textbook per-token recurrence in
fp64 (values and, through autograd, gradients), the scalar-gate operator it reduces to when every channel decays
alike, invariants (chunk size, padding, state continuity, packing, state layout), a library triangular solve,
closed forms of the gate, and committed golden vectors."""
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import gdn_oracle as GO
from oracle import kda_oracle as KO

GOLD = os.path.join(os.path.dirname(__file__), "golden")
F64 = torch.float64


def make(B, T, H, K, V, seed=0, N=None, slow=False):
    gen = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=gen, dtype=F64)
    q, k, v = r(B, T, H, K), r(B, T, H, K), r(B, T, H, V)
    q, k = GO.l2norm(q), GO.l2norm(k)
    a = torch.empty(H, 1, dtype=F64).uniform_(0.0 if not slow else -1.0, math.log(16.0) if not slow else 0.5, generator=gen)
    g = -a.exp() * F.softplus(r(B, T, H, K) + torch.empty(H, K, dtype=F64).uniform_(-4.0, -2.0, generator=gen))
    beta = torch.sigmoid(r(B, T, H))
    h0 = 0.5 * r(N if N is not None else B, H, K, V)
    return q, k, v, g, beta, h0


def ref64(q, k, v, g, beta, h0=None, **kw):
    return KO.chunk_kda_ref(q, k, v, g, beta, initial_state=h0, output_final_state=True, compute_dtype=F64,
                            round_output=False, **kw)


@pytest.mark.parametrize("B,T,H,K,V", [(1, 64, 2, 16, 16), (2, 100, 3, 16, 24), (1, 193, 1, 8, 12), (1, 1, 2, 16, 16)])
def test_chunk_equals_recurrence(B, T, H, K, V):
    q, k, v, g, beta, h0 = make(B, T, H, K, V, seed=1)
    o1, s1 = KO.naive_kda_recurrence(q, k, v, g, beta, initial_state=h0, output_final_state=True)
    o2, s2 = ref64(q, k, v, g, beta, h0)
    torch.testing.assert_close(o2, o1, rtol=1e-9, atol=1e-11)
    torch.testing.assert_close(s2, s1, rtol=1e-9, atol=1e-11)


def test_gradients_equal_recurrence_autograd():
    q, k, v, g, beta, h0 = make(1, 80, 2, 8, 8, seed=2, slow=True)
    gen = torch.Generator().manual_seed(3)
    do, dht = torch.randn(1, 80, 2, 8, generator=gen, dtype=F64), torch.randn(1, 2, 8, 8, generator=gen, dtype=F64)
    grads = []
    for fn in (lambda *a: KO.naive_kda_recurrence(*a[:5], initial_state=a[5], output_final_state=True),
               lambda *a: ref64(*a[:5], a[5])):
        leaves = [x.clone().requires_grad_(True) for x in (q, k, v, g, beta, h0)]
        o, ht = fn(*leaves)
        ((o * do).sum() + (ht * dht).sum()).backward()
        grads.append([x.grad for x in leaves])
    for a, b in zip(*grads):
        torch.testing.assert_close(b, a, rtol=1e-8, atol=1e-10)


def test_gradcheck_small():
    q, k, v, g, beta, h0 = make(1, 20, 1, 4, 4, seed=4, slow=True)
    leaves = [x.clone().requires_grad_(True) for x in (q, k, v, g, beta, h0)]
    f = lambda *a: ref64(*a[:5], a[5], chunk_size=8)
    assert torch.autograd.gradcheck(f, leaves, eps=1e-6, atol=1e-6, rtol=1e-4)


def test_same_gate_on_every_channel_is_the_scalar_gate_operator():
    """g[d] = g for all d: diag(e^g) S = e^g S, the gated delta rule, whose oracle is pinned to the reference."""
    B, T, H, K, V = 2, 150, 2, 16, 16
    q, k, v, g, beta, h0 = make(B, T, H, K, V, seed=5)
    gs = g[..., 0]
    o1, s1 = GO.chunk_gated_delta_rule_ref(q, k, v, gs, beta, initial_state=h0, output_final_state=True, dtype=F64)
    o2, s2 = ref64(q, k, v, gs[..., None].expand(B, T, H, K), beta, h0)
    torch.testing.assert_close(o2, o1, rtol=1e-9, atol=1e-11)
    torch.testing.assert_close(s2, s1, rtol=1e-9, atol=1e-11)


def test_chunk_size_and_padding_invariance():
    q, k, v, g, beta, h0 = make(1, 128, 2, 8, 8, seed=6)
    o64, s64 = ref64(q, k, v, g, beta, h0)
    for c in (16, 32):
        o, s = ref64(q, k, v, g, beta, h0, chunk_size=c)
        torch.testing.assert_close(o, o64, rtol=1e-9, atol=1e-11)
        torch.testing.assert_close(s, s64, rtol=1e-9, atol=1e-11)
    # beta = 0 and g = 0 on appended tokens leave the state alone
    z = lambda x: torch.cat([x, torch.zeros(1, 7, *x.shape[2:], dtype=F64)], 1)
    o, s = ref64(z(q), z(k), z(v), z(g), z(beta), h0)
    torch.testing.assert_close(o[:, :128], o64, rtol=1e-9, atol=1e-11)
    torch.testing.assert_close(s, s64, rtol=1e-9, atol=1e-11)


def test_state_continuity_and_packing_and_layout():
    q, k, v, g, beta, h0 = make(1, 170, 2, 8, 12, seed=7)
    o, s = ref64(q, k, v, g, beta, h0)
    oa, sa = ref64(q[:, :70], k[:, :70], v[:, :70], g[:, :70], beta[:, :70], h0)
    ob, sb = ref64(q[:, 70:], k[:, 70:], v[:, 70:], g[:, 70:], beta[:, 70:], sa)
    torch.testing.assert_close(torch.cat([oa, ob], 1), o, rtol=1e-9, atol=1e-11)
    torch.testing.assert_close(sb, s, rtol=1e-9, atol=1e-11)
    # packed: three sequences, one of them of length 1, one empty
    cu = [0, 1, 1, 70, 170]
    h4 = 0.5 * torch.randn(4, 2, 8, 12, dtype=F64, generator=torch.Generator().manual_seed(8))
    op, sp = ref64(q, k, v, g, beta, h4, cu_seqlens=cu)
    for n in range(4):
        a, b = cu[n], cu[n + 1]
        if b == a:
            torch.testing.assert_close(sp[n], h4[n])
            continue
        on, sn = ref64(q[:, a:b], k[:, a:b], v[:, a:b], g[:, a:b], beta[:, a:b], h4[n:n + 1])
        torch.testing.assert_close(op[:, a:b], on, rtol=1e-9, atol=1e-11)
        torch.testing.assert_close(sp[n:n + 1], sn, rtol=1e-9, atol=1e-11)
    ot, st = ref64(q, k, v, g, beta, h4.transpose(-1, -2).contiguous(), cu_seqlens=cu, transpose_state_layout=True)
    torch.testing.assert_close(ot, op)
    torch.testing.assert_close(st, sp.transpose(-1, -2))


def test_tm_is_the_inverse_of_i_plus_l():
    """U = (I+L)^-1 (beta v): with S0 = 0 the first chunk's v_new is U; check through o of a single chunk with q = k
    chosen so that o = Aq U, against torch.linalg.solve_triangular."""
    T, H, K, V = 64, 1, 8, 8
    q, k, v, g, beta, _ = make(1, T, H, K, V, seed=9)
    G = g[0, :, 0].cumsum(0)
    gam = (G[:, None, :] - G[None, :, :]).clamp(max=80).exp()
    kk = torch.einsum("id,jd,ijd->ij", k[0, :, 0], k[0, :, 0], gam)
    L = torch.tril(beta[0, :, 0, None] * kk, -1)
    U = torch.linalg.solve_triangular(torch.eye(T, dtype=F64) + L, beta[0, :, 0, None] * v[0, :, 0], upper=False)
    Aq = torch.tril(torch.einsum("id,jd,ijd->ij", q[0, :, 0], k[0, :, 0], gam)) * K ** -0.5
    o, _ = ref64(q, k, v, g, beta, None)
    torch.testing.assert_close(o[0, :, 0], Aq @ U, rtol=1e-9, atol=1e-11)


def test_gate_closed_forms_and_library_routines():
    H, K = 3, 5
    gen = torch.Generator().manual_seed(10)
    A_log = torch.randn(H, generator=gen, dtype=F64)
    dt_bias = torch.randn(H * K, generator=gen, dtype=F64)
    x = torch.randn(2, 7, H, K, generator=gen, dtype=F64)
    zero = -dt_bias.reshape(H, K).expand(2, 7, H, K)
    torch.testing.assert_close(KO.kda_gate_ref(zero, A_log, dt_bias, dtype=F64),
                               (-A_log.exp() * math.log(2.0))[:, None].expand(2, 7, H, K))
    torch.testing.assert_close(KO.kda_gate_ref(zero, A_log, dt_bias, lower_bound=-5.0, dtype=F64),
                               torch.full((2, 7, H, K), -2.5, dtype=F64))
    y = x + dt_bias.reshape(H, K)
    a = A_log.exp()[:, None]
    torch.testing.assert_close(KO.kda_gate_ref(x, A_log, dt_bias, dtype=F64), -a * torch.logaddexp(y, torch.zeros_like(y)))
    torch.testing.assert_close(KO.kda_gate_ref(x, A_log, dt_bias, lower_bound=-5.0, dtype=F64), -5.0 * torch.special.expit(a * y))
    torch.testing.assert_close(KO.kda_gate_ref(x, A_log, None, dtype=F64), -a * torch.logaddexp(x, torch.zeros_like(x)))
    leaves = [t.clone().requires_grad_(True) for t in (x, A_log, dt_bias)]
    assert torch.autograd.gradcheck(lambda a_, b_, c_: KO.kda_gate_ref(a_, b_, c_, dtype=F64), leaves)
    assert torch.autograd.gradcheck(lambda a_, b_, c_: KO.kda_gate_ref(a_, b_, c_, lower_bound=-5.0, dtype=F64), leaves)


def test_operator_options_equal_preprocessed_inputs():
    """l2 norm, gate, sigmoid of beta applied by the operator == applied by the caller."""
    B, T, H, K, V = 1, 90, 2, 8, 8
    gen = torch.Generator().manual_seed(11)
    r = lambda *s: torch.randn(*s, generator=gen, dtype=F64)
    q, k, v, graw, braw = r(B, T, H, K), r(B, T, H, K), r(B, T, H, V), r(B, T, H, K), r(B, T, H)
    A_log, dt_bias = r(H), r(H * K)
    o1, s1 = ref64(q, k, v, graw, braw, None, use_qk_l2norm_in_kernel=True, use_gate_in_kernel=True,
                   use_beta_sigmoid_in_kernel=True, allow_neg_eigval=True, A_log=A_log, dt_bias=dt_bias)
    # the operator normalises in fp32 and rounds to the input type, as the reference does
    qn, kn = (GO.l2norm(x.float()).to(F64) for x in (q, k))
    o2, s2 = ref64(qn, kn, v, KO.kda_gate_ref(graw, A_log, dt_bias, dtype=F64), 2.0 * torch.sigmoid(braw), None)
    torch.testing.assert_close(o1, o2, rtol=1e-9, atol=1e-11)
    torch.testing.assert_close(s1, s2, rtol=1e-9, atol=1e-11)
    with pytest.raises(ValueError):
        ref64(q, k, v, graw, braw, None, allow_neg_eigval=True)
    with pytest.raises(ValueError):
        ref64(q, k, v, graw, braw, None, use_gate_in_kernel=True)


def test_fp32_close_to_fp64_and_output_dtype():
    q, k, v, g, beta, h0 = make(1, 256, 2, 32, 32, seed=12)
    o1, s1 = KO.naive_kda_recurrence(q, k, v, g, beta, initial_state=h0, output_final_state=True)
    o2, s2 = KO.chunk_kda_ref(q.float(), k.float(), v.float(), g.float(), beta.float(), initial_state=h0.float(),
                              output_final_state=True)
    assert o2.dtype == torch.float32 and s2.dtype == torch.float32
    assert (o2.double() - o1).abs().max() / o1.abs().max() < 1e-5
    assert (s2.double() - s1).abs().max() / s1.abs().max() < 1e-5
    o3, _ = KO.chunk_kda_ref(q.bfloat16(), k.bfloat16(), v.bfloat16(), g.float(), beta.float())
    assert o3.dtype == torch.bfloat16


def test_golden_vectors():
    z = np.load(os.path.join(GOLD, "kda_T96_H2_d16.npz"))
    t = {n: torch.from_numpy(z[n]) for n in z.files}
    cu = t["cu_seqlens"].tolist()
    leaves = [t[n].clone().requires_grad_(True) for n in ("q", "k", "v", "g", "beta", "h0", "A_log", "dt_bias")]
    lq, lk, lv, lg, lb, lh, la, ld = leaves
    qn, kn = GO.l2norm(lq), GO.l2norm(lk)   # unrounded: the vectors are fp64
    o, ht = ref64(qn, kn, lv, lg, lb, lh, use_gate_in_kernel=True, use_beta_sigmoid_in_kernel=True, A_log=la, dt_bias=ld,
                  cu_seqlens=cu)
    torch.testing.assert_close(o, t["o"], rtol=1e-8, atol=1e-10)
    torch.testing.assert_close(ht, t["ht"], rtol=1e-8, atol=1e-10)
    ((o * t["do"]).sum() + (ht * t["dht"]).sum()).backward()
    for n, leaf in zip(("dq", "dk", "dv", "dg", "dbeta", "dh0", "dA_log", "ddt_bias"), leaves):
        torch.testing.assert_close(leaf.grad, t[n], rtol=1e-7, atol=1e-9)


def test_intermediate_states_are_the_recurrence_states_at_chunk_entries():
    """h[:, c] is the state the per-token recurrence holds after 64 c tokens of the sequence (chunk_kda_naive.py:287-303):
    dense batches, packed sequences (chunks of all sequences in order; an empty sequence contributes none), the
    transposed layout, the cast to the input type."""
    q, k, v, g, beta, h0 = make(2, 150, 2, 8, 12, seed=11)
    o, s, h = ref64(q, k, v, g, beta, h0, return_intermediate_states=True)
    assert h.shape == (2, 3, 2, 8, 12)
    for c in range(3):
        if c == 0:
            want = h0
        else:
            _, want = KO.naive_kda_recurrence(q[:, :64 * c], k[:, :64 * c], v[:, :64 * c], g[:, :64 * c], beta[:, :64 * c],
                                              initial_state=h0, output_final_state=True)
        torch.testing.assert_close(h[:, c], want, rtol=1e-9, atol=1e-11)
    cu = [0, 1, 1, 70, 150]
    h4 = 0.5 * torch.randn(4, 2, 8, 12, dtype=F64, generator=torch.Generator().manual_seed(12))
    _, _, hp = ref64(q[:1], k[:1], v[:1], g[:1], beta[:1], h4, cu_seqlens=cu, return_intermediate_states=True)
    assert hp.shape == (1, 1 + 0 + 2 + 2, 2, 8, 12)
    at = 0
    for n in range(4):
        a, b = cu[n], cu[n + 1]
        for c in range((b - a + 63) // 64):
            if c == 0:
                want = h4[n:n + 1]
            else:
                _, want = KO.naive_kda_recurrence(q[:1, a:a + 64 * c], k[:1, a:a + 64 * c], v[:1, a:a + 64 * c],
                                                  g[:1, a:a + 64 * c], beta[:1, a:a + 64 * c], initial_state=h4[n:n + 1],
                                                  output_final_state=True)
            torch.testing.assert_close(hp[:, at], want, rtol=1e-9, atol=1e-11)
            at += 1
    _, _, ht = ref64(q[:1], k[:1], v[:1], g[:1], beta[:1], h4.transpose(-1, -2).contiguous(), cu_seqlens=cu,
                     transpose_state_layout=True, return_intermediate_states=True)
    torch.testing.assert_close(ht, hp.transpose(-1, -2))
    qb, kb, vb = q.to(torch.bfloat16), k.to(torch.bfloat16), v.to(torch.bfloat16)
    _, _, hb = KO.chunk_kda_ref(qb, kb, vb, g.float(), beta.float(), initial_state=h0.float(), return_intermediate_states=True)
    assert hb.dtype == torch.bfloat16 and hb.shape == h.shape
