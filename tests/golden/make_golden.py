"""Writes the golden vectors under tests/golden/.

The vectors come from the fp64 textbook recurrence (``naive_gated_delta_rule``) and autograd through
it -- an algorithm independent of the chunked algebra that both the chunked oracle and the HIP kernels
use.  The reference holds no stored vectors for this path, and nothing from the reference is imported.

    python tests/golden/make_golden.py
"""
import math
import os
import sys

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import gdn_oracle as O  # noqa: E402
from oracle import kda_oracle as KO  # noqa: E402


def make(name, T, Hqk, Hv, K, V, seed, cu=None):
    gen = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float64)
    N = (len(cu) - 1) if cu else 1
    q, k, v = r(1, T, Hqk, K), r(1, T, Hqk, K), r(1, T, Hv, V)
    beta = torch.sigmoid(r(1, T, Hv))
    A_log = torch.empty(Hv, dtype=torch.float64).uniform_(0.0, math.log(16.0), generator=gen)
    dt_bias = torch.empty(Hv, dtype=torch.float64).uniform_(-4.0, -2.0, generator=gen)
    g = -A_log.exp() * F.softplus(r(1, T, Hv) + dt_bias)
    h0 = 0.5 * r(N, Hv, K, V)
    do, dht = r(1, T, Hv, V), r(N, Hv, K, V)
    leaves = [x.clone().requires_grad_(True) for x in (q, k, v, g, beta, h0)]
    o, ht = O.naive_gated_delta_rule(*leaves[:5], initial_state=leaves[5], output_final_state=True,
                                     use_qk_l2norm_in_kernel=True, cu_seqlens=cu)
    ((o * do).sum() + (ht * dht).sum()).backward()
    out = dict(q=q, k=k, v=v, g=g, beta=beta, h0=h0, do=do, dht=dht, o=o.detach(), ht=ht.detach())
    for n, leaf in zip(("dq", "dk", "dv", "dg", "dbeta", "dh0"), leaves):
        out[n] = leaf.grad
    out = {k_: v_.numpy() for k_, v_ in out.items()}
    if cu:
        out["cu_seqlens"] = np.asarray(cu, dtype=np.int64)
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **out)


def make_kda(name, T, H, K, V, seed, cu=None):
    """KDA: raw gate input per key channel, the gate and the sigmoid of beta applied before the fp64 per-token
    recurrence (the vectors hold the raw inputs and the gradients with respect to them)."""
    gen = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float64)
    N = (len(cu) - 1) if cu else 1
    q, k, v, g = r(1, T, H, K), r(1, T, H, K), r(1, T, H, V), r(1, T, H, K)
    beta = r(1, T, H)
    A_log = torch.empty(H, dtype=torch.float64).uniform_(0.0, math.log(16.0), generator=gen)
    dt_bias = torch.empty(H * K, dtype=torch.float64).uniform_(-4.0, -2.0, generator=gen)
    h0 = 0.5 * r(N, H, K, V)
    do, dht = r(1, T, H, V), r(N, H, K, V)
    leaves = [x.clone().requires_grad_(True) for x in (q, k, v, g, beta, h0, A_log, dt_bias)]
    lq, lk, lv, lg, lb, lh, la, ld = leaves
    qn = lq * torch.rsqrt((lq * lq).sum(-1, keepdim=True) + 1e-6)
    kn = lk * torch.rsqrt((lk * lk).sum(-1, keepdim=True) + 1e-6)
    gl = -la.exp().reshape(H, 1) * F.softplus(lg + ld.reshape(H, K))
    o, ht = KO.naive_kda_recurrence(qn, kn, lv, gl, torch.sigmoid(lb), initial_state=lh, output_final_state=True,
                                    cu_seqlens=cu)
    ((o * do).sum() + (ht * dht).sum()).backward()
    out = dict(q=q, k=k, v=v, g=g, beta=beta, h0=h0, A_log=A_log, dt_bias=dt_bias, do=do, dht=dht, o=o.detach(),
               ht=ht.detach())
    for n, leaf in zip(("dq", "dk", "dv", "dg", "dbeta", "dh0", "dA_log", "ddt_bias"), leaves):
        out[n] = leaf.grad
    out = {k_: v_.numpy() for k_, v_ in out.items()}
    if cu:
        out["cu_seqlens"] = np.asarray(cu, dtype=np.int64)
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **out)


if __name__ == "__main__":
    make("gdn_T128_H2_d16", T=128, Hqk=1, Hv=2, K=16, V=16, seed=0)
    make("gdn_varlen_T96_H2_d16", T=96, Hqk=2, Hv=2, K=16, V=16, seed=1, cu=[0, 1, 38, 96])
    make_kda("kda_T96_H2_d16", T=96, H=2, K=16, V=16, seed=2, cu=[0, 1, 38, 96])
