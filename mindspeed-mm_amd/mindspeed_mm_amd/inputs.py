"""Synthetic inputs of the benchmark configurations (CPU-generated from one seeded generator, so host and
device runs see identical bits).  Caller-side recipe of the reference module:
beta = sigmoid(b), g = -exp(A_log) * softplus(a + dt_bias)  (mindspeed_mm/fsdp/models/qwen3_5/modeling_qwen3_5.py:833-841)."""
import math

import torch
import torch.nn.functional as F


def gdn_inputs(B, T, Hqk, Hv, K, V, dtype, seed=0, N=None, l2norm_in_kernel=True, a_log=(1.0, 16.0),
               dt_bias=(-4.0, -2.0), h0_std=0.02):
    """q,k ~ N(0,1) (L2-normalised here when the kernel is not asked to), v ~ N(0,1), beta = sigmoid(N(0,1)),
    g = -exp(A_log) softplus(N(0,1) + dt_bias) with per-head A_log ~ U(log a0, log a1), dt_bias ~ U(b0, b1);
    h0, dht ~ N(0, h0_std) fp32; do ~ N(0,1)."""
    gen = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=gen)
    q, k, v = r(B, T, Hqk, K), r(B, T, Hqk, K), r(B, T, Hv, V)
    if not l2norm_in_kernel:
        q = q * torch.rsqrt((q * q).sum(-1, keepdim=True) + 1e-6)
        k = k * torch.rsqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(r(B, T, Hv))
    A_log = torch.empty(Hv).uniform_(math.log(a_log[0]), math.log(a_log[1]), generator=gen)
    bias = torch.empty(Hv).uniform_(dt_bias[0], dt_bias[1], generator=gen)
    g = -A_log.exp() * F.softplus(r(B, T, Hv) + bias)
    n = N if N is not None else B
    h0 = h0_std * r(n, Hv, K, V)
    do = r(B, T, Hv, V)
    dht = h0_std * r(n, Hv, K, V)
    return dict(q=q.to(dtype), k=k.to(dtype), v=v.to(dtype), g=g, beta=beta.to(dtype), h0=h0, do=do.to(dtype),
                dht=dht)


def packed_lengths(n_seq=24, total=32768, lo=64, hi=4096, seed=0):
    """Sequence lengths log-uniform in [lo, hi] whose sum is exactly `total` (last ones adjusted); deterministic."""
    gen = torch.Generator().manual_seed(seed)
    u = torch.empty(n_seq).uniform_(math.log(lo), math.log(hi), generator=gen)
    lens = [int(round(x)) for x in u.exp().tolist()]
    scale = total / sum(lens)
    lens = [max(lo, min(hi, int(round(x * scale)))) for x in lens]
    i = 0
    while sum(lens) != total:                      # spread the rounding remainder, staying inside [lo, hi]
        d = 1 if sum(lens) < total else -1
        if lo <= lens[i % n_seq] + d <= hi:
            lens[i % n_seq] += d
        i += 1
    cu = [0]
    for x in lens:
        cu.append(cu[-1] + x)
    return cu


def kda_inputs(B, T, H, K, V, dtype, seed=0, N=None, a_log=(1.0, 16.0), dt_bias=(-4.0, -2.0), h0_std=0.02):
    """Inputs of the KDA operator as its layer hands them over (mindspeed_mm/fsdp/models/kimi_k3/
    modeling_kimi_linear.py:584-596, 665-671): q, k, v ~ N(0,1); the raw gate input g ~ N(0,1) per key channel with
    A_log ~ U(log a0, log a1) per head and dt_bias ~ U(b0, b1) per head and channel; beta raw ~ N(0,1) (the
    operator applies the sigmoid); h0, dht ~ N(0, h0_std) fp32 in [N,H,K,V]; do ~ N(0,1)."""
    gen = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=gen)
    q, k, v, g = r(B, T, H, K), r(B, T, H, K), r(B, T, H, V), r(B, T, H, K)
    beta = r(B, T, H)
    A_log = torch.empty(H).uniform_(math.log(a_log[0]), math.log(a_log[1]), generator=gen)
    bias = torch.empty(H * K).uniform_(dt_bias[0], dt_bias[1], generator=gen)
    n = N if N is not None else B
    h0 = h0_std * r(n, H, K, V)
    do = r(B, T, H, V)
    dht = h0_std * r(n, H, K, V)
    return dict(q=q.to(dtype), k=k.to(dtype), v=v.to(dtype), g=g.to(dtype), beta=beta.to(dtype), A_log=A_log,
                dt_bias=bias, h0=h0, do=do.to(dtype), dht=dht)
