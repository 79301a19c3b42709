"""CPU oracle for the KDA (Kimi delta attention) operator.  TEST INFRASTRUCTURE ONLY.

This file is the checker, never the product: only ``tests/``, the smoke entry
and the ``cpu_baseline`` leg of the benchmark may import it.  The shipped
operator lives in the HIP library and refuses to run without it.

A from-scratch restatement, in plain PyTorch on the CPU, of the reference's
pure-PyTorch KDA (paths relative to the reference checkout):

* ``kda_gate_ref``   mindspeed_mm/fsdp/ops/kda/chunk_kda_naive.py:76-104  (``kda_gate``)
* ``chunk_kda_ref``  chunk_kda_naive.py:106-221 (``_chunk_kda_core``: WY form per chunk of 64 tokens, the state
                     carried from chunk to chunk) and :223-381 (``chunk_kda_naive``: l2 norm rounded to the input
                     type, gate and beta transforms in fp32, the [N,H,V,K] state layout, packed sequences run one
                     by one, output cast back to the input type)

KDA is the gated delta rule with one decay per key channel: the state S [K,V] of a head evolves per token as

    S <- diag(e^{g_t}) S;   S <- S + beta_t k_t (v_t - S^T k_t)^T;   o_t = scale S^T q_t.

``naive_kda_recurrence`` states exactly that, token by token in fp64, independently of the chunk algebra.

How each function is pinned (tests/test_oracle_kda.py):

* chunked form == the fp64 per-token recurrence (outputs, final state and, through autograd, all gradients);
* a gate that is the same for every channel reduces KDA to the scalar-gate operator: equal to
  ``gdn_oracle.chunk_gated_delta_rule_ref``, which is itself pinned to the reference's functions;
* invariance to the chunk size (16, 32, 64) and to zero padding, state continuity across a split sequence,
  packed == one by one, the transposed state layout;
* ``(I+L)^-1`` == ``torch.linalg.solve_triangular``;
* gate closed forms: x + dt_bias = 0 gives -e^{A_log} ln 2, with a lower bound lb/2; against
  ``torch.logaddexp`` / ``torch.special.expit`` in fp64; ``gradcheck``;
* committed vectors ``tests/golden/kda_T96_H2_d16.npz`` (made by the fp64 recurrence) guard against drift.

The reference holds no test or stored vector for KDA and its fused kernels (``triton_ascend_kernels``) are absent:
parity is defined against the PyTorch function cited above.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn.functional as F


def _l2norm_rounded(x: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """fp32 normalisation, result rounded to the input type (chunk_kda_naive.py:65-71)."""
    xf = x.float()
    return (xf * torch.rsqrt((xf * xf).sum(-1, keepdim=True) + eps)).to(x.dtype)


def kda_gate_ref(g: torch.Tensor, A_log: torch.Tensor, dt_bias: Optional[torch.Tensor] = None,
                 lower_bound: Optional[float] = None, dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Log decay per key channel from the raw gate input g [..., H, K] (chunk_kda_naive.py:76-104):
    -e^{A_log[h]} softplus(g + dt_bias), or with a lower bound  lb * sigmoid(e^{A_log[h]} (g + dt_bias))."""
    H, K = g.shape[-2:]
    x = g.to(dtype)
    if dt_bias is not None:
        x = x + dt_bias.to(dtype).reshape(H, K)
    a = A_log.to(dtype).reshape(H, 1).exp()
    if lower_bound is not None:
        return lower_bound * torch.sigmoid(a * x)
    return -a * F.softplus(x)


def _seqs(cu_seqlens, B: int, T: int):
    if cu_seqlens is None:
        return [(b, 0, T) for b in range(B)]
    cu = [int(c) for c in (cu_seqlens.tolist() if torch.is_tensor(cu_seqlens) else cu_seqlens)]
    return [(0, cu[i], cu[i + 1]) for i in range(len(cu) - 1)]


def naive_kda_recurrence(q, k, v, g, beta, scale: Optional[float] = None,
                         initial_state: Optional[torch.Tensor] = None, output_final_state: bool = False,
                         cu_seqlens=None, dtype: torch.dtype = torch.float64
                         ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Textbook per-token recurrence.  q,k,g [B,T,H,K] (g the log decay), v [B,T,H,V], beta [B,T,H],
    state [N,H,K,V].  Differentiable in ``dtype``."""
    B, T, H, K = k.shape
    V = v.shape[-1]
    q, k, v, g, beta = (x.to(dtype) for x in (q, k, v, g, beta))
    if scale is None:
        scale = K ** -0.5
    rows = [[None] * T for _ in range(B)]
    finals = []
    for n, (b, s, e) in enumerate(_seqs(cu_seqlens, B, T)):
        S = torch.zeros(H, K, V, dtype=dtype) if initial_state is None else initial_state[n].to(dtype)
        for t in range(s, e):
            S = S * g[b, t].exp()[:, :, None]
            err = v[b, t] - torch.einsum("hkv,hk->hv", S, k[b, t])
            S = S + k[b, t][:, :, None] * (beta[b, t][:, None] * err)[:, None, :]
            rows[b][t] = scale * torch.einsum("hkv,hk->hv", S, q[b, t])
        finals.append(S)
    zero = torch.zeros(H, V, dtype=dtype)
    o = torch.stack([torch.stack([r if r is not None else zero for r in rs]) for rs in rows])
    return o, (torch.stack(finals) if output_final_state else None)


def _kda_chunks(q, k, v, g, beta, scale, S0, chunk: int):
    """One sequence, all heads: q,k,g [T,H,K], v [T,H,V], beta [T,H] in the compute type; S0 [H,K,V].
    Returns o [T,H,V], the final state and the state at the entry of every chunk [nc,H,K,V]
    (chunk_kda_naive.py:139-216)."""
    T, H, K = k.shape
    V = v.shape[-1]
    dt = k.dtype
    pad = (-T) % chunk
    if pad:
        q, k, v, g = (torch.cat([x, x.new_zeros(pad, *x.shape[1:])]) for x in (q, k, v, g))
        beta = torch.cat([beta, beta.new_zeros(pad, H)])
    nc = (T + pad) // chunk
    # [H, nc, C, .]
    q, k, v, g = (x.reshape(nc, chunk, H, -1).permute(2, 0, 1, 3) for x in (q, k, v, g))
    beta = beta.reshape(nc, chunk, H).permute(2, 0, 1)
    G = g.cumsum(-2)                                             # decay from the chunk start up to and including token i
    idx = torch.arange(chunk)
    # Gam[i, j, d] = e^{G_i[d] - G_j[d]}: only i >= j is ever used; the exponent of the rest is clamped, not read
    diff = (G[..., :, None, :] - G[..., None, :, :]).clamp(max=80.0)
    gam = diff.exp()
    kk = torch.einsum("hcid,hcjd,hcijd->hcij", k, k, gam)
    qk = torch.einsum("hcid,hcjd,hcijd->hcij", q, k, gam)
    strict = (idx[:, None] > idx[None, :]).to(dt)
    lower = (idx[:, None] >= idx[None, :]).to(dt)
    L = beta[..., :, None] * kk * strict                         # strictly lower triangular
    # Tm = (I + L)^-1 row by row: row i of (I + L) Tm = I reads  Tm[i] = e_i - sum_{m<i} L[i,m] Tm[m]
    eye = torch.eye(chunk, dtype=dt)
    tm_rows = []
    for i in range(chunk):
        r = eye[i].expand(H, nc, chunk)
        if i:
            r = r - torch.einsum("hcm,hcmj->hcj", L[..., i, :i], torch.stack(tm_rows, dim=-2))
        tm_rows.append(r)
    Tm = torch.stack(tm_rows, dim=-2)
    U = Tm @ (beta[..., None] * v)                               # [H, nc, C, V]
    W = Tm @ (beta[..., None] * k * G.exp())                     # [H, nc, C, K]
    Aq = scale * qk * lower
    S = S0
    outs, entries = [], []
    for c in range(nc):
        entries.append(S)
        vn = U[:, c] - W[:, c] @ S                               # what the chunk writes, net of what the state holds
        outs.append(scale * (q[:, c] * G[:, c].exp()) @ S + Aq[:, c] @ vn)
        glast = G[:, c, -1]                                      # [H, K]
        S = glast.exp()[:, :, None] * S + (k[:, c] * (glast[:, None, :] - G[:, c]).exp()).transpose(-1, -2) @ vn
    o = torch.stack(outs, dim=1).reshape(H, nc * chunk, V)[:, :T].permute(1, 0, 2)
    return o, S, torch.stack(entries)


def chunk_kda_ref(q, k, v, g, beta, scale: Optional[float] = None, initial_state: Optional[torch.Tensor] = None,
                  output_final_state: bool = False, use_qk_l2norm_in_kernel: bool = False,
                  use_gate_in_kernel: bool = False, use_beta_sigmoid_in_kernel: bool = False,
                  allow_neg_eigval: bool = False, cu_seqlens=None, lower_bound: Optional[float] = None,
                  transpose_state_layout: bool = False, A_log: Optional[torch.Tensor] = None,
                  dt_bias: Optional[torch.Tensor] = None, chunk_size: int = 64,
                  compute_dtype: torch.dtype = torch.float32, round_output: bool = True,
                  return_intermediate_states: bool = False):
    """The operator as the reference states it (chunk_kda_naive.py:223-381).  ``compute_dtype`` float64 and
    ``round_output=False`` turn it into a differentiable high-precision version of the same algebra.
    ``return_intermediate_states`` adds a third result, the state at the entry of every chunk, [B, NT, H, K, V]
    ([.., V, K] with the transposed layout) in the input type, packed input: B = 1 and the chunks of all sequences in
    order, as the reference documents it (:287-303, :375-380).  (Its own loop stores them with ``h[:, :, i] = S`` into
    a [B, NT, H, K, V] buffer, :196-203, which only runs where NT == H; the documented meaning is what is stated here.)"""
    B, T, H, K = k.shape
    if allow_neg_eigval and not use_beta_sigmoid_in_kernel:
        raise ValueError("allow_neg_eigval needs use_beta_sigmoid_in_kernel")
    if cu_seqlens is not None and B != 1:
        raise ValueError("packed input needs batch size 1")
    if use_gate_in_kernel and A_log is None:
        raise ValueError("A_log is needed for the in-kernel gate")
    if scale is None:
        scale = K ** -0.5
    in_dtype = q.dtype
    if use_qk_l2norm_in_kernel:
        q, k = _l2norm_rounded(q), _l2norm_rounded(k)
    gl = kda_gate_ref(g, A_log, dt_bias, lower_bound, compute_dtype) if use_gate_in_kernel else g.to(compute_dtype)
    q, k, v, beta = (x.to(compute_dtype) for x in (q, k, v, beta))
    if use_beta_sigmoid_in_kernel:
        beta = torch.sigmoid(beta) * (2.0 if allow_neg_eigval else 1.0)
    h0 = initial_state
    if h0 is not None and transpose_state_layout:
        h0 = h0.transpose(-1, -2)
    V = v.shape[-1]
    o = torch.zeros(B, T, H, V, dtype=compute_dtype)
    pieces = [[] for _ in range(B)]
    finals, entries = [], [[] for _ in range(B)]
    for n, (b, s, e) in enumerate(_seqs(cu_seqlens, B, T)):
        S0 = torch.zeros(H, K, V, dtype=compute_dtype) if h0 is None else h0[n].to(compute_dtype)
        if e > s:
            on, S0, hs = _kda_chunks(q[b, s:e], k[b, s:e], v[b, s:e], gl[b, s:e], beta[b, s:e], scale, S0, chunk_size)
            pieces[b].append((s, e, on))
            entries[b].append(hs)
        finals.append(S0)
    rows = []
    for b in range(B):
        cur, parts = 0, []
        for s, e, on in pieces[b]:
            if s > cur:
                parts.append(o.new_zeros(s - cur, H, V))
            parts.append(on)
            cur = e
        if cur < T:
            parts.append(o.new_zeros(T - cur, H, V))
        rows.append(torch.cat(parts) if parts else o.new_zeros(T, H, V))
    o = torch.stack(rows)
    if round_output:
        o = o.to(in_dtype)
    ht = None
    if output_final_state:
        ht = torch.stack(finals)
        if transpose_state_layout:
            ht = ht.transpose(-1, -2)
    if return_intermediate_states:
        h = torch.stack([torch.cat(e) if e else o.new_zeros(0, H, K, V) for e in entries])
        if transpose_state_layout:
            h = h.transpose(-1, -2)
        return o, ht, (h.to(in_dtype) if round_output else h)
    return o, ht
