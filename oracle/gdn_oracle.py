"""CPU oracle for the Gated DeltaNet operator path.  TEST INFRASTRUCTURE ONLY.

This file is the checker, never the product: only ``tests/``, the smoke entry
and the ``cpu_baseline`` leg of the benchmark may import it.  The shipped ops
live in the HIP library and refuse to run without it.

Everything here is a from-scratch restatement, in plain PyTorch on the CPU, of
the reference's own PyTorch implementation of the gated delta rule (paths are
relative to the reference checkout):

* ``l2norm``                       mindspeed_mm/fsdp/models/qwen3_5/modeling_qwen3_5.py:392-395
* ``chunk_gated_delta_rule_ref``   modeling_qwen3_5.py:398-475 (chunked form)
* ``recurrent_gated_delta_rule_ref`` modeling_qwen3_5.py:478-517 (per-token form)
* ``causal_conv1d_ref``            tests/ut_fsdp/models/qwen3_5/test_causal_conv1d/reference_impl.py:18-59
                                   and the eager branch modeling_qwen3_5.py:803-806
* ``causal_conv1d_final_state_ref`` reference_impl.py:81-102
* ``causal_conv1d_update_ref``     modeling_qwen3_5.py:373-389
* ``pad_and_batch``                tests/ut_fsdp/models/qwen3_5/test_chunk_gated_delta_rule.py:14-28
* ``rms_norm_gated_ref``           Qwen3_5RMSNormGated.forward, modeling_qwen3_5.py:341-349 (the non-NPU branch)
* ``gdn_gates_ref``                g / beta recipe of Qwen3_5GatedDeltaNet.forward, modeling_qwen3_5.py:833-841

The reference functions take neither ``scale``, ``cu_seqlens`` nor grouped
(GQA) q/k heads; the operator entry does
(mindspeed_mm/fsdp/ops/gdn/chunk_gated_delta_rule.py:297-311, and the caller
expands heads at modeling_qwen3_5.py:842-848).  Those three are added here in
the only way consistent with the reference: ``scale`` replaces ``K**-0.5``,
packed sequences are run one by one (equal to the reference test's
pad-and-batch construction), grouped heads are ``repeat_interleave``d.

How each function is pinned (tests/test_oracle_*.py):

* chunked form == independent fp64 textbook recurrence
  (``naive_gated_delta_rule``), closed forms (beta=0, orthonormal keys, T=1,
  overwrite property), chunk-size / zero-padding invariance, state
  continuity, explicit ``(I+A)^-1`` by ``torch.linalg.solve_triangular``;
* backward == autograd through the fp64 recurrence + ``gradcheck``;
* conv1d == ``F.conv1d(groups=D)`` library routine and autograd thereof;
* gated RMSNorm == ``F.rms_norm`` (library routine) times ``F.silu(gate)`` in fp64, the closed form for a constant
  row, scale invariance in x, ``gradcheck``;
* gate recipe == ``torch.special.expit`` / ``torch.logaddexp(x, 0)`` (library routines other than the ones it
  calls) in fp64, closed forms at a + dt_bias = 0 and b = 0, the benchmark input generator's own g, ``gradcheck``;
* committed golden vectors under ``tests/golden`` (made by the fp64
  recurrence) guard against drift.

The reference holds no stored vectors for this path, and its third-party
``fla``/``causal_conv1d`` kernels are absent: parity is defined against the
PyTorch functions cited above, all of which are pinned as listed.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------
# helpers
# --------------------------------------------------------------------------

def l2norm(x: torch.Tensor, dim: int = -1, eps: float = 1e-6) -> torch.Tensor:
    """x * rsqrt(sum(x^2) + eps)  (modeling_qwen3_5.py:392-395)."""
    return x * torch.rsqrt((x * x).sum(dim=dim, keepdim=True) + eps)


def _seq_bounds(cu_seqlens, B: int, T: int):
    """List of (batch index, start, end) per sequence."""
    if cu_seqlens is None:
        return [(b, 0, T) for b in range(B)]
    cu = [int(c) for c in (cu_seqlens.tolist() if torch.is_tensor(cu_seqlens) else cu_seqlens)]
    return [(0, cu[i], cu[i + 1]) for i in range(len(cu) - 1)]


def _expand_heads(x: torch.Tensor, Hv: int) -> torch.Tensor:
    """GQA expansion as the caller does it (modeling_qwen3_5.py:842-848)."""
    H = x.shape[2]
    if H == Hv:
        return x
    assert Hv % H == 0
    return x.repeat_interleave(Hv // H, dim=2)


def pad_and_batch(cu_seqlens: Sequence[int], *inputs: torch.Tensor):
    """Packed [1, T, ...] -> zero padded [N, max_len, ...]
    (test_chunk_gated_delta_rule.py:14-28)."""
    cu = [int(c) for c in cu_seqlens]
    N = len(cu) - 1
    max_len = max(cu[i + 1] - cu[i] for i in range(N))
    outs = [x.new_zeros(N, max_len, *x.shape[2:]) for x in inputs]
    for i in range(N):
        s, e = cu[i], cu[i + 1]
        for o, x in zip(outs, inputs):
            o[i, : e - s] = x[0, s:e]
    return outs


# --------------------------------------------------------------------------
# ground truth: textbook per-token recurrence (independent of the chunk algebra)
# --------------------------------------------------------------------------

def naive_gated_delta_rule(
    q, k, v, g, beta,
    scale: Optional[float] = None,
    initial_state: Optional[torch.Tensor] = None,
    output_final_state: bool = False,
    use_qk_l2norm_in_kernel: bool = False,
    cu_seqlens=None,
    dtype: torch.dtype = torch.float64,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """S <- e^g S;  S <- S + k (beta (v - S^T k))^T;  o = scale * S^T q.

    q,k [B,T,Hqk,K]; v [B,T,Hv,V]; g,beta [B,T,Hv]; state [N,Hv,K,V].
    Differentiable (autograd) in ``dtype``.
    """
    B, T, Hv, V = v.shape
    K = k.shape[-1]
    # The reference normalises before its cast to fp32 (:410-415), i.e. in the input dtype; here the cast comes first,
    # so that a 16-bit input is normalised without an extra rounding (the kernels do the same, in fp32 registers).
    # For fp32 / fp64 inputs, which the oracle tests use, the two orders coincide.
    q, k, v, g, beta = (x.to(dtype) for x in (q, k, v, g, beta))
    if use_qk_l2norm_in_kernel:
        q, k = l2norm(q), l2norm(k)
    q, k = _expand_heads(q, Hv), _expand_heads(k, Hv)
    if scale is None:
        scale = K ** -0.5
    bounds = _seq_bounds(cu_seqlens, B, T)
    o_rows = [[None] * T for _ in range(B)]
    finals = []
    for n, (b, s, e) in enumerate(bounds):
        S = (torch.zeros(Hv, K, V, dtype=dtype) if initial_state is None
             else initial_state[n].to(dtype))
        for t in range(s, e):
            S = S * g[b, t].exp()[:, None, None]
            kv = torch.einsum("hkv,hk->hv", S, k[b, t])
            delta = (v[b, t] - kv) * beta[b, t][:, None]
            S = S + k[b, t][:, :, None] * delta[:, None, :]
            o_rows[b][t] = scale * torch.einsum("hkv,hk->hv", S, q[b, t])
        finals.append(S)
    zero = torch.zeros(Hv, V, dtype=dtype)
    o = torch.stack([torch.stack([r if r is not None else zero for r in rows]) for rows in o_rows])
    ht = torch.stack(finals) if output_final_state else None
    return o, ht


# --------------------------------------------------------------------------
# chunked form, following the reference's torch function line by line in math
# --------------------------------------------------------------------------

def _chunk_one(q, k, v, g, beta, S, chunk_size):
    """One batch of equal-length sequences.  q,k,v head-first [B,H,T,*], q
    pre-scaled; S [B,H,K,V].  Returns (o [B,H,T,V], S)."""
    B, H, T, K = k.shape
    V = v.shape[-1]
    C = chunk_size
    pad = (C - T % C) % C                                    # :419-425
    q = F.pad(q, (0, 0, 0, pad))
    k = F.pad(k, (0, 0, 0, pad))
    v = F.pad(v, (0, 0, 0, pad))
    beta = F.pad(beta, (0, pad))
    g = F.pad(g, (0, pad))
    Tp = T + pad
    v_beta = v * beta[..., None]                             # :429-430
    k_beta = k * beta[..., None]
    q, k, v, k_beta, v_beta = (x.reshape(B, H, Tp // C, C, x.shape[-1]) for x in (q, k, v, k_beta, v_beta))
    g = g.reshape(B, H, Tp // C, C).cumsum(-1)               # :435-439
    diff = g[..., :, None] - g[..., None, :]
    tril0 = torch.ones(C, C, dtype=torch.bool).tril(0)
    tril1 = torch.ones(C, C, dtype=torch.bool).tril(-1)
    # mask before exp: upper-triangle exponents are positive and may overflow (:440)
    decay = torch.where(tril0, diff, torch.zeros_like(diff)).exp() * tril0
    A = -(k_beta @ k.transpose(-1, -2)) * decay * tril1      # :441
    # rows of (I - A)^{-1} by forward substitution (:442-446), built without
    # in-place writes so autograd stays valid
    rows = [A[..., 0, :]]
    for i in range(1, C):
        prev = torch.stack(rows, dim=-2)                     # [.., i, C]
        row = A[..., i, :]
        rows.append(row + (row[..., :i, None] * prev).sum(-2))
    Tm = torch.stack(rows, dim=-2) + torch.eye(C, dtype=A.dtype)
    u = Tm @ v_beta                                          # :447
    w = Tm @ (k_beta * g.exp()[..., None])                   # :448
    outs = []
    for i in range(Tp // C):                                 # :458-468
        q_i, k_i, u_i, w_i, g_i = q[:, :, i], k[:, :, i], u[:, :, i], w[:, :, i], g[:, :, i]
        attn = (q_i @ k_i.transpose(-1, -2)) * decay[:, :, i]
        v_new = u_i - w_i @ S
        outs.append((q_i * g_i.exp()[..., None]) @ S + attn @ v_new)
        S = S * g_i[..., -1, None, None].exp() + \
            (k_i * (g_i[..., -1, None] - g_i).exp()[..., None]).transpose(-1, -2) @ v_new
    o = torch.cat(outs, dim=2)[:, :, :T]
    return o, S


def chunk_gated_delta_rule_ref(
    q, k, v, g, beta,
    scale: Optional[float] = None,
    initial_state: Optional[torch.Tensor] = None,
    output_final_state: bool = False,
    use_qk_l2norm_in_kernel: bool = False,
    cu_seqlens=None,
    chunk_size: int = 64,
    dtype: torch.dtype = torch.float32,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Chunked gated delta rule (modeling_qwen3_5.py:398-475), with ``scale``,
    packed sequences and grouped q/k heads added as described in the module
    docstring.  Returns o [B,T,Hv,V] in ``dtype`` and the state in ``dtype``."""
    B, T, Hv, V = v.shape
    K = k.shape[-1]
    # The reference normalises before its cast to fp32 (:410-415), i.e. in the input dtype; here the cast comes first,
    # so that a 16-bit input is normalised without an extra rounding (the kernels do the same, in fp32 registers).
    # For fp32 / fp64 inputs, which the oracle tests use, the two orders coincide.
    q, k, v, g, beta = (x.to(dtype) for x in (q, k, v, g, beta))
    if use_qk_l2norm_in_kernel:
        q, k = l2norm(q), l2norm(k)
    q, k = _expand_heads(q, Hv), _expand_heads(k, Hv)
    if scale is None:
        scale = K ** -0.5
    q = q * scale
    hf = lambda x: x.transpose(1, 2)                         # :413-415
    if cu_seqlens is None:
        S0 = (torch.zeros(B, Hv, K, V, dtype=dtype) if initial_state is None else initial_state.to(dtype))
        o, S = _chunk_one(hf(q), hf(k), hf(v), hf(g), hf(beta), S0, chunk_size)
        return o.transpose(1, 2), (S if output_final_state else None)
    outs, finals = [], []
    for n, (b, s, e) in enumerate(_seq_bounds(cu_seqlens, B, T)):
        S0 = (torch.zeros(1, Hv, K, V, dtype=dtype) if initial_state is None else initial_state[n:n + 1].to(dtype))
        if e > s:
            sl = lambda x: hf(x[b:b + 1, s:e])
            o, S0 = _chunk_one(sl(q), sl(k), sl(v), sl(g), sl(beta), S0, chunk_size)
            outs.append(o.transpose(1, 2))
        finals.append(S0)
    o = torch.cat(outs, dim=1)
    return o, (torch.cat(finals, 0) if output_final_state else None)


def recurrent_gated_delta_rule_ref(
    q, k, v, g, beta,
    initial_state: Optional[torch.Tensor] = None,
    output_final_state: bool = False,
    use_qk_l2norm_in_kernel: bool = False,
    scale: Optional[float] = None,
    dtype: torch.dtype = torch.float32,
):
    """Per-token decode rule (modeling_qwen3_5.py:478-517): batched over B,
    scale = K**-0.5 unless given, new state tensor returned."""
    B, T, Hv, V = v.shape
    K = k.shape[-1]
    # The reference normalises before its cast to fp32 (:410-415), i.e. in the input dtype; here the cast comes first,
    # so that a 16-bit input is normalised without an extra rounding (the kernels do the same, in fp32 registers).
    # For fp32 / fp64 inputs, which the oracle tests use, the two orders coincide.
    q, k, v, g, beta = (x.to(dtype) for x in (q, k, v, g, beta))
    if use_qk_l2norm_in_kernel:
        q, k = l2norm(q), l2norm(k)
    q, k = _expand_heads(q, Hv), _expand_heads(k, Hv)
    q = q * (K ** -0.5 if scale is None else scale)
    S = torch.zeros(B, Hv, K, V, dtype=dtype) if initial_state is None else initial_state.to(dtype)
    outs = []
    for t in range(T):                                       # :501-512
        S = S * g[:, t].exp()[..., None, None]
        kv = (S * k[:, t][..., None]).sum(-2)
        delta = (v[:, t] - kv) * beta[:, t][..., None]
        S = S + k[:, t][..., None] * delta[..., None, :]
        outs.append((S * q[:, t][..., None]).sum(-2))
    o = torch.stack(outs, dim=1)
    return o, (S if output_final_state else None)


# --------------------------------------------------------------------------
# causal short conv1d
# --------------------------------------------------------------------------

def _act(y, activation):
    if activation in ("silu", "swish"):
        return y * torch.sigmoid(y)
    if activation is None:
        return y
    raise ValueError(f"unknown activation {activation!r}")


def causal_conv1d_ref(
    x, weight, bias=None, residual=None, initial_state=None, activation=None,
    cu_seqlens=None, output_final_state: bool = False, dtype: torch.dtype = torch.float32,
):
    """y[t,d] = act(sum_w xpad[t+w,d] * weight[w,d] + bias[d]) (+ residual).

    x [B,T,D]; weight [W,D]; initial_state [N,D,W] where entry ``j`` is the
    input at step ``j - W`` relative to the sequence start (only j >= 1 is
    read); final_state[n,d,w] = x[T_n - W + w] falling back to the initial
    state / zero for short sequences (reference_impl.py:18-59, 81-102).
    Differentiable in ``dtype``.
    """
    B, T, D = x.shape
    W = weight.shape[0]
    xf, wf = x.to(dtype), weight.to(dtype)
    ys, finals = [], []
    for n, (b, s, e) in enumerate(_seq_bounds(cu_seqlens, B, T)):
        xs = xf[b, s:e]                                      # [Tn, D]
        Tn = e - s
        if initial_state is not None:
            hist = initial_state[n].to(dtype).transpose(0, 1)  # [W, D], row j = step j-W
        else:
            hist = torch.zeros(W, D, dtype=dtype)
        xp = torch.cat([hist, xs], 0)                        # row W+t = x[t]
        y = torch.zeros(Tn, D, dtype=dtype)
        for w in range(W):
            y = y + xp[w + 1: w + 1 + Tn] * wf[w]
        ys.append(y)
        finals.append(xp[Tn: Tn + W].transpose(0, 1))        # [D, W]
    if cu_seqlens is None:
        y = torch.stack(ys, 0)
    else:
        y = torch.cat(ys, 0)[None]
    if bias is not None:
        y = y + bias.to(dtype)
    y = _act(y, activation)
    if residual is not None:
        y = y + residual.to(dtype)
    fs = torch.stack(finals, 0) if output_final_state else None
    return y, fs


def causal_conv1d_update_ref(hidden_states, conv_state, weight, bias=None, activation=None):
    """Decode-time update (modeling_qwen3_5.py:373-389).  hidden_states
    [B,T,D]; conv_state [B,D,S] is rolled IN PLACE; weight [D,W].  Returns
    [B,T,D] in hidden_states.dtype."""
    hs = hidden_states.transpose(1, 2)
    Tn = hs.shape[-1]
    S = conv_state.shape[-1]
    cat = torch.cat([conv_state, hs], dim=-1).to(weight.dtype)
    conv_state.copy_(cat[:, :, -S:])
    out = F.conv1d(cat, weight.unsqueeze(1), bias, padding=0, groups=hs.shape[1])
    out = _act(out[:, :, -Tn:], activation)
    return out.to(hidden_states.dtype).transpose(1, 2).contiguous()


# --------------------------------------------------------------------------
# gated RMSNorm (the step after the gated delta rule in the layer)
# --------------------------------------------------------------------------
def rms_norm_gated_ref(hidden_states: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor,
                       eps: float = 1e-6) -> torch.Tensor:
    """Qwen3_5RMSNormGated.forward (modeling_qwen3_5.py:341-349): normalise in fp32, cast back to the input dtype,
    scale by ``weight``, multiply with ``silu(gate)`` taken in fp32, cast to the input dtype.  Differentiable."""
    input_dtype = hidden_states.dtype
    x = hidden_states.to(torch.float32)
    variance = x.pow(2).mean(-1, keepdim=True)
    x = x * torch.rsqrt(variance + eps)
    x = weight * x.to(input_dtype)
    x = x * F.silu(gate.to(torch.float32))
    return x.to(input_dtype)


def rms_norm_sigmoid_gated_ref(hidden_states: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor,
                               eps: float = 1e-6) -> torch.Tensor:
    """KimiK_3_MoeRMSNormGated.forward, the branch without NPU operators (mindspeed_mm/fsdp/models/kimi_k3/
    modeling_kimi_linear.py:89-94): normalise in fp32, cast back to the input dtype, scale by ``weight``, multiply with
    ``sigmoid(gate)`` taken in fp32 and cast to the input dtype.  The reference leaves the product in the promoted dtype
    of weight and input; the operator returns the input dtype, so does this.  Differentiable."""
    input_dtype = hidden_states.dtype
    x = hidden_states.to(torch.float32)
    variance = x.pow(2).mean(-1, keepdim=True)
    x = x * torch.rsqrt(variance + eps)
    x = weight * x.to(input_dtype)
    x = x * torch.sigmoid(gate.to(torch.float32)).to(input_dtype)
    return x.to(input_dtype)


def gdn_gates_ref(a: torch.Tensor, b: torch.Tensor, A_log: torch.Tensor,
                  dt_bias: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """(g, beta) as Qwen3_5GatedDeltaNet.forward forms them (modeling_qwen3_5.py:833-841, the branch without sequence
    parallelism): ``beta = b.sigmoid()`` in b's dtype, ``g = -A_log.float().exp() * softplus(a.float() + dt_bias)``
    in fp32 (fp64 inputs stay fp64).  Differentiable."""
    beta = b.sigmoid()
    up = torch.float64 if a.dtype == torch.float64 else torch.float32
    g = -A_log.to(up).exp() * F.softplus(a.to(up) + dt_bias)
    return g, beta
