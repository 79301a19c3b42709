"""torch.library registration of the three entry points the layer binds: the chunked gated delta rule (forward and
backward), the fused recurrent decode rule and the causal short convolution (forward, backward, decode update), as
custom operators `torch.ops.mindspeed_mm_amd.*`.

Each operator is a thin call through the C ABI of libgdn_mi355x.so (the same calls the autograd functions of ops.py
make) with a fake implementation (shapes and dtypes only) and, where the reference differentiates, an autograd
formula that calls the backward operator: a traced program (torch.compile, export) carries them as opaque nodes.
Operators take and return tensors only: an absent optional result is an empty tensor of 0 elements, and
`cu_seqlens` is an int64 tensor.  The functions at the end give them the reference's call signatures
(chunk_gated_delta_rule.py:297-311; causal_conv1d.py:100-119; the recurrent slot called at
modeling_qwen3_5.py:877-886) and turn the empty tensors back into None.

The workspace a forward call keeps for its backward pass (the part that depends on the inputs only, see
gdn_chunk_workspace_bytes) is an output of the forward operator, so autograd owns it like any saved tensor.
"""
from typing import Optional, Tuple

import torch
from torch import Tensor

from . import ops as _ops
from ._lib import DTYPE_CODE

NS = "mindspeed_mm_amd"


def _empty(ref, dtype=None):
    return torch.empty(0, dtype=dtype or ref.dtype, device=ref.device)


# ------------------------------------------------------------------ chunk rule
@torch.library.custom_op(f"{NS}::chunk_gated_delta_rule_fwd", mutates_args=())
def chunk_gated_delta_rule_fwd(q: Tensor, k: Tensor, v: Tensor, g: Tensor, beta: Tensor, scale: float,
                               initial_state: Optional[Tensor], output_final_state: bool,
                               cu_seqlens: Optional[Tensor], use_qk_l2norm_in_kernel: bool,
                               for_backward: bool) -> Tuple[Tensor, Tensor, Tensor]:
    """(o, final_state, workspace).  final_state is empty unless asked for; workspace is what a backward call on the
    same inputs can reuse (empty when for_backward is false or the dtype is float32, whose backward pass refills)."""
    gops = _ops._default_ops()
    with torch.cuda.device(q.device):
        o, ht, saved, _ = _ops._chunk_forward_call(gops, q, k, v, g, beta, float(scale), initial_state,
                                                   bool(output_final_state), cu_seqlens, bool(use_qk_l2norm_in_kernel),
                                                   bool(for_backward), False)
    ws = saved[7] if for_backward else None
    return o, (ht if ht is not None else _empty(q, torch.float32)), (ws if ws is not None else _empty(q, torch.uint8))


@chunk_gated_delta_rule_fwd.register_fake
def _(q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, use_qk_l2norm_in_kernel, for_backward):
    B, T, Hqk, K = q.shape
    Hv, V = v.shape[2], v.shape[3]
    N = (cu_seqlens.shape[0] - 1) if cu_seqlens is not None else B
    o = q.new_empty(B, T, Hv, V)
    ht = q.new_empty((N, Hv, K, V) if output_final_state else (0,), dtype=torch.float32)
    nbytes = 0
    if for_backward and q.dtype != torch.float32:
        nbytes = _ops._default_ops().lib.gdn_chunk_workspace_bytes(B, T, N, Hqk, Hv, K, V, DTYPE_CODE[q.dtype], 2)
    return o, ht, q.new_empty(nbytes, dtype=torch.uint8)


@torch.library.custom_op(f"{NS}::chunk_gated_delta_rule_bwd", mutates_args=())
def chunk_gated_delta_rule_bwd(q: Tensor, k: Tensor, v: Tensor, g: Tensor, beta: Tensor, scale: float,
                               initial_state: Optional[Tensor], cu_seqlens: Optional[Tensor],
                               use_qk_l2norm_in_kernel: bool, workspace: Tensor, d_o: Tensor,
                               d_final_state: Optional[Tensor]) -> Tuple[Tensor, Tensor, Tensor, Tensor, Tensor, Tensor]:
    """(dq, dk, dv, dg, dbeta, d initial_state) of chunk_gated_delta_rule_fwd; the last is empty without an initial
    state.  `workspace` is the forward operator's third result (may be empty: the pass then refills one)."""
    gops = _ops._default_ops()
    lib = gops.lib
    B, T, Hqk, K = q.shape
    Hv, V = v.shape[2], v.shape[3]
    N = (cu_seqlens.shape[0] - 1) if cu_seqlens is not None else B
    with torch.cuda.device(q.device):
        (qc, sq), (kc, sk), (vc, sv) = _ops._token_view(q), _ops._token_view(k), _ops._token_view(v)
        bc, bcode = _ops._beta_arg(beta, q.dtype)
        code = DTYPE_CODE[q.dtype]
        ws, nbytes = None, 0
        if workspace.numel():
            nbytes = lib.gdn_chunk_workspace_bytes(B, T, N, Hqk, Hv, K, V, code, 2)
            if workspace.numel() != nbytes:
                raise ValueError(f"workspace of {workspace.numel()} bytes, expected {nbytes}")
            ws = workspace if workspace.data_ptr() % 256 == 0 else _aligned_copy(workspace)
        saved = (qc, kc, vc, gops._f32(g), bc, gops._f32(initial_state), _ops._i64(cu_seqlens, q), ws)
        meta = (B, T, N, Hqk, Hv, K, V, float(scale), int(use_qk_l2norm_in_kernel), code, nbytes, g.dtype, beta.dtype,
                None if initial_state is None else initial_state.dtype, sq, sk, sv, bcode, ws is not None)
        dq, dk, dv, dg, db, dh0 = _ops._chunk_backward_call(gops, saved, meta, d_o, d_final_state)
    return dq, dk, dv, dg, db, (dh0 if dh0 is not None else _empty(q, torch.float32))


def _aligned_copy(t):
    buf = torch.empty(t.numel() + 256, dtype=torch.uint8, device=t.device)
    off = (-buf.data_ptr()) % 256
    out = buf[off:off + t.numel()]
    out.copy_(t)
    return out


@chunk_gated_delta_rule_bwd.register_fake
def _(q, k, v, g, beta, scale, initial_state, cu_seqlens, use_qk_l2norm_in_kernel, workspace, d_o, d_final_state):
    dh0 = q.new_empty(0, dtype=torch.float32) if initial_state is None else torch.empty_like(initial_state)
    return torch.empty_like(q), torch.empty_like(k), torch.empty_like(v), torch.empty_like(g), torch.empty_like(beta), dh0


def _chunk_setup(ctx, inputs, output):
    q, k, v, g, beta, scale, h0, out_final, cu, l2, _ = inputs
    ctx.save_for_backward(q, k, v, g, beta, h0, cu, output[2])
    ctx.scale, ctx.l2, ctx.out_final = scale, l2, out_final


def _chunk_backward(ctx, d_o, d_ht, _d_ws):
    q, k, v, g, beta, h0, cu, ws = ctx.saved_tensors
    dht = d_ht if (ctx.out_final and d_ht is not None) else None
    dq, dk, dv, dg, db, dh0 = torch.ops.mindspeed_mm_amd.chunk_gated_delta_rule_bwd(
        q, k, v, g, beta, ctx.scale, h0, cu, ctx.l2, ws, d_o, dht)
    return dq, dk, dv, dg, db, None, (dh0 if h0 is not None else None), None, None, None, None


chunk_gated_delta_rule_fwd.register_autograd(_chunk_backward, setup_context=_chunk_setup)


# ------------------------------------------------------------------ decode
@torch.library.custom_op(f"{NS}::fused_recurrent_gated_delta_rule", mutates_args=())
def fused_recurrent_gated_delta_rule_op(q: Tensor, k: Tensor, v: Tensor, g: Tensor, beta: Tensor, scale: float,
                                        initial_state: Optional[Tensor], output_final_state: bool,
                                        cu_seqlens: Optional[Tensor],
                                        use_qk_l2norm_in_kernel: bool) -> Tuple[Tensor, Tensor]:
    """(o, final_state); final_state (a new float32 tensor) is empty unless asked for."""
    with torch.cuda.device(q.device):
        o, s = _ops._default_ops().fused_recurrent_gated_delta_rule(
            q, k, v, g, beta, scale=float(scale), initial_state=initial_state, output_final_state=bool(output_final_state),
            cu_seqlens=cu_seqlens, use_qk_l2norm_in_kernel=bool(use_qk_l2norm_in_kernel))
    return o, (s if s is not None else _empty(q, torch.float32))


@fused_recurrent_gated_delta_rule_op.register_fake
def _(q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens, use_qk_l2norm_in_kernel):
    B, _, _, K = q.shape
    Hv, V = v.shape[2], v.shape[3]
    N = (cu_seqlens.shape[0] - 1) if cu_seqlens is not None else B
    return torch.empty_like(v), q.new_empty((N, Hv, K, V) if output_final_state else (0,), dtype=torch.float32)


# ------------------------------------------------------------------ causal short convolution
def _act_name(code: int):
    return "silu" if code else None


@torch.library.custom_op(f"{NS}::causal_conv1d_fwd", mutates_args=())
def causal_conv1d_fwd(x: Tensor, weight: Tensor, bias: Optional[Tensor], residual: Optional[Tensor],
                      initial_state: Optional[Tensor], silu: bool, cu_seqlens: Optional[Tensor],
                      output_final_state: bool) -> Tuple[Tensor, Tensor]:
    """(y, final_state [N,D,W] or empty).  weight [W,D]."""
    with torch.cuda.device(x.device), torch.no_grad():
        y, fs = _ops._CausalConv1d.apply(x, weight, bias, residual, initial_state, _act_name(int(silu)), cu_seqlens,
                                         bool(output_final_state), _ops._default_ops())
    return y, (fs if fs is not None else _empty(x))


@causal_conv1d_fwd.register_fake
def _(x, weight, bias, residual, initial_state, silu, cu_seqlens, output_final_state):
    B, _, D = x.shape
    N = (cu_seqlens.shape[0] - 1) if cu_seqlens is not None else B
    return torch.empty_like(x), x.new_empty((N, D, weight.shape[0]) if output_final_state else (0,))


@torch.library.custom_op(f"{NS}::causal_conv1d_bwd", mutates_args=())
def causal_conv1d_bwd(x: Tensor, weight: Tensor, bias: Optional[Tensor], initial_state: Optional[Tensor], silu: bool,
                      cu_seqlens: Optional[Tensor], dy: Tensor,
                      d_final_state: Optional[Tensor]) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """(dx, dweight, dbias, d initial_state); the last two are empty without a bias / an initial state.  The gradient
    of the residual is dy itself."""
    gops = _ops._default_ops()
    lib = gops.lib
    B, T, D = x.shape
    W = weight.shape[0]
    N = (cu_seqlens.shape[0] - 1) if cu_seqlens is not None else B
    dt = x.dtype
    with torch.cuda.device(x.device):
        xc, wc = x.contiguous(), weight.to(dt).contiguous()
        bc = None if bias is None else bias.to(dt).contiguous()
        h0 = None if initial_state is None else initial_state.to(dt).contiguous()
        cu = _ops._i64(cu_seqlens, x)
        dyc = dy.to(dt).contiguous()
        dfs = None if d_final_state is None else d_final_state.to(dt).contiguous()
        dx = torch.empty_like(xc)
        dw = torch.empty(W, D, dtype=torch.float32, device=x.device)
        db = torch.empty(D, dtype=torch.float32, device=x.device) if bc is not None else None
        dh0 = torch.empty(N, D, W, dtype=dt, device=x.device) if h0 is not None else None
        nbytes = lib.gdn_conv1d_bwd_workspace_bytes(B, T, D, W)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
        p = _ops.ptr
        code = lib.gdn_conv1d_bwd(p(xc), p(dyc), p(wc), p(bc), p(h0), p(dfs), p(cu), p(dx), p(dw), p(db), p(dh0), p(ws),
                                  nbytes, B, T, N, D, W, int(silu), DTYPE_CODE[dt], lib.stream())
        lib.check(code, "gdn_conv1d_bwd")
    return (dx, dw.to(weight.dtype), db.to(bias.dtype) if db is not None else _empty(x),
            dh0.to(initial_state.dtype) if dh0 is not None else _empty(x))


@causal_conv1d_bwd.register_fake
def _(x, weight, bias, initial_state, silu, cu_seqlens, dy, d_final_state):
    return (torch.empty_like(x), torch.empty_like(weight), x.new_empty(0) if bias is None else torch.empty_like(bias),
            x.new_empty(0) if initial_state is None else torch.empty_like(initial_state))


def _conv_setup(ctx, inputs, output):
    x, weight, bias, residual, h0, silu, cu, out_final = inputs
    ctx.save_for_backward(x, weight, bias, h0, cu)
    ctx.silu, ctx.out_final, ctx.res_dtype = silu, out_final, (None if residual is None else residual.dtype)


def _conv_backward(ctx, dy, dfs):
    x, weight, bias, h0, cu = ctx.saved_tensors
    dfs = dfs if ctx.out_final else None
    dx, dw, db, dh0 = torch.ops.mindspeed_mm_amd.causal_conv1d_bwd(x, weight, bias, h0, ctx.silu, cu, dy, dfs)
    return (dx, dw, db if bias is not None else None, dy.to(ctx.res_dtype) if ctx.res_dtype is not None else None,
            dh0 if h0 is not None else None, None, None, None)


causal_conv1d_fwd.register_autograd(_conv_backward, setup_context=_conv_setup)


@torch.library.custom_op(f"{NS}::causal_conv1d_update", mutates_args=("conv_state",))
def causal_conv1d_update_op(x: Tensor, conv_state: Tensor, weight: Tensor, bias: Optional[Tensor], silu: bool) -> Tensor:
    """One decode step per sequence: conv_state [N,D,W] is rolled in place, the result has x's shape."""
    with torch.cuda.device(x.device):
        return _ops._default_ops().causal_conv1d_update(x, conv_state, weight, bias, _act_name(int(silu)))


@causal_conv1d_update_op.register_fake
def _(x, conv_state, weight, bias, silu):
    return torch.empty_like(x)


# ------------------------------------------------------------------ the reference's signatures
def _cu_tensor(cu_seqlens, ref):
    if cu_seqlens is None:
        return None
    return torch.as_tensor(cu_seqlens).to(device=ref.device, dtype=torch.int64)


def chunk_gated_delta_rule(q, k, v, g, beta, scale=None, initial_state=None, output_final_state=False,
                           cu_seqlens=None, use_qk_l2norm_in_kernel=False):
    """chunk_gated_delta_rule (chunk_gated_delta_rule.py:297-311) through the registered operator: (o, final_state)."""
    if scale is None:
        scale = k.shape[-1] ** -0.5
    need = torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in (q, k, v, g, beta, initial_state))
    o, ht, _ = torch.ops.mindspeed_mm_amd.chunk_gated_delta_rule_fwd(
        q, k, v, g, beta, float(scale), initial_state, bool(output_final_state), _cu_tensor(cu_seqlens, q),
        bool(use_qk_l2norm_in_kernel), bool(need))
    return o, (ht if output_final_state else None)


def fused_recurrent_gated_delta_rule(q, k, v, g, beta=None, scale=None, initial_state=None, output_final_state=False,
                                     cu_seqlens=None, use_qk_l2norm_in_kernel=False):
    """The decode slot (called at modeling_qwen3_5.py:877-886) through the registered operator: (o, final_state)."""
    if scale is None:
        scale = k.shape[-1] ** -0.5
    if beta is None:
        beta = torch.ones(v.shape[:3], dtype=torch.float32, device=q.device)
    o, s = torch.ops.mindspeed_mm_amd.fused_recurrent_gated_delta_rule(
        q, k, v, g, beta, float(scale), initial_state, bool(output_final_state), _cu_tensor(cu_seqlens, q),
        bool(use_qk_l2norm_in_kernel))
    return o, (s if output_final_state else None)


def causal_conv1d(x, weight, bias=None, residual=None, initial_state=None, activation=None, cu_seqlens=None,
                  output_final_state=False):
    """causal_conv1d (models/qwen3_5/causal_conv1d.py:100-119) through the registered operator: (y, final_state)."""
    y, fs = torch.ops.mindspeed_mm_amd.causal_conv1d_fwd(x, weight, bias, residual, initial_state,
                                                         bool(_ops._act_code(activation)), _cu_tensor(cu_seqlens, x),
                                                         bool(output_final_state))
    return y, (fs if output_final_state else None)


def causal_conv1d_update(x, conv_state, weight, bias=None, activation=None):
    """The decode update of the convolution (modeling_qwen3_5.py:373-389) through the registered operator."""
    return torch.ops.mindspeed_mm_amd.causal_conv1d_update(x, conv_state, weight, bias, bool(_ops._act_code(activation)))
