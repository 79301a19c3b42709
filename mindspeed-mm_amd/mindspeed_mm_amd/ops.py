"""Python entry points of the Gated DeltaNet operator path, with the reference's signatures.

    chunk_gated_delta_rule            mindspeed_mm/fsdp/ops/gdn/chunk_gated_delta_rule.py:296-443
    fused_recurrent_gated_delta_rule  call site mindspeed_mm/fsdp/models/qwen3_5/modeling_qwen3_5.py:877-886
                                      (semantics of torch_recurrent_gated_delta_rule, :478-517)
    causal_conv1d                     mindspeed_mm/fsdp/models/qwen3_5/causal_conv1d.py:100-119
    causal_conv1d_update              modeling_qwen3_5.py:373-389, called at :738-744
    rms_norm_gated / RMSNormGated     Qwen3_5RMSNormGated, modeling_qwen3_5.py:330-349, called at :897-900
    gdn_gates                         g / beta recipe of the layer, modeling_qwen3_5.py:833-841
    chunk_gated_delta_rule_qkv        the rule on the unsplit convolution output (split at :818-831)
    chunk_kda                         mindspeed_mm/fsdp/ops/kda/triton_ascend/chunk.py:215-407 (the fused operator),
                                      mindspeed_mm/fsdp/ops/kda/chunk_kda_naive.py:223-381 (its pure-PyTorch statement)
    fused_recurrent_gated_delta_rule_qkv / decode_step / GdnDecodeCache
                                      the layer's decode branch (:738-744, :808-848, :877-890) and the
                                      linear-attention part of Qwen3_5DynamicCache (:134-221)

Everything here is host glue: validation, output/workspace allocation with torch, and one call into the
C ABI per operator.  The kernels themselves are the HIP library; nothing in this file computes.
"""
import functools
import os
import warnings
from typing import Optional

import torch

from ._lib import DTYPE_CODE, GdnLibrary, default_library, ptr


def _input_guard(fn):
    """Runs an autograd function's forward / backward with the device of its first tensor argument current, as the
    reference's input_guard does (mindspeed_mm/fsdp/ops/gdn/triton/utils.py:210-239): the backward pass is called
    from the autograd engine's thread, where another device may be current."""
    @functools.wraps(fn)
    def wrapper(ctx, *args):
        dev = next((a.device for a in args if isinstance(a, torch.Tensor)), None)
        if dev is not None and dev.type == "cuda":
            with torch.cuda.device(dev):
                return fn(ctx, *args)
        return fn(ctx, *args)
    return wrapper


# forward and backward keep the autocast state of the forward call (triton/utils.py:194-197)
_custom_fwd = functools.partial(torch.amp.custom_fwd, device_type="cuda")
_custom_bwd = functools.partial(torch.amp.custom_bwd, device_type="cuda")


def _out_grad(grad, like):
    """The gradient of the main output, for autograd functions that ask for undefined gradients to stay None (the final
    state is rarely used: its zero gradient is then neither filled nor read): zeros only when the output itself went
    unused while the final state was used.  `like` = (shape, dtype, device) of that output."""
    if grad is not None:
        return grad.contiguous()
    return torch.zeros(like[0], dtype=like[1], device=like[2])


def _beta_arg(beta, act_dtype):
    """beta as handed to the kernels: in place when it has the 16-bit dtype of q, k, v (the layer's beta = b.sigmoid()
    is bf16, modeling_qwen3_5.py:833), else as float32.  Returns (tensor, dtype code)."""
    if beta.dtype == act_dtype and act_dtype == torch.bfloat16:
        return beta.detach().contiguous(), 1
    return beta.detach().to(torch.float32).contiguous(), 0


def _check_packed_length(cu_seqlens, tokens):
    """cu_seqlens must start at 0, not decrease and stay within the packed tokens; rows past cu_seqlens[-1] (a padded
    batch) are cleared by the kernels.  Checked where it costs no device synchronisation (lists and host tensors); a
    device tensor must satisfy it too."""
    if cu_seqlens is None:
        return
    if isinstance(cu_seqlens, torch.Tensor):
        if cu_seqlens.device.type != "cpu" or cu_seqlens.numel() == 0:
            return
        cu = [int(c) for c in cu_seqlens.tolist()]
    else:
        cu = [int(c) for c in cu_seqlens]
    if cu[0] != 0 or cu[-1] > tokens or any(b < a for a, b in zip(cu[:-1], cu[1:])):
        raise ValueError(f"cu_seqlens must start at 0, not decrease and end at or before the number of packed tokens "
                         f"({tokens}), got {cu[0]} ... {cu[-1]}")


def _act_code(activation):
    if activation in ("silu", "swish"):
        return 1
    if activation is None:
        return 0
    raise ValueError(f"unsupported activation {activation!r} (None, 'silu' or 'swish')")


class GdnOps:
    """The operators bound to one loaded kernel library."""

    def __init__(self, lib: GdnLibrary):
        self.lib = lib
        self._helpers = {}
        # False: the backward pass of the chunked rule runs its two recurrences one after the other on the caller's stream
        self.two_stream_backward = os.environ.get("GDN_TWO_STREAM_BACKWARD", "1") != "0"

    def helper_stream(self, device):
        """A second stream on `device` (default priority, made once) for work that may run beside the caller's stream;
        None where there are no streams (the host build of the kernels) or two_stream_backward is off."""
        if self.lib.device_type != "cuda" or not self.two_stream_backward:
            return None
        key = torch.device(device).index
        if key is None:
            key = torch.cuda.current_device()
        if key not in self._helpers:
            self._helpers[key] = torch.cuda.Stream(device=key)
        return self._helpers[key]

    # ------------------------------------------------------------------ helpers
    def _need(self, *tensors):
        for t in tensors:
            if not isinstance(t, torch.Tensor):   # None, or cu_seqlens given as a list
                continue
            if t.device.type != self.lib.device_type:
                raise RuntimeError(
                    f"tensor on {t.device}; these operators run only on {self.lib.device_type} tensors "
                    "(there is no host fallback)")

    @staticmethod
    def _f32(t):
        return None if t is None else t.detach().to(torch.float32).contiguous()

    @staticmethod
    def _no_grad_views(*tensors):
        """Under torch.no_grad() a tensor still reports requires_grad, and an autograd function would take that as a
        backward pass to prepare for (extra operands written by the forward kernels): hand it detached views then."""
        if torch.is_grad_enabled():
            return tensors
        return tuple(None if t is None else t.detach() for t in tensors)

    # ------------------------------------------------------------------ chunked rule
    def chunk_gated_delta_rule(self, q, k, v, g, beta, scale=None, initial_state=None, output_final_state=False,
                               use_qk_l2norm_in_kernel=False, cu_seqlens=None, chunk_size=64, head_first=False,
                               skip_recompute=False):
        scale = self._check_chunk_args(q, k, v, g, beta, scale, initial_state, cu_seqlens, chunk_size, head_first)
        if q.dtype == torch.float16:
            # float16 (which the reference's entry accepts, chunk_gated_delta_rule.py:379-386) runs on the float32
            # kernels: q, k, v are widened, o comes back in float16, and autograd carries the casts
            o, ht = self.chunk_gated_delta_rule(q.float(), k.float(), v.float(), g, beta, scale, initial_state,
                                                output_final_state, use_qk_l2norm_in_kernel, cu_seqlens, chunk_size,
                                                False, skip_recompute)
            return o.to(torch.float16), ht
        q, k, v, g, beta, initial_state = self._no_grad_views(q, k, v, g, beta, initial_state)
        return _ChunkGatedDeltaRule.apply(q, k, v, g, beta, float(scale), initial_state, bool(output_final_state),
                                          cu_seqlens, bool(use_qk_l2norm_in_kernel), bool(skip_recompute), self)

    def chunk_gated_delta_rule_norm(self, q, k, v, g, beta, gate, norm_weight, eps=1e-6, scale=None,
                                    initial_state=None, output_final_state=False, use_qk_l2norm_in_kernel=False,
                                    cu_seqlens=None, in_output_kernel=False, skip_recompute=False):
        """The rule followed by the layer's gated RMSNorm over head_v_dim (modeling_qwen3_5.py:886-900:
        `core_attn_out = self.norm(core_attn_out.reshape(-1, head_v_dim), z.reshape(-1, head_v_dim))`).
        Returns (y [B,T,Hv,V], final_state).  By default the two operators run in sequence (the rule's output comes
        from the recurrence kernel itself, which is the faster arrangement); with in_output_kernel=True the stand-alone
        output kernel forms it from the stored per-chunk states and normalises and gates the rows before they leave
        (one launch less, head_v_dim 64 or 128).  Both give the same bits."""
        if not in_output_kernel:
            o, ht = self.chunk_gated_delta_rule(q, k, v, g, beta, scale, initial_state, output_final_state,
                                                use_qk_l2norm_in_kernel, cu_seqlens, skip_recompute=skip_recompute)
            V = v.shape[-1]
            y = self.rms_norm_gated(o.reshape(-1, V), gate.reshape(-1, V).to(o.dtype), norm_weight, eps)
            return y.view(o.shape), ht
        scale = self._check_chunk_args(q, k, v, g, beta, scale, initial_state, cu_seqlens, 64, False)
        V = v.shape[-1]
        if V not in (64, 128):
            raise ValueError(f"the fused norm needs head_v_dim 64 or 128, got {V}; use the two operators in sequence")
        if gate.numel() != v.numel():
            raise ValueError(f"gate has {gate.numel()} elements, expected {v.numel()} (one per element of v)")
        if tuple(norm_weight.shape) != (V,):
            raise ValueError(f"norm_weight shape {tuple(norm_weight.shape)}, expected ({V},)")
        self._need(gate, norm_weight)
        q, k, v, g, beta, gate, norm_weight, initial_state = self._no_grad_views(q, k, v, g, beta, gate, norm_weight,
                                                                                 initial_state)
        return _ChunkGatedDeltaRuleNorm.apply(q, k, v, g, beta, gate, norm_weight, float(eps), float(scale),
                                              initial_state, bool(output_final_state), cu_seqlens,
                                              bool(use_qk_l2norm_in_kernel), self)

    def _check_chunk_args(self, q, k, v, g, beta, scale, initial_state, cu_seqlens, chunk_size, head_first):
        """Argument checks of chunk_gated_delta_rule (chunk_gated_delta_rule.py:379-414); returns the scale."""
        if q.dtype != k.dtype or k.dtype != v.dtype:
            raise ValueError(
                f"q current type is {q.dtype} , k current type is {k.dtype} ,v current type is {v.dtype} , "
                "they should are equal")
        if q.dtype not in (torch.float32, torch.bfloat16, torch.float16):
            raise ValueError(f"chunk_gated_delta_rule supports bfloat16, float16 and float32, got {q.dtype}")
        if len(beta.shape) != 3:
            raise ValueError(
                f"beta current shape len is {len(beta.shape)}, beta must be of shape [B, T, H] if head_first=False, "
                "or [B, H, T] otherwise.")
        if head_first:   # as the reference: a warning, and the tensors are taken as [B, T, H, ...] all the same
            warnings.warn(
                "head_first is deprecated and will be removed in a future version. "
                "Please use head_first=False for now instead.")
        if chunk_size != 64:
            raise ValueError("only chunk_size=64 is supported")
        if not head_first and q.shape[1] < q.shape[2]:
            warnings.warn(
                f"Input tensor shape suggests potential format mismatch: seq_len ({q.shape[1]}) < num_heads "
                f"({q.shape[2]}). Please verify your input tensor format matches the expected shape [B, T, H, ...].")
        if cu_seqlens is not None:
            if q.shape[0] != 1:
                raise ValueError(
                    f"The batch size is expected to be 1 rather than {q.shape[0]} when using `cu_seqlens`."
                    f"Please flatten variable-length inputs before processing.")
            if initial_state is not None and initial_state.shape[0] != len(cu_seqlens) - 1:
                raise ValueError(
                    f"The number of initial states is expected to be equal to the number of input sequences, "
                    f"i.e., {len(cu_seqlens) - 1} rather than {initial_state.shape[0]}.")
        if v.shape[2] % q.shape[2] != 0 or k.shape != q.shape or g.shape != beta.shape or \
                tuple(g.shape) != tuple(v.shape[:3]):
            raise ValueError("expected q,k [B,T,Hqk,K], v [B,T,Hv,V], g,beta [B,T,Hv] with Hv % Hqk == 0")
        if scale is None:
            scale = k.shape[-1] ** -0.5
        _check_packed_length(cu_seqlens, q.shape[1])
        self._need(q, k, v, g, beta, initial_state, cu_seqlens if isinstance(cu_seqlens, torch.Tensor) and
                   cu_seqlens.device.type != "cpu" else None)
        return scale

    def chunk_gated_delta_rule_qkv(self, mixed_qkv, g, beta, num_k_heads, num_v_heads, head_k_dim, head_v_dim,
                                   scale=None, initial_state=None, output_final_state=False,
                                   use_qk_l2norm_in_kernel=False, cu_seqlens=None, gate=None, norm_weight=None,
                                   norm_eps=1e-6):
        """chunk_gated_delta_rule on the unsplit [B,T,2 Hqk K + Hv V] output of the convolution: equal to splitting it
        into q, k, v as modeling_qwen3_5.py:818-831 does and calling chunk_gated_delta_rule, without the copies.
        With gate (the layer's z) and norm_weight the gated RMSNorm of modeling_qwen3_5.py:897-900 follows."""
        if (gate is None) != (norm_weight is None):
            raise ValueError("gate and norm_weight go together")
        if mixed_qkv.dim() != 3 or mixed_qkv.shape[-1] < 2 * num_k_heads * head_k_dim + num_v_heads * head_v_dim:
            raise ValueError("expected mixed_qkv [B, T, D] with D >= 2 * num_k_heads * head_k_dim + num_v_heads * head_v_dim")
        if mixed_qkv.dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"chunk_gated_delta_rule supports bfloat16 and float32, got {mixed_qkv.dtype}")
        if len(beta.shape) != 3 or g.shape != beta.shape or \
                tuple(g.shape) != (mixed_qkv.shape[0], mixed_qkv.shape[1], num_v_heads) or num_v_heads % num_k_heads:
            raise ValueError("expected g, beta [B, T, Hv] with Hv % Hqk == 0")
        if cu_seqlens is not None:
            if mixed_qkv.shape[0] != 1:
                raise ValueError(
                    f"The batch size is expected to be 1 rather than {mixed_qkv.shape[0]} when using `cu_seqlens`."
                    f"Please flatten variable-length inputs before processing.")
            if initial_state is not None and initial_state.shape[0] != len(cu_seqlens) - 1:
                raise ValueError(
                    f"The number of initial states is expected to be equal to the number of input sequences, "
                    f"i.e., {len(cu_seqlens) - 1} rather than {initial_state.shape[0]}.")
        if scale is None:
            scale = head_k_dim ** -0.5
        _check_packed_length(cu_seqlens, mixed_qkv.shape[1])
        self._need(mixed_qkv, g, beta, initial_state, cu_seqlens if isinstance(cu_seqlens, torch.Tensor) and
                   cu_seqlens.device.type != "cpu" else None)
        mixed_qkv, g, beta, initial_state = self._no_grad_views(mixed_qkv, g, beta, initial_state)
        o, ht = _ChunkGatedDeltaRuleQKV.apply(mixed_qkv, g, beta, int(num_k_heads), int(num_v_heads), int(head_k_dim),
                                              int(head_v_dim), float(scale), initial_state, bool(output_final_state),
                                              cu_seqlens, bool(use_qk_l2norm_in_kernel), self)
        if gate is None:
            return o, ht
        y = self.rms_norm_gated(o.reshape(-1, head_v_dim), gate.reshape(-1, head_v_dim).to(o.dtype), norm_weight,
                                norm_eps)
        return y.view(o.shape), ht

    # ------------------------------------------------------------------ KDA
    def chunk_kda(self, q, k, v, g, beta, scale=None, initial_state=None, output_final_state=False,
                  use_qk_l2norm_in_kernel=False, use_gate_in_kernel=False, use_beta_sigmoid_in_kernel=False,
                  allow_neg_eigval=False, cu_seqlens=None, cu_seqlens_cpu=None, safe_gate=False, lower_bound=None,
                  disable_recompute=False, return_intermediate_states=False, transpose_state_layout=False,
                  skip_recompute=False, chunk_size=64, **kwargs):
        """Kimi delta attention, chunked: the delta rule with one decay per key channel.  Signature and argument
        checks of chunk_kda (triton_ascend/chunk.py:215-407) and chunk_kda_naive (chunk_kda_naive.py:223-381):
        q, k, g [B,T,H,K], v [B,T,H,V], beta [B,T,H]; A_log [H] and dt_bias [H*K] come as keyword arguments when
        use_gate_in_kernel is set.  safe_gate, disable_recompute, skip_recompute and cu_seqlens_cpu are hints of the
        reference's kernels without effect on the result and are accepted and ignored.
        return_intermediate_states=True adds a third result: the state at the entry of every chunk of 64 tokens,
        [B, NT, H, K, V] ([B, NT, H, V, K] with transpose_state_layout) in the dtype of q; packed input: B = 1 and NT
        counts the chunks of all sequences (chunk_kda_naive.py:287-303).  It carries no gradient."""
        A_log, dt_bias = kwargs.get("A_log"), kwargs.get("dt_bias")
        if use_gate_in_kernel and A_log is None:
            raise ValueError("A_log must be provided when use_gate_in_kernel=True.")
        if allow_neg_eigval and not use_beta_sigmoid_in_kernel:
            raise ValueError("`allow_neg_eigval=True` requires `use_beta_sigmoid_in_kernel=True`.")
        if not (q.shape == k.shape == g.shape):
            raise ValueError("q, k, g must have the same shape.")
        if beta.shape != q.shape[:3]:
            raise ValueError("beta must be of shape (batch size, seq len, num of head).")
        if tuple(v.shape[:3]) != tuple(q.shape[:3]) or v.dim() != 4:
            raise ValueError("v must be of shape (batch size, seq len, num of head, head dim).")
        if q.dtype != k.dtype or k.dtype != v.dtype or q.dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"chunk_kda supports bfloat16 and float32 q, k, v of one dtype, got {q.dtype}, {k.dtype}, {v.dtype}")
        if chunk_size != 64:
            raise ValueError("only chunk_size=64 is supported")
        if safe_gate and use_gate_in_kernel:   # triton_ascend/chunk.py:373-377
            if lower_bound is None:
                raise ValueError("`lower_bound` must be specified when `safe_gate=True` and `use_gate_in_kernel=True`.")
            if not (-5 <= lower_bound < 0):
                raise ValueError(f"`lower_bound` must be in the safe range [-5, 0), got {lower_bound}.")
        N = q.shape[0]
        if cu_seqlens is not None:
            if q.shape[0] != 1:
                raise ValueError(
                    f"The batch size is expected to be 1 rather than {q.shape[0]} when using `cu_seqlens`."
                    f"Please flatten variable-length inputs before processing.")
            N = len(cu_seqlens) - 1
            if initial_state is not None and initial_state.shape[0] != N:
                raise ValueError(
                    f"The number of initial states is expected to be equal to the number of input sequences, "
                    f"i.e., {N} rather than {initial_state.shape[0]}.")
        if initial_state is not None and initial_state.dtype != torch.float32:
            raise ValueError("initial_state must be in float32.")
        if scale is None:
            scale = k.shape[-1] ** -0.5
        _check_packed_length(cu_seqlens, q.shape[1])
        self._need(q, k, v, g, beta, initial_state, A_log, dt_bias)
        q, k, v, g, beta, initial_state, A_log, dt_bias = self._no_grad_views(q, k, v, g, beta, initial_state, A_log, dt_bias)
        if transpose_state_layout and initial_state is not None:
            initial_state = initial_state.transpose(-1, -2)
        o, ht, hs = _ChunkKda.apply(q, k, v, g, beta, A_log, dt_bias, float(scale), initial_state,
                                    bool(output_final_state), bool(use_qk_l2norm_in_kernel), bool(use_gate_in_kernel),
                                    bool(use_beta_sigmoid_in_kernel), bool(allow_neg_eigval), cu_seqlens, lower_bound,
                                    bool(return_intermediate_states), bool(transpose_state_layout), self)
        if ht is not None and transpose_state_layout:
            ht = ht.transpose(-1, -2)
        if return_intermediate_states:
            return o, ht, hs
        return o, ht

    def gdn_gates(self, a, b, A_log, dt_bias):
        """(g, beta) of the layer from its projections a, b [..., Hv] and parameters A_log, dt_bias [Hv]:
        beta = b.sigmoid(), g = -A_log.float().exp() * softplus(a.float() + dt_bias) (modeling_qwen3_5.py:833-841)."""
        if a.shape != b.shape or a.dtype != b.dtype or A_log.shape != (a.shape[-1],) or dt_bias.shape != A_log.shape:
            raise ValueError("expected a, b [..., Hv] of one dtype and A_log, dt_bias [Hv]")
        if a.dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"gdn_gates supports bfloat16 and float32, got {a.dtype}")
        self._need(a, b, A_log, dt_bias)
        return _GdnGates.apply(a, b, A_log, dt_bias, self)

    # ------------------------------------------------------------------ decode
    def fused_recurrent_gated_delta_rule(self, q, k, v, g, beta=None, scale=None, initial_state=None,
                                         output_final_state=False, cu_seqlens=None, use_qk_l2norm_in_kernel=False,
                                         inplace_state=False):
        """One or more decode tokens per sequence.  Returns (o, final_state); final_state is a new fp32 tensor
        unless inplace_state=True, in which case initial_state (fp32, contiguous) is updated and returned.
        cu_seqlens (list or int64 tensor [N+1]): the batch is one row of packed sequences, each run from its own
        state [N,Hv,K,V], as at the chunk entry (chunk_gated_delta_rule.py:297-311, :398-411)."""
        if q.dtype != k.dtype or k.dtype != v.dtype or q.dtype not in (torch.float32, torch.bfloat16):
            raise ValueError("q, k, v must share a dtype, bfloat16 or float32")
        B, T, Hqk, K = q.shape
        Hv, V = v.shape[2], v.shape[3]
        N = B
        if cu_seqlens is not None:
            if B != 1:
                raise ValueError(
                    f"The batch size is expected to be 1 rather than {B} when using `cu_seqlens`."
                    f"Please flatten variable-length inputs before processing.")
            N = len(cu_seqlens) - 1
            if initial_state is not None and initial_state.shape[0] != N:
                raise ValueError(
                    f"The number of initial states is expected to be equal to the number of input sequences, "
                    f"i.e., {N} rather than {initial_state.shape[0]}.")
            _check_packed_length(cu_seqlens, T)
        if beta is None:
            beta = torch.ones(B, T, Hv, dtype=torch.float32, device=q.device)
        self._need(q, k, v, g, beta, initial_state)
        if scale is None:
            scale = K ** -0.5
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        # rows outside every listed sequence (a padded packed batch) are not visited by the kernel
        o = torch.zeros_like(v) if cu_seqlens is not None else torch.empty_like(v)
        s_in = None
        if initial_state is not None:
            if inplace_state:
                if initial_state.dtype != torch.float32 or not initial_state.is_contiguous():
                    raise ValueError("inplace_state needs a contiguous float32 state")
                s_in = initial_state
            else:
                s_in = self._f32(initial_state)
        s_out = None
        if output_final_state or inplace_state:
            s_out = s_in if (inplace_state and s_in is not None) else \
                torch.empty(N, Hv, K, V, dtype=torch.float32, device=q.device)
        g32, b32 = self._f32(g), self._f32(beta)   # named: temporaries must outlive the launch
        if cu_seqlens is not None:
            cu = _i64(cu_seqlens, q)
            code = self.lib.gdn_recurrent_fwd_packed(ptr(q), ptr(k), ptr(v), ptr(g32), ptr(b32), ptr(s_in), ptr(s_out),
                                                     ptr(o), ptr(cu), N, T, Hqk, Hv, K, V, float(scale),
                                                     int(use_qk_l2norm_in_kernel), DTYPE_CODE[q.dtype], self.lib.stream())
            self.lib.check(code, "gdn_recurrent_fwd_packed")
            return o, (s_out if output_final_state else None)
        code = self.lib.gdn_recurrent_fwd(ptr(q), ptr(k), ptr(v), ptr(g32), ptr(b32), ptr(s_in),
                                          ptr(s_out), ptr(o), B, T, Hqk, Hv, K, V, float(scale),
                                          int(use_qk_l2norm_in_kernel), DTYPE_CODE[q.dtype], self.lib.stream())
        self.lib.check(code, "gdn_recurrent_fwd")
        return o, (s_out if output_final_state else None)

    def fused_recurrent_gated_delta_rule_qkv(self, mixed_qkv, a, b, A_log, dt_bias, num_k_heads, num_v_heads,
                                             head_k_dim, head_v_dim, scale=None, initial_state=None,
                                             output_final_state=False, use_qk_l2norm_in_kernel=False,
                                             inplace_state=False):
        """fused_recurrent_gated_delta_rule on the convolution's unsplit output [B,T,D] with the gates formed in the
        kernel from the projections a, b [B,T,Hv] and the parameters A_log, dt_bias [Hv]: equal to the layer's chain
        split -> sigmoid / softplus recipe -> rule (modeling_qwen3_5.py:808-848, 877-886) without its copies."""
        Hqk, Hv, K, V = int(num_k_heads), int(num_v_heads), int(head_k_dim), int(head_v_dim)
        if mixed_qkv.dim() != 3 or mixed_qkv.shape[-1] < 2 * Hqk * K + Hv * V:
            raise ValueError("expected mixed_qkv [B, T, D] with D >= 2 * num_k_heads * head_k_dim + num_v_heads * head_v_dim")
        B, T, D = mixed_qkv.shape
        dt = mixed_qkv.dtype
        if dt not in (torch.float32, torch.bfloat16) or a.dtype != dt or b.dtype != dt:
            raise ValueError("mixed_qkv, a, b must share a dtype, bfloat16 or float32")
        if tuple(a.shape) != (B, T, Hv) or a.shape != b.shape or A_log.shape != (Hv,) or dt_bias.shape != (Hv,):
            raise ValueError("expected a, b [B, T, Hv] and A_log, dt_bias [Hv]")
        self._need(mixed_qkv, a, b, A_log, dt_bias, initial_state)
        if scale is None:
            scale = K ** -0.5
        vec = 16 // mixed_qkv.element_size()
        x = mixed_qkv if (mixed_qkv.is_contiguous() and D % vec == 0 and mixed_qkv.data_ptr() % 16 == 0) \
            else mixed_qkv.contiguous()
        if D % vec != 0:
            raise ValueError(f"the width of mixed_qkv must be a multiple of {vec} elements")
        pdt = dt if (A_log.dtype == dt and dt_bias.dtype == dt) else torch.float32
        Ac, dc = A_log.detach().to(pdt).contiguous(), dt_bias.detach().to(pdt).contiguous()
        ac, bc = a.contiguous(), b.contiguous()
        o = torch.empty(B, T, Hv, V, dtype=dt, device=x.device)
        s_in = None
        if initial_state is not None:
            if inplace_state:
                if initial_state.dtype != torch.float32 or not initial_state.is_contiguous():
                    raise ValueError("inplace_state needs a contiguous float32 state")
                s_in = initial_state
            else:
                s_in = self._f32(initial_state)
        s_out = None
        if output_final_state or inplace_state:
            s_out = s_in if (inplace_state and s_in is not None) else \
                torch.empty(B, Hv, K, V, dtype=torch.float32, device=x.device)
        code = self.lib.gdn_recurrent_fwd_qkv(ptr(x), D, ptr(ac), ptr(bc), ptr(Ac), ptr(dc), ptr(s_in), ptr(s_out),
                                              ptr(o), B, T, Hqk, Hv, K, V, float(scale),
                                              int(use_qk_l2norm_in_kernel), DTYPE_CODE[dt], DTYPE_CODE[pdt],
                                              self.lib.stream())
        self.lib.check(code, "gdn_recurrent_fwd_qkv")
        return o, (s_out if output_final_state else None)

    def decode_step(self, mixed_qkv, a, b, conv_state, recurrent_state, conv_weight, conv_bias, A_log, dt_bias,
                    num_k_heads, num_v_heads, head_k_dim, head_v_dim, activation="silu"):
        """The decode branch of Qwen3_5GatedDeltaNet.forward between the input projections and the gated norm
        (modeling_qwen3_5.py:738-744, 808-848, 877-890) in two launches: convolution update (conv_state [B,D,S] rolled
        in place), then the rule on its unsplit output with the gates formed in the kernel (recurrent_state
        [B,Hv,K,V] fp32 updated in place).  mixed_qkv [B,T,D], a, b [B,T,Hv]; conv_weight [D,W].  Returns o [B,T,Hv,V]."""
        y = self.causal_conv1d_update(mixed_qkv, conv_state, conv_weight, conv_bias, activation)
        o, _ = self.fused_recurrent_gated_delta_rule_qkv(y, a, b, A_log, dt_bias, num_k_heads, num_v_heads, head_k_dim,
                                                         head_v_dim, initial_state=recurrent_state,
                                                         use_qk_l2norm_in_kernel=True, inplace_state=True)
        return o

    # ------------------------------------------------------------------ conv1d
    def causal_conv1d(self, x, weight, bias=None, residual=None, initial_state=None, activation=None,
                      cu_seqlens=None, output_final_state=False):
        if x.shape[-1] != weight.shape[-1]:
            raise ValueError("x [B, T, D], weight [W, D], please check.")
        if cu_seqlens is not None and x.shape[0] != 1:
            raise ValueError("cu_seqlens needs batch size 1 (packed input)")
        _act_code(activation)
        self._need(x, weight, bias, residual, initial_state)   # cu_seqlens: a list or a tensor on any device
        return _CausalConv1d.apply(x, weight, bias, residual, initial_state, activation, cu_seqlens,
                                   bool(output_final_state), self)

    def causal_conv1d_update(self, hidden_states, conv_state, weight, bias=None, activation=None):
        """hidden_states [B,T,D]; conv_state [B,D,S] updated in place; weight [D,W]."""
        self._need(hidden_states, conv_state, weight, bias)
        B, T, D = hidden_states.shape
        W, S = weight.shape[1], conv_state.shape[-1]
        dt = hidden_states.dtype
        if not conv_state.is_contiguous():
            raise ValueError("conv_state must be contiguous (it is updated in place)")
        x = hidden_states.contiguous()
        state = conv_state if conv_state.dtype == dt else conv_state.to(dt)
        out = torch.empty_like(x)
        wc = weight.to(dt).contiguous()
        bc = None if bias is None else bias.to(dt).contiguous()
        code = self.lib.gdn_conv1d_update(ptr(x), ptr(state), ptr(wc), ptr(bc), ptr(out), B, T, D,
                                          W, S, _act_code(activation), DTYPE_CODE[dt], self.lib.stream())
        self.lib.check(code, "gdn_conv1d_update")
        if state is not conv_state:
            conv_state.copy_(state)
        return out

    # ------------------------------------------------------------------ gated RMSNorm
    def rms_norm_gated(self, hidden_states, gate, weight, eps=1e-6, activation="silu"):
        if gate is None:
            raise ValueError("rms_norm_gated needs a gate (the reference layer always passes one)")
        if activation not in _GATE_ACTIVATION:
            raise ValueError(f"gate activation {activation!r}: 'silu' (Qwen3_5RMSNormGated) or 'sigmoid' (KimiK_3_MoeRMSNormGated)")
        self._need(hidden_states, gate, weight)
        return _RMSNormGated.apply(hidden_states, gate, weight, eps, self, _GATE_ACTIVATION[activation])


def _i64(cu, ref):
    if cu is None:
        return None
    return torch.as_tensor(cu).to(device=ref.device, dtype=torch.int64).contiguous()


def _token_view(x):
    """(tensor, token stride in elements) for a [B,T,H,D] tensor whose heads are contiguous within a token and whose
    tokens are evenly spaced (a column slice of a wider [B,T,*] tensor qualifies); anything else is copied."""
    B, T, H, D = x.shape
    vec = 16 // x.element_size()
    ok = (x.stride(3) == 1 and x.stride(2) == D and x.stride(1) >= H * D and x.stride(1) % vec == 0
          and (B == 1 or x.stride(0) == T * x.stride(1)) and x.data_ptr() % 16 == 0)
    if not ok:
        x = x.contiguous()
    return x, x.stride(1)


def _chunk_workspace(lib, device, B, T, N, Hqk, Hv, K, V, code, need_grad):
    """A 256-byte aligned workspace; need_grad: False / True for a forward-only or a forward + backward workspace,
    2 / 3 for its prep part / state part alone (gdn_chunk_workspace_bytes)."""
    nbytes = lib.gdn_chunk_workspace_bytes(B, T, N, Hqk, Hv, K, V, code, int(need_grad))
    ws = torch.empty(nbytes + 256, dtype=torch.uint8, device=device)
    off = (-ws.data_ptr()) % 256
    return ws[off:off + nbytes], nbytes


def _chunk_forward_call(ops, q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens,
                        use_qk_l2norm_in_kernel, need_grad, skip_recompute):
    """One forward call of the chunk rule through the C ABI.  Returns (o, final_state or None, the tensors a backward
    call needs, their description); shared by the autograd function and the torch.library operator."""
    lib = ops.lib
    B, T, Hqk, K = q.shape
    Hv, V = v.shape[2], v.shape[3]
    N = (len(cu_seqlens) - 1) if cu_seqlens is not None else B
    keep = need_grad and skip_recompute
    prep_only = q.dtype != torch.float32 and not keep   # the recurrence writes o itself: no state leaves it
    (qc, sq), (kc, sk), (vc, sv) = _token_view(q), _token_view(k), _token_view(v)
    g32, h0 = ops._f32(g), ops._f32(initial_state)
    bc, bcode = _beta_arg(beta, q.dtype)
    cu = _i64(cu_seqlens, q)
    code = DTYPE_CODE[q.dtype]
    ws, nbytes = _chunk_workspace(lib, q.device, B, T, N, Hqk, Hv, K, V, code, 2 if prep_only else keep)
    o = torch.empty(B, T, Hv, V, dtype=v.dtype, device=v.device)
    ht = torch.empty(N, Hv, K, V, dtype=torch.float32, device=q.device) if output_final_state else None
    rc = lib.gdn_chunk_fwd_strided(ptr(qc), ptr(kc), ptr(vc), sq, sk, sv, ptr(g32), ptr(bc), ptr(h0), ptr(cu),
                                   ptr(o), ptr(ht), ptr(ws), nbytes, B, T, N, Hqk, Hv, K, V, scale,
                                   int(use_qk_l2norm_in_kernel), code, bcode, lib.stream())
    lib.check(rc, "gdn_chunk_fwd_strided")
    saved = (qc, kc, vc, g32, bc, h0, cu, ws if (keep or prep_only) else None)
    meta = (B, T, N, Hqk, Hv, K, V, scale, int(use_qk_l2norm_in_kernel), code, nbytes,
            g.dtype, beta.dtype, None if initial_state is None else initial_state.dtype, sq, sk, sv, bcode, prep_only)
    return o, ht, saved, meta


def _chunk_backward_call(ops, saved, meta, do, dht):
    """The backward pass for a forward call described by (saved, meta) of _chunk_forward_call.
    Returns (dq, dk, dv, dg, dbeta, d initial_state or None) in the dtypes of the forward call's arguments."""
    qc, kc, vc, g32, bc, h0, cu, ws = saved
    B, T, N, Hqk, Hv, K, V, scale, l2, code, nbytes, g_dt, b_dt, h_dt, sq, sk, sv, bcode, prep_only = meta
    lib = ops.lib
    dev = qc.device
    do = do.contiguous()
    dht = ops._f32(dht)
    dq = torch.empty(B, T, Hqk, K, dtype=qc.dtype, device=dev)
    dk = torch.empty(B, T, Hqk, K, dtype=qc.dtype, device=dev)
    dv = torch.empty(B, T, Hv, V, dtype=qc.dtype, device=dev)
    dg = torch.empty(B, T, Hv, dtype=torch.float32, device=dev)
    db = torch.empty(B, T, Hv, dtype=bc.dtype, device=dev)
    dh0 = torch.empty(N, Hv, K, V, dtype=torch.float32, device=dev) if h0 is not None else None
    if ws is not None and prep_only:
        # the prep part was kept: the state part is rebuilt beside the reverse recurrence, then the chunk-local kernels
        ws_state, nstate = _chunk_workspace(lib, dev, B, T, N, Hqk, Hv, K, V, code, 3)

        def phase(ph):
            rc = lib.gdn_chunk_bwd_parts(ptr(qc), ptr(kc), ptr(vc), sq, sk, sv, ptr(g32), ptr(bc), ptr(h0), ptr(cu),
                                         ptr(do), ptr(dht), ptr(dq), ptr(dk), ptr(dv), 0, 0, 0, ptr(dg), ptr(db),
                                         ptr(dh0), ptr(ws), nbytes, ptr(ws_state), nstate, ph, 1, B, T, N, Hqk, Hv, K,
                                         V, scale, l2, code, bcode, lib.stream())
            lib.check(rc, "gdn_chunk_bwd_parts")
        helper = ops.helper_stream(dev)
        if helper is None:
            phase(7)
        else:
            main = torch.cuda.current_stream(dev)
            helper.wait_stream(main)
            with torch.cuda.stream(helper):
                phase(1)
            phase(2)
            main.wait_stream(helper)
            phase(4)
        return dq, dk, dv, dg.to(g_dt), db.to(b_dt), None if dh0 is None else dh0.to(h_dt)
    if ws is None:   # nothing was kept: refill a workspace (no output is written when o is null)
        ws, nbytes = _chunk_workspace(lib, dev, B, T, N, Hqk, Hv, K, V, code, True)
        rc = lib.gdn_chunk_fwd_strided(ptr(qc), ptr(kc), ptr(vc), sq, sk, sv, ptr(g32), ptr(bc), ptr(h0), ptr(cu),
                                       None, None, ptr(ws), nbytes, B, T, N, Hqk, Hv, K, V, scale, l2, code, bcode,
                                       lib.stream())
        lib.check(rc, "gdn_chunk_fwd_strided (recompute)")
    rc = lib.gdn_chunk_bwd_strided(ptr(qc), ptr(kc), ptr(vc), sq, sk, sv, ptr(g32), ptr(bc), ptr(h0), ptr(cu),
                                   ptr(do), ptr(dht), ptr(dq), ptr(dk), ptr(dv), 0, 0, 0, ptr(dg), ptr(db),
                                   ptr(dh0), ptr(ws), nbytes, B, T, N, Hqk, Hv, K, V, scale, l2, code, bcode,
                                   lib.stream())
    lib.check(rc, "gdn_chunk_bwd_strided")
    return dq, dk, dv, dg.to(g_dt), db.to(b_dt), None if dh0 is None else dh0.to(h_dt)


class _ChunkGatedDeltaRule(torch.autograd.Function):
    """Positional order as ChunkGatedDeltaRuleFunction.forward (chunk_gated_delta_rule.py:182-196).

    skip_recompute=False (the default, as in the reference, which saves q, k, v, g_cum, beta, Ai, h0 and recomputes w,
    u, h and v_new in its backward pass, chunk_gated_delta_rule.py:102-119, :264): in the 16-bit dtypes the forward pass
    keeps the prep part of its workspace (cumulative decay, Tm, the intra-chunk tiles and the K / Q^T images: everything
    that does not depend on v or on the state) and the backward pass rebuilds the per-chunk states and v_new with the
    forward recurrence on a second stream while the reverse recurrence runs on the caller's; both are latency-bound and
    fit the device side by side.  In fp32 nothing but the inputs is kept and the backward pass refills the whole
    workspace first.  skip_recompute=True keeps the whole forward workspace instead (per-chunk states and v_new too:
    gdn_chunk_workspace_bytes with with_backward=1) and skips that work.  All give the same gradients, bit for bit."""

    @staticmethod
    @_input_guard
    @_custom_fwd
    def forward(ctx, q, k, v, g, beta, scale, initial_state, output_final_state, cu_seqlens,
                use_qk_l2norm_in_kernel, skip_recompute, ops):
        need_grad = any(ctx.needs_input_grad[:5]) or (initial_state is not None and ctx.needs_input_grad[6])
        o, ht, saved, meta = _chunk_forward_call(ops, q, k, v, g, beta, scale, initial_state, output_final_state,
                                                 cu_seqlens, use_qk_l2norm_in_kernel, need_grad, skip_recompute)
        if need_grad:
            ctx.save_for_backward(*saved)
            ctx.meta = meta
            ctx.ops = ops
            ctx.set_materialize_grads(False)
            ctx.o_like = (o.shape, o.dtype, o.device)
        return o, ht

    @staticmethod
    @_input_guard
    @_custom_bwd
    def backward(ctx, do, dht):
        do = _out_grad(do, ctx.o_like)
        dq, dk, dv, dg, db, dh0 = _chunk_backward_call(ctx.ops, ctx.saved_tensors, ctx.meta, do, dht)
        return dq, dk, dv, dg, db, None, dh0, None, None, None, None, None


class _ChunkGatedDeltaRuleNorm(torch.autograd.Function):
    """Rule + gated RMSNorm in one forward pass; the backward pass is the two operators' backward passes in turn
    (the forward then also writes `o` and 1/rms, which they need)."""

    @staticmethod
    @_input_guard
    @_custom_fwd
    def forward(ctx, q, k, v, g, beta, gate, norm_weight, eps, scale, initial_state, output_final_state, cu_seqlens,
                use_qk_l2norm_in_kernel, ops):
        lib = ops.lib
        B, T, Hqk, K = q.shape
        Hv, V = v.shape[2], v.shape[3]
        N = (len(cu_seqlens) - 1) if cu_seqlens is not None else B
        rule_grad = any(ctx.needs_input_grad[:5]) or (initial_state is not None and ctx.needs_input_grad[9])
        need_grad = rule_grad or ctx.needs_input_grad[5] or ctx.needs_input_grad[6]
        (qc, sq), (kc, sk), (vc, sv) = _token_view(q), _token_view(k), _token_view(v)
        g32, h0 = ops._f32(g), ops._f32(initial_state)
        b32, bcode = _beta_arg(beta, q.dtype)
        cu = _i64(cu_seqlens, q)
        dt = q.dtype
        code = DTYPE_CODE[dt]
        w_dt = dt if norm_weight.dtype == dt else torch.float32
        gc = gate.detach().to(dt).contiguous().view(B, T, Hv, V)
        wc = norm_weight.detach().to(w_dt).contiguous()
        ws, nbytes = _chunk_workspace(lib, q.device, B, T, N, Hqk, Hv, K, V, code, rule_grad)
        y = torch.empty(B, T, Hv, V, dtype=dt, device=v.device)
        o = torch.empty(B, T, Hv, V, dtype=dt, device=v.device) if need_grad else None
        rstd = torch.empty(B * T * Hv, dtype=torch.float32, device=v.device) if need_grad else None
        ht = torch.empty(N, Hv, K, V, dtype=torch.float32, device=q.device) if output_final_state else None
        rc = lib.gdn_chunk_fwd_norm_strided(ptr(qc), ptr(kc), ptr(vc), sq, sk, sv, ptr(g32), ptr(b32), ptr(h0),
                                            ptr(cu), ptr(gc), ptr(wc), ptr(o), ptr(y), ptr(rstd), ptr(ht), ptr(ws),
                                            nbytes, B, T, N, Hqk, Hv, K, V, scale, eps,
                                            int(use_qk_l2norm_in_kernel), code, DTYPE_CODE[w_dt], bcode, lib.stream())
        lib.check(rc, "gdn_chunk_fwd_norm_strided")
        if need_grad:
            ctx.save_for_backward(qc, kc, vc, g32, b32, h0, cu, ws if rule_grad else None, o, gc, wc, rstd)
            ctx.meta = (B, T, N, Hqk, Hv, K, V, scale, int(use_qk_l2norm_in_kernel), code, nbytes, g.dtype,
                        beta.dtype, None if initial_state is None else initial_state.dtype, sq, sk, sv, w_dt,
                        norm_weight.dtype, gate.dtype, gate.shape, rule_grad, bcode)
            ctx.ops = ops
            ctx.set_materialize_grads(False)
            ctx.o_like = (y.shape, y.dtype, y.device)
        return y, ht

    @staticmethod
    @_input_guard
    @_custom_bwd
    def backward(ctx, dy, dht):
        qc, kc, vc, g32, b32, h0, cu, ws, o, gc, wc, rstd = ctx.saved_tensors
        (B, T, N, Hqk, Hv, K, V, scale, l2, code, nbytes, g_dt, b_dt, h_dt, sq, sk, sv, w_dt, weight_dt, gate_dt,
         gate_shape, rule_grad, bcode) = ctx.meta
        lib = ctx.ops.lib
        dev, dt = qc.device, qc.dtype
        rows = B * T * Hv
        dyc = _out_grad(dy, ctx.o_like).to(dt).contiguous()
        do = torch.empty_like(o)
        dgate = torch.empty_like(o)
        dw = torch.empty(V, dtype=torch.float32, device=dev)
        nb = lib.gdn_rmsnorm_gated_bwd_workspace_bytes(rows, V)
        nws = torch.empty(nb, dtype=torch.uint8, device=dev)
        rc = lib.gdn_rmsnorm_gated_bwd(ptr(o), ptr(gc), ptr(wc), ptr(rstd), ptr(dyc), ptr(do), ptr(dgate), ptr(dw),
                                       ptr(nws), nb, rows, V, code, DTYPE_CODE[w_dt], 0, lib.stream())
        lib.check(rc, "gdn_rmsnorm_gated_bwd")
        dq = dk = dv = dg = db = dh0 = None
        if rule_grad:
            dht = ctx.ops._f32(dht)
            dq = torch.empty(B, T, Hqk, K, dtype=dt, device=dev)
            dk = torch.empty(B, T, Hqk, K, dtype=dt, device=dev)
            dv = torch.empty(B, T, Hv, V, dtype=dt, device=dev)
            dg = torch.empty(B, T, Hv, dtype=torch.float32, device=dev)
            db = torch.empty(B, T, Hv, dtype=b32.dtype, device=dev)
            dh0 = torch.empty(N, Hv, K, V, dtype=torch.float32, device=dev) if h0 is not None else None
            rc = lib.gdn_chunk_bwd_strided(ptr(qc), ptr(kc), ptr(vc), sq, sk, sv, ptr(g32), ptr(b32), ptr(h0),
                                           ptr(cu), ptr(do), ptr(dht), ptr(dq), ptr(dk), ptr(dv), 0, 0, 0, ptr(dg),
                                           ptr(db), ptr(dh0), ptr(ws), nbytes, B, T, N, Hqk, Hv, K, V, scale, l2,
                                           code, bcode, lib.stream())
            lib.check(rc, "gdn_chunk_bwd_strided")
            dg, db = dg.to(g_dt), db.to(b_dt)
            dh0 = None if dh0 is None else dh0.to(h_dt)
        return (dq, dk, dv, dg, db, dgate.view(gate_shape).to(gate_dt), dw.to(weight_dt), None, None, dh0, None,
                None, None, None)


class _ChunkGatedDeltaRuleQKV(torch.autograd.Function):
    """The rule on the convolution's output as it is: q, k, v are the column ranges [0, Hqk K), [Hqk K, 2 Hqk K),
    [2 Hqk K, 2 Hqk K + Hv V) of mixed_qkv [B,T,D] (the split of modeling_qwen3_5.py:818-831), read in place; the
    backward pass writes dq, dk, dv into one [B,T,D] gradient, so neither the split nor its backward copies."""

    @staticmethod
    @_input_guard
    @_custom_fwd
    def forward(ctx, qkv, g, beta, Hqk, Hv, K, V, scale, initial_state, output_final_state, cu_seqlens,
                use_qk_l2norm_in_kernel, ops):
        lib = ops.lib
        B, T, D = qkv.shape
        nq, nv = Hqk * K, Hv * V
        N = (len(cu_seqlens) - 1) if cu_seqlens is not None else B
        need_grad = any(ctx.needs_input_grad[:3]) or (initial_state is not None and ctx.needs_input_grad[8])
        vec = 16 // qkv.element_size()
        x = qkv if (qkv.is_contiguous() and D % vec == 0 and qkv.data_ptr() % 16 == 0) else qkv.contiguous()
        g32, h0 = ops._f32(g), ops._f32(initial_state)
        b32, bcode = _beta_arg(beta, qkv.dtype)
        cu = _i64(cu_seqlens, qkv)
        code = DTYPE_CODE[qkv.dtype]
        es = x.element_size()
        ws, nbytes = _chunk_workspace(lib, qkv.device, B, T, N, Hqk, Hv, K, V, code, need_grad)
        o = torch.empty(B, T, Hv, V, dtype=qkv.dtype, device=qkv.device)
        ht = torch.empty(N, Hv, K, V, dtype=torch.float32, device=qkv.device) if output_final_state else None
        base = x.data_ptr()
        rc = lib.gdn_chunk_fwd_strided(base, base + nq * es, base + 2 * nq * es, D, D, D, ptr(g32), ptr(b32), ptr(h0),
                                       ptr(cu), ptr(o), ptr(ht), ptr(ws), nbytes, B, T, N, Hqk, Hv, K, V, scale,
                                       int(use_qk_l2norm_in_kernel), code, bcode, lib.stream())
        lib.check(rc, "gdn_chunk_fwd_strided")
        if need_grad:
            ctx.save_for_backward(x, g32, b32, h0, cu, ws)
            ctx.meta = (B, T, D, N, Hqk, Hv, K, V, scale, int(use_qk_l2norm_in_kernel), code, nbytes,
                        g.dtype, beta.dtype, None if initial_state is None else initial_state.dtype, bcode)
            ctx.ops = ops
            ctx.set_materialize_grads(False)
            ctx.o_like = (o.shape, o.dtype, o.device)
        return o, ht

    @staticmethod
    @_input_guard
    @_custom_bwd
    def backward(ctx, do, dht):
        x, g32, b32, h0, cu, ws = ctx.saved_tensors
        B, T, D, N, Hqk, Hv, K, V, scale, l2, code, nbytes, g_dt, b_dt, h_dt, bcode = ctx.meta
        lib = ctx.ops.lib
        nq, nv, es, dev = Hqk * K, Hv * V, x.element_size(), x.device
        do = _out_grad(do, ctx.o_like)
        dht = ctx.ops._f32(dht)
        # columns past q, k, v (none in the layer) receive no gradient
        dx = torch.empty_like(x) if D == 2 * nq + nv else torch.zeros_like(x)
        dg = torch.empty(B, T, Hv, dtype=torch.float32, device=dev)
        db = torch.empty(B, T, Hv, dtype=b32.dtype, device=dev)
        dh0 = torch.empty(N, Hv, K, V, dtype=torch.float32, device=dev) if h0 is not None else None
        base, dbase = x.data_ptr(), dx.data_ptr()
        rc = lib.gdn_chunk_bwd_strided(base, base + nq * es, base + 2 * nq * es, D, D, D, ptr(g32), ptr(b32), ptr(h0),
                                       ptr(cu), ptr(do), ptr(dht), dbase, dbase + nq * es, dbase + 2 * nq * es, D, D,
                                       D, ptr(dg), ptr(db), ptr(dh0), ptr(ws), nbytes, B, T, N, Hqk, Hv, K, V, scale,
                                       l2, code, bcode, lib.stream())
        lib.check(rc, "gdn_chunk_bwd_strided")
        return (dx, dg.to(g_dt), db.to(b_dt), None, None, None, None, None, None if dh0 is None else dh0.to(h_dt),
                None, None, None, None)


class _ChunkKda(torch.autograd.Function):
    """KDA through the HIP library: gdn_kda_fwd, and gdn_kda_bwd on the workspace the forward call filled (it is kept
    between the passes when a gradient is asked for)."""

    @staticmethod
    @_input_guard
    @_custom_fwd
    def forward(ctx, q, k, v, g, beta, A_log, dt_bias, scale, initial_state, output_final_state, l2norm, use_gate,
                beta_sigmoid, allow_neg, cu_seqlens, lower_bound, want_states, transposed_states, ops):
        lib = ops.lib
        B, T, H, K = q.shape
        V = v.shape[3]
        N = (len(cu_seqlens) - 1) if cu_seqlens is not None else B
        code = DTYPE_CODE[q.dtype]
        need_grad = any(ctx.needs_input_grad[:7]) or (initial_state is not None and ctx.needs_input_grad[8])
        qc, kc, vc = q.detach().contiguous(), k.detach().contiguous(), v.detach().contiguous()
        gc = g.detach().contiguous() if g.dtype == q.dtype else g.detach().to(torch.float32).contiguous()
        gcode = code if g.dtype == q.dtype else 0
        bc, bcode = _beta_arg(beta, q.dtype)
        a32, d32, h0 = ops._f32(A_log), ops._f32(dt_bias), ops._f32(initial_state)
        cu = _i64(cu_seqlens, q)
        # the per-chunk states stay in the workspace only when it has the size that serves a backward pass
        nbytes = lib.gdn_kda_workspace_bytes(B, T, N, H, K, V, int(need_grad or want_states), code)
        ws = torch.empty(nbytes + 256, dtype=torch.uint8, device=q.device)
        off = (-ws.data_ptr()) % 256
        ws = ws[off:off + nbytes]
        o = torch.empty(B, T, H, V, dtype=v.dtype, device=v.device)
        ht = torch.empty(N, H, K, V, dtype=torch.float32, device=q.device) if output_final_state else None
        opts = (int(l2norm), int(use_gate), int(lower_bound is not None),
                float(lower_bound if lower_bound is not None else 0.0), int(beta_sigmoid), int(allow_neg), code, gcode, bcode)
        rc = lib.gdn_kda_fwd(ptr(qc), ptr(kc), ptr(vc), ptr(gc), ptr(bc), ptr(a32), ptr(d32), ptr(h0), ptr(cu), ptr(o),
                             ptr(ht), ptr(ws), nbytes, B, T, N, H, K, V, scale, *opts, lib.stream())
        lib.check(rc, "gdn_kda_fwd")
        hs = None
        if want_states:
            # the states at chunk entries, from the tiles the recurrence left in the workspace; the number of chunks of a
            # packed batch needs the sequence lengths on the host (the reference reads them there as well)
            if cu_seqlens is None:
                rows, nt = B, (T + 63) // 64
            else:
                c = cu_seqlens.tolist() if torch.is_tensor(cu_seqlens) else list(cu_seqlens)
                rows, nt = 1, sum((int(b) - int(a) + 63) // 64 for a, b in zip(c[:-1], c[1:]))
            hs = torch.empty((rows, nt, H, V, K) if transposed_states else (rows, nt, H, K, V), dtype=q.dtype, device=q.device)
            rc = lib.gdn_kda_intermediate_states(ptr(ws), nbytes, ptr(cu), ptr(hs), rows * nt, B, T, N, H, K, V,
                                                 int(transposed_states), code, lib.stream())
            lib.check(rc, "gdn_kda_intermediate_states")
            ctx.mark_non_differentiable(hs)
        if need_grad:
            ctx.save_for_backward(qc, kc, vc, gc, a32, d32, cu, ws)
            ctx.meta = (B, T, N, H, K, V, scale, opts, nbytes, g.dtype, beta.dtype, bc.dtype,
                        None if A_log is None else A_log.dtype, None if dt_bias is None else (dt_bias.dtype, dt_bias.shape),
                        None if initial_state is None else initial_state.dtype)
            ctx.ops = ops
            ctx.set_materialize_grads(False)
            ctx.o_like = (o.shape, o.dtype, o.device)
        return o, ht, hs

    @staticmethod
    @_input_guard
    @_custom_bwd
    def backward(ctx, do, dht, _dhs=None):
        qc, kc, vc, gc, a32, d32, cu, ws = ctx.saved_tensors
        B, T, N, H, K, V, scale, opts, nbytes, g_dt, b_dt, bc_dt, a_dt, d_dt, h_dt = ctx.meta
        lib = ctx.ops.lib
        dev = qc.device
        do = _out_grad(do, ctx.o_like)
        dht = ctx.ops._f32(dht)
        dq, dk, dv, dg = torch.empty_like(qc), torch.empty_like(kc), torch.empty_like(vc), torch.empty_like(gc)
        db = torch.empty(B, T, H, dtype=bc_dt, device=dev)
        use_gate = bool(opts[1])
        dA = torch.empty(H, dtype=torch.float32, device=dev) if (use_gate and a32 is not None) else None
        dD = torch.empty(H * K, dtype=torch.float32, device=dev) if (use_gate and d32 is not None) else None
        dh0 = torch.empty(N, H, K, V, dtype=torch.float32, device=dev) if h_dt is not None else None
        rc = lib.gdn_kda_bwd(ptr(qc), ptr(kc), ptr(vc), ptr(gc), ptr(a32), ptr(d32), ptr(cu), ptr(do), ptr(dht), ptr(dq),
                             ptr(dk), ptr(dv), ptr(dg), ptr(db), ptr(dA), ptr(dD), ptr(dh0), ptr(ws), nbytes, B, T, N, H, K,
                             V, scale, *opts, lib.stream())
        lib.check(rc, "gdn_kda_bwd")
        return (dq, dk, dv, dg.to(g_dt), db.to(b_dt), None if dA is None else dA.to(a_dt),
                None if dD is None else dD.to(d_dt[0]).reshape(d_dt[1]), None, None if dh0 is None else dh0.to(h_dt),
                None, None, None, None, None, None, None, None, None, None)


class _GdnGates(torch.autograd.Function):
    """beta = sigmoid(b), g = -exp(A_log.float()) * softplus(a.float() + dt_bias), modeling_qwen3_5.py:833-841."""

    @staticmethod
    @_input_guard
    @_custom_fwd
    def forward(ctx, a, b, A_log, dt_bias, ops):
        lib = ops.lib
        Hv = a.shape[-1]
        ac, bc = a.contiguous(), b.contiguous()
        pdt = a.dtype if (A_log.dtype == a.dtype and dt_bias.dtype == a.dtype) else torch.float32
        Ac, dc = A_log.detach().to(pdt).contiguous(), dt_bias.detach().to(pdt).contiguous()
        tokens = ac.numel() // Hv
        g = torch.empty(ac.shape, dtype=torch.float32, device=a.device)
        beta = torch.empty_like(bc)
        rc = lib.gdn_gate_fwd(ptr(ac), ptr(bc), ptr(Ac), ptr(dc), ptr(g), ptr(beta), tokens, Hv, DTYPE_CODE[a.dtype],
                              DTYPE_CODE[pdt], lib.stream())
        lib.check(rc, "gdn_gate_fwd")
        ctx.save_for_backward(ac, bc, Ac, dc)
        ctx.meta = (tokens, Hv, A_log.dtype, dt_bias.dtype)
        ctx.ops = ops
        return g, beta

    @staticmethod
    @_input_guard
    @_custom_bwd
    def backward(ctx, dg, dbeta):
        ac, bc, Ac, dc = ctx.saved_tensors
        tokens, Hv, A_dt, d_dt = ctx.meta
        lib = ctx.ops.lib
        dg = dg.to(torch.float32).contiguous()
        dbeta = dbeta.to(bc.dtype).contiguous()
        da, db = torch.empty_like(ac), torch.empty_like(bc)
        dA = torch.empty(Hv, dtype=torch.float32, device=ac.device)
        dd = torch.empty(Hv, dtype=torch.float32, device=ac.device)
        nbytes = lib.gdn_gate_bwd_workspace_bytes(tokens, Hv)
        ws = torch.empty(max(nbytes, 4), dtype=torch.uint8, device=ac.device)
        rc = lib.gdn_gate_bwd(ptr(ac), ptr(bc), ptr(Ac), ptr(dc), ptr(dg), ptr(dbeta), ptr(da), ptr(db), ptr(dA),
                              ptr(dd), ptr(ws), nbytes, tokens, Hv, DTYPE_CODE[ac.dtype], DTYPE_CODE[Ac.dtype],
                              lib.stream())
        lib.check(rc, "gdn_gate_bwd")
        return da, db, dA.to(A_dt), dd.to(d_dt), None


class _CausalConv1d(torch.autograd.Function):
    """Argument order as CausalConv1dFunction.forward (models/qwen3_5/causal_conv1d.py:27-38)."""

    @staticmethod
    @_input_guard
    @_custom_fwd
    def forward(ctx, x, weight, bias, residual, initial_state, activation, cu_seqlens, output_final_state, ops):
        lib = ops.lib
        B, T, D = x.shape
        W = weight.shape[0]
        N = (len(cu_seqlens) - 1) if cu_seqlens is not None else B
        dt = x.dtype
        xc = x.contiguous()
        wc = weight.to(dt).contiguous()
        bc = None if bias is None else bias.to(dt).contiguous()
        rc_ = None if residual is None else residual.to(dt).contiguous()
        h0 = None if initial_state is None else initial_state.to(dt).contiguous()
        cu = _i64(cu_seqlens, x)
        y = torch.empty_like(xc)
        fs = torch.empty(N, D, W, dtype=dt, device=x.device) if output_final_state else None
        code = lib.gdn_conv1d_fwd(ptr(xc), ptr(wc), ptr(bc), ptr(rc_), ptr(h0), ptr(cu), ptr(y), ptr(fs), B, T, N, D,
                                  W, _act_code(activation), DTYPE_CODE[dt], lib.stream())
        lib.check(code, "gdn_conv1d_fwd")
        ctx.save_for_backward(xc, wc, bc, h0, cu)
        ctx.meta = (B, T, N, D, W, _act_code(activation), dt, weight.dtype, None if bias is None else bias.dtype,
                    residual is not None, None if residual is None else residual.dtype,
                    None if initial_state is None else initial_state.dtype)
        ctx.ops = ops
        return y, fs

    @staticmethod
    @_input_guard
    @_custom_bwd
    def backward(ctx, dy, dfs):
        xc, wc, bc, h0, cu = ctx.saved_tensors
        B, T, N, D, W, act, dt, w_dt, b_dt, has_res, r_dt, h_dt = ctx.meta
        lib = ctx.ops.lib
        dy = dy.to(dt).contiguous()
        dfs = None if dfs is None else dfs.to(dt).contiguous()
        dx = torch.empty_like(xc)
        dw = torch.empty(W, D, dtype=torch.float32, device=xc.device)
        db = torch.empty(D, dtype=torch.float32, device=xc.device) if bc is not None else None
        dh0 = torch.empty(N, D, W, dtype=dt, device=xc.device) if h0 is not None else None
        nbytes = lib.gdn_conv1d_bwd_workspace_bytes(B, T, D, W)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=xc.device)
        code = lib.gdn_conv1d_bwd(ptr(xc), ptr(dy), ptr(wc), ptr(bc), ptr(h0), ptr(dfs), ptr(cu), ptr(dx), ptr(dw),
                                  ptr(db), ptr(dh0), ptr(ws), nbytes, B, T, N, D, W, act, DTYPE_CODE[dt], lib.stream())
        lib.check(code, "gdn_conv1d_bwd")
        return (dx, dw.to(w_dt), None if db is None else db.to(b_dt), dy.to(r_dt) if has_res else None,
                None if dh0 is None else dh0.to(h_dt), None, None, None, None)


_GATE_ACTIVATION = {"silu": 0, "swish": 0, "sigmoid": 1}


class _RMSNormGated(torch.autograd.Function):
    """y = (weight * rmsnorm(x)) * act(gate) over the last axis, act = silu (code 0) or sigmoid (code 1)."""

    @staticmethod
    @_input_guard
    @_custom_fwd
    def forward(ctx, x, gate, weight, eps, ops, act=0):
        lib = ops.lib
        dt = x.dtype
        if dt not in (torch.float32, torch.bfloat16):
            raise ValueError(f"rms_norm_gated supports float32 and bfloat16, got {dt}")
        if gate.shape != x.shape:
            raise ValueError(f"gate shape {tuple(gate.shape)} differs from hidden_states shape {tuple(x.shape)}")
        N = x.shape[-1]
        if weight.shape != (N,):
            raise ValueError(f"weight shape {tuple(weight.shape)}, expected ({N},)")
        w_dt = dt if weight.dtype == dt else torch.float32   # same dtype as the input, else fp32 as in the reference
        xc = x.contiguous().view(-1, N)
        gc = gate.to(dt).contiguous().view(-1, N)
        wc = weight.detach().to(w_dt).contiguous()
        rows = xc.shape[0]
        y = torch.empty_like(xc)
        rstd = torch.empty(rows, dtype=torch.float32, device=x.device)
        code = lib.gdn_rmsnorm_gated_fwd(ptr(xc), ptr(gc), ptr(wc), ptr(y), ptr(rstd), rows, N, float(eps),
                                         DTYPE_CODE[dt], DTYPE_CODE[w_dt], act, lib.stream())
        lib.check(code, "gdn_rmsnorm_gated_fwd")
        ctx.save_for_backward(xc, gc, wc, rstd)
        ctx.meta = (rows, N, dt, w_dt, weight.dtype, gate.dtype, x.shape, act)
        ctx.ops = ops
        return y.view(x.shape)

    @staticmethod
    @_input_guard
    @_custom_bwd
    def backward(ctx, dy):
        xc, gc, wc, rstd = ctx.saved_tensors
        rows, N, dt, w_dt, weight_dt, gate_dt, shape, act = ctx.meta
        lib = ctx.ops.lib
        dyc = dy.to(dt).contiguous().view(-1, N)
        dx = torch.empty_like(xc)
        dg = torch.empty_like(xc)
        dw = torch.empty(N, dtype=torch.float32, device=xc.device)
        nbytes = lib.gdn_rmsnorm_gated_bwd_workspace_bytes(rows, N)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=xc.device)
        code = lib.gdn_rmsnorm_gated_bwd(ptr(xc), ptr(gc), ptr(wc), ptr(rstd), ptr(dyc), ptr(dx), ptr(dg), ptr(dw),
                                         ptr(ws), nbytes, rows, N, DTYPE_CODE[dt], DTYPE_CODE[w_dt], act, lib.stream())
        lib.check(code, "gdn_rmsnorm_gated_bwd")
        return dx.view(shape), dg.view(shape).to(gate_dt), dw.to(weight_dt), None, None, None


# ---------------------------------------------------------------------- module-level entry points
_ops: Optional[GdnOps] = None


def _default_ops() -> GdnOps:
    global _ops
    if _ops is None:
        _ops = GdnOps(default_library())
    return _ops


@torch.compiler.disable
def chunk_gated_delta_rule(q, k, v, g, beta, scale=None, initial_state=None, output_final_state=False,
                           use_qk_l2norm_in_kernel=False, cu_seqlens=None, chunk_size=64, head_first=False,
                           skip_recompute=False):
    """Drop-in for mindspeed_mm.fsdp.ops.gdn.chunk_gated_delta_rule.chunk_gated_delta_rule.

    q,k [B,T,Hqk,K]; v [B,T,Hv,V]; g,beta [B,T,Hv]; Hv may be a multiple of Hqk (grouped heads are read in
    place; dq/dk come back summed over each group).  float32 is accepted as well as bfloat16.
    skip_recompute=False (default, as in the reference): nothing but the inputs is kept for the backward pass, which
    recomputes Tm, the per-chunk states and v_new; skip_recompute=True keeps the forward pass's workspace instead
    (gdn_chunk_workspace_bytes with with_backward=1: 1.2 GB at B=2, T=8192, H_v=32, d=128) for a faster backward pass.
    The gradients are the same bits either way."""
    return _default_ops().chunk_gated_delta_rule(q, k, v, g, beta, scale, initial_state, output_final_state,
                                                 use_qk_l2norm_in_kernel, cu_seqlens, chunk_size, head_first,
                                                 skip_recompute)


@torch.compiler.disable
def chunk_gated_delta_rule_norm(q, k, v, g, beta, gate, norm_weight, eps=1e-6, scale=None, initial_state=None,
                                output_final_state=False, use_qk_l2norm_in_kernel=False, cu_seqlens=None,
                                in_output_kernel=False, skip_recompute=False):
    return _default_ops().chunk_gated_delta_rule_norm(q, k, v, g, beta, gate, norm_weight, eps, scale, initial_state,
                                                      output_final_state, use_qk_l2norm_in_kernel, cu_seqlens,
                                                      in_output_kernel, skip_recompute)


@torch.compiler.disable
def chunk_gated_delta_rule_qkv(mixed_qkv, g, beta, num_k_heads, num_v_heads, head_k_dim, head_v_dim, scale=None,
                               initial_state=None, output_final_state=False, use_qk_l2norm_in_kernel=False,
                               cu_seqlens=None, gate=None, norm_weight=None, norm_eps=1e-6):
    return _default_ops().chunk_gated_delta_rule_qkv(mixed_qkv, g, beta, num_k_heads, num_v_heads, head_k_dim,
                                                     head_v_dim, scale, initial_state, output_final_state,
                                                     use_qk_l2norm_in_kernel, cu_seqlens, gate, norm_weight, norm_eps)


@torch.compiler.disable
def chunk_kda(q, k, v, g, beta, scale=None, initial_state=None, output_final_state=False, **kwargs):
    return _default_ops().chunk_kda(q, k, v, g, beta, scale, initial_state, output_final_state, **kwargs)


@torch.compiler.disable
def gdn_gates(a, b, A_log, dt_bias):
    return _default_ops().gdn_gates(a, b, A_log, dt_bias)


@torch.compiler.disable
def fused_recurrent_gated_delta_rule(q, k, v, g, beta=None, scale=None, initial_state=None,
                                     output_final_state=False, cu_seqlens=None, use_qk_l2norm_in_kernel=False,
                                     inplace_state=False):
    return _default_ops().fused_recurrent_gated_delta_rule(q, k, v, g, beta, scale, initial_state,
                                                           output_final_state, cu_seqlens, use_qk_l2norm_in_kernel,
                                                           inplace_state)


@torch.compiler.disable
def fused_recurrent_gated_delta_rule_qkv(mixed_qkv, a, b, A_log, dt_bias, num_k_heads, num_v_heads, head_k_dim,
                                         head_v_dim, scale=None, initial_state=None, output_final_state=False,
                                         use_qk_l2norm_in_kernel=False, inplace_state=False):
    return _default_ops().fused_recurrent_gated_delta_rule_qkv(
        mixed_qkv, a, b, A_log, dt_bias, num_k_heads, num_v_heads, head_k_dim, head_v_dim, scale, initial_state,
        output_final_state, use_qk_l2norm_in_kernel, inplace_state)


@torch.compiler.disable
def decode_step(mixed_qkv, a, b, conv_state, recurrent_state, conv_weight, conv_bias, A_log, dt_bias, num_k_heads,
                num_v_heads, head_k_dim, head_v_dim, activation="silu"):
    return _default_ops().decode_step(mixed_qkv, a, b, conv_state, recurrent_state, conv_weight, conv_bias, A_log,
                                      dt_bias, num_k_heads, num_v_heads, head_k_dim, head_v_dim, activation)


class GdnDecodeCache:
    """The linear-attention half of Qwen3_5DynamicCache (modeling_qwen3_5.py:134-221): per layer a convolution state
    [B, D, W] and a recurrent state [B, Hv, K, V], created by the prefill, updated in place by decode_step, reordered
    along the batch for beam search.  Host-side bookkeeping only."""

    def __init__(self, num_layers):
        self.conv_states = [None] * num_layers
        self.recurrent_states = [None] * num_layers

    def __len__(self):
        return len(self.conv_states)

    def set_prefill(self, layer_idx, conv_final_state, recurrent_final_state):
        """conv_final_state: the final_state causal_conv1d returns with output_final_state=True, which is the layer's
        zero-left-padded last W inputs (modeling_qwen3_5.py:746-750); recurrent_final_state: the rule's final_state."""
        self.conv_states[layer_idx] = conv_final_state.contiguous()
        self.recurrent_states[layer_idx] = recurrent_final_state.to(torch.float32).contiguous()

    def has_previous_state(self, layer_idx):
        return self.conv_states[layer_idx] is not None

    def reorder_cache(self, beam_idx):
        """index_select along the batch of every state (modeling_qwen3_5.py:183-196)."""
        for i, c in enumerate(self.conv_states):
            if c is not None:
                idx = beam_idx.to(c.device)
                self.conv_states[i] = c.index_select(0, idx)
                self.recurrent_states[i] = self.recurrent_states[i].index_select(0, idx)


@torch.compiler.disable
def causal_conv1d(x, weight, bias=None, residual=None, initial_state=None, activation=None, cu_seqlens=None,
                  output_final_state=False):
    return _default_ops().causal_conv1d(x, weight, bias, residual, initial_state, activation, cu_seqlens,
                                        output_final_state)


@torch.compiler.disable
def causal_conv1d_update(hidden_states, conv_state, weight, bias=None, activation=None):
    return _default_ops().causal_conv1d_update(hidden_states, conv_state, weight, bias, activation)


@torch.compiler.disable
def rms_norm_gated(hidden_states, gate, weight, eps=1e-6, activation="silu"):
    """Functional form of Qwen3_5RMSNormGated.forward (modeling_qwen3_5.py:341-349):
    (weight * rmsnorm(hidden_states)) * silu(gate) over the last axis, in the input dtype; with activation="sigmoid"
    that of KimiK_3_MoeRMSNormGated.forward (modeling_kimi_linear.py:83-96), whose gate passes through a sigmoid."""
    return _default_ops().rms_norm_gated(hidden_states, gate, weight, eps, activation)


class RMSNormGated(torch.nn.Module):
    """Drop-in for Qwen3_5RMSNormGated (modeling_qwen3_5.py:330-349) and, constructed with activation="sigmoid" as the
    KDA layer constructs its norm (modeling_kimi_linear.py:603-604), for KimiK_3_MoeRMSNormGated (:75-96): same
    constructor, parameter and forward."""

    def __init__(self, hidden_size, eps=1e-6, activation="silu", **kwargs):
        super().__init__()
        if activation not in _GATE_ACTIVATION:
            raise ValueError(f"gate activation {activation!r}: 'silu' or 'sigmoid'")
        self.weight = torch.nn.Parameter(torch.ones(hidden_size))
        self.variance_epsilon = eps
        self.activation = activation

    def forward(self, hidden_states, gate=None):
        return rms_norm_gated(hidden_states, gate, self.weight, self.variance_epsilon, self.activation)


class ShortConvolution(torch.nn.Conv1d):
    """Drop-in for the KDA layer's ShortConvolution (mindspeed_mm/fsdp/ops/kda/short_conv.py:18-218): the same
    constructor, parameters (a depthwise nn.Conv1d weight [D, 1, W], optional bias) and forward, over causal_conv1d /
    causal_conv1d_update of this package.  `backend` is accepted and reported as 'mi355x'."""

    def __init__(self, hidden_size, kernel_size, bias=False, activation="silu", backend="triton", device=None,
                 dtype=None, **kwargs):
        super().__init__(in_channels=hidden_size, out_channels=hidden_size, kernel_size=kernel_size,
                         groups=hidden_size, bias=bias, padding=kernel_size - 1, device=device, dtype=dtype)
        self.hidden_size = hidden_size
        self.activation = None
        if activation is not None:
            if activation not in ("silu", "swish"):
                raise AssertionError(f"Activation `{activation}` not supported yet.")   # short_conv.py:72
            self.activation = activation
        self.backend = "mi355x"

    def extra_repr(self):
        return (f"{self.in_channels}, {self.out_channels}, kernel_size={self.kernel_size}, groups={self.groups}, "
                f"bias={self.bias is not None}, activation={self.activation}, backend={self.backend}")

    def forward(self, x, residual=None, mask=None, cache=None, output_final_state=False, cu_seqlens=None,
                chunk_indices=None, **kwargs):
        """x [B, T, D] (B = 1 with cu_seqlens); cache [N, D, W], updated in place in the decoding case (one token per
        sequence, short_conv.py:145-154); returns (y [B, T, D], final state [N, D, W] or None)."""
        B, T = x.shape[0], x.shape[1]
        N = B if cu_seqlens is None else len(cu_seqlens) - 1
        if mask is not None:
            if cu_seqlens is not None:
                raise ValueError("`mask` and `cu_seqlens` cannot be provided at the same time")
            x = x.mul_(mask.unsqueeze(-1))     # in place, as the reference does (short_conv.py:143)
        if B * T == N:
            return self.step(x, residual, cache, output_final_state, cu_seqlens)
        weight = self.weight.squeeze(1).transpose(0, 1).contiguous()      # [D, 1, W] -> [W, D]
        # further keywords (the reference hands them to a kernel that ignores them, short_conv.py:155-166) are dropped
        return causal_conv1d(x=x, weight=weight, bias=self.bias, residual=residual, initial_state=cache,
                             output_final_state=output_final_state, activation=self.activation,
                             cu_seqlens=cu_seqlens)

    def step(self, x, residual, cache, output_final_state=False, cu_seqlens=None):
        """One token per sequence: the cache rolls by one and takes the token (short_conv.py:185-213)."""
        D, W = x.shape[-1], self.kernel_size[0]
        N = x.shape[0] if cu_seqlens is None else len(cu_seqlens) - 1
        if cache is None:
            cache = x.new_zeros(N, D, W)
        y = causal_conv1d_update(x.reshape(N, 1, D), cache, self.weight.squeeze(1), self.bias, self.activation)
        y = y.reshape(x.shape)
        if residual is not None:
            y = y + residual
        return y, (cache if output_final_state else None)

    @property
    def state_size(self):
        return self.hidden_size * self.kernel_size[0]

