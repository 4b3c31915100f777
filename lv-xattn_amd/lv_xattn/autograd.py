"""The two autograd wrappers the reference's harnesses build around
`_attn_forward` / `_attn_backward`:

* `create_attention_class_save_qkv` - classic save-(q,k,v,o,L) function
  (test.py:38-77 and test_llama3.py:125-178 there);
* `create_attention_class`          - the K/V-RECOMPUTE variant
  (test_llama3.py:180-245): forward keeps only (x, o, L); backward re-runs the
  projection of the shared visual hidden states instead of loading stored K/V.

Unlike the reference's recompute wrapper, which returns no gradients at all
(test_llama3.py:243), backward here returns real ones, including the gradient
that flows into the visual hidden states (dX_vis) and the projection weights.
"""
from __future__ import annotations

from typing import Callable, Optional

import torch

from . import ops
from ._lib import LvxError
from .attn import Mask, _attn_backward, _attn_forward, _reject_unsupported
from .async_communication import reset_global_memory_buffer


def create_attention_class_save_qkv(attention_mode: str = "lv_xattn", no_overlap: bool = False,
                                    rounds: Optional[int] = None, batched: bool = False):
    """apply(q, k, v, causal, sm_scale, bias_func=None, local_bias_args=[],
    remote_bias_args=[], mask=None) -> o"""
    if attention_mode != "lv_xattn":
        raise ValueError("only attention_mode='lv_xattn' exists on this path")

    class _attention(torch.autograd.Function):
        @staticmethod
        def forward(ctx, q, k, v, causal, sm_scale, bias_func=None, local_bias_args=[],
                    remote_bias_args=[], mask=None):
            q, k, v, o, L = _attn_forward(q, k, v, causal, sm_scale, None, bias_func, local_bias_args,
                                          remote_bias_args, no_overlap, rounds=rounds, mask=mask,
                                          batched=batched)
            # like the reference (test_llama3.py:144-149): the bias arguments are kept and the
            # bias is rebuilt in backward
            ctx.save_for_backward(q, k, v, o, L, *local_bias_args, *remote_bias_args)
            ctx.n_local = len(local_bias_args)
            ctx.bias_func = bias_func
            ctx.sm_scale, ctx.causal, ctx.mask = sm_scale, causal, mask
            return o

        @staticmethod
        def backward(ctx, do):
            q, k, v, o, L, *bias_args = ctx.saved_tensors
            dq, dk, dv = _attn_backward(do, q, k, v, o, L, ctx.causal, ctx.sm_scale, None, "flash",
                                        ctx.bias_func, bias_args[:ctx.n_local], bias_args[ctx.n_local:],
                                        no_overlap=no_overlap, rounds=rounds, mask=ctx.mask, batched=batched)
            return dq, dk, dv, None, None, None, None, None, None

    return _attention


class KVProjection:
    """The K/V half of the reference's `project` closure
    (test_llama3.py:395-398): K = X_vis W_k, V = X_vis W_v, computed by the
    gfx950 GEMM and handed to attention in [B, Lkv, Hkv, D] memory order."""

    def __init__(self, w_k: torch.Tensor, w_v: torch.Tensor, n_kv_heads: int, w_in_major: bool = True):
        self.w_k, self.w_v, self.n_kv_heads, self.w_in_major = w_k, w_v, n_kv_heads, w_in_major

    def __call__(self, x_vis: torch.Tensor):
        return ops.kv_proj(x_vis, self.w_k, self.w_v, self.n_kv_heads, self.w_in_major)


def create_attention_class(attention_mode: str = "lv_xattn", no_overlap: bool = False,
                           rounds: Optional[int] = None, batched: bool = False,
                           weight_grads: bool = False, w_in_major: bool = True):
    """Two call shapes, told apart by their arguments.

    apply(x, run_function, is_causal) -> o: the reference's (test_llama3.py:184-243, called at
    :459 as attention(hidden_states, project, is_causal)).  q, k, v = run_function(x,
    get_global_cross_attention_states()); saves (x, o, L) only; backward runs run_function
    again and sends dq, dk, dv back through it (real gradients, where the reference returns
    None).  Build run_function from `create_q_projection_class` / `create_kv_projection_class`
    to keep every GEMM on this library's kernels.

    apply(q, x_vis, w_k, w_v, n_kv_heads, sm_scale, mask=None, k_norm_weight=None,
    k_norm_eps=1e-5, bias_func=None, *bias_args) -> o: q given, K/V recomputed:

    Forward: K, V = kv_proj(x_vis); o, L = attention; saves (q, x_vis, w_k, w_v,
    o, L) - K and V are dropped.  (q stays: [B, Hq, Lq, D], 32 MiB at B1 Hq32 Lq4096, which is
    more than the 25 MiB of K and V at Lkv 6404 that are not kept; the run_function form above
    saves the layer input instead and recomputes q as well.)  Backward: recomputes K, V by the same GEMMs,
    runs the attention backward, then dX_vis = dK W_k^T + dV W_v^T (and, with
    `weight_grads`, dW_k = X^T dK, dW_v = X^T dV).  With `k_norm_weight` K is
    RMS-normalised per head in the projection's epilogue (the k_norm of
    test_llama3.py:418) and backward goes through the norm before dX_vis
    (weight_grads: also returns the norm weight's gradient).  `w_in_major`:
    W is [Dm, Hkv*D]; False: [Hkv*D, Dm] (torch.nn.Linear.weight).
    `bias_func(*bias_args)` gives the dense additive bias, as for
    `_attn_forward`; the arguments are kept and the bias is rebuilt in backward."""
    if attention_mode != "lv_xattn":
        raise ValueError("only attention_mode='lv_xattn' exists on this path")

    class _attention_by_tensors(torch.autograd.Function):
        @staticmethod
        def forward(ctx, q, x_vis, w_k, w_v, n_kv_heads, sm_scale, mask=None, k_norm_weight=None,
                    k_norm_eps=1e-5, bias_func=None, *bias_args):
            k, v = ops.kv_proj(x_vis, w_k, w_v, n_kv_heads, w_in_major, k_norm_weight=k_norm_weight,
                               eps=k_norm_eps)
            _, _, _, o, L = _attn_forward(q, k, v, False, sm_scale, None, bias_func, list(bias_args), [],
                                          no_overlap, rounds=rounds, mask=mask, batched=batched)
            ctx.has_norm = k_norm_weight is not None
            ctx.save_for_backward(q, x_vis, w_k, w_v, o, L, *([k_norm_weight] if ctx.has_norm else []), *bias_args)
            ctx.k_norm_eps, ctx.bias_func, ctx.n_bias = k_norm_eps, bias_func, len(bias_args)
            ctx.n_kv_heads, ctx.sm_scale, ctx.mask = n_kv_heads, sm_scale, mask
            reset_global_memory_buffer(attention_mode)
            return o

        @staticmethod
        def backward(ctx, do):
            q, x_vis, w_k, w_v, o, L, *rest = ctx.saved_tensors
            norm_w = rest[0] if ctx.has_norm else None
            bias_args = rest[1:] if ctx.has_norm else rest
            dwn = None
            if ctx.has_norm:                                             # recompute, keeping x and r
                k, v, k_raw, k_rstd = ops.kv_proj(x_vis, w_k, w_v, ctx.n_kv_heads, w_in_major,
                                                  k_norm_weight=norm_w, eps=ctx.k_norm_eps, for_backward=True)
            else:
                k, v = ops.kv_proj(x_vis, w_k, w_v, ctx.n_kv_heads, w_in_major)
            dq, dk, dv = _attn_backward(do, q, k, v, o, L, False, ctx.sm_scale, None, "flash",
                                        ctx.bias_func, list(bias_args), [], no_overlap,
                                        rounds=rounds, mask=ctx.mask, batched=batched)
            if ctx.has_norm:
                dk, dwn = ops.k_norm_bwd(dk, k_raw, k_rstd, norm_w, want_dw=weight_grads)
                if dwn is not None:
                    dwn = dwn.to(norm_w.dtype)
            dx = ops.dx_vis(dk, dv, w_k, w_v, w_in_major)
            dwk = dwv = None
            if weight_grads:
                dwk, dwv = ops.dw_kv(x_vis, dk, dv, w_in_major)
            return (dq, dx, dwk, dwv, None, None, None, dwn, None, None) + (None,) * ctx.n_bias

    class _attention_by_run_function(torch.autograd.Function):
        # The reference's own call shape (test_llama3.py:184-243): apply(x, run_function, is_causal)
        # with q, k, v = run_function(x, get_global_cross_attention_states()) and
        # sm_scale = head_dim ** -0.5.  Only (x, o, L) are kept; backward runs run_function again -
        # under autograd, on a detached x - and pushes dq, dk, dv back through it, so x gets its
        # gradient and so does whatever else run_function's graph reaches (projection weights,
        # norm weights, the visual states), where the reference returns none (:243).
        # backward only runs when the output has a grad_fn, i.e. when x requires grad: with a frozen
        # x (a frozen trunk under trainable projections) the parameters run_function reaches would
        # silently get no gradient, so that case is refused while gradients are being recorded.
        @staticmethod
        def forward(ctx, x, run_function, is_causal):
            _reject_unsupported(is_causal)
            if torch.is_grad_enabled() and not x.requires_grad:
                raise LvxError("create_attention_class(...).apply(x, run_function, is_causal): x does not require "
                               "grad, so backward would never run and run_function's parameters would get no "
                               "gradient; pass x.requires_grad_() (its gradient can be discarded) or call under "
                               "torch.no_grad()")
            q, k, v = run_function(x, get_global_cross_attention_states())
            sm_scale = q.size(-1) ** -0.5
            _, _, _, o, L = _attn_forward(q, k, v, is_causal, sm_scale, None, None, [], [], no_overlap,
                                          rounds=rounds, batched=batched)
            ctx.save_for_backward(x, o, L)
            ctx.run_function, ctx.causal = run_function, is_causal
            reset_global_memory_buffer(attention_mode)
            return o

        @staticmethod
        def backward(ctx, do):
            x, o, L = ctx.saved_tensors
            x_ = x.detach().requires_grad_(x.requires_grad)
            with torch.enable_grad():
                q, k, v = ctx.run_function(x_, get_global_cross_attention_states())
            sm_scale = q.size(-1) ** -0.5
            dq, dk, dv = _attn_backward(do, q.detach(), k.detach(), v.detach(), o, L, ctx.causal, sm_scale, None,
                                        "flash", None, [], [], no_overlap, rounds=rounds, batched=batched)
            outs = [(t, g) for t, g in ((q, dq), (k, dk), (v, dv)) if t.requires_grad]
            if outs:
                torch.autograd.backward([t for t, _ in outs], [g for _, g in outs])
            reset_global_memory_buffer(attention_mode)
            return x_.grad, None, None

    class _attention:
        """`apply` takes either call shape: (x, run_function, is_causal) - the reference's - or
        (q, x_vis, w_k, w_v, n_kv_heads, sm_scale, ...)."""
        by_tensors, by_run_function = _attention_by_tensors, _attention_by_run_function

        @staticmethod
        def apply(*args):
            if len(args) == 3 and callable(args[1]):
                return _attention_by_run_function.apply(*args)
            return _attention_by_tensors.apply(*args)

    return _attention


_global_cross_attention_states = None


def set_global_cross_attention_states(vision_features):
    """The visual hidden states every cross-attention layer projects its K and V from
    (test_llama3.py:69-79): set once per step, read by the run_function wrapper in both passes."""
    global _global_cross_attention_states
    _global_cross_attention_states = vision_features


def get_global_cross_attention_states():
    return _global_cross_attention_states


def clear_global_cross_attention_states():
    global _global_cross_attention_states
    _global_cross_attention_states = None


def create_kv_projection_class(w_in_major: bool = True, weight_grads: bool = True):
    """apply(x_vis, w_k, w_v, n_kv_heads, k_norm_weight=None, eps=1e-5) -> k, v [B, Hkv, Lkv, D]

    The visual side of the reference's `project` (test_llama3.py:395-398, 418) as one autograd
    function over the fused GEMMs: K = k_norm(X_vis W_k), V = X_vis W_v.  Nothing but the inputs
    is kept; backward re-runs the projection for the raw K and its r when there is a norm, goes
    back through the norm, then dX_vis = dK W_k^T + dV W_v^T and (weight_grads) dW_k, dW_v and
    the norm weight's gradient."""

    class _kv_projection(torch.autograd.Function):
        @staticmethod
        def forward(ctx, x_vis, w_k, w_v, n_kv_heads, k_norm_weight=None, eps=1e-5):
            ctx.has_norm = k_norm_weight is not None
            ctx.save_for_backward(x_vis, w_k, w_v, *([k_norm_weight] if ctx.has_norm else []))
            ctx.n_kv_heads, ctx.eps = n_kv_heads, eps
            return ops.kv_proj(x_vis, w_k, w_v, n_kv_heads, w_in_major, k_norm_weight=k_norm_weight, eps=eps)

        @staticmethod
        def backward(ctx, dk, dv):
            x_vis, w_k, w_v, *rest = ctx.saved_tensors
            dwn = None

            def token_major(t):      # [B, H, L, D] gradients in [B, L, H, D] memory order, as the GEMMs read them
                return t if t.transpose(1, 2).is_contiguous() else t.transpose(1, 2).contiguous().transpose(1, 2)

            dk, dv = token_major(dk), token_major(dv)
            if ctx.has_norm:
                _, _, k_raw, k_rstd = ops.kv_proj(x_vis, w_k, w_v, ctx.n_kv_heads, w_in_major, k_norm_weight=rest[0],
                                                  eps=ctx.eps, for_backward=True)
                dk, dwn = ops.k_norm_bwd(dk, k_raw, k_rstd, rest[0], want_dw=weight_grads)
                if dwn is not None:
                    dwn = dwn.to(rest[0].dtype)
            dx = ops.dx_vis(dk, dv, w_k, w_v, w_in_major)
            dwk = dwv = None
            if weight_grads:
                dwk, dwv = ops.dw_kv(x_vis, dk, dv, w_in_major)
            return dx, dwk, dwv, None, dwn, None

    return _kv_projection


def create_q_projection_class(w_in_major: bool = True, weight_grads: bool = True):
    """apply(x, w_q, n_heads, q_norm_weight, eps) -> q [B, Hq, Lq, D]

    The text side of the reference's `project` (test_llama3.py:390-393),
    Q = q_norm(X W_q), with the reference's recompute discipline
    (test_llama3.py:184-243: only the layer input is kept): forward saves
    (x, w_q, norm weight); backward re-runs the fused GEMM to get the raw
    projection and r, goes back through the norm, then dX = dQ_raw W_q^T and
    dW_q = X^T dQ_raw."""

    class _q_projection(torch.autograd.Function):
        @staticmethod
        def forward(ctx, x, w_q, n_heads, q_norm_weight, eps=1e-5):
            ctx.save_for_backward(x, w_q, q_norm_weight)
            ctx.n_heads, ctx.eps = n_heads, eps
            return ops.q_proj(x, w_q, n_heads, w_in_major, q_norm_weight, eps)

        @staticmethod
        def backward(ctx, dq):
            x, w_q, wn = ctx.saved_tensors
            _, q_raw, rstd = ops.q_proj(x, w_q, ctx.n_heads, w_in_major, wn, ctx.eps, for_backward=True)
            dq_tm = dq if dq.transpose(1, 2).is_contiguous() else dq.transpose(1, 2).contiguous().transpose(1, 2)
            dq_raw, dwn = ops.k_norm_bwd(dq_tm, q_raw, rstd, wn, want_dw=weight_grads)
            dx, dw = ops.q_proj_bwd(x, dq_raw, w_q, w_in_major, want_dw=weight_grads)
            return dx, dw, None, (dwn.to(wn.dtype) if dwn is not None else None), None

    return _q_projection
