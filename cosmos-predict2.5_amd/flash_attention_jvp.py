"""Drop-in for the reference's Triton flash-attention-with-JVP entry point.

Reference: cosmos_predict2/_src/predict2/utils/flash_attention_jvp_triton.py
  ``attention = _attention.apply`` (:564), ``_attention.forward(ctx, q, k, v, tq, tk, tv, causal=False,
  sm_scale=None) -> (o, to)`` (:436-502), tensors ``[batch, heads, seq, head_dim]`` (:425-431).

Same names, argument order, defaults, assertions and return values; the computation runs in the
hand-written gfx950 kernels behind the C ABI.  ``attention_with_lse`` additionally returns the
log-sum-exp the reference keeps for its backward (:455, :499) and accepts ``key_lens``.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import ops


class _attention(torch.autograd.Function):
    """
    Arguments:
        q, tq: (batch_size, nheads, seqlen_q, d_qk)
        k, tk: (batch_size, nheads, seqlen_kv, d_qk)
        v, tv: (batch_size, nheads, seqlen_kv, d_v)
    Returns:
        o, to: (batch_size, nheads, seqlen_q, d_v)
    """

    @staticmethod
    def forward(ctx, q, k, v, tq, tk, tv, causal=False, sm_scale=None):
        is_grad = any(x.requires_grad for x in [q, k, v])
        # the reference asserts matching tangent shapes and strides (…jvp_triton.py:447-448)
        assert tq.shape == q.shape and tk.shape == k.shape and tv.shape == v.shape
        assert tq.stride() == q.stride() and tk.stride() == k.stride() and tv.stride() == v.stride()
        if sm_scale is None:
            sm_scale = q.shape[-1] ** (-0.5)
        o, to, lse = ops.fwd_jvp(q, k, v, tq, tk, tv, causal=causal, sm_scale=sm_scale)
        if is_grad:
            ctx.save_for_backward(q, k, v, o, lse)
            ctx.sm_scale = sm_scale
            ctx.causal = causal
        ctx.mark_non_differentiable(to)
        return o, to

    @staticmethod
    def backward(ctx, dout, *args):
        # The reference hands the saved (q, k, v, o, lse) and dout to flash-attn's backward and returns
        # (dq, dk, dv, None, ...) (…jvp_triton.py:505-561): gradient through o only, equal head dims only.
        q, k, v, out, softmax_lse = ctx.saved_tensors
        assert q.shape[-1] == k.shape[-1] and k.shape[-1] == v.shape[-1], (
            "Backward not supported with different headdim."
        )
        dq, dk, dv = ops.bwd(q, k, v, out, softmax_lse, dout, causal=ctx.causal, sm_scale=ctx.sm_scale)
        return dq, dk, dv, None, None, None, None, None


attention = _attention.apply


def attention_with_lse(q, k, v, tq=None, tk=None, tv=None, causal=False, sm_scale=None,
                       key_lens: Optional[torch.Tensor] = None):
    """(o, to, lse): forward + JVP plus the log-sum-exp; tangents optional; optional key-padding lengths."""
    return ops.fwd_jvp(q, k, v, tq, tk, tv, causal=causal, sm_scale=sm_scale, key_lens=key_lens)
