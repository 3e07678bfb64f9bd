"""Drop-in for the reference's forward attention entry used by the DiT blocks.

Reference: cosmos_predict2/_src/predict2/networks/attention.py ``attention(q, k, v, q_lens=None,
k_lens=None, dropout_p=0.0, softmax_scale=None, q_scale=None, causal=False, deterministic=False,
dtype=torch.bfloat16) -> out`` (:90-181), tensors ``[B, S, H, D]``, output contiguous ``[B, S, H, D]`` (:180).

Behaviour kept: cast of q,k,v to ``dtype`` (:110-112), ``q_scale`` (:114-115), ``NotImplementedError`` for
unsupported dtypes (:107-108), ``q_lens`` / ``k_lens`` accepted and ignored (:94-95 -- the reference never
reads them).  The gfx950 kernels are deterministic (no atomics, fixed reduction order), so
``deterministic=True`` is honoured instead of raising (:151-154).  fp32 is not built: NotImplementedError.
``dropout_p != 0`` raises NotImplementedError: the reference's SDPA branch applies it (:176), the HIP kernels have no
dropout, and silently returning unregularised attention would be the worse deviation.
"""
from __future__ import annotations

import contextlib
import threading

import torch

from . import ops


class _KeptResults(threading.local):
    """Per host thread: where attention results (o, log-sum-exp) are being recorded, or replayed from."""

    record = None     # list that every attention call appends (o, lse) to
    replay = None     # list of (o, lse) that the next differentiable attention calls take instead of running the kernel


_kept = _KeptResults()


def results_are_kept() -> bool:
    """Is a recording or a replay of attention results under way on this thread?  (Callers that have another way to the
    kernels than ``attention()`` must not take it then.)"""
    return _kept.record is not None or _kept.replay is not None


@contextlib.contextmanager
def record_attention_results(store: list):
    """Every ``attention()`` call inside appends its ``(o [B,H,S,D] view of [B,S,H,D] memory, lse [B,H,S])`` to ``store``."""
    prev, _kept.record = _kept.record, store
    try:
        yield store
    finally:
        _kept.record = prev


@contextlib.contextmanager
def replay_attention_results(store: list):
    """The differentiable ``attention()`` calls inside take their forward results from ``store`` (in call order) instead
    of running the forward kernel again: activation recomputation that keeps the one expensive result of a block."""
    prev, _kept.replay = _kept.replay, list(store)
    try:
        yield
        assert not _kept.replay, "fewer attention calls in the recomputation than were recorded"
    finally:
        _kept.replay = prev


class _AttentionFn(torch.autograd.Function):
    """Forward-only attention on ``[B, S, H, D]`` tensors with a reverse-mode rule: the forward keeps o and the
    log-sum-exp, the backward is the HIP backward (equal head dims only)."""

    @staticmethod
    def forward(ctx, q, k, v, causal, softmax_scale):
        if _kept.replay is not None:
            if not _kept.replay:
                raise RuntimeError("more attention calls in the recomputation than were recorded")
            o, lse = _kept.replay.pop(0)
            if o.shape != (q.shape[0], q.shape[2], q.shape[1], v.shape[3]) or o.dtype != q.dtype:
                raise RuntimeError("recorded attention result of another call (shape or type differs)")
        else:
            o, _, lse = ops.fwd_jvp(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2),
                                    causal=causal, sm_scale=softmax_scale, out_layout="blhd", need_lse=True)
            if _kept.record is not None:
                _kept.record.append((o, lse))
        ctx.save_for_backward(q, k, v, o, lse)
        ctx.causal, ctx.softmax_scale = causal, softmax_scale
        return o.transpose(1, 2)

    @staticmethod
    def backward(ctx, dout):
        q, k, v, o, lse = ctx.saved_tensors
        t = lambda x: x.transpose(1, 2)
        dq, dk, dv = ops.bwd(t(q), t(k), t(v), o, lse, t(dout), causal=ctx.causal, sm_scale=ctx.softmax_scale)
        return t(dq), t(dk), t(dv), None, None


def attention(
    q,
    k,
    v,
    q_lens=None,
    k_lens=None,
    dropout_p=0.0,
    softmax_scale=None,
    q_scale=None,
    causal=False,
    deterministic=False,
    dtype=torch.bfloat16,
):
    supported_dtypes = [torch.bfloat16, torch.float16]
    if dtype not in supported_dtypes:
        # the reference also lists float32 (served by SDPA's efficient-attention backend, attention.py:145-148); the HIP
        # kernels compute from 16-bit operands only
        raise NotImplementedError(f"{dtype=} is not supported.")
    if dropout_p != 0.0:
        # On a ROCm build the reference takes its SDPA branch (get_device_cc() returns 0, attention.py:84-87, :127), which
        # applies dropout_p (:176).  The HIP kernels have no dropout: refuse loudly rather than train unregularised.
        raise NotImplementedError(f"attention(): dropout_p={dropout_p} is not supported by the HIP kernels (pass 0.0)")
    del q_lens, k_lens, deterministic

    q = q.to(dtype)
    k = k.to(dtype)
    v = v.to(dtype)
    if q_scale is not None:
        q = q * q_scale

    if torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad):
        return _AttentionFn.apply(q, k, v, causal, softmax_scale)   # the SDPA path of the reference is differentiable too

    # [B, S, H, D] -> heads-first views (no copy); the kernel writes [B, S, H, D] memory directly
    if _kept.replay is not None:      # a recomputation in which q, k, v happen not to need gradients
        if not _kept.replay:
            raise RuntimeError("more attention calls in the recomputation than were recorded")
        return _kept.replay.pop(0)[0].transpose(1, 2)
    recording = _kept.record is not None
    o, _, lse = ops.fwd_jvp(
        q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2),
        causal=causal, sm_scale=softmax_scale, out_layout="blhd", need_lse=recording,
    )
    if recording:
        _kept.record.append((o, lse))
    return o.transpose(1, 2)
