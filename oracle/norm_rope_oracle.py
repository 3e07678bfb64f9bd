"""CPU oracle for the per-head RMSNorm + rotary embedding step (and its forward-mode tangent).

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this module; only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may use it, as the checker.

What it restates
----------------
``Attention.compute_qkv`` in ``cosmos_predict2/_src/predict2/networks/minimal_v4_dit.py`` (below "DIT"):
``q_norm`` / ``k_norm`` are ``te.pytorch.RMSNorm(head_dim, eps=1e-6)`` (DIT:350-356), applied to the
``[B, S, H, D]`` heads (DIT:400-407), followed for self-attention by Transformer Engine's
``apply_rotary_pos_emb(t, rope_emb, tensor_format="bshd", fused=True)`` (DIT:409-414) with
``rope_emb`` the angles ``[S, 1, 1, D] = cat([t, h, w] * 2)`` (DIT:648-658).

Transformer Engine (pinned by the reference's Dockerfile / pyproject to the 1.13 line) is a third-party
dependency that is not part of the reference checkout and is not installed here.  Its two ops are
restated from their published semantics:

* ``RMSNorm``: ``y = x / sqrt(mean(x^2, -1) + eps) * weight`` computed in fp32, returned in the input type.
* ``apply_rotary_pos_emb`` (default, non-interleaved): ``t * cos(freqs) + rotate_half(t) * sin(freqs)`` with
  ``rotate_half(t) = cat(-t[..., D/2:], t[..., :D/2])``.  The reference's own call site fixes the variant:
  the angle vector is the half-vector repeated twice (DIT:648-656), which is the layout of the rotate-half
  form (channel j pairs with channel j + D/2), not of the interleaved one.

Functions
---------
``norm_rope_torch``         torch fp32: ``torch.nn.functional.rms_norm`` + rotate-half rotation under
                            ``torch.func.jvp`` -- the oracle the tolerance is quoted against.
``norm_rope_closed_form``   numpy fp64 closed form of value and tangent, independent of autograd; optional
                            16-bit rounding of the normalised tensor (RMSNorm's output type).
``norm_rope_grads_torch``   torch autograd (reverse mode) of the same function: (dx, dweight) for a cotangent dy.
``norm_rope_grads_closed_form``  numpy fp64 closed form of the reverse mode.

Parity status: the mathematics is pinned in ``tests/test_oracle_norm_rope.py`` (closed form against torch forward AD
and torch's own ``rms_norm``, finite differences, brute-force scalar loops, rotation invariants: zero angle,
pair-norm preservation, angle additivity, relative-position property; RMSNorm invariants: scale invariance
and the zero tangent along x; the reverse mode against torch autograd, the adjoint identity <dy, J tx> = <J^T dy, tx>
with the pinned forward-mode closed form as J, and finite differences in the weight).  Against Transformer Engine's
binaries themselves -- in particular the exact rounding points of its fused kernels -- PARITY UNPINNED: the library is absent and the reference holds no
stored outputs of this step.
"""
from __future__ import annotations

from typing import Optional

import numpy as np


def _rotate_half_np(t: np.ndarray) -> np.ndarray:
    d = t.shape[-1] // 2
    return np.concatenate([-t[..., d:], t[..., :d]], axis=-1)


def _round_half(x: np.ndarray, half: Optional[str]) -> np.ndarray:
    if half is None:
        return x
    import torch

    dt = {"bf16": torch.bfloat16, "fp16": torch.float16}[half]
    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(dt).to(torch.float64).numpy()


def norm_rope_closed_form(x, weight=None, angles=None, tx=None, eps: float = 1e-6, half: Optional[str] = None):
    """numpy fp64.  x, tx: [B, S, H, D]; weight: [D] or None; angles: [S, D] or None.  Returns (y, ty or None).

    ``half`` ("bf16" / "fp16") rounds the normalised tensor (and its tangent) to that type before the
    rotation, which is where RMSNorm hands a 16-bit tensor to the rotary op (DIT:405-414)."""
    x = np.asarray(x, dtype=np.float64)
    B, S, H, D = x.shape
    g = np.ones(D) if weight is None else np.asarray(weight, dtype=np.float64)
    ms = (x * x).mean(axis=-1, keepdims=True)
    r = 1.0 / np.sqrt(ms + eps)
    n = _round_half(x * r * g, half)
    dn = None
    if tx is not None:
        tx = np.asarray(tx, dtype=np.float64)
        # d/de [ (x + e tx) (mean((x + e tx)^2) + eps)^(-1/2) ] = tx r - x r^3 mean(x tx)
        dn = _round_half(g * (tx * r - x * r**3 * (x * tx).mean(axis=-1, keepdims=True)), half)
    if angles is None:
        return n, dn
    a = np.asarray(angles, dtype=np.float64).reshape(1, S, 1, D)
    c, s = np.cos(a), np.sin(a)
    y = n * c + _rotate_half_np(n) * s
    ty = None if dn is None else dn * c + _rotate_half_np(dn) * s   # the rotation is linear in n
    return y, ty


def norm_rope_torch(x, weight=None, angles=None, tx=None, eps: float = 1e-6):
    """torch fp32 on the CPU: library rms_norm, rotate-half rotation, tangent by ``torch.func.jvp``."""
    import torch
    import torch.nn.functional as F

    x = torch.as_tensor(np.asarray(x, dtype=np.float32)) if not isinstance(x, torch.Tensor) else x.detach().float().cpu()
    B, S, H, D = x.shape
    w = None if weight is None else torch.as_tensor(np.asarray(weight, dtype=np.float32))
    a = None if angles is None else torch.as_tensor(np.asarray(angles, dtype=np.float32)).reshape(1, S, 1, D)

    def f(t):
        n = F.rms_norm(t, (D,), weight=w, eps=eps)
        if a is None:
            return n
        n1, n2 = n[..., : D // 2], n[..., D // 2 :]
        return n * torch.cos(a) + torch.cat([-n2, n1], dim=-1) * torch.sin(a)

    if tx is None:
        return f(x), None
    tx = torch.as_tensor(np.asarray(tx, dtype=np.float32)) if not isinstance(tx, torch.Tensor) else tx.detach().float().cpu()
    y, ty = torch.func.jvp(f, (x,), (tx,))
    return y, ty


def norm_rope_grads_closed_form(x, weight=None, angles=None, dy=None, eps: float = 1e-6):
    """numpy fp64 reverse mode: (dx, dweight) with dy the cotangent of y.
        dn = R^T dy,   dx = r (g dn) - x r^3 mean(x g dn),   dweight = sum_rows dn x r."""
    x = np.asarray(x, dtype=np.float64)
    dy = np.asarray(dy, dtype=np.float64)
    B, S, H, D = x.shape
    g = np.ones(D) if weight is None else np.asarray(weight, dtype=np.float64)
    if angles is None:
        dn = dy
    else:
        a = np.asarray(angles, dtype=np.float64).reshape(1, S, 1, D)
        # y = n cos(a) + rotate_half(n) sin(a);  the adjoint of rotate_half is its negative
        dn = dy * np.cos(a) - _rotate_half_np(dy * np.sin(a))
    r = 1.0 / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)
    gdn = g * dn
    dx = r * gdn - x * r**3 * (x * gdn).mean(axis=-1, keepdims=True)
    dweight = (dn * x * r).sum(axis=(0, 1, 2))
    return dx, dweight


def norm_rope_grads_torch(x, weight=None, angles=None, dy=None, eps: float = 1e-6, dtype=None):
    """torch autograd of rms_norm + rotate-half rotation: (dx, dweight) for the cotangent dy (fp32 unless ``dtype``)."""
    import torch
    import torch.nn.functional as F

    dt = dtype or torch.float32
    t = lambda z: torch.as_tensor(np.asarray(z)).to(dt) if not isinstance(z, torch.Tensor) else z.detach().cpu().to(dt)
    x = t(x).requires_grad_(True)
    B, S, H, D = x.shape
    w = (torch.ones(D, dtype=dt) if weight is None else t(weight)).requires_grad_(True)
    n = F.rms_norm(x, (D,), weight=w, eps=eps)
    if angles is not None:
        a = t(angles).reshape(1, S, 1, D)
        n = n * torch.cos(a) + torch.cat([-n[..., D // 2:], n[..., : D // 2]], dim=-1) * torch.sin(a)
    dx, dw = torch.autograd.grad(n, (x, w), grad_outputs=t(dy))
    return dx, dw


def rope_angles_3d(T: int, Hh: int, W: int, D: int, theta: float = 10000.0) -> np.ndarray:
    """Angles with the reference's layout (DIT:600-658, without its NTK / fps rescaling): per position
    (t, h, w) the vector cat([t f_t, h f_h, w f_w] * 2) with dim_h = dim_w = D/6*2, dim_t = D - 2 dim_h.
    Returns [T*Hh*W, D] fp32.  Used by tests and the bench to get angles of realistic magnitude."""
    dim_h = D // 6 * 2
    dim_w = dim_h
    dim_t = D - 2 * dim_h

    def freqs(dim):
        return 1.0 / theta ** (np.arange(0, dim, 2)[: dim // 2].astype(np.float64) / dim)

    et = np.outer(np.arange(T), freqs(dim_t))
    eh = np.outer(np.arange(Hh), freqs(dim_h))
    ew = np.outer(np.arange(W), freqs(dim_w))
    half = np.concatenate(
        [
            np.broadcast_to(et[:, None, None, :], (T, Hh, W, et.shape[1])),
            np.broadcast_to(eh[None, :, None, :], (T, Hh, W, eh.shape[1])),
            np.broadcast_to(ew[None, None, :, :], (T, Hh, W, ew.shape[1])),
        ],
        axis=-1,
    )
    return np.concatenate([half, half], axis=-1).reshape(T * Hh * W, D).astype(np.float32)
