"""CPU oracle for the DiT ``Attention`` module (projections, per-head RMSNorm, RoPE, attention, output projection)
and its forward-mode tangent.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this module; only ``tests/``,
``__graft_entry__.smoke()`` and ``bench.py`` may use it, as the checker.

What it restates: ``Attention.forward`` of cosmos_predict2/_src/predict2/networks/minimal_v4_dit.py
(``compute_qkv`` :395-419, ``compute_attention`` :421-427, ``forward`` :429-445) with the ``torch`` backend
(``torch_attention_op`` :252-283: SDPA on ``[B, H, S, D]``, result flattened to ``[B, S, H*D]``), written as one
pure function of the weights so that ``torch.func.jvp`` gives the tangent.  RMSNorm and the rotary embedding are the
published semantics of the Transformer Engine ops the reference calls (see norm_rope_oracle.py).

``attention_module_grads_torch`` is torch autograd (reverse mode) of the same function.

Parity status: pinned in tests/test_oracle_dit_attention.py against the composition of the separately pinned fp64
closed forms (norm_rope_oracle.norm_rope_closed_form, attention_oracle.closed_form) with numpy matmuls, and by central
finite differences; the reverse mode by the adjoint identity against the forward-mode result and by finite differences
in the weights.  Against Transformer Engine's own kernels: PARITY UNPINNED, as for norm_rope_oracle.py.
"""
from __future__ import annotations

from typing import Dict, Optional


def attention_module_torch(weights: Dict[str, "torch.Tensor"], x, context=None, rope_angles=None, n_heads: int = 8,
                           head_dim: int = 64, tx=None, tcontext=None, eps: float = 1e-6, dtype=None):
    """weights: q_proj.weight, k_proj.weight, v_proj.weight, output_proj.weight, q_norm.weight, k_norm.weight
    (the module's state-dict names).  x: [B, Mq, K]; context: [B, Mk, Kc] or None (self-attention);
    rope_angles: [Mq, D] or None (applied for self-attention only, minimal_v4_dit.py:409).  fp32 unless ``dtype``.
    Returns (out, tout); tout is None without tx."""
    import torch
    import torch.nn.functional as F
    from torch.nn.attention import SDPBackend, sdpa_kernel

    dt = dtype or torch.float32
    w = {k: v.detach().to("cpu", dt) for k, v in weights.items()}
    f = lambda t: None if t is None else torch.as_tensor(t).detach().to("cpu", dt)
    x, context, tx, tcontext = f(x), f(context), f(tx), f(tcontext)
    selfattn = context is None
    a = None
    if rope_angles is not None and selfattn:
        a = torch.as_tensor(rope_angles).detach().to("cpu", dt).reshape(1, -1, 1, head_dim)

    def heads(t):
        return t.reshape(t.shape[0], -1, n_heads, head_dim)

    def norm_rope(t, g):
        n = F.rms_norm(t, (head_dim,), weight=g, eps=eps)
        if a is None:
            return n
        n1, n2 = n[..., : head_dim // 2], n[..., head_dim // 2:]
        return n * torch.cos(a) + torch.cat([-n2, n1], dim=-1) * torch.sin(a)

    def fwd(x_, c_):
        c_ = x_ if selfattn else c_
        q = norm_rope(heads(F.linear(x_, w["q_proj.weight"])), w["q_norm.weight"])
        k = norm_rope(heads(F.linear(c_, w["k_proj.weight"])), w["k_norm.weight"])
        v = heads(F.linear(c_, w["v_proj.weight"]))
        with sdpa_kernel([SDPBackend.MATH]):
            o = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2))
        o = o.transpose(1, 2).flatten(-2)
        return F.linear(o, w["output_proj.weight"])

    if tx is None:
        return fwd(x, context), None
    if selfattn:
        return torch.func.jvp(lambda x_: fwd(x_, None), (x,), (tx,))
    if tcontext is None:
        return torch.func.jvp(lambda x_: fwd(x_, context), (x,), (tx,))
    return torch.func.jvp(fwd, (x, context), (tx, tcontext))


def attention_module_grads_torch(weights, x, dout, context=None, rope_angles=None, n_heads: int = 8, head_dim: int = 64,
                                 eps: float = 1e-6, dtype=None):
    """Reverse mode of the module for the cotangent ``dout`` of its output: a dict with the gradients of ``x``,
    ``context`` (if given) and every weight (state-dict names).  fp32 unless ``dtype``."""
    import torch
    import torch.nn.functional as F
    from torch.nn.attention import SDPBackend, sdpa_kernel

    dt = dtype or torch.float32
    f = lambda t: None if t is None else torch.as_tensor(t).detach().to("cpu", dt)
    w = {k: f(v).requires_grad_(True) for k, v in weights.items()}
    x = f(x).requires_grad_(True)
    context = None if context is None else f(context).requires_grad_(True)
    selfattn = context is None
    a = None
    if rope_angles is not None and selfattn:
        a = f(rope_angles).reshape(1, -1, 1, head_dim)
    heads = lambda t: t.reshape(t.shape[0], -1, n_heads, head_dim)

    def norm_rope(t, g):
        n = F.rms_norm(t, (head_dim,), weight=g, eps=eps)
        if a is None:
            return n
        return n * torch.cos(a) + torch.cat([-n[..., head_dim // 2:], n[..., : head_dim // 2]], dim=-1) * torch.sin(a)

    c = x if selfattn else context
    q = norm_rope(heads(F.linear(x, w["q_proj.weight"])), w["q_norm.weight"])
    k = norm_rope(heads(F.linear(c, w["k_proj.weight"])), w["k_norm.weight"])
    v = heads(F.linear(c, w["v_proj.weight"]))
    with sdpa_kernel([SDPBackend.MATH]):
        o = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2))
    out = F.linear(o.transpose(1, 2).flatten(-2), w["output_proj.weight"])
    names = ["x"] + ([] if selfattn else ["context"]) + list(w)
    leaves = [x] + ([] if selfattn else [context]) + [w[k_] for k_ in w]
    grads = torch.autograd.grad(out, leaves, grad_outputs=f(dout))
    return dict(zip(names, grads))
